"""The inference tenant of the colocation benchmark: forward-only requests that arrive as a Poisson process and run
ahead of training's queued launches.

The reference colocates a C++ inference server with the training process and lets inference kernels overtake
training ones through xsched: training's stream is a queue that hands at most 16 launches to the hardware at a
time, and is suspended while a request runs (common/xsched_ctrl.cc:27-108,
third_party/xsched/preempt/xqueue/xqueue.cpp:80-137, worker.cpp:155-260).  Here the same happens inside one
process: training's stream is registered with the launch queue (torch_col.xsched.register_stream), the requests
run on a stream of their own that is not, and around every request the queues are suspended and resumed.  The
launches training already handed to the hardware (at most the queue's depth) finish beside the request; nothing
of training starts behind them until the request is done.
"""
import threading
import time

import numpy as np
import torch

from .torch_col import xsched


def poisson_arrivals(rate_per_s, n, seed=0):
    """Arrival times in seconds from 0: cumulative sums of n exponential gaps of mean 1 / rate (seeded)."""
    gaps = np.random.default_rng(seed).exponential(1.0 / rate_per_s, n)
    return np.cumsum(gaps)


class ColocatedInference:
    """Serves `engine.forward_eval` on batches of `batch` images at the given arrival times, from a thread.

    preempt: suspend training's launch queues for the length of a request (the colocation mode); False lets the
    request compete with whatever training has queued (for comparison).
    sync_hw: also wait for the launches training already handed to the hardware before the request starts."""

    def __init__(self, engine, arrivals_s, batch=1, preempt=True, sync_hw=False, seed=0):
        self.engine, self.arrivals, self.batch = engine, np.asarray(arrivals_s, dtype=np.float64), batch
        self.preempt, self.sync_hw = preempt, sync_hw
        g = torch.Generator().manual_seed(seed)
        self.image = torch.randn(batch, 3, engine.image_size, engine.image_size, generator=g).pin_memory()
        # the engine's own stream (default priority): it must not be a registered (preemptible) one
        self.stream = engine.ctx.stream
        self.latencies_ms, self.service_ms, self.started_late_ms = [], [], []
        self.last_logits = None
        self._thread, self._stop = None, threading.Event()
        self.error = None

    def warm_up(self, n=3):
        with torch.cuda.stream(self.stream):
            for _ in range(n):
                self.engine.forward_eval(self.image.to(self.engine.dev, non_blocking=True))
            self.engine.ctx.synchronize()

    def _serve_one(self, arrival_abs):
        t_begin = time.perf_counter()
        if self.preempt:
            xsched.suspend_all_streams(self.sync_hw)
        try:
            with torch.cuda.stream(self.stream):
                plan = self.engine.forward_eval(self.image.to(self.engine.dev, non_blocking=True))
                self.engine.ctx.synchronize()
        finally:
            if self.preempt:
                xsched.resume_all_streams()
        t_end = time.perf_counter()
        self.latencies_ms.append((t_end - arrival_abs) * 1e3)
        self.service_ms.append((t_end - t_begin) * 1e3)
        self.started_late_ms.append((t_begin - arrival_abs) * 1e3)
        self.last_logits = plan.logits

    def _run(self):
        try:
            torch.cuda.set_device(self.engine.dev)
            t0 = time.perf_counter()
            for a in self.arrivals:
                if self._stop.is_set():
                    break
                # requests queue up behind one another: a request that arrives while the one before is still
                # being served starts late, and that wait is part of its latency
                while True:
                    left = t0 + a - time.perf_counter()
                    if left <= 0 or self._stop.is_set():
                        break
                    time.sleep(min(left, 0.002) if left > 0.0005 else 0)
                if self._stop.is_set():
                    break
                self._serve_one(t0 + a)
        except Exception as e:   # surfaced by stop()
            self.error = e

    def start(self):
        self._thread = threading.Thread(target=self._run, name="colocated-inference", daemon=True)
        self._thread.start()
        return self

    def stop(self):
        self._stop.set()
        if self._thread is not None:
            self._thread.join(timeout=30.0)
            if self._thread.is_alive():
                raise RuntimeError("the inference thread did not stop")
        if self.preempt:
            xsched.resume_all_streams()
        if self.error is not None:
            raise self.error

    def join(self):
        """Serve every arrival, then return."""
        if self._thread is not None:
            self._thread.join()
        if self.error is not None:
            raise self.error

    def summary(self):
        lat = np.asarray(self.latencies_ms)
        if lat.size == 0:
            return {"requests": 0}
        return {"requests": int(lat.size), "p50_ms": float(np.percentile(lat, 50)), "p99_ms": float(np.percentile(lat, 99)),
                "mean_ms": float(lat.mean()), "max_ms": float(lat.max()),
                "service_p50_ms": float(np.percentile(self.service_ms, 50))}
