"""What the training scripts of this package share: set-up / tear-down of the colocation runtime, the
in-process stand-in for the inference server, and the epoch loop with its per-epoch report line (the
reference's scripts repeat these: train/swin_b.py:97-138, train/resnet152.py:93-153, train/gpt2.py:75-150).
"""
import os
import threading
import time
from typing import Optional

from .. import torch_col
from ..torch_col import EventManager, MemoryPool


def setup():
    torch_col.info(f'[Train PID {os.getpid()}] setup')
    return torch_col.setup_colocate_training(0, 1, False, False)


def cleanup():
    torch_col.cleanup_colocate_training(False)


class PeerScript:
    """Stand-in inference server: `at` maps a micro-batch index to ('l1' | 'l2' | 'exit', batch size) or to
    ('switch', milliseconds until the resume), or to ('cus', compute units inference wants for itself).
    The command is sent from a side thread `delay_ms` after the micro-batch began, so that it lands
    while kernels are queued, as a real request would; with `delay_ms` <= 0 it is sent on the spot, before
    the micro-batch's first launch (no thread, no dependence on how the threads are scheduled)."""

    def __init__(self, at, delay_ms=5.0, verbose=False):
        self.server = torch_col.DebugServer(1, verbose=verbose)
        self.at = dict(at)
        self.delay_ms = delay_ms
        self.sent = []
        self._threads = []

    def on_batch(self, idx):
        cmd = self.at.pop(idx, None)
        if cmd is None:
            return
        kind, bs = cmd

        def fire():
            time.sleep(self.delay_ms / 1e3)
            t = torch_col.get_unix_timestamp_us()
            if kind == "switch":
                # task switch: interrupt now, resume `bs` milliseconds later (training stands still in
                # between, so no micro-batch index could trigger the resume)
                self.server.interrupt_train()
                self.sent.append((t, "interrupt", 0))
                time.sleep(bs / 1e3)
                self.server.resume_train()
                self.sent.append((torch_col.get_unix_timestamp_us(), "resume", 0))
                return
            {"l1": self.server.colocate_l1, "l2": self.server.colocate_l2, "exit": self.server.infer_exit,
             "cus": self.server.set_infer_required_cus}[kind](bs)
            self.sent.append((t, kind, bs))
        if self.delay_ms <= 0:
            fire()
            return
        t = threading.Thread(target=fire, daemon=True)
        self._threads.append(t)
        t.start()

    def stop(self):
        # a command still on its way must not reach the communicator after the runtime is shut down
        for t in self._threads:
            t.join(timeout=5.0)
        alive = [t for t in self._threads if t.is_alive()]
        self.server.stop()
        if alive:
            raise RuntimeError(f"PeerScript.stop: {len(alive)} command thread(s) still running after 5 s")


def autotune_requested():
    """COLTRAIN_AUTOTUNE=1 (train/resnet152.py): the engine times every tiling of each distinct layer shape whenever it builds the plan
    of a new batch size and keeps the fastest (a few tenths of a second per plan, scratch tensors from the same
    allocator as the activations).  Off by default: a colocated run rebuilds plans while the inference side waits
    for memory."""
    return os.environ.get("COLTRAIN_AUTOTUNE", "0") == "1"


def attach_cu_partition(model):
    """With COLTRAIN_DYNAMIC_SM_PARTITION the engine asks the shared board before every launch segment how
    many compute units training may use (csrc/init.cc:43-71 + common/sm_partition.cc:96-112)."""
    if torch_col.sm_partition_enabled():
        model.set_cu_share_provider(torch_col.get_train_avail_cus)


def run_epochs(tag, model, iter_train_fn, col_ctrl, train_mode, num_epoch: int, batch_size: int,
               global_batch_size: Optional[int]):
    """Trainer.train_one_epoch per epoch with the reference's report line; ends the control session, dumps
    the event profile and returns what the callers and tests look at."""
    trainer = torch_col.Trainer(model, iter_train_fn)
    for epoch in range(num_epoch):
        trainer.train_one_epoch(epoch)
        model.synchronize()
        running_loss = model.last_loss()
        epoch_stat = trainer.get_last_epoch_stat()
        epoch_duration = trainer.get_last_epoch_duration()
        mem_info = f'mem {MemoryPool.get_memory_usage():.2f}Gb'
        batch_info = (f'batch cnt {epoch_stat.finished_batch} '
                      f'avg {epoch_duration / max(1, epoch_stat.finished_batch):.1f}ms')
        if train_mode.is_kill_batch():
            batch_info += (f' | try {epoch_stat.tried_batch} kill {epoch_stat.killed_batch}, '
                           f'{epoch_stat.killed_time*1e3:.1f}ms finish {epoch_stat.finished_batch}, '
                           f'{epoch_stat.finished_time*1e3:.1f}ms')
        if global_batch_size is not None:
            batch_info += f' | num_rollback_sampels {epoch_stat.num_rollback_batch}'
        print(f'[{tag} epoch {epoch}] {epoch_duration / 1e3:.3f}s | {batch_info} | batch-size {batch_size} '
              f'| {mem_info} | thpt {epoch_stat.finished_sample / (epoch_duration / 1e3):.3f} '
              f'| loss {running_loss:.6f}', flush=True)
        if col_ctrl.can_exit_after_infer_worklaod_done():
            print('[hook] inference workload done, will exit training', flush=True)
            break

    if train_mode.is_kill_batch():
        overall_stat = trainer.get_overall_stat()
        print("[" + tag + "] Epoch x Batch {} | Batch Total Tried {} Killed {} Finished {}".format(
            num_epoch * batch_size, overall_stat.tried_batch, overall_stat.killed_batch,
            overall_stat.finished_batch), flush=True)
    col_ctrl.train_end()
    col_ctrl.stop()
    path = EventManager.dump(None, train_mode)
    cleanup()
    return {"trainer": trainer, "model": model, "ctrl": col_ctrl, "profile": path}


