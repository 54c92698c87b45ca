#!/usr/bin/env python3
"""bench.py -- ResNet-152 bf16 batch-64 training step on one MI355X.

    python bench.py [--gpus 1] [--steps 20] [--warmup 5]

A step is one pass of the hot path over one synthetic batch that already sits in HBM:
NCHW->NHWC conversion, forward, softmax-CE, hand-written backward, SGD-momentum with the
bf16 shadow refresh.  Prints ONE JSON line.  After the timed region the same programs
are replayed with a HIP event between any two launches to attribute time to kernels
(`roofline`, `conv_mfma_util`), and the CPU oracle step is timed on the host cores
(`cpu_baseline`).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_FLOPS = 2.5e15   # MI355X dense bf16 MFMA
PEAK_HBM_BYTES = 8.0e12    # MI355X HBM3E
METRIC = "ResNet-152 bf16 bs64 train images/sec on 1 GPU; conv MFMA util %"
# HBM bytes per launch of the kernels that can top the step, from two rocprofv3 --pmc runs of this file
# (FETCH_SIZE and WRITE_SIZE, KiB per dispatch, scaled by what the same counters read for the --calibrate
# copy of known size: factors 2.000 and 1.000); the summary is profiles/resnet152_bf16_bs64_step_kernel_stats_and_traffic.txt
# The handover measurement: a pool of nearly the whole part in 128 MB pages (the reference's 32 MB page costs one
# driver call per page on the way out: 9 GB take 68 ms there, 18 ms in 128 MB pages).
HANDOVER_POOL_GB = 256
HANDOVER_PAGE_MB = 128
# The rocprofv3 summaries of this file's default run: kernel trace (average durations inside the step) and the
# FETCH_SIZE / WRITE_SIZE counter runs the traffic figures below are taken from.
PROFILE_FILE = "profiles/resnet152_bf16_bs64_step_kernel_stats_and_traffic.txt"
MEASURED_TRAFFIC_MIB = {
    "wgrad_kernel<bf16,128x128>": 44.18 + 15.41,
    "wgrad_kernel<bf16,64x64>": 93.22 + 6.32,
    "igemm2_kernel<bf16,dgrad,128x64,3buf,k32>": 73.34 + 33.50,
    "igemm2_kernel<bf16,dgrad,128x128,2buf>": 63.51 + 30.53,
    "igemm2_kernel<bf16,dgrad,128x128,3buf,k32>": 66.89 + 35.55,
    "igemm2_kernel<bf16,dgrad,128x128,2buf,k32>": 89.75 + 34.04,
    "igemm2_kernel<bf16,dgrad,128x64,3buf>": 70.39 + 31.94,
    "igemm2_kernel<bf16,fwd,128x128,2buf>": 28.05 + 15.45,
    "igemm2_kernel<bf16,fwd,128x128,2buf,k32>": 32.77 + 29.51,
    "igemm2_kernel<bf16,fwd,128x64,3buf>": 37.96 + 16.22,
    "igemm3_kernel<bf16,dgrad,128x64,3buf,patch160>": 29.50 + 5.99,
    "bn_fin_apply_kernel<bf16,bwd>": 24.39 + 11.91,
    "bn_fin_apply_kernel<bf16,fwd>": 20.39 + 12.03,
}


def grouped_wgrad_step(batch, x, y, steps, warmup, tile_cache):
    """The same step with the weight gradients of a whole stage as ONE launch over a table
    (`ResNetEngine(group_wgrad=True)`) instead of one launch (+ one split reduction) per layer: what the grouped
    kernel does to the weight gradients' kernel time, and what it does to the step."""
    import torch
    from sirius_amd.resnet import ResNetEngine
    eng = ResNetEngine((3, 8, 36, 3), 1000, 64, dtype=torch.bfloat16, image_size=224, lr=0.1, momentum=0.9,
                       weight_decay=1e-4, autotune=True, group_wgrad=True, wgrad_group_blocks=0, wgrad_group_wgs=1024)
    eng._tile_cache.update(tile_cache)          # the tilings the headline run measured
    eng.init_kaiming(seed=0)
    for _ in range(warmup):
        eng.forward_backward(x, y)
        eng.optimizer_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.forward_backward(x, y)
        eng.optimizer_step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    plan = eng.plan(batch)
    rows = eng.ctx.profile(plan.prog, 1) + eng.ctx.profile(eng._opt_prog, 1)
    wg = [r for r in rows if r["name"].startswith(("wgrad_", "splitk_reduce"))]
    conv = [r for r in rows if r["name"].startswith(("igemm_kernel", "igemm2_kernel", "igemm3_kernel", "wgrad_"))]
    grp = [r for r in rows if r["name"].startswith("wgrad_group_kernel<bf16,128x128>")]
    res = {"ms_per_step": ms, "images_per_s": batch / (ms * 1e-3), "launches_per_step": len(plan.prog) + len(eng._opt_prog),
           "wgrad_and_reduce_kernel_ms": sum(r["total_ms"] for r in wg),
           "conv_mfma_util": sum(r["work"] for r in conv) / (sum(r["total_ms"] for r in conv) * 1e-3) / PEAK_BF16_FLOPS,
           "wgrad_group_128x128_tflops": (sum(r["work"] for r in grp) / (sum(r["total_ms"] for r in grp) * 1e-3) / 1e12) if grp else None,
           "groups": len(plan.wgrad_groups),
           "layers_without_partial_filters": sum(sum(1 for sp in g["splits"] if sp == 1) for g in plan.wgrad_groups),
           "layers_grouped": sum(len(g["splits"]) for g in plan.wgrad_groups)}
    del eng, plan
    torch.cuda.empty_cache()
    return res


def cpu_model():
    """The host processor as the kernel reports it: model name, and family / model / stepping numbers (a guest
    system may be shown a generic name only)."""
    fields = {}
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if ":" not in line:
                    if fields:
                        break       # one processor entry is enough
                    continue
                k, v = line.split(":", 1)
                fields.setdefault(k.strip().lower(), v.strip())
    except OSError:
        pass
    if "model name" in fields:
        ids = ", ".join(f"{k} {fields[k]}" for k in ("cpu family", "model", "stepping") if k in fields)
        return fields["model name"] + (f" ({ids})" if ids else "")
    import platform
    return platform.processor() or platform.machine()


def cpu_baseline(batch, timed_steps):
    """The CPU oracle step (oracle/resnet.py: plain torch.nn ResNet-152, fp32, SGD) on the
    host cores of this box: 1 warm-up step + `timed_steps` timed steps at the bench batch."""
    import torch
    from oracle import resnet as R
    cores = torch.get_num_threads()
    model = R.make_model((3, 8, 36, 3), 1000, 64, seed=0)
    x, y = R.make_batch(batch, 224, 1000, seed=0)
    R.train_steps(model, x, y, 1)
    t0 = time.perf_counter()
    R.train_steps(model, x, y, timed_steps)
    dt = time.perf_counter() - t0
    return {"value": batch * timed_steps / dt, "unit": "images/s", "cores": cores, "cpu_model": cpu_model(),
            "kind": "port", "sample": f"ResNet-152 fp32 batch {batch} @224, torch CPU oracle step, 1 warm-up + {timed_steps} timed steps"}


def handover(batch, pool_gb=None, page_mb=None, lazy=False):
    """BASELINE configs[2]: ResNet-152 bf16 under the colocation protocol, global batch fixed at
    `batch`; a stand-in inference peer asks for memory (target batch 16) during the 4th micro-batch
    and leaves later (target back to `batch`).  Reports request -> AdjustL1Done as the server sees
    it, split into wait (request received -> release starts) and release, and the bytes returned.
    lazy: the pool answers first and removes its mappings of the pages it handed back right after the reply (a peer
    waits for a page's flag before it maps it); `request_to_last_page_usable_ms` then says when the last one was gone."""
    import contextlib
    import csv
    import tempfile

    import torch
    from sirius_amd import torch_col
    from sirius_amd.train import resnet152 as script

    tmp = tempfile.mkdtemp(prefix="tch_bench_")
    env = {"COLTRAIN_MODE": "colocate-l1", "COLTRAIN_HOOK_MODE": "xsched-sync", "COLTRAIN_USE_XSCHED": "1",
           "COLTRAIN_HAS_INFER_SERVER": "1", "COLTRAIN_USE_SHARED_TENSOR": "1",
           "COLTRAIN_SHARED_TENSOR_POOL_GB": str(pool_gb or HANDOVER_POOL_GB),
           "COLTRAIN_POOL_PAGE_MB": str(page_mb or HANDOVER_PAGE_MB), "COLTRAIN_POOL_LAZY_UNMAP": "1" if lazy else "0",
           "COLTRAIN_PROFILE_LOG_PATH": os.path.join(tmp, "train-profile.csv"),
           "SIRIUS_PORT": str(18000 + os.getpid() % 1000)}
    os.environ.update(env)
    peer = script.PeerScript({3: ("l1", 16), 14: ("exit", batch)}, delay_ms=8.0)
    try:
        with contextlib.redirect_stdout(sys.stderr):
            out = script.train(1, batch, dataset_size=batch * 10, dtype=torch.bfloat16, peer=peer,
                               num_distinct_samples=batch)
    finally:
        peer.stop()
    req, fin = torch_col.get_adjust_request_time_stamp(), torch_col.get_adjust_done_time_stamp()
    rows = list(csv.DictReader(open(out["profile"])))
    adj = [r for r in rows if r["name"] == "adjust_l1"]
    sizes = [int(r["name"].split("_")[-1]) for r in rows if r["name"].startswith("batch_0")]
    stat = out["trainer"].get_last_epoch_stat()
    res = {
        "request_to_done_ms": (fin[0] - req[0]) / 1e3 if req and fin else None,
        "wait_ms": float(adj[0]["timestamp"]) - req[0] / 1e3 if adj and req else None,
        "release_ms": float(adj[0]["duration"]) if adj else None,
        "stages_ms": {k: round(v, 3) for k, v in out["ctrl"].last_adjust.items() if k.endswith("_ms")},
        "activation_bytes_released": out["ctrl"].last_adjust.get("released_bytes"),
        "pool_bytes_returned": out["ctrl"].last_adjust.get("pool_bytes_returned"),
        "micro_batch_sizes": sizes,
        "killed_batches": stat.killed_batch,
        "finished_samples": stat.finished_sample,
        "bound_ms": 50.0,
        "pool_gb": pool_gb or HANDOVER_POOL_GB,
        "page_mb": page_mb or HANDOVER_PAGE_MB,
        "unmapping": ("after the reply: the pages are FREE and claimable at once, each flagged in the shared page table until "
                      "training's mapping of it is gone; a peer waits for the flag of the page it maps") if lazy else
                     "eager: every page handed back is unmapped from training's address range before the reply",
        "stale_pages_after": out["ctrl"].last_adjust.get("stale_pages_after"),
    }
    la = out["ctrl"].last_adjust
    if lazy and res["request_to_done_ms"] is not None:
        res["request_to_last_page_usable_ms"] = res["request_to_done_ms"] + la.get("stat_ms", 0.0) + la.get("trim_after_reply_ms", 0.0)
        res["pages_unmapped_after_reply"] = la.get("trimmed_after_reply")
    del out
    torch_col.reset_for_tests()
    torch_col.torch_col_shutdown()
    return res


def through_plugin(batch, batches=30, skip=8):
    """The same step through the plugin path, as the reference's train script drives it: colocate-l1 mode with the
    allocator hook and the launch queue, micro-batches copied from pinned host memory (the next one ahead of
    time on a copy stream), forward + backward + accumulate + optimizer, one synchronisation per micro-batch,
    no inference peer.  Images per second over the micro-batch durations the profile records (the first
    `skip` left out)."""
    import contextlib
    import csv
    import tempfile

    import torch
    from sirius_amd import torch_col
    from sirius_amd.train import resnet152 as script

    tmp = tempfile.mkdtemp(prefix="tch_bench_")
    os.environ.update({"COLTRAIN_MODE": "colocate-l1", "COLTRAIN_HOOK_MODE": "xsched-sync", "COLTRAIN_USE_XSCHED": "1",
                       "COLTRAIN_HAS_INFER_SERVER": "0", "COLTRAIN_USE_SHARED_TENSOR": "1",
                       "COLTRAIN_SHARED_TENSOR_POOL_GB": "48", "COLTRAIN_POOL_PAGE_MB": "32", "COLTRAIN_AUTOTUNE": "1",
                       "COLTRAIN_PROFILE_LOG_PATH": os.path.join(tmp, "train-profile.csv"),
                       "SIRIUS_PORT": str(19000 + os.getpid() % 1000)})
    with contextlib.redirect_stdout(sys.stderr):
        out = script.train(1, batch, dataset_size=batch * batches, dtype=torch.bfloat16, num_distinct_samples=batch * 2)
    rows = [r for r in csv.DictReader(open(out["profile"])) if r["name"].startswith("batch_0")]
    dur = [float(r["duration"]) for r in rows][skip:]
    t_first, t_last = float(rows[skip]["timestamp"]), float(rows[-1]["timestamp"]) + float(rows[-1]["duration"])
    res = {"images_per_s": batch * len(dur) / ((t_last - t_first) * 1e-3), "micro_batches_timed": len(dur),
           "ms_per_micro_batch": sum(dur) / len(dur),
           "ms_per_micro_batch_wall": (t_last - t_first) / len(dur),
           "note": "train script + Trainer + dataset: H2D copy of the next micro-batch overlapped on a copy stream, "
                   "gradient accumulation, one synchronisation per micro-batch; wall = first timed micro-batch's "
                   "begin to the last one's end, dataset and bookkeeping between micro-batches included"}
    del out
    torch_col.reset_for_tests()
    torch_col.torch_col_shutdown()
    return res


def gpt2_step(batch=8, seq_len=1024, warmup=2, steps=5):
    """BASELINE configs[4]'s training side: GPT-2 small (124.4 M parameters), bf16 compute with fp32 master
    weights, token ids uniform in [0, 50257) of shape [8, 1024], AdamW.  Reported beside the headline figure."""
    import torch
    from sirius_amd.gpt2 import GPT2Engine
    eng = GPT2Engine(seq_len=seq_len, dtype=torch.bfloat16, optimizer="adamw")
    eng.init_normal(0)
    g = torch.Generator(device="cuda")
    g.manual_seed(2)
    ids = torch.randint(0, eng.vocab, (batch, seq_len), device="cuda", generator=g)
    for _ in range(warmup):
        eng.forward_backward(ids)
        eng.optimizer_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.forward_backward(ids)
        eng.optimizer_step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    plan = eng.plan(batch)
    rows = eng.ctx.profile(plan.prog, 1) + eng.ctx.profile(eng._opt_prog, 1)
    rows.sort(key=lambda r: -r["total_ms"])
    gemm = [r for r in rows if not r["work_is_bytes"]]
    flops = sum(r["work"] for r in gemm)
    res = {
        "workload": f"GPT-2 small training step, bf16, ids [{batch}, {seq_len}], AdamW(lr 1e-3, wd 0.01)",
        "tokens_per_s": batch * seq_len / dt, "ms_per_step": dt * 1e3, "loss_after_run": eng.last_loss(),
        "parameters": eng.num_parameters(), "launches_per_step": len(plan.prog) + len(eng._opt_prog),
        "mfma_tflop_per_step": flops / 1e12,
        "mfma_kernel_ms_per_step": sum(r["total_ms"] for r in gemm),
        "mfma_util": flops / (sum(r["total_ms"] for r in gemm) * 1e-3) / PEAK_BF16_FLOPS,
        "breakdown": [{"kernel": r["name"], "ms_per_step": round(r["total_ms"], 4), "launches": r["launches"]}
                      for r in rows[:8]],
    }
    del eng, plan
    torch.cuda.empty_cache()
    return res


def interleaving(batch=8, seq_len=1024, rate_per_s=50.0, train_s=3.0):
    """BASELINE configs[4] whole: the GPT-2 small training step (bf16, ids [8, 1024], AdamW) on a stream that is
    registered with the launch queue, while batch-1 ResNet-152 forward-only requests arrive as a seeded Poisson
    process at `rate_per_s` and suspend that queue for as long as each of them runs.  Reports the request
    latencies (arrival to logits) and what the requests cost training: steps per second alone against steps
    per second beside the requests, both over about `train_s` seconds of steps."""
    import torch
    from sirius_amd.gpt2 import GPT2Engine
    from sirius_amd.resnet import ResNetEngine
    from sirius_amd.serve import ColocatedInference, poisson_arrivals
    from sirius_amd.torch_col import xsched
    train_stream, infer_stream = torch.cuda.Stream(), torch.cuda.Stream()
    xsched.register_stream(train_stream, False)
    server = None
    try:
        eng = GPT2Engine(seq_len=seq_len, dtype=torch.bfloat16, optimizer="adamw", stream=train_stream)
        eng.init_normal(0)
        g = torch.Generator(device="cuda")
        g.manual_seed(2)
        ids = torch.randint(0, eng.vocab, (batch, seq_len), device="cuda", generator=g)

        def run(seconds):
            n = 0
            with torch.cuda.stream(train_stream):
                t0 = time.perf_counter()
                while time.perf_counter() - t0 < seconds:
                    eng.forward_backward(ids)
                    eng.optimizer_step()
                    n += 1
                    if n % 8 == 0:
                        eng.synchronize()      # keep the host no more than a few steps ahead of the device
                eng.synchronize()
                return n, time.perf_counter() - t0

        run(0.2)
        n_alone, s_alone = run(train_s)
        infer = ResNetEngine(dtype=torch.bfloat16, stream=infer_stream)
        infer.init_kaiming(seed=9)
        arrivals = poisson_arrivals(rate_per_s, int(rate_per_s * train_s * 4) + 16, seed=7)
        server = ColocatedInference(infer, arrivals, batch=1, preempt=True)
        server.warm_up()
        idle = []
        for _ in range(20):                      # the request alone on the chip
            t0 = time.perf_counter()
            server._serve_one(t0)
            idle.append(server.latencies_ms.pop())
            server.service_ms.pop(), server.started_late_ms.pop()
        server.start()
        n_mixed, s_mixed = run(train_s)
        served = len(server.latencies_ms)
        server.stop()
        lat = server.summary()
        res = {
            "workload": f"GPT-2 small training, bf16, ids [{batch}, {seq_len}], AdamW, beside batch-1 ResNet-152 bf16 "
                        f"forward-only requests, Poisson {rate_per_s:g}/s (seed 7), each suspending training's launch queue",
            "requests_served": served,
            "infer_p50_ms": lat.get("p50_ms"), "infer_p99_ms": lat.get("p99_ms"), "infer_max_ms": lat.get("max_ms"),
            "infer_alone_p50_ms": sorted(idle)[len(idle) // 2],
            "train_ms_per_step_alone": s_alone / n_alone * 1e3,
            "train_ms_per_step_interleaved": s_mixed / n_mixed * 1e3,
            "train_slowdown": (s_mixed / n_mixed) / (s_alone / n_alone),
            "tokens_per_s_interleaved": batch * seq_len * n_mixed / s_mixed,
        }
        del eng, infer
        return res
    finally:
        if server is not None and server._thread is not None and server._thread.is_alive():
            server._stop.set()
            server._thread.join(10)
        xsched.resume_all_streams()
        torch.cuda.synchronize()
        xsched.unregister_stream(train_stream)
        torch.cuda.empty_cache()


def swin_b_step(batch=32, warmup=2, steps=5):
    """BASELINE configs[3]: Swin-B (87.77 M parameters), bf16 compute with fp32 master weights, images
    [32, 3, 224, 224] N(0,1), AdamW(lr 1e-3, wd 0.05), stochastic depth 0.  Reported beside the headline figure."""
    import torch
    from sirius_amd.swin import SwinEngine
    eng = SwinEngine(dtype=torch.bfloat16)
    eng.init_normal(0)
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    x = torch.randn(batch, 3, 224, 224, device="cuda", generator=g)
    y = torch.randint(0, 1000, (batch,), device="cuda", generator=g)
    for _ in range(warmup):
        eng.forward_backward(x, y)
        eng.optimizer_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.forward_backward(x, y)
        eng.optimizer_step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    plan = eng.plan(batch)
    rows = eng.ctx.profile(plan.prog, 1) + eng.ctx.profile(eng._opt_prog, 1)
    rows.sort(key=lambda r: -r["total_ms"])
    gemm = [r for r in rows if not r["work_is_bytes"]]
    flops = sum(r["work"] for r in gemm)
    res = {
        "workload": f"Swin-B training step, bf16, images [{batch}, 3, 224, 224], AdamW(lr 1e-3, wd 0.05)",
        "images_per_s": batch / dt, "ms_per_step": dt * 1e3, "loss_after_run": eng.last_loss(),
        "parameters": eng.num_parameters(), "launches_per_step": len(plan.prog) + len(eng._opt_prog),
        "mfma_tflop_per_step": flops / 1e12,
        "mfma_util": flops / (sum(r["total_ms"] for r in gemm) * 1e-3) / PEAK_BF16_FLOPS,
        "breakdown": [{"kernel": r["name"], "ms_per_step": round(r["total_ms"], 4), "launches": r["launches"]}
                      for r in rows[:8]],
    }
    del eng, plan
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-handover", action="store_true", help="skip the 64 -> 16 -> 64 handover measurement")
    ap.add_argument("--no-plugin", action="store_true", help="skip the run of the same step through the train script")
    ap.add_argument("--no-gpt2", action="store_true", help="skip the GPT-2 step measurement")
    ap.add_argument("--only-gpt2", action="store_true", help="run the GPT-2 step measurement alone (for profiling it)")
    ap.add_argument("--no-interleave", action="store_true", help="skip GPT-2 training beside Poisson ResNet-152 requests")
    ap.add_argument("--no-swin", action="store_true", help="skip the Swin-B step measurement")
    ap.add_argument("--only-swin", action="store_true", help="run the Swin-B step measurement alone (for profiling it)")
    ap.add_argument("--no-autotune", action="store_true", help="keep the library's tiling heuristic")
    ap.add_argument("--no-overlap", action="store_true", help="record weight gradients on the main lane (one stream)")
    ap.add_argument("--no-grouped", action="store_true", help="skip the extra run of the step with grouped weight gradients")
    ap.add_argument("--group-wgrad", action="store_true", help="grouped weight-gradient launches instead of one per layer")
    ap.add_argument("--wgrad-group-blocks", type=int, default=None, help="bottleneck blocks per grouped weight-gradient launch (0: a stage)")
    ap.add_argument("--wgrad-group-wgs", type=int, default=None, help="workgroups a grouped weight-gradient launch aims for")
    ap.add_argument("--wgrad-group-max-wgs", type=int, default=None, help="cap on the workgroups of a grouped weight-gradient launch")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch accumulate_kernel once over two 512 MiB buffers (reads 1 GiB, writes 1 GiB): "
                         "the known-size dispatch that scales FETCH_SIZE / WRITE_SIZE counter readings")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--profile-reps", type=int, default=2)
    ap.add_argument("--cpu-steps", type=int, default=2, help="timed CPU oracle steps (0 = skip the CPU baseline)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from sirius_amd.resnet import ResNetEngine

    assert torch.cuda.is_available(), "bench.py needs the GPU; there is no CPU fallback"
    torch.cuda.set_device(0)
    if args.only_gpt2:
        print(json.dumps({"gpt2": gpt2_step(steps=args.steps, warmup=args.warmup)}), flush=True)
        return
    if args.only_swin:
        print(json.dumps({"swin_b": swin_b_step(steps=args.steps, warmup=args.warmup)}), flush=True)
        return
    B = args.batch
    eng = ResNetEngine((3, 8, 36, 3), 1000, 64, dtype=torch.bfloat16, image_size=224, lr=0.1, momentum=0.9,
                       weight_decay=1e-4, overlap_wgrad=not args.no_overlap, autotune=not args.no_autotune,
                       group_wgrad=args.group_wgrad,
                       **({} if args.wgrad_group_blocks is None else {"wgrad_group_blocks": args.wgrad_group_blocks}),
                       **({} if args.wgrad_group_wgs is None else {"wgrad_group_wgs": args.wgrad_group_wgs}),
                       **({} if args.wgrad_group_max_wgs is None else {"wgrad_group_max_wgs": args.wgrad_group_max_wgs}))
    eng.init_kaiming(seed=0)
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    x = torch.randn(B, 3, 224, 224, device="cuda", generator=g)
    y = torch.randint(0, 1000, (B,), device="cuda", generator=g)
    torch.cuda.synchronize()

    def step():
        eng.forward_backward(x, y)
        eng.optimizer_step()

    if args.calibrate:
        from sirius_amd import ops
        a = torch.zeros(128 << 20, device="cuda")
        b = torch.ones(128 << 20, device="cuda")
        ops.grad_accumulate(eng.ctx, a, b)
        torch.cuda.synchronize()
        del a, b

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = dt / args.steps * 1e3
    plan = eng.plan(B)
    loss = plan.loss.item()

    # ---- per-kernel attribution (HIP events on the stream the kernels run on) ----
    reps = max(1, args.profile_reps)
    rows = eng.ctx.profile(plan.prog, reps) + eng.ctx.profile(eng._opt_prog, reps)
    rows.sort(key=lambda r: -r["total_ms"])
    total_ms = sum(r["total_ms"] for r in rows) / reps
    conv = [r for r in rows if r["name"].startswith(("igemm_kernel", "igemm2_kernel", "igemm3_kernel", "wgrad_kernel"))]
    conv_ms = sum(r["total_ms"] for r in conv) / reps
    conv_flops = sum(r["work"] for r in conv) / reps
    top = rows[0]
    alone_s = top["total_ms"] / top["launches"] * 1e-3
    # The leader's launches INSIDE the step, both lanes running: begin / end timestamps of each of its launches in
    # plain replays of the step's program (what a kernel trace of this run shows); the figures below are quoted
    # on that duration, the one-at-a-time replay is kept beside them as `alone`.
    in_step_us, in_step_n = eng.ctx.time_kernel(plan.prog, top["name"], max(3, reps))
    if in_step_n == 0:
        in_step_us, in_step_n = eng.ctx.time_kernel(eng._opt_prog, top["name"], max(3, reps))
    per_launch_s = in_step_us * 1e-6 if in_step_n else alone_s
    # A kernel annotated with flops also states its algorithmic bytes: the roof that binds is the one that
    # alone would need more time (flops / MFMA peak against bytes / HBM bandwidth), and `frac` is quoted on it.
    flops = 0.0 if top["work_is_bytes"] else top["work"] / top["launches"]
    nbytes = top["bytes"] / top["launches"]
    hbm_bound = nbytes / PEAK_HBM_BYTES >= flops / PEAK_BF16_FLOPS
    peak = PEAK_HBM_BYTES if hbm_bound else PEAK_BF16_FLOPS
    work = nbytes if hbm_bound else flops
    achieved = work / per_launch_s
    roofline = {
        "kernel": top["name"],
        "bound": "hbm" if hbm_bound else "mfma",
        "achieved": achieved / (1e9 if hbm_bound else 1e12),
        "peak": peak / (1e9 if hbm_bound else 1e12),
        "unit": "GB/s" if hbm_bound else "TFLOP/s",
        "frac": achieved / peak,
        "traffic": MEASURED_TRAFFIC_MIB[top["name"]] * 2 ** 20 if top["name"] in MEASURED_TRAFFIC_MIB else None,
        "traffic_unit": "bytes per launch (HBM, rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated)",
        "algorithmic_bytes_per_launch": nbytes,
        "algorithmic_flops_per_launch": flops,
        "frac_of_other_roof": (flops / per_launch_s / PEAK_BF16_FLOPS) if hbm_bound else (nbytes / per_launch_s / PEAK_HBM_BYTES),
        "avg_launch_us": per_launch_s * 1e6,
        "measured": "inside the step (both lanes running): HIP start / stop events of each launch of this kernel, "
                    "on the stream it is launched on" if in_step_n else "one launch at a time (HIP events between launches)",
        "launches_per_step": top["launches"] // reps,
        "share_of_step_kernel_time": top["total_ms"] / reps / total_ms,
        "alone": {"avg_launch_us": alone_s * 1e6, "achieved": work / alone_s / (1e9 if hbm_bound else 1e12),
                  "frac": work / alone_s / peak,
                  "measured": "the same launches replayed one at a time with a HIP event between any two"},
        "profile": PROFILE_FILE,
    }
    breakdown = [{"kernel": r["name"], "ms_per_step": round(r["total_ms"] / reps, 4), "launches": r["launches"] // reps,
                  ("GB/s" if r["work_is_bytes"] else "TFLOP/s"):
                      round(r["work"] / (r["total_ms"] * 1e-3) / (1e9 if r["work_is_bytes"] else 1e12), 2)
                  if r["total_ms"] > 0 else None,
                  **({} if r["work_is_bytes"] or r["total_ms"] <= 0 else
                     {"GB/s": round(r["bytes"] / (r["total_ms"] * 1e-3) / 1e9, 2)})}
                 for r in rows[:24]]

    out = {
        "metric": METRIC,
        "value": B * args.steps / dt,
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"ResNet-152 training step, bf16 compute with fp32 master weights, batch {B} @ 3x224x224 "
                               "N(0,1), labels uniform [0,1000), SGD-momentum(0.9, lr 0.1, wd 1e-4), Kaiming-normal init "
                               "(BASELINE configs[1])",
                   "global_batch": B, "launches_per_step": len(plan.prog) + len(eng._opt_prog)},
        "loss_after_run": loss,
        "roofline": roofline,
        "conv_mfma_util": conv_flops / (conv_ms * 1e-3) / PEAK_BF16_FLOPS if conv_ms > 0 else None,
        "conv_ms_per_step": conv_ms,
        "conv_tflop_per_step": conv_flops / 1e12,
        "kernel_ms_per_step": total_ms,
        "breakdown": breakdown,
    }
    if not args.no_grouped and not args.group_wgrad:
        try:
            out["grouped_wgrad"] = grouped_wgrad_step(B, x, y, max(4, args.steps // 2), 2, eng._tile_cache)
        except Exception as e:
            out["grouped_wgrad"] = {"error": repr(e)}
    if args.cpu_steps > 0:
        out["cpu_baseline"] = cpu_baseline(B, args.cpu_steps)
    else:
        out["cpu_baseline"] = None
    del eng, plan, x, y
    torch.cuda.empty_cache()
    if not args.no_plugin:
        try:
            out["value_through_plugin"] = through_plugin(B)
        except Exception as e:
            out["value_through_plugin"] = {"error": repr(e)}
    if not args.no_handover:
        try:
            out["handover"] = handover(B)
        except Exception as e:  # the headline figure stands on its own; say what went wrong
            out["handover"] = {"error": repr(e)}
        try:    # the reference's page size: 32 MB pages, the reply first, the unmapping right behind it
            out["handover_32mb_pages"] = handover(B, pool_gb=48, page_mb=32, lazy=True)
        except Exception as e:
            out["handover_32mb_pages"] = {"error": repr(e)}
    if not args.no_gpt2:
        try:
            out["gpt2"] = gpt2_step()
        except Exception as e:
            out["gpt2"] = {"error": repr(e)}
    if not args.no_gpt2 and not args.no_interleave:
        try:
            out["gpt2"]["interleaving"] = interleaving()
        except Exception as e:
            out["gpt2"]["interleaving"] = {"error": repr(e)}
    if not args.no_swin:
        try:
            out["swin_b"] = swin_b_step()
        except Exception as e:
            out["swin_b"] = {"error": repr(e)}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
