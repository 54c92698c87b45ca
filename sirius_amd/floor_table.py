"""Per-launch roofline table of a recorded training step.

For every launch of the step: the work it states (algorithmic flops and bytes), the time either roof of the chip
would need for it alone (flops / 2.5 PFLOP/s bf16 MFMA, bytes / 8 TB/s HBM), the larger of the two as its floor,
the time it takes alone on the chip (HIP events around it in a one-at-a-time replay), and the gap.  Summed per
phase (forward / backward), per stage of the network and per kernel family, next to the wall time of the step
as it runs (two lanes): where the step's time goes.

    python -m sirius_amd.floor_table [--batch 64] [--reps 3] [--out floor_table.txt]
"""
import argparse
import collections
import re
import sys
import time

PEAK_FLOPS = 2.5e15
PEAK_BYTES = 8.0e12


def family(name):
    """Kernel family of a launch: what the kernel does, without its tiling."""
    if name.startswith(("igemm2_kernel", "igemm3_kernel", "igemm_kernel")):
        return "conv data gradient" if ",dgrad" in name else "conv forward"
    if name.startswith("wgrad"):
        return "conv weight gradient"
    if name.startswith("splitk"):
        return "split reduction"
    direction = "bwd" if ",bwd" in name else "fwd"
    if name.startswith(("bn_fin_apply", "bn_acc_apply")):
        return f"bn coefficients+apply {direction}"
    if name.startswith("bn_apply"):
        return f"bn apply {direction}"
    if "finalize" in name:
        return "bn finalize"
    return name.split("<")[0]


def stage_of(layer):
    m = re.match(r"layer(\d)", layer)
    return f"stage {m.group(1)}" if m else "stem/head"


def build_rows(eng, plan, reps):
    stats = eng.ctx.profile_launches(plan.prog, reps)
    # marks: (launch index one past the layer, phase, layer) in program order
    marks = sorted(plan.marks)
    rows, mi = [], 0
    for i, s in enumerate(stats):
        while mi < len(marks) and marks[mi][0] <= i:
            mi += 1
        phase, layer = (marks[mi][1], marks[mi][2]) if mi < len(marks) else ("bwd", "tail")
        if not s["name"]:
            continue
        t_flop, t_byte = s["flops"] / PEAK_FLOPS, s["bytes"] / PEAK_BYTES
        rows.append(dict(i=i, phase=phase, layer=layer, kernel=s["name"], lane=s["lane"], wgs=s["workgroups"],
                         gflop=s["flops"] / 1e9, mb=s["bytes"] / 1e6, floor_us=max(t_flop, t_byte) * 1e6,
                         bound="mfma" if t_flop >= t_byte else "hbm", us=s["ms"] * 1e3))
    return rows


def summarise(rows, key):
    agg = collections.OrderedDict()
    for r in rows:
        a = agg.setdefault(key(r), dict(n=0, us=0.0, floor=0.0, gflop=0.0, mb=0.0))
        a["n"] += 1
        a["us"] += r["us"]
        a["floor"] += r["floor_us"]
        a["gflop"] += r["gflop"]
        a["mb"] += r["mb"]
    return agg


def fmt_summary(title, agg):
    out = [title, f"{'':44s} {'launches':>8s} {'alone ms':>9s} {'floor ms':>9s} {'gap ms':>8s} {'us/launch':>9s} "
                  f"{'TFLOP/s':>8s} {'TB/s':>6s}"]
    for k, a in agg.items():
        s = a["us"] * 1e-6
        out.append(f"{str(k):44s} {a['n']:8d} {a['us'] / 1e3:9.3f} {a['floor'] / 1e3:9.3f} "
                   f"{(a['us'] - a['floor']) / 1e3:8.3f} {a['us'] / a['n']:9.1f} "
                   f"{a['gflop'] / 1e3 / s if s else 0:8.0f} {a['mb'] / 1e6 / s if s else 0:6.2f}")
    return "\n".join(out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--reps", type=int, default=3)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--no-autotune", action="store_true")
    ap.add_argument("--out", default="")
    args = ap.parse_args()
    import torch
    from sirius_amd.resnet import ResNetEngine
    assert torch.cuda.is_available(), "needs the GPU"
    B = args.batch
    eng = ResNetEngine((3, 8, 36, 3), 1000, 64, dtype=torch.bfloat16, image_size=224, autotune=not args.no_autotune)
    eng.init_kaiming(0)
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    x = torch.randn(B, 3, 224, 224, device="cuda", generator=g)
    y = torch.randint(0, 1000, (B,), device="cuda", generator=g)
    for _ in range(5):
        eng.forward_backward(x, y)
        eng.optimizer_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        eng.forward_backward(x, y)
        eng.optimizer_step()
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) / args.steps * 1e3
    plan = eng.plan(B)
    # forward alone, as it runs (one lane): wall time of the first n_forward launches
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        eng.ctx.run(plan.prog, 0, plan.n_forward)
    eng.ctx.synchronize()
    fwd_ms = (time.perf_counter() - t0) / args.steps * 1e3
    rows = build_rows(eng, plan, args.reps)
    main_rows = [r for r in rows if r["lane"] == 0]
    text = [f"ResNet-152 bf16 batch {B} training step on MI355X: {step_ms:.3f} ms per step as it runs (two lanes), "
            f"forward part alone {fwd_ms:.3f} ms; {len(rows)} launches in the forward/backward program "
            f"({len(main_rows)} on the main lane).",
            "alone = HIP events around the launch in a one-at-a-time replay (includes the launch-to-launch floor of "
            "about 5 us); floor = max(flops / 2.5 PFLOP/s, algorithmic bytes / 8 TB/s).", ""]
    text.append(fmt_summary("main lane by phase", summarise(main_rows, lambda r: r["phase"])))
    text.append("")
    text.append(fmt_summary("main lane by phase and stage", summarise(main_rows, lambda r: (r["phase"], stage_of(r["layer"])))))
    text.append("")
    text.append(fmt_summary("main lane by phase and kernel family", summarise(main_rows, lambda r: (r["phase"], family(r["kernel"])))))
    text.append("")
    text.append(fmt_summary("second lane by kernel family", summarise([r for r in rows if r["lane"] == 1], lambda r: family(r["kernel"]))))
    text.append("")
    text.append(fmt_summary("stage 3, main lane, by layer kind and kernel family",
                            summarise([r for r in main_rows if r["layer"].startswith("layer3.") and not r["layer"].startswith("layer3.0.")],
                                      lambda r: (r["phase"], r["layer"].split(".")[-1], family(r["kernel"])))))
    text.append("")
    text.append("every launch (program order)")
    text.append(f"{'#':>5s} {'ph':3s} {'layer':22s} {'lane':>4s} {'wgs':>6s} {'GFLOP':>8s} {'MB':>8s} {'bound':>5s} "
                f"{'floor us':>8s} {'alone us':>8s}  kernel")
    for r in rows:
        text.append(f"{r['i']:5d} {r['phase']:3s} {r['layer']:22s} {r['lane']:4d} {r['wgs']:6d} {r['gflop']:8.2f} "
                    f"{r['mb']:8.2f} {r['bound']:>5s} {r['floor_us']:8.2f} {r['us']:8.2f}  {r['kernel']}")
    text = "\n".join(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text + "\n")
        print("\n".join(text.split("\n")[:70]))
    else:
        print(text)


if __name__ == "__main__":
    sys.exit(main())
