"""Whole-step parity: the HIP ResNet engine against the CPU oracle step (oracle/resnet.py)
on identical seeded weights and inputs, 3 optimizer steps, SGD(lr 0.1, momentum 0.9,
weight decay 1e-4), BatchNorm in training mode.

Two kinds of bound are used, and each test says which:

* DIRECT -- fp32 rtol 1e-3 / bf16 rtol 2e-2 against the CPU step, on the loss and, per
  parameter tensor relative to that tensor's largest oracle magnitude, on every gradient,
  every updated weight and every BatchNorm running statistic.  Used wherever the step is
  well conditioned, and for every layer of ResNet-152 at its real shapes when the layer is
  fed the oracle's own activations (teacher forcing).

* ANCHORED -- for the end-to-end step wherever it is ill conditioned.  At random init with
  lr 0.1 it is: the CPU oracle run in fp32 differs from the same oracle run in fp64 by
  10-35 % in the ResNet-152 gradients after ONE step at batch 4, by more than 100 % from
  the second step on, and the CPU bf16-autocast gradients are uncorrelated with fp64 from the
  first step (all measured, see the table each test prints), so no implementation of that
  precision can sit within rtol of another one.  Those tests anchor on the fp64 oracle and
  require the HIP path to be as close to it as the CPU path of the same precision is
  (factor 2), and to meet the DIRECT bound outright on the steps where the CPU path does.
"""
import pytest
import torch

from oracle import nn_ops as O
from oracle import resnet as R

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2}


def rel_err(got, ref):
    ref = ref.float()
    return ((got.float().cpu() - ref).abs().max() / (ref.abs().max() + 1e-12)).item()


def worst(got_dict, ref_dict, keys):
    w, name = 0.0, None
    for k in keys:
        e = rel_err(got_dict[k], ref_dict[k])
        assert e == e, f"{k}: NaN"
        if e > w:
            w, name = e, k
    return w, name


def median_err(got_dict, ref_dict, keys):
    errs = sorted(rel_err(got_dict[k], ref_dict[k]) for k in keys)
    return errs[len(errs) // 2]


def engine_steps(eng, x, y, steps, micro_batches):
    """The engine's side of oracle.resnet.train_steps: per step (losses, grads at the optimizer step)."""
    batch = x.shape[0]
    mb = batch // micro_batches
    xd, yd = x.cuda(), y.cuda()
    out = []
    for _ in range(steps):
        losses = []
        for i in range(micro_batches):
            plan, cut = eng.forward_backward(xd[i * mb:(i + 1) * mb].contiguous(),
                                             yd[i * mb:(i + 1) * mb].contiguous(), loss_scale=mb / batch)
            assert not cut
            losses.append(plan.loss.item())
            if micro_batches > 1:
                eng.accumulate()
        grads = eng.grads_dict(use_global=micro_batches > 1)
        eng.optimizer_step(use_global=micro_batches > 1)
        out.append((losses, grads))
    return out


def run_parity(depths, width, classes, image, batch, dtype, steps, micro_batches=1, direct_steps=0, **engine_kw):
    """HIP path and CPU path of the same precision on the same seeded weights and inputs, both
    measured against the fp64 oracle.  Per step: the loss is held to the DIRECT bound against
    the CPU path while the CPU path itself is that close to fp64; the worst and the median
    per-tensor gradient error of the HIP path must be within max(rtol, 2 x the CPU path's).
    The first `direct_steps` steps must in addition meet the DIRECT bound outright
    (gradients within rtol of the CPU path)."""
    from sirius_amd.resnet import ResNetEngine
    rtol = RTOL[dtype]
    x, y = R.make_batch(batch, image, classes, seed=0)
    m64 = R.make_model(depths, classes, width, seed=0).double()
    mcpu = R.make_model(depths, classes, width, seed=0)
    eng = ResNetEngine(depths, classes, width, dtype=dtype, image_size=image, **engine_kw)
    eng.load_state_dict(mcpu.state_dict())
    assert eng.num_parameters() == sum(p.numel() for p in mcpu.parameters())
    names = [k for k, _ in mcpu.named_parameters()]
    h64 = R.train_steps(m64, x.double(), y, steps, micro_batches=micro_batches)
    hcpu = R.train_steps(mcpu, x, y, steps, micro_batches=micro_batches, autocast_bf16=(dtype == torch.bfloat16))
    got = engine_steps(eng, x, y, steps, micro_batches)
    decorrelated = False
    print("step | loss fp64 / cpu / hip | median grad err cpu / hip | worst grad err cpu / hip | hip vs cpu worst")
    for s in range(steps):
        l64, lcpu, lgot = h64[s][0], hcpu[s][0], got[s][0]
        g_cpu, g_got = median_err(hcpu[s][1], h64[s][1], names), median_err(got[s][1], h64[s][1], names)
        w_cpu, _ = worst(hcpu[s][1], h64[s][1], names)
        w_got, wname = worst(got[s][1], h64[s][1], names)
        d_got, dname = worst(got[s][1], hcpu[s][1], names)
        print(s, l64, lcpu, lgot, f"{g_cpu:.3e} {g_got:.3e} | {w_cpu:.3e} {w_got:.3e} ({wname}) | {d_got:.3e} ({dname})",
              flush=True)
        for a, b, c in zip(lgot, lcpu, l64):
            assert a == a and abs(a) < 1e6, f"step {s}: loss {a}"
            tol = max(rtol * abs(c), 2.0 * abs(b - c))
            # once the CPU path's own gradients have decorrelated from fp64 (median error
            # above one half) the weights of the three runs are unrelated: only finiteness
            # of the loss can be asked of the following steps
            if not decorrelated:
                assert abs(a - c) <= tol, f"step {s}: loss {a} vs fp64 {c} (CPU path {b})"
        if decorrelated:
            # weights already unrelated: gradients of this step are finite (checked by worst()), no more
            continue
        decorrelated = g_cpu >= 0.5
        assert g_got <= max(rtol, 2.0 * g_cpu), f"step {s}: median gradient error {g_got:.3e} vs CPU path {g_cpu:.3e}"
        assert w_got <= max(rtol, 2.0 * w_cpu), f"step {s}: worst gradient error {w_got:.3e} ({wname}) vs CPU {w_cpu:.3e}"
        if s < direct_steps:
            assert d_got <= rtol, f"step {s}: gradient {dname} off the CPU path by {d_got:.3e} (DIRECT bound {rtol})"
    sd, ref_sd, cpu_sd = eng.state_dict(), m64.state_dict(), mcpu.state_dict()
    keys = names + [k for k in ref_sd if k.endswith("running_mean") or k.endswith("running_var")]
    w_cpu, _ = worst(cpu_sd, ref_sd, keys)
    w_got, wname = worst(sd, ref_sd, keys)
    print("final weights / running stats: worst err cpu", w_cpu, "hip", w_got, wname, flush=True)
    if not decorrelated:
        assert w_got <= max(rtol, 2.0 * w_cpu), \
            f"updated weight / statistic {wname} off by {w_got:.3e} (CPU path {w_cpu:.3e})"
    if direct_steps >= steps:
        d, dname = worst(sd, cpu_sd, keys)
        assert d <= rtol, f"updated weight / statistic {dname} off the CPU path by {d:.3e}"


def test_fp32_four_stages_direct():
    """3 steps, every gradient / weight / statistic within 1e-3 of the CPU step"""
    run_parity((1, 1, 1, 1), 16, 16, 64, 4, torch.float32, 3, direct_steps=3)


@pytest.mark.parametrize("blocks,wgs,cap", [(0, 1024, 0), (1, 8, 0), (2, 300, 16)])
def test_fp32_grouped_weight_gradients(blocks, wgs, cap):
    """the weight gradients of a stage (or of every `blocks` blocks) as one launch over a table, split to about
    `wgs` workgroups, optionally capped: same bounds as the layer-by-layer plan"""
    run_parity((2, 2, 2), 16, 16, 64, 8, torch.float32, 3, direct_steps=2, group_wgrad=True, wgrad_group_blocks=blocks,
               wgrad_group_wgs=wgs, wgrad_group_max_wgs=cap)


def test_fp32_identity_blocks():
    run_parity((2, 2, 2), 16, 16, 64, 8, torch.float32, 3, direct_steps=2)


def test_fp32_micro_batches():
    """global batch 16 as 4 micro-batches of 4: scaled losses, accumulated gradients, one step
    per global batch (pytorch/torch_col/dynamic_batch.py:112-153, accumulate.py:20-47)"""
    run_parity((1, 2, 1), 16, 16, 64, 16, torch.float32, 3, micro_batches=4, direct_steps=1)


def test_fp32_full_width_shallow():
    """the real channel widths (64..2048) and image size, one block per stage"""
    run_parity((1, 1, 1, 1), 64, 1000, 224, 4, torch.float32, 2)


def test_bf16_four_stages():
    run_parity((1, 1, 1, 1), 16, 16, 64, 8, torch.bfloat16, 3)


def test_resnet152_fp32_batch4():
    """BASELINE configs[0]: ResNet-152, fp32, batch 4 @ 224, 3 steps"""
    run_parity((3, 8, 36, 3), 64, 1000, 224, 4, torch.float32, 3)


def test_resnet152_bf16_batch8():
    """the bf16 path (fp32 master weights) at a batch the CPU oracle can afford"""
    run_parity((3, 8, 36, 3), 64, 1000, 224, 8, torch.bfloat16, 2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_teacher_forced_resnet152_layers(ctx, dtype):
    """Every convolution and BatchNorm of ResNet-152 at its real shape (batch 4 @ 224), fed the
    oracle's own activations and output gradients: forward, data gradient, weight gradient,
    BN forward / backward -- DIRECT bound per layer."""
    from sirius_amd import ops
    rtol = RTOL[dtype]
    model = R.make_model((3, 8, 36, 3), 1000, 64, seed=0)
    x, y = R.make_batch(4, 224, 1000, seed=0)
    cap = {}

    def fwd_hook(name):
        def hook(mod, inp, out):
            cap[name] = [inp[0].detach(), None]
            out.register_hook(lambda g: cap[name].__setitem__(1, g.detach()))
        return hook

    mods = {n: m for n, m in model.named_modules() if isinstance(m, (torch.nn.Conv2d, torch.nn.BatchNorm2d))}
    for n, m in mods.items():
        m.register_forward_hook(fwd_hook(n))
    model.train()
    torch.nn.functional.cross_entropy(model(x), y).backward()
    nhwc = lambda t: t.permute(0, 2, 3, 1).contiguous()
    worst_seen = {}

    def check(kind, name, got, ref):
        e = rel_err(got, ref)
        assert e <= rtol, f"{kind} {name}: {e:.3e} > {rtol}"
        worst_seen[kind] = max(worst_seen.get(kind, 0.0), e)

    code = ops.dtype_code(torch.empty(0, dtype=dtype))
    for n, m in mods.items():
        xin, gout = cap[n]
        if isinstance(m, torch.nn.Conv2d):
            xs = nhwc(xin)
            if xs.shape[3] < 8:
                xs = torch.nn.functional.pad(xs, (0, 8 - xs.shape[3]))
            w = m.weight.detach().permute(0, 2, 3, 1).contiguous()
            if w.shape[3] < 8:
                w = torch.nn.functional.pad(w, (0, 8 - w.shape[3]))
            xs, w, dy = xs.to(dtype), w.to(dtype), nhwc(gout)
            dy = (dy / dy.abs().max()).to(dtype)
            st, pad = m.stride[0], m.padding[0]
            y_ref = O.conv2d_fwd(xs, w, st, pad)
            yd = torch.empty(y_ref.shape, dtype=dtype, device="cuda")
            ops.conv2d_fwd(ctx, xs.cuda(), w.cuda(), yd, st, pad)
            check("conv_fwd", n, yd, y_ref)
            dx = torch.empty(xs.shape, dtype=dtype, device="cuda")
            ops.conv2d_dgrad(ctx, dy.cuda(), ops.filter_transpose(ctx, w.cuda()), dx, st, pad)
            check("conv_dgrad", n, dx, O.conv2d_dgrad(dy, w, xs.shape, st, pad))
            K, Rr, Ss, C = w.shape
            sp = ops.conv2d_wgrad_splits(xs, K, Rr, Ss, st, pad)
            ws = torch.empty(max(1, ops.conv2d_wgrad_workspace_bytes(code, K, Rr, Ss, C, sp) // 4), device="cuda")
            dw = torch.empty(w.shape, dtype=torch.float32, device="cuda")
            ops.conv2d_wgrad(ctx, xs.cuda(), dy.cuda(), dw, st, pad, workspace=ws)
            check("conv_wgrad", n, dw, O.conv2d_wgrad(xs, dy, w.shape, st, pad))
        else:
            C = xin.shape[1]
            xs = nhwc(xin).to(dtype)
            dy = nhwc(gout)
            dy = (dy / dy.abs().max()).to(dtype)
            gamma, beta = m.weight.detach().clone(), m.bias.detach().clone()
            rm, rv = torch.zeros(C), torch.ones(C)
            y_ref, mean_ref, invstd_ref = O.bn_fwd_train(xs, gamma, beta, rm, rv)
            rows = xs.numel() // C
            yd = torch.empty(xs.shape, dtype=dtype, device="cuda")
            sm, si = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
            rmd, rvd = torch.zeros(C, device="cuda"), torch.ones(C, device="cuda")
            ws = torch.empty(ops.bn_workspace_bytes(code, rows, C) // 4, device="cuda")
            ops.bn_fwd_train(ctx, xs.cuda(), yd, gamma.cuda(), beta.cuda(), rmd, rvd, sm, si, ws)
            check("bn_fwd", n, yd, y_ref)
            check("bn_running_var", n, rvd, rv)
            dx_ref, dg_ref, db_ref = O.bn_bwd(dy, xs, gamma)
            dx = torch.empty(xs.shape, dtype=dtype, device="cuda")
            dg, db = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
            ops.bn_bwd(ctx, dy.cuda(), xs.cuda(), dx, gamma.cuda(), sm, si, dg, db, ws)
            check("bn_dx", n, dx, dx_ref)
            check("bn_dgamma", n, dg, dg_ref)
            check("bn_dbeta", n, db, db_ref)
        torch.cuda.synchronize()
    print(dtype, worst_seen, flush=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("options", [
    dict(fuse_bn_stats=False, fuse_bn_bwd=False, overlap_wgrad=False),   # every BatchNorm pass as its own launch
    dict(fuse_bn_bwd=False),
    dict(overlap_wgrad=False),
    dict(fuse_bn_finalize=True),                                         # coefficients inside the convolutions
    dict(autotune=True),
])
def test_engine_options_agree(dtype, options):
    """Where a reduction is taken (own pass, convolution epilogue, last workgroup) and on which lane a kernel
    runs changes summation order at most.  One step of each variant against the default engine: same loss, and
    per-tensor gradient differences at rounding level in the median.  The worst tensor gets a loose bound:
    a last-bit difference in a BatchNorm output flips the ReLU of an element that sits at zero (seen: one
    element of 262144 at 2e-6), and the gradient of the layers below changes by a whole term."""
    from sirius_amd.resnet import ResNetEngine
    depths, width, classes, image, batch = (1, 2, 1, 1), 64, 16, 64, 8
    x, y = R.make_batch(batch, image, classes, seed=3)
    sd = R.make_model(depths, classes, width, seed=3).state_dict()
    outs = []
    for kw in ({}, options):
        eng = ResNetEngine(depths, classes, width, dtype=dtype, image_size=image, **kw)
        eng.load_state_dict(sd)
        outs.append(engine_steps(eng, x, y, 1, 1) + [eng.state_dict()])
    names = list(outs[0][0][1])
    assert abs(outs[0][0][0][0] - outs[1][0][0][0]) <= (1e-5 if dtype == torch.float32 else 2e-2) * abs(outs[0][0][0][0])
    # a flip in the first stage shifts every gradient below it by ~1e-3 of its size: the median bound is the
    # path's tolerance, not rounding level
    med = median_err(outs[1][0][1], outs[0][0][1], names)
    w, name = worst(outs[1][0][1], outs[0][0][1], names)
    print(f"median {med:.3e} worst {w:.3e} ({name})", flush=True)
    if dtype == torch.bfloat16:
        # in bf16 a last-bit difference of the statistics moves stored activations by whole bf16 steps and
        # the two runs drift apart layer by layer (as two CPU bf16 runs do): only sanity is asked here
        assert med <= 0.5
        return
    assert med <= 2e-3
    assert w <= 5e-2, f"gradient {name} differs by {w:.3e}"
    w, name = worst(outs[1][1], outs[0][1], list(outs[0][1]))
    assert w <= 5e-2, f"weights / statistics: {name} differs by {w:.3e}"
