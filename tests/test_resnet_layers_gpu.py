"""Layer-local parity of the ResNet-152 engine AS THE BENCHMARK RUNS IT: the real plan (tilings picked by
measurement, BatchNorm statistics in the forward epilogues, ReLU gate + BatchNorm-backward sums in the
data-gradient epilogues, finalize + apply in one launch, weight gradients on the second lane), bf16 with fp32
master weights, at batch 8 and at the benchmark's batch 64.

One training step runs on the GPU.  Then, for every layer of the network, the layer's input is read back from
the plan's own buffers, that ONE layer is recomputed on the CPU with oracle/nn_ops.py from exactly that input,
and the engine's output buffer is held to the bf16 bound (2e-2 of the largest magnitude of the oracle tensor):
forward convolutions, BatchNorm statistics / outputs / running statistics, pools (argmax indices bit for bit),
logits and loss, and in the backward every data gradient, weight gradient, BatchNorm input gradient and
BatchNorm parameter gradient.  One layer deep, so the chaos of the 152-layer step at random init (CPU fp32
against CPU fp64 differ by 10-35 % end to end) does not enter; what is checked is every kernel of the timed
step at its real shape, on real data, with the tiling the step uses.
"""
import pytest
import torch

from oracle import nn_ops as O

pytestmark = pytest.mark.gpu

TOL = 2e-2


def _f(t):
    return t.detach().float().cpu()


class _Check:
    def __init__(self):
        self.worst = {}
        self.count = 0

    def __call__(self, kind, name, got, ref, tol=TOL):
        got, ref = _f(got), ref.float()
        assert got.shape == ref.shape, (kind, name, got.shape, ref.shape)
        assert torch.isfinite(got).all(), f"{kind} {name}: not finite"
        e = ((got - ref).abs().max() / (ref.abs().max() + 1e-20)).item()
        assert e <= tol, f"{kind} {name}: {e:.3e} > {tol}"
        if e > self.worst.get(kind, (0.0, ""))[0]:
            self.worst[kind] = (e, name)
        self.count += 1


def _layer_local(batch, depths=(3, 8, 36, 3), width=64, classes=1000, image=224, autotune=True):
    from sirius_amd.resnet import ResNetEngine
    eng = ResNetEngine(depths, classes, width, dtype=torch.bfloat16, image_size=image, autotune=autotune,
                       retain_gradients=True)
    assert eng.fuse_bn_stats and eng.fuse_bn_bwd and eng.overlap_wgrad and not eng.fuse_bn_finalize
    eng.init_kaiming(seed=5)
    g = torch.Generator()
    g.manual_seed(17)
    x = torch.randn(batch, 3, image, image, generator=g)
    y = torch.randint(0, classes, (batch,), generator=g)
    rm0, rv0 = _f(eng.running_mean), _f(eng.running_var)
    plan, cut = eng.forward_backward(x.cuda(), y.cuda())
    assert not cut
    eng.synchronize()
    torch.cuda.synchronize()
    T = plan.tensors
    head = T["head"]
    nbn = eng.running_mean.numel()
    save = _f(plan.bn_save)
    rm1, rv1 = _f(eng.running_mean), _f(eng.running_var)
    chk = _Check()

    def w_of(c):                       # the filter the kernels read (bf16 shadow), [K,R,S,C]
        return _f(eng._w(c.name + ".weight"))

    def gamma_beta(name):
        return _f(eng._view(eng.params, name + ".weight")), _f(eng._view(eng.params, name + ".bias"))

    def grad_of(name):
        return _f(eng._view(eng.grads, name))

    def conv_fwd(c, xin, z):
        chk("conv_fwd", c.name, z, O.conv2d_fwd(_f(xin), w_of(c), c.stride, c.pad))

    def bn_fwd(name, z, yout, residual=None, relu=True):
        o, ch = eng._bn_off[name]
        gm, bt = gamma_beta(name)
        rm, rv = rm0[o:o + ch].clone(), rv0[o:o + ch].clone()
        y_ref, mean, invstd = O.bn_fwd_train(_f(z), gm, bt, rm, rv, eng.bn_momentum, eng.bn_eps,
                                             residual=None if residual is None else _f(residual), relu=relu)
        chk("bn_mean", name, save[o:o + ch], mean, tol=1e-3)
        chk("bn_invstd", name, save[nbn + o:nbn + o + ch], invstd, tol=1e-3)
        chk("bn_running_mean", name, rm1[o:o + ch], rm, tol=1e-3)
        chk("bn_running_var", name, rv1[o:o + ch], rv, tol=1e-3)
        # an element whose normalised value is within rounding of zero sits on either side of the ReLU
        chk("bn_fwd", name, yout, y_ref)

    def bn_bwd(name, g_eff, z, dz):
        gm, _ = gamma_beta(name)
        dx, dg, db = O.bn_bwd(g_eff, _f(z), gm, eng.bn_eps)
        chk("bn_dx", name, dz, dx)
        chk("bn_dgamma", name, grad_of(name + ".weight"), dg)
        chk("bn_dbeta", name, grad_of(name + ".bias"), db)

    def conv_wgrad(c, xin, dy):
        wshape = eng.spec[c.name + ".weight"].store_shape
        chk("conv_wgrad", c.name, grad_of(c.name + ".weight"), O.conv2d_wgrad(_f(xin), _f(dy), wshape, c.stride, c.pad))

    def conv_dgrad(c, dy, xin):
        return O.conv2d_dgrad(_f(dy), w_of(c), tuple(xin.shape), c.stride, c.pad)

    # ---------------- forward ----------------
    xs = torch.nn.functional.pad(x.permute(0, 2, 3, 1), (0, 8 - 3)).to(torch.bfloat16)
    assert torch.equal(_f(head["x0"]), xs.float()), "image conversion NCHW fp32 -> NHWC bf16, channels padded to 8"
    conv_fwd(eng.stem, head["x0"], head["z0"])
    bn_fwd("bn1", head["z0"], head["a0"])
    p_ref, idx_ref = O.maxpool_fwd(_f(head["a0"]), 3, 2, 1)
    assert torch.equal(_f(head["p0"]), p_ref), "max-pool values"
    assert torch.equal(head["p0_idx"].cpu().long(), idx_ref.long()), "max-pool argmax indices"
    for blk in eng.blocks:
        t, pre = T[blk.prefix], blk.prefix
        conv_fwd(blk.c1, t["x"], t["z1"])
        bn_fwd(pre + ".bn1", t["z1"], t["a1"])
        conv_fwd(blk.c2, t["a1"], t["z2"])
        bn_fwd(pre + ".bn2", t["z2"], t["a2"])
        conv_fwd(blk.c3, t["a2"], t["z3"])
        if blk.cd is not None:
            conv_fwd(blk.cd, t["x"], t["zd"])
            bn_fwd(pre + ".downsample.1", t["zd"], t["idn"], relu=False)
        bn_fwd(pre + ".bn3", t["z3"], t["out"], residual=t["idn"], relu=True)
    last = T[eng.blocks[-1].prefix]["out"]
    chk("avgpool", "avgpool", head["pooled"], O.avgpool_fwd(_f(last)))
    fcw, fcb = _f(eng._w("fc.weight")).view(classes, -1), _f(eng._view(eng.params, "fc.bias"))
    chk("fc", "fc", head["logits"], _f(head["pooled"]) @ fcw.t() + fcb)
    rows, mean, dlog = O.softmax_ce(_f(head["logits"]), y)
    chk("loss", "loss", plan.loss, mean.reshape(1), tol=1e-4)
    chk("dlogits", "dlogits", head["dlogits"], dlog)

    # ---------------- backward ----------------
    dl = _f(head["dlogits"])
    chk("fc_wgrad", "fc.weight", grad_of("fc.weight").view(classes, -1), dl.t() @ _f(head["pooled"]))
    chk("fc_bgrad", "fc.bias", grad_of("fc.bias"), dl.sum(0))
    chk("fc_dgrad", "fc", head["g_pooled"], dl @ fcw)
    chk("avgpool_bwd", "avgpool", head["g_feat"], O.avgpool_bwd(_f(head["g_pooled"]), tuple(last.shape)))
    for blk in reversed(eng.blocks):
        t, pre = T[blk.prefix], blk.prefix
        relu = lambda a: (_f(a) > 0).float()
        G = _f(t["g_out"]) if t["g_out_gated"] else _f(t["g_out"]) * relu(t["out"])
        bn_bwd(pre + ".bn3", G, t["z3"], t["dz3"])
        conv_wgrad(blk.c3, t["a2"], t["dz3"])
        chk("conv_dgrad_gate", blk.c3.name, t["g_a2"], conv_dgrad(blk.c3, t["dz3"], t["a2"]) * relu(t["a2"]))
        bn_bwd(pre + ".bn2", _f(t["g_a2"]), t["z2"], t["dz2"])
        conv_wgrad(blk.c2, t["a1"], t["dz2"])
        chk("conv_dgrad_gate", blk.c2.name, t["g_a1"], conv_dgrad(blk.c2, t["dz2"], t["a1"]) * relu(t["a1"]))
        bn_bwd(pre + ".bn1", _f(t["g_a1"]), t["z1"], t["dz1"])
        conv_wgrad(blk.c1, t["x"], t["dz1"])
        if blk.cd is not None:
            bn_bwd(pre + ".downsample.1", G, t["zd"], t["dzd"])
            conv_wgrad(blk.cd, t["x"], t["dzd"])
            ref_id = conv_dgrad(blk.cd, t["dzd"], t["x"])
            got_id = _f(t["gx_id"])
            if got_id.shape != ref_id.shape:
                # the engine keeps the gradient of a stride-2 downsample convolution on the small grid: the even
                # pixels of the oracle's tensor, whose other pixels are exactly zero
                assert float(ref_id[:, 1::2].abs().max()) == 0.0 and float(ref_id[:, :, 1::2].abs().max()) == 0.0
                chk("conv_dgrad", blk.cd.name, t["gx_id"], ref_id[:, ::2, ::2])
                shortcut = torch.zeros_like(ref_id)
                shortcut[:, ::2, ::2] = got_id
            else:
                chk("conv_dgrad", blk.cd.name, t["gx_id"], ref_id)
                shortcut = got_id
        else:
            shortcut = G
        gx_ref = conv_dgrad(blk.c1, t["dz1"], t["x"]) + shortcut
        if t["gx_gated"]:
            gx_ref = gx_ref * relu(t["x"])
        chk("conv_dgrad_add", blk.c1.name, t["gx"], gx_ref)
    chk("maxpool_bwd", "maxpool", head["g_a0"], O.maxpool_bwd(_f(head["g_p0"]), _f(head["a0"]), 3, 2, 1))
    bn_bwd("bn1", _f(head["g_a0"]) * (_f(head["a0"]) > 0).float(), head["z0"], head["dz0"])
    conv_wgrad(eng.stem, head["x0"], head["dz0"])

    names = [r["name"] for r in eng.ctx.profile(plan.prog, 1)]
    kinds = {n.split("<")[0] for n in names}
    # the plan under test is the fused one: convolutions on the direct-to-LDS kernels, BatchNorm sums in their
    # epilogues, the BatchNorm itself as one launch from the accumulators (or from per-tile sums, bn_acc off)
    bn_kind = "bn_acc_apply_kernel" if eng.bn_acc else "bn_fin_apply_kernel"
    for must in ("igemm2_kernel", "igemm3_kernel", "wgrad_kernel", bn_kind, "splitk_reduce_kernel"):
        assert must in kinds, (must, sorted(kinds))
    print(f"batch {batch}: {chk.count} tensors checked; worst per kind:", flush=True)
    for kind, (e, name) in sorted(chk.worst.items()):
        print(f"  {kind:18s} {e:.3e}  {name}", flush=True)
    print("  tilings in use:", sorted({v for v in plan.tiles.values()}), flush=True)


def test_resnet152_bf16_batch8_every_layer_of_the_tuned_fused_plan():
    _layer_local(8)


def test_resnet152_bf16_batch64_every_layer_of_the_tuned_fused_plan():
    """BASELINE configs[1] at its own batch size: the plan the benchmark times."""
    _layer_local(64)
