"""Convolution -> BatchNorm pairs through exact per-channel accumulators (tch_conv2d_fwd_bnacc /
tch_conv2d_dgrad_bnacc -> tch_bn_fwd_train_acc / tch_bn_bwd_acc), through the C ABI.

What is checked:
* the accumulators (their copies added up) hold the SUM OF THE PER-TILE PARTIALS the per-tile form of the same convolution leaves
  (same tiling, same fp32 partials), to the last bit the split keeps: compared with math.fsum of those
  partials (exact summation on the host), a bound of 2^-60 relative -- not with a second floating-point sum;
* they are integers: two runs give the same words bit for bit, although the order the workgroups add in is
  not fixed;
* BatchNorm from them agrees with the oracle's conv -> BatchNorm(train) (-> backward) chain on the same
  inputs (fp32 1e-3, bf16 2e-2 of the tensor's largest magnitude) and, elementwise, with the per-tile form
  (the two differ only in how the per-channel totals were rounded to fp64);
* many row tiles (more than the fused per-tile form takes) and a residual + ReLU epilogue.
"""
import math

import pytest
import torch

from oracle import nn_ops as O

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2}

CASES = [
    # N, H, W, C, K, R, S, stride, pad
    (2, 14, 14, 64, 64, 3, 3, 1, 1),
    (2, 14, 14, 256, 64, 1, 1, 1, 0),
    (2, 14, 14, 64, 256, 1, 1, 1, 0),
    (2, 16, 16, 64, 128, 3, 3, 2, 1),
    (3, 14, 14, 128, 128, 3, 3, 1, 1),
    (2, 7, 7, 128, 64, 3, 3, 1, 1),
    (5, 9, 11, 64, 64, 1, 1, 1, 0),       # ragged last row tile
]


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def rnd(shape, dtype, g, scale=1.0):
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(got, ref, rtol, what):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    assert got.shape == ref.shape, what
    assert torch.isfinite(got).all(), f"{what}: non-finite"
    scale = ref.abs().max().item() + 1e-30
    err = (got - ref).abs().max().item()
    assert err <= rtol * scale, f"{what}: max err {err:.3e} > {rtol:g} * {scale:.3e}"


def decode(acc, C):
    """[C][2] python floats from the [copies, 4, C] int64 words: the copies are added up as integers, then
    hi * 2^-24 + lo * 2^-66 (both exact in binary)."""
    w = acc.cpu().reshape(-1, 4, C).sum(0).tolist()
    return [[w[0][c] * 2.0 ** -24 + w[1][c] * 2.0 ** -66, w[2][c] * 2.0 ** -24 + w[3][c] * 2.0 ** -66] for c in range(C)]


def exact_sums(partial, rb, C):
    p = partial.cpu().reshape(rb, C, 2).double()
    return [[math.fsum(p[:, c, j].tolist()) for j in range(2)] for c in range(C)]


def assert_totals(acc, partial, rb, C, what):
    got, want = decode(acc, C), exact_sums(partial, rb, C)
    for c in range(C):
        for j in range(2):
            # every partial loses at most 2^-67 in the split; rb of them, and the decode rounds once to fp64
            bound = rb * 2.0 ** -66 + abs(want[c][j]) * 2.0 ** -51
            assert abs(got[c][j] - want[c][j]) <= bound, (what, c, j, got[c][j], want[c][j])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("tile_cfg,copies", [(-1, 1), (0, 4), (1, 2), (2, 8), (5, 1), (11, 4), (13, 16)])
def test_forward_statistics_through_accumulators(ctx, dtype, case, tile_cfg, copies):
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    print("case", case, dtype, tile_cfg, copies, flush=True)
    g = _gen(31)
    x = rnd((N, H, W, C), dtype, g)
    w = rnd((K, R, S, C), dtype, g, (R * S * C) ** -0.5)
    gamma, beta = torch.rand(K, generator=g) + 0.5, torch.randn(K, generator=g) * 0.1
    res = rnd((N,) + ops.conv_out_hw(H, W, R, S, st, pad) + (K,), dtype, g)
    z_ref = O.conv2d_fwd(x, w, st, pad).to(dtype)
    y_ref, mean_ref, invstd_ref = O.bn_fwd_train(z_ref, gamma, beta, torch.zeros(K), torch.ones(K), relu=True,
                                                 residual=res)
    xd, wd = x.cuda(), w.cuda()
    # per-tile form: the reference for the totals
    rb = ops.conv2d_fwd_stat_rows(xd, K, R, S, st, pad, tile_cfg)
    partial = torch.zeros(rb * K * 2, device="cuda")
    z0 = torch.empty(z_ref.shape, dtype=dtype, device="cuda")
    ops.conv2d_fwd_bnstats(ctx, xd, wd, z0, st, pad, partial, tile_cfg=tile_cfg)
    y0 = torch.empty_like(z0)
    rm0, rv0 = torch.zeros(K, device="cuda"), torch.ones(K, device="cuda")
    sm0, si0 = torch.empty(K, device="cuda"), torch.empty(K, device="cuda")
    ops.bn_fwd_train_partials(ctx, z0, y0, gamma.cuda(), beta.cuda(), rm0, rv0, sm0, si0, partial, rb,
                              torch.empty(2 * K, device="cuda"), residual=res.cuda(), relu=True)
    # accumulator form, twice
    accs = []
    for _ in range(2):
        acc = torch.zeros(copies * 4 * K, dtype=torch.int64, device="cuda")
        z = torch.empty_like(z0)
        ops.conv2d_fwd_bnacc(ctx, xd, wd, z, st, pad, acc, tile_cfg=tile_cfg)
        y = torch.empty_like(z)
        rm, rv = torch.zeros(K, device="cuda"), torch.ones(K, device="cuda")
        sm, si = torch.empty(K, device="cuda"), torch.empty(K, device="cuda")
        ops.bn_fwd_train_acc(ctx, z, y, gamma.cuda(), beta.cuda(), rm, rv, sm, si, acc, residual=res.cuda(), relu=True)
        torch.cuda.synchronize()
        accs.append(acc.clone())
        assert torch.equal(z, z0), "the convolution output does not depend on where the sums go"
    assert torch.equal(accs[0], accs[1]), "integer accumulators: identical from run to run"
    assert_totals(accs[0], partial, rb, K, "forward")
    tol = RTOL[dtype]
    close(sm, mean_ref, tol, "mean")
    close(si, invstd_ref, tol, "invstd")
    close(y, y_ref, tol, "y")
    close(sm, sm0, 1e-6, "mean vs per-tile form")
    close(si, si0, 1e-6, "invstd vs per-tile form")
    close(rm, rm0, 1e-6, "running mean vs per-tile form")
    close(rv, rv0, 1e-6, "running var vs per-tile form")
    # elementwise: the two forms may round a coefficient differently in its last bit
    d = (y.float() - y0.float()).abs()
    lim = (1e-5 if dtype == torch.float32 else 8e-3) * y0.float().abs().clamp_min(1.0)
    assert (d <= lim).all(), f"y vs per-tile form: {d.max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("tile_cfg,copies", [(-1, 4), (0, 1), (1, 8), (2, 2), (5, 4), (11, 1), (13, 2)])
def test_backward_sums_through_accumulators(ctx, dtype, case, tile_cfg, copies):
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    print("case", case, dtype, tile_cfg, copies, flush=True)
    g = _gen(32)
    Ho, Wo = ops.conv_out_hw(H, W, R, S, st, pad)
    dy = rnd((N, Ho, Wo, K), dtype, g, 1e-3)     # gradients are small: the split must keep them
    w = rnd((K, R, S, C), dtype, g, (R * S * K) ** -0.5)
    add = rnd((N, H, W, C), dtype, g, 1e-3)
    z = (rnd((N, H, W, C), dtype, g) * 1.3 - 0.2).to(dtype)
    relu_out = rnd((N, H, W, C), dtype, g)
    gamma = torch.rand(C, generator=g) + 0.5
    z2 = z.float().reshape(-1, C)
    mean, invstd = z2.mean(0), 1.0 / torch.sqrt(z2.var(0, unbiased=False) + 1e-5)
    g_ref = (O.conv2d_dgrad(dy, w, (N, H, W, C), st, pad) + add.float()).to(dtype)
    dz_ref, dg_ref, db_ref = O.bn_bwd(g_ref, z, gamma, relu_mask=relu_out)

    wt = ops.filter_transpose(ctx, w.cuda())
    zd = z.cuda()
    gx0 = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    rb = ops.conv2d_dgrad_stat_rows(gx0, K, R, S, st, pad, tile_cfg)
    partial = torch.zeros(rb * C * 2, device="cuda")
    ops.conv2d_dgrad_bnsums(ctx, dy.cuda(), wt, gx0, st, pad, zd, mean.cuda(), invstd.cuda(), partial,
                            bn_mask=relu_out.cuda(), add=add.cuda(), tile_cfg=tile_cfg)
    dz0 = torch.empty_like(gx0)
    dg0, db0 = torch.zeros(C, device="cuda"), torch.zeros(C, device="cuda")
    ops.bn_bwd_partials(ctx, gx0, zd, dz0, gamma.cuda(), mean.cuda(), invstd.cuda(), dg0, db0, partial, rb,
                        torch.empty(3 * C, device="cuda"))
    accs = []
    for _ in range(2):
        acc = torch.zeros(copies * 4 * C, dtype=torch.int64, device="cuda")
        gx = torch.empty_like(gx0)
        ops.conv2d_dgrad_bnacc(ctx, dy.cuda(), wt, gx, st, pad, zd, mean.cuda(), invstd.cuda(), acc,
                               bn_mask=relu_out.cuda(), add=add.cuda(), tile_cfg=tile_cfg)
        dz = torch.empty_like(gx)
        dg, db = torch.ones(C, device="cuda"), torch.ones(C, device="cuda")
        ops.bn_bwd_acc(ctx, gx, zd, dz, gamma.cuda(), mean.cuda(), invstd.cuda(), dg, db, acc, accumulate=True)
        torch.cuda.synchronize()
        accs.append(acc.clone())
        assert torch.equal(gx, gx0)
    assert torch.equal(accs[0], accs[1])
    assert_totals(accs[0], partial, rb, C, "backward")
    tol = RTOL[dtype]
    close(dg - 1.0, dg_ref, tol, "dgamma (accumulated onto ones)")
    close(db - 1.0, db_ref, tol, "dbeta (accumulated onto ones)")
    close(dz, dz_ref, tol, "dx")
    close(dg - 1.0, dg0, 1e-5, "dgamma vs per-tile form")
    close(db - 1.0, db0, 1e-5, "dbeta vs per-tile form")
    d = (dz.float() - dz0.float()).abs()
    lim = (1e-5 if dtype == torch.float32 else 8e-3) * dz0.float().abs().max().clamp_min(1e-12)
    assert (d <= lim).all(), f"dx vs per-tile form: {d.max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_many_row_tiles_and_large_values(ctx, dtype):
    """1568 row tiles add to the same accumulators (a 56x56 layer at batch 8 has as many); activations of a few
    hundred (sums of squares near 1e9 per tile) and of 1e-4 in neighbouring channels."""
    from sirius_amd import ops
    N, H, W, C, K = 8, 112, 112, 64, 64
    g = _gen(33)
    x = rnd((N, H, W, C), dtype, g)
    col_scale = torch.ones(K)
    col_scale[::3] = 300.0
    col_scale[1::3] = 1e-4
    w = (torch.randn(K, 1, 1, C, generator=g) * C ** -0.5 * col_scale.view(K, 1, 1, 1)).to(dtype)
    gamma, beta = torch.rand(K, generator=g) + 0.5, torch.randn(K, generator=g) * 0.1
    xd, wd = x.cuda(), w.cuda()
    z = torch.empty((N, H, W, K), dtype=dtype, device="cuda")
    acc = torch.zeros(8 * 4 * K, dtype=torch.int64, device="cuda")     # eight copies
    ops.conv2d_fwd_bnacc(ctx, xd, wd, z, 1, 0, acc, tile_cfg=2)
    y = torch.empty_like(z)
    rm, rv = torch.zeros(K, device="cuda"), torch.ones(K, device="cuda")
    sm, si = torch.empty(K, device="cuda"), torch.empty(K, device="cuda")
    ops.bn_fwd_train_acc(ctx, z, y, gamma.cuda(), beta.cuda(), rm, rv, sm, si, acc, relu=False)
    torch.cuda.synchronize()
    zz = z.double().cpu().reshape(-1, K)
    tot = decode(acc, K)
    s_ref, q_ref = zz.sum(0), (zz * zz).sum(0)
    for c in range(K):
        # the per-tile partials are fp32 sums over 64 rows: 1e-6 relative is their own rounding
        assert abs(tot[c][0] - s_ref[c].item()) <= 2e-6 * zz[:, c].abs().sum().item() + 1e-12, c
        assert abs(tot[c][1] - q_ref[c].item()) <= 2e-6 * q_ref[c].item() + 1e-18, c
    y_ref, mean_ref, invstd_ref = O.bn_fwd_train(z.cpu(), gamma, beta, torch.zeros(K), torch.ones(K), relu=False)
    close(sm, mean_ref, 1e-4, "mean")
    close(si, invstd_ref, 1e-4, "invstd")
    close(y, y_ref, RTOL[dtype], "y")


def test_accumulator_arguments_are_checked(ctx):
    from sirius_amd import ops
    from sirius_amd._lib import TorchColHipError
    x = torch.zeros((1, 8, 8, 64), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((48, 1, 1, 64), dtype=torch.bfloat16, device="cuda")
    z = torch.zeros((1, 8, 8, 48), dtype=torch.bfloat16, device="cuda")
    acc = torch.zeros(48 * 4, dtype=torch.int64, device="cuda")
    f = torch.zeros(48, device="cuda")
    # 48 channels are not a whole group of eight chunks: the one-launch BatchNorm refuses them
    with pytest.raises(TorchColHipError):
        ops.bn_fwd_train_acc(ctx, z, z.clone(), f, f, None, None, f.clone(), f.clone(), acc)
    with pytest.raises(AssertionError):
        ops.conv2d_fwd_bnacc(ctx, x, w, z, 1, 0, acc[:-1])
    with pytest.raises(AssertionError):      # three copies: not a power of two
        ops.conv2d_fwd_bnacc(ctx, x, w, z, 1, 0, torch.zeros(3 * 48 * 4, dtype=torch.int64, device="cuda"))
