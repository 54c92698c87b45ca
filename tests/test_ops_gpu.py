"""Operator parity on the GPU: every HIP kernel, called through the C ABI, against the
CPU oracle (oracle/nn_ops.py) on the same seeded inputs.

Tolerances (stated per the path's contract): fp32 rtol 1e-3; bf16 rtol 2e-2, measured
twice for every tensor:

* norm-wise: |got - ref| <= rtol * max|ref| over the whole tensor, the meaningful bound
  for sums of thousands of products;
* per channel (the last dimension: output channels of a convolution, channels of a
  BatchNorm, classes of a loss): |got - ref| <= rtol * max(max|ref| within that channel,
  1 % of the tensor's maximum).  A channel of small magnitude that is wrong throughout
  passes the first bound and fails this one; the 1 % floor keeps channels that are (nearly)
  zero by cancellation from being held to their own rounding noise.

Integer results (argmax indices) must be bit-exact.
"""
import pytest
import torch

from oracle import nn_ops as O

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2}


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def rnd(shape, dtype, g, scale=1.0):
    """Seeded N(0,1) values, rounded to `dtype` so that oracle and kernel see identical inputs."""
    t = torch.randn(shape, generator=g) * scale
    return t.to(dtype)


def close(got, ref, dtype, what, rtol=None):
    rtol = RTOL[dtype] if rtol is None else rtol
    got = got.detach().float().cpu()
    ref = ref.detach().float()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    scale = ref.abs().max().item() + 1e-12
    err = (got - ref).abs().max().item()
    assert err <= rtol * scale, f"{what}: max err {err:.3e} > {rtol:g} * {scale:.3e}"
    if ref.dim() >= 2 and ref.shape[-1] > 1:
        r2, g2 = ref.reshape(-1, ref.shape[-1]), got.reshape(-1, ref.shape[-1])
        col_scale = torch.clamp(r2.abs().amax(0), min=1e-2 * scale)
        col_err = (g2 - r2).abs().amax(0)
        over = col_err / (rtol * col_scale)
        c = int(over.argmax())
        assert over[c] <= 1.0, (f"{what}: channel {c} max err {col_err[c].item():.3e} > {rtol:g} * {col_scale[c].item():.3e} "
                                f"(its own scale; the tensor's is {scale:.3e})")


CONV_CASES = [
    # N, H, W, C, K, R, S, stride, pad
    (2, 14, 14, 64, 64, 3, 3, 1, 1),      # the dominant ResNet shape family
    (2, 14, 14, 256, 64, 1, 1, 1, 0),     # pointwise reduce
    (2, 14, 14, 64, 256, 1, 1, 1, 0),     # pointwise expand
    (2, 16, 16, 64, 128, 3, 3, 2, 1),     # strided 3x3
    (2, 16, 16, 64, 128, 1, 1, 2, 0),     # strided 1x1 (downsample)
    (2, 32, 32, 8, 64, 7, 7, 2, 3),       # stem with the channel dim padded to one chunk
    (3, 7, 7, 32, 40, 3, 3, 1, 1),        # ragged: rows, cols and reduction all off-tile
    (5, 1, 1, 64, 1000, 1, 1, 1, 0),      # fully connected as a 1x1 convolution
    (1, 9, 11, 16, 24, 3, 3, 1, 1),       # non-square
    (2, 16, 16, 8, 32, 4, 4, 4, 0),       # patch embedding: 4x4 patches, stride 4, channels padded to one chunk
    (3, 14, 14, 128, 96, 3, 3, 1, 1),     # 3x3 over two channel blocks, tiles that span images, ragged columns
    (1, 28, 28, 64, 64, 3, 3, 1, 1),      # 3x3 with 28-pixel rows (the longer patch of tiling 5)
    (1, 56, 56, 64, 64, 3, 3, 1, 1),      # 3x3 with 56-pixel rows (the longest patch)
    (2, 7, 7, 128, 64, 3, 3, 1, 1),       # 3x3 on 7x7 images: every tile holds image borders
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("tile_cfg", [-1, 0, 1, 2, 3, 5, 6, 7, 9, 10, 11, 12, 13, 14])
def test_conv_fwd(ctx, dtype, case, tile_cfg):
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    print("case", case, dtype, tile_cfg, flush=True)
    g = _gen(1)
    x = rnd((N, H, W, C), dtype, g)
    w = rnd((K, R, S, C), dtype, g, (R * S * C) ** -0.5)
    ref = O.conv2d_fwd(x, w, st, pad)
    y = torch.empty(ref.shape, dtype=dtype, device="cuda")
    ops.conv2d_fwd(ctx, x.cuda(), w.cuda(), y, st, pad, tile_cfg=tile_cfg)
    torch.cuda.synchronize()
    close(y, ref, dtype, "conv fwd")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tile_cfg", [-1, 0, 2, 5])
def test_conv_channels_of_very_different_scale(ctx, dtype, tile_cfg):
    """Output channels that differ by 1e4 in magnitude, forward, data gradient and weight gradient: the per-channel
    bound of close() holds the small ones to their own scale."""
    from sirius_amd import ops
    N, H, W, C, K = 2, 14, 14, 64, 128
    g = _gen(77)
    scale_k = torch.ones(K)
    scale_k[::2] = 1e-4
    x = rnd((N, H, W, C), dtype, g)
    w = (torch.randn(K, 3, 3, C, generator=g) * (9 * C) ** -0.5 * scale_k.view(K, 1, 1, 1)).to(dtype)
    y = torch.empty((N, H, W, K), dtype=dtype, device="cuda")
    ops.conv2d_fwd(ctx, x.cuda(), w.cuda(), y, 1, 1, tile_cfg=tile_cfg)
    torch.cuda.synchronize()
    close(y, O.conv2d_fwd(x, w, 1, 1), dtype, "conv fwd, mixed channel scales")
    # data gradient into input channels of mixed scale: scale the filter over its input channels instead
    scale_c = torch.ones(C)
    scale_c[1::2] = 1e-4
    w2 = (torch.randn(K, 3, 3, C, generator=g) * (9 * K) ** -0.5 * scale_c.view(1, 1, 1, C)).to(dtype)
    dy = rnd((N, H, W, K), dtype, g)
    dx = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    ops.conv2d_dgrad(ctx, dy.cuda(), ops.filter_transpose(ctx, w2.cuda()), dx, 1, 1, tile_cfg=tile_cfg)
    torch.cuda.synchronize()
    close(dx, O.conv2d_dgrad(dy, w2, (N, H, W, C), 1, 1), dtype, "conv dgrad, mixed channel scales")
    # weight gradient with input channels of mixed scale
    x3 = (torch.randn(N, H, W, C, generator=g) * scale_c).to(dtype)
    dw = torch.empty((K, 3, 3, C), device="cuda")
    ops.conv2d_wgrad(ctx, x3.cuda(), dy.cuda(), dw, 1, 1)
    torch.cuda.synchronize()
    close(dw, O.conv2d_wgrad(x3, dy, (K, 3, 3, C), 1, 1), dtype, "conv wgrad, mixed channel scales")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_fwd_epilogue(ctx, dtype):
    """bias, fp32 output, gated addend"""
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = 2, 8, 8, 32, 48, 3, 3, 1, 1
    g = _gen(2)
    x, w = rnd((N, H, W, C), dtype, g), rnd((K, R, S, C), dtype, g, 0.06)
    bias = torch.randn(K, generator=g)
    add = rnd((N, H, W, K), dtype, g)
    mask = rnd((N, H, W, K), dtype, g)
    ref = O.conv2d_fwd(x, w, st, pad, bias) + add.float() * (mask.float() > 0)
    y = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
    ops.conv2d_fwd(ctx, x.cuda(), w.cuda(), y, st, pad, add=add.cuda(), mask=mask.cuda(), bias=bias.cuda())
    torch.cuda.synchronize()
    close(y, ref, dtype, "conv fwd epilogue", rtol=1e-3 if dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("tile_cfg", [-1, 0, 1, 2, 3, 5, 6, 7, 9, 10, 11, 12, 13, 14])
def test_conv_dgrad(ctx, dtype, case, tile_cfg):
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    print("case", case, dtype, tile_cfg, flush=True)
    g = _gen(3)
    Ho, Wo = ops.conv_out_hw(H, W, R, S, st, pad)
    dy = rnd((N, Ho, Wo, K), dtype, g)
    w = rnd((K, R, S, C), dtype, g, (R * S * K) ** -0.5)
    ref = O.conv2d_dgrad(dy, w, (N, H, W, C), st, pad)
    dx = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    ops.conv2d_dgrad(ctx, dy.cuda(), ops.filter_transpose(ctx, w.cuda()), dx, st, pad, tile_cfg=tile_cfg)
    torch.cuda.synchronize()
    close(dx, ref, dtype, "conv dgrad")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_dgrad_residual(ctx, dtype):
    """dx = dgrad + addend gated by a ReLU mask (the identity branch of a bottleneck)"""
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = 2, 8, 8, 64, 32, 1, 1, 1, 0
    g = _gen(4)
    dy, w = rnd((N, H, W, K), dtype, g), rnd((K, R, S, C), dtype, g, 0.2)
    add, mask = rnd((N, H, W, C), dtype, g), rnd((N, H, W, C), dtype, g)
    ref = O.conv2d_dgrad(dy, w, (N, H, W, C), st, pad) + add.float() * (mask.float() > 0)
    dx = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    ops.conv2d_dgrad(ctx, dy.cuda(), ops.filter_transpose(ctx, w.cuda()), dx, st, pad, add=add.cuda(), mask=mask.cuda())
    torch.cuda.synchronize()
    close(dx, ref, dtype, "conv dgrad + residual")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [CONV_CASES[0], CONV_CASES[2], CONV_CASES[3], CONV_CASES[5], CONV_CASES[6], CONV_CASES[10]])
@pytest.mark.parametrize("tile_cfg", [-1, 0, 2, 5])
def test_conv_fwd_with_inference_batchnorm_in_the_epilogue(ctx, dtype, case, tile_cfg):
    """conv -> BatchNorm(eval) -> (+ residual) -> ReLU as one launch: scale, shift, residual and ReLU act on the
    fp32 accumulators; against the oracle's convolution followed by the same arithmetic in fp32."""
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    g = _gen(23)
    x = rnd((N, H, W, C), dtype, g)
    w = rnd((K, R, S, C), dtype, g, (R * S * C) ** -0.5)
    Ho, Wo = ops.conv_out_hw(H, W, R, S, st, pad)
    res = rnd((N, Ho, Wo, K), dtype, g)
    scale = torch.rand(K, generator=g) + 0.5
    shift = torch.randn(K, generator=g)
    conv = O.conv2d_fwd(x, w, st, pad)
    for use_res, relu in ((False, True), (True, True), (True, False), (False, False)):
        ref = conv * scale + shift + (res.float() if use_res else 0.0)
        if relu:
            ref = ref.clamp_min(0.0)
        y = torch.full((N, Ho, Wo, K), -5.0, dtype=dtype, device="cuda")
        ops.conv2d_fwd_affine(ctx, x.cuda(), w.cuda(), y, st, pad, scale=scale.cuda(), shift=shift.cuda(),
                              residual=res.cuda() if use_res else None, relu=relu, tile_cfg=tile_cfg)
        torch.cuda.synchronize()
        close(y, ref, dtype, f"conv + affine (residual {use_res}, relu {relu})")
        if relu:
            assert float(y.float().min()) >= 0.0
    # no scale, no shift: the plain convolution
    y = torch.empty((N, Ho, Wo, K), dtype=dtype, device="cuda")
    y2 = torch.empty_like(y)
    ops.conv2d_fwd_affine(ctx, x.cuda(), w.cuda(), y, st, pad, tile_cfg=tile_cfg)
    ops.conv2d_fwd(ctx, x.cuda(), w.cuda(), y2, st, pad, tile_cfg=tile_cfg)
    torch.cuda.synchronize()
    assert torch.equal(y, y2)


@pytest.mark.parametrize("shape", [(1000, 128, 520), (2048, 192, 1024), (300, 64, 72), (1100, 64, 1200), (2900, 64, 2320)])
def test_huge_tile_equals_the_128_tile(ctx, shape):
    """The 256 x 256 tilings (plain and rotated loop, eight wavefronts) and the tilings with 32-element reduction
    steps (11 - 14) on products with several such tiles and ragged edges: within the bf16 bound of the oracle and
    bit-equal to the 128 x 128 tiling (same order of additions per output), forward and data gradient, with the
    grouped tile order on and off (wide and narrow N)."""
    from sirius_amd import ops
    M, C, K = shape
    g = _gen(17)
    x = rnd((1, 1, M, C), torch.bfloat16, g)
    w = rnd((K, 1, 1, C), torch.bfloat16, g, C ** -0.5)
    ref = O.conv2d_fwd(x, w, 1, 0)
    outs = {}
    for cfg in (0, 9, 10, 11, 12, 13, 14):
        y = torch.full((1, 1, M, K), 3.0, dtype=torch.bfloat16, device="cuda")
        ops.conv2d_fwd(ctx, x.cuda(), w.cuda(), y, 1, 0, tile_cfg=cfg)
        torch.cuda.synchronize()
        close(y, ref, torch.bfloat16, f"forward tiling {cfg}")
        outs[cfg] = y
    assert all(torch.equal(outs[c], outs[0]) for c in outs), [c for c in outs if not torch.equal(outs[c], outs[0])]
    dy = rnd((1, 1, M, K), torch.bfloat16, g)
    ref_dx = O.conv2d_dgrad(dy, w, (1, 1, M, C), 1, 0)
    wt = ops.filter_transpose(ctx, w.cuda())
    outs = {}
    for cfg in (0, 9, 10, 11, 12, 13, 14):
        dx = torch.full((1, 1, M, C), 3.0, dtype=torch.bfloat16, device="cuda")
        ops.conv2d_dgrad(ctx, dy.cuda(), wt, dx, 1, 0, tile_cfg=cfg)
        torch.cuda.synchronize()
        close(dx, ref_dx, torch.bfloat16, f"data gradient tiling {cfg}")
        outs[cfg] = dx
    assert all(torch.equal(outs[c], outs[0]) for c in outs), [c for c in outs if not torch.equal(outs[c], outs[0])]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hw", [(14, 14), (7, 9), (5, 5)])
@pytest.mark.parametrize("tile_cfg", [-1, 0, 2, 6])
def test_conv_dgrad_with_a_compact_addend(ctx, dtype, hw, tile_cfg):
    """The data gradient of a stride-2 1x1 convolution is non-zero at the even pixels only: kept on the small grid
    (odd sizes: ceil(H/2) x ceil(W/2)) and added from there by the data gradient it joins -- same result as adding
    the full-size tensor, bit for bit; also with the BatchNorm-backward sums in the epilogue."""
    from sirius_amd import ops
    H, W = hw
    N, C, K, Kd = 3, 64, 64, 128
    g = _gen(31)
    dy = rnd((N, H, W, K), dtype, g, K ** -0.5)
    w = rnd((K, 1, 1, C), dtype, g)
    Hs, Ws = (H + 1) // 2, (W + 1) // 2
    dyd = rnd((N, Hs, Ws, Kd), dtype, g, Kd ** -0.5)         # gradient of the downsample branch's output
    wd = rnd((Kd, 1, 1, C), dtype, g)
    wt, wdt = ops.filter_transpose(ctx, w.cuda()), ops.filter_transpose(ctx, wd.cuda())
    # full-size route: stride-2 data gradient blown up to the input grid, then added
    full = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    ops.conv2d_dgrad(ctx, dyd.cuda(), wdt, full, 2, 0)
    ref_full = O.conv2d_dgrad(dyd, wd, (N, H, W, C), 2, 0)
    torch.cuda.synchronize()
    close(full, ref_full, dtype, "stride-2 data gradient")
    assert float(full[:, 1::2].float().abs().max()) == 0.0 and float(full[:, :, 1::2].float().abs().max()) == 0.0
    dx_a = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    ops.conv2d_dgrad(ctx, dy.cuda(), wt, dx_a, 1, 0, add=full, tile_cfg=tile_cfg)
    # compact route
    small = torch.empty((N, Hs, Ws, C), dtype=dtype, device="cuda")
    ops.conv2d_dgrad(ctx, dyd.cuda(), wdt, small, 1, 0)
    dx_b = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    ops.conv2d_dgrad(ctx, dy.cuda(), wt, dx_b, 1, 0, add=small, add_stride=2, tile_cfg=tile_cfg)
    torch.cuda.synchronize()
    assert torch.equal(small, full[:, ::2, ::2])
    assert torch.equal(dx_a, dx_b)
    close(dx_b, O.conv2d_dgrad(dy, w, (N, H, W, C), 1, 0) + ref_full, dtype, "data gradient + compact addend")
    # the same with the BatchNorm-backward sums and the ReLU gate in the epilogue
    bn_x, relu_out = rnd((N, H, W, C), dtype, g), rnd((N, H, W, C), dtype, g)
    mean, invstd = torch.randn(C, generator=g), torch.rand(C, generator=g) + 0.5
    outs = []
    for add, stride in ((full, 1), (small, 2)):
        dx = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
        rb = ops.conv2d_dgrad_stat_rows(dx, K, 1, 1, 1, 0, tile_cfg)
        partial = torch.zeros(rb * C * 2, dtype=torch.float32, device="cuda")
        ops.conv2d_dgrad_bnsums(ctx, dy.cuda(), wt, dx, 1, 0, bn_x.cuda(), mean.cuda(), invstd.cuda(), partial,
                                bn_mask=relu_out.cuda(), add=add, add_stride=stride, tile_cfg=tile_cfg)
        torch.cuda.synchronize()
        outs.append((dx, partial))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("splits", [1, 0, 3])
def test_conv_wgrad(ctx, dtype, case, splits):
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    print("case", case, dtype, splits, flush=True)
    g = _gen(5)
    Ho, Wo = ops.conv_out_hw(H, W, R, S, st, pad)
    x = rnd((N, H, W, C), dtype, g)
    dy = rnd((N, Ho, Wo, K), dtype, g, (N * Ho * Wo) ** -0.5)
    ref = O.conv2d_wgrad(x, dy, (K, R, S, C), st, pad)
    dw = torch.full((K, R, S, C), 7.0, dtype=torch.float32, device="cuda")
    ws = None
    if splits != 1:
        n_split = splits if splits > 0 else ops.conv2d_wgrad_splits(x, K, R, S, st, pad)
        nbytes = max(4, ops.conv2d_wgrad_workspace_bytes(ops.dtype_code(x), K, R, S, C, n_split))
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device="cuda")
    ops.conv2d_wgrad(ctx, x.cuda(), dy.cuda(), dw, st, pad, workspace=ws, splits=splits)
    torch.cuda.synchronize()
    close(dw, ref, dtype, "conv wgrad", rtol=1e-3 if dtype == torch.float32 else 5e-3)
    # accumulate: a second pass adds the same gradient on top; this one also asks for the bias gradient
    # (column sums of dy), first plain into a filled buffer, then accumulated
    db_ref = dy.float().sum(dim=(0, 1, 2))
    db = torch.full((K,), -3.0, dtype=torch.float32, device="cuda")
    dw2 = torch.full((K, R, S, C), 7.0, dtype=torch.float32, device="cuda")
    ops.conv2d_wgrad(ctx, x.cuda(), dy.cuda(), dw2, st, pad, workspace=ws, splits=splits, dbias=db)
    torch.cuda.synchronize()
    assert torch.equal(dw2, dw), "asking for the bias gradient changes the filter gradient"
    close(db, db_ref, torch.float32, "bias gradient", rtol=1e-4)
    ops.conv2d_wgrad(ctx, x.cuda(), dy.cuda(), dw, st, pad, workspace=ws, splits=splits, accumulate=True, dbias=db)
    torch.cuda.synchronize()
    close(dw, 2 * ref, dtype, "conv wgrad accumulate", rtol=1e-3 if dtype == torch.float32 else 5e-3)
    close(db, 2 * db_ref, torch.float32, "bias gradient accumulate", rtol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_wgrad_with_trailing_reductions(ctx, dtype):
    """A run of weight gradients whose split reductions ride the launches behind them (tch_conv2d_wgrad_trailing):
    every dw / dbias equals the one-call-per-layer result BIT FOR BIT (same splits, same order of additions), with
    and without bias gradients, accumulating and not, a layer without splits in the middle of the run, twice in a row
    on the same workspaces; and no reduction launch is left in the run except the flush."""
    from sirius_amd import ops
    g = _gen(61)
    layers = [  # N, H, W, C, K, R, stride, pad, with bias
        (4, 14, 14, 256, 64, 1, 1, 0, False),
        (4, 14, 14, 64, 64, 3, 1, 1, True),
        (1, 4, 4, 64, 256, 1, 1, 0, False),       # few pixels: one split, nothing to reduce
        (4, 14, 14, 64, 256, 1, 1, 0, True),
        (2, 16, 16, 64, 128, 3, 2, 1, False),
    ]
    data = []
    for N, H, W, C, K, R, st, pad, bias in layers:
        Ho, Wo = ops.conv_out_hw(H, W, R, R, st, pad)
        data.append((rnd((N, H, W, C), dtype, g).cuda(), rnd((N, Ho, Wo, K), dtype, g).cuda()))
    code = ops.dtype_code(data[0][0])
    half = 0
    for (x, dy), (N, H, W, C, K, R, st, pad, bias) in zip(data, layers):
        sp = ops.conv2d_wgrad_splits(x, K, R, R, st, pad)
        half = max(half, ops.conv2d_wgrad_workspace_bytes(code, K, R, R, C, sp) // 4)
    half = (half + 63) // 64 * 64
    ws_ref = torch.empty(half, device="cuda")
    ws = torch.full((2 * half,), float("nan"), device="cuda")
    for accumulate in (False, True):
        ref, got = [], []
        for (x, dy), (N, H, W, C, K, R, st, pad, bias) in zip(data, layers):
            dw = torch.full((K, R, R, C), 0.5, device="cuda")
            db = torch.full((K,), 0.25, device="cuda") if bias else None
            ops.conv2d_wgrad(ctx, x, dy, dw, st, pad, workspace=ws_ref, accumulate=accumulate, dbias=db)
            ref.append((dw, db))
        prog = ops.Program()
        ctx.begin_record(prog)
        try:
            trail = ops.TrailingWgrad(ctx, ws, half)
            for (x, dy), (N, H, W, C, K, R, st, pad, bias) in zip(data, layers):
                dw = torch.full((K, R, R, C), 0.5, device="cuda")
                db = torch.full((K,), 0.25, device="cuda") if bias else None
                trail.wgrad(x, dy, dw, st, pad, accumulate=accumulate, dbias=db)
                got.append((dw, db))
            trail.flush()
        finally:
            ctx.end_record()
        names = [r["name"] for r in ctx.profile(prog, 1)]
        # at most the flush: nothing is left for it when the last layer of the run has a single split
        assert sum(r["launches"] for r in ctx.profile(prog, 1) if r["name"].startswith("splitk_reduce")) <= 1, names
        for t, _ in got:        # the profile replays ran the program: start again from the initial values
            t.fill_(0.5)
        for _, b in got:
            if b is not None:
                b.fill_(0.25)
        ctx.run(prog)
        ctx.synchronize()
        torch.cuda.synchronize()
        for i, ((dw, db), (rw, rb)) in enumerate(zip(got, ref)):
            assert torch.equal(dw, rw), f"layer {i}, accumulate {accumulate}: dw"
            assert (db is None) or torch.equal(db, rb), f"layer {i}, accumulate {accumulate}: dbias"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("target_wgs,tile_cfg,max_wgs", [(0, -1, 0), (40, -1, 0), (300, 0, 0), (64, 2, 0), (0, -1, 37), (300, 0, 8)])
def test_conv_wgrad_group(ctx, dtype, target_wgs, tile_cfg, max_wgs):
    """Several weight gradients in one launch over a table: each layer's result equals the oracle's, and equals
    the one-layer call with the same split count and tiling bit for bit (same kernel body, same split ranges,
    same order of additions in the reduction); bias gradients ride along for the layers that ask.  max_wgs: the
    launch is capped at that many workgroups, which share the tiles out among themselves."""
    from sirius_amd import ops
    cases = [c for c in CONV_CASES if c[7] in (1, 2)]
    if tile_cfg == 0:
        cases = [c for c in cases if c[4] >= 128 or c[3] * c[5] * c[6] >= 128]   # any shape runs, these fill tiles
    g = _gen(11)
    items, refs, singles = [], [], []
    for i, (N, H, W, C, K, R, S, st, pad) in enumerate(cases):
        Ho, Wo = ops.conv_out_hw(H, W, R, S, st, pad)
        x = rnd((N, H, W, C), dtype, g)
        dy = rnd((N, Ho, Wo, K), dtype, g, (N * Ho * Wo) ** -0.5)
        dw = torch.full((K, R, S, C), float(i), dtype=torch.float32, device="cuda")
        db = torch.full((K,), -1.0, dtype=torch.float32, device="cuda") if i % 2 == 0 else None
        items.append((x.cuda(), dy.cuda(), dw, st, pad, db))
        refs.append((O.conv2d_wgrad(x, dy, (K, R, S, C), st, pad), dy.float().sum(dim=(0, 1, 2))))
    splits, tile, table_bytes, ws_bytes = ops.conv2d_wgrad_group_plan(items, target_wgs, tile_cfg)
    print("group", dtype, target_wgs, tile_cfg, "->", tile, splits, table_bytes, ws_bytes, flush=True)
    assert tile in (0, 2) and all(sp >= 1 for sp in splits)
    if target_wgs == 0:
        assert max(splits) > 1, "a small group is split to fill the chip"
    table = torch.empty(table_bytes, dtype=torch.uint8, device="cuda")
    ws = torch.full((max(ws_bytes // 4, 1),), float("nan"), dtype=torch.float32, device="cuda")
    ops.conv2d_wgrad_group(ctx, items, splits, tile, ws, table, max_wgs=max_wgs)
    torch.cuda.synchronize()
    rt = 1e-3 if dtype == torch.float32 else 5e-3
    for (x, dy, dw, st, pad, db), (ref, db_ref), sp, case in zip(items, refs, splits, cases):
        close(dw, ref, dtype, f"grouped wgrad {case}", rtol=rt)
        if db is not None:
            close(db, db_ref, torch.float32, f"grouped bias gradient {case}", rtol=1e-4)
        one = torch.empty_like(dw)
        one_b = torch.empty_like(db) if db is not None else None
        K, R, S, C = dw.shape
        w1 = torch.empty(max(4, ops.conv2d_wgrad_workspace_bytes(ops.dtype_code(x), K, R, S, C, sp)) // 4,
                         dtype=torch.float32, device="cuda")
        ops.conv2d_wgrad(ctx, x, dy, one, st, pad, workspace=w1, splits=sp, tile_cfg=tile, dbias=one_b)
        torch.cuda.synchronize()
        assert torch.equal(one, dw), f"grouped and single launch differ for {case} at {sp} splits"
        if db is not None:
            assert torch.equal(one_b, db)
    # a second run over the same table accumulates on top
    ops.conv2d_wgrad_group(ctx, items, splits, tile, ws, table, accumulate=True, max_wgs=max_wgs)
    torch.cuda.synchronize()
    for (x, dy, dw, st, pad, db), (ref, db_ref), case in zip(items, refs, cases):
        close(dw, 2 * ref, dtype, f"grouped wgrad accumulate {case}", rtol=rt)
        if db is not None:
            close(db, 2 * db_ref, torch.float32, f"grouped bias gradient accumulate {case}", rtol=1e-4)


BN_CASES = [(2 * 14 * 14, 64), (4 * 28 * 28, 128), (3 * 7 * 7, 2048), (37, 8), (100000, 64), (1024 + 37, 256)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,C", BN_CASES)
@pytest.mark.parametrize("fuse", ["plain", "relu", "residual_relu"])
def test_bn_fwd(ctx, dtype, rows, C, fuse):
    from sirius_amd import ops
    g = _gen(6)
    x = rnd((1, 1, rows, C), dtype, g) * 1.7 + 0.3
    x = x.to(dtype)
    gamma, beta = torch.rand(C, generator=g) + 0.5, torch.randn(C, generator=g) * 0.1
    rm, rv = torch.randn(C, generator=g) * 0.1, torch.rand(C, generator=g) + 0.5
    res = rnd(x.shape, dtype, g) if fuse == "residual_relu" else None
    relu = fuse != "plain"
    rm_ref, rv_ref = rm.clone(), rv.clone()
    y_ref, mean_ref, invstd_ref = O.bn_fwd_train(x, gamma, beta, rm_ref, rv_ref, residual=res, relu=relu)
    d = lambda t: t.cuda() if t is not None else None
    y = torch.empty(x.shape, dtype=dtype, device="cuda")
    rm_d, rv_d = rm.cuda(), rv.cuda()
    sm, si = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    ws = torch.empty(ops.bn_workspace_bytes(ops.dtype_code(x), rows, C) // 4, dtype=torch.float32, device="cuda")
    ops.bn_fwd_train(ctx, x.cuda(), y, gamma.cuda(), beta.cuda(), rm_d, rv_d, sm, si, ws, residual=d(res), relu=relu)
    torch.cuda.synchronize()
    close(sm, mean_ref, torch.float32, "bn mean", rtol=1e-4)
    close(si, invstd_ref, torch.float32, "bn invstd", rtol=1e-4)
    close(rm_d, rm_ref, torch.float32, "bn running_mean", rtol=1e-4)
    close(rv_d, rv_ref, torch.float32, "bn running_var", rtol=1e-4)
    close(y, y_ref, dtype, "bn y", rtol=1e-4 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [CONV_CASES[0], CONV_CASES[2], CONV_CASES[3], CONV_CASES[5], CONV_CASES[6], CONV_CASES[10], CONV_CASES[13]])
@pytest.mark.parametrize("tile_cfg", [-1, 0, 1, 2, 3, 5, 6, 7, 9, 10, 11, 12, 13, 14])
def test_conv_with_bn_statistics(ctx, dtype, case, tile_cfg):
    """The convolution leaves per-tile sums of its stored output; BatchNorm starts from them.
    Checked against the oracle's conv -> BatchNorm(train) on the same inputs; the statistics must be
    those of the ROUNDED convolution output (what the unfused pair would see)."""
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    print("case", case, dtype, tile_cfg, flush=True)
    g = _gen(21)
    x = rnd((N, H, W, C), dtype, g)
    w = rnd((K, R, S, C), dtype, g, (R * S * C) ** -0.5)
    gamma, beta = torch.rand(K, generator=g) + 0.5, torch.randn(K, generator=g) * 0.1
    z_ref = O.conv2d_fwd(x, w, st, pad).to(dtype)
    rm_ref, rv_ref = torch.zeros(K), torch.ones(K)
    y_ref, mean_ref, invstd_ref = O.bn_fwd_train(z_ref, gamma, beta, rm_ref, rv_ref, relu=True)
    xd, wd = x.cuda(), w.cuda()
    z = torch.empty(z_ref.shape, dtype=dtype, device="cuda")
    rb = ops.conv2d_fwd_stat_rows(xd, K, R, S, st, pad, tile_cfg)
    partial = torch.full((rb * K * 2,), float("nan"), device="cuda")
    assert ops.conv2d_fwd_bnstats(ctx, xd, wd, z, st, pad, partial, tile_cfg=tile_cfg) == rb
    y = torch.empty_like(z)
    rm, rv = torch.zeros(K, device="cuda"), torch.ones(K, device="cuda")
    sm, si = torch.empty(K, device="cuda"), torch.empty(K, device="cuda")
    scratch = torch.empty(2 * K, device="cuda")
    ops.bn_fwd_train_partials(ctx, z, y, gamma.cuda(), beta.cuda(), rm, rv, sm, si, partial, rb, scratch, relu=True)
    torch.cuda.synchronize()
    close(z, z_ref, dtype, "conv out")
    # statistics of what was stored, exactly: compare with sums over the kernel's own z
    z32 = z.float().cpu().reshape(-1, K)
    sums = partial.cpu().reshape(rb, K, 2).double().sum(0)
    close(sums[:, 0].float(), z32.double().sum(0).float(), torch.float32, "sum", rtol=1e-5)
    close(sums[:, 1].float(), (z32.double() ** 2).sum(0).float(), torch.float32, "sum of squares", rtol=1e-5)
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    close(sm, mean_ref, torch.float32, "bn mean", rtol=tol)
    close(si, invstd_ref, torch.float32, "bn invstd", rtol=tol)
    close(y, y_ref, dtype, "bn y", rtol=tol)
    # the same with the coefficients computed as part of the convolution call; twice, on the same counters
    counters = torch.zeros(K // 64 + 1, dtype=torch.int32, device="cuda")
    for _ in range(2):
        rm2, rv2 = torch.zeros(K, device="cuda"), torch.ones(K, device="cuda")
        sm2, si2 = torch.empty(K, device="cuda"), torch.empty(K, device="cuda")
        coef = torch.full((2 * K,), float("nan"), device="cuda")
        z2, y2 = torch.empty_like(z), torch.empty_like(z)
        partial.fill_(float("nan"))
        ops.conv2d_fwd_bn(ctx, xd, wd, z2, st, pad, partial, counters, gamma.cuda(), beta.cuda(), rm2, rv2, sm2, si2, coef,
                          tile_cfg=tile_cfg)
        ops.bn_apply_fwd(ctx, z2, y2, coef, relu=True)
        torch.cuda.synchronize()
        assert torch.equal(z2, z) and torch.all(counters == 0)
        close(sm2, sm.cpu(), torch.float32, "fused finalize: mean", rtol=1e-6)
        close(si2, si.cpu(), torch.float32, "fused finalize: invstd", rtol=1e-6)
        close(rm2, rm.cpu(), torch.float32, "fused finalize: running mean", rtol=1e-6)
        close(rv2, rv.cpu(), torch.float32, "fused finalize: running var", rtol=1e-6)
        close(y2, y.float().cpu(), dtype, "fused finalize: y", rtol=1e-6 if dtype == torch.float32 else 8e-3)


def test_bn_finalize_over_more_row_tiles_than_one_trip(ctx):
    """2 400 row tiles of 64 rows: the finalize kernels' lanes take more than one trip over their row tiles
    (a trip covers 2 048).  Forward statistics and backward sums against the oracle."""
    from sirius_amd import ops
    dtype = torch.bfloat16
    N, H, W, C, K = 6, 160, 160, 64, 64     # 153 600 output rows
    g = _gen(29)
    x = rnd((N, H, W, C), dtype, g)
    w = rnd((K, 1, 1, C), dtype, g, C ** -0.5)
    gamma, beta = torch.rand(K, generator=g) + 0.5, torch.randn(K, generator=g) * 0.1
    z_ref = O.conv2d_fwd(x, w, 1, 0).to(dtype)
    y_ref, mean_ref, invstd_ref = O.bn_fwd_train(z_ref, gamma, beta, torch.zeros(K), torch.ones(K), relu=True)
    xd, wd = x.cuda(), w.cuda()
    z = torch.empty(z_ref.shape, dtype=dtype, device="cuda")
    rb = ops.conv2d_fwd_stat_rows(xd, K, 1, 1, 1, 0, 2)
    assert rb == 2400
    partial = torch.full((rb * K * 2,), float("nan"), device="cuda")
    ops.conv2d_fwd_bnstats(ctx, xd, wd, z, 1, 0, partial, tile_cfg=2)
    y = torch.empty_like(z)
    rm, rv = torch.zeros(K, device="cuda"), torch.ones(K, device="cuda")
    sm, si = torch.empty(K, device="cuda"), torch.empty(K, device="cuda")
    scratch = torch.empty(2 * K, device="cuda")
    ops.bn_fwd_train_partials(ctx, z, y, gamma.cuda(), beta.cuda(), rm, rv, sm, si, partial, rb, scratch, relu=True)
    torch.cuda.synchronize()
    close(sm, mean_ref, torch.float32, "bn mean", rtol=2e-2)
    close(si, invstd_ref, torch.float32, "bn invstd", rtol=2e-2)
    close(y, y_ref, dtype, "bn y", rtol=2e-2)
    z32 = z.float().cpu().reshape(-1, K).double()
    close(sm, z32.mean(0).float(), torch.float32, "mean of the stored output", rtol=1e-5)
    # backward: data gradient of a 1x1 convolution behind that BatchNorm + ReLU, sums over 2 400 row tiles
    dy2 = rnd((N, H, W, K), dtype, g)
    w2 = rnd((K, 1, 1, K), dtype, g, K ** -0.5)
    g_ref = O.conv2d_dgrad(dy2, w2, (N, H, W, K), 1, 0)
    dz_ref, dg_ref, db_ref = O.bn_bwd(g_ref, z_ref, gamma, relu_mask=y_ref)
    gx = torch.empty((N, H, W, K), dtype=dtype, device="cuda")
    rb2 = ops.conv2d_dgrad_stat_rows(gx, K, 1, 1, 1, 0, 2)
    assert rb2 == 2400
    partial2 = torch.full((rb2 * K * 2,), float("nan"), device="cuda")
    ops.conv2d_dgrad_bnsums(ctx, dy2.cuda(), ops.filter_transpose(ctx, w2.cuda()), gx, 1, 0, z, sm, si, partial2,
                            bn_mask=y, tile_cfg=2)
    dz = torch.empty_like(z)
    dgm, dbt = torch.empty(K, device="cuda"), torch.empty(K, device="cuda")
    ops.bn_bwd_partials(ctx, gx, z, dz, gamma.cuda(), sm, si, dgm, dbt, partial2, rb2, torch.empty(3 * K, device="cuda"))
    torch.cuda.synchronize()
    close(dgm, dg_ref, torch.float32, "bn dgamma", rtol=2e-2)
    close(dbt, db_ref, torch.float32, "bn dbeta", rtol=2e-2)
    close(dz, dz_ref, dtype, "bn dz", rtol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_bn_finalize_with_many_row_tiles(ctx, dtype):
    """More row tiles than one workgroup should sum (> 256): the convolution call finishes the coefficients
    with a launch of its own; same results, same interface."""
    from sirius_amd import ops
    N, H, W, C, K = 2, 96, 96, 64, 64     # 18432 output rows: 288 tiles of 64 rows
    g = _gen(23)
    x = rnd((N, H, W, C), dtype, g)
    w = rnd((K, 1, 1, C), dtype, g, C ** -0.5)
    gamma, beta = torch.rand(K, generator=g) + 0.5, torch.randn(K, generator=g) * 0.1
    z_ref = O.conv2d_fwd(x, w, 1, 0).to(dtype)
    rm_ref, rv_ref = torch.zeros(K), torch.ones(K)
    y_ref, mean_ref, invstd_ref = O.bn_fwd_train(z_ref, gamma, beta, rm_ref, rv_ref, relu=True)
    xd, wd = x.cuda(), w.cuda()
    assert ops.conv2d_fwd_stat_rows(xd, K, 1, 1, 1, 0, 2) > 256
    partial = torch.empty(ops.conv2d_fwd_stat_rows(xd, K, 1, 1, 1, 0, 2) * K * 2, device="cuda")
    counters = torch.zeros(2, dtype=torch.int32, device="cuda")
    z, y = (torch.empty(z_ref.shape, dtype=dtype, device="cuda") for _ in range(2))
    rm, rv = torch.zeros(K, device="cuda"), torch.ones(K, device="cuda")
    sm, si, coef = torch.empty(K, device="cuda"), torch.empty(K, device="cuda"), torch.empty(2 * K, device="cuda")
    ops.conv2d_fwd_bn(ctx, xd, wd, z, 1, 0, partial, counters, gamma.cuda(), beta.cuda(), rm, rv, sm, si, coef, tile_cfg=2)
    ops.bn_apply_fwd(ctx, z, y, coef, relu=True)
    torch.cuda.synchronize()
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    close(sm, mean_ref, torch.float32, "bn mean", rtol=tol)
    close(si, invstd_ref, torch.float32, "bn invstd", rtol=tol)
    close(rv, rv_ref, torch.float32, "running var", rtol=tol)
    close(y, y_ref, dtype, "bn y", rtol=tol)
    assert torch.all(counters == 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,C", BN_CASES)
@pytest.mark.parametrize("masked", [False, True])
def test_bn_bwd(ctx, dtype, rows, C, masked):
    from sirius_amd import ops
    g = _gen(7)
    x = (rnd((1, 1, rows, C), dtype, g) * 1.3 - 0.2).to(dtype)
    dy = rnd(x.shape, dtype, g)
    mask = rnd(x.shape, dtype, g) if masked else None
    gamma = torch.rand(C, generator=g) + 0.5
    dx_ref, dg_ref, db_ref = O.bn_bwd(dy, x, gamma, relu_mask=mask)
    x2 = x.float().reshape(-1, C)
    mean, invstd = x2.mean(0), 1.0 / torch.sqrt(x2.var(0, unbiased=False) + 1e-5)
    dx = torch.empty(x.shape, dtype=dtype, device="cuda")
    dg, db = torch.zeros(C, device="cuda"), torch.zeros(C, device="cuda")
    ws = torch.empty(ops.bn_workspace_bytes(ops.dtype_code(x), rows, C) // 4, dtype=torch.float32, device="cuda")
    ops.bn_bwd(ctx, dy.cuda(), x.cuda(), dx, gamma.cuda(), mean.cuda(), invstd.cuda(), dg, db, ws,
               relu_mask=mask.cuda() if masked else None)
    torch.cuda.synchronize()
    close(dg, dg_ref, torch.float32, "bn dgamma", rtol=1e-3)
    close(db, db_ref, torch.float32, "bn dbeta", rtol=1e-3)
    close(dx, dx_ref, dtype, "bn dx", rtol=1e-3 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [CONV_CASES[0], CONV_CASES[1], CONV_CASES[3], CONV_CASES[4], CONV_CASES[6], CONV_CASES[10], CONV_CASES[13]])
@pytest.mark.parametrize("tile_cfg", [-1, 0, 1, 2, 3, 5, 6, 7, 9, 10, 11, 12, 13, 14])
@pytest.mark.parametrize("with_add", [False, True])
def test_conv_dgrad_with_bn_backward_sums(ctx, dtype, case, tile_cfg, with_add):
    """The data-gradient convolution gates its output by the ReLU of the BatchNorm it flows into and
    leaves that BatchNorm's two reductions; the BatchNorm backward starts from them.  Checked against
    the oracle's dgrad -> (ReLU gate) -> BatchNorm backward chain on the same inputs."""
    from sirius_amd import ops
    N, H, W, C, K, R, S, st, pad = case
    print("case", case, dtype, tile_cfg, with_add, flush=True)
    g = _gen(22)
    Ho, Wo = ops.conv_out_hw(H, W, R, S, st, pad)
    dy = rnd((N, Ho, Wo, K), dtype, g)
    w = rnd((K, R, S, C), dtype, g, (R * S * K) ** -0.5)
    add = rnd((N, H, W, C), dtype, g) if with_add else None
    z = (rnd((N, H, W, C), dtype, g) * 1.3 - 0.2).to(dtype)     # the BatchNorm's input
    relu_out = rnd((N, H, W, C), dtype, g)                        # its ReLU output: only the sign matters
    gamma = torch.rand(C, generator=g) + 0.5
    z2 = z.float().reshape(-1, C)
    mean, invstd = z2.mean(0), 1.0 / torch.sqrt(z2.var(0, unbiased=False) + 1e-5)
    # oracle chain; the gradient is rounded to the storage type between the two operators
    g_ref = O.conv2d_dgrad(dy, w, (N, H, W, C), st, pad)
    if with_add:
        g_ref = g_ref + add.float()
    g_ref = g_ref.to(dtype)
    dz_ref, dg_ref, db_ref = O.bn_bwd(g_ref, z, gamma, relu_mask=relu_out)
    gated_ref = g_ref.float() * (relu_out.float() > 0)

    d = lambda t: t.cuda() if t is not None else None
    gx = torch.empty((N, H, W, C), dtype=dtype, device="cuda")
    rb = ops.conv2d_dgrad_stat_rows(gx, K, R, S, st, pad, tile_cfg)
    partial = torch.full((rb * C * 2,), float("nan"), device="cuda")
    zd = z.cuda()
    got_rb = ops.conv2d_dgrad_bnsums(ctx, dy.cuda(), ops.filter_transpose(ctx, w.cuda()), gx, st, pad, zd, mean.cuda(),
                                     invstd.cuda(), partial, bn_mask=relu_out.cuda(), add=d(add), tile_cfg=tile_cfg)
    assert got_rb == rb
    dz = torch.empty_like(gx)
    dg, db = torch.zeros(C, device="cuda"), torch.zeros(C, device="cuda")
    scratch = torch.empty(3 * C, device="cuda")
    ops.bn_bwd_partials(ctx, gx, zd, dz, gamma.cuda(), mean.cuda(), invstd.cuda(), dg, db, partial, rb, scratch)
    torch.cuda.synchronize()
    close(gx, gated_ref, dtype, "gated gradient")
    assert ((gx.float().cpu() == 0) | (relu_out.float() > 0)).all(), "the gradient must be zero behind a closed ReLU"
    # the sums are those of what was stored, exactly
    g32 = gx.float().cpu().reshape(-1, C).double()
    xhat = (z2 - mean).double() * invstd.double()
    sums = partial.cpu().reshape(rb, C, 2).double().sum(0)
    close(sums[:, 0].float(), g32.sum(0).float(), torch.float32, "sum g", rtol=1e-4)
    close(sums[:, 1].float(), (g32 * xhat).sum(0).float(), torch.float32, "sum g*xhat", rtol=1e-4)
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    close(dg, dg_ref, torch.float32, "bn dgamma", rtol=tol)
    close(db, db_ref, torch.float32, "bn dbeta", rtol=tol)
    close(dz, dz_ref, dtype, "bn dx", rtol=tol)
    # the same with the coefficients computed as part of the convolution call; twice, on the same counters
    counters = torch.zeros(C // 64 + 1, dtype=torch.int32, device="cuda")
    for _ in range(2):
        gx2, dz2 = torch.empty_like(gx), torch.empty_like(gx)
        dg2, db2 = torch.zeros(C, device="cuda"), torch.zeros(C, device="cuda")
        coef = torch.full((3 * C,), float("nan"), device="cuda")
        partial.fill_(float("nan"))
        ops.conv2d_dgrad_bn(ctx, dy.cuda(), ops.filter_transpose(ctx, w.cuda()), gx2, st, pad, zd, mean.cuda(),
                            invstd.cuda(), partial, counters, gamma.cuda(), dg2, db2, coef, bn_mask=relu_out.cuda(),
                            add=d(add), tile_cfg=tile_cfg)
        ops.bn_apply_bwd(ctx, gx2, zd, dz2, coef)
        torch.cuda.synchronize()
        assert torch.equal(gx2, gx) and torch.all(counters == 0)
        close(dg2, dg.cpu(), torch.float32, "fused finalize: dgamma", rtol=1e-6)
        close(db2, db.cpu(), torch.float32, "fused finalize: dbeta", rtol=1e-6)
        close(dz2, dz.float().cpu(), dtype, "fused finalize: dx", rtol=1e-5 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 16, 16, 64), (1, 7, 9, 8), (3, 112, 112, 16)])
def test_maxpool(ctx, dtype, shape):
    from sirius_amd import ops
    g = _gen(8)
    x = torch.relu(rnd(shape, dtype, g))  # post-ReLU: zeros tie constantly
    y_ref, idx_ref = O.maxpool_fwd(x, 3, 2, 1)
    N, Ho, Wo, C = y_ref.shape
    y = torch.empty(y_ref.shape, dtype=dtype, device="cuda")
    idx = torch.empty(y_ref.shape, dtype=torch.int32, device="cuda")
    ops.maxpool_fwd(ctx, x.cuda(), y, idx, 3, 2, 1)
    torch.cuda.synchronize()
    assert torch.equal(y.float().cpu(), y_ref), "maxpool values must be exact"
    assert torch.equal(idx.cpu().long(), idx_ref), "maxpool argmax indices must be bit-exact (first maximum wins)"
    dy = rnd(y_ref.shape, dtype, g)
    dx_ref = O.maxpool_bwd(dy, x, 3, 2, 1)
    dx = torch.empty(shape, dtype=dtype, device="cuda")
    ops.maxpool_bwd(ctx, dy.cuda(), idx, dx, 3, 2, 1)
    torch.cuda.synchronize()
    close(dx, dx_ref, dtype, "maxpool bwd", rtol=1e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_avgpool(ctx, dtype):
    from sirius_amd import ops
    g = _gen(9)
    x = rnd((3, 7, 7, 64), dtype, g)
    y = torch.empty((3, 64), dtype=dtype, device="cuda")
    ops.avgpool_fwd(ctx, x.cuda(), y)
    dy = rnd((3, 64), dtype, g)
    dx = torch.empty(x.shape, dtype=dtype, device="cuda")
    ops.avgpool_bwd(ctx, dy.cuda(), dx)
    torch.cuda.synchronize()
    close(y, O.avgpool_fwd(x), dtype, "avgpool fwd", rtol=1e-5 if dtype == torch.float32 else 1e-2)
    close(dx, O.avgpool_bwd(dy, x.shape), dtype, "avgpool bwd", rtol=1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,classes,scale", [(4, 1000, 1.0), (64, 1000, 0.25), (3, 10, 1.0)])
def test_softmax_ce(ctx, dtype, rows, classes, scale):
    from sirius_amd import ops
    g = _gen(10)
    z = torch.randn(rows, classes, generator=g) * 3
    labels = torch.randint(0, classes, (rows,), generator=g)
    rows_ref, mean_ref, g_ref = O.softmax_ce(z, labels, scale)
    loss_rows, loss_mean = torch.empty(rows, device="cuda"), torch.empty(1, device="cuda")
    ld = (classes + 7) // 8 * 8
    dz = torch.zeros(rows, ld, dtype=dtype, device="cuda")
    ops.softmax_ce_fwd_bwd(ctx, z.cuda(), labels.cuda(), loss_rows, loss_mean, dz, loss_scale=scale)
    torch.cuda.synchronize()
    close(loss_rows, rows_ref, torch.float32, "ce rows", rtol=1e-5)
    close(loss_mean, mean_ref.reshape(1), torch.float32, "ce mean", rtol=1e-5)
    close(dz[:, :classes], g_ref, dtype, "ce grad", rtol=1e-4 if dtype == torch.float32 else 1e-2)
    assert (dz[:, classes:] == 0).all()


@pytest.mark.parametrize("n", [1024, 1000003])
@pytest.mark.parametrize("offset", [0, 1])   # 1: the buffers start 4 bytes past a 16-byte boundary (scalar accesses)
def test_sgd_and_accumulate(ctx, n, offset):
    from sirius_amd import ops
    g = _gen(11)
    p, gr, buf = torch.randn(n, generator=g), torch.randn(n, generator=g), torch.zeros(n)
    p_ref, buf_ref = O.sgd_momentum(p, gr, buf, 0.1, 0.9, 1e-4, steps=2)

    def dev(t):
        d = torch.zeros(n + offset, device="cuda")[offset:]
        d.copy_(t)
        return d
    p_d, g_d, b_d = dev(p), dev(gr), dev(buf)
    shadow = torch.empty(n + offset, dtype=torch.bfloat16, device="cuda")[offset:]
    for _ in range(2):
        ops.sgd_momentum_step(ctx, p_d, g_d, b_d, 0.1, 0.9, 1e-4, shadow=shadow)
    torch.cuda.synchronize()
    close(p_d, p_ref, torch.float32, "sgd param", rtol=1e-6)
    close(b_d, buf_ref, torch.float32, "sgd momentum", rtol=1e-6)
    assert torch.equal(shadow.cpu(), p_d.cpu().to(torch.bfloat16)), "bf16 shadow must be the RNE rounding of the master"
    acc = torch.randn(n, generator=g)
    acc_d, g_al = acc.cuda(), gr.cuda()
    ops.grad_accumulate(ctx, acc_d, g_al)
    torch.cuda.synchronize()
    assert torch.equal(acc_d.cpu(), acc + gr) and (g_al == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layout_and_cast(ctx, dtype):
    from sirius_amd import ops
    g = _gen(12)
    x = torch.randn(2, 3, 10, 12, generator=g)
    y = torch.empty(2, 10, 12, 8, dtype=dtype, device="cuda")
    ops.nchw_to_nhwc_pad(ctx, x.cuda(), y)
    torch.cuda.synchronize()
    ref = torch.zeros(2, 10, 12, 8)
    ref[..., :3] = x.permute(0, 2, 3, 1)
    assert torch.equal(y.cpu(), ref.to(dtype)), "layout conversion must round exactly like torch"
    src = torch.randn(1001, generator=g)
    dst = torch.empty(1001, dtype=dtype, device="cuda")
    back = torch.empty(1001, device="cuda")
    ops.cast_from_f32(ctx, src.cuda(), dst)
    ops.cast_to_f32(ctx, dst, back)
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), src.to(dtype)) and torch.equal(back.cpu(), src.to(dtype).float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(16, 1000), (8192, 2304), (1000, 72), (257, 8)])
def test_bias_grad(ctx, dtype, rows, cols):
    """few rows (a batch of logits) and many rows (tokens of a transformer projection)"""
    from sirius_amd import ops
    g = _gen(13)
    dy = rnd((rows, cols), dtype, g)
    db = torch.ones(cols, device="cuda")
    ops.bias_grad(ctx, dy.cuda(), db)
    torch.cuda.synchronize()
    close(db, dy.double().sum(0).float(), torch.float32, "bias grad", rtol=1e-5)
    ops.bias_grad(ctx, dy.cuda(), db, accumulate=True)
    torch.cuda.synchronize()
    close(db, 2 * dy.double().sum(0).float(), torch.float32, "bias grad accumulated", rtol=1e-5)
    # with scratch memory (rows summed in slabs); a scratch too small for two slabs falls back to one
    for floats in (64 * cols, 3 * cols, cols):
        ws = torch.full((floats,), float("nan"), device="cuda")
        db2 = torch.ones(cols, device="cuda")
        ops.bias_grad(ctx, dy.cuda(), db2, accumulate=True, workspace=ws)
        torch.cuda.synchronize()
        close(db2, 1 + dy.double().sum(0).float(), torch.float32, "bias grad with scratch", rtol=1e-5)


def test_program_record_replay(ctx):
    """A recorded program replays the same launches: results equal the eager ones."""
    from sirius_amd import ops
    g = _gen(14)
    x, w = rnd((2, 8, 8, 32), torch.bfloat16, g).cuda(), rnd((64, 3, 3, 32), torch.bfloat16, g, 0.06).cuda()
    y_eager = torch.empty((2, 8, 8, 64), dtype=torch.bfloat16, device="cuda")
    ops.conv2d_fwd(ctx, x, w, y_eager, 1, 1)
    prog = ops.Program()
    y_prog = torch.zeros_like(y_eager)
    ctx.begin_record(prog)
    ops.conv2d_fwd(ctx, x, w, y_prog, 1, 1)
    ctx.end_record()
    torch.cuda.synchronize()
    assert len(prog) == 1 and (y_prog == 0).all(), "recording must not launch"
    for _ in range(3):
        y_prog.zero_()
        assert ctx.run(prog) is False
        torch.cuda.synchronize()
        assert torch.equal(y_prog, y_eager)


def test_kernel_timed_inside_a_two_lane_program(ctx):
    """tch_program_time_kernel: the launches of one kernel timed by their own begin / end timestamps while the
    program runs on its two lanes -- every launch of that name is counted, the duration is a kernel's (more than
    nothing, far less than the replay's wall time), the results stay those of a plain replay, and a name no
    launch carries counts nothing."""
    import time
    from sirius_amd import ops
    g = _gen(15)
    x = rnd((8, 28, 28, 64), torch.bfloat16, g).cuda()
    w = rnd((64, 3, 3, 64), torch.bfloat16, g, 0.04).cuda()
    ys = [torch.zeros((8, 28, 28, 64), dtype=torch.bfloat16, device="cuda") for _ in range(6)]
    dws = [torch.zeros((64, 3, 3, 64), device="cuda") for _ in range(6)]
    ws = torch.empty(ops.conv2d_wgrad_workspace_bytes(ops.dtype_code(x), 64, 3, 3, 64, ops.conv2d_wgrad_splits(x, 64, 3, 3, 1, 1)) // 4 + 64,
                     device="cuda")
    prog = ops.Program()
    ctx.begin_record(prog)
    try:
        for y, dw in zip(ys, dws):
            ops.conv2d_fwd(ctx, x, w, y, 1, 1)
            with ctx.side_lane(wait_main=True):     # reads what the main-lane launch before it wrote
                ops.conv2d_wgrad(ctx, x, y, dw, 1, 1, workspace=ws)
        ctx.join()
    finally:
        ctx.end_record()
    ctx.run(prog)
    ctx.synchronize()
    torch.cuda.synchronize()
    want_y, want_dw = [y.clone() for y in ys], [d.clone() for d in dws]
    names = {r["name"]: r["launches"] for r in ctx.profile(prog, 1)}
    fwd = next(n for n in names if "fwd" in n)
    wg = next(n for n in names if n.startswith("wgrad_kernel"))
    t0 = time.perf_counter()
    us_fwd, n_fwd = ctx.time_kernel(prog, fwd, 2)        # main-lane kernel whose stop event is also the fork
    wall_us = (time.perf_counter() - t0) * 1e6
    us_wg, n_wg = ctx.time_kernel(prog, wg, 2)           # second-lane kernel
    assert n_fwd == names[fwd] == 6 and n_wg == names[wg] == 6
    assert 1.0 < us_fwd < wall_us / 2 and 1.0 < us_wg < 5000.0, (us_fwd, us_wg, wall_us)
    assert ctx.time_kernel(prog, "no_such_kernel", 1) == (0.0, 0)
    torch.cuda.synchronize()
    for y, d, wy, wd in zip(ys, dws, want_y, want_dw):
        assert torch.equal(y, wy) and torch.equal(d, wd)
