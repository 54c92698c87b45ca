"""tch_conv2d_wgrad_static: the weight gradient for callers that cannot allocate (split-K partials in the library's
static device buffer) against tch_conv2d_wgrad with a caller-provided workspace, through the C ABI.

Same kernels, same split count => the two results are equal bit for bit.  Two calls in a row, the second on a
smaller problem (the buffer still holds the first call's partials), then once more the large one; device memory in
use does not change across the calls; a split count whose partials exceed the buffer is refused with a message."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(ctx, dtype, N, H, W, C, K, R, stride, pad, splits, seed):
    from sirius_amd import ops
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, H, W, C, generator=g).to(dtype).cuda()
    Ho, Wo = ops.conv_out_hw(H, W, R, R, stride, pad)
    dy = torch.randn(N, Ho, Wo, K, generator=g).to(dtype).cuda()
    code = ops.dtype_code(x)
    if splits <= 0:
        splits = ops.conv2d_wgrad_splits(x, K, R, R, stride, pad)
    need = ops.conv2d_wgrad_workspace_bytes(code, K, R, R, C, splits)
    assert need <= ops.conv2d_wgrad_static_capacity_bytes()
    ws = torch.empty(max(1, need // 4), device="cuda")
    ref = torch.full((K, R, R, C), 3.0, device="cuda")
    ops.conv2d_wgrad(ctx, x, dy, ref, stride, pad, workspace=ws, splits=splits)
    got = torch.full((K, R, R, C), -7.0, device="cuda")
    ctx.synchronize()
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0 = torch.cuda.memory_allocated()
    ops.conv2d_wgrad_static(ctx, x, dy, got, stride, pad, splits=splits)
    ctx.synchronize()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == alloc0
    free1, _ = torch.cuda.mem_get_info()
    return got, ref, splits, free0 - free1


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_weight_gradient_equals_the_workspace_one(ctx, dtype):
    from sirius_amd import ops
    from sirius_amd._lib import TorchColHipError
    # warm-up: the first use on a device looks the buffer's address up (no allocation, but the code object loads)
    _case(ctx, dtype, 2, 8, 8, 64, 64, 1, 1, 0, 4, 0)
    big = (16, 28, 28, 128, 128, 3, 1, 1, 12, 1)      # 3x3, 12 splits of 147 456 + 128 floats
    small = (4, 14, 14, 64, 256, 1, 1, 0, 5, 2)       # 1x1, fewer and smaller partials
    grown = []
    for i, case in enumerate((big, small, big)):
        print("case", dtype, case, flush=True)
        got, ref, splits, used = _case(ctx, dtype, *case)
        assert splits > 1
        assert torch.equal(got, ref), f"call {i}: static-scratch result differs from the workspace result"
        grown.append(used)
    assert grown[1] <= 0 and grown[2] <= 0, f"device memory in use grew across the calls: {grown}"
    # library-chosen split count, accumulate on top of existing values
    g = torch.Generator().manual_seed(9)
    x = torch.randn(8, 14, 14, 256, generator=g).to(dtype).cuda()
    dy = torch.randn(8, 14, 14, 512, generator=g).to(dtype).cuda()
    code = ops.dtype_code(x)
    sp = ops.conv2d_wgrad_splits(x, 512, 1, 1, 1, 0)
    ws = torch.empty(max(1, ops.conv2d_wgrad_workspace_bytes(code, 512, 1, 1, 256, sp) // 4), device="cuda")
    ref = torch.ones(512, 1, 1, 256, device="cuda")
    got = torch.ones(512, 1, 1, 256, device="cuda")
    ops.conv2d_wgrad(ctx, x, dy, ref, 1, 0, workspace=ws, accumulate=True)
    ops.conv2d_wgrad_static(ctx, x, dy, got, 1, 0, accumulate=True)
    ctx.synchronize()
    assert torch.equal(got, ref)
    # beyond the buffer: 512 x 3 x 3 x 512 filter = 9.4 MB of partials per split, 8 splits = 75 MB > 64 MiB
    xb = torch.zeros(8, 7, 7, 512, dtype=dtype, device="cuda")
    dyb = torch.zeros(8, 7, 7, 512, dtype=dtype, device="cuda")
    dwb = torch.zeros(512, 3, 3, 512, device="cuda")
    with pytest.raises(TorchColHipError, match="static buffer holds"):
        ops.conv2d_wgrad_static(ctx, xb, dyb, dwb, 1, 1, splits=8)
    # the library's own choice is lowered to what fits instead
    ops.conv2d_wgrad_static(ctx, xb, dyb, dwb, 1, 1)
    ctx.synchronize()
    assert float(dwb.abs().max()) == 0.0


def test_two_streams_share_the_static_buffer_in_order():
    """Calls that launch at once on two different streams of one GPU: the library makes the second wait for the first
    one's reduction (on the device, no host synchronisation in between), so both results equal the workspace form bit
    for bit although the two problems overwrite each other's partials."""
    from sirius_amd import ops
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    c1, c2 = ops.Context(s1), ops.Context(s2)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(5)
    xa = torch.randn(16, 28, 28, 128, generator=g).to(dtype).cuda()
    dya = torch.randn(16, 28, 28, 128, generator=g).to(dtype).cuda()
    xb = torch.randn(8, 14, 14, 256, generator=g).to(dtype).cuda()
    dyb = torch.randn(8, 14, 14, 512, generator=g).to(dtype).cuda()
    main = ops.Context(torch.cuda.current_stream())
    code = ops.dtype_code(xa)
    wsa = torch.empty(ops.conv2d_wgrad_workspace_bytes(code, 128, 3, 3, 128, 12) // 4, device="cuda")
    wsb = torch.empty(ops.conv2d_wgrad_workspace_bytes(code, 512, 1, 1, 256, 6) // 4, device="cuda")
    refa = torch.zeros(128, 3, 3, 128, device="cuda")
    refb = torch.zeros(512, 1, 1, 256, device="cuda")
    ops.conv2d_wgrad(main, xa, dya, refa, 1, 1, workspace=wsa, splits=12)
    ops.conv2d_wgrad(main, xb, dyb, refb, 1, 0, workspace=wsb, splits=6)
    main.synchronize()
    torch.cuda.synchronize()
    gota = [torch.empty_like(refa) for _ in range(6)]
    gotb = [torch.empty_like(refb) for _ in range(6)]
    print("two streams, 6 rounds", flush=True)
    for i in range(6):          # no host synchronisation inside the loop
        ops.conv2d_wgrad_static(c1, xa, dya, gota[i], 1, 1, splits=12)
        ops.conv2d_wgrad_static(c2, xb, dyb, gotb[i], 1, 0, splits=6)
    c1.synchronize()
    c2.synchronize()
    torch.cuda.synchronize()
    for i in range(6):
        assert torch.equal(gota[i], refa), f"round {i}: the 3x3 problem on stream 1"
        assert torch.equal(gotb[i], refb), f"round {i}: the 1x1 problem on stream 2"
