"""Compute-unit partitioning between training and the colocated tenant (the reference's SMPartitioner,
common/sm_partition.cc:26-112, with compute units in the place of TPCs).  CPU part: the share arithmetic and
the demand field of the shared board.  GPU part: a context with a limit runs the same kernels, with the same
results, on fewer compute units (slower), and an engine step under a limit equals the unrestricted one."""
import os

import pytest
import torch

from sirius_amd._lib import lib


def test_train_share_arithmetic():
    L = lib()
    assert L.tch_cu_partition_init(256, 8, 0) == 0
    assert L.tch_cu_partition_total() == 256
    # GetTrainAvailTpcNum: max(min, total - required) capped at max (sm_partition.cc:96-106)
    assert [L.tch_cu_partition_train_avail(r) for r in (0, 100, 248, 255, 300, -5)] == [256, 156, 8, 8, 8, 256]
    assert L.tch_cu_partition_init(256, 16, 128) == 0
    assert [L.tch_cu_partition_train_avail(r) for r in (0, 128, 200, 250)] == [128, 128, 56, 16]
    assert L.tch_cu_partition_init(64, 100, 32) < 0          # min above max
    assert L.tch_cu_partition_init(256, 8, 0) == 0


def test_required_compute_units_on_the_board(monkeypatch):
    L = lib()
    monkeypatch.setenv("SIRIUS_PORT", str(42000 + os.getpid() % 1000))
    L.tch_TorchColShutdown()
    assert L.tch_InfTraCommunicator_Init(1, 1, 1) == 0
    try:
        assert L.tch_infer_required_cus_get(0) == 0
        assert L.tch_infer_required_cus_set(0, 96) == 0
        assert L.tch_infer_required_cus_add(0, 32) == 128 and L.tch_infer_required_cus_add(0, -64) == 64
        assert L.tch_infer_required_cus_get(0) == 64 and L.tch_infer_required_cus_get(1) == 0
        assert L.tch_infer_required_cus_set(0, -1) < 0
    finally:
        L.tch_TorchColShutdown()


@pytest.mark.gpu
def test_limited_context_runs_the_same_kernels_slower(ctx):
    from sirius_amd import ops
    L = lib()
    assert L.tch_cu_partition_init(0, 8, 0) == 0
    total = L.tch_cu_partition_total()
    assert total >= 64
    g = torch.Generator()
    g.manual_seed(0)
    x = torch.randn(32, 56, 56, 256, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(256, 3, 3, 256, generator=g) * 0.02).to(torch.bfloat16).cuda()
    prog = ops.Program()
    y = torch.empty(32, 56, 56, 256, dtype=torch.bfloat16, device="cuda")
    ctx.begin_record(prog)
    for _ in range(4):
        ops.conv2d_fwd(ctx, x, w, y, 1, 1)
    ctx.end_record()

    def timed(limit):
        ctx.set_cu_limit(limit)
        assert ctx.cu_limit() == (0 if limit in (0, total) else limit)
        y.zero_()
        ctx.run(prog)
        ctx.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        ctx.run(prog)
        e1.record()
        ctx.synchronize()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1), y.clone()

    try:
        t_full, y_full = timed(0)
        t_half, y_half = timed(total // 2)
        t_eighth, y_eighth = timed(total // 8)
        t_back, y_back = timed(0)
    finally:
        ctx.set_cu_limit(0)
    print(f"conv 4x: all CUs {t_full:.3f} ms, half {t_half:.3f} ms, an eighth {t_eighth:.3f} ms, all again {t_back:.3f} ms",
          flush=True)
    assert torch.equal(y_full, y_half) and torch.equal(y_full, y_eighth) and torch.equal(y_full, y_back)
    assert t_half > 1.4 * t_full and t_eighth > 2.0 * t_half
    assert t_back < 1.3 * t_full


@pytest.mark.gpu
def test_engine_step_under_a_share_equals_the_unrestricted_step():
    from sirius_amd.resnet import ResNetEngine
    L = lib()
    assert L.tch_cu_partition_init(0, 8, 0) == 0
    total = L.tch_cu_partition_total()
    g = torch.Generator()
    g.manual_seed(1)
    x, y = torch.randn(8, 3, 64, 64, generator=g).cuda(), torch.randint(0, 16, (8,), generator=g).cuda()
    outs = []
    for share in (None, [total // 4, total // 2, total]):
        eng = ResNetEngine((1, 1, 1, 1), 16, 16, dtype=torch.bfloat16, image_size=64)
        eng.init_kaiming(2)
        if share is not None:
            it = iter(share * 1000)
            eng.set_cu_share_provider(lambda: next(it))          # a different share at every launch segment
            eng.set_checkpoint_hook(lambda phase, name: None)    # cut the program into per-layer segments
        p, cut = eng.forward_backward(x, y)
        eng.synchronize()
        outs.append((p.loss.item(), eng.grads.clone()))
        eng.ctx.set_cu_limit(0)
    assert outs[0][0] == outs[1][0] and torch.equal(outs[0][1], outs[1][1])

