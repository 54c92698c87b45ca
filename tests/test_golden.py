"""Committed golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py) against
(a) the torch-CPU oracle -- CPU tests, and (b) the HIP kernels through the C ABI -- GPU tests.

The vectors come from float64 brute force (operators) and a float64 torch step (tiny ResNet); the
oracle and the kernels compute in fp32, so the bars are: oracle vs vector 1e-5 (norm-wise), HIP
fp32 vs vector 1e-3, integer indices bit-exact."""
import os

import numpy as np
import pytest
import torch

from oracle import nn_ops as O
from oracle import resnet as oracle_resnet

HERE = os.path.dirname(os.path.abspath(__file__))
TINY = dict(depths=(1, 1, 1, 1), num_classes=8, width=8)


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(HERE, "golden", "ops_small.npz"))


@pytest.fixture(scope="module")
def tiny():
    return np.load(os.path.join(HERE, "golden", "resnet_tiny.npz"))


def t32(a):
    return torch.from_numpy(np.asarray(a)).float()


def close(got, ref, rtol, what):
    got = torch.as_tensor(got).detach().double().cpu()
    ref = torch.as_tensor(np.asarray(ref)).double()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    scale = ref.abs().max().item() + 1e-30
    err = (got - ref).abs().max().item()
    assert err <= rtol * scale, f"{what}: max err {err:.3e} > {rtol:g} * {scale:.3e}"


# ------------------------------------------------------------------ oracle vs vectors (CPU)

@pytest.mark.parametrize("i", range(4))
def test_oracle_conv_against_vectors(vec, i):
    N, H, W, C, K, R, s, p = (int(v) for v in vec[f"conv{i}_cfg"])
    x, w, dy = t32(vec[f"conv{i}_x"]), t32(vec[f"conv{i}_w"]), t32(vec[f"conv{i}_dy"])
    close(O.conv2d_fwd(x, w, s, p), vec[f"conv{i}_y"], 1e-5, "conv fwd")
    close(O.conv2d_dgrad(dy, w, x.shape, s, p), vec[f"conv{i}_dx"], 1e-5, "conv dgrad")
    close(O.conv2d_wgrad(x, dy, w.shape, s, p), vec[f"conv{i}_dw"], 1e-5, "conv wgrad")


@pytest.mark.parametrize("i", range(2))
def test_oracle_bn_against_vectors(vec, i):
    g = lambda k: vec[f"bn{i}_{k}"]
    x, gamma, beta = t32(g("x")), t32(g("gamma")), t32(g("beta"))
    C = x.shape[1]
    rm, rv = torch.zeros(C), torch.ones(C)
    y, mean, invstd = O.bn_fwd_train(x.reshape(1, 1, -1, C), gamma, beta, rm, rv)
    close(y.reshape(-1, C), g("y"), 1e-5, "bn y")
    close(mean, g("mean"), 1e-5, "bn mean")
    close(invstd, 1.0 / np.sqrt(g("var") + 1e-5), 1e-5, "bn invstd")
    # running statistics: momentum 0.1, unbiased variance (what F.batch_norm stores)
    close(rm, 0.1 * g("mean"), 1e-5, "running mean")
    close(rv, 0.9 + 0.1 * g("var_unbiased"), 1e-5, "running var")
    dx, dg, db = O.bn_bwd(t32(g("dy")).reshape(1, 1, -1, C), x.reshape(1, 1, -1, C), gamma)
    close(dx.reshape(-1, C), g("dx"), 1e-4, "bn dx")
    close(dg, g("dgamma"), 1e-5, "bn dgamma")
    close(db, g("dbeta"), 1e-5, "bn dbeta")


def test_oracle_pool_ce_sgd_against_vectors(vec):
    y, idx = O.maxpool_fwd(t32(vec["pool_x"]), 3, 2, 1)
    assert np.array_equal(y.numpy(), vec["pool_y"].astype(np.float32))
    assert np.array_equal(idx.numpy(), vec["pool_idx"]), "first maximum wins on ties"
    rows, mean, dz = O.softmax_ce(t32(vec["ce_logits"]), torch.from_numpy(vec["ce_labels"]))
    close(rows, vec["ce_rows"], 1e-6, "ce rows")
    close(mean, vec["ce_mean"], 1e-6, "ce mean")
    close(dz, vec["ce_dlogits"], 1e-6, "ce grad")
    p, _ = O.sgd_momentum(t32(vec["sgd_p"]), t32(vec["sgd_g"]), torch.zeros(32), 0.1, 0.9, 1e-4, steps=3)
    close(p, vec["sgd_p3"], 1e-6, "sgd three steps")


def _tiny_state(tiny, prefix):
    return {k[len(prefix):]: torch.from_numpy(tiny[k]) for k in tiny.files if k.startswith(prefix)}


def test_oracle_resnet_step_against_vectors(tiny):
    model = oracle_resnet.ResNet(**TINY)
    sd = _tiny_state(tiny, "w0/")
    missing = model.load_state_dict(sd, strict=False)
    assert all("num_batches_tracked" in k for k in missing.missing_keys) and not missing.unexpected_keys
    x, y = torch.from_numpy(tiny["x"]), torch.from_numpy(tiny["y"])
    (losses, grads), = oracle_resnet.train_steps(model, x, y, 1, lr=0.1, momentum=0.9, weight_decay=1e-4)
    assert abs(losses[0] - float(tiny["loss"][0])) <= 1e-5 * abs(float(tiny["loss"][0]))
    for k, g in grads.items():
        close(g, tiny["grad/" + k], 2e-4, "grad " + k)
    after = model.state_dict()
    for k, v in _tiny_state(tiny, "w1/").items():
        close(after[k], v, 1e-4, "after step " + k)


# ------------------------------------------------------------------ HIP vs vectors (GPU)

@pytest.mark.gpu
@pytest.mark.parametrize("i", range(4))
def test_hip_conv_against_vectors(ctx, vec, i):
    from sirius_amd import ops
    N, H, W, C, K, R, s, p = (int(v) for v in vec[f"conv{i}_cfg"])
    print("golden conv", i, (N, H, W, C, K, R, s, p), flush=True)
    x, w, dy = t32(vec[f"conv{i}_x"]), t32(vec[f"conv{i}_w"]), t32(vec[f"conv{i}_dy"])
    if C % 4:
        pytest.skip("channel count below one 16-byte chunk")
    xd, wd, dyd = x.cuda(), w.cuda(), dy.cuda()
    y = torch.empty(dy.shape, device="cuda")
    ops.conv2d_fwd(ctx, xd, wd, y, s, p)
    dx = torch.empty(x.shape, device="cuda")
    ops.conv2d_dgrad(ctx, dyd, ops.filter_transpose(ctx, wd), dx, s, p)
    dw = torch.empty(w.shape, device="cuda")
    ops.conv2d_wgrad(ctx, xd, dyd, dw, s, p)
    torch.cuda.synchronize()
    close(y, vec[f"conv{i}_y"], 1e-3, "conv fwd")
    close(dx, vec[f"conv{i}_dx"], 1e-3, "conv dgrad")
    close(dw, vec[f"conv{i}_dw"], 1e-3, "conv wgrad")


@pytest.mark.gpu
@pytest.mark.parametrize("i", range(2))
def test_hip_bn_against_vectors(ctx, vec, i):
    from sirius_amd import ops
    g = lambda k: vec[f"bn{i}_{k}"]
    x = t32(g("x"))
    rows, C = x.shape
    x4 = x.reshape(1, 1, rows, C).cuda()
    y = torch.empty_like(x4)
    rm, rv = torch.zeros(C, device="cuda"), torch.ones(C, device="cuda")
    sm, si = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    ws = torch.empty(ops.bn_workspace_bytes(ops.dtype_code(x4), rows, C) // 4, dtype=torch.float32, device="cuda")
    gamma = t32(g("gamma")).cuda()
    ops.bn_fwd_train(ctx, x4, y, gamma, t32(g("beta")).cuda(), rm, rv, sm, si, ws, relu=False)
    dx = torch.empty_like(x4)
    dg, db = torch.zeros(C, device="cuda"), torch.zeros(C, device="cuda")
    ops.bn_bwd(ctx, t32(g("dy")).reshape(1, 1, rows, C).cuda(), x4, dx, gamma, sm, si, dg, db, ws)
    torch.cuda.synchronize()
    close(y.reshape(rows, C), g("y"), 1e-4, "bn y")
    close(sm, g("mean"), 1e-5, "bn mean")
    close(si, 1.0 / np.sqrt(g("var") + 1e-5), 1e-5, "bn invstd")
    close(rm, 0.1 * g("mean"), 1e-5, "running mean")
    close(rv, 0.9 + 0.1 * g("var_unbiased"), 1e-5, "running var")
    close(dx.reshape(rows, C), g("dx"), 1e-3, "bn dx")
    close(dg, g("dgamma"), 1e-4, "bn dgamma")
    close(db, g("dbeta"), 1e-4, "bn dbeta")


@pytest.mark.gpu
def test_hip_pool_ce_sgd_against_vectors(ctx, vec):
    from sirius_amd import ops
    x = t32(vec["pool_x"]).cuda()
    y = torch.empty(vec["pool_y"].shape, device="cuda")
    idx = torch.empty(vec["pool_y"].shape, dtype=torch.int32, device="cuda")
    ops.maxpool_fwd(ctx, x, y, idx, 3, 2, 1)
    z = t32(vec["ce_logits"]).cuda()
    rows, classes = z.shape
    loss_rows, loss_mean = torch.empty(rows, device="cuda"), torch.empty(1, device="cuda")
    dz = torch.zeros(rows, classes, device="cuda")
    ops.softmax_ce_fwd_bwd(ctx, z, torch.from_numpy(vec["ce_labels"]).cuda(), loss_rows, loss_mean, dz)
    p, gr, buf = t32(vec["sgd_p"]).cuda(), t32(vec["sgd_g"]).cuda(), torch.zeros(32, device="cuda")
    for _ in range(3):
        ops.sgd_momentum_step(ctx, p, gr, buf, 0.1, 0.9, 1e-4)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), vec["pool_y"].astype(np.float32))
    assert np.array_equal(idx.cpu().numpy().astype(np.int64), vec["pool_idx"]), "indices must be bit-exact"
    close(loss_rows, vec["ce_rows"], 1e-5, "ce rows")
    close(loss_mean.reshape(()), vec["ce_mean"], 1e-5, "ce mean")
    close(dz, vec["ce_dlogits"], 1e-4, "ce grad")
    close(p, vec["sgd_p3"], 1e-6, "sgd three steps")


@pytest.mark.gpu
def test_hip_resnet_step_against_vectors(tiny):
    from sirius_amd.resnet import ResNetEngine
    eng = ResNetEngine(dtype=torch.float32, image_size=32, lr=0.1, momentum=0.9, weight_decay=1e-4, **TINY)
    eng.load_state_dict(_tiny_state(tiny, "w0/"))
    x, y = torch.from_numpy(tiny["x"]).cuda(), torch.from_numpy(tiny["y"]).cuda()
    plan, cut = eng.forward_backward(x, y)
    assert not cut
    torch.cuda.synchronize()
    loss = float(plan.loss.item())
    assert abs(loss - float(tiny["loss"][0])) <= 1e-4 * abs(float(tiny["loss"][0]))
    grads = eng.grads_dict()
    for k in (k[5:] for k in tiny.files if k.startswith("grad/")):
        close(grads[k], tiny["grad/" + k], 1e-3, "grad " + k)
    eng.optimizer_step()
    after = eng.state_dict()
    for k, v in _tiny_state(tiny, "w1/").items():
        close(after[k], v, 1e-3, "after step " + k)
