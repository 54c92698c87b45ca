"""CPU: pin the operator oracle (oracle/nn_ops.py) against closed forms and brute force
(oracle/brute.py), and the ResNet oracle against what the architecture fixes.

The reference's own tests hold no vectors for this path (its scripts compare unseeded GPU
and CPU runs), so these pins are what stands between the oracle and a plausible mistake.
"""
import numpy as np
import pytest
import torch

from oracle import brute as B
from oracle import nn_ops as O
from oracle import resnet as R


def _t(a):
    return torch.from_numpy(np.asarray(a)).float()


CASES = [(1, 5, 6, 3, 4, 3, 3, 1, 1), (2, 6, 6, 2, 3, 3, 3, 2, 1), (1, 7, 5, 2, 2, 1, 1, 2, 0), (1, 8, 8, 3, 2, 7, 7, 2, 3)]


@pytest.mark.parametrize("case", CASES)
def test_conv_oracle_against_seven_loops(case):
    N, H, W, C, K, Rr, S, st, pad = case
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal((N, H, W, C)), rng.standard_normal((K, Rr, S, C))
    y = B.conv2d_fwd(x, w, st, pad)
    np.testing.assert_allclose(O.conv2d_fwd(_t(x), _t(w), st, pad).numpy(), y, rtol=1e-4, atol=1e-5)
    dy = rng.standard_normal(y.shape)
    np.testing.assert_allclose(O.conv2d_dgrad(_t(dy), _t(w), x.shape, st, pad).numpy(),
                               B.conv2d_dgrad(dy, w, x.shape, st, pad), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(O.conv2d_wgrad(_t(x), _t(dy), w.shape, st, pad).numpy(),
                               B.conv2d_wgrad(x, dy, w.shape, st, pad), rtol=1e-4, atol=1e-5)


def test_conv_gradients_are_adjoint():
    """<conv(x,w), dy> = <x, dgrad(dy,w)> = <w, wgrad(x,dy)>: fails on a transposed operand or a flipped tap."""
    rng = np.random.default_rng(1)
    x, w = rng.standard_normal((2, 9, 7, 4)), rng.standard_normal((5, 3, 3, 4))
    for st, pad in ((1, 1), (2, 1), (2, 0)):
        y = O.conv2d_fwd(_t(x), _t(w), st, pad)
        dy = torch.randn(y.shape, generator=torch.Generator().manual_seed(2))
        lhs = (y * dy).sum().item()
        assert abs(lhs - (_t(x) * O.conv2d_dgrad(dy, _t(w), x.shape, st, pad)).sum().item()) < 1e-3 * abs(lhs) + 1e-3
        assert abs(lhs - (_t(w) * O.conv2d_wgrad(_t(x), dy, w.shape, st, pad)).sum().item()) < 1e-3 * abs(lhs) + 1e-3


def test_bn_oracle_against_fp64_statistics():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 4, 6)) * 2 + 0.5
    gamma, beta = rng.random(6) + 0.5, rng.standard_normal(6)
    y, mean, var, var_unb = B.bn_train(x, gamma, beta, 1e-5)
    rm, rv = torch.zeros(6), torch.ones(6)
    y_o, mean_o, invstd_o = O.bn_fwd_train(_t(x), _t(gamma), _t(beta), rm, rv)
    np.testing.assert_allclose(y_o.numpy(), y, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(mean_o.numpy(), mean, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(invstd_o.numpy(), 1 / np.sqrt(var + 1e-5), rtol=1e-5)
    # running statistics: momentum 0.1, UNBIASED variance
    np.testing.assert_allclose(rm.numpy(), 0.1 * mean, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(rv.numpy(), 0.9 + 0.1 * var_unb, rtol=1e-5)
    dy = rng.standard_normal(x.shape)
    dx, dg, db = B.bn_bwd(dy, x, gamma, 1e-5)
    dx_o, dg_o, db_o = O.bn_bwd(_t(dy), _t(x), _t(gamma))
    np.testing.assert_allclose(dx_o.numpy(), dx, rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(dg_o.numpy(), dg, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(db_o.numpy(), db, rtol=1e-4, atol=1e-5)
    # ReLU gate: the oracle's mask argument is dy * (mask > 0)
    mask = rng.standard_normal(x.shape)
    dx_m, _, _ = B.bn_bwd(dy * (mask > 0), x, gamma, 1e-5)
    np.testing.assert_allclose(O.bn_bwd(_t(dy), _t(x), _t(gamma), relu_mask=_t(mask))[0].numpy(), dx_m, rtol=1e-3,
                               atol=1e-5)


def test_maxpool_first_maximum_rule():
    # the documented probe: zeros 4x4, k3 s2 p1 -> [[0, 1], [4, 5]]
    y, idx = O.maxpool_fwd(torch.zeros(1, 4, 4, 1), 3, 2, 1)
    assert idx[0, :, :, 0].tolist() == [[0, 1], [4, 5]]
    rng = np.random.default_rng(4)
    x = np.maximum(rng.standard_normal((2, 9, 8, 3)), 0).astype(np.float32)  # ties at zero
    x[0, 3, 3, 1] = np.nan
    yb, ib = B.maxpool_first_max(x, 3, 2, 1)
    yo, io = O.maxpool_fwd(torch.from_numpy(x), 3, 2, 1)
    assert np.array_equal(io.numpy(), ib)
    np.testing.assert_array_equal(np.nan_to_num(yo.numpy(), nan=-7), np.nan_to_num(yb, nan=-7))


def test_cross_entropy_and_sgd_closed_forms():
    rng = np.random.default_rng(5)
    z, labels = rng.standard_normal((6, 11)) * 3, rng.integers(0, 11, 6)
    rows, mean, grad = B.cross_entropy(z, labels)
    rows_o, mean_o, grad_o = O.softmax_ce(_t(z), torch.from_numpy(labels), 0.25)
    np.testing.assert_allclose(rows_o.numpy(), rows, rtol=1e-5)
    np.testing.assert_allclose(mean_o.item(), mean, rtol=1e-5)
    np.testing.assert_allclose(grad_o.numpy(), 0.25 * grad, rtol=1e-4, atol=1e-7)
    # a hand-computed probe: p=1, g=1, lr .1, mu .9, wd 1e-4 -> 0.89999 then 0.70997
    p1, _ = B.sgd_scalar(1.0, 1.0, 0.1, 0.9, 1e-4, 1)
    p2, _ = B.sgd_scalar(1.0, 1.0, 0.1, 0.9, 1e-4, 2)
    assert abs(p1 - 0.89999) < 1e-6 and abs(p2 - 0.70997) < 2e-5
    po, _ = O.sgd_momentum(torch.ones(1), torch.ones(1), torch.zeros(1), 0.1, 0.9, 1e-4, steps=2)
    assert abs(po.item() - p2) < 1e-6


def test_resnet_oracle_matches_the_architecture():
    m = R.make_model()
    assert sum(p.numel() for p in m.parameters()) == 60192808
    convs = [c for c in m.modules() if isinstance(c, torch.nn.Conv2d)]
    assert len(convs) == 155
    assert [len(getattr(m, f"layer{i}")) for i in (1, 2, 3, 4)] == [3, 8, 36, 3]
    assert m.layer2[0].conv2.stride == (2, 2) and m.layer2[0].conv1.stride == (1, 1)  # stride on the 3x3
    small = R.make_model((1, 1, 1, 1), 16, 16)
    x, y = R.make_batch(2, 64, 16)
    assert small(x).shape == (2, 16)
    # micro-batching with scaled losses reproduces the full-batch gradient when BN sees the same
    # statistics, i.e. for micro_batches == 1; and exactly one optimizer step is taken per call
    before = {k: v.clone() for k, v in small.state_dict().items()}
    (losses, grads), = R.train_steps(small, x, y, 1, micro_batches=2)
    assert len(losses) == 2
    after = small.state_dict()
    k = "fc.bias"
    expect = before[k] - 0.1 * (grads[k] + 1e-4 * before[k])
    assert torch.allclose(after[k], expect, rtol=1e-5, atol=1e-7)
