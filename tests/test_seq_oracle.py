"""Pins for the transformer-operator oracle (oracle/seq_ops.py), on the CPU.

The reference holds no stored expectations for these operators (its tests compare GPU with CPU on
unseeded inputs), so each oracle function is checked against what the mathematics fixes: closed
forms in float64, scalar recurrences, brute-force loops on tiny inputs.
"""
import math

import numpy as np
import torch

from oracle import seq_ops as S


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def test_layernorm_closed_form_fp64():
    g = _gen(0)
    x = torch.randn(5, 24, generator=g) * 2 + 0.5
    gamma, beta = torch.rand(24, generator=g) + 0.5, torch.randn(24, generator=g)
    y, mean, rstd = S.layernorm(x, gamma, beta)
    xn = x.double().numpy()
    mu = xn.mean(-1, keepdims=True)
    var = ((xn - mu) ** 2).mean(-1, keepdims=True)          # biased
    ref = (xn - mu) / np.sqrt(var + 1e-5) * gamma.double().numpy() + beta.double().numpy()
    np.testing.assert_allclose(y.numpy(), ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(mean.numpy(), mu[:, 0], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(rstd.numpy(), 1 / np.sqrt(var[:, 0] + 1e-5), rtol=1e-5)


def test_layernorm_bwd_closed_form_fp64():
    g = _gen(1)
    x, dy = torch.randn(4, 16, generator=g), torch.randn(4, 16, generator=g)
    gamma = torch.rand(16, generator=g) + 0.5
    dx, dg, db = S.layernorm_bwd(dy, x, gamma)
    xn, gn, gam = x.double().numpy(), dy.double().numpy(), gamma.double().numpy()
    mu = xn.mean(-1, keepdims=True)
    rstd = 1 / np.sqrt(((xn - mu) ** 2).mean(-1, keepdims=True) + 1e-5)
    xh = (xn - mu) * rstd
    gg = gn * gam
    ref = rstd * (gg - gg.mean(-1, keepdims=True) - xh * (gg * xh).mean(-1, keepdims=True))
    np.testing.assert_allclose(dx.numpy(), ref, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dg.numpy(), (gn * xh).sum(0), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(db.numpy(), gn.sum(0), rtol=1e-4, atol=1e-5)


def test_gelu_forms():
    x = torch.linspace(-6, 6, 241)
    erf_form = 0.5 * x.double() * (1 + torch.erf(x.double() / math.sqrt(2)))
    assert torch.allclose(S.gelu(x).double(), erf_form, atol=1e-6)
    assert torch.allclose(S.gelu(x, tanh_form=True), S.gelu_new_closed_form(x), atol=1e-6)
    # the two forms differ: a mix-up must fail
    assert (S.gelu(x) - S.gelu(x, tanh_form=True)).abs().max() > 1e-4
    # derivative by central differences in float64
    for tanh_form in (False, True):
        h = 1e-4
        xd = x.double()
        f = (lambda t: 0.5 * t * (1 + torch.tanh(math.sqrt(2 / math.pi) * (t + 0.044715 * t ** 3)))) if tanh_form else \
            (lambda t: 0.5 * t * (1 + torch.erf(t / math.sqrt(2))))
        num = (f(xd + h) - f(xd - h)) / (2 * h)
        got = S.gelu_bwd(torch.ones_like(x), x, tanh_form)
        assert torch.allclose(got.double(), num, atol=1e-5)


def test_attention_brute_force():
    """attention() against scalar loops on a tiny causal problem, and its gradients against central differences."""
    g = torch.Generator().manual_seed(5)
    B, H, T, d = 1, 2, 5, 3
    q, k, v = (torch.randn(B, H, T, d, generator=g, dtype=torch.float64) for _ in range(3))
    scale = 0.7
    o, lse = S.attention(q.float(), k.float(), v.float(), scale, causal=True)

    def brute(q, k, v):
        out = torch.zeros(B, H, T, d, dtype=torch.float64)
        ls = torch.zeros(B, H, T, dtype=torch.float64)
        for b in range(B):
            for h in range(H):
                for i in range(T):
                    w = [math.exp(scale * sum(q[b, h, i, e] * k[b, h, j, e] for e in range(d))) for j in range(i + 1)]
                    tot = sum(w)
                    ls[b, h, i] = math.log(tot)
                    for e in range(d):
                        out[b, h, i, e] = sum(w[j] * v[b, h, j, e] for j in range(i + 1)) / tot
        return out, ls
    ob, lb = brute(q, k, v)
    assert torch.allclose(o.double(), ob, atol=1e-5) and torch.allclose(lse.double(), lb, atol=1e-5)
    dout = torch.randn(B, H, T, d, generator=g, dtype=torch.float64)
    dq, dk, dv = S.attention_bwd(q.float(), k.float(), v.float(), dout.float(), scale, causal=True)
    eps = 1e-5
    for name, t, got in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for idx in [(0, 0, 4, 1), (0, 1, 2, 0), (0, 1, 0, 2)]:
            tp, tm = t.clone(), t.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = [tp if n == name else x for n, x in (("q", q), ("k", k), ("v", v))]
            args_m = [tm if n == name else x for n, x in (("q", q), ("k", k), ("v", v))]
            num = ((brute(*args_p)[0] - brute(*args_m)[0]) * dout).sum().item() / (2 * eps)
            assert abs(got[idx].item() - num) <= 1e-4 * max(1.0, abs(num)), (name, idx, got[idx].item(), num)


def test_attn_softmax_brute_force():
    g = _gen(2)
    Bn, Hn, L, nW = 4, 2, 5, 2
    s = torch.randn(Bn, Hn, L, L, generator=g)
    bias = torch.randn(Hn, L, L, generator=g)
    mask = torch.where(torch.rand(nW, L, L, generator=g) > 0.7, -100.0, 0.0)
    p = S.attn_softmax(s, 0.3, bias, mask)
    for b in range(Bn):
        for h in range(Hn):
            for i in range(L):
                z = [0.3 * s[b, h, i, j].item() + bias[h, i, j].item() + mask[b % nW, i, j].item() for j in range(L)]
                m = max(z)
                e = [math.exp(v - m) for v in z]
                for j in range(L):
                    assert abs(p[b, h, i, j].item() - e[j] / sum(e)) < 1e-6
    pc = S.attn_softmax(s, 0.3, causal=True)
    assert torch.all(pc.triu(1) == 0) and torch.allclose(pc.sum(-1), torch.ones(Bn, Hn, L))
    assert abs(pc[0, 0, 0, 0].item() - 1.0) < 1e-7
    # backward: dS = scale * P * (dP - sum(dP * P))
    dp = torch.randn(Bn, Hn, L, L, generator=g)
    ds = S.attn_softmax_bwd(s, dp, 0.3, bias, mask)
    ref = 0.3 * p * (dp - (dp * p).sum(-1, keepdim=True))
    assert torch.allclose(ds, ref, atol=1e-6)


def test_adamw_scalar_recurrence():
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.05
    p0, g0 = 1.0, 0.5
    for steps in (1, 2, 7):
        ref = S.adamw_scalar(p0, g0, lr, b1, b2, eps, wd, steps)
        p, m, v = S.adamw(torch.tensor([p0]), [torch.tensor([g0])] * steps, lr, b1, b2, eps, wd)
        assert abs(p.item() - ref) < 1e-6
    # first step with a constant gradient moves by ~lr (after decay): m_hat / sqrt(v_hat) = sign(g)
    p, _, _ = S.adamw(torch.tensor([p0]), [torch.tensor([g0])], lr, b1, b2, eps, wd)
    assert abs(p.item() - (p0 * (1 - lr * wd) - lr)) < 1e-6


def test_embedding_brute_force():
    g = _gen(3)
    vocab, C, B, T = 11, 8, 2, 5
    wte, wpe = torch.randn(vocab, C, generator=g), torch.randn(7, C, generator=g)
    ids = torch.randint(0, vocab, (B, T), generator=g)
    ids[0, 1] = ids[1, 3] = 4   # a token that repeats
    out = S.embedding(ids, wte, wpe)
    for b in range(B):
        for t in range(T):
            assert torch.equal(out[b, t], wte[ids[b, t]] + wpe[t])
    dy = torch.randn(B, T, C, generator=g)
    dwte, dwpe = S.embedding_bwd(ids, dy, vocab, 7)
    ref = torch.zeros(vocab, C)
    for b in range(B):
        for t in range(T):
            ref[ids[b, t]] += dy[b, t]
    assert torch.allclose(dwte, ref, atol=1e-6)
    assert torch.allclose(dwpe[:T], dy.sum(0), atol=1e-6) and torch.all(dwpe[T:] == 0)
