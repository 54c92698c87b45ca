"""Transformer operators on the GPU (LayerNorm, GELU, attention softmax, AdamW, embedding, batched GEMM),
called through the C ABI, against the CPU oracle (oracle/seq_ops.py) on the same seeded inputs.

Tolerances: fp32 rtol 1e-3, bf16 rtol 2e-2 against the largest magnitude of the oracle tensor (the
path's stated bound); tighter where an operator is purely elementwise.
"""
import pytest
import torch

from oracle import seq_ops as S

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2}


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def rnd(shape, dtype, g, scale=1.0):
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(got, ref, dtype, what, rtol=None):
    rtol = RTOL[dtype] if rtol is None else rtol
    got, ref = got.detach().float().cpu(), ref.detach().float()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    scale = ref.abs().max().item() + 1e-12
    err = (got - ref).abs().max().item()
    assert err <= rtol * scale, f"{what}: max err {err:.3e} > {rtol:g} * {scale:.3e}"


LN_CASES = [(8 * 49, 128), (3 * 197, 768), (1000, 1024), (5, 8), (4100, 256)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,C", LN_CASES)
def test_layernorm(ctx, dtype, rows, C):
    from sirius_amd import ops
    print("case", rows, C, dtype, flush=True)
    g = _gen(31)
    x = (rnd((rows, C), dtype, g) * 1.5 + 0.3).to(dtype)
    gamma, beta = torch.rand(C, generator=g) + 0.5, torch.randn(C, generator=g) * 0.2
    y_ref, mean_ref, rstd_ref = S.layernorm(x, gamma, beta)
    xd = x.cuda()
    y = torch.empty_like(xd)
    mean, rstd = torch.empty(rows, device="cuda"), torch.empty(rows, device="cuda")
    ops.layernorm_fwd(ctx, xd, y, gamma.cuda(), beta.cuda(), mean, rstd)
    dy = rnd((rows, C), dtype, g)
    dx_ref, dg_ref, db_ref = S.layernorm_bwd(dy, x, gamma)
    dx = torch.empty_like(xd)
    dg, db = torch.full((C,), 3.0, device="cuda"), torch.full((C,), -2.0, device="cuda")
    partial = torch.empty(ops.layernorm_bwd_partial_rows(rows) * C * 2, device="cuda")
    ops.layernorm_bwd(ctx, dy.cuda(), xd, dx, gamma.cuda(), mean, rstd, dg, db, partial)
    # accumulate on top
    dg2, db2 = dg.clone(), db.clone()
    torch.cuda.synchronize()
    res = rnd((rows, C), dtype, g)
    dx_res = torch.empty_like(xd)
    ops.layernorm_bwd(ctx, dy.cuda(), xd, dx_res, gamma.cuda(), mean, rstd, dg2, db2, partial, accumulate=True,
                      residual=res.cuda())
    torch.cuda.synchronize()
    close(dx_res, dx_ref + res.float(), dtype, "ln dx + residual", rtol=1e-3 if dtype == torch.float32 else 1e-2)
    close(mean, mean_ref, torch.float32, "ln mean", rtol=1e-4)
    close(rstd, rstd_ref, torch.float32, "ln rstd", rtol=1e-4)
    close(y, y_ref, dtype, "ln y", rtol=1e-4 if dtype == torch.float32 else 1e-2)
    close(dx, dx_ref, dtype, "ln dx", rtol=1e-3 if dtype == torch.float32 else 1e-2)
    close(dg, dg_ref, torch.float32, "ln dgamma", rtol=1e-3)
    close(db, db_ref, torch.float32, "ln dbeta", rtol=1e-3)
    close(dg2, 2 * dg_ref, torch.float32, "ln dgamma accumulated", rtol=1e-3)
    close(db2, 2 * db_ref, torch.float32, "ln dbeta accumulated", rtol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tanh_form", [False, True])
@pytest.mark.parametrize("n", [8, 4096 * 3 + 8, 1 << 20])
def test_gelu(ctx, dtype, tanh_form, n):
    from sirius_amd import ops
    g = _gen(32)
    x = rnd((n,), dtype, g, 2.0)
    x[:8] = torch.tensor([0.0, -0.0, 1e-4, -1e-4, 6.0, -6.0, 12.0, -12.0]).to(dtype)
    dy = rnd((n,), dtype, g)
    y, dx = torch.empty(n, dtype=dtype, device="cuda"), torch.empty(n, dtype=dtype, device="cuda")
    ops.gelu_fwd(ctx, x.cuda(), y, tanh_form)
    ops.gelu_bwd(ctx, dy.cuda(), x.cuda(), dx, tanh_form)
    torch.cuda.synchronize()
    tol = 1e-5 if dtype == torch.float32 else 8e-3   # bf16: one rounding of the output
    close(y, S.gelu(x, tanh_form), dtype, "gelu", rtol=tol)
    close(dx, S.gelu_bwd(dy, x, tanh_form), dtype, "gelu bwd", rtol=tol)


SOFTMAX_CASES = [
    # batch, heads, L, windows (0: no mask), bias, causal
    (8, 4, 49, 4, True, False),     # Swin window attention with the shift mask
    (6, 3, 49, 0, True, False),     # unshifted block
    (2, 12, 128, 0, False, True),   # GPT-2, short
    (1, 2, 1024, 0, False, True),   # GPT-2 sequence length
    (3, 1, 7, 0, False, False),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", SOFTMAX_CASES)
def test_attn_softmax(ctx, dtype, case):
    from sirius_amd import ops
    Bn, Hn, L, nW, with_bias, causal = case
    print("case", case, dtype, flush=True)
    g = _gen(33)
    s = rnd((Bn, Hn, L, L), dtype, g, 3.0)
    bias = torch.randn(Hn, L, L, generator=g) if with_bias else None
    mask = torch.where(torch.rand(nW, L, L, generator=g) > 0.6, -100.0, 0.0) if nW else None
    scale = 0.17
    p_ref = S.attn_softmax(s, scale, bias, mask, causal)
    d = lambda t: t.cuda() if t is not None else None
    p = torch.empty((Bn, Hn, L, L), dtype=dtype, device="cuda")
    ops.attn_softmax_fwd(ctx, s.cuda(), p, scale, d(bias), d(mask), causal)
    torch.cuda.synchronize()
    close(p, p_ref, dtype, "softmax", rtol=1e-5 if dtype == torch.float32 else 8e-3)
    if causal:
        assert torch.all(p.float().cpu().triu(1) == 0), "keys after the query must get probability zero"
    # in place
    s2 = s.cuda()
    ops.attn_softmax_fwd(ctx, s2, s2, scale, d(bias), d(mask), causal)
    torch.cuda.synchronize()
    assert torch.equal(s2, p), "in-place softmax must match the out-of-place one bit for bit"
    # backward from the kernel's own (rounded) probabilities
    dp = rnd((Bn, Hn, L, L), dtype, g)
    pf = p.float().cpu()
    ds_ref = scale * pf * (dp.float() - (dp.float() * pf).sum(-1, keepdim=True))
    ds = torch.empty_like(p)
    ops.attn_softmax_bwd(ctx, p, dp.cuda(), ds, scale)
    torch.cuda.synchronize()
    close(ds, ds_ref, dtype, "softmax bwd", rtol=1e-4 if dtype == torch.float32 else 1e-2)
    if dtype == torch.float32:
        close(ds, S.attn_softmax_bwd(s, dp, scale, bias, mask, causal), dtype, "softmax bwd vs autograd", rtol=1e-4)
    if causal:
        # the causal form never reads dp beyond the query's own position: poison it
        poisoned = dp.clone().float()
        poisoned[..., torch.triu(torch.ones(L, L, dtype=torch.bool), 1)] = float("nan")
        ds2 = torch.full_like(p, 5.0)
        ops.attn_softmax_bwd(ctx, p, poisoned.to(dtype).cuda(), ds2, scale, causal=True)
        torch.cuda.synchronize()
        close(ds2, ds_ref, dtype, "causal softmax bwd", rtol=1e-4 if dtype == torch.float32 else 1e-2)
        assert torch.all(ds2.float().cpu().triu(1) == 0)


@pytest.mark.parametrize("n", [5, 1000, (1 << 20) + 3])
@pytest.mark.parametrize("with_shadow", [False, True])
@pytest.mark.parametrize("offset", [0, 1])   # 1: the buffers start 4 bytes past a 16-byte boundary (scalar accesses)
def test_adamw(ctx, n, with_shadow, offset):
    from sirius_amd import ops
    g = _gen(34)
    p0 = torch.randn(n, generator=g)
    grads = [torch.randn(n, generator=g) * (0.1 + i) for i in range(3)]
    hp = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.05)
    p_ref, m_ref, v_ref = S.adamw(p0, grads, hp["lr"], hp["beta1"], hp["beta2"], hp["eps"], hp["weight_decay"])
    p = torch.zeros(n + offset, device="cuda")[offset:]
    p.copy_(p0)
    m, v = torch.zeros(n + offset, device="cuda")[offset:], torch.zeros(n + offset, device="cuda")[offset:]
    step, scal = torch.zeros(1, dtype=torch.int32, device="cuda"), torch.zeros(2, device="cuda")
    shadow = torch.empty(n + offset, dtype=torch.bfloat16, device="cuda")[offset:] if with_shadow else None
    for gi in grads:
        ops.adamw_step(ctx, p, gi.cuda(), m, v, step, scal, shadow=shadow, **hp)
        torch.cuda.synchronize()
    assert step.item() == 3
    close(p, p_ref, torch.float32, "adamw param", rtol=1e-5)
    close(m, m_ref, torch.float32, "adamw exp_avg", rtol=1e-5)
    close(v, v_ref, torch.float32, "adamw exp_avg_sq", rtol=1e-5)
    if with_shadow:
        assert torch.equal(shadow, p.to(torch.bfloat16)), "the bf16 shadow is the rounded parameter, bit for bit"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,C,vocab", [(2, 16, 64, 101), (3, 37, 768, 5000), (1, 1, 8, 3)])
def test_embedding(ctx, dtype, B, T, C, vocab):
    from sirius_amd import ops
    g = _gen(35)
    wte, wpe = rnd((vocab, C), dtype, g), rnd((T + 3, C), dtype, g)
    ids = torch.randint(0, vocab, (B, T), generator=g)
    if B * T > 4:
        ids.view(-1)[:4] = ids.view(-1)[0]   # a token that repeats
    out = torch.empty((B, T, C), dtype=dtype, device="cuda")
    ops.embedding_fwd(ctx, ids.cuda(), wte.cuda(), wpe.cuda(), out)
    torch.cuda.synchronize()
    close(out, S.embedding(ids, wte, wpe), dtype, "embedding", rtol=1e-6 if dtype == torch.float32 else 8e-3)
    dy = rnd((B, T, C), dtype, g)
    dwte_ref, dwpe_ref = S.embedding_bwd(ids, dy, vocab, T + 3)
    dwte = torch.zeros((vocab, C), device="cuda")
    dwpe = torch.full((T + 3, C), 9.0, device="cuda")
    ops.embedding_bwd(ctx, ids.cuda(), dy.cuda(), dwte, dwpe)
    torch.cuda.synchronize()
    close(dwte, dwte_ref, torch.float32, "dwte", rtol=1e-5)
    close(dwpe[:T], dwpe_ref[:T], torch.float32, "dwpe", rtol=1e-5)
    assert torch.all(dwpe[T:] == 9.0), "positions past the sequence are not touched"
    # with the chain scratch: the same values, on top of what the rows already hold (the tied head's gradient), and
    # the same bits on every run -- one thread adds the rows of a repeated token in position order
    base = rnd((vocab, C), torch.float32, g)
    chain = torch.full((2 * B * T,), -7, dtype=torch.int32, device="cuda")
    runs = []
    for _ in range(3):
        d = base.clone().cuda()
        dp = torch.zeros((T + 3, C), device="cuda")
        ops.embedding_bwd(ctx, ids.cuda(), dy.cuda(), d, dp, chain=chain)
        torch.cuda.synchronize()
        runs.append((d.clone(), dp.clone()))
    close(runs[0][0] - base.cuda(), dwte_ref, torch.float32, "dwte (chained)", rtol=1e-4)
    close(runs[0][1][:T], dwpe_ref[:T], torch.float32, "dwpe (chained)", rtol=1e-5)
    assert all(torch.equal(runs[0][0], r[0]) and torch.equal(runs[0][1], r[1]) for r in runs[1:])


def _attention_layouts(B, H, T, D):
    """Offsets of head h of sample b inside a packed [B, T, 3, H, D] projection (GPT-2's c_attn output)."""
    C = H * D
    return dict(row=3 * C, batch=(T * 3 * C, D), q0=0, k0=C, v0=2 * C)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,H,T,D", [(2, 3, 49, 32), (1, 2, 200, 64), (2, 2, 64, 64), (1, 1, 5, 8)])
def test_batched_gemm_attention_products(ctx, dtype, B, H, T, D):
    """Every product of an attention layer and of its backward, on strided views of one packed qkv tensor,
    against einsum on the CPU: Q K^T, P V, P^T dO, dO V^T, dS K, dS^T Q."""
    from sirius_amd import ops
    print("case", B, H, T, D, dtype, flush=True)
    g = _gen(36)
    C = H * D
    qkv = rnd((B, T, 3, H, D), dtype, g)
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3).float() for i in range(3))     # [B, H, T, D]
    lay = _attention_layouts(B, H, T, D)
    qkv_d = qkv.cuda()
    flat = qkv_d.view(-1)
    qv, kv, vv = flat[lay["q0"]:], flat[lay["k0"]:], flat[lay["v0"]:]
    sb = (H * T * T, T * T)   # scores [B, H, T, T]
    ob = (T * C, D)           # output [B, T, H, D]
    tol = 1e-3 if dtype == torch.float32 else 2e-2

    s = torch.full((B, H, T, T), 7.0, dtype=dtype, device="cuda")
    ops.batched_gemm(ctx, qv, kv, s, T, T, D, (lay["row"], 1), (lay["row"], 1), T, (B, H), lay["batch"], lay["batch"], sb,
                     alpha=0.25)
    torch.cuda.synchronize()
    close(s, 0.25 * torch.einsum("bhtd,bhsd->bhts", q, k), dtype, "Q K^T", rtol=tol)

    p = rnd((B, H, T, T), dtype, g, 0.2)
    p_d = p.cuda()
    o = torch.empty((B, T, H, D), dtype=dtype, device="cuda")
    ops.batched_gemm(ctx, p_d, vv, o, T, D, T, (T, 1), (1, lay["row"]), C, (B, H), sb, lay["batch"], ob)
    torch.cuda.synchronize()
    o_ref = torch.einsum("bhts,bhsd->bthd", p.float(), v)
    close(o, o_ref, dtype, "P V", rtol=tol)

    do = rnd((B, T, H, D), dtype, g)
    do_d = do.cuda()
    dof = do.float().permute(0, 2, 1, 3)                                        # [B, H, T, D]
    dqkv = torch.zeros((B, T, 3, H, D), dtype=dtype, device="cuda")
    dflat = dqkv.view(-1)
    # dV[s, d] = sum_t P[t, s] dO[t, d]
    ops.batched_gemm(ctx, p_d, do_d, dflat[lay["v0"]:], T, D, T, (1, T), (1, C), lay["row"], (B, H), sb, ob, lay["batch"])
    # dP[t, s] = sum_d dO[t, d] V[s, d]
    dp = torch.empty((B, H, T, T), dtype=dtype, device="cuda")
    ops.batched_gemm(ctx, do_d, vv, dp, T, T, D, (C, 1), (lay["row"], 1), T, (B, H), ob, lay["batch"], sb)
    ds = rnd((B, H, T, T), dtype, g, 0.3)
    ds_d = ds.cuda()
    # dQ[t, d] = sum_s dS[t, s] K[s, d];  dK[s, d] = sum_t dS[t, s] Q[t, d]
    ops.batched_gemm(ctx, ds_d, kv, dflat[lay["q0"]:], T, D, T, (T, 1), (1, lay["row"]), lay["row"], (B, H), sb,
                     lay["batch"], lay["batch"])
    ops.batched_gemm(ctx, ds_d, qv, dflat[lay["k0"]:], T, D, T, (1, T), (1, lay["row"]), lay["row"], (B, H), sb,
                     lay["batch"], lay["batch"])
    torch.cuda.synchronize()
    close(dp, torch.einsum("bhtd,bhsd->bhts", dof, v), dtype, "dO V^T", rtol=tol)
    got = dqkv.float().cpu()
    close(got[:, :, 2], torch.einsum("bhts,bhtd->bshd", p.float(), dof), dtype, "P^T dO", rtol=tol)
    close(got[:, :, 0], torch.einsum("bhts,bhsd->bthd", ds.float(), k), dtype, "dS K", rtol=tol)
    close(got[:, :, 1], torch.einsum("bhts,bhtd->bshd", ds.float(), q), dtype, "dS^T Q", rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D", [(200, 64), (64, 16), (130, 32)])
def test_batched_gemm_causal_forms(ctx, dtype, T, D):
    """What a causal mask leaves of a square problem: (1) only the lower triangle of the output is wanted and the
    tiles above the diagonal stay untouched; (2) / (3) A is lower / upper triangular and the reduction is cut."""
    from sirius_amd import ops
    g = _gen(38)
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    Z = 3
    q, k = rnd((Z, T, D), dtype, g), rnd((Z, T, D), dtype, g)
    s = torch.full((Z, T, T), 7.0, dtype=dtype, device="cuda")
    ops.batched_gemm(ctx, q.cuda(), k.cuda(), s, T, T, D, (D, 1), (D, 1), T, (Z, 1), (T * D, 0), (T * D, 0), (T * T, 0),
                     causal=1)
    torch.cuda.synchronize()
    ref = torch.einsum("ztd,zsd->zts", q.float(), k.float())
    low = torch.tril(torch.ones(T, T, dtype=torch.bool))
    got = s.float().cpu()
    close(got * low, ref * low, dtype, "lower triangle", rtol=tol)
    tiles = (torch.arange(T)[None, :] // 64) > (torch.arange(T)[:, None] // 64)      # tiles wholly above the diagonal
    assert torch.all(got[:, tiles] == 7.0), "tiles above the diagonal must be left unwritten"
    p_low = (rnd((Z, T, T), dtype, g, 0.3).float() * low).to(dtype)
    v = rnd((Z, T, D), dtype, g)
    o = torch.empty((Z, T, D), dtype=dtype, device="cuda")
    ops.batched_gemm(ctx, p_low.cuda(), v.cuda(), o, T, D, T, (T, 1), (1, D), D, (Z, 1), (T * T, 0), (T * D, 0),
                     (T * D, 0), causal=2)
    o_t = torch.empty((Z, T, D), dtype=dtype, device="cuda")
    ops.batched_gemm(ctx, p_low.cuda(), v.cuda(), o_t, T, D, T, (1, T), (1, D), D, (Z, 1), (T * T, 0), (T * D, 0),
                     (T * D, 0), causal=3)
    torch.cuda.synchronize()
    close(o, torch.einsum("zts,zsd->ztd", p_low.float(), v.float()), dtype, "P V, lower-triangular P", rtol=tol)
    close(o_t, torch.einsum("zts,ztd->zsd", p_low.float(), v.float()), dtype, "P^T dO, lower-triangular P", rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_batched_gemm_accumulate_and_edges(ctx, dtype):
    """Sizes off every tile edge, an unaligned base, accumulate on top of existing values."""
    from sirius_amd import ops
    g = _gen(37)
    M, N, K = 70, 33, 45
    a, b = rnd((M * K + 1,), dtype, g), rnd((N, K), dtype, g)
    a_d = a.cuda()
    c = torch.ones((M, N), dtype=dtype, device="cuda")
    ops.batched_gemm(ctx, a_d[1:], b.cuda(), c, M, N, K, (K, 1), (K, 1), N, accumulate=True, alpha=0.5)
    torch.cuda.synchronize()
    ref = 1.0 + 0.5 * a[1:].float().view(M, K) @ b.float().t()
    close(c, ref, dtype, "accumulate", rtol=1e-3 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,T,packed", [(2, 3, 256, True), (1, 2, 128, False), (1, 1, 512, True)])
def test_flash_attention(ctx, B, H, T, packed, causal):
    """Fused attention forward and backward against the oracle's scores -> softmax -> context chain.  The
    oracle sees the same bf16-rounded inputs; bf16 tolerance (2e-2 of the largest magnitude per tensor)."""
    from sirius_amd import ops
    D, C = 64, H * 64
    g = _gen(40 + T + B)
    dtype = torch.bfloat16
    scale = 1.0 / 8.0
    if packed:
        qkv = rnd((B, T, 3 * C), dtype, g)
        q, k, v = qkv[..., :C], qkv[..., C:2 * C], qkv[..., 2 * C:]
        dev = qkv.cuda()
        flat = dev.view(-1)
        dq_, dk_, dv_ = flat, flat[C:], flat[2 * C:]
        strides = (3 * C, T * 3 * C)
        dgrad = torch.zeros_like(dev)
        gflat = dgrad.view(-1)
        gq, gk, gv = gflat, gflat[C:], gflat[2 * C:]
    else:
        q, k, v = (rnd((B, T, C), dtype, g) for _ in range(3))
        dq_, dk_, dv_ = (t.cuda().view(-1) for t in (q, k, v))
        strides = (C, T * C)
        gq, gk, gv = (torch.zeros(B * T * C, dtype=dtype, device="cuda") for _ in range(3))
    dout = rnd((B, T, C), dtype, g)

    def heads(t):
        return t.reshape(B, T, H, D).permute(0, 2, 1, 3)
    o_ref, lse_ref = S.attention(heads(q), heads(k), heads(v), scale, causal)
    dq_ref, dk_ref, dv_ref = S.attention_bwd(heads(q), heads(k), heads(v), heads(dout), scale, causal)

    o = torch.zeros(B, T, C, dtype=dtype, device="cuda")
    lse = torch.zeros(B * H, T, dtype=torch.float32, device="cuda")
    delta = torch.zeros(B * H, T, dtype=torch.float32, device="cuda")
    ops.flash_attn_fwd(ctx, dq_, dk_, dv_, o.view(-1), lse, B, H, T, strides, (C, T * C), scale, causal)
    ctx.synchronize()
    close(heads(o.cpu()), o_ref, dtype, "context")
    close(lse.view(B, H, T), lse_ref, torch.float32, "log-sum-exp", rtol=2e-3)
    d_dev = dout.cuda()
    ops.flash_attn_bwd(ctx, dq_, dk_, dv_, o.view(-1), d_dev.view(-1), lse, delta, gq, gk, gv, B, H, T, strides,
                       (C, T * C), scale, causal)
    ctx.synchronize()
    delta_ref = (heads(dout).float() * o_ref).sum(-1)
    close(delta.view(B, H, T), delta_ref, dtype, "delta")
    if packed:
        got = dgrad.cpu()
        got_q, got_k, got_v = got[..., :C], got[..., C:2 * C], got[..., 2 * C:]
    else:
        got_q, got_k, got_v = (t.cpu().view(B, T, C) for t in (gq, gk, gv))
    close(heads(got_q), dq_ref, dtype, "dq")
    close(heads(got_k), dk_ref, dtype, "dk")
    close(heads(got_v), dv_ref, dtype, "dv")


def test_flash_attention_rejects_bad_shapes(ctx):
    from sirius_amd import ops
    t = torch.zeros(2 * 100 * 64, dtype=torch.bfloat16, device="cuda")
    lse = torch.zeros(2 * 100, dtype=torch.float32, device="cuda")
    with pytest.raises(Exception, match="multiple of 128"):
        ops.flash_attn_fwd(ctx, t, t, t, t, lse, 2, 1, 100, (64, 100 * 64), (64, 100 * 64), 0.125)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,classes,ld", [(37, 50257, 50304), (64, 97, 128), (19, 1001, 1001), (8, 70001, 70008)])
def test_softmax_ce_lm(ctx, dtype, rows, classes, ld):
    """Language-model cross entropy (mean over rows with a label >= 0) and its gradient against torch's CPU
    cross_entropy with ignore_index; covers the rows-in-registers kernel (aligned rows of at most 65536 classes)
    and the looping one (unaligned leading dimension, longer rows)."""
    from sirius_amd import ops
    g = _gen(rows + classes)
    z = torch.randn(rows, ld, generator=g) * 3.0
    labels = torch.randint(0, classes, (rows,), generator=g)
    labels[::5] = -100
    valid = int((labels >= 0).sum())
    zr = z[:, :classes].clone().requires_grad_(True)
    loss_ref = torch.nn.functional.cross_entropy(zr, labels, ignore_index=-100) * 0.5
    (g_ref,) = torch.autograd.grad(loss_ref, zr)
    zd = z.cuda()
    dl = torch.full((rows, ld), 7.0, dtype=dtype, device="cuda")
    loss_rows = torch.zeros(rows, device="cuda")
    loss = torch.zeros(1, device="cuda")
    ops.softmax_ce_lm(ctx, zd, labels.cuda(), loss_rows, loss, dl, classes, valid, loss_scale=0.5)
    ctx.synchronize()
    assert abs(loss.item() * 0.5 - loss_ref.item()) <= 1e-4 * abs(loss_ref.item()), (loss.item(), loss_ref.item())
    close(dl[:, :classes], g_ref, dtype, "dlogits")
    assert torch.all(dl[labels.cuda() < 0][:, :classes] == 0)
    pad = dl[:, (classes + 3) // 4 * 4:]
    assert torch.all(pad == 7.0), "columns beyond the last four-float piece are not touched"
