"""Transformer operator oracle on CPU fp32 (test infrastructure only; see oracle/__init__.py).

Each function is the PyTorch CPU routine the reference's Swin-B / GPT-2 training steps end up in
(reference call sites: train/swin_b.py:38-45, train/gpt2.py:26-33; window attention as written out
in train/swin_b_tiny.py:66-110), with gradients taken by autograd through that same routine.
"""
import torch
import torch.nn.functional as F


def layernorm(x, gamma, beta, eps=1e-5):
    """nn.LayerNorm over the last dimension -> (y, mean, rstd)."""
    xf = x.float()
    y = F.layer_norm(xf, (xf.shape[-1],), gamma, beta, eps)
    mean = xf.mean(-1)
    rstd = 1.0 / torch.sqrt(xf.var(-1, unbiased=False) + eps)
    return y, mean.reshape(-1), rstd.reshape(-1)


def layernorm_bwd(dy, x, gamma, eps=1e-5):
    xf = x.float().clone().requires_grad_(True)
    g = gamma.clone().requires_grad_(True)
    b = torch.zeros_like(gamma).requires_grad_(True)
    y = F.layer_norm(xf, (xf.shape[-1],), g, b, eps)
    dx, dg, db = torch.autograd.grad(y, (xf, g, b), dy.float())
    return dx, dg, db


def gelu(x, tanh_form=False):
    """nn.GELU (exact erf) or GPT-2's gelu_new (the tanh form)."""
    return F.gelu(x.float(), approximate="tanh" if tanh_form else "none")


def gelu_bwd(dy, x, tanh_form=False):
    xf = x.float().clone().requires_grad_(True)
    (dx,) = torch.autograd.grad(gelu(xf, tanh_form), xf, dy.float())
    return dx


def gelu_new_closed_form(x):
    """transformers' NewGELUActivation written out: pins that the tanh form above is the one GPT-2 uses."""
    xf = x.double()
    return (0.5 * xf * (1.0 + torch.tanh((2.0 / torch.pi) ** 0.5 * (xf + 0.044715 * xf ** 3)))).float()


def attn_logits(scores, scale, bias=None, mask=None, causal=False):
    """scale * scores [B_, heads, Lq, Lk] + bias [heads, Lq, Lk] + mask [nW, Lq, Lk] (window = b % nW), causal fill."""
    z = scores.float() * scale
    Bn, Hn, Lq, Lk = z.shape
    if bias is not None:
        z = z + bias.unsqueeze(0)
    if mask is not None:
        nW = mask.shape[0]
        z = (z.view(Bn // nW, nW, Hn, Lq, Lk) + mask.unsqueeze(1).unsqueeze(0)).view(Bn, Hn, Lq, Lk)
    if causal:
        keep = torch.tril(torch.ones(Lq, Lk, dtype=torch.bool))
        z = z.masked_fill(~keep, float("-inf"))
    return z


def attn_softmax(scores, scale, bias=None, mask=None, causal=False):
    return torch.softmax(attn_logits(scores, scale, bias, mask, causal), dim=-1)


def attn_softmax_bwd(scores, dprobs, scale, bias=None, mask=None, causal=False):
    s = scores.float().clone().requires_grad_(True)
    p = attn_softmax(s, scale, bias, mask, causal)
    (ds,) = torch.autograd.grad(p, s, dprobs.float())
    return ds


def attention(q, k, v, scale, causal=False):
    """q, k, v [B, heads, T, d] -> (context [B, heads, T, d], log-sum-exp of the scaled scores [B, heads, T]):
    the scores / mask / softmax / context chain of transformers' GPT2Attention as train/gpt2.py:26 runs it."""
    z = attn_logits(q.float() @ k.float().transpose(-1, -2), scale, causal=causal)
    return torch.softmax(z, dim=-1) @ v.float(), torch.logsumexp(z, dim=-1)


def attention_bwd(q, k, v, dout, scale, causal=False):
    qs, ks, vs = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    o, _ = attention(qs, ks, vs, scale, causal)
    return torch.autograd.grad(o, (qs, ks, vs), dout.float())


def adamw(param, grads, lr, beta1, beta2, eps, weight_decay):
    """torch.optim.AdamW over one flat parameter, one step per entry of `grads`."""
    p = param.clone().requires_grad_(True)
    opt = torch.optim.AdamW([p], lr=lr, betas=(beta1, beta2), eps=eps, weight_decay=weight_decay)
    for g in grads:
        p.grad = g.clone()
        opt.step()
    st = opt.state[p]
    return p.detach(), st["exp_avg"], st["exp_avg_sq"]


def adamw_scalar(p, g, lr, beta1, beta2, eps, wd, steps):
    """The AdamW recurrence on one scalar in Python floats (fp64): pins the formula itself."""
    m = v = 0.0
    for t in range(1, steps + 1):
        p *= 1.0 - lr * wd
        m = beta1 * m + (1 - beta1) * g
        v = beta2 * v + (1 - beta2) * g * g
        p -= lr / (1 - beta1 ** t) * m / ((v ** 0.5) / ((1 - beta2 ** t) ** 0.5) + eps)
    return p


def embedding(ids, wte, wpe):
    T = ids.shape[1]
    return F.embedding(ids, wte.float()) + wpe.float()[:T].unsqueeze(0)


def embedding_bwd(ids, dy, vocab, n_pos):
    wte = torch.zeros(vocab, dy.shape[-1], requires_grad=True)
    wpe = torch.zeros(n_pos, dy.shape[-1], requires_grad=True)
    out = embedding(ids, wte, wpe)
    dwte, dwpe = torch.autograd.grad(out, (wte, wpe), dy.float())
    return dwte, dwpe
