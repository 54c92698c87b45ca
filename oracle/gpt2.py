"""GPT-2 training-step oracle on CPU fp32 (test infrastructure only; see oracle/__init__.py).

A plain torch.nn statement of the model the reference trains through
``GPT2LMHeadModel`` (train/gpt2.py:26, loss = output.loss at :93): learned token and position
embeddings, pre-LayerNorm blocks with causal multi-head attention and a gelu_new MLP, a final
LayerNorm, the token embedding reused as output projection, and the mean cross entropy of
position t's logits against token t+1.  Parameter names and the [in, out] orientation of the
projection weights follow the transformers state dict, so that a state dict moves between the
three of them (transformers, this oracle, the HIP engine) unchanged.  Dropout is off.

tests/test_gpt2_oracle.py pins this definition against transformers' own GPT2LMHeadModel
(random weights, no download) on logits, loss and every gradient.
"""
import math

import torch
import torch.nn.functional as F


def make_state_dict(vocab, n_pos, n_embd, n_layer, seed=0):
    """GPT-2's initialisation: N(0, 0.02) weights (residual projections scaled by 1/sqrt(2 n_layer)),
    zero biases, LayerNorm gamma 1 / beta 0."""
    g = torch.Generator()
    g.manual_seed(seed)
    C = n_embd
    n = lambda *s, std=0.02: torch.randn(*s, generator=g) * std
    sd = {"transformer.wte.weight": n(vocab, C), "transformer.wpe.weight": n(n_pos, C)}
    for i in range(n_layer):
        p = f"transformer.h.{i}."
        sd[p + "ln_1.weight"], sd[p + "ln_1.bias"] = torch.ones(C), torch.zeros(C)
        sd[p + "attn.c_attn.weight"], sd[p + "attn.c_attn.bias"] = n(C, 3 * C), torch.zeros(3 * C)
        sd[p + "attn.c_proj.weight"] = n(C, C, std=0.02 / math.sqrt(2 * n_layer))
        sd[p + "attn.c_proj.bias"] = torch.zeros(C)
        sd[p + "ln_2.weight"], sd[p + "ln_2.bias"] = torch.ones(C), torch.zeros(C)
        sd[p + "mlp.c_fc.weight"], sd[p + "mlp.c_fc.bias"] = n(C, 4 * C), torch.zeros(4 * C)
        sd[p + "mlp.c_proj.weight"] = n(4 * C, C, std=0.02 / math.sqrt(2 * n_layer))
        sd[p + "mlp.c_proj.bias"] = torch.zeros(C)
    sd["transformer.ln_f.weight"], sd["transformer.ln_f.bias"] = torch.ones(C), torch.zeros(C)
    return sd


def forward(sd, ids, n_head, n_layer):
    """Logits [B, T, vocab] from a state dict of (possibly requires_grad) fp32 tensors."""
    B, T = ids.shape
    wte = sd["transformer.wte.weight"]
    C = wte.shape[1]
    D = C // n_head
    h = F.embedding(ids, wte) + sd["transformer.wpe.weight"][:T].unsqueeze(0)
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for i in range(n_layer):
        p = f"transformer.h.{i}."
        a = F.layer_norm(h, (C,), sd[p + "ln_1.weight"], sd[p + "ln_1.bias"], 1e-5)
        qkv = a @ sd[p + "attn.c_attn.weight"] + sd[p + "attn.c_attn.bias"]
        q, k, v = (t.view(B, T, n_head, D).transpose(1, 2) for t in qkv.split(C, dim=2))
        att = (q @ k.transpose(-1, -2)) / math.sqrt(D)
        att = torch.softmax(att.masked_fill(~causal, float("-inf")), dim=-1)
        o = (att @ v).transpose(1, 2).reshape(B, T, C)
        h = h + o @ sd[p + "attn.c_proj.weight"] + sd[p + "attn.c_proj.bias"]
        m = F.layer_norm(h, (C,), sd[p + "ln_2.weight"], sd[p + "ln_2.bias"], 1e-5)
        f = F.gelu(m @ sd[p + "mlp.c_fc.weight"] + sd[p + "mlp.c_fc.bias"], approximate="tanh")
        h = h + f @ sd[p + "mlp.c_proj.weight"] + sd[p + "mlp.c_proj.bias"]
    h = F.layer_norm(h, (C,), sd["transformer.ln_f.weight"], sd["transformer.ln_f.bias"], 1e-5)
    return h @ wte.t()


def loss_of(logits, ids):
    """transformers' causal LM loss: logits of position t against token t+1, mean over B * (T-1)."""
    V = logits.shape[-1]
    return F.cross_entropy(logits[:, :-1].reshape(-1, V), ids[:, 1:].reshape(-1))


def loss_and_grads(sd, ids, n_head, n_layer, loss_scale=1.0):
    leaf = {k: v.detach().clone().float().requires_grad_(True) for k, v in sd.items()}
    loss = loss_of(forward(leaf, ids, n_head, n_layer), ids)
    (loss * loss_scale).backward()
    return loss.detach(), {k: v.grad for k, v in leaf.items()}


def train_steps(sd, batches, n_head, n_layer, optimizer="adamw", lr=1e-3, weight_decay=0.01, momentum=0.9):
    """`len(batches)` optimizer steps; returns (losses, final state dict).  AdamW with PyTorch's defaults
    (betas 0.9 / 0.999, eps 1e-8), or SGD-momentum as the reference's script configures it
    (train/gpt2.py:31-32)."""
    leaf = {k: v.detach().clone().float().requires_grad_(True) for k, v in sd.items()}
    params = list(leaf.values())
    opt = (torch.optim.AdamW(params, lr=lr, weight_decay=weight_decay) if optimizer == "adamw"
           else torch.optim.SGD(params, lr=lr, momentum=momentum, weight_decay=weight_decay))
    losses = []
    for ids in batches:
        opt.zero_grad(set_to_none=False)
        loss = loss_of(forward(leaf, ids, n_head, n_layer), ids)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    return losses, {k: v.detach() for k, v in leaf.items()}
