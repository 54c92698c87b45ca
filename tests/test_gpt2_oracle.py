"""Pins the GPT-2 oracle (oracle/gpt2.py) against transformers' GPT2LMHeadModel on the CPU:
same random weights (no download), same token ids -> same logits, loss and gradients.  A wrong weight
orientation, a wrong GELU form, a missing label shift or a wrong attention scale fails this test."""
import pytest
import torch

from oracle import gpt2 as G

transformers = pytest.importorskip("transformers")


def test_oracle_matches_transformers_gpt2():
    cfg = transformers.GPT2Config(vocab_size=97, n_positions=24, n_embd=32, n_layer=2, n_head=4,
                                  resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
    torch.manual_seed(0)
    model = transformers.GPT2LMHeadModel(cfg).train()
    # give biases and LayerNorm parameters non-trivial values so that they take part
    g = torch.Generator()
    g.manual_seed(1)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() == 1:
                p.add_(torch.randn(p.shape, generator=g) * 0.1)
    sd = {k: v.detach().clone() for k, v in model.state_dict().items()
          if not k.endswith(".attn.bias") and not k.endswith("masked_bias") and k != "lm_head.weight"}
    assert set(sd) == set(G.make_state_dict(97, 24, 32, 2)), "state-dict names must be those of transformers"
    ids = torch.randint(0, 97, (3, 24), generator=g)
    out = model(input_ids=ids, labels=ids)
    out.loss.backward()
    logits = G.forward(sd, ids, 4, 2)
    assert torch.allclose(logits, out.logits, atol=2e-5), (logits - out.logits).abs().max()
    loss, grads = G.loss_and_grads(sd, ids, 4, 2)
    assert abs(loss.item() - out.loss.item()) < 1e-5
    named = dict(model.named_parameters())
    for k, gk in grads.items():
        ref = named[k].grad
        assert torch.allclose(gk, ref, atol=1e-5 + 1e-4 * ref.abs().max().item()), k


def test_oracle_init_statistics():
    sd = G.make_state_dict(1000, 64, 128, 4, seed=3)
    assert abs(sd["transformer.wte.weight"].std().item() - 0.02) < 1e-3
    assert abs(sd["transformer.h.0.mlp.c_proj.weight"].std().item() - 0.02 / (8 ** 0.5)) < 5e-4
    assert torch.all(sd["transformer.h.1.ln_1.weight"] == 1) and torch.all(sd["transformer.h.1.attn.c_attn.bias"] == 0)
