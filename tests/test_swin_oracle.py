"""Pins for the Swin oracle (oracle/swin.py), on the CPU.

* tests/golden/swin_block.npz: vectors written by the reference's own readable Swin block
  (train/swin_b_tiny.py, through tests/golden/make_swin_fixtures.py): the oracle's block must reproduce them,
  unshifted and shifted (the toy shifts without a mask, so the mask is switched off for that comparison);
* the attention mask of shifted windows, patch merging (odd sides too) and the window round trip by brute force;
* a block on a feature map the window does not tile (zero padding to whole windows, crop) by loops over the frame;
* the parameter table against the published size of Swin-B (87,768,224 parameters).
"""
import math
import os

import numpy as np
import torch

from oracle import swin as S

FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "swin_block.npz"))


def _block_params(tag):
    pre = f"{tag}.param."
    return {"b." + k[len(pre):]: torch.from_numpy(FIX[k]) for k in FIX.files if k.startswith(pre)}


def test_block_matches_the_reference_toy_vectors():
    dim, heads, ws, H, W, B, shift = (int(v) for v in FIX["meta"])
    for tag, s in (("plain", 0), ("shifted", shift)):
        sd = _block_params(tag)
        x = torch.from_numpy(FIX[f"{tag}.x"])
        y = S.block(sd, "b.", x.view(B, H, W, dim), heads, ws, s, use_mask=False).reshape(B, H * W, dim)
        assert torch.allclose(y, torch.from_numpy(FIX[f"{tag}.y"]), atol=1e-10), tag
        assert np.array_equal(S.relative_position_index(ws).numpy(), FIX[f"{tag}.index"])
    # the shift changes the result, and so does the mask: neither can be dropped unnoticed
    sd = _block_params("shifted")
    x = torch.from_numpy(FIX["shifted.x"]).view(B, H, W, dim)
    y_shift = S.block(sd, "b.", x, heads, ws, shift, use_mask=False)
    assert (y_shift - S.block(sd, "b.", x, heads, ws, 0)).abs().max() > 1e-3
    assert (y_shift - S.block(sd, "b.", x, heads, ws, shift, use_mask=True)).abs().max() > 1e-3


def test_shift_mask_brute_force():
    H, W, ws, shift = 12, 8, 4, 2
    m = S.shift_mask(H, W, ws, shift)
    nW = (H // ws) * (W // ws)
    assert m.shape == (nW, ws * ws, ws * ws)
    for w in range(nW):
        wh, ww = divmod(w, W // ws)
        for a in range(ws * ws):
            for b in range(ws * ws):
                # position in the rolled image, then whether it wrapped round the border when it was rolled
                pa = (wh * ws + a // ws, ww * ws + a % ws)
                pb = (wh * ws + b // ws, ww * ws + b % ws)
                wrap = lambda p: (p[0] + shift >= H, p[1] + shift >= W)
                same = wrap(pa) == wrap(pb)
                assert m[w, a, b].item() == (0.0 if same else -100.0), (w, a, b)


def test_window_round_trip_and_patch_merging():
    g = torch.Generator()
    g.manual_seed(0)
    x = torch.randn(2, 8, 12, 5, generator=g)
    win = S.window_partition(x, 4)
    assert win.shape == (2 * 2 * 3, 16, 5)
    assert torch.equal(S.window_reverse(win, 4, 2, 8, 12), x)
    # window 1 of image 0 is rows 0..3, columns 4..7
    assert torch.equal(win[1].view(4, 4, 5), x[0, 0:4, 4:8])
    C = 5
    sd = {"m.norm.weight": torch.ones(4 * C), "m.norm.bias": torch.zeros(4 * C), "m.reduction.weight": torch.eye(4 * C)}
    y = S.patch_merging(sd, "m.", x)
    assert y.shape == (2, 4, 6, 4 * C)
    for b in range(2):
        for h in range(4):
            for w in range(6):
                cat = torch.cat([x[b, 2 * h, 2 * w], x[b, 2 * h + 1, 2 * w], x[b, 2 * h, 2 * w + 1], x[b, 2 * h + 1, 2 * w + 1]])
                ref = (cat - cat.mean()) / torch.sqrt(cat.var(unbiased=False) + 1e-5)
                assert torch.allclose(y[b, h, w], ref, atol=1e-5)


def test_padded_block_by_brute_force():
    """A feature map the window does not tile (10 x 6 under a 4 x 4 window -> a 12 x 8 frame), shifted and not: the
    attention half of oracle.swin.block against loops over the padded frame -- every frame position is a token (zeros
    behind norm1 where the image ends, so q, k, v there are the bias), a token attends to the tokens of its window
    in the frame rolled by the shift, pairs from different sides of the border are masked, and only the image's own
    positions get the result added."""
    for H, W, shifts in ((10, 6, (0, 2)), (3, 3, (2,))):        # the second: smaller than the window, one padded window
        _padded_block_case(H, W, shifts)


def _padded_block_case(H, W, shifts):
    g = torch.Generator()
    g.manual_seed(5)
    B, C, heads, ws = 2, 8, 2, 4
    Hp, Wp, D, N = -(-H // ws) * ws, -(-W // ws) * ws, C // heads, ws * ws
    sd = {"b.norm1.weight": torch.rand(C, generator=g) + 0.5, "b.norm1.bias": torch.randn(C, generator=g) * 0.1,
          "b.attn.qkv.weight": torch.randn(3 * C, C, generator=g) * 0.3, "b.attn.qkv.bias": torch.randn(3 * C, generator=g) * 0.3,
          "b.attn.proj.weight": torch.randn(C, C, generator=g) * 0.3, "b.attn.proj.bias": torch.randn(C, generator=g) * 0.1,
          "b.attn.relative_position_bias_table": torch.randn((2 * ws - 1) ** 2, heads, generator=g),
          "b.norm2.weight": torch.ones(C), "b.norm2.bias": torch.zeros(C),
          "b.mlp.0.weight": torch.zeros(4 * C, C), "b.mlp.0.bias": torch.zeros(4 * C),      # MLP switched off:
          "b.mlp.3.weight": torch.zeros(C, 4 * C), "b.mlp.3.bias": torch.zeros(C)}          # block = x + attention
    x = torch.randn(B, H, W, C, generator=g)
    for asked in shifts:
        got = S.block(sd, "b.", x, heads, ws, asked)
        shift = 0 if (ws >= Hp and ws >= Wp) else asked        # one window covers the frame: nothing to shift
        want = x.clone()
        for b in range(B):
            frame = torch.zeros(Hp, Wp, C)
            for h in range(H):
                for w in range(W):
                    v = x[b, h, w]
                    frame[h, w] = (v - v.mean()) / torch.sqrt(v.var(unbiased=False) + 1e-5) * sd["b.norm1.weight"] + sd["b.norm1.bias"]
            qkv = frame @ sd["b.attn.qkv.weight"].T + sd["b.attn.qkv.bias"]               # [Hp, Wp, 3C]
            out = torch.zeros(Hp, Wp, C)
            for h in range(Hp):
                for w in range(Wp):
                    # position in the rolled frame, its window there, and the frame positions of that window's tokens
                    rh, rw = (h - shift) % Hp, (w - shift) % Wp
                    keys = [(((rh // ws) * ws + i + shift) % Hp, ((rw // ws) * ws + j + shift) % Wp, i, j)
                            for i in range(ws) for j in range(ws)]
                    qi, qj = rh % ws, rw % ws
                    side = lambda r, c: (r + shift >= Hp if shift else False, c + shift >= Wp if shift else False)
                    for hd in range(heads):
                        q = qkv[h, w, hd * D:(hd + 1) * D] * D ** -0.5
                        logits = []
                        for kh, kw, i, j in keys:
                            k = qkv[kh, kw, C + hd * D:C + (hd + 1) * D]
                            rel = (qi - i + ws - 1) * (2 * ws - 1) + (qj - j + ws - 1)
                            rolled_q = (rh, rw)
                            rolled_k = ((kh - shift) % Hp, (kw - shift) % Wp)
                            masked = side(*rolled_q) != side(*rolled_k)
                            logits.append(q @ k + sd["b.attn.relative_position_bias_table"][rel, hd] + (-100.0 if masked else 0.0))
                        pr = torch.softmax(torch.stack(logits), 0)
                        out[h, w, hd * D:(hd + 1) * D] = sum(p_ * qkv[kh, kw, 2 * C + hd * D:2 * C + (hd + 1) * D]
                                                             for p_, (kh, kw, _, _) in zip(pr, keys))
            proj = out @ sd["b.attn.proj.weight"].T + sd["b.attn.proj.bias"]
            want[b] += proj[:H, :W]
        assert torch.allclose(got, want, atol=2e-5), (shift, (got - want).abs().max())


def test_patch_merging_pads_odd_sides_with_zeros():
    g = torch.Generator()
    g.manual_seed(1)
    C = 3
    x = torch.randn(1, 5, 3, C, generator=g)
    sd = {"m.norm.weight": torch.ones(4 * C), "m.norm.bias": torch.zeros(4 * C), "m.reduction.weight": torch.eye(4 * C)}
    y = S.patch_merging(sd, "m.", x)
    assert y.shape == (1, 3, 2, 4 * C)
    at = lambda h, w: x[0, h, w] if h < 5 and w < 3 else torch.zeros(C)
    for h in range(3):
        for w in range(2):
            cat = torch.cat([at(2 * h, 2 * w), at(2 * h + 1, 2 * w), at(2 * h, 2 * w + 1), at(2 * h + 1, 2 * w + 1)])
            ref = (cat - cat.mean()) / torch.sqrt(cat.var(unbiased=False) + 1e-5)
            assert torch.allclose(y[0, h, w], ref, atol=1e-5)


def test_swin_b_parameter_table():
    shapes = S.param_shapes(S.config())
    assert sum(math.prod(s) for s in shapes.values()) == 87_768_224
    assert shapes["features.5.17.attn.relative_position_bias_table"] == (169, 16)
    assert shapes["features.6.reduction.weight"] == (1024, 2048) and shapes["head.weight"] == (1000, 1024)


def test_forward_shapes_tiny():
    cfg = S.config(embed=16, depths=(2, 2), heads=(2, 4), window=4, patch=2, image=32, classes=10)
    sd = S.make_state_dict(cfg)
    x = torch.randn(3, 3, 32, 32)
    assert S.forward(sd, x, cfg).shape == (3, 10)
    loss, grads = S.loss_and_grads(sd, x, torch.tensor([1, 2, 3]), cfg)
    assert set(grads) == set(sd) and all(torch.isfinite(g).all() and g.abs().sum() > 0 for g in grads.values())
