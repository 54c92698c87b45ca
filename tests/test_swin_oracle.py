"""Pins for the Swin oracle (oracle/swin.py), on the CPU.

* tests/golden/swin_block.npz: vectors written by the reference's own readable Swin block
  (train/swin_b_tiny.py, through tests/golden/make_swin_fixtures.py): the oracle's block must reproduce them,
  unshifted and shifted (the toy shifts without a mask, so the mask is switched off for that comparison);
* the attention mask of shifted windows, patch merging and the window round trip by brute force;
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
