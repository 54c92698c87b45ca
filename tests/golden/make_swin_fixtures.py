"""Writes tests/golden/swin_block.npz: inputs, parameters and outputs of the reference's own readable Swin
block (train/swin_b_tiny.py: WindowAttention :22-76 and SwinTransformerBlock :78-137), evaluated here on the
CPU in float64 with seeded values.  Only this script reads the reference; the fixture it writes is data.

    python tests/golden/make_swin_fixtures.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("swin_b_tiny", os.path.join(ref_root, "train", "swin_b_tiny.py"))
    toy = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(toy)
    torch.manual_seed(0)
    out = {}
    dim, heads, ws, H, W, B = 32, 4, 4, 8, 8, 2
    for tag, shift in (("plain", 0), ("shifted", 2)):
        blk = toy.SwinTransformerBlock(dim, (H, W), heads, window_size=ws, shift_size=shift, num_mlp=4 * dim).double()
        with torch.no_grad():
            for p in blk.parameters():       # zeros (the table) and ones would hide a wrong gather
                p.copy_(torch.randn(p.shape, dtype=torch.float64) * (0.2 if p.dim() > 1 else 0.1))
        x = torch.randn(B, H * W, dim, dtype=torch.float64)
        with torch.no_grad():
            y = blk(x)
            a = blk.attn(toy.window_partition(blk.norm1(x).view(B, H, W, dim), ws).view(-1, ws * ws, dim))
        out[f"{tag}.x"], out[f"{tag}.y"], out[f"{tag}.attn_of_norm1_windows"] = x.numpy(), y.numpy(), a.numpy()
        for k, v in blk.state_dict().items():
            out[f"{tag}.param.{k}"] = v.numpy()
        out[f"{tag}.index"] = blk.attn.relative_position_index.numpy()
    out["meta"] = np.array([dim, heads, ws, H, W, B, 2])
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "swin_block.npz"), **out)
    print("wrote swin_block.npz with", len(out), "arrays")


if __name__ == "__main__":
    main()
