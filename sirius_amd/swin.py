"""Swin Transformer training-step engine over the HIP operators.

What the reference does with ``torchvision.models.swin_b`` + autograd + an optimizer (train/swin_b.py:38-45,
83-95), this engine does with one recorded program of hand-written kernels per batch size.  The block
mathematics is the one the reference spells out in train/swin_b_tiny.py (window partition :8-19, relative
position bias :35-59, attention :49-76, pre-norm block with cyclic shift :104-137), plus what the full model
adds: the attention mask of shifted windows, patch merging, patch embedding.

* tokens are rows: activations are [B*H*W, C]; a block gathers its LayerNorm output into window order (cyclic
  shift and partition in one pass), runs every projection as a 1x1 convolution on the MFMA kernels, the
  attention products as batched strided GEMMs on the packed [B_, N, 3, heads, D] projection, and scatters
  the result back with the residual add fused; where one window covers the image (the last stage at 224) the
  gathers vanish; a feature map the window does not tile is padded with zero tokens at the bottom and the right to
  whole windows (torchvision's rule; window-ordered tensors then have the padded frame's rows), an odd side is
  padded by the merge;
* the relative-position bias is gathered from its table into a dense [heads, N, N] fp32 tensor per block
  (read by the softmax kernel); its gradient is the column sum of the logit gradients over the windows,
  scattered back through the index;
* parameters / gradients / AdamW state are flat fp32 buffers with torchvision's state-dict names; bf16 mode
  keeps a flat bf16 shadow; backward is written out by hand.

torch supplies device memory and streams only.  Stochastic depth and dropout are off.
"""
import contextlib
import math
import os

import torch

from . import ops
from .engine_base import EngineBase

PATCH_CIN_PAD = 8


class _Param:
    __slots__ = ("name", "kind", "shape", "store_shape", "offset", "numel")

    def __init__(self, name, kind, shape, store_shape, offset):
        self.name, self.kind, self.shape, self.store_shape, self.offset = name, kind, shape, store_shape, offset
        self.numel = int(math.prod(store_shape))


class _Plan:
    pass


def relative_position_index(ws):
    """[ws*ws, ws*ws] int: which row of the bias table a (query, key) pair of a window reads
    (train/swin_b_tiny.py:35-46)."""
    coords = torch.stack(torch.meshgrid([torch.arange(ws), torch.arange(ws)], indexing="ij")).flatten(1)
    rel = (coords[:, :, None] - coords[:, None, :]).permute(1, 2, 0).contiguous()
    rel[:, :, 0] += ws - 1
    rel[:, :, 1] += ws - 1
    rel[:, :, 0] *= 2 * ws - 1
    return rel.sum(-1)


def shifted_window_mask(H, W, ws, shift):
    """[nW, ws*ws, ws*ws] fp32, 0 or -100: token pairs of a shifted window that come from different sides of
    the image border must not attend to each other."""
    region = torch.zeros(H, W)
    n = 0
    for hs in (slice(0, -ws), slice(-ws, -shift), slice(-shift, None)):
        for wsl in (slice(0, -ws), slice(-ws, -shift), slice(-shift, None)):
            region[hs, wsl] = n
            n += 1
    win = region.view(H // ws, ws, W // ws, ws).permute(0, 2, 1, 3).reshape(-1, ws * ws)
    diff = win.unsqueeze(1) - win.unsqueeze(2)
    return torch.where(diff != 0, torch.tensor(-100.0), torch.tensor(0.0)).contiguous()


class SwinEngine(EngineBase):
    def __init__(self, embed=128, depths=(2, 2, 18, 2), heads=(4, 8, 16, 32), window=7, patch=4, image_size=224,
                 num_classes=1000, dtype=torch.bfloat16, lr=1e-3, weight_decay=0.05, betas=(0.9, 0.999), eps=1e-8,
                 stream=None, allocator=None, overlap_wgrad=True, fused_attention=True, fuse_window_ln=True,
                 batch_bias_gather=True, trailing_reduce=None):
        self._init_engine(dtype, stream, allocator)
        # trailing_reduce: the split reduction of a weight gradient rides the next weight-gradient launch as extra
        # workgroups instead of being a launch of its own (same bits)
        self.trailing_reduce = (os.environ.get("TCH_TRAILING_REDUCE", "1") != "0") if trailing_reduce is None \
            else bool(trailing_reduce)
        # weight / bias / bias-table gradients on a second lane beside the data-gradient chain; the lanes meet
        # at the end of every block, before its gradient buffers are handed round again
        self.overlap_wgrad = overlap_wgrad
        # fuse_window_ln: the LayerNorms next to a window partition read / write window order themselves
        self.fuse_window_ln = fuse_window_ln
        # batch_bias_gather: the dense bias of every block is gathered from its table at the start of the forward
        # pass, eight tables per launch, instead of one launch per block in front of its attention
        self.batch_bias_gather = batch_bias_gather
        self.fused_attention = fused_attention
        assert len(depths) == len(heads) and image_size % patch == 0 and num_classes % 8 == 0 and embed % 8 == 0
        self.embed, self.depths, self.heads = embed, tuple(depths), tuple(heads)
        self.window, self.patch, self.image_size, self.num_classes = window, patch, image_size, num_classes
        self.lr, self.weight_decay, self.betas, self.eps = lr, weight_decay, betas, eps

        # ---- stages: (feature index, depth, heads, C, resolution, effective window) ----
        self.stages = []
        C, R = embed, image_size // patch
        for s, (depth, nh) in enumerate(zip(self.depths, self.heads)):
            assert C % nh == 0 and (C // nh) % 8 == 0, "head dimension must be a multiple of one 16-byte chunk"
            # A feature map the window does not tile (or one smaller than the window) is padded at the bottom and the
            # right to whole windows (Rp), the way torchvision's shifted_window_attention pads its input; the window,
            # and with it the bias table, stays what it is.  Not needed at the reference's 224 x 224
            # (train/swin_b.py:59), where the stages are 56, 28, 14 and 7 wide under a 7 x 7 window.
            ws = window
            Rp = -(-R // ws) * ws
            assert Rp == R or fuse_window_ln, "padded windows are built into the LayerNorms next to the partitions only"
            self.stages.append(dict(f=1 + 2 * s, depth=depth, heads=nh, C=C, R=R, ws=ws, Rp=Rp))
            if s + 1 < len(self.depths):
                C, R = 2 * C, (R + 1) // 2      # an odd side is padded with a zero row / column by the merge
        self.feat = C

        # ---- parameter table (torchvision naming) ----
        self._specs, self._off = [], 0
        self._add("features.0.0.weight", "conv", (embed, 3, patch, patch), (embed, patch, patch, PATCH_CIN_PAD))
        self._add_vec("features.0.0.bias", embed)
        self._add_vec("features.0.2.weight", embed)
        self._add_vec("features.0.2.bias", embed)
        for st in self.stages:
            C = st["C"]
            for i in range(st["depth"]):
                p = f"features.{st['f']}.{i}."
                self._add_vec(p + "norm1.weight", C)
                self._add_vec(p + "norm1.bias", C)
                self._add_linear(p + "attn.qkv", C, 3 * C)
                self._add_linear(p + "attn.proj", C, C)
                self._add(p + "attn.relative_position_bias_table", "plain", ((2 * window - 1) ** 2, st["heads"]),
                          ((2 * window - 1) ** 2, st["heads"]))
                self._add_vec(p + "norm2.weight", C)
                self._add_vec(p + "norm2.bias", C)
                self._add_linear(p + "mlp.0", C, 4 * C)
                self._add_linear(p + "mlp.3", 4 * C, C)
            if st is not self.stages[-1]:
                p = f"features.{st['f'] + 1}."
                self._add_vec(p + "norm.weight", 4 * C)
                self._add_vec(p + "norm.bias", 4 * C)
                self._add(p + "reduction.weight", "linear", (2 * C, 4 * C), (2 * C, 1, 1, 4 * C))
        self._add_vec("norm.weight", self.feat)
        self._add_vec("norm.bias", self.feat)
        self._add_linear("head", self.feat, num_classes)
        self.n_store = self._off
        self.spec = {p.name: p for p in self._specs}

        def zeros(n, dt=torch.float32):
            return self._alloc((n,), dt).zero_()
        self.params, self.grads = zeros(self.n_store), zeros(self.n_store)
        self.exp_avg, self.exp_avg_sq = zeros(self.n_store), zeros(self.n_store)
        self.step_dev = self._alloc((1,), torch.int32).zero_()
        self.adam_scalars = zeros(2)
        self.shadow = zeros(self.n_store, torch.bfloat16) if dtype == torch.bfloat16 else None
        self.wt = zeros(self.n_store, dtype)
        self._tt = ops.FilterTransposeTable(
            [(p.offset, p.store_shape[0], 1, p.store_shape[3]) for p in self._specs if p.kind == "linear"], self.dev)

    # ------------------------------------------------------------------ parameter table
    def _add(self, name, kind, shape, store_shape):
        p = _Param(name, kind, shape, store_shape, self._off)
        self._specs.append(p)
        self._off += (p.numel + 7) // 8 * 8
        return p

    def _add_vec(self, name, n):
        self._add(name, "vec", (n,), (n,))

    def _add_linear(self, name, cin, cout):
        self._add(name + ".weight", "linear", (cout, cin), (cout, 1, 1, cin))
        self._add_vec(name + ".bias", cout)

    def num_parameters(self):
        return sum(int(math.prod(p.shape)) for p in self._specs)

    def _view(self, flat, name):
        p = self.spec[name]
        return flat[p.offset:p.offset + p.numel].view(p.store_shape)

    def _w(self, name):
        return self._view(self.shadow if self.shadow is not None else self.params, name)

    def _wt(self, name):
        p = self.spec[name]
        K, _, _, C = p.store_shape
        return self.wt[p.offset:p.offset + p.numel].view(C, 1, 1, K)

    def _to_store(self, p, t):
        t = t.detach().to(torch.float32)
        if p.kind == "conv":
            t = torch.nn.functional.pad(t.permute(0, 2, 3, 1), (0, p.store_shape[3] - t.shape[1]))
        return t.reshape(p.store_shape).contiguous()

    def _from_store(self, p, flat):
        t = flat[p.offset:p.offset + p.numel].view(p.store_shape)
        if p.kind == "conv":
            t = t[..., :p.shape[1]].permute(0, 3, 1, 2)
        return t.reshape(p.shape).contiguous().cpu()

    def load_state_dict(self, sd):
        host = torch.zeros(self.n_store, dtype=torch.float32)
        for p in self._specs:
            host[p.offset:p.offset + p.numel] = self._to_store(p, sd[p.name]).reshape(-1)
        self.params.copy_(host)
        self._reset()

    def init_normal(self, seed=0):
        """N(0, 0.02) weights and bias tables, zero biases, LayerNorm gamma 1 / beta 0, generated on the GPU."""
        g = torch.Generator(device=self.dev)
        g.manual_seed(seed)
        for p in self._specs:
            v = self._view(self.params, p.name)
            if p.kind == "vec":
                is_gamma = p.name.endswith(("norm1.weight", "norm2.weight", "norm.weight", "features.0.2.weight"))
                v.fill_(1.0 if is_gamma else 0.0)
            else:
                v.normal_(0.0, 0.02, generator=g)
                if p.kind == "conv":
                    v[..., p.shape[1]:] = 0
        self._reset()

    def _reset(self):
        self.grads.zero_()
        self.exp_avg.zero_()
        self.exp_avg_sq.zero_()
        self.step_dev.zero_()
        self.refresh_shadow()
        torch.cuda.synchronize()

    def refresh_shadow(self):
        self.ctx.synchronize()      # nothing of an earlier step (either lane) still reads or writes the copies
        if self.shadow is not None:
            ops.cast_from_f32(self.ctx, self.params, self.shadow)
        self._refresh_transposed()

    def _refresh_transposed(self):
        ops.filter_transpose_batched(self.ctx, self.shadow if self.shadow is not None else self.params, self.wt,
                                     self._tt)

    def state_dict(self):
        torch.cuda.synchronize()
        return {p.name: self._from_store(p, self.params) for p in self._specs}

    def grads_dict(self, use_global=False):
        torch.cuda.synchronize()
        flat = self.global_grads if use_global else self.grads
        return {p.name: self._from_store(p, flat) for p in self._specs}

    # ------------------------------------------------------------------ the plan for one batch size
    def _build_plan(self, B, loss_scale):
        T_, ctx, dev = self.dtype, self.ctx, self.dev
        S, P = self.image_size, self.patch
        plan = _Plan()
        plan.batch, plan.loss_scale = B, loss_scale
        keep = []

        def act(*shape, dtype=T_):
            t = self._alloc(tuple(shape), dtype)
            keep.append(t)
            return t

        code = ops.dtype_code(torch.empty(0, dtype=T_))
        plan.x_in = act(B, 3, S, S, dtype=torch.float32)
        plan.labels = act(B, dtype=torch.int64).zero_()
        plan.loss_rows = act(B, dtype=torch.float32)
        plan.loss = act(1, dtype=torch.float32)

        st0 = self.stages[0]
        rows0 = B * st0["R"] ** 2
        max_rc = max(B * st["Rp"] ** 2 * st["C"] for st in self.stages)         # elements of the largest [rows, C]
        n_ln = 2 + sum(2 * st["depth"] for st in self.stages) + (len(self.stages) - 1)
        ln_mean, ln_rstd = act(n_ln * rows0, dtype=torch.float32), act(n_ln * rows0, dtype=torch.float32)
        ln_partial = act(max(ops.layernorm_bwd_partial_rows(B * st["R"] ** 2) * 4 * st["C"] * 2 for st in self.stages),
                         dtype=torch.float32)
        ln_slot = [0]

        def new_ln(rows):
            i = ln_slot[0]
            ln_slot[0] += 1
            return ln_mean[i * rows0:i * rows0 + rows], ln_rstd[i * rows0:i * rows0 + rows]

        # weight-gradient workspace: the largest need over every projection call of the plan
        calls = [(B, S, S, PATCH_CIN_PAD, self.embed, P, P, P), (B, 1, 1, self.feat, self.num_classes, 1, 1, 1)]
        for si, st in enumerate(self.stages):
            rows, C = B * st["Rp"] ** 2, st["C"]    # window-ordered operands have the padded frame's rows
            calls += [(rows, 1, 1, C, 3 * C, 1, 1, 1), (rows, 1, 1, C, C, 1, 1, 1), (rows, 1, 1, C, 4 * C, 1, 1, 1),
                      (rows, 1, 1, 4 * C, C, 1, 1, 1)]
            if si + 1 < len(self.stages):
                calls.append((B * ((st["R"] + 1) // 2) ** 2, 1, 1, 4 * C, 2 * C, 1, 1, 1))
        ws_bytes = 4
        for n_, h_, w_, cin, k_, r_, s_, stride in calls:
            sp = int(ops.lib().tch_conv2d_wgrad_pick_splits(code, n_, h_, w_, cin, k_, r_, s_, stride, 0))
            ws_bytes = max(ws_bytes, ops.conv2d_wgrad_workspace_bytes(code, k_, r_, s_, cin, sp))
        wg_half = (ws_bytes // 4 + 63) // 64 * 64
        wg_ws = act(2 * wg_half, dtype=torch.float32)     # two workspaces taken in turn (trailing reductions)
        trail = ops.TrailingWgrad(ctx, wg_ws, wg_half) if self.trailing_reduce else None

        def wgrad(x4, dy4, dw, stride=1, dbias=None, c_logical=0):
            if trail is not None:
                return trail.wgrad(x4, dy4, dw, stride, 0, dbias=dbias, c_logical=c_logical)
            ops.conv2d_wgrad(ctx, x4, dy4, dw, stride, 0, workspace=wg_ws, dbias=dbias, c_logical=c_logical)
        bias_ws = act(64 * 4 * self.feat, dtype=torch.float32)

        def ln_fwd(name, x, y, stats, window=None, **kw):
            ops.layernorm_fwd(ctx, x, y, self._view(self.params, name + ".weight"), self._view(self.params, name + ".bias"),
                              stats[0], stats[1], window=window, **kw)

        def ln_bwd(name, dy, x, dx, stats, residual=None, window=None, windowed=()):
            ops.layernorm_bwd(ctx, dy, x, dx, self._view(self.params, name + ".weight"), stats[0], stats[1],
                              self._view(self.grads, name + ".weight"), self._view(self.grads, name + ".bias"), ln_partial,
                              residual=residual, window=window, windowed=windowed)

        def as4(t):
            return t.view(t.shape[0], 1, 1, t.shape[1])

        def lin_fwd(name, x, y, add=None, bias=True):
            ops.conv2d_fwd(ctx, as4(x), self._w(name + ".weight"), as4(y), 1, 0,
                           bias=self._view(self.params, name + ".bias") if bias else None,
                           add=None if add is None else as4(add))

        def side():
            return ctx.side_lane(wait_main=True) if self.overlap_wgrad else contextlib.nullcontext()

        def lin_bwd(name, x, dy, dx, bias=True):
            with side():
                wgrad(as4(x), as4(dy), self._view(self.grads, name + ".weight"),
                      dbias=self._view(self.grads, name + ".bias") if bias else None)
            if dx is not None:
                ops.conv2d_dgrad(ctx, as4(dy), self._wt(name + ".weight"), as4(dx), 1, 0)

        # scratch the blocks share (program order is the only hazard: one lane)
        def flat(n):
            return act(n)
        s_n1 = flat(max_rc)                                    # LayerNorm output before it is gathered
        # gradients of [rows, C] tensors, handed round; six, so that inside a block nothing the second lane
        # still reads (the block's incoming gradient, the gathered projection gradient) is written again
        g_bufs = [flat(max_rc) for _ in range(6)]
        g_3c, g_4c_a, g_4c_b = flat(3 * max_rc), flat(4 * max_rc), flat(4 * max_rc)
        # One launch per direction for the attention of a block where the kernel's limits hold (bf16, heads 32
        # wide and even in number, at most 64 tokens per window): score rows are then padded to 64 keys.
        for st in self.stages:
            st["fused"] = (self.fused_attention and self.dtype == torch.bfloat16 and st["C"] // st["heads"] == 32 and
                           st["heads"] % 2 == 0 and st["ws"] ** 2 <= 64)
            st["keys_ld"] = 64 if st["fused"] else st["ws"] ** 2      # leading dimension of a score row
            st["bias_elems"] = st["heads"] * (64 * 64 if st["fused"] else st["ws"] ** 4)
        max_scores = max(B * (st["Rp"] // st["ws"]) ** 2 * st["heads"] * st["ws"] ** 2 * st["keys_ld"] for st in self.stages)
        d_scores = flat(max_scores)
        max_bias = max(st["bias_elems"] for st in self.stages)
        bias_buf = act(max_bias, dtype=torch.float32)
        dbias_buf = act(max_bias, dtype=torch.float32)
        colsum_ws = act(max(ops.column_sum_workspace_floats(B * (st["Rp"] // st["ws"]) ** 2,
                                                            st["heads"] * st["ws"] ** 2 * st["keys_ld"])
                            for st in self.stages), dtype=torch.float32)

        def v2(buf, r, c):
            return buf[:r * c].view(r, c)

        # constants per stage: index of the bias table, mask of the shifted windows
        for st in self.stages:
            ws = st["ws"]
            st["index"] = relative_position_index(ws)
            st["index_dev"] = st["index"].to(torch.int32).contiguous().to(dev)
            keep.append(st["index_dev"])
            shift = ws // 2 if ws < st["Rp"] else 0
            st["shift"] = shift
            mask = shifted_window_mask(st["Rp"], st["Rp"], ws, shift) if shift else None     # over the padded frame
            if st["fused"]:
                # (query, key) pairs in rows of 64 keys: -1 = padding (gathers -inf, which masks the padded keys)
                pairs = torch.full((64, 64), -1, dtype=torch.int32)
                pairs[:ws * ws, :ws * ws] = st["index"].to(torch.int32)
                st["pairs_dev"] = pairs.reshape(-1).to(dev)
                ptr, plist = ops.relpos_inverse_index(pairs[:ws * ws], (2 * self.window - 1) ** 2)
                st["inv_ptr_dev"], st["inv_list_dev"] = ptr.to(dev), plist.to(dev)
                keep += [st["inv_ptr_dev"], st["inv_list_dev"]]
                keep.append(st["pairs_dev"])
                if mask is not None:
                    padded = torch.zeros(mask.shape[0], 64, 64)
                    padded[:, :ws * ws, :ws * ws] = mask
                    mask = padded
            st["mask_dev"] = mask.contiguous().to(dev) if mask is not None else None
            if st["mask_dev"] is not None:
                keep.append(st["mask_dev"])

        prog = ops.Program()
        marks = []

        def mark(phase, name):
            marks.append((len(prog), phase, name))

        ctx.begin_record(prog)
        try:
            # ================= forward =================
            x0 = act(B, S, S, PATCH_CIN_PAD)
            ops.nchw_to_nhwc_pad(ctx, plan.x_in, x0)
            R0, C0 = st0["R"], st0["C"]
            e0 = act(rows0, C0)
            ops.conv2d_fwd(ctx, x0, self._w("features.0.0.weight"), e0.view(B, R0, R0, C0), P, 0,
                           bias=self._view(self.params, "features.0.0.bias"), c_logical=3)
            x = act(rows0, C0)
            embed_stats = new_ln(rows0)
            ln_fwd("features.0.2", e0, x, embed_stats)
            mark("fwd", "features.0")
            saved_blocks, saved_merges = [], []
            block_bias = {}
            if self.batch_bias_gather:
                fused = [(f"features.{st['f']}.{i}.", st) for st in self.stages if st["fused"] for i in range(st["depth"])]
                for pre, st in fused:
                    block_bias[pre] = act(st["heads"] * 64 * 64, dtype=torch.float32)
                if fused:
                    ops.relpos_bias_gather_batch(
                        ctx, [self._view(self.params, pre + "attn.relative_position_bias_table") for pre, _ in fused],
                        [st["pairs_dev"] for _, st in fused], [block_bias[pre] for pre, _ in fused])
            for si, st in enumerate(self.stages):
                C, R, ws, Hh = st["C"], st["R"], st["ws"], st["heads"]
                rows, N, D = B * R * R, ws * ws, C // Hh
                wrows = B * st["Rp"] ** 2       # rows of a window-ordered tensor: the frame padded to whole windows
                padded = wrows != rows
                B_ = wrows // N
                whole = ws == R                 # one window covers the image: window order == image order
                qkv_row, qkv_b = 3 * C, (N * 3 * C, D)
                s_b, o_b = (Hh * N * N, N * N), (N * C, D)
                scale = D ** -0.5
                for i in range(st["depth"]):
                    pre = f"features.{st['f']}.{i}."
                    shift = st["shift"] if i % 2 == 1 else 0
                    stats1, stats2 = new_ln(rows), new_ln(rows)
                    if whole:
                        xw = act(rows, C)
                        ln_fwd(pre + "norm1", x, xw, stats1)
                    elif self.fuse_window_ln:
                        xw = act(wrows, C)   # LayerNorm and window partition in one pass
                        if padded:
                            ops.fill_zero(ctx, xw)      # the tokens of the padding are zeros behind norm1
                        ln_fwd(pre + "norm1", x, xw, stats1, window=(R, R, ws, shift))
                    else:
                        n1, xw = v2(s_n1, rows, C), act(rows, C)
                        ln_fwd(pre + "norm1", x, n1, stats1)
                        ops.window_partition(ctx, n1, xw, ws, shift, image_shape=(B, R, R, C))
                    qkv = act(wrows, 3 * C)
                    lin_fwd(pre + "attn.qkv", xw, qkv)
                    fq = qkv.view(-1)
                    o = act(wrows, C)
                    if st["fused"]:
                        Pm = act(B_ * Hh, N, 64)
                        bias = block_bias.get(pre)
                        if bias is None:
                            bias = bias_buf[:Hh * 64 * 64]
                            ops.relpos_bias_gather_pairs(ctx, self._view(self.params, pre + "attn.relative_position_bias_table"),
                                                         st["pairs_dev"], bias)
                        ops.window_attn_fwd(ctx, qkv, o, Pm, bias, st["mask_dev"] if shift else None, B_, Hh, N, scale)
                    else:
                        Pm = act(B_, Hh, N, N)
                        ops.batched_gemm(ctx, fq, fq[C:], Pm, N, N, D, (qkv_row, 1), (qkv_row, 1), N, (B_, Hh), qkv_b, qkv_b,
                                         s_b, alpha=scale)
                        bias = bias_buf[:Hh * N * N].view(Hh, N, N)
                        ops.relpos_bias_gather(ctx, self._view(self.params, pre + "attn.relative_position_bias_table"),
                                               st["index_dev"], bias)
                        ops.attn_softmax_fwd(ctx, Pm, Pm, 1.0, bias=bias, mask=st["mask_dev"] if shift else None)
                        ops.batched_gemm(ctx, Pm, fq[2 * C:], o, N, D, N, (N, 1), (1, qkv_row), C, (B_, Hh), s_b, qkv_b, o_b)
                    x1 = act(rows, C)
                    n2, f1, f2, x2 = act(rows, C), act(rows, 4 * C), act(rows, 4 * C), act(rows, C)
                    if whole:
                        lin_fwd(pre + "attn.proj", o, x1, add=x)
                        ln_fwd(pre + "norm2", x1, n2, stats2)
                    elif self.fuse_window_ln:
                        # x1 = x + window_reverse(projection) and n2 = LayerNorm(x1) in one pass (what the projection
                        # left on the tokens of the padding is never read: the crop)
                        pr = v2(s_n1, wrows, C)
                        lin_fwd(pre + "attn.proj", o, pr)
                        ln_fwd(pre + "norm2", x, n2, stats2, window=(R, R, ws, shift), windowed=("add",), add=pr, sum_out=x1)
                    else:
                        pr = v2(s_n1, rows, C)
                        lin_fwd(pre + "attn.proj", o, pr)
                        ops.window_partition(ctx, pr, x1, ws, shift, reverse=True, add=x, image_shape=(B, R, R, C))
                        ln_fwd(pre + "norm2", x1, n2, stats2)
                    lin_fwd(pre + "mlp.0", n2, f1)
                    ops.gelu_fwd(ctx, f1, f2, tanh_form=False)
                    lin_fwd(pre + "mlp.3", f2, x2, add=x1)
                    saved_blocks.append((si, i, shift, x, xw, qkv, Pm, o, x1, n2, f1, f2, stats1, stats2))
                    x = x2
                    mark("fwd", pre[:-1])
                if si + 1 < len(self.stages):
                    pre = f"features.{st['f'] + 1}."
                    mrows = B * ((R + 1) // 2) ** 2
                    xm, nm, y = act(mrows, 4 * C), act(mrows, 4 * C), act(mrows, 2 * C)
                    mstats = new_ln(mrows)
                    ops.patch_merge_gather(ctx, x, xm, (B, R, R, C))
                    ln_fwd(pre + "norm", xm, nm, mstats)
                    lin_fwd(pre + "reduction", nm, y, bias=False)
                    saved_merges.append((si, xm, nm, mstats))
                    x = y
                    mark("fwd", pre[:-1])
            stL = self.stages[-1]
            rowsL, CL = B * stL["R"] ** 2, stL["C"]
            hf, pooled = act(rowsL, CL), act(B, CL)
            final_stats = new_ln(rowsL)
            ln_fwd("norm", x, hf, final_stats)
            ops.avgpool_fwd(ctx, hf.view(B, stL["R"], stL["R"], CL), pooled)
            logits = act(B, self.num_classes, dtype=torch.float32)
            ops.conv2d_fwd(ctx, pooled.view(B, 1, 1, CL), self._w("head.weight"), logits.view(B, 1, 1, self.num_classes), 1, 0,
                           bias=self._view(self.params, "head.bias"))
            dlogits = act(B, self.num_classes)
            ops.softmax_ce_fwd_bwd(ctx, logits, plan.labels, plan.loss_rows, plan.loss, dlogits, loss_scale=loss_scale)
            plan.n_forward = len(prog)
            mark("fwd", "loss")

            # ================= backward =================
            if self.overlap_wgrad:
                ctx.join()      # the second lane may still be writing the transposed filters of the last optimizer step
            g_pooled = v2(g_bufs[0], B, CL)
            lin_bwd("head", pooled, dlogits, g_pooled)
            g_hf = v2(g_bufs[1], rowsL, CL)
            ops.avgpool_bwd(ctx, g_pooled, g_hf.view(B, stL["R"], stL["R"], CL))
            gi = 2                                            # index of the buffer that holds the running gradient
            g = v2(g_bufs[gi], rowsL, CL)
            ln_bwd("norm", g_hf, x, g, final_stats)
            mark("bwd", "norm")
            merges = {si: m for si, *m in saved_merges}
            bi = len(saved_blocks)
            for si in range(len(self.stages) - 1, -1, -1):
                st = self.stages[si]
                C, R, ws, Hh = st["C"], st["R"], st["ws"], st["heads"]
                rows, N, D = B * R * R, ws * ws, C // Hh
                wrows = B * st["Rp"] ** 2
                padded = wrows != rows
                mrows = B * ((R + 1) // 2) ** 2
                B_ = wrows // N
                whole = ws == R
                qkv_row, qkv_b = 3 * C, (N * 3 * C, D)
                s_b, o_b = (Hh * N * N, N * N), (N * C, D)
                scale = D ** -0.5
                if si + 1 < len(self.stages):
                    # g is the gradient of the merged tokens [rows/4, 2C]
                    xm, nm, mstats = merges[si]
                    pre = f"features.{st['f'] + 1}."
                    spare = [k for k in range(len(g_bufs)) if k != gi]
                    d_nm = v2(g_4c_a, mrows, 4 * C)
                    with side():
                        wgrad(as4(nm), as4(g), self._view(self.grads, pre + "reduction.weight"))
                    ops.conv2d_dgrad(ctx, as4(g), self._wt(pre + "reduction.weight"), as4(d_nm), 1, 0)
                    d_xm = v2(g_4c_b, mrows, 4 * C)
                    ln_bwd(pre + "norm", d_nm, xm, d_xm, mstats)
                    gi = spare[0]
                    g = v2(g_bufs[gi], rows, C)
                    ops.patch_merge_gather(ctx, d_xm, g, (B, R, R, C), reverse=True)
                    if self.overlap_wgrad:
                        ctx.join()
                    mark("bwd", pre[:-1])
                for i in range(st["depth"] - 1, -1, -1):
                    bi -= 1
                    _, _, shift, x_in, xw, qkv, Pm, o, x1, n2, f1, f2, stats1, stats2 = saved_blocks[bi]
                    pre = f"features.{st['f']}.{i}."
                    spare = [k for k in range(len(g_bufs)) if k != gi]
                    # t_b, t_c, t_d carry window-ordered gradients (the padded frame's rows) wherever the block has windows
                    t_a, t_e = v2(g_bufs[spare[0]], rows, C), v2(g_bufs[spare[4]], rows, C)
                    t_b, t_c, t_d = (v2(g_bufs[k], wrows, C) for k in spare[1:4])
                    d_f2, d_f1, d_qkv = v2(g_4c_a, rows, 4 * C), v2(g_4c_b, rows, 4 * C), v2(g_3c, wrows, 3 * C)
                    fq, fg = qkv.view(-1), d_qkv.view(-1)
                    dP = d_scores[:B_ * Hh * N * st["keys_ld"]].view(B_, Hh, N, st["keys_ld"])
                    # MLP
                    lin_bwd(pre + "mlp.3", f2, g, d_f2)
                    ops.gelu_bwd(ctx, d_f2, f1, d_f1, tanh_form=False)
                    lin_bwd(pre + "mlp.0", n2, d_f1, t_a)
                    g1 = t_b
                    fuse_w = self.fuse_window_ln and not whole
                    win = (R, R, ws, shift)
                    # attention
                    if fuse_w:
                        # the gradient behind norm2 is written as window tokens right away: the projection's gradients
                        # want it in that order, and norm1's backward reads its residual through the same map
                        if padded:
                            ops.fill_zero(ctx, g1)      # no gradient reaches the projection's output on the padding
                        ln_bwd(pre + "norm2", t_a, x1, g1, stats2, residual=g, window=win, windowed=("dx",))
                        d_pr = g1
                    elif whole:
                        ln_bwd(pre + "norm2", t_a, x1, g1, stats2, residual=g)
                        d_pr = g1
                    else:
                        ln_bwd(pre + "norm2", t_a, x1, g1, stats2, residual=g)
                        d_pr = t_a
                        ops.window_partition(ctx, g1, d_pr, ws, shift, image_shape=(B, R, R, C))
                    d_o = t_c
                    lin_bwd(pre + "attn.proj", o, d_pr, d_o)
                    if st["fused"]:
                        ops.window_attn_bwd(ctx, qkv, Pm, d_o, d_qkv, dP, B_, Hh, N, scale)
                        dbias = dbias_buf[:Hh * N * 64]
                        with side():
                            # the sum over the windows in 16-byte pieces (rows are a multiple of 8 wide), then
                            # each table entry collects its pairs through the inverse index
                            ops.bias_grad(ctx, dP.view(B_, Hh * N * 64), dbias, workspace=colsum_ws)
                            ops.relpos_bias_scatter_csr(ctx, dbias, st["inv_ptr_dev"], st["inv_list_dev"],
                                                        self._view(self.grads, pre + "attn.relative_position_bias_table")
                                                        .view(-1, Hh), N * 64)
                    else:
                        ops.batched_gemm(ctx, Pm, d_o, fg[2 * C:], N, D, N, (1, N), (1, C), qkv_row, (B_, Hh), s_b, o_b, qkv_b)
                        ops.batched_gemm(ctx, d_o, fq[2 * C:], dP, N, N, D, (C, 1), (qkv_row, 1), N, (B_, Hh), o_b, qkv_b, s_b)
                        ops.attn_softmax_bwd(ctx, Pm, dP, dP, 1.0)
                        dbias = dbias_buf[:Hh * N * N]
                        with side():
                            ops.column_sum(ctx, dP.view(B_, Hh * N * N), dbias, colsum_ws)
                            ops.relpos_bias_scatter(ctx, dbias, st["index_dev"],
                                                    self._view(self.grads, pre + "attn.relative_position_bias_table"))
                        ops.batched_gemm(ctx, dP, fq[C:], fg, N, D, N, (N, 1), (1, qkv_row), qkv_row, (B_, Hh), s_b, qkv_b,
                                         qkv_b, alpha=scale)
                        ops.batched_gemm(ctx, dP, fq, fg[C:], N, D, N, (1, N), (1, qkv_row), qkv_row, (B_, Hh), s_b, qkv_b,
                                         qkv_b, alpha=scale)
                    d_xw = t_d
                    lin_bwd(pre + "attn.qkv", xw, d_qkv, d_xw)
                    # the new running gradient goes into a buffer of its own: the old one may still be read by
                    # this block's first weight gradient on the second lane
                    g_next = t_e
                    if fuse_w:
                        ln_bwd(pre + "norm1", d_xw, x_in, g_next, stats1, residual=g1, window=win,
                               windowed=("dy", "residual"))
                    else:
                        if whole:
                            d_n1 = d_xw
                        else:
                            d_n1 = t_c
                            ops.window_partition(ctx, d_xw, d_n1, ws, shift, reverse=True, image_shape=(B, R, R, C))
                        ln_bwd(pre + "norm1", d_n1, x_in, g_next, stats1, residual=g1)
                    g, gi = g_next, spare[4]
                    if self.overlap_wgrad:
                        ctx.join()
                    mark("bwd", pre[:-1])
            # patch embedding: LayerNorm, then the 4x4 stride-4 convolution (no data gradient: it is the input)
            spare = [k for k in range(len(g_bufs)) if k != gi]
            d_e0 = v2(g_bufs[spare[0]], rows0, C0)
            ln_bwd("features.0.2", g, e0, d_e0, embed_stats)
            # on the main lane, behind the join that ended the last block: the second lane's last weight gradient has
            # finished, so its pending reduction may ride this launch; this one's own reduction follows at once
            wgrad(x0, d_e0.view(B, R0, R0, C0), self._view(self.grads, "features.0.0.weight"), stride=P, c_logical=3)
            if trail is not None:
                trail.flush()
            ops.bias_grad(ctx, d_e0, self._view(self.grads, "features.0.0.bias"), workspace=bias_ws)
            if self.overlap_wgrad:
                ctx.join()
            mark("bwd", "features.0")
        finally:
            ctx.end_record()
        plan.prog, plan.marks, plan.keep, plan.logits = prog, marks, keep, logits
        plan.bytes = sum(t.numel() * t.element_size() for t in keep)
        return plan

    # ------------------------------------------------------------------ the step
    def forward_backward(self, x, y, loss_scale=1.0):
        """x [B,3,S,S] fp32 and y [B] int64 on the GPU.  Returns (plan, cut_short)."""
        p = self._last_plan = self.plan(x.shape[0], loss_scale)
        self.ctx.flush()
        p.x_in.copy_(x, non_blocking=True)
        p.labels.copy_(y, non_blocking=True)
        return p, self._run_plan(p)

    def _record_optimizer(self, grads):
        ops.adamw_step(self.ctx, self.params, grads, self.exp_avg, self.exp_avg_sq, self.step_dev, self.adam_scalars,
                       lr=self.lr, beta1=self.betas[0], beta2=self.betas[1], eps=self.eps,
                       weight_decay=self.weight_decay, shadow=self.shadow)
        # the transposed copies are read by the data gradients only: made on the second lane, beside the next
        # step's forward pass; the backward program joins the lanes before its first data gradient
        if self.overlap_wgrad:
            with self.ctx.side_lane(wait_main=True):
                self._refresh_transposed()
        else:
            self._refresh_transposed()
