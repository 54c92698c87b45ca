"""GPT-2 training-step engine over the HIP operators.

What the reference does with ``GPT2LMHeadModel`` + autograd + an optimizer (train/gpt2.py:26-33,
90-97: forward with labels = input ids, ``output.loss``, backward, step), this engine does with one
recorded program of hand-written kernels per batch size:

* parameters, gradients and optimizer state live in flat fp32 buffers; projection weights are kept
  [out, in] (the filter layout of the 1x1 convolution kernels, which run every projection and the
  output head on MFMA); bf16 mode keeps a flat bf16 shadow the kernels read;
* the vocabulary is padded to a multiple of 128 rows of zeros (they never receive a gradient), so the
  output head and its two gradients run on the direct-to-LDS GEMM kernel;
* attention reads the packed [B, T, 3, heads, head_dim] projection in place: in bf16 with heads 64 wide
  and a sequence length that is a multiple of 128 it is one fused launch forward (scores never leave the
  chip, the log-sum-exp is kept) and two backward; otherwise batched strided GEMMs and a causal softmax
  over materialised [B, heads, T, T] scores (kept for the backward);
* backward is written out by hand; the gradient that bypasses a LayerNorm is added inside the
  LayerNorm backward; the token embedding receives the head's weight gradient and then the scattered
  embedding gradient (tied weights);
* state dicts use transformers' names and its [in, out] orientation of the projection weights.

torch supplies device memory and streams only.  Dropout is off (probabilities 0).
"""
import contextlib
import math
import os

import torch

from . import ops
from .engine_base import EngineBase


class _Param:
    __slots__ = ("name", "kind", "shape", "store_shape", "offset", "numel")

    def __init__(self, name, kind, shape, store_shape, offset):
        self.name, self.kind, self.shape, self.store_shape, self.offset = name, kind, shape, store_shape, offset
        self.numel = int(math.prod(store_shape))


class _Plan:
    pass


class GPT2Engine(EngineBase):
    def __init__(self, vocab=50257, n_pos=1024, n_embd=768, n_layer=12, n_head=12, seq_len=1024, dtype=torch.bfloat16,
                 optimizer="adamw", lr=1e-3, weight_decay=0.01, betas=(0.9, 0.999), eps=1e-8, momentum=0.9,
                 stream=None, allocator=None, overlap_wgrad=True, fused_attention=True, trailing_wgrad=True,
                 trailing_reduce=None):
        self._init_engine(dtype, stream, allocator)
        # trailing_reduce: the split reduction of a weight gradient rides the next weight-gradient launch as extra
        # workgroups instead of being a launch of its own (same bits)
        self.trailing_reduce = (os.environ.get("TCH_TRAILING_REDUCE", "1") != "0") if trailing_reduce is None \
            else bool(trailing_reduce)
        # weight and bias gradients depend only on a saved activation and on a gradient that stays put until
        # the layer is done: recorded on a second lane, they run beside the data-gradient chain; the lanes
        # meet at the end of every layer, before its gradient buffers are handed round again
        self.overlap_wgrad = overlap_wgrad
        # trailing_wgrad: three sets of gradient buffers taken in turn, so that the second lane may trail the first
        # by a layer instead of meeting it at the end of every layer
        self.trailing_wgrad = trailing_wgrad and overlap_wgrad
        self.fused_attention = fused_attention
        assert n_embd % n_head == 0 and n_embd % 8 == 0 and seq_len <= n_pos
        assert optimizer in ("adamw", "sgd")
        self.vocab, self.n_pos, self.C, self.n_layer, self.n_head = vocab, n_pos, n_embd, n_layer, n_head
        self.D = n_embd // n_head
        self.T = seq_len
        self.vocab_pad = (vocab + 127) // 128 * 128
        self.optimizer, self.lr, self.weight_decay = optimizer, lr, weight_decay
        self.betas, self.eps, self.momentum = betas, eps, momentum
        C = n_embd

        self._specs, self._off = [], 0
        self._add("transformer.wte.weight", "embed", (vocab, C), (self.vocab_pad, 1, 1, C))
        self._add("transformer.wpe.weight", "plain", (n_pos, C), (n_pos, C))
        for i in range(n_layer):
            p = f"transformer.h.{i}."
            self._add_vec(p + "ln_1.weight", C)
            self._add_vec(p + "ln_1.bias", C)
            self._add_linear(p + "attn.c_attn", C, 3 * C)
            self._add_linear(p + "attn.c_proj", C, C)
            self._add_vec(p + "ln_2.weight", C)
            self._add_vec(p + "ln_2.bias", C)
            self._add_linear(p + "mlp.c_fc", C, 4 * C)
            self._add_linear(p + "mlp.c_proj", 4 * C, C)
        self._add_vec("transformer.ln_f.weight", C)
        self._add_vec("transformer.ln_f.bias", C)
        self.n_store = self._off
        self.spec = {p.name: p for p in self._specs}

        def zeros(n, dt=torch.float32):
            return self._alloc((n,), dt).zero_()
        self.params = zeros(self.n_store)
        self.grads = zeros(self.n_store)
        self.shadow = zeros(self.n_store, torch.bfloat16) if dtype == torch.bfloat16 else None
        self.wt = zeros(self.n_store, dtype)   # projection weights transposed to [in, out] for the data gradients
        self._tt = ops.FilterTransposeTable(
            [(p.offset, p.store_shape[0], 1, p.store_shape[3]) for p in self._specs if p.kind in ("linear", "embed")],
            self.dev)
        if optimizer == "adamw":
            self.exp_avg, self.exp_avg_sq = zeros(self.n_store), zeros(self.n_store)
            self.step_dev = self._alloc((1,), torch.int32).zero_()
            self.adam_scalars = zeros(2)
        else:
            self.momentum_buf = zeros(self.n_store)

    # ------------------------------------------------------------------ parameter table
    def _add(self, name, kind, shape, store_shape):
        p = _Param(name, kind, shape, store_shape, self._off)
        self._specs.append(p)
        self._off += (p.numel + 7) // 8 * 8
        return p

    def _add_vec(self, name, n):
        self._add(name, "vec", (n,), (n,))

    def _add_linear(self, name, cin, cout):
        self._add(name + ".weight", "linear", (cin, cout), (cout, 1, 1, cin))
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
        if p.kind == "linear":
            t = t.t()
        elif p.kind == "embed":
            t = torch.nn.functional.pad(t, (0, 0, 0, p.store_shape[0] - t.shape[0]))
        return t.reshape(p.store_shape).contiguous()

    def _from_store(self, p, flat):
        t = flat[p.offset:p.offset + p.numel].view(p.store_shape)
        if p.kind == "linear":
            t = t.view(p.store_shape[0], p.store_shape[3]).t()
        elif p.kind == "embed":
            t = t.view(p.store_shape[0], p.store_shape[3])[:p.shape[0]]
        return t.reshape(p.shape).contiguous().cpu()

    def load_state_dict(self, sd):
        """Weights from a transformers-style state dict (CPU tensors, projection weights [in, out])."""
        host = torch.zeros(self.n_store, dtype=torch.float32)
        for p in self._specs:
            host[p.offset:p.offset + p.numel] = self._to_store(p, sd[p.name]).reshape(-1)
        self.params.copy_(host)
        self.grads.zero_()
        self._reset_optimizer_state()
        self.refresh_shadow()
        torch.cuda.synchronize()

    def init_normal(self, seed=0):
        """GPT-2's initialisation, generated on the GPU: N(0, 0.02) weights, residual projections scaled by
        1/sqrt(2 n_layer), zero biases, LayerNorm gamma 1 / beta 0."""
        g = torch.Generator(device=self.dev)
        g.manual_seed(seed)
        for p in self._specs:
            v = self._view(self.params, p.name)
            if p.kind == "vec":
                v.fill_(1.0 if p.name.endswith(("ln_1.weight", "ln_2.weight", "ln_f.weight")) else 0.0)
            else:
                std = 0.02 / math.sqrt(2 * self.n_layer) if p.name.endswith("c_proj.weight") else 0.02
                v.normal_(0.0, std, generator=g)
                if p.kind == "embed":
                    v[p.shape[0]:] = 0
        self.grads.zero_()
        self._reset_optimizer_state()
        self.refresh_shadow()
        torch.cuda.synchronize()

    def _reset_optimizer_state(self):
        if self.optimizer == "adamw":
            self.exp_avg.zero_()
            self.exp_avg_sq.zero_()
            self.step_dev.zero_()
        else:
            self.momentum_buf.zero_()

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
        T_, ctx = self.dtype, self.ctx
        T, C, H, D, L, V, Vp = self.T, self.C, self.n_head, self.D, self.n_layer, self.vocab, self.vocab_pad
        R = B * T
        plan = _Plan()
        plan.batch, plan.loss_scale = B, loss_scale
        keep = []

        def act(*shape, dtype=T_):
            t = self._alloc(tuple(shape), dtype)
            keep.append(t)
            return t

        code = ops.dtype_code(torch.empty(0, dtype=T_))
        plan.ids = act(B, T, dtype=torch.int64).zero_()
        plan.labels = act(R, dtype=torch.int64).zero_()
        plan.loss_rows = act(R, dtype=torch.float32)
        plan.loss = act(1, dtype=torch.float32)
        ln_mean, ln_rstd = act((2 * L + 1) * R, dtype=torch.float32), act((2 * L + 1) * R, dtype=torch.float32)
        ln_partial = act(ops.layernorm_bwd_partial_rows(R) * C * 2, dtype=torch.float32)

        # the weight-gradient workspace over every projection of the plan
        ws_bytes = 4
        for p in self._specs:
            if p.kind in ("linear", "embed"):
                K, _, _, Cin = p.store_shape
                sp = int(ops.lib().tch_conv2d_wgrad_pick_splits(code, R, 1, 1, Cin, K, 1, 1, 1, 0))
                ws_bytes = max(ws_bytes, ops.conv2d_wgrad_workspace_bytes(code, K, 1, 1, Cin, sp))
        # two workspaces taken in turn: the split reduction of a weight gradient rides the launch of the next one
        wg_half = (ws_bytes // 4 + 63) // 64 * 64
        wg_ws = act(2 * wg_half, dtype=torch.float32)
        trail = ops.TrailingWgrad(ctx, wg_ws, wg_half) if self.trailing_reduce else None

        def wgrad(x4, dy4, dw, dbias=None):
            if trail is not None:
                return trail.wgrad(x4, dy4, dw, 1, 0, dbias=dbias)
            ops.conv2d_wgrad(ctx, x4, dy4, dw, 1, 0, workspace=wg_ws, dbias=dbias)

        def ln_stats(i):
            return ln_mean[i * R:(i + 1) * R], ln_rstd[i * R:(i + 1) * R]

        def ln_fwd(name, idx, x, y):
            m, r = ln_stats(idx)
            ops.layernorm_fwd(ctx, x, y, self._view(self.params, name + ".weight"), self._view(self.params, name + ".bias"),
                              m, r)

        def ln_bwd(name, idx, dy, x, dx, residual=None):
            m, r = ln_stats(idx)
            ops.layernorm_bwd(ctx, dy, x, dx, self._view(self.params, name + ".weight"), m, r,
                              self._view(self.grads, name + ".weight"), self._view(self.grads, name + ".bias"), ln_partial,
                              residual=residual)

        def as4(t):
            return t.view(t.shape[0], 1, 1, t.shape[1])

        def lin_fwd(name, x, y, add=None):
            ops.conv2d_fwd(ctx, as4(x), self._w(name + ".weight"), as4(y), 1, 0,
                           bias=self._view(self.params, name + ".bias"), add=None if add is None else as4(add))

        def side():
            return ctx.side_lane(wait_main=True) if self.overlap_wgrad else contextlib.nullcontext()

        def lin_bwd(name, x, dy, dx):
            """dW, db from (x, dy); dx = dy W"""
            with side():
                wgrad(as4(x), as4(dy), self._view(self.grads, name + ".weight"), self._view(self.grads, name + ".bias"))
            ops.conv2d_dgrad(ctx, as4(dy), self._wt(name + ".weight"), as4(dx), 1, 0)

        # strides / batch offsets of head h of sample b inside the packed projection and the score tensor
        qkv_row, qkv_b = 3 * C, (T * 3 * C, D)
        s_b, o_b = (H * T * T, T * T), (T * C, D)
        scale = 1.0 / math.sqrt(D)
        # one fused pass per direction where the kernel's shape limits hold; the three-launch chain otherwise
        fused = self.fused_attention and self.dtype == torch.bfloat16 and D == 64 and T % 128 == 0

        prog = ops.Program()
        marks = []

        def mark(phase, name):
            marks.append((len(prog), phase, name))

        ctx.begin_record(prog)
        try:
            # ================= forward =================
            h = act(R, C)
            ops.embedding_fwd(ctx, plan.ids, self._w("transformer.wte.weight").view(Vp, C),
                              self._w("transformer.wpe.weight"), h.view(B, T, C))
            saved = []
            for i in range(L):
                pre = f"transformer.h.{i}."
                a, qkv = act(R, C), act(R, 3 * C)
                ln_fwd(pre + "ln_1", 2 * i, h, a)
                lin_fwd(pre + "attn.c_attn", a, qkv)
                flat = qkv.view(-1)
                o = act(R, C)
                if fused:
                    # P is the log-sum-exp here: all the backward needs to rebuild the probabilities
                    P = act(B * H, T, dtype=torch.float32)
                    ops.flash_attn_fwd(ctx, flat, flat[C:], flat[2 * C:], o.view(-1), P, B, H, T, (qkv_row, T * qkv_row),
                                       (C, T * C), scale, causal=True)
                else:
                    P = act(B, H, T, T)
                    ops.batched_gemm(ctx, flat, flat[C:], P, T, T, D, (qkv_row, 1), (qkv_row, 1), T, (B, H), qkv_b, qkv_b,
                                     s_b, causal=1)
                    ops.attn_softmax_fwd(ctx, P, P, scale, causal=True)
                    ops.batched_gemm(ctx, P, flat[2 * C:], o, T, D, T, (T, 1), (1, qkv_row), C, (B, H), s_b, qkv_b, o_b,
                                     causal=2)
                h1 = act(R, C)
                lin_fwd(pre + "attn.c_proj", o, h1, add=h)
                m, f1, f2 = act(R, C), act(R, 4 * C), act(R, 4 * C)
                ln_fwd(pre + "ln_2", 2 * i + 1, h1, m)
                lin_fwd(pre + "mlp.c_fc", m, f1)
                ops.gelu_fwd(ctx, f1, f2, tanh_form=True)
                h2 = act(R, C)
                lin_fwd(pre + "mlp.c_proj", f2, h2, add=h1)
                saved.append((h, a, qkv, P, o, h1, m, f1, f2))
                h = h2
                mark("fwd", f"h.{i}")
            hf = act(R, C)
            ln_fwd("transformer.ln_f", 2 * L, h, hf)
            logits = act(R, Vp, dtype=torch.float32)
            ops.conv2d_fwd(ctx, as4(hf), self._w("transformer.wte.weight"), as4(logits), 1, 0)
            dlogits = act(R, Vp).zero_()   # the padding columns stay zero: no kernel writes them
            ops.softmax_ce_lm(ctx, logits, plan.labels, plan.loss_rows, plan.loss, dlogits, V, B * (T - 1), loss_scale)
            plan.n_forward = len(prog)
            mark("fwd", "loss")

            # ================= backward =================
            if self.overlap_wgrad:
                ctx.join()      # the second lane may still be writing the transposed filters of the last optimizer step
            # Gradient buffers, handed round.  The second lane reads a layer's incoming gradient and three of the
            # layer's own (the right-hand sides of its four weight gradients).  With one set the lanes would have
            # to meet at the end of every layer; with three sets taken in turn the second lane may trail the first
            # by a layer: what layer j reads lies in the sets of layers j-1 and j, layer j+1 writes a third set,
            # and before layer j+2 takes the first set again the main lane has waited for layer j's weight gradients.
            n_sets = 3 if self.trailing_wgrad else 1
            g_sets = [([act(R, C) for _ in range(4 if k == 0 else 3)], act(R, 4 * C), act(R, 3 * C)) for k in range(n_sets)]
            g_c = g_sets[0][0]
            g_f2 = act(R, 4 * C)                      # main lane only
            dP = act(B * H, T, dtype=torch.float32) if fused else act(B, H, T, T)   # fused: the delta scratch
            d_hf, g = g_c[0], g_c[1]
            with side():
                wgrad(as4(hf), as4(dlogits), self._view(self.grads, "transformer.wte.weight"))
            ops.conv2d_dgrad(ctx, as4(dlogits), self._wt("transformer.wte.weight"), as4(d_hf), 1, 0)
            ln_bwd("transformer.ln_f", 2 * L, d_hf, h, g)
            mark("bwd", "ln_f")
            for i in range(L - 1, -1, -1):
                pre = f"transformer.h.{i}."
                h_in, a, qkv, P, o, h1, m, f1, f2 = saved[i]
                own_c, g_f1, g_qkv = g_sets[(L - i) % n_sets]
                flat, gflat = qkv.view(-1), g_qkv.view(-1)
                spare = [t for t in own_c if t is not g]
                d_m, g1, d_o = spare[0], spare[1], spare[2]
                # MLP
                lin_bwd(pre + "mlp.c_proj", f2, g, g_f2)
                ops.gelu_bwd(ctx, g_f2, f1, g_f1, tanh_form=True)
                lin_bwd(pre + "mlp.c_fc", m, g_f1, d_m)
                ln_bwd(pre + "ln_2", 2 * i + 1, d_m, h1, g1, residual=g)
                # attention
                lin_bwd(pre + "attn.c_proj", o, g1, d_o)
                if fused:
                    ops.flash_attn_bwd(ctx, flat, flat[C:], flat[2 * C:], o.view(-1), d_o.view(-1), P, dP, gflat,
                                       gflat[C:], gflat[2 * C:], B, H, T, (qkv_row, T * qkv_row), (C, T * C), scale,
                                       causal=True)
                else:
                    ops.batched_gemm(ctx, P, d_o, gflat[2 * C:], T, D, T, (1, T), (1, C), qkv_row, (B, H), s_b, o_b, qkv_b,
                                     causal=3)
                    ops.batched_gemm(ctx, d_o, flat[2 * C:], dP, T, T, D, (C, 1), (qkv_row, 1), T, (B, H), o_b, qkv_b, s_b,
                                     causal=1)
                    ops.attn_softmax_bwd(ctx, P, dP, dP, scale, causal=True)
                    ops.batched_gemm(ctx, dP, flat[C:], gflat, T, D, T, (T, 1), (1, qkv_row), qkv_row, (B, H), s_b, qkv_b,
                                     qkv_b, causal=2)
                    ops.batched_gemm(ctx, dP, flat, gflat[C:], T, D, T, (1, T), (1, qkv_row), qkv_row, (B, H), s_b, qkv_b,
                                     qkv_b, causal=3)
                d_a = d_m   # free again
                lin_bwd(pre + "attn.c_attn", a, g_qkv, d_a)
                g_next = d_o
                ln_bwd(pre + "ln_1", 2 * i, d_a, h_in, g_next, residual=g1)
                g = g_next
                if self.overlap_wgrad:
                    ctx.join(behind=self.trailing_wgrad)
                mark("bwd", f"h.{i}")
            if trail is not None:
                with side():
                    trail.flush()     # the last weight gradient's own reduction
            if self.overlap_wgrad:
                ctx.join()
            # tied weights: the scattered embedding gradient lands on top of the head's weight gradient
            ops.embedding_bwd(ctx, plan.ids, g.view(B, T, C), self._view(self.grads, "transformer.wte.weight").view(Vp, C),
                              self._view(self.grads, "transformer.wpe.weight"), chain=act(2 * B * T, dtype=torch.int32))
        finally:
            ctx.end_record()
        plan.prog, plan.marks, plan.keep, plan.logits = prog, marks, keep, logits
        plan.bytes = sum(t.numel() * t.element_size() for t in keep)
        return plan

    # ------------------------------------------------------------------ the step
    def forward_backward(self, ids, loss_scale=1.0):
        """ids [B, T] int64 on the GPU; labels are the ids shifted by one (transformers' causal LM loss).
        Returns (plan, cut_short)."""
        B, T = ids.shape
        assert T == self.T, f"this engine was built for sequences of {self.T} tokens"
        p = self._last_plan = self.plan(B, loss_scale)
        self.ctx.flush()
        p.ids.copy_(ids, non_blocking=True)
        lab = p.labels.view(B, T)
        lab[:, :-1].copy_(ids[:, 1:], non_blocking=True)
        lab[:, -1].fill_(-100)
        return p, self._run_plan(p)

    def _record_optimizer(self, grads):
        if self.optimizer == "adamw":
            ops.adamw_step(self.ctx, self.params, grads, self.exp_avg, self.exp_avg_sq, self.step_dev, self.adam_scalars,
                           lr=self.lr, beta1=self.betas[0], beta2=self.betas[1], eps=self.eps,
                           weight_decay=self.weight_decay, shadow=self.shadow)
        else:
            ops.sgd_momentum_step(self.ctx, self.params, grads, self.momentum_buf, self.lr, self.momentum,
                                  self.weight_decay, shadow=self.shadow)
        # the transposed copies are read by the data gradients only: made on the second lane, beside the next
        # step's forward pass; the backward program joins the lanes before its first data gradient
        if self.overlap_wgrad:
            with self.ctx.side_lane(wait_main=True):
                self._refresh_transposed()
        else:
            self._refresh_transposed()
