"""ResNet (Bottleneck) training-step engine over the HIP operators.

What the reference does with ``torchvision.models.resnet152`` + autograd +
``torch.optim.SGD`` (train/resnet152.py:22-29,84-91), this engine does with one
recorded program of hand-written kernels per batch size:

* parameters, gradients and momentum live in three flat fp32 buffers (filters in
  [K,R,S,C] order, the stem's 3 input channels zero-padded to one 16-byte chunk);
  bf16 mode keeps a flat bf16 shadow the kernels read, rewritten by the optimizer;
* activations are NHWC in the compute dtype; per batch size a static plan owns
  them, so a step is a replay of pre-bound launches (no Python per kernel);
* backward is written out by hand (no autograd): BatchNorm backward takes the
  ReLU mask of the block output, the identity branch is added in the epilogue of
  the first convolution's data gradient;
* the reject flag of the launch queues is a checkpoint between any two launches:
  a replay that was cut short reports it, the caller frees the plan
  (``release_activations``) and the memory returns to the pool.

torch supplies device memory and streams only.
"""
import math
import os

import torch

from . import ops
from .engine_base import EngineBase

STEM_CIN_PAD = 8


class _Conv:
    def __init__(self, name, cin, cout, k, stride, pad):
        self.name, self.cin, self.cout, self.k, self.stride, self.pad = name, cin, cout, k, stride, pad
        self.cin_store = max(cin, STEM_CIN_PAD) if cin < STEM_CIN_PAD else cin


class _Param:
    __slots__ = ("name", "kind", "shape", "store_shape", "offset", "numel")

    def __init__(self, name, kind, shape, store_shape, offset):
        self.name, self.kind, self.shape, self.store_shape, self.offset = name, kind, shape, store_shape, offset
        self.numel = int(math.prod(store_shape))


class _Block:
    pass


class ResNetEngine(EngineBase):
    def __init__(self, depths=(3, 8, 36, 3), num_classes=1000, width=64, dtype=torch.bfloat16, image_size=224,
                 lr=0.1, momentum=0.9, weight_decay=1e-4, bn_momentum=0.1, bn_eps=1e-5, stream=None, allocator=None,
                 overlap_wgrad=True, fuse_bn_stats=True, fuse_bn_bwd=True, fuse_bn_finalize=False, autotune=False,
                 retain_gradients=False, group_wgrad=False, wgrad_group_wgs=256, wgrad_group_blocks=2,
                 wgrad_group_max_wgs=0, bn_acc=None, trailing_reduce=None):
        self._init_engine(dtype, stream, allocator)
        assert num_classes % 8 == 0, "class count must be a multiple of one 16-byte chunk"
        self.image_size, self.num_classes = image_size, num_classes
        self.lr, self.momentum, self.weight_decay = lr, momentum, weight_decay
        self.bn_momentum, self.bn_eps = bn_momentum, bn_eps
        self.depths, self.width = tuple(depths), width
        # weight gradients depend only on dy and the saved input: recorded on a second lane so that
        # they run beside the data-gradient chain (each kernel alone leaves CUs idle at batch 64);
        # costs the recycling of the dy buffers (they stay alive until the lanes join)
        self.overlap_wgrad = overlap_wgrad
        # group_wgrad: the weight gradients of the bottleneck convolutions are not launched layer by layer but
        # collected, and launched together once the data-gradient chain has left a stage (or every
        # wgrad_group_blocks blocks, if not 0): one launch over a table for all of them, sized for about
        # wgrad_group_wgs workgroups of equal length, so that a layer is split only where a whole stage would
        # not fill the chip.  Needs the second lane's rule that no dy buffer is handed out twice.  Off by default:
        # measured on ResNet-152 at batch 64, the grouped launches need 2.4 ms of kernel time per step instead of
        # 6.3 ms (745 against 320 TFLOP/s, no partial filters in stages 3 and 4, 300 launches fewer), but the step
        # is 16.5-17.1 ms against 16.3 ms: the many short launches run in the gaps of the data-gradient chain,
        # which is the critical path, while a launch that fills the chip holds that chain up for as long as it runs
        # (also when it is capped to one workgroup per compute unit).
        # fuse_eval_bn: the forward-only (inference) plan runs convolution + BatchNorm (+ residual) (+ ReLU) as one
        # launch each instead of two
        self.fuse_eval_bn = True
        # compact_downsample_dgrad: the data gradient of a stride-2 downsample convolution stays on the small grid
        self.compact_downsample_dgrad = True
        self.group_wgrad = group_wgrad and overlap_wgrad
        self.wgrad_group_wgs, self.wgrad_group_blocks = wgrad_group_wgs, wgrad_group_blocks
        self.wgrad_group_max_wgs = wgrad_group_max_wgs
        self.fuse_bn_stats = fuse_bn_stats
        # trailing_reduce: the split reduction of a weight gradient is not a launch of its own but rides the next
        # weight-gradient launch of the step as extra workgroups (two workspaces taken in turn); same bits
        self.trailing_reduce = (os.environ.get("TCH_TRAILING_REDUCE", "1") != "0") if trailing_reduce is None \
            else bool(trailing_reduce)
        # fuse_bn_bwd: a data-gradient convolution whose output flows into a BatchNorm(+ReLU) backward applies
        # the ReLU gate and takes that BatchNorm's two reductions in its epilogue (no reduction pass)
        self.fuse_bn_bwd = fuse_bn_bwd
        # fuse_bn_finalize: the convolution that leaves the sums also turns them into the BatchNorm's
        # coefficients (its last workgroup per column tile), so that only the apply launch follows.
        # Off by default: measured on MI355X at batch 64, the tail it adds to every convolution (two
        # round trips of device-scope atomics, then a few batches of uncached loads in one workgroup)
        # costs as much as the finalize launch it saves (20.2 ms per step against 19.3 ms)
        self.fuse_bn_finalize = fuse_bn_finalize
        # bn_acc: the convolution epilogues ADD their BatchNorm sums to exact integer accumulators (one pair per
        # channel, zeroed by one launch at the head of the step) instead of leaving them per row tile, and the
        # BatchNorm that follows is ONE launch that derives its coefficients from the two totals: no finalize
        # launch in the large stages, no pass over per-tile partials in the small ones.  bn_acc_max_rows bounds
        # the layers that take this form by their number of rows (0: all of them).
        # Off by default: measured on MI355X at batch 64 (same box, alternating runs), 20.4 ms per step with every
        # layer in this form, 17.8 ms with the layers of up to 60 000 rows, 16.8 ms with the 14x14 and 7x7 stages
        # only, against 15.6 ms without.  The BatchNorm launch gets 1.6 us shorter (12.9 -> 11.3 us) and 77
        # finalize launches go, but every convolution that adds to the accumulators gets 6-8 us LONGER: the
        # integer atomics of all row tiles of a channel meet at one address, a device-scope read-modify-write on
        # one address takes about 70 ns, and the kernel is not done before the last of them is (98 row tiles x 70 ns
        # = 7 us at 14x14, 1568 tiles at 56x56) -- that with one pair of words per channel, interleaved.  With the
        # words laid out in planes (512 contiguous bytes per atomic instruction) and the row tiles spread over 4 / 8
        # copies per channel the 14x14 and 7x7 stages alone cost 15.61 / 15.79 ms against 15.52 ms: still no gain,
        # what the shorter BatchNorm launch wins the tail of the convolution loses.  Same bits in the loss as the
        # per-tile form in every variant.
        self.bn_acc = (os.environ.get("TCH_BN_ACC", "0") != "0") if bn_acc is None else bool(bn_acc)
        self.bn_acc_max_rows = int(os.environ.get("TCH_BN_ACC_MAX_ROWS", "0"))
        self.bn_acc_copies = int(os.environ.get("TCH_BN_ACC_COPIES", "4"))   # row tile t adds to copy t % copies
        # autotune: when a plan is built, time each distinct convolution shape with every tiling and
        # keep the fastest (forward and data gradient separately); off = the library's heuristic
        self.autotune = autotune
        # tile_margin: see _pick_tiling (measured on the batch-64 step: 0 / 3 / 6 / 10 % -> 15.87 / 15.82 / 15.77 / 15.83 ms)
        self.tile_margin = float(os.environ.get("TCH_TILE_MARGIN", "0.05"))
        # retain_gradients: no gradient buffer of a plan is handed out twice, and the plan lists every
        # intermediate tensor of the step by name (plan.tensors): for inspection layer by layer; the launches,
        # their order and their tilings are those of the ordinary plan
        self.retain_gradients = retain_gradients
        self._tile_cache = {}
        self.tile_timings = {}   # what the tuner measured: {shape key: {"fwd_ms": {cfg: ms}, "dgrad_ms": {cfg: ms}}}

        # ---- architecture + parameter table (torchvision naming and order) ----
        self._specs, self._bn_names = [], []
        self._off = 0
        self.stem = _Conv("conv1", 3, width, 7, 2, 3)
        self._add_conv(self.stem)
        self._add_bn("bn1", width)
        self.blocks = []
        inplanes = width
        for i, depth in enumerate(self.depths):
            planes = width * (2 ** i)
            for b in range(depth):
                s = (1 if i == 0 else 2) if b == 0 else 1
                blk = _Block()
                pre = f"layer{i + 1}.{b}"
                blk.c1 = _Conv(pre + ".conv1", inplanes, planes, 1, 1, 0)
                blk.c2 = _Conv(pre + ".conv2", planes, planes, 3, s, 1)
                blk.c3 = _Conv(pre + ".conv3", planes, planes * 4, 1, 1, 0)
                for j, c in enumerate((blk.c1, blk.c2, blk.c3)):
                    self._add_conv(c)
                    self._add_bn(f"{pre}.bn{j + 1}", c.cout)
                blk.cd = None
                if b == 0 and (s != 1 or inplanes != planes * 4):
                    blk.cd = _Conv(pre + ".downsample.0", inplanes, planes * 4, 1, s, 0)
                    self._add_conv(blk.cd)
                    self._add_bn(pre + ".downsample.1", planes * 4)
                blk.stride, blk.cin, blk.planes, blk.prefix = s, inplanes, planes, pre
                self.blocks.append(blk)
                inplanes = planes * 4
        self.feat = inplanes
        self._add_param("fc.weight", "fc_w", (num_classes, inplanes), (num_classes, 1, 1, inplanes))
        self._add_param("fc.bias", "fc_b", (num_classes,), (num_classes,))
        self.n_store = self._off
        self.spec = {p.name: p for p in self._specs}

        def zeros(n, dt=torch.float32):
            return self._alloc((n,), dt).zero_()
        self.params = zeros(self.n_store)
        self.grads = zeros(self.n_store)
        self.momentum_buf = zeros(self.n_store)
        self.global_grads = None
        self.shadow = zeros(self.n_store, torch.bfloat16) if dtype == torch.bfloat16 else None
        # filters transposed to [C,R,S,K] for the data-gradient GEMM, same offsets, rewritten
        # in one launch whenever the weights change
        self.wt = zeros(self.n_store, dtype)
        self._tt = ops.FilterTransposeTable(
            [(p.offset, p.store_shape[0], p.store_shape[1] * p.store_shape[2], p.store_shape[3])
             for p in self._specs if p.kind in ("conv", "fc_w")], self.dev)
        nbn = sum(c for _, c in self._bn_names)
        self.running_mean = zeros(nbn)
        self.running_var = zeros(nbn).fill_(1.0)
        self._bn_off, o = {}, 0
        for name, c in self._bn_names:
            self._bn_off[name] = (o, c)
            o += c

    # ------------------------------------------------------------------ parameter table
    def _add_param(self, name, kind, shape, store_shape):
        p = _Param(name, kind, shape, store_shape, self._off)
        self._specs.append(p)
        self._off += (p.numel + 3) // 4 * 4
        return p

    def _add_conv(self, c):
        self._add_param(c.name + ".weight", "conv", (c.cout, c.cin, c.k, c.k), (c.cout, c.k, c.k, c.cin_store))

    def _add_bn(self, name, c):
        self._add_param(name + ".weight", "bn_w", (c,), (c,))
        self._add_param(name + ".bias", "bn_b", (c,), (c,))
        self._bn_names.append((name, c))

    def num_parameters(self):
        return sum(int(math.prod(p.shape)) for p in self._specs)

    def _view(self, flat, name):
        p = self.spec[name]
        return flat[p.offset:p.offset + p.numel].view(p.store_shape)

    def _w(self, name):
        """The tensor the kernels read for a filter: bf16 shadow or the fp32 master."""
        return self._view(self.shadow if self.shadow is not None else self.params, name)

    def _to_store(self, p, t):
        t = t.detach().to(torch.float32)
        if p.kind == "conv":
            t = t.permute(0, 2, 3, 1)  # OIHW -> KRSC
            if p.store_shape[3] != t.shape[3]:
                t = torch.nn.functional.pad(t, (0, p.store_shape[3] - t.shape[3]))
        return t.reshape(p.store_shape).contiguous()

    def _from_store(self, p, flat):
        t = flat[p.offset:p.offset + p.numel].view(p.store_shape)
        if p.kind == "conv":
            t = t[..., :p.shape[1]].permute(0, 3, 1, 2)  # KRSC -> OIHW, padding stripped
        return t.reshape(p.shape).contiguous().cpu()

    def load_state_dict(self, sd):
        """Take weights and BN statistics from a torchvision-style state dict (CPU, OIHW)."""
        host = torch.zeros(self.n_store, dtype=torch.float32)
        for p in self._specs:
            host[p.offset:p.offset + p.numel] = self._to_store(p, sd[p.name]).reshape(-1)
        self.params.copy_(host)
        for name, (o, c) in self._bn_off.items():
            self.running_mean[o:o + c].copy_(sd[name + ".running_mean"])
            self.running_var[o:o + c].copy_(sd[name + ".running_var"])
        self.momentum_buf.zero_()
        self.grads.zero_()
        self.refresh_shadow()
        torch.cuda.synchronize()

    def init_kaiming(self, seed=0):
        """Random initial weights generated on the GPU: convolutions N(0, 2/fan_out) (Kaiming
        normal, fan_out, relu), BatchNorm gamma 1 / beta 0, fc U(-1/sqrt(fan_in), 1/sqrt(fan_in)).
        Same distribution as the oracle's init, different stream of random numbers."""
        g = torch.Generator(device=self.dev)
        g.manual_seed(seed)
        for p in self._specs:
            v = self._view(self.params, p.name)
            if p.kind == "conv":
                K, R, S, C = p.store_shape
                v.normal_(0.0, math.sqrt(2.0 / (K * R * S)), generator=g)
                if p.shape[1] != C:
                    v[..., p.shape[1]:] = 0
            elif p.kind == "bn_w":
                v.fill_(1.0)
            elif p.kind == "bn_b":
                v.zero_()
            else:
                bound = 1.0 / math.sqrt(self.feat)
                v.uniform_(-bound, bound, generator=g)
        self.running_mean.zero_()
        self.running_var.fill_(1.0)
        self.momentum_buf.zero_()
        self.grads.zero_()
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

    def _wt(self, name):
        p = self.spec[name]
        K, R, S, C = p.store_shape
        return self.wt[p.offset:p.offset + p.numel].view(C, R, S, K)

    def state_dict(self):
        torch.cuda.synchronize()
        sd = {p.name: self._from_store(p, self.params) for p in self._specs}
        for name, (o, c) in self._bn_off.items():
            sd[name + ".running_mean"] = self.running_mean[o:o + c].cpu()
            sd[name + ".running_var"] = self.running_var[o:o + c].cpu()
        return sd

    def grads_dict(self, use_global=False):
        torch.cuda.synchronize()
        flat = self.global_grads if use_global else self.grads
        return {p.name: self._from_store(p, flat) for p in self._specs}

    # ------------------------------------------------------------------ tiling choice
    def _pick_tiling(self, timings):
        """The fastest tiling, or a larger tile that is within `tile_margin` of it: alone on the chip a small tile
        can win by a few percent and still lose in the step, where it shares L2 bandwidth with the weight gradients
        (a larger tile fetches fewer operand bytes per flop)."""
        area = lambda cfg: {0: 4, 11: 4, 12: 4, 9: 16, 10: 16, 1: 2, 5: 2, 6: 2, 13: 2}.get(cfg, 1)
        best = min(timings.values())
        ok = [cfg for cfg, t in timings.items() if t <= best * (1.0 + self.tile_margin)]
        return min(ok, key=lambda cfg: (-area(cfg), timings[cfg]))

    def _tune_conv(self, c, n, h, w):
        """(forward tiling, data-gradient tiling) for one convolution at one input shape."""
        key = (c.cin_store, c.cout, c.k, c.stride, c.pad, n, h, w)
        hit = self._tile_cache.get(key)
        if hit is not None:
            return hit
        T, ctx = self.dtype, self.ctx
        ho, wo = ops.conv_out_hw(h, w, c.k, c.k, c.stride, c.pad)
        # scratch operands from the engine's allocator (the shared pool when there is one), dropped on return
        x = self._scratch((n, h, w, c.cin_store), T)
        z = self._scratch((n, ho, wo, c.cout), T)
        wgt, wt = self._w(c.name + ".weight"), self._wt(c.name + ".weight")
        part = self._scratch((ops.conv2d_fwd_stat_rows(x, c.cout, c.k, c.k, c.stride, c.pad, 2) * c.cout * 2,),
                             torch.float32)
        reps = 4

        def fwd(cfg):
            def rec():
                for _ in range(reps):
                    ops.conv2d_fwd_bnstats(ctx, x, wgt, z, c.stride, c.pad, part, tile_cfg=cfg, c_logical=c.cin)
            return rec

        mean = self._scratch((c.cin_store,), torch.float32)
        invstd = self._scratch((c.cin_store,), torch.float32, 1.0)
        x2 = self._scratch(tuple(x.shape), T, 1.0)
        dpart = self._scratch((ops.conv2d_dgrad_stat_rows(x, c.cout, c.k, c.k, c.stride, c.pad, 2) * c.cin_store * 2,),
                              torch.float32)
        torch.cuda.synchronize()

        def dgrad(cfg):
            def rec():
                for _ in range(reps):
                    if self.fuse_bn_bwd:   # nearly every data gradient of the plan runs in this form
                        ops.conv2d_dgrad_bnsums(ctx, z, wt, x, c.stride, c.pad, x2, mean, invstd, dpart, bn_mask=x2,
                                                tile_cfg=cfg, c_logical=c.cin)
                    else:
                        ops.conv2d_dgrad(ctx, z, wt, x, c.stride, c.pad, tile_cfg=cfg, c_logical=c.cin)
            return rec
        # 5 = the 3x3 patch kernel (stride-1 3x3 layers; elsewhere the library runs tiling 1 for it)
        patch = (5,) if (c.k == 3 and c.stride == 1 and c.pad == 1) else ()
        # 6 / 7 = tilings 1 / 2 with two LDS tiles in flight (more workgroups per CU)
        # 11 - 14 = 128 x 128 (three / two LDS tiles), 128 x 64, 64 x 64 with 32-element reduction steps: half the LDS
        # per workgroup, which the wide, shallow products of the first two stages prefer
        cfgs = ((0, 1, 2, 3, 6, 7, 11, 12, 13, 14) if c.cout > 64 else (1, 2, 3, 6, 7, 13, 14)) + patch
        t_f = {cfg: self._time_program(fwd(cfg)) / reps for cfg in cfgs}
        tf = self._pick_tiling(t_f)
        cfgs_d = ((0, 1, 2, 3, 6, 7, 11, 12, 13, 14) if c.cin_store > 64 else (1, 2, 3, 6, 7, 13, 14)) + patch
        t_d = {cfg: self._time_program(dgrad(cfg)) / reps for cfg in cfgs_d} if c.cin_store >= 64 else {-1: 0.0}
        td = self._pick_tiling(t_d)
        self._tile_cache[key] = (tf, td)
        self.tile_timings[key] = {"fwd_ms": t_f, "dgrad_ms": t_d}
        return tf, td

    # ------------------------------------------------------------------ the plan for one batch size
    def _build_plan(self, B, loss_scale):
        T, dev, ctx = self.dtype, self.dev, self.ctx
        S = self.image_size
        plan = _Block()
        plan.batch, plan.loss_scale = B, loss_scale
        keep = []

        def act(*shape, dtype=T):
            t = self._alloc(tuple(shape), dtype)
            keep.append(t)
            return t

        # gradient buffers are recycled through a size-keyed free list: the program is
        # one in-order stream of launches, so program order is the only hazard
        free = {}

        def galloc(shape):
            n = int(math.prod(shape))
            lst = free.get(n)
            if lst:
                return lst.pop().view(shape)
            t = self._alloc((n,), T)
            keep.append(t)
            return t.view(shape)

        def gfree(t, read_by_wgrad=False):
            # a buffer the side lane still reads must not be handed out again before the join
            if (read_by_wgrad and (self.overlap_wgrad or self.group_wgrad)) or self.retain_gradients:
                return
            free.setdefault(t.numel(), []).append(t.reshape(-1))

        code = ops.dtype_code(torch.empty(0, dtype=T))
        plan.x_in = act(B, 3, S, S, dtype=torch.float32)
        plan.labels = act(B, dtype=torch.int64).zero_()
        plan.loss_rows = act(B, dtype=torch.float32)
        plan.loss = act(1, dtype=torch.float32)
        bn_save = act(2 * self.running_mean.numel(), dtype=torch.float32)
        nbn = self.running_mean.numel()

        # workspaces sized over every layer of the plan
        bn_ws_bytes, wg_ws_bytes = [0], [4]
        geo = []  # (conv, x_shape) for the workspace pass

        def conv_shape(c, H, W):
            Ho, Wo = ops.conv_out_hw(H, W, c.k, c.k, c.stride, c.pad)
            return Ho, Wo

        # ---- shapes ----
        H0, W0 = conv_shape(self.stem, S, S)
        Hp, Wp = ops.conv_out_hw(H0, W0, 3, 3, 2, 1)
        shapes = []
        H, W = Hp, Wp
        for blk in self.blocks:
            Ho, Wo = conv_shape(blk.c2, H, W)
            shapes.append((H, W, Ho, Wo))
            H, W = Ho, Wo
        Hl, Wl = H, W

        def wg_need(c, N, H, W):
            x_like = torch.empty((N, H, W, c.cin_store), dtype=T, device="meta")
            sp = int(ops.lib().tch_conv2d_wgrad_pick_splits(code, N, H, W, c.cin_store, c.cout, c.k, c.k, c.stride, c.pad))
            wg_ws_bytes[0] = max(wg_ws_bytes[0], ops.conv2d_wgrad_workspace_bytes(code, c.cout, c.k, c.k, c.cin_store, sp))
            del x_like

        def bn_need(rows, C):
            bn_ws_bytes[0] = max(bn_ws_bytes[0], ops.bn_workspace_bytes(code, rows, C))

        conv_inputs = [(self.stem, (B, S, S))]
        wg_need(self.stem, B, S, S)
        bn_need(B * H0 * W0, self.width)
        for blk, (H, W, Ho, Wo) in zip(self.blocks, shapes):
            conv_inputs += [(blk.c1, (B, H, W)), (blk.c2, (B, H, W)), (blk.c3, (B, Ho, Wo))]
            if blk.cd is not None:
                conv_inputs.append((blk.cd, (B, H, W)))
            wg_need(blk.c1, B, H, W)
            wg_need(blk.c2, B, H, W)
            wg_need(blk.c3, B, Ho, Wo)
            bn_need(B * H * W, blk.planes)
            bn_need(B * Ho * Wo, blk.planes * 4)
            if blk.cd is not None:
                wg_need(blk.cd, B, H, W)
        fc = _Conv("fc", self.feat, self.num_classes, 1, 1, 0)
        wg_need(fc, B, 1, 1)
        bn_ws = act(bn_ws_bytes[0] // 4, dtype=torch.float32)
        wg_half = (wg_ws_bytes[0] // 4 + 63) // 64 * 64
        wg_ws = act(2 * wg_half, dtype=torch.float32)
        trail = ops.TrailingWgrad(ctx, wg_ws, wg_half) if self.trailing_reduce else None

        def bn_fwd(name, x, y, residual=None, relu=True):
            o, c = self._bn_off[name]
            ops.bn_fwd_train(ctx, x, y, self._view(self.params, name + ".weight"), self._view(self.params, name + ".bias"),
                             self.running_mean[o:o + c], self.running_var[o:o + c], bn_save[o:o + c],
                             bn_save[nbn + o:nbn + o + c], bn_ws, residual=residual, relu=relu,
                             momentum=self.bn_momentum, eps=self.bn_eps)

        def bn_bwd(name, dy, x, dx, mask):
            o, c = self._bn_off[name]
            ops.bn_bwd(ctx, dy, x, dx, self._view(self.params, name + ".weight"), bn_save[o:o + c],
                       bn_save[nbn + o:nbn + o + c], self._view(self.grads, name + ".weight"),
                       self._view(self.grads, name + ".bias"), bn_ws, relu_mask=mask)

        def conv_fwd(c, x, y, **kw):
            ops.conv2d_fwd(ctx, x, self._w(c.name + ".weight"), y, c.stride, c.pad, c_logical=c.cin, **kw)

        # convolution -> BatchNorm pairs: the convolution's epilogue leaves the per-tile batch sums,
        # the BatchNorm starts at its finalize (no statistics pass over the convolution's output)
        stat_elems = [0]
        tiles = {}
        for c_, (n_, h_, w_) in conv_inputs:
            xm = torch.empty((n_, h_, w_, c_.cin_store), dtype=T, device="meta")
            # sized for the smallest row tile, whichever tiling is picked
            stat_elems[0] = max(stat_elems[0],
                                ops.conv2d_fwd_stat_rows(xm, c_.cout, c_.k, c_.k, c_.stride, c_.pad, 2) * c_.cout * 2,
                                ops.conv2d_dgrad_stat_rows(xm, c_.cout, c_.k, c_.k, c_.stride, c_.pad, 2) * c_.cin_store * 2)
            tiles[c_.name] = self._tune_conv(c_, n_, h_, w_) if self.autotune else (-1, -1)
        stat_partial = act(max(stat_elems[0], 2), dtype=torch.float32)
        bn_scratch = act(3 * max(max(c_.cout, c_.cin_store) for c_, _ in conv_inputs), dtype=torch.float32)
        bn_counters = act(max(max(c_.cout, c_.cin_store) for c_, _ in conv_inputs) // 64 + 1, dtype=torch.int32).zero_()

        # exact accumulators: [forward | backward][BatchNorm channel][2 sums][2 words]
        use_acc = self.bn_acc and self.fuse_bn_stats and not self.fuse_bn_finalize
        copies = self.bn_acc_copies
        acc_all = act(2 * nbn * 4 * copies, dtype=torch.int64) if use_acc else None
        plan.bn_acc = acc_all

        def acc_of(name, backward, rows):
            """The accumulators of one BatchNorm ([copies, 4, channels]), or None where the layer keeps the per-tile form."""
            o, ch = self._bn_off[name]
            if not use_acc or ch % 64 or (self.bn_acc_max_rows and rows > self.bn_acc_max_rows):
                return None
            base = ((nbn if backward else 0) + o) * 4 * copies
            return acc_all[base:base + 4 * copies * ch]

        def conv_bn_fwd(c, name, x, z, y, residual=None, relu=True):
            if not self.fuse_bn_stats:
                conv_fwd(c, x, z)
                return bn_fwd(name, z, y, residual=residual, relu=relu)
            o, ch = self._bn_off[name]
            acc = acc_of(name, False, z.numel() // ch)
            if acc is not None:
                ops.conv2d_fwd_bnacc(ctx, x, self._w(c.name + ".weight"), z, c.stride, c.pad, acc,
                                     tile_cfg=tiles[c.name][0], c_logical=c.cin)
                return ops.bn_fwd_train_acc(ctx, z, y, self._view(self.params, name + ".weight"),
                                            self._view(self.params, name + ".bias"), self.running_mean[o:o + ch],
                                            self.running_var[o:o + ch], bn_save[o:o + ch], bn_save[nbn + o:nbn + o + ch],
                                            acc, residual=residual, relu=relu, momentum=self.bn_momentum, eps=self.bn_eps)
            if self.fuse_bn_finalize:
                ops.conv2d_fwd_bn(ctx, x, self._w(c.name + ".weight"), z, c.stride, c.pad, stat_partial, bn_counters,
                                  self._view(self.params, name + ".weight"), self._view(self.params, name + ".bias"),
                                  self.running_mean[o:o + ch], self.running_var[o:o + ch], bn_save[o:o + ch],
                                  bn_save[nbn + o:nbn + o + ch], bn_scratch, momentum=self.bn_momentum, eps=self.bn_eps,
                                  tile_cfg=tiles[c.name][0], c_logical=c.cin)
                return ops.bn_apply_fwd(ctx, z, y, bn_scratch, residual=residual, relu=relu)
            rb = ops.conv2d_fwd_bnstats(ctx, x, self._w(c.name + ".weight"), z, c.stride, c.pad, stat_partial,
                                        tile_cfg=tiles[c.name][0], c_logical=c.cin)
            ops.bn_fwd_train_partials(ctx, z, y, self._view(self.params, name + ".weight"),
                                      self._view(self.params, name + ".bias"), self.running_mean[o:o + ch],
                                      self.running_var[o:o + ch], bn_save[o:o + ch], bn_save[nbn + o:nbn + o + ch],
                                      stat_partial, rb, bn_scratch, residual=residual, relu=relu,
                                      momentum=self.bn_momentum, eps=self.bn_eps)

        pending = []   # (convolution, its input, the gradient of its output): weight gradients not launched yet

        def flush_wgrads():
            if not pending:
                return
            items = [(x_, dy_, self._view(self.grads, c_.name + ".weight"), c_.stride, c_.pad) for c_, x_, dy_ in pending]
            splits, tile, table_bytes, ws_bytes = ops.conv2d_wgrad_group_plan(items, self.wgrad_group_wgs)
            table = act(table_bytes, dtype=torch.uint8)
            ws = act(max(ws_bytes // 4, 1), dtype=torch.float32)
            with ctx.side_lane(wait_main=True):
                ops.conv2d_wgrad_group(ctx, items, splits, tile, ws, table, max_wgs=self.wgrad_group_max_wgs)
            plan.wgrad_groups.append(dict(layers=[c_.name for c_, _, _ in pending], splits=splits, tile=tile,
                                          workspace_bytes=ws_bytes))
            pending.clear()

        plan.wgrad_groups = []

        def conv_wgrad(c, x, dy, grouped=False):
            if grouped and self.group_wgrad:
                pending.append((c, x, dy))
                return
            def one():
                if trail is not None:
                    return trail.wgrad(x, dy, self._view(self.grads, c.name + ".weight"), c.stride, c.pad, c_logical=c.cin)
                ops.conv2d_wgrad(ctx, x, dy, self._view(self.grads, c.name + ".weight"), c.stride, c.pad,
                                 workspace=wg_ws, c_logical=c.cin)
            if self.overlap_wgrad:
                with ctx.side_lane(wait_main=True):
                    one()
            else:
                one()

        def conv_dgrad(c, dy, dx, **kw):
            ops.conv2d_dgrad(ctx, dy, self._wt(c.name + ".weight"), dx, c.stride, c.pad, c_logical=c.cin,
                             tile_cfg=tiles.get(c.name, (-1, -1))[1], **kw)

        # data gradient -> BatchNorm backward pairs: conv_dgrad_bn leaves dx gated by the ReLU of the
        # BatchNorm `name` (output `relu_out`, input `z`) together with its two reductions; bn_bwd_sums
        # is that BatchNorm's backward from there (finalize + apply)
        def conv_dgrad_bn(c, dy, dx, name, z, relu_out, **kw):
            o, ch = self._bn_off[name]
            acc = acc_of(name, True, z.numel() // ch)
            if acc is not None:
                ops.conv2d_dgrad_bnacc(ctx, dy, self._wt(c.name + ".weight"), dx, c.stride, c.pad, z, bn_save[o:o + ch],
                                       bn_save[nbn + o:nbn + o + ch], acc, bn_mask=relu_out, c_logical=c.cin,
                                       tile_cfg=tiles.get(c.name, (-1, -1))[1], **kw)
                return -2   # the sums are in the accumulators
            if self.fuse_bn_finalize:
                ops.conv2d_dgrad_bn(ctx, dy, self._wt(c.name + ".weight"), dx, c.stride, c.pad, z, bn_save[o:o + ch],
                                    bn_save[nbn + o:nbn + o + ch], stat_partial, bn_counters,
                                    self._view(self.params, name + ".weight"), self._view(self.grads, name + ".weight"),
                                    self._view(self.grads, name + ".bias"), bn_scratch, bn_mask=relu_out,
                                    c_logical=c.cin, tile_cfg=tiles.get(c.name, (-1, -1))[1], **kw)
                return -1   # the coefficients are in bn_scratch already
            return ops.conv2d_dgrad_bnsums(ctx, dy, self._wt(c.name + ".weight"), dx, c.stride, c.pad, z,
                                           bn_save[o:o + ch], bn_save[nbn + o:nbn + o + ch], stat_partial,
                                           bn_mask=relu_out, c_logical=c.cin,
                                           tile_cfg=tiles.get(c.name, (-1, -1))[1], **kw)

        def bn_bwd_sums(name, g, x, dx, rb):
            if rb == -1:
                return ops.bn_apply_bwd(ctx, g, x, dx, bn_scratch)
            o, c = self._bn_off[name]
            if rb == -2:
                return ops.bn_bwd_acc(ctx, g, x, dx, self._view(self.params, name + ".weight"), bn_save[o:o + c],
                                      bn_save[nbn + o:nbn + o + c], self._view(self.grads, name + ".weight"),
                                      self._view(self.grads, name + ".bias"), acc_of(name, True, x.numel() // c))
            ops.bn_bwd_partials(ctx, g, x, dx, self._view(self.params, name + ".weight"), bn_save[o:o + c],
                                bn_save[nbn + o:nbn + o + c], self._view(self.grads, name + ".weight"),
                                self._view(self.grads, name + ".bias"), stat_partial, rb, bn_scratch)

        prog = ops.Program()
        marks = []  # (launch index one past the layer, 'fwd' | 'bwd', layer name): checkpoint positions
        named = {}  # retain_gradients: every intermediate tensor of the step by name

        def mark(phase, name):
            marks.append((len(prog), phase, name))

        ctx.begin_record(prog)
        try:
            # ================= forward =================
            if acc_all is not None:
                ops.fill_zero(ctx, acc_all)
            x0 = act(B, S, S, STEM_CIN_PAD)
            ops.nchw_to_nhwc_pad(ctx, plan.x_in, x0)
            z0, a0 = act(B, H0, W0, self.width), act(B, H0, W0, self.width)
            conv_bn_fwd(self.stem, "bn1", x0, z0, a0)
            mark("fwd", "bn1")
            p0 = act(B, Hp, Wp, self.width)
            p0_idx = act(B, Hp, Wp, self.width, dtype=torch.int32)
            ops.maxpool_fwd(ctx, a0, p0, p0_idx, 3, 2, 1)
            x = p0
            saved = []
            for blk, (H, W, Ho, Wo) in zip(self.blocks, shapes):
                P, pre = blk.planes, blk.prefix
                z1, a1 = act(B, H, W, P), act(B, H, W, P)
                conv_bn_fwd(blk.c1, pre + ".bn1", x, z1, a1)
                mark("fwd", pre + ".bn1")
                z2, a2 = act(B, Ho, Wo, P), act(B, Ho, Wo, P)
                conv_bn_fwd(blk.c2, pre + ".bn2", a1, z2, a2)
                mark("fwd", pre + ".bn2")
                z3, out = act(B, Ho, Wo, 4 * P), act(B, Ho, Wo, 4 * P)
                zd = None
                if blk.cd is not None:
                    zd, idn = act(B, Ho, Wo, 4 * P), act(B, Ho, Wo, 4 * P)
                    conv_bn_fwd(blk.cd, pre + ".downsample.1", x, zd, idn, relu=False)
                else:
                    idn = x
                conv_bn_fwd(blk.c3, pre + ".bn3", a2, z3, out, residual=idn, relu=True)
                mark("fwd", pre + ".bn3")
                saved.append((x, z1, a1, z2, a2, z3, zd, out))
                named[pre] = dict(x=x, z1=z1, a1=a1, z2=z2, a2=a2, z3=z3, zd=zd, idn=idn, out=out)
                x = out
            pooled = act(B, self.feat)
            ops.avgpool_fwd(ctx, x, pooled)
            logits = act(B, self.num_classes, dtype=torch.float32)
            ops.conv2d_fwd(ctx, pooled.view(B, 1, 1, self.feat), self._w("fc.weight"),
                           logits.view(B, 1, 1, self.num_classes), 1, 0, bias=self._view(self.params, "fc.bias"))
            dlogits = act(B, self.num_classes)
            ops.softmax_ce_fwd_bwd(ctx, logits, plan.labels, plan.loss_rows, plan.loss, dlogits, loss_scale=loss_scale)
            plan.n_forward = len(prog)
            mark("fwd", "loss")

            # ================= backward =================
            if self.overlap_wgrad:
                ctx.join()      # the second lane may still be writing the transposed filters of the last optimizer step
            fc_conv = _Conv("fc", self.feat, self.num_classes, 1, 1, 0)
            conv_wgrad(fc_conv, pooled.view(B, 1, 1, self.feat), dlogits.view(B, 1, 1, self.num_classes))
            ops.bias_grad(ctx, dlogits, self._view(self.grads, "fc.bias"))
            g_pooled = galloc((B, self.feat))
            ops.conv2d_dgrad(ctx, dlogits.view(B, 1, 1, self.num_classes), self._wt("fc.weight"),
                             g_pooled.view(B, 1, 1, self.feat), 1, 0)
            g_out = galloc((B, Hl, Wl, self.feat))
            ops.avgpool_bwd(ctx, g_pooled, g_out)
            named["head"] = dict(x0=x0, z0=z0, a0=a0, p0=p0, p0_idx=p0_idx, pooled=pooled, logits=logits,
                                 dlogits=dlogits, g_pooled=g_pooled, g_feat=g_out)
            gfree(g_pooled)
            # g_rb: g_out is already gated by the block's final ReLU and stat_partial holds g_rb row tiles of
            # the sums of this block's bn3 (left by the c1 data gradient of the block after it); None = neither
            g_rb = None
            fuse = self.fuse_bn_bwd
            since_flush = 0
            for bi in range(len(self.blocks) - 1, -1, -1):
                blk, (H, W, Ho, Wo), sv = self.blocks[bi], shapes[bi], saved[bi]
                xin, z1, a1, z2, a2, z3, zd, out = sv
                P, pre = blk.planes, blk.prefix
                dz3 = galloc(z3.shape)
                if g_rb is None:
                    bn_bwd(pre + ".bn3", g_out, z3, dz3, out)
                else:
                    bn_bwd_sums(pre + ".bn3", g_out, z3, dz3, g_rb)
                out_gate = out if g_rb is None else None   # what still has to gate g_out
                conv_wgrad(blk.c3, a2, dz3, grouped=True)
                g_a2 = galloc(a2.shape)
                dz2 = galloc(z2.shape)
                if fuse:
                    rb = conv_dgrad_bn(blk.c3, dz3, g_a2, pre + ".bn2", z2, a2)
                    mark("bwd", pre + ".conv3")
                    bn_bwd_sums(pre + ".bn2", g_a2, z2, dz2, rb)
                else:
                    conv_dgrad(blk.c3, dz3, g_a2)
                    mark("bwd", pre + ".conv3")
                    bn_bwd(pre + ".bn2", g_a2, z2, dz2, a2)
                gfree(dz3, True)
                gfree(g_a2)
                conv_wgrad(blk.c2, a1, dz2, grouped=True)
                g_a1 = galloc(a1.shape)
                dz1 = galloc(z1.shape)
                if fuse:
                    rb = conv_dgrad_bn(blk.c2, dz2, g_a1, pre + ".bn1", z1, a1)
                    mark("bwd", pre + ".conv2")
                    bn_bwd_sums(pre + ".bn1", g_a1, z1, dz1, rb)
                else:
                    conv_dgrad(blk.c2, dz2, g_a1)
                    mark("bwd", pre + ".conv2")
                    bn_bwd(pre + ".bn1", g_a1, z1, dz1, a1)
                gfree(dz2, True)
                gfree(g_a1)
                conv_wgrad(blk.c1, xin, dz1, grouped=True)
                gx = galloc(xin.shape)
                # xin is the output of the block before (its bn3 + residual + ReLU), whose bn3 input is z3 there
                prev = (self.blocks[bi - 1].prefix + ".bn3", saved[bi - 1][5]) if (fuse and bi > 0) else None
                if blk.cd is not None:
                    dzd = galloc(zd.shape)
                    bn_bwd(pre + ".downsample.1", g_out, zd, dzd, out_gate)
                    conv_wgrad(blk.cd, xin, dzd, grouped=True)
                    if blk.cd.stride == 2 and self.compact_downsample_dgrad:
                        # a stride-2 1x1 convolution sends gradient to the even pixels of its input only: computed
                        # as the stride-1 data gradient on dzd's own grid and added from there
                        gx_id = galloc((B, Ho, Wo, xin.shape[3]))
                        ops.conv2d_dgrad(ctx, dzd, self._wt(blk.cd.name + ".weight"), gx_id, 1, 0)
                        add_kw = dict(add=gx_id, add_stride=2)
                    else:
                        gx_id = galloc(xin.shape)
                        conv_dgrad(blk.cd, dzd, gx_id)
                        add_kw = dict(add=gx_id)
                    gfree(dzd, True)
                else:
                    gx_id = None
                    add_kw = dict(add=g_out, mask=out_gate)
                if prev is not None:
                    g_rb = conv_dgrad_bn(blk.c1, dz1, gx, prev[0], prev[1], xin, **add_kw)
                else:
                    conv_dgrad(blk.c1, dz1, gx, **add_kw)
                    g_rb = None
                if gx_id is not None:
                    gfree(gx_id)
                mark("bwd", pre + ".conv1")
                # g_out_gated: g_out arrived with this block's final ReLU applied (by the data gradient that wrote it);
                # gx_gated: gx leaves with the ReLU of the block before applied
                named[pre].update(g_out=g_out, g_out_gated=out_gate is None, dz3=dz3, g_a2=g_a2, dz2=dz2, g_a1=g_a1,
                                  dz1=dz1, gx=gx, gx_gated=prev is not None, dzd=dzd if blk.cd is not None else None,
                                  gx_id=gx_id)
                gfree(dz1, True)
                gfree(g_out)
                g_out = gx
                since_flush += 1
                if blk.cd is not None or (self.wgrad_group_blocks and since_flush >= self.wgrad_group_blocks):
                    flush_wgrads()      # the stage ends here (its first block is the last one of the backward)
                    since_flush = 0
            flush_wgrads()
            g_a0 = galloc(a0.shape)
            ops.maxpool_bwd(ctx, g_out, p0_idx, g_a0, 3, 2, 1)
            gfree(g_out)
            dz0 = galloc(z0.shape)
            bn_bwd("bn1", g_a0, z0, dz0, a0)
            gfree(g_a0)
            conv_wgrad(self.stem, x0, dz0)
            if trail is not None:      # the stem's own reduction: nothing behind it to ride on
                if self.overlap_wgrad:
                    with ctx.side_lane(wait_main=False):
                        trail.flush()
                else:
                    trail.flush()
            named["head"].update(g_p0=g_out, g_a0=g_a0, dz0=dz0)
            gfree(dz0, True)
            ctx.join()
        finally:
            ctx.end_record()
        plan.prog = prog
        plan.marks = marks
        plan.keep = keep
        plan.logits = logits
        plan.tensors = named if self.retain_gradients else None
        plan.tiles = tiles
        plan.bn_save = bn_save   # [2][sum of BatchNorm widths]: saved batch mean, then inverse std
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

    def forward_backward_resident(self, batch, loss_scale=1.0):
        """Replay on whatever already sits in the plan's input buffers."""
        p = self.plan(batch, loss_scale)
        return p, self._run_plan(p)

    # ------------------------------------------------------------------ inference (model.eval())
    def prepare_eval(self):
        """Turn every BatchNorm into one scale and one shift per channel from its running statistics (what
        model.eval() makes of it).  Run again whenever weights or statistics changed."""
        if getattr(self, "_eval_coef", None) is None:
            self._eval_coef = self._alloc((2 * self.running_mean.numel(),), torch.float32)
        nbn = self.running_mean.numel()
        for name, (o, c) in self._bn_off.items():
            # (scale, shift) of a BatchNorm sit next to each other: coef[2o : 2o + 2c]
            ops.bn_eval_coef(self.ctx, self._view(self.params, name + ".weight"), self._view(self.params, name + ".bias"),
                             self.running_mean[o:o + c], self.running_var[o:o + c], self._eval_coef[2 * o:2 * o + 2 * c],
                             eps=self.bn_eps)
        assert 2 * nbn == self._eval_coef.numel()

    def _build_eval_plan(self, B):
        """Forward only, BatchNorm from the running statistics, nothing kept for a backward: the program of
        one inference request (the batch-1 ResNet-152 requests that share the GPU with training)."""
        T, ctx, S = self.dtype, self.ctx, self.image_size
        plan = _Block()
        keep = []

        def act(*shape, dtype=T):
            t = self._alloc(tuple(shape), dtype)
            keep.append(t)
            return t

        def conv_bn(c, name, x, residual=None, relu=True):
            Ho, Wo = ops.conv_out_hw(x.shape[1], x.shape[2], c.k, c.k, c.stride, c.pad)
            y = act(B, Ho, Wo, c.cout)
            o, ch = self._bn_off[name]
            coef = self._eval_coef[2 * o:2 * o + 2 * ch]
            if self.fuse_eval_bn:
                # the BatchNorm is a per-channel scale and shift here: applied to the accumulators in the epilogue
                ops.conv2d_fwd_affine(ctx, x, self._w(c.name + ".weight"), y, c.stride, c.pad, scale=coef[:ch], shift=coef[ch:],
                                      residual=residual, relu=relu, c_logical=c.cin)
                return y
            z = act(B, Ho, Wo, c.cout)
            ops.conv2d_fwd(ctx, x, self._w(c.name + ".weight"), z, c.stride, c.pad, c_logical=c.cin)
            ops.bn_apply_fwd(ctx, z, y, coef, residual=residual, relu=relu)
            return y

        plan.x_in = act(B, 3, S, S, dtype=torch.float32)
        prog = ops.Program()
        ctx.begin_record(prog)
        try:
            x0 = act(B, S, S, STEM_CIN_PAD)
            ops.nchw_to_nhwc_pad(ctx, plan.x_in, x0)
            a0 = conv_bn(self.stem, "bn1", x0)
            Hp, Wp = ops.conv_out_hw(a0.shape[1], a0.shape[2], 3, 3, 2, 1)
            x = act(B, Hp, Wp, self.width)
            idx = act(B, Hp, Wp, self.width, dtype=torch.int32)
            ops.maxpool_fwd(ctx, a0, x, idx, 3, 2, 1)
            for blk in self.blocks:
                pre = blk.prefix
                a1 = conv_bn(blk.c1, pre + ".bn1", x)
                a2 = conv_bn(blk.c2, pre + ".bn2", a1)
                idn = conv_bn(blk.cd, pre + ".downsample.1", x, relu=False) if blk.cd is not None else x
                x = conv_bn(blk.c3, pre + ".bn3", a2, residual=idn, relu=True)
            pooled = act(B, self.feat)
            ops.avgpool_fwd(ctx, x, pooled)
            plan.logits = act(B, self.num_classes, dtype=torch.float32)
            ops.conv2d_fwd(ctx, pooled.view(B, 1, 1, self.feat), self._w("fc.weight"),
                           plan.logits.view(B, 1, 1, self.num_classes), 1, 0, bias=self._view(self.params, "fc.bias"))
        finally:
            ctx.end_record()
        plan.prog, plan.keep, plan.batch = prog, keep, B
        plan.bytes = sum(t.numel() * t.element_size() for t in keep)
        return plan

    def eval_plan(self, batch):
        plans = self.__dict__.setdefault("_eval_plans", {})
        if batch not in plans:
            if getattr(self, "_eval_coef", None) is None:
                self.prepare_eval()
            plans[batch] = self._build_eval_plan(batch)
        return plans[batch]

    def forward_eval(self, x):
        """x [B,3,S,S] fp32 on the GPU -> the plan whose `logits` [B, classes] (fp32) the launches fill.  The
        caller synchronises (ctx.synchronize()) before reading them."""
        p = self.eval_plan(x.shape[0])
        p.x_in.copy_(x, non_blocking=True)
        self.ctx.run(p.prog)
        return p

    def _record_optimizer(self, grads):
        ops.sgd_momentum_step(self.ctx, self.params, grads, self.momentum_buf, self.lr, self.momentum,
                              self.weight_decay, shadow=self.shadow)
        # the transposed copies are read by the data gradients only: made on the second lane, beside the next
        # step's forward pass; the backward program joins the lanes before its first data gradient
        if self.overlap_wgrad:
            with self.ctx.side_lane(wait_main=True):
                self._refresh_transposed()
        else:
            self._refresh_transposed()
