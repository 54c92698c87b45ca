"""Tensor-level wrappers over the C ABI (include/torch_col_hip.h).

torch is used for device memory and streams only: every function takes tensors
that already live on the GPU, passes their raw pointers to the shared library,
and the library enqueues hand-written HIP kernels.  Layout is NHWC throughout;
filters are [K, R, S, C].
"""
import contextlib
import ctypes
import time

import torch

from ._lib import check, lib

F32, BF16 = 0, 1


def dtype_code(t):
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"unsupported dtype {t.dtype}")


def chunk_elems(dtype):
    return 8 if dtype in (BF16, torch.bfloat16) else 4


def _p(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("device operators need GPU tensors")
    if not t.is_contiguous():
        raise ValueError("device operators need contiguous tensors")
    return ctypes.c_void_p(t.data_ptr())


class Program:
    """A recorded sequence of launches (replayed without touching Python per launch)."""

    def __init__(self):
        h = ctypes.c_void_p()
        check(lib().tch_program_create(ctypes.byref(h)), "tch_program_create")
        self.handle = h
        self.keepalive = []  # tensors whose addresses are baked into the launches

    def __len__(self):
        return int(lib().tch_program_size(self.handle))

    def __del__(self):
        try:
            if self.handle:
                lib().tch_program_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class Context:
    """Launch target: a HIP stream, optionally behind a preemptible launch queue."""

    def __init__(self, stream=None):
        if stream is None:
            stream = torch.cuda.current_stream()
        self.stream = stream
        h = ctypes.c_void_p()
        check(lib().tch_context_create(ctypes.c_void_p(stream.cuda_stream), ctypes.byref(h)), "tch_context_create")
        self.handle = h
        self._recording = None

    def __del__(self):
        try:
            if self.handle:
                lib().tch_context_destroy(self.handle)
                self.handle = None
        except Exception:
            pass

    def begin_record(self, program):
        check(lib().tch_program_begin_record(self.handle, program.handle), "tch_program_begin_record")
        self._recording = program

    def end_record(self):
        check(lib().tch_program_end_record(self.handle), "tch_program_end_record")
        self._recording = None

    def run(self, program, first=0, last=-1):
        """Replay; returns True when the reject flag made the library skip launches."""
        return check(lib().tch_program_run(self.handle, program.handle, first, last), "tch_program_run") == 1

    def take_rejected(self):
        return int(lib().tch_context_take_rejected(self.handle))

    def flush(self):
        """Wait until every queued launch has been handed to the HIP stream.  Work torch puts on
        the stream itself (copies, fills, read-backs) does not pass through the launch queue, so
        stream order only covers it once the queue is empty.  No-op for an unregistered stream."""
        s = self.stream.cuda_stream
        while lib().tch_GetXQueueSize(s):
            time.sleep(0)

    def synchronize(self):
        """Everything submitted so far, queued or not, on either lane, has finished on the GPU."""
        self.flush()
        check(lib().tch_context_synchronize(self.handle), "tch_context_synchronize")

    @contextlib.contextmanager
    def side_lane(self, wait_main=True):
        """While recording: the launches inside may run beside the main ones on a second stream;
        the first of them waits for everything recorded before it.  `join()` is where the main
        lane waits for them."""
        check(lib().tch_context_set_lane(self.handle, 1, int(wait_main)), "tch_context_set_lane")
        try:
            yield
        finally:
            check(lib().tch_context_set_lane(self.handle, 0, 0), "tch_context_set_lane")

    def join(self, behind=False):
        """While recording: the main lane waits for everything the second lane was given so far.  With `behind`
        it waits for what the second lane had been given at the previous join(behind=True) only, so the second
        lane may trail by one such section (whose buffers must then stay untouched for one section more)."""
        if behind:
            check(lib().tch_context_join_behind(self.handle), "tch_context_join_behind")
        else:
            check(lib().tch_context_join(self.handle), "tch_context_join")

    def set_cu_limit(self, n_cus):
        """From the next launch on, run on at most n_cus compute units (0 lifts the limit); needs
        tch_cu_partition_init.  Ordered with what was launched before."""
        check(lib().tch_context_set_cu_limit(self.handle, int(n_cus)), "tch_context_set_cu_limit")

    def cu_limit(self):
        return int(lib().tch_context_get_cu_limit(self.handle))

    def profile(self, program, reps=1):
        """Per-kernel HIP-event timing of `reps` replays: list of dicts with name, total_ms,
        launches, work (algorithmic flops or bytes, summed), work_is_bytes and bytes (algorithmic bytes,
        summed; 0 where a kernel annotated with flops states none)."""
        from ._lib import KernelStat
        cap = 256
        buf = (KernelStat * cap)()
        n = ctypes.c_int(0)
        check(lib().tch_program_profile(self.handle, program.handle, reps, buf, cap, ctypes.byref(n)),
              "tch_program_profile")
        return [dict(name=buf[i].name.decode(), total_ms=buf[i].total_ms, launches=int(buf[i].launches),
                     work=buf[i].work, work_is_bytes=bool(buf[i].work_is_bytes), bytes=buf[i].bytes) for i in range(n.value)]

    def time_kernel(self, program, kernel_name, reps=1):
        """Mean duration (microseconds) of the launches of one kernel inside plain replays of the program, both
        lanes running, measured with each launch's own begin / end timestamps; and their number per replay."""
        us, n = ctypes.c_double(0.0), ctypes.c_int64(0)
        check(lib().tch_program_time_kernel(self.handle, program.handle, kernel_name.encode(), int(reps),
                                            ctypes.byref(us), ctypes.byref(n)), "tch_program_time_kernel")
        return us.value, int(n.value)

    def profile_launches(self, program, reps=1):
        """The same replay, one dict per program position: name ('' for an entry that launches nothing), ms
        (mean over the repetitions, the launch alone on the chip), flops, bytes (algorithmic), lane, workgroups."""
        from ._lib import LaunchStat
        cap = len(program)
        buf = (LaunchStat * cap)()
        n = ctypes.c_int64(0)
        check(lib().tch_program_profile_launches(self.handle, program.handle, reps, buf, cap, ctypes.byref(n)),
              "tch_program_profile_launches")
        return [dict(name=buf[i].name.decode(), ms=buf[i].ms, flops=buf[i].flops, bytes=buf[i].bytes,
                     lane=int(buf[i].lane), workgroups=int(buf[i].workgroups)) for i in range(n.value)]


# ---------------------------------------------------------------------------
# convolution
# ---------------------------------------------------------------------------

def conv_out_hw(H, W, R, S, stride, pad):
    return (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1


def conv2d_fwd(ctx, x, w, y, stride, pad, add=None, mask=None, bias=None, tile_cfg=-1, c_logical=0):
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    assert C == C2, "filter / input channel mismatch"
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(y.shape) == (N, Ho, Wo, K), f"output shape {tuple(y.shape)} != {(N, Ho, Wo, K)}"
    assert w.dtype == x.dtype
    out_f32 = int(y.dtype == torch.float32 and x.dtype != torch.float32)
    for t in (add, mask):
        assert t is None or (t.shape == y.shape and t.dtype == x.dtype)
    assert bias is None or (bias.dtype == torch.float32 and bias.numel() == K)
    check(lib().tch_conv2d_fwd(ctx.handle, dtype_code(x), _p(x), _p(w), _p(y), _p(add), _p(mask), _p(bias), out_f32,
                               N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical), "tch_conv2d_fwd")


def conv2d_fwd_stat_rows(x, K, R, S, stride, pad, tile_cfg=-1):
    N, H, W, C = x.shape
    return int(lib().tch_conv2d_fwd_stat_rows(dtype_code(x), N, H, W, C, K, R, S, stride, pad, tile_cfg))


def conv2d_fwd_affine(ctx, x, w, y, stride, pad, scale=None, shift=None, residual=None, relu=False, tile_cfg=-1,
                      c_logical=0):
    """y = relu?(conv(x, w) * scale + shift + residual?) in one launch (inference-mode BatchNorm folded into the
    convolution's epilogue)."""
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    assert C == C2 and w.dtype == x.dtype == y.dtype
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(y.shape) == (N, Ho, Wo, K)
    for t in (scale, shift):
        assert t is None or (t.dtype == torch.float32 and t.numel() == K)
    assert residual is None or (residual.shape == y.shape and residual.dtype == y.dtype)
    check(lib().tch_conv2d_fwd_affine(ctx.handle, dtype_code(x), _p(x), _p(w), _p(y), _p(scale), _p(shift), _p(residual),
                                      int(relu), N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical),
          "tch_conv2d_fwd_affine")


def conv2d_fwd_bnstats(ctx, x, w, y, stride, pad, partial, tile_cfg=-1, c_logical=0):
    """conv2d_fwd that also leaves the per-row-tile BatchNorm sums of y in `partial`
    ([row tiles, K, 2] fp32); returns the number of row tiles."""
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    assert C == C2 and w.dtype == x.dtype == y.dtype
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(y.shape) == (N, Ho, Wo, K)
    rb = conv2d_fwd_stat_rows(x, K, R, S, stride, pad, tile_cfg)
    assert partial.dtype == torch.float32 and partial.numel() >= rb * K * 2
    check(lib().tch_conv2d_fwd_bnstats(ctx.handle, dtype_code(x), _p(x), _p(w), _p(y), N, H, W, C, K, R, S, stride, pad,
                                       tile_cfg, c_logical, _p(partial)), "tch_conv2d_fwd_bnstats")
    return rb


def _check_acc(acc, C):
    """copies of an accumulator set [copies, 4, C] int64 (copies a power of two)."""
    assert acc.dtype == torch.int64 and acc.is_contiguous() and acc.numel() % (4 * C) == 0, "accumulators: [copies, 4, C] int64"
    copies = acc.numel() // (4 * C)
    assert copies >= 1 and copies & (copies - 1) == 0, "accumulator copies: a power of two"
    return copies


def conv2d_fwd_bnacc(ctx, x, w, y, stride, pad, acc, tile_cfg=-1, c_logical=0):
    """conv2d_fwd that also ADDS the BatchNorm sums of y (sum, sum of squares per output channel) to the exact
    accumulators `acc` ([copies, 4, K] int64, zero before the call): no per-tile partials, see bn_fwd_train_acc."""
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    assert C == C2 and w.dtype == x.dtype == y.dtype
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(y.shape) == (N, Ho, Wo, K)
    copies = _check_acc(acc, K)
    check(lib().tch_conv2d_fwd_bnacc(ctx.handle, dtype_code(x), _p(x), _p(w), _p(y), N, H, W, C, K, R, S, stride, pad,
                                     tile_cfg, c_logical, _p(acc), copies), "tch_conv2d_fwd_bnacc")


def _check_addend(add, dx, add_stride):
    """add is laid out like dx, or (add_stride 2) holds the even (h, w) of dx's grid only."""
    assert add_stride in (1, 2)
    if add is None:
        return
    N, H, W, C = dx.shape
    want = (N, H, W, C) if add_stride == 1 else (N, (H + 1) // 2, (W + 1) // 2, C)
    assert tuple(add.shape) == want and add.dtype == dx.dtype, (tuple(add.shape), want)


def conv2d_dgrad(ctx, dy, wt, dx, stride, pad, add=None, mask=None, tile_cfg=-1, c_logical=0, add_stride=1):
    """wt is the filter transposed to [C,R,S,K] (filter_transpose).  add_stride=2: `add` is [N, ceil(H/2), ceil(W/2), C]
    and counts at the even pixels of dx's grid (the compact data gradient of a stride-2 1x1 convolution)."""
    w = wt
    N, H, W, C = dx.shape
    C2, R, S, K = wt.shape
    assert C == C2
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(dy.shape) == (N, Ho, Wo, K)
    assert dy.dtype == w.dtype == dx.dtype
    assert mask is None or (mask.shape == dx.shape and mask.dtype == dx.dtype)
    _check_addend(add, dx, add_stride)
    check(lib().tch_conv2d_dgrad(ctx.handle, dtype_code(dy), _p(dy), _p(w), _p(dx), _p(add), _p(mask),
                                 N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical, add_stride), "tch_conv2d_dgrad")


def conv2d_dgrad_stat_rows(dx, K, R, S, stride, pad, tile_cfg=-1):
    N, H, W, C = dx.shape
    return int(lib().tch_conv2d_dgrad_stat_rows(dtype_code(dx), N, H, W, C, K, R, S, stride, pad, tile_cfg))


def conv2d_dgrad_bnsums(ctx, dy, wt, dx, stride, pad, bn_x, bn_mean, bn_invstd, partial, bn_mask=None, add=None,
                        mask=None, tile_cfg=-1, c_logical=0, add_stride=1):
    """conv2d_dgrad whose output is the gradient behind a BatchNorm(+ReLU) with input bn_x and ReLU output
    bn_mask: dx is stored already gated by the ReLU, and `partial` ([row tiles, C, 2] fp32) receives the two
    reductions of that BatchNorm's backward.  Returns the number of row tiles."""
    N, H, W, C = dx.shape
    C2, R, S, K = wt.shape
    assert C == C2
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(dy.shape) == (N, Ho, Wo, K)
    assert dy.dtype == wt.dtype == dx.dtype
    for t in (mask, bn_mask, bn_x):
        assert t is None or (t.shape == dx.shape and t.dtype == dx.dtype)
    _check_addend(add, dx, add_stride)
    assert bn_x is not None and bn_mean.numel() == C and bn_invstd.numel() == C
    assert bn_mean.dtype == bn_invstd.dtype == torch.float32
    rb = conv2d_dgrad_stat_rows(dx, K, R, S, stride, pad, tile_cfg)
    assert partial.dtype == torch.float32 and partial.numel() >= rb * C * 2
    check(lib().tch_conv2d_dgrad_bnsums(ctx.handle, dtype_code(dy), _p(dy), _p(wt), _p(dx), _p(add), _p(mask),
                                        N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical, _p(bn_mask), _p(bn_x),
                                        _p(bn_mean), _p(bn_invstd), _p(partial), add_stride), "tch_conv2d_dgrad_bnsums")
    return rb


def conv2d_dgrad_bnacc(ctx, dy, wt, dx, stride, pad, bn_x, bn_mean, bn_invstd, acc, bn_mask=None, add=None,
                       mask=None, tile_cfg=-1, c_logical=0, add_stride=1):
    """conv2d_dgrad_bnsums with the two reductions ADDED to the exact accumulators `acc` ([copies, 4, C] int64, zero before
    the call) instead of left per row tile; see bn_bwd_acc."""
    N, H, W, C = dx.shape
    C2, R, S, K = wt.shape
    assert C == C2
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(dy.shape) == (N, Ho, Wo, K)
    assert dy.dtype == wt.dtype == dx.dtype
    for t in (mask, bn_mask, bn_x):
        assert t is None or (t.shape == dx.shape and t.dtype == dx.dtype)
    _check_addend(add, dx, add_stride)
    assert bn_x is not None and bn_mean.numel() == C and bn_invstd.numel() == C
    assert bn_mean.dtype == bn_invstd.dtype == torch.float32
    copies = _check_acc(acc, C)
    check(lib().tch_conv2d_dgrad_bnacc(ctx.handle, dtype_code(dy), _p(dy), _p(wt), _p(dx), _p(add), _p(mask),
                                       N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical, _p(bn_mask), _p(bn_x),
                                       _p(bn_mean), _p(bn_invstd), _p(acc), copies, add_stride), "tch_conv2d_dgrad_bnacc")


def conv2d_fwd_bn(ctx, x, w, y, stride, pad, partial, counters, gamma, beta, running_mean, running_var, save_mean,
                  save_invstd, coef, momentum=0.1, eps=1e-5, tile_cfg=-1, c_logical=0):
    """conv2d_fwd + batch statistics + the BatchNorm's scale / shift (coef [2, K]); finish with bn_apply_fwd."""
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    assert C == C2 and w.dtype == x.dtype == y.dtype
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(y.shape) == (N, Ho, Wo, K)
    rb = conv2d_fwd_stat_rows(x, K, R, S, stride, pad, tile_cfg)
    assert partial.dtype == torch.float32 and partial.numel() >= rb * K * 2
    assert counters.dtype == torch.int32 and counters.numel() >= (K + 63) // 64 and coef.numel() >= 2 * K
    for t in (gamma, beta, save_mean, save_invstd):
        assert t.dtype == torch.float32 and t.numel() == K
    check(lib().tch_conv2d_fwd_bn(ctx.handle, dtype_code(x), _p(x), _p(w), _p(y), N, H, W, C, K, R, S, stride, pad,
                                  tile_cfg, c_logical, _p(partial), _p(counters), _p(gamma), _p(beta), _p(running_mean),
                                  _p(running_var), _p(save_mean), _p(save_invstd), momentum, eps, _p(coef)),
          "tch_conv2d_fwd_bn")


def conv2d_dgrad_bn(ctx, dy, wt, dx, stride, pad, bn_x, bn_mean, bn_invstd, partial, counters, gamma, dgamma, dbeta, coef,
                    bn_mask=None, add=None, mask=None, accumulate=False, tile_cfg=-1, c_logical=0, add_stride=1):
    """conv2d_dgrad_bnsums + dgamma / dbeta + the coefficients of the BatchNorm input gradient (coef [3, C]);
    finish with bn_apply_bwd."""
    N, H, W, C = dx.shape
    C2, R, S, K = wt.shape
    assert C == C2
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(dy.shape) == (N, Ho, Wo, K) and dy.dtype == wt.dtype == dx.dtype
    for t in (mask, bn_mask, bn_x):
        assert t is None or (t.shape == dx.shape and t.dtype == dx.dtype)
    _check_addend(add, dx, add_stride)
    assert bn_x is not None and bn_mean.numel() == C and bn_invstd.numel() == C
    rb = conv2d_dgrad_stat_rows(dx, K, R, S, stride, pad, tile_cfg)
    assert partial.dtype == torch.float32 and partial.numel() >= rb * C * 2
    assert counters.dtype == torch.int32 and counters.numel() >= (C + 63) // 64 and coef.numel() >= 3 * C
    check(lib().tch_conv2d_dgrad_bn(ctx.handle, dtype_code(dy), _p(dy), _p(wt), _p(dx), _p(add), _p(mask),
                                    N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical, _p(bn_mask), _p(bn_x),
                                    _p(bn_mean), _p(bn_invstd), _p(partial), _p(counters), _p(gamma), _p(dgamma),
                                    _p(dbeta), int(accumulate), _p(coef), add_stride), "tch_conv2d_dgrad_bn")


def bn_apply_fwd(ctx, x, y, coef, residual=None, relu=True):
    C = x.shape[-1]
    assert y.shape == x.shape and y.dtype == x.dtype and coef.numel() >= 2 * C
    assert residual is None or (residual.shape == x.shape and residual.dtype == x.dtype)
    check(lib().tch_bn_apply_fwd(ctx.handle, dtype_code(x), _p(x), _p(y), _p(residual), int(relu), x.numel() // C, C,
                                 _p(coef)), "tch_bn_apply_fwd")


def bn_eval_coef(ctx, gamma, beta, running_mean, running_var, coef, eps=1e-5):
    """coef [2, C] fp32 = (scale, shift) of inference-mode BatchNorm from the running statistics."""
    C = gamma.numel()
    assert coef.dtype == torch.float32 and coef.numel() >= 2 * C
    check(lib().tch_bn_eval_coef(ctx.handle, _p(gamma), _p(beta), _p(running_mean), _p(running_var), _p(coef), C,
                                 float(eps)), "tch_bn_eval_coef")


def bn_apply_bwd(ctx, g, x, dx, coef):
    C = x.shape[-1]
    assert g.shape == x.shape == dx.shape and g.dtype == x.dtype == dx.dtype and coef.numel() >= 3 * C
    check(lib().tch_bn_apply_bwd(ctx.handle, dtype_code(x), _p(g), _p(x), _p(dx), x.numel() // C, C, _p(coef)),
          "tch_bn_apply_bwd")


def conv2d_wgrad_splits(x, K, R, S, stride, pad):
    N, H, W, C = x.shape
    return int(lib().tch_conv2d_wgrad_pick_splits(dtype_code(x), N, H, W, C, K, R, S, stride, pad))


def conv2d_wgrad_workspace_bytes(dtype, K, R, S, C, splits):
    return int(lib().tch_conv2d_wgrad_workspace_bytes(dtype, K, R, S, C, splits))


def conv2d_wgrad(ctx, x, dy, dw, stride, pad, workspace=None, splits=0, accumulate=False, tile_cfg=-1, c_logical=0,
                 dbias=None):
    """dw (+)= dy^T x over the pixels; with dbias [K] fp32 also dbias (+)= column sums of dy."""
    N, H, W, C = x.shape
    K, R, S, C2 = dw.shape
    assert C == C2 and dw.dtype == torch.float32
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(dy.shape) == (N, Ho, Wo, K) and dy.dtype == x.dtype
    if workspace is not None:
        if splits <= 0:
            splits = conv2d_wgrad_splits(x, K, R, S, stride, pad)
        need = conv2d_wgrad_workspace_bytes(dtype_code(x), K, R, S, C, splits)
        assert workspace.numel() * workspace.element_size() >= need, "wgrad workspace too small"
    if dbias is not None:
        assert dbias.dtype == torch.float32 and dbias.numel() == K
        check(lib().tch_conv2d_wgrad_bias(ctx.handle, dtype_code(x), _p(x), _p(dy), _p(dw), _p(dbias), _p(workspace),
                                          splits, int(accumulate), N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical),
              "tch_conv2d_wgrad_bias")
        return
    check(lib().tch_conv2d_wgrad(ctx.handle, dtype_code(x), _p(x), _p(dy), _p(dw), _p(workspace), splits,
                                 int(accumulate), N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical),
          "tch_conv2d_wgrad")


class TrailingWgrad:
    """A run of weight gradients on one context whose split reductions ride the launches behind them
    (tch_conv2d_wgrad_trailing): `workspace` holds TWO workspaces of `half` floats each, taken in turn (the partials
    of a call are read by the call after it).  flush() launches the last reduction; until then the last dw is
    incomplete."""

    def __init__(self, ctx, workspace, half):
        assert workspace.dtype == torch.float32 and workspace.numel() >= 2 * half
        self.ctx, self.ws, self.half, self.turn = ctx, workspace, half, 0

    def wgrad(self, x, dy, dw, stride, pad, accumulate=False, tile_cfg=-1, c_logical=0, dbias=None):
        N, H, W, C = x.shape
        K, R, S, C2 = dw.shape
        assert C == C2 and dw.dtype == torch.float32
        Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
        assert tuple(dy.shape) == (N, Ho, Wo, K) and dy.dtype == x.dtype
        assert dbias is None or (dbias.dtype == torch.float32 and dbias.numel() == K)
        splits = conv2d_wgrad_splits(x, K, R, S, stride, pad)
        assert self.half * 4 >= conv2d_wgrad_workspace_bytes(dtype_code(x), K, R, S, C, splits), "wgrad workspace too small"
        ws = self.ws[self.turn * self.half:(self.turn + 1) * self.half]
        self.turn ^= 1
        check(lib().tch_conv2d_wgrad_trailing(self.ctx.handle, dtype_code(x), _p(x), _p(dy), _p(dw), _p(dbias), _p(ws),
                                              splits, int(accumulate), N, H, W, C, K, R, S, stride, pad, tile_cfg,
                                              c_logical), "tch_conv2d_wgrad_trailing")

    def flush(self):
        check(lib().tch_conv2d_wgrad_flush(self.ctx.handle), "tch_conv2d_wgrad_flush")


def _wgrad_group_shapes(items):
    import ctypes
    flat = []
    for it in items:
        x, dy, dw, stride, pad = it[:5]
        N, H, W, C = x.shape
        K, R, S, C2 = dw.shape
        assert C == C2 and dw.dtype == torch.float32 and dy.dtype == x.dtype
        Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
        assert tuple(dy.shape) == (N, Ho, Wo, K), (tuple(dy.shape), (N, Ho, Wo, K))
        flat += [N, H, W, C, K, R, S, stride, pad]
    return (ctypes.c_int * len(flat))(*flat)


def conv2d_wgrad_group_plan(items, target_wgs=0, tile_cfg=-1):
    """items: (x, dy, dw, stride, pad[, dbias]) per convolution (tensors may be on the meta device).  Returns
    (splits per convolution, tiling, table bytes, workspace bytes) for conv2d_wgrad_group."""
    import ctypes
    n = len(items)
    shapes = _wgrad_group_shapes(items)
    splits = (ctypes.c_int * n)()
    tb, wb = ctypes.c_int64(0), ctypes.c_int64(0)
    tile = check(lib().tch_conv2d_wgrad_group_plan(dtype_code(items[0][0]), n, shapes, target_wgs, tile_cfg, splits,
                                                   ctypes.byref(tb), ctypes.byref(wb)), "tch_conv2d_wgrad_group_plan")
    return list(splits), tile, tb.value, wb.value


def conv2d_wgrad_group(ctx, items, splits, tile_cfg, workspace, table, accumulate=False, max_wgs=0):
    """The weight gradients of every (x, dy, dw, stride, pad[, dbias]) of `items` in one launch (+ one for the
    split reductions): dw (+)= dy^T x, dbias (+)= column sums of dy.  `table` (uint8, device) and `workspace`
    (fp32, device) sized by conv2d_wgrad_group_plan; the table is written here and must stay untouched while a
    recorded program holds the launches.  max_wgs > 0: at most that many workgroups, which share the tiles out
    among themselves (a launch that runs beside others instead of flooding the chip)."""
    import ctypes
    n = len(items)
    assert n == len(splits) and table.dtype == torch.uint8 and table.is_cuda
    shapes = _wgrad_group_shapes(items)
    arr = ctypes.c_uint64 * n
    xs = arr(*[it[0].data_ptr() for it in items])
    dys = arr(*[it[1].data_ptr() for it in items])
    dws = arr(*[it[2].data_ptr() for it in items])
    with_bias = any(len(it) > 5 and it[5] is not None for it in items)
    dbs = arr(*[(it[5].data_ptr() if len(it) > 5 and it[5] is not None else 0) for it in items]) if with_bias else None
    sp = (ctypes.c_int * n)(*splits)
    check(lib().tch_conv2d_wgrad_group(ctx.handle, dtype_code(items[0][0]), n, shapes, xs, dys, dws, dbs, sp, tile_cfg,
                                       int(accumulate), _p(workspace), _p(table), max_wgs), "tch_conv2d_wgrad_group")


def conv2d_wgrad_static_capacity_bytes():
    return int(lib().tch_conv2d_wgrad_static_capacity_bytes())


def conv2d_wgrad_static(ctx, x, dy, dw, stride, pad, splits=0, accumulate=False, tile_cfg=-1, c_logical=0):
    """conv2d_wgrad with the split-K partials in the library's static device buffer: nothing is allocated and no
    workspace is passed (for callers that cannot allocate)."""
    N, H, W, C = x.shape
    K, R, S, C2 = dw.shape
    assert C == C2 and dw.dtype == torch.float32
    Ho, Wo = conv_out_hw(H, W, R, S, stride, pad)
    assert tuple(dy.shape) == (N, Ho, Wo, K) and dy.dtype == x.dtype
    check(lib().tch_conv2d_wgrad_static(ctx.handle, dtype_code(x), _p(x), _p(dy), _p(dw), splits, int(accumulate),
                                        N, H, W, C, K, R, S, stride, pad, tile_cfg, c_logical),
          "tch_conv2d_wgrad_static")


# ---------------------------------------------------------------------------
# BatchNorm
# ---------------------------------------------------------------------------

def bn_workspace_bytes(dtype, rows, C):
    return int(lib().tch_bn_workspace_bytes(dtype, rows, C))


def bn_fwd_train(ctx, x, y, gamma, beta, running_mean, running_var, save_mean, save_invstd, workspace,
                 residual=None, relu=False, momentum=0.1, eps=1e-5):
    C = x.shape[-1]
    rows = x.numel() // C
    assert y.shape == x.shape and y.dtype == x.dtype
    assert residual is None or (residual.shape == x.shape and residual.dtype == x.dtype)
    for t in (gamma, beta, save_mean, save_invstd):
        assert t.dtype == torch.float32 and t.numel() == C
    assert workspace.numel() * workspace.element_size() >= bn_workspace_bytes(dtype_code(x), rows, C)
    check(lib().tch_bn_fwd_train(ctx.handle, dtype_code(x), _p(x), _p(y), _p(residual), int(relu), rows, C,
                                 _p(gamma), _p(beta), _p(running_mean), _p(running_var), _p(save_mean),
                                 _p(save_invstd), momentum, eps, _p(workspace)), "tch_bn_fwd_train")


def bn_fwd_train_partials(ctx, x, y, gamma, beta, running_mean, running_var, save_mean, save_invstd, partial,
                          row_blocks, scratch, residual=None, relu=False, momentum=0.1, eps=1e-5):
    """bn_fwd_train on statistics the producer of x has already summed per row block."""
    C = x.shape[-1]
    rows = x.numel() // C
    assert y.shape == x.shape and y.dtype == x.dtype
    assert residual is None or (residual.shape == x.shape and residual.dtype == x.dtype)
    for t in (gamma, beta, save_mean, save_invstd):
        assert t.dtype == torch.float32 and t.numel() == C
    assert partial.dtype == torch.float32 and partial.numel() >= row_blocks * C * 2
    assert scratch.dtype == torch.float32 and scratch.numel() >= 2 * C
    check(lib().tch_bn_fwd_train_partials(ctx.handle, dtype_code(x), _p(x), _p(y), _p(residual), int(relu), rows, C,
                                          _p(gamma), _p(beta), _p(running_mean), _p(running_var), _p(save_mean),
                                          _p(save_invstd), momentum, eps, _p(partial), int(row_blocks), _p(scratch)),
          "tch_bn_fwd_train_partials")


def bn_fwd_train_acc(ctx, x, y, gamma, beta, running_mean, running_var, save_mean, save_invstd, acc, residual=None,
                     relu=False, momentum=0.1, eps=1e-5):
    """bn_fwd_train from the accumulators conv2d_fwd_bnacc added the statistics of x to: one launch."""
    C = x.shape[-1]
    rows = x.numel() // C
    assert y.shape == x.shape and y.dtype == x.dtype
    assert residual is None or (residual.shape == x.shape and residual.dtype == x.dtype)
    for t in (gamma, beta, save_mean, save_invstd):
        assert t.dtype == torch.float32 and t.numel() == C
    copies = _check_acc(acc, C)
    check(lib().tch_bn_fwd_train_acc(ctx.handle, dtype_code(x), _p(x), _p(y), _p(residual), int(relu), rows, C,
                                     _p(gamma), _p(beta), _p(running_mean), _p(running_var), _p(save_mean),
                                     _p(save_invstd), momentum, eps, _p(acc), copies), "tch_bn_fwd_train_acc")


def bn_bwd_acc(ctx, g, x, dx, gamma, save_mean, save_invstd, dgamma, dbeta, acc, accumulate=False):
    """bn_bwd from the accumulators conv2d_dgrad_bnacc added the two sums to; g is already gated by the ReLU."""
    C = x.shape[-1]
    rows = x.numel() // C
    assert g.shape == x.shape == dx.shape and g.dtype == x.dtype == dx.dtype
    copies = _check_acc(acc, C)
    check(lib().tch_bn_bwd_acc(ctx.handle, dtype_code(x), _p(g), _p(x), _p(dx), rows, C, _p(gamma), _p(save_mean),
                               _p(save_invstd), _p(dgamma), _p(dbeta), int(accumulate), _p(acc), copies), "tch_bn_bwd_acc")


def bn_bwd(ctx, dy, x, dx, gamma, save_mean, save_invstd, dgamma, dbeta, workspace, relu_mask=None,
           accumulate=False):
    C = x.shape[-1]
    rows = x.numel() // C
    assert dy.shape == x.shape == dx.shape and dy.dtype == x.dtype == dx.dtype
    assert relu_mask is None or (relu_mask.shape == x.shape and relu_mask.dtype == x.dtype)
    assert workspace.numel() * workspace.element_size() >= bn_workspace_bytes(dtype_code(x), rows, C)
    check(lib().tch_bn_bwd(ctx.handle, dtype_code(x), _p(dy), _p(relu_mask), _p(x), _p(dx), rows, C, _p(gamma),
                           _p(save_mean), _p(save_invstd), _p(dgamma), _p(dbeta), int(accumulate), _p(workspace)),
          "tch_bn_bwd")


def bn_bwd_partials(ctx, g, x, dx, gamma, save_mean, save_invstd, dgamma, dbeta, partial, row_blocks, scratch,
                    accumulate=False):
    """bn_bwd from the sums conv2d_dgrad_bnsums left in `partial`; g is already gated by the ReLU."""
    C = x.shape[-1]
    rows = x.numel() // C
    assert g.shape == x.shape == dx.shape and g.dtype == x.dtype == dx.dtype
    assert partial.numel() >= row_blocks * C * 2 and scratch.numel() >= 3 * C
    check(lib().tch_bn_bwd_partials(ctx.handle, dtype_code(x), _p(g), _p(x), _p(dx), rows, C, _p(gamma), _p(save_mean),
                                    _p(save_invstd), _p(dgamma), _p(dbeta), int(accumulate), _p(partial),
                                    int(row_blocks), _p(scratch)), "tch_bn_bwd_partials")


# ---------------------------------------------------------------------------
# pooling
# ---------------------------------------------------------------------------

def maxpool_fwd(ctx, x, y, index, ksize, stride, pad):
    N, H, W, C = x.shape
    Ho, Wo = conv_out_hw(H, W, ksize, ksize, stride, pad)
    assert tuple(y.shape) == (N, Ho, Wo, C) and tuple(index.shape) == (N, Ho, Wo, C)
    assert index.dtype == torch.int32 and y.dtype == x.dtype
    check(lib().tch_maxpool_fwd(ctx.handle, dtype_code(x), _p(x), _p(y), _p(index), N, H, W, C, ksize, stride, pad),
          "tch_maxpool_fwd")


def maxpool_bwd(ctx, dy, index, dx, ksize, stride, pad):
    N, H, W, C = dx.shape
    Ho, Wo = conv_out_hw(H, W, ksize, ksize, stride, pad)
    assert tuple(dy.shape) == (N, Ho, Wo, C) and tuple(index.shape) == (N, Ho, Wo, C)
    assert index.dtype == torch.int32 and dy.dtype == dx.dtype
    check(lib().tch_maxpool_bwd(ctx.handle, dtype_code(dy), _p(dy), _p(index), _p(dx), N, H, W, C, ksize, stride,
                                pad), "tch_maxpool_bwd")


def avgpool_fwd(ctx, x, y):
    N, H, W, C = x.shape
    assert tuple(y.shape) == (N, C) and y.dtype == x.dtype
    check(lib().tch_avgpool_fwd(ctx.handle, dtype_code(x), _p(x), _p(y), N, H * W, C), "tch_avgpool_fwd")


def avgpool_bwd(ctx, dy, dx):
    N, H, W, C = dx.shape
    assert tuple(dy.shape) == (N, C) and dy.dtype == dx.dtype
    check(lib().tch_avgpool_bwd(ctx.handle, dtype_code(dy), _p(dy), _p(dx), N, H * W, C), "tch_avgpool_bwd")


# ---------------------------------------------------------------------------
# loss / optimizer / helpers
# ---------------------------------------------------------------------------

def softmax_ce_fwd_bwd(ctx, logits, labels, loss_rows, loss_mean, dlogits, loss_scale=1.0):
    rows, classes = logits.shape
    assert logits.dtype == torch.float32 and labels.dtype == torch.int64 and labels.numel() == rows
    assert loss_rows.dtype == torch.float32 and loss_rows.numel() >= rows and loss_mean.dtype == torch.float32
    assert dlogits.shape[0] == rows and dlogits.shape[1] >= classes and dlogits.stride(0) == dlogits.shape[1]
    check(lib().tch_softmax_ce_fwd_bwd(ctx.handle, dtype_code(dlogits), _p(logits), _p(labels), _p(loss_rows),
                                       _p(loss_mean), _p(dlogits), rows, classes, dlogits.shape[1],
                                       float(loss_scale) / rows), "tch_softmax_ce_fwd_bwd")


def softmax_ce_lm(ctx, logits, labels, loss_rows, loss_mean, dlogits, classes, valid_rows, loss_scale=1.0):
    """logits [rows, ld] fp32 and dlogits [rows, ld'] with ld, ld' >= classes; labels < 0 are ignored."""
    rows = logits.shape[0]
    assert logits.dtype == torch.float32 and labels.dtype == torch.int64 and labels.numel() == rows
    assert logits.stride(0) == logits.shape[1] >= classes and dlogits.stride(0) == dlogits.shape[1] >= classes
    assert dlogits.shape[0] == rows and loss_rows.numel() >= rows
    check(lib().tch_softmax_ce_lm(ctx.handle, dtype_code(dlogits), _p(logits), logits.shape[1], _p(labels), _p(loss_rows),
                                  _p(loss_mean), _p(dlogits), dlogits.shape[1], rows, classes, int(valid_rows),
                                  float(loss_scale)), "tch_softmax_ce_lm")


def sgd_momentum_step(ctx, param, grad, buf, lr, momentum, weight_decay, shadow=None):
    n = param.numel()
    assert param.dtype == grad.dtype == buf.dtype == torch.float32 and grad.numel() == n and buf.numel() == n
    assert shadow is None or (shadow.dtype == torch.bfloat16 and shadow.numel() == n)
    check(lib().tch_sgd_momentum_step(ctx.handle, _p(param), _p(grad), _p(buf), _p(shadow), n, lr, momentum,
                                      weight_decay), "tch_sgd_momentum_step")


def grad_accumulate(ctx, global_grad, grad):
    assert global_grad.dtype == grad.dtype == torch.float32 and global_grad.numel() == grad.numel()
    check(lib().tch_grad_accumulate(ctx.handle, _p(global_grad), _p(grad), grad.numel()), "tch_grad_accumulate")


def fill_zero(ctx, t):
    check(lib().tch_fill_zero(ctx.handle, _p(t), t.numel() * t.element_size()), "tch_fill_zero")


def bias_grad(ctx, dy, dbias, cols=None, accumulate=False, workspace=None):
    rows, ld = dy.shape
    cols = ld if cols is None else cols
    if workspace is not None:
        assert workspace.dtype == torch.float32
        check(lib().tch_bias_grad_ws(ctx.handle, dtype_code(dy), _p(dy), _p(dbias), rows, cols, ld, int(accumulate),
                                     _p(workspace), workspace.numel()), "tch_bias_grad_ws")
        return
    check(lib().tch_bias_grad(ctx.handle, dtype_code(dy), _p(dy), _p(dbias), rows, cols, ld, int(accumulate)),
          "tch_bias_grad")


def nchw_to_nhwc_pad(ctx, x_nchw, y_nhwc):
    N, C, H, W = x_nchw.shape
    assert x_nchw.dtype == torch.float32 and tuple(y_nhwc.shape[:3]) == (N, H, W)
    check(lib().tch_nchw_to_nhwc_pad(ctx.handle, dtype_code(y_nhwc), _p(x_nchw), _p(y_nhwc), N, C, H, W,
                                     y_nhwc.shape[3]), "tch_nchw_to_nhwc_pad")


class FilterTransposeTable:
    """Device table for tch_filter_transpose_batched: filters [(element offset, K, RS, C), ...]
    that sit at the same offsets inside a flat source and a flat destination buffer."""

    def __init__(self, filters, device):
        rows, tile = [], 0
        self.total_elems = 0
        for off, K, RS, C in filters:
            rows.append([tile, off, K, RS, C])
            tile += RS * ((K + 31) // 32) * ((C + 31) // 32)
            self.total_elems += K * RS * C
        self.total_tiles = tile
        self.n = len(rows)
        self.table = torch.tensor(rows, dtype=torch.int64).to(device)


def filter_transpose_batched(ctx, src, dst, table):
    """dst[C][RS][K] = src[K][RS][C] for every filter of the table (one launch)."""
    assert src.dtype == dst.dtype and src.numel() == dst.numel()
    check(lib().tch_filter_transpose_batched(ctx.handle, dtype_code(src), _p(src), _p(dst), _p(table.table), table.n,
                                             table.total_tiles, table.total_elems), "tch_filter_transpose_batched")


def filter_transpose(ctx, w):
    """[K,R,S,C] -> [C,R,S,K] (the layout conv2d_dgrad reads)."""
    K, R, S, C = w.shape
    out = torch.empty((C, R, S, K), dtype=w.dtype, device=w.device)
    filter_transpose_batched(ctx, w, out, FilterTransposeTable([(0, K, R * S, C)], w.device))
    return out


def cast_from_f32(ctx, src, dst):
    assert src.dtype == torch.float32 and src.numel() == dst.numel()
    check(lib().tch_cast_from_f32(ctx.handle, dtype_code(dst), _p(src), _p(dst), src.numel()), "tch_cast_from_f32")


def cast_to_f32(ctx, src, dst):
    assert dst.dtype == torch.float32 and src.numel() == dst.numel()
    check(lib().tch_cast_to_f32(ctx.handle, dtype_code(src), _p(src), _p(dst), src.numel()), "tch_cast_to_f32")


# ---------------------------------------------------------------------------
# transformer operators (Swin-B / GPT-2 steps)
# ---------------------------------------------------------------------------

def window_token_rows(rows, H, W, ws):
    """Rows of a window-ordered tensor that belongs to `rows` = B * H * W pixels: the frame is padded at the bottom and
    the right to whole ws x ws windows."""
    assert rows % (H * W) == 0
    return rows // (H * W) * (-(-H // ws) * ws) * (-(-W // ws) * ws)


def layernorm_fwd(ctx, x, y, gamma, beta, mean, rstd, eps=1e-5, window=None, windowed=("y",), add=None, sum_out=None):
    """window = (H, W, window size, shift): x is [B*H*W, C] in pixel order; the tensors named in `windowed` ("y",
    "add") are laid out as window tokens (the LayerNorm and the window partition next to it in a Swin block in one
    pass).  add / sum_out: sum_out = x + add (pixel order, rounded to the tensors' type), y = LayerNorm(sum_out)."""
    C = x.shape[-1]
    rows = x.numel() // C
    assert y.dtype == x.dtype and x.is_contiguous() and y.is_contiguous()
    assert gamma.numel() == C and beta.numel() == C and gamma.dtype == beta.dtype == torch.float32
    assert mean.numel() == rows and rstd.numel() == rows and mean.dtype == rstd.dtype == torch.float32
    if window is not None:
        H, W, ws, shift = window
        wrows = window_token_rows(rows, H, W, ws)      # rows of a window-ordered tensor (more than rows when padded)
        assert (add is None) == (sum_out is None)
        assert y.numel() == (wrows if "y" in windowed else rows) * C
        assert add is None or (add.numel() == (wrows if "add" in windowed else rows) * C and sum_out.numel() == x.numel()
                               and add.dtype == sum_out.dtype == x.dtype)
        flags = sum({"y": 1, "add": 4}[t] for t in windowed)
        check(lib().tch_layernorm_fwd_windowed(ctx.handle, dtype_code(x), _p(x), _p(y), _p(gamma), _p(beta), _p(mean),
                                               _p(rstd), rows, C, eps, H, W, ws, shift, flags, _p(add), _p(sum_out)),
              "tch_layernorm_fwd_windowed")
        return
    assert add is None and sum_out is None, "the residual sum comes with the windowed form"
    assert y.shape == x.shape
    check(lib().tch_layernorm_fwd(ctx.handle, dtype_code(x), _p(x), _p(y), _p(gamma), _p(beta), _p(mean), _p(rstd),
                                  rows, C, eps), "tch_layernorm_fwd")


def layernorm_bwd_partial_rows(rows):
    return int(lib().tch_layernorm_bwd_partial_rows(rows))


def layernorm_bwd(ctx, dy, x, dx, gamma, mean, rstd, dgamma, dbeta, partial, accumulate=False, residual=None,
                  window=None, windowed=()):
    """window = (H, W, window size, shift) and windowed, a subset of ("dx", "dy", "residual"): those tensors are laid
    out as window tokens, everything else ([B*H*W, C] x, the statistics) in pixel order."""
    C = x.shape[-1]
    rows = x.numel() // C
    assert dy.dtype == x.dtype == dx.dtype and (residual is None or residual.dtype == x.dtype)
    assert partial.dtype == torch.float32 and partial.numel() >= layernorm_bwd_partial_rows(rows) * C * 2
    if window is not None:
        H, W, ws, shift = window
        wrows = window_token_rows(rows, H, W, ws)      # rows of a window-ordered tensor (more than rows when padded)
        for name, t in (("dx", dx), ("dy", dy), ("residual", residual)):
            assert t is None or t.numel() == (wrows if name in windowed else rows) * C, name
        flags = sum({"dx": 1, "dy": 2, "residual": 4}[t] for t in windowed)
        check(lib().tch_layernorm_bwd_windowed(ctx.handle, dtype_code(x), _p(dy), _p(x), _p(dx), _p(residual), _p(gamma),
                                               _p(mean), _p(rstd), _p(dgamma), _p(dbeta), int(accumulate), rows, C,
                                               _p(partial), H, W, ws, shift, flags), "tch_layernorm_bwd_windowed")
        return
    assert dy.shape == x.shape == dx.shape and (residual is None or residual.shape == x.shape)
    check(lib().tch_layernorm_bwd(ctx.handle, dtype_code(x), _p(dy), _p(x), _p(dx), _p(residual), _p(gamma), _p(mean), _p(rstd),
                                  _p(dgamma), _p(dbeta), int(accumulate), rows, C, _p(partial)), "tch_layernorm_bwd")


def gelu_fwd(ctx, x, y, tanh_form=False):
    assert y.shape == x.shape and y.dtype == x.dtype
    check(lib().tch_gelu_fwd(ctx.handle, dtype_code(x), _p(x), _p(y), x.numel(), int(tanh_form)), "tch_gelu_fwd")


def gelu_bwd(ctx, dy, x, dx, tanh_form=False):
    assert dy.shape == x.shape == dx.shape and dy.dtype == x.dtype == dx.dtype
    check(lib().tch_gelu_bwd(ctx.handle, dtype_code(x), _p(dy), _p(x), _p(dx), x.numel(), int(tanh_form)), "tch_gelu_bwd")


def attn_softmax_fwd(ctx, scores, probs, scale=1.0, bias=None, mask=None, causal=False):
    """scores / probs [batch, heads, Lq, Lk]; bias [heads, Lq, Lk] fp32; mask [windows, Lq, Lk] fp32."""
    Bn, Hn, Lq, Lk = scores.shape
    assert probs.shape == scores.shape and probs.dtype == scores.dtype and scores.is_contiguous()
    windows = 1
    if bias is not None:
        assert tuple(bias.shape) == (Hn, Lq, Lk) and bias.dtype == torch.float32
    if mask is not None:
        assert tuple(mask.shape[1:]) == (Lq, Lk) and mask.dtype == torch.float32
        windows = mask.shape[0]
    check(lib().tch_attn_softmax_fwd(ctx.handle, dtype_code(scores), _p(scores), _p(probs), Bn, Hn, Lq, Lk, scale,
                                     _p(bias), _p(mask), windows, int(causal)), "tch_attn_softmax_fwd")


def attn_softmax_bwd(ctx, probs, dprobs, dscores, scale=1.0, causal=False):
    Lq, Lk = probs.shape[-2:]
    assert probs.shape == dprobs.shape == dscores.shape and probs.dtype == dprobs.dtype == dscores.dtype
    check(lib().tch_attn_softmax_bwd(ctx.handle, dtype_code(probs), _p(probs), _p(dprobs), _p(dscores),
                                     probs.numel() // Lk, Lq, Lk, scale, int(causal)), "tch_attn_softmax_bwd")


def adamw_step(ctx, param, grad, exp_avg, exp_avg_sq, step_dev, scalars_dev, lr, beta1=0.9, beta2=0.999, eps=1e-8,
               weight_decay=0.01, shadow=None):
    n = param.numel()
    for t in (grad, exp_avg, exp_avg_sq):
        assert t.dtype == torch.float32 and t.numel() == n
    assert param.dtype == torch.float32 and step_dev.dtype == torch.int32 and scalars_dev.dtype == torch.float32
    assert step_dev.numel() >= 1 and scalars_dev.numel() >= 2
    assert shadow is None or (shadow.dtype == torch.bfloat16 and shadow.numel() == n)
    check(lib().tch_adamw_step(ctx.handle, _p(param), _p(grad), _p(exp_avg), _p(exp_avg_sq), _p(shadow), n, lr, beta1,
                               beta2, eps, weight_decay, _p(step_dev), _p(scalars_dev)), "tch_adamw_step")


def embedding_fwd(ctx, ids, wte, wpe, out):
    B, T = ids.shape
    vocab, C = wte.shape
    assert ids.dtype == torch.int64 and wpe.shape[0] >= T and wpe.shape[1] == C
    assert tuple(out.shape) == (B, T, C) and out.dtype == wte.dtype == wpe.dtype
    check(lib().tch_embedding_fwd(ctx.handle, dtype_code(wte), _p(ids), _p(wte), _p(wpe), _p(out), B, T, C, vocab),
          "tch_embedding_fwd")


def embedding_bwd(ctx, ids, dy, dwte, dwpe, accumulate_wpe=False, chain=None):
    """chain: int32 scratch of 2 * B * T elements; with it the result is the same bit for bit every run (rows that
    share a token are added in position order), without it fp32 atomics decide the order."""
    B, T = ids.shape
    vocab, C = dwte.shape
    assert tuple(dy.shape) == (B, T, C) and dwte.dtype == dwpe.dtype == torch.float32 and dwpe.shape[0] >= T
    assert chain is None or (chain.dtype == torch.int32 and chain.numel() >= 2 * B * T)
    check(lib().tch_embedding_bwd(ctx.handle, dtype_code(dy), _p(ids), _p(dy), _p(dwte), _p(dwpe), B, T, C, vocab,
                                  int(accumulate_wpe), _p(chain)), "tch_embedding_bwd")


def batched_gemm(ctx, a, b, c, M, N, K, a_strides, b_strides, ldc, batch=(1, 1), a_batch=(0, 0), b_batch=(0, 0),
                 c_batch=(0, 0), alpha=1.0, accumulate=False, causal=0):
    """C[z](m, n) (+)= alpha * sum_k A[z](m, k) * B[z](n, k); strides are (row, k) in elements, batch offsets are
    (outer, inner) in elements, z = outer * batch[1] + inner.  The caller vouches that every address the
    strides reach lies inside the tensors; what can be checked from the tensor sizes is checked here."""
    assert a.dtype == b.dtype == c.dtype
    bo, bi = batch

    def extent(strides, rows, batch_off):
        return (bo - 1) * batch_off[0] + (bi - 1) * batch_off[1] + (rows - 1) * strides[0] + (K - 1) * strides[1] + 1
    assert extent(a_strides, M, a_batch) <= a.numel(), "batched_gemm: A reaches past its tensor"
    assert extent(b_strides, N, b_batch) <= b.numel(), "batched_gemm: B reaches past its tensor"
    assert (bo - 1) * c_batch[0] + (bi - 1) * c_batch[1] + (M - 1) * ldc + N <= c.numel(), \
        "batched_gemm: C reaches past its tensor"
    check(lib().tch_batched_gemm(ctx.handle, dtype_code(a), _p(a), _p(b), _p(c), M, N, K, a_strides[0], a_strides[1],
                                 b_strides[0], b_strides[1], ldc, bo, bi, a_batch[0], a_batch[1], b_batch[0], b_batch[1],
                                 c_batch[0], c_batch[1], alpha, int(accumulate), int(causal)), "tch_batched_gemm")


def _flash_check(name, t, B, H, T, strides):
    rs, bs = strides
    assert t.dtype == torch.bfloat16, f"flash attention: {name} must be bf16"
    assert (B - 1) * bs + (T - 1) * rs + H * 64 <= t.numel(), f"flash attention: {name} reaches past its tensor"


def flash_attn_fwd(ctx, q, k, v, o, lse, B, H, T, qkv_strides, o_strides, scale, causal=True):
    """o = softmax(scale * q k^T [+ causal mask]) v per head without the [T, T] scores in memory (bf16, heads 64
    wide, T a multiple of 128).  q, k, v are views that start at head 0 of sample 0; element (b, t, h, d) sits at
    b * strides[1] + t * strides[0] + 64 h + d, so the three may be slices of one packed projection.  lse
    [B * H, T] fp32 receives the log-sum-exp of the scaled scores for the backward."""
    for name, t in (("q", q), ("k", k), ("v", v)):
        _flash_check(name, t, B, H, T, qkv_strides)
    _flash_check("o", o, B, H, T, o_strides)
    assert lse.dtype == torch.float32 and lse.numel() >= B * H * T
    check(lib().tch_flash_attn_fwd(ctx.handle, dtype_code(q), _p(q), _p(k), _p(v), _p(o), _p(lse), B, H, T, qkv_strides[0],
                                   qkv_strides[1], o_strides[0], o_strides[1], scale, int(causal)), "tch_flash_attn_fwd")


def flash_attn_bwd(ctx, q, k, v, o, dout, lse, delta, dq, dk, dv, B, H, T, qkv_strides, o_strides, scale, causal=True):
    """Gradients of flash_attn_fwd; dq, dk, dv are laid out like q, k, v and o, dout like o.  delta [B * H, T]
    fp32 is scratch (row sums of dout * o)."""
    for name, t in (("q", q), ("k", k), ("v", v), ("dq", dq), ("dk", dk), ("dv", dv)):
        _flash_check(name, t, B, H, T, qkv_strides)
    for name, t in (("o", o), ("dout", dout)):
        _flash_check(name, t, B, H, T, o_strides)
    assert lse.dtype == delta.dtype == torch.float32 and lse.numel() >= B * H * T and delta.numel() >= B * H * T
    check(lib().tch_flash_attn_bwd(ctx.handle, dtype_code(q), _p(q), _p(k), _p(v), _p(o), _p(dout), _p(lse), _p(delta),
                                   _p(dq), _p(dk), _p(dv), B, H, T, qkv_strides[0], qkv_strides[1], o_strides[0],
                                   o_strides[1], scale, int(causal)), "tch_flash_attn_bwd")


# ---------------------------------------------------------------------------
# Swin-B data movement
# ---------------------------------------------------------------------------

def window_partition(ctx, src, dst, window, shift, reverse=False, add=None, image_shape=None):
    """reverse=False: src [B,H,W,C] -> dst [B*nW*window*window, C] (cyclic shift by -shift, then windows);
    reverse=True: src windows -> dst [B,H,W,C] (+ add).  image_shape = (B, H, W, C) when neither tensor says."""
    B, H, W, C = image_shape if image_shape is not None else (dst.shape if reverse else src.shape)
    assert src.numel() == dst.numel() == B * H * W * C and src.dtype == dst.dtype
    assert add is None or (add.numel() == dst.numel() and add.dtype == dst.dtype)
    check(lib().tch_window_partition(ctx.handle, dtype_code(src), _p(src), _p(dst), _p(add), B, H, W, C, window, shift,
                                     int(reverse)), "tch_window_partition")


def patch_merge_gather(ctx, src, dst, image_shape, reverse=False):
    """image_shape = (B, H, W, C) of the unmerged side; the merged side is [B, (H+1)//2, (W+1)//2, 4C] (an odd side
    is padded with zeros)."""
    B, H, W, C = image_shape
    merged = B * ((H + 1) // 2) * ((W + 1) // 2) * 4 * C
    a, b = (merged, B * H * W * C) if reverse else (B * H * W * C, merged)
    assert src.numel() == a and dst.numel() == b and src.dtype == dst.dtype
    check(lib().tch_patch_merge_gather(ctx.handle, dtype_code(src), _p(src), _p(dst), B, H, W, C, int(reverse)),
          "tch_patch_merge_gather")


def relpos_bias_gather(ctx, table, index, bias):
    entries, heads = table.shape
    nn = index.numel()
    tokens = int(round(nn ** 0.5))
    assert tokens * tokens == nn and index.dtype == torch.int32 and bias.numel() == heads * nn
    assert table.dtype == bias.dtype == torch.float32
    check(lib().tch_relpos_bias_gather(ctx.handle, _p(table), _p(index), _p(bias), heads, tokens, entries),
          "tch_relpos_bias_gather")


def relpos_bias_scatter(ctx, dbias, index, dtable, accumulate=False):
    entries, heads = dtable.shape
    nn = index.numel()
    tokens = int(round(nn ** 0.5))
    assert dbias.numel() == heads * nn and dbias.dtype == dtable.dtype == torch.float32 and index.dtype == torch.int32
    check(lib().tch_relpos_bias_scatter(ctx.handle, _p(dbias), _p(index), _p(dtable), heads, tokens, entries,
                                        int(accumulate)), "tch_relpos_bias_scatter")


def relpos_bias_gather_pairs(ctx, table, index, bias):
    """bias[h, pair] = table[index[pair], h], -inf where index[pair] < 0 (padding)."""
    entries, heads = table.shape
    assert index.dtype == torch.int32 and bias.numel() == heads * index.numel()
    assert table.dtype == bias.dtype == torch.float32
    check(lib().tch_relpos_bias_gather_pairs(ctx.handle, _p(table), _p(index), _p(bias), heads, index.numel(), entries),
          "tch_relpos_bias_gather_pairs")


def relpos_bias_gather_batch(ctx, tables, indices, biases):
    """relpos_bias_gather_pairs for lists of tables / indices / bias tensors, eight tables per launch."""
    count = len(tables)
    assert count > 0 and len(indices) == len(biases) == count
    entries, pairs = tables[0].shape[0], indices[0].numel()
    for t, ix, b in zip(tables, indices, biases):
        assert t.shape[0] == entries and ix.numel() == pairs and ix.dtype == torch.int32
        assert t.dtype == b.dtype == torch.float32 and b.numel() == t.shape[1] * pairs
        assert t.is_contiguous() and ix.is_contiguous() and b.is_contiguous()
    ptrs = ctypes.c_void_p * count
    heads = (ctypes.c_int * count)(*[t.shape[1] for t in tables])
    check(lib().tch_relpos_bias_gather_batch(ctx.handle, ptrs(*[t.data_ptr() for t in tables]),
                                             ptrs(*[ix.data_ptr() for ix in indices]),
                                             ptrs(*[b.data_ptr() for b in biases]), heads, count, pairs, entries),
          "tch_relpos_bias_gather_batch")


def relpos_bias_scatter_pairs(ctx, dbias, index, dtable, accumulate=False):
    """dtable[entry, h] (+)= sum of dbias[h, pair] over the pairs with index[pair] == entry."""
    entries, heads = dtable.shape
    assert dbias.numel() == heads * index.numel() and dbias.dtype == dtable.dtype == torch.float32
    assert index.dtype == torch.int32
    check(lib().tch_relpos_bias_scatter_pairs(ctx.handle, _p(dbias), _p(index), _p(dtable), heads, index.numel(), entries,
                                              int(accumulate)), "tch_relpos_bias_scatter_pairs")


def relpos_inverse_index(index, entries):
    """(ptr [entries + 1], list) int32 on the CPU: list[ptr[e]:ptr[e + 1]] are the positions of `index` (any
    shape, negative = padding) that hold e, in ascending order."""
    flat = index.reshape(-1).to(torch.int64).cpu()
    pos = torch.nonzero(flat >= 0).reshape(-1)
    order = torch.argsort(flat[pos], stable=True)
    counts = torch.bincount(flat[pos], minlength=entries)
    assert counts.numel() == entries, "index refers to entries beyond the table"
    ptr = torch.zeros(entries + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(counts, 0)
    return ptr.to(torch.int32), pos[order].to(torch.int32)


def relpos_bias_scatter_csr(ctx, dbias, ptr, pair_list, dtable, pairs, accumulate=False):
    """dtable[e, h] (+)= sum of dbias[h, pair] over pair in list[ptr[e]:ptr[e + 1]] (relpos_inverse_index)."""
    entries, heads = dtable.shape
    assert dbias.numel() == heads * pairs and dbias.dtype == dtable.dtype == torch.float32
    assert ptr.dtype == pair_list.dtype == torch.int32 and ptr.numel() == entries + 1
    check(lib().tch_relpos_bias_scatter_csr(ctx.handle, _p(dbias), _p(ptr), _p(pair_list), _p(dtable), heads, pairs,
                                            entries, int(accumulate)), "tch_relpos_bias_scatter_csr")


def window_attn_fwd(ctx, qkv, o, probs, bias, mask, windows, heads, N, scale):
    """Window attention forward in one launch (bf16, heads 32 wide, N <= 64): qkv [windows * N, 3C] ->
    o [windows * N, C]; probs [windows * heads, N, 64] keeps the probabilities; bias [heads, 64, 64] fp32 with -inf
    from key column N on; mask [nW, 64, 64] fp32 or None."""
    C = heads * 32
    assert qkv.dtype == o.dtype == probs.dtype == torch.bfloat16 and bias.dtype == torch.float32
    assert qkv.numel() == windows * N * 3 * C and o.numel() == windows * N * C
    assert probs.numel() == windows * heads * N * 64 and bias.numel() == heads * 64 * 64
    nW = 1
    if mask is not None:
        assert mask.dtype == torch.float32 and mask.numel() % (64 * 64) == 0
        nW = mask.numel() // (64 * 64)
    check(lib().tch_window_attn_fwd(ctx.handle, dtype_code(qkv), _p(qkv), _p(o), _p(probs), _p(bias), _p(mask), windows,
                                    heads, N, C, nW, scale), "tch_window_attn_fwd")


def window_attn_bwd(ctx, qkv, probs, dout, dqkv, ds, windows, heads, N, scale):
    """Gradients of window_attn_fwd: dqkv like qkv, ds [windows * heads, N, 64] = gradient of the logits (its sum
    over the windows is the bias gradient in the padded pair layout)."""
    C = heads * 32
    assert qkv.dtype == probs.dtype == dout.dtype == dqkv.dtype == ds.dtype == torch.bfloat16
    assert qkv.numel() == dqkv.numel() == windows * N * 3 * C and dout.numel() == windows * N * C
    assert probs.numel() == ds.numel() == windows * heads * N * 64
    check(lib().tch_window_attn_bwd(ctx.handle, dtype_code(qkv), _p(qkv), _p(probs), _p(dout), _p(dqkv), _p(ds), windows,
                                    heads, N, C, scale), "tch_window_attn_bwd")


def column_sum_workspace_floats(rows, cols):
    return int(lib().tch_column_sum_workspace_floats(rows, cols))


def column_sum(ctx, x, out, workspace, accumulate=False):
    rows, cols = x.shape
    assert out.numel() == cols and out.dtype == workspace.dtype == torch.float32 and x.is_contiguous()
    assert workspace.numel() >= column_sum_workspace_floats(rows, cols)
    check(lib().tch_column_sum(ctx.handle, dtype_code(x), _p(x), _p(out), rows, cols, int(accumulate), _p(workspace)),
          "tch_column_sum")
