"""What every training-step engine of this package shares: the plan cache (one recorded program
per batch size), the checkpoints between launch segments, the flat gradient buffers with the
micro-batch accumulator, and the optimizer program.

A subclass provides
  * ``_build_plan(batch, loss_scale)`` -> an object with ``prog``, ``marks``, ``keep`` (the tensors the
    plan owns), ``loss`` (1-element fp32 tensor), ``bytes``;
  * the flat fp32 buffers ``params`` / ``grads`` of ``n_store`` elements;
  * ``_record_optimizer(grads)``: the launches of one optimizer step that consumes ``grads``.
"""
import torch

from . import ops


class EngineBase:
    def _init_engine(self, dtype, stream, allocator):
        if not torch.cuda.is_available():
            raise RuntimeError(f"{type(self).__name__} runs on the GPU only; there is no CPU path")
        assert dtype in (torch.bfloat16, torch.float32)
        self.dtype = dtype
        self.dev = torch.device("cuda", torch.cuda.current_device())
        self.ctx = ops.Context(stream if stream is not None else torch.cuda.current_stream())
        # allocator(shape, dtype) -> uninitialised device tensor; the shared HBM pool plugs in here
        # (torch_col.pool_empty), torch's own allocator is the default
        self._alloc = allocator if allocator is not None else (
            lambda shape, dtype: torch.empty(shape, dtype=dtype, device=self.dev))
        self._hook = None
        self._cut_exception = None
        self._plans = {}
        self._last_plan = None
        self._opt_prog = None
        self._acc_prog = None
        self._opt_global_prog = None
        self.global_grads = None

    def plan(self, batch, loss_scale=1.0):
        key = (int(batch), float(loss_scale))
        p = self._plans.get(key)
        if p is None:
            # plans of other batch sizes own activation memory: drop them first
            for k in [k for k in self._plans if k[0] != key[0]]:
                del self._plans[k]
            p = self._plans[key] = self._build_plan(*key)
        return p

    def release_activations(self):
        """Drop every plan (and with it all activation / gradient-scratch memory)."""
        n = sum(p.bytes for p in self._plans.values())
        # an exception in flight may still hold a plan through its traceback: with an allocator
        # that can release a block under a live tensor, give the memory back now
        release = getattr(self._alloc, "release", None)
        if release is not None:
            self.ctx.synchronize()
            for p in self._plans.values():
                for t in p.keep:
                    release(t)
                p.keep = []
        self._plans.clear()
        self._last_plan = None
        return n

    def last_loss(self):
        """Mean loss of the most recent micro-batch (nan once its plan has been released)."""
        p = getattr(self, "_last_plan", None)
        if p is None or not p.keep:
            return float("nan")
        self.ctx.synchronize()
        return float(p.loss.item())

    def set_checkpoint_hook(self, fn):
        """fn(phase, layer name) runs between the launch segments of forward_backward, once per
        layer and direction: the place of the forward / backward module hooks of the reference
        (torch_col/colocate_ctrl.py:360-402).  An exception raised by fn ends the step there."""
        self._hook = fn

    def set_cut_exception(self, exc_type):
        """Raise exc_type from forward_backward when the reject flag cut the replay short (the
        control thread killed the batch on receipt of a request): what the reference's autograd
        engine hook does with EngineColocateAdjustL1Exception (csrc/mem_tagging.cc:54-58)."""
        self._cut_exception = exc_type

    def set_cu_share_provider(self, fn):
        """fn() -> compute units training may use right now (0 = all); asked before every launch segment,
        as the reference sets the TPC mask of the training stream before each launch
        (common/sm_partition.cc:108-112)."""
        self._cu_share = fn

    def _apply_cu_share(self):
        fn = getattr(self, "_cu_share", None)
        if fn is not None:
            self.ctx.set_cu_limit(fn())

    def _run_plan(self, p):
        self._apply_cu_share()
        if self._hook is None:
            cut = self.ctx.run(p.prog)
        else:
            first, cut = 0, False
            for idx, phase, name in p.marks:
                cut = self.ctx.run(p.prog, first, idx) or cut
                first = idx
                self._hook(phase, name)
                self._apply_cu_share()
                if cut and self._cut_exception is not None:
                    break
            if first < len(p.prog) and not (cut and self._cut_exception is not None):
                cut = self.ctx.run(p.prog, first, len(p.prog)) or cut
        if cut and self._cut_exception is not None:
            raise self._cut_exception("launches rejected: batch killed on request")
        return cut

    def _flat_prog(self, fn):
        prog = ops.Program()
        self.ctx.begin_record(prog)
        try:
            fn()
        finally:
            self.ctx.end_record()
        return prog

    # ------------------------------------------------------------------ tiling choice by measurement
    def _time_program(self, fn, reps=3):
        """Best-of-`reps` milliseconds of the launches `fn` records, replayed alone on this engine's stream."""
        prog = self._flat_prog(fn)
        self.ctx.run(prog)
        self.ctx.synchronize()
        best = float("inf")
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(self.ctx.stream)
            self.ctx.run(prog)
            # behind a launch queue the launches reach the stream from the queue's own thread: the closing event
            # must not overtake them
            self.ctx.flush()
            e1.record(self.ctx.stream)
            e1.synchronize()
            best = min(best, e0.elapsed_time(e1))
        return best

    def _scratch(self, shape, dtype, fill=0.0):
        """A filled tensor from this engine's allocator, for measurements made while a plan is built."""
        return self._alloc(tuple(shape), dtype).fill_(fill)

    def ensure_global_grads(self):
        if self.global_grads is None:
            self.global_grads = self._alloc((self.n_store,), torch.float32).zero_()

    def zero_global_grads(self):
        if self.global_grads is not None:
            ops.fill_zero(self.ctx, self.global_grads)

    def synchronize(self):
        self.ctx.synchronize()

    def zero_grad(self):
        ops.fill_zero(self.ctx, self.grads)

    def discard_partial_grads(self):
        """After a killed micro-batch: its gradients are partial.  Every backward overwrites the
        whole gradient buffer, so zeroing is only for the reader of grads_dict()."""
        ops.fill_zero(self.ctx, self.grads)

    def accumulate(self):
        """global += grads; grads = 0   (GradAccumulator.accumulate)"""
        self.ensure_global_grads()
        if self._acc_prog is None:
            self._acc_prog = self._flat_prog(lambda: ops.grad_accumulate(self.ctx, self.global_grads, self.grads))
        return self.ctx.run(self._acc_prog)

    def optimizer_step(self, use_global=False, zero_global=True):
        """One optimizer step over the flat buffers; with use_global the accumulated gradients are
        consumed and zeroed (GradAccumulator.step)."""
        if use_global:
            if self.global_grads is None:
                raise RuntimeError("optimizer_step(use_global=True) before any accumulate()")
            if self._opt_global_prog is None:
                self._opt_global_prog = self._flat_prog(lambda: self._record_optimizer(self.global_grads))
            cut = self.ctx.run(self._opt_global_prog)
            if zero_global:
                ops.fill_zero(self.ctx, self.global_grads)
            return cut
        if self._opt_prog is None:
            self._opt_prog = self._flat_prog(lambda: self._record_optimizer(self.grads))
        return self.ctx.run(self._opt_prog)
