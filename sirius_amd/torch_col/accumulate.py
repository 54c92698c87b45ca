"""Gradient accumulation across the micro-batches of one global batch
(pytorch/torch_col/accumulate.py:8-51), over the engine's flat gradient buffers: one fused
`global += grad; grad = 0` launch instead of a Python loop over parameters."""
from typing import Optional


class GradAccumulator:
    def __init__(self, model):
        # the engine owns params / grads / momentum as flat fp32 buffers; the extra buffer the
        # reference allocates per parameter ('global') is one more flat buffer of the same size
        self.model = model
        model.ensure_global_grads()

    def accumulate(self):
        """global += p.grad; p.grad.zero_()  (accumulate.py:19-23)"""
        return self.model.accumulate()

    def step(self, optmizer=None, scaler=None, do_zero_grad=True):
        """Optimizer step on the accumulated gradients (accumulate.py:25-45).  `optmizer` (sic) and
        `scaler` keep the reference's signature: the engine's own SGD runs the step; a scaler is
        not needed because the bf16 path keeps fp32 master weights and fp32 gradients."""
        return self.model.optimizer_step(use_global=True, zero_global=do_zero_grad)

    def zero_grad(self):
        self.model.zero_global_grads()
