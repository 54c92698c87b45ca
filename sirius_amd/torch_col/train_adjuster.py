"""The inference side's adjust arithmetic, for a stand-in peer that asks for memory in megabytes
the way the real server does (server/train_adjuster.cc:69-145,521-538,642-736): memory <-> batch
size through a linear model `MB = base + slope * batch_size` per training model.

`MODEL_MEM_PARAM` keeps the reference's table (fitted on its GPUs with fp16 autocast);
`MODEL_MEM_PARAM_MI355X` is re-fitted for this engine from pool readings on MI355X.
"""
import math

from . import _C

# (base MB, slope MB / sample), shared-tensor mode (train_adjuster.cc:647-698)
MODEL_MEM_PARAM = {"resnet152": (1150, 85), "swin_b": (1700, 145), "swin_b_ddp": (2560, 140),
                   "gpt2": (2700, 490), "qwen": (9000, 600)}
# This engine on MI355X, bf16 compute with fp32 master state, from pool readings (bytes held by torch before any
# plan exists, and the bytes of the plans at three batch sizes; the plan grows linearly, its intercept is < 30 MB):
#   resnet152  state 920 MB (+ 241 MB of accumulated gradients in colocate mode), plans 1109 / 2190 / 8673 MB at
#              batch 8 / 16 / 64
#   swin_b     state 1675 MB (+ 351 MB), plans 544 / 1083 / 4200 MB at batch 4 / 8 / 32
#   gpt2       state 2375 MB (+ 498 MB); 256-token rows as train/gpt2.py:45 builds them: plans 1306 / 2585 / 10258 MB
#              at batch 8 / 16 / 64 (1024-token rows: 640 MB per row)
# base = state + accumulated gradients + the plan's intercept, slope = plan bytes per sample.
MODEL_MEM_PARAM_MI355X = {"resnet152": (1190, 136), "swin_b": (2050, 131), "gpt2": (2900, 160)}


class TrainAdjuster:
    def __init__(self, model_name=None, table=None, min_train_bs=0):
        self.table = dict(MODEL_MEM_PARAM if table is None else table)
        self.model_name = model_name
        self.min_train_bs = min_train_bs

    def get_model_mem_param(self):
        name = self.model_name or _C.get_train_info_model_name(0)
        if name not in self.table:
            raise KeyError(f"Unsupported model: {name}")
        return self.table[name]

    def predict_train_mem_usage_mb(self, batch_size):
        base, slope = self.get_model_mem_param()
        return base if batch_size <= 0 else base + slope * batch_size

    def predict_target_batch_size(self, memory_mb):
        base, slope = self.get_model_mem_param()
        init_bs = _C.get_train_info(0, "init_batch_size")
        return max(0, min(int((memory_mb - base) / slope), init_bs))

    def get_delta_batch_size(self, memory_mb):
        _, slope = self.get_model_mem_param()
        return int(math.ceil(memory_mb / slope))

    def infer_require_mem_adjust_plan(self, required_mem_mb):
        """Target batch size after inference asked for required_mem_mb, or None when nothing is
        to be done (already at the limit, or nothing required).  One training rank."""
        cur = _C.get_train_info(0, "target_batch_size_unpublished")
        if cur <= self.min_train_bs or required_mem_mb <= 0:
            return None
        return cur - self.get_delta_batch_size(required_mem_mb)

    def infer_release_mem_adjust_plan(self, avail_mem_mb):
        """Target batch size when inference gives memory back: what fits into avail_mem_mb,
        never more than the initial batch size."""
        return self.predict_target_batch_size(avail_mem_mb)
