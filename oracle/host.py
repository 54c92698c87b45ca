"""Pure-Python restatements of the plugin's integer / closed-form bookkeeping.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py): the C++ host runtime is checked against these,
they are never on the product path.

Pins: the reference's tests hold no expectations for any of these (parity unpinned by the
reference); each restatement is the published rule of the cited lines, and the tests check the
product against it on random walks plus hand-evaluated cases.
"""
import math


class DistributorModel:
    """Single-rank view of DynamicBatchDistirbutor (pytorch/torch_col/csrc/dynamic_batch.cc):
    an ordered set of unprocessed sample ranges; GetBatch takes from the lowest index and slices
    the last range it touches (:352-383); the batch that empties the unprocessed set is the one
    that steps (:396-398); AbortBatch puts the ranges back as they are, neighbours are never
    merged (:533-563); FinishBatch moves them to the processed set (:470-500)."""

    def __init__(self, lo, hi):
        self.unproc = [(lo, hi)] if hi > lo else []
        self.procing, self.proced = [], []

    def query(self, bs):
        return min(bs, sum(b - a for a, b in self.unproc))

    def get(self, bs):
        out, need = [], bs
        while need > 0 and self.unproc:
            a, b = self.unproc[0]
            take = min(need, b - a)
            out.append((a, a + take))
            need -= take
            if a + take == b:
                self.unproc.pop(0)
            else:
                self.unproc[0] = (a + take, b)
        self.procing += out
        return out, not self.unproc

    def finish(self, r):
        for x in r:
            self.procing.remove(x)
        self.proced = sorted(self.proced + list(r))

    def abort(self, r):
        for x in r:
            self.procing.remove(x)
        self.unproc = sorted(self.unproc + list(r))


def split_global_batch(n, world, policy="fix", ratios=None):
    """How many samples of a global batch of n each rank gets (dynamic_batch.cc:254-314).
    fix / simple: q = n // W, the first n % W ranks one more (:262-275).
    by_performance: max(1, int(n * ratio_i)), then +-1 round-robin until the sum is n (:277-312)."""
    if policy in ("fix", "simple") or not ratios:
        q, r = divmod(n, world)
        return [q + (1 if i < r else 0) for i in range(world)]
    total = sum(ratios)
    out = [max(1, int(n * x / total)) for x in ratios]
    i = 0
    while sum(out) != n:
        if sum(out) < n:
            out[i % world] += 1
        elif out[i % world] > 1:
            out[i % world] -= 1
        i += 1
    return out


def num_global_batches(dataset_size, global_batch_size):
    """ceil(ds / gbs) (dynamic_batch.cc:79-80); the last one is cut to ds - done (:668-671)."""
    return (dataset_size + global_batch_size - 1) // global_batch_size


class PerfModelOracle:
    """csrc/perf_model.cc:25-94: thpt = bs / ms, running mean per batch size; lookup: empty -> -1,
    bs <= 0 -> 0, outside the recorded range proportional to the nearest key, else linear
    interpolation between the neighbouring keys."""

    def __init__(self):
        self.m = {}

    def record(self, bs, ms):
        if bs <= 0 or ms <= 0:
            return
        mean, n = self.m.get(bs, (0.0, 0))
        self.m[bs] = ((mean * n + bs / ms) / (n + 1), n + 1)

    def get(self, bs):
        if not self.m:
            return -1.0
        if bs <= 0:
            return 0.0
        keys = sorted(self.m)
        if bs <= keys[0]:
            return self.m[keys[0]][0] / keys[0] * bs
        if bs >= keys[-1]:
            return self.m[keys[-1]][0] / keys[-1] * bs
        hi = next(k for k in keys if k >= bs)
        if hi == bs:
            return self.m[hi][0]
        lo = max(k for k in keys if k < bs)
        t0, t1 = self.m[lo][0], self.m[hi][0]
        return (t1 - t0) / (hi - lo) * (bs - lo) + t0


# ---- the inference side's adjust arithmetic (server/train_adjuster.cc) ----

# (base MB, slope MB per sample) with shared tensors (:647-698) / without (:699-734)
MODEL_MEM_PARAM_SHARED = {"resnet152": (1150, 85), "swin_b": (1700, 145), "swin_b_ddp": (2560, 140),
                          "gpt2": (2700, 490), "qwen": (9000, 600)}
MODEL_MEM_PARAM_PLAIN = {"resnet152": (2396, 85), "swin_b": (3000, 200), "swin_b_ddp": (3800, 200),
                         "qwen": (9000, 600)}


def predict_train_mem_usage_mb(base, slope, batch_size):
    """train_adjuster.cc:69-80: base for bs <= 0, else base + slope * bs."""
    return base if batch_size <= 0 else base + slope * batch_size


def predict_target_batch_size(base, slope, memory_mb, init_batch_size):
    """train_adjuster.cc:521-533: clamp(int((MB - base) / slope), 0, init_bs)."""
    return max(0, min(int((memory_mb - base) / slope), init_batch_size))


def delta_batch_size(slope, memory_mb):
    """train_adjuster.cc:535-538: ceil(MB / slope)."""
    return int(math.ceil(memory_mb / slope))


def infer_require_mem_target(cur_target_bs, required_mem_mb, slope, min_train_bs=0, num_gpus=1):
    """train_adjuster.cc:97-145: nothing to do when already at the limit or nothing is required;
    else target = cur - ceil(MB / slope), floored at the limit on multi-GPU hosts only (on one GPU
    it may go to zero or below: training then waits for a valid batch size)."""
    if cur_target_bs <= min_train_bs or required_mem_mb <= 0:
        return None
    t = cur_target_bs - delta_batch_size(slope, required_mem_mb)
    if num_gpus > 1:
        t = max(t, min_train_bs)
    return t
