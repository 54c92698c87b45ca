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


class PoolModel:
    """Independent model of where the training allocator places blocks and which physical pages back them.

    Configuration as the reference gives it to the allocator it delegates to (common/cuda_allocator.cc:61-85):
    32 MB pages (`PageNbytes`, cuda_allocator.h:81-87), small-block threshold = page / 16 = 2 MB, 1024-byte
    alignment, virtual range 8x the pool; zero-byte requests are null (cuda_allocator.cc:129-132);
    `FreeTrainLocals` = empty the cache (cuda_allocator.cc:304-307); page states train-local-free -> free <->
    infer, free -> train (cuda_allocator.h:48-58).  The allocator itself (third_party/mpool) is not in the
    reference tree, so the policy inside those constants is THIS BUILD'S and is stated here in full -- parity with
    mpool's own tie-breaking is unpinned; what this model pins is that the C++ pool (CPU backend and HIP
    virtual-memory backend alike) follows the stated policy offset for offset and page for page:

    * two segments of the range: [0, range/8 rounded up to a page) for requests < 2 MB after rounding to 1024,
      the rest for the others; each grows at its end, in whole pages;
    * a request takes the smallest free block that fits (lowest offset among equals); if none fits the segment
      grows, extending a trailing free block rather than leaving it behind; the block is split when at least
      one alignment unit remains;
    * a freed block merges with free neighbours and keeps its pages; empty_cache() returns every page that
      lies wholly inside free blocks;
    * a block is backed page by page: a slot that still carries the (stale, lazy mode) mapping of a page
      nobody took gets that page back; otherwise the lowest-numbered free page that carries no stale mapping,
      and only then the lowest-numbered one that does;
    * a request that finds too few free pages empties the cache first and fails (leaving the block free and
      merged) if that is not enough.

    Written with plain lists and linear scans on purpose (the C++ uses ordered maps and a size index): a shared
    data-structure mistake cannot hide in both.
    """
    ALIGN = 1024
    FREE, TRAIN, INFER = 0, 1, 2

    def __init__(self, pool_bytes, page_bytes=32 << 20, lazy_unmap=False):
        self.page = page_bytes
        self.small_limit_bytes = 2 << 20      # the reference's page / 16 at ITS page size; kept when the page size is a parameter
        self.n_pages = pool_bytes // page_bytes
        va = self.n_pages * page_bytes * 8
        small = -(-(va // 8) // page_bytes) * page_bytes
        # segment: [begin, limit), frontier, blocks = list of [offset, size, allocated] in address order
        self.segs = [dict(begin=0, limit=small, frontier=0, blocks=[]),
                     dict(begin=small, limit=va, frontier=small, blocks=[])]
        self.owner = [self.FREE] * self.n_pages
        self.slot_page = {}      # slot -> page mapped there (live or stale)
        self.slot_live = set()   # slots whose page training owns
        self.lazy = lazy_unmap
        self.train_usage = 0
        self.maps = self.unmaps = self.revives = 0

    # -- pages ---------------------------------------------------------------------------------------
    def free_pages(self):
        return sum(1 for o in self.owner if o == self.FREE)

    def train_pages(self):
        return sum(1 for o in self.owner if o == self.TRAIN)

    def _stale_pages(self):
        return {p for s, p in self.slot_page.items() if s not in self.slot_live}

    def _take_free_page(self):
        stale = self._stale_pages()
        free = [i for i, o in enumerate(self.owner) if o == self.FREE]
        clean = [i for i in free if i not in stale]
        if clean:
            return clean[0]
        if not free:
            return None
        page = free[0]
        slot = next(s for s, p in self.slot_page.items() if p == page)
        del self.slot_page[slot]
        self.unmaps += 1
        return page

    def _back(self, off, size):
        slots = range(off // self.page, (off + size - 1) // self.page + 1)
        if all(s in self.slot_live for s in slots):
            return True
        for s in slots:     # a stale mapping whose page is still free comes back as it is
            if s in self.slot_page and s not in self.slot_live and self.owner[self.slot_page[s]] == self.FREE:
                self.owner[self.slot_page[s]] = self.TRAIN
                self.slot_live.add(s)
                self.revives += 1
        missing = [s for s in slots if s not in self.slot_live]
        if not missing:
            return True
        if self.free_pages() < len(missing):
            self.empty_cache()
            missing = [s for s in slots if s not in self.slot_live]
            if self.free_pages() < len(missing):
                return False
        for s in missing:
            if s in self.slot_page:          # stale mapping of a page that went elsewhere
                del self.slot_page[s]
                self.unmaps += 1
            page = self._take_free_page()
            self.owner[page] = self.TRAIN
            self.slot_page[s] = page
            self.slot_live.add(s)
            self.maps += 1
        return True

    # -- blocks --------------------------------------------------------------------------------------
    def _seg_of(self, off):
        return self.segs[0] if off < self.segs[0]["limit"] else self.segs[1]

    def _merge_free(self, seg, i):
        b = seg["blocks"]
        if i + 1 < len(b) and not b[i + 1][2]:
            b[i][1] += b[i + 1][1]
            del b[i + 1]
        if i > 0 and not b[i - 1][2]:
            b[i - 1][1] += b[i][1]
            del b[i]

    def alloc(self, nbytes):
        """Offset of the block, or None (zero bytes, out of range, out of pages)."""
        if nbytes == 0:
            return None
        n = -(-nbytes // self.ALIGN) * self.ALIGN
        seg = self.segs[0] if n < self.small_limit_bytes else self.segs[1]
        b = seg["blocks"]
        fits = [(blk[1], blk[0], i) for i, blk in enumerate(b) if not blk[2] and blk[1] >= n]
        if fits:
            i = min(fits)[2]
        else:
            start = seg["frontier"]
            if b and not b[-1][2]:
                start = b[-1][0]
            frontier = -(-(start + n) // self.page) * self.page
            if frontier > seg["limit"]:
                return None
            if b and not b[-1][2]:
                b.pop()
            b.append([start, frontier - start, False])
            seg["frontier"] = frontier
            i = len(b) - 1
        if b[i][1] - n >= self.ALIGN:
            b.insert(i + 1, [b[i][0] + n, b[i][1] - n, False])
            b[i][1] = n
        if not self._back(b[i][0], b[i][1]):
            # empty_cache inside _back may have changed nothing about the blocks; the block stays free, merged
            self._merge_free(seg, i)
            return None
        b[i][2] = True
        self.train_usage += n
        return b[i][0]

    def free(self, off):
        seg = self._seg_of(off)
        i = next(k for k, blk in enumerate(seg["blocks"]) if blk[0] == off and blk[2])
        seg["blocks"][i][2] = False
        self.train_usage -= seg["blocks"][i][1]
        self._merge_free(seg, i)

    def empty_cache(self):
        """Bytes of pages handed back."""
        slots = []
        for seg in self.segs:
            for off, size, allocated in seg["blocks"]:
                if allocated:
                    continue
                lo = -(-off // self.page)
                hi = (off + size) // self.page
                slots += [s for s in range(lo, hi) if s in self.slot_live]
        for s in slots:
            self.owner[self.slot_page[s]] = self.FREE
            self.slot_live.discard(s)
            if not self.lazy:
                del self.slot_page[s]
                self.unmaps += 1
        return len(slots) * self.page

    # -- the other tenant ----------------------------------------------------------------------------
    def infer_claim(self, n):
        moved = 0
        for i in range(self.n_pages):
            if moved == n:
                break
            if self.owner[i] == self.FREE:
                self.owner[i] = self.INFER
                moved += 1
        return moved

    def infer_release(self, n):
        moved = 0
        for i in range(self.n_pages - 1, -1, -1):
            if moved == n:
                break
            if self.owner[i] == self.INFER:
                self.owner[i] = self.FREE
                moved += 1
        return moved
