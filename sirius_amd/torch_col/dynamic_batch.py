"""The dataset whose batch size follows inference's demand, and the bookkeeping of micro-batches inside a global
batch.  Class / function names, `Batch` keys, event names (`batch_EE_BBB_SS`, `global_batch_...`,
`optimizer_step`, `wait_valid_batch`) and tags (`finish`, `cancel`, `global`, `local`) are the reference's
(pytorch/torch_col/dynamic_batch.py:27-625); sample ranges come from the C++ distributor; the optimizer step
is the engine's fused kernel, so "optimizer" below is the engine itself.

Layout of this module:
  _HostSamples        the synthetic samples, resident in pinned host memory, gathered by ring index
  _Span               one open event of the profile (begin ... end with a tag)
  _GlobalBatchLedger  which sample ranges the current global batch has consumed so far, and what the
                      distributor must be told when a micro-batch finishes, is cut, or the whole global batch is
                      rolled back
  MicroBatchManager   the reference's facade over the ledger + the optimizer step in its critical section
  DynamicBatchDataset the iterator that sizes every micro-batch by the controller's current target
"""
from __future__ import annotations

import contextlib
import dataclasses
import os
import sys
import time
from enum import Enum, IntEnum
from typing import Iterator, List, Optional, Tuple, Union

import torch

from . import _C, dist
from ._C import CtrlEvent, TrainMode
from .colocate_ctrl import CtrlBase, get_colocate_ctrl
from .dist import _DynamicBatchDistirbutor as _Distributor
from .dist import _PerfModel
from .util import EventManager, MemoryPool

_BATCH_FINISH_TAG = 'finish'
_BATCH_CANCEL_TAG = 'cancel'

RangeVec = List[Tuple[int, int]]


class BatchDistributePolicy(Enum):
    FIX = 'fix'
    SIMPLE = 'simple'
    BY_PERFORMANCE = 'by_performance'


class DatasetType(IntEnum):
    VISION = 0
    TEXT_GEN = 1
    TEXT_CLS = 2
    DYNAMIC_BATCH = 3


class DatasetState(IntEnum):
    INIT = 0
    ITER = 1
    NEXT = 2


@dataclasses.dataclass
class VisionDatasetConfig:
    input_shape: tuple
    num_class: int


@dataclasses.dataclass
class TextDatasetConfig:
    seq_len: int


def _num_sample_of_batch_range_vec(batch_range_vec: RangeVec) -> int:
    return sum(hi - lo for lo, hi in batch_range_vec)


def _num_sample_of_batch_range(batch_range) -> int:
    """One (lo, hi) pair, or -- as the reference's callers pass it -- a whole vector of them."""
    if batch_range and isinstance(batch_range[0], (tuple, list)):
        return _num_sample_of_batch_range_vec(batch_range)
    return batch_range[1] - batch_range[0]


class Batch(dict):
    """What `iter_train_fn` receives: the input tensors on the device, plus 'range' (the sample ranges) and
    'do_step' (this micro-batch closes its global batch)."""

    def __init__(self, inputs: Optional[dict] = None):
        super().__init__(inputs or {})

    def should_update_param(self):
        return self.get('do_step', True)

    def get_range(self) -> RangeVec:
        return self['range']

    def __len__(self) -> int:
        return DynamicBatchDataset._dynamic_batch_dataset.get_batch_size(self)


# ----------------------------------------------------------------------------------------------------------------
def _hand_over_queued_launches(stream):
    """Wait until the preemptible launch queue of `stream` (if it has one) holds nothing that has not reached the
    stream yet.  Does not wait for the GPU."""
    import time
    from .._lib import lib
    handle = stream.cuda_stream
    while lib().tch_GetXQueueSize(handle):
        time.sleep(0)


class _HostSamples:
    """`resident` rows per input tensor in pinned host memory; sample i of the dataset is row i % resident
    (the reference's ring repeat, dynamic_batch.py:449-454), so a small resident set stands for a dataset of
    any size."""

    def __init__(self, tensors: dict, pinned: bool):
        self.tensors = {k: (t.pin_memory() if pinned else t) for k, t in tensors.items()}
        self.resident = len(next(iter(self.tensors.values())))
        self.pinned = pinned
        self.prefetch = os.environ.get('COLTRAIN_PREFETCH_BATCH', '1') != '0'
        self._copy_stream = None
        self._ahead = None      # (first row, rows, device tensors, copy-done event) of the guessed next batch

    def rows_of(self, range_vec: RangeVec) -> torch.Tensor:
        return torch.cat([torch.arange(lo, hi) for lo, hi in range_vec]) % self.resident if range_vec \
            else torch.empty(0, dtype=torch.long)

    def _copy_run(self, first: int, n: int, device, copy_stream=None) -> dict:
        """Rows [first, first + n) on the device.  The tensors are always allocated on the CURRENT (training) stream,
        which is the stream that will read them: the allocator then orders their reuse against that stream.  With a
        copy stream the copy alone is issued there, and the copy stream is recorded as a second user."""
        out = {}
        for key, src in self.tensors.items():
            dst = torch.empty((n, *src.shape[1:]), dtype=src.dtype, device=device)
            if copy_stream is None:
                dst.copy_(src[first:first + n], non_blocking=True)
            else:
                with torch.cuda.stream(copy_stream):
                    dst.copy_(src[first:first + n], non_blocking=True)
                dst.record_stream(copy_stream)
            out[key] = dst
        return out

    def _prefetch(self, first: int, n: int, device):
        """Start copying rows [first, first + n) on the copy stream: the guess for the next micro-batch (the run
        that follows this one, same size).  The destination is allocated on the training stream; the copy stream
        first waits for everything the training stream has been given -- including launches that still sit in the
        stream's preemptible launch queue, which are handed over first (a stream wait only covers what is ON the
        stream) -- so memory the allocator hands out again is not still in use by a cut or killed batch; the copy
        then runs beside the micro-batch that is launched next."""
        if self._copy_stream is None:
            self._copy_stream = torch.cuda.Stream(device=device)
        train_stream = torch.cuda.current_stream(device)
        _hand_over_queued_launches(train_stream)
        self._copy_stream.wait_stream(train_stream)
        tensors = self._copy_run(first, n, device, copy_stream=self._copy_stream)
        done = torch.cuda.Event()
        done.record(self._copy_stream)
        self._ahead = (first, n, tensors, done)

    def drop_prefetched(self):
        """Give the guessed batch's memory back (before memory is handed to inference)."""
        if self._ahead is not None:
            self._ahead[3].synchronize()
            self._ahead = None

    def to_device(self, range_vec: RangeVec, device) -> dict:
        rows = self.rows_of(range_vec)
        n = rows.numel()
        # one ascending run is a slice of the pinned tensor: a single asynchronous copy, no gather on the host
        run = n > 0 and int(rows[-1]) - int(rows[0]) == n - 1 and bool((rows[1:] > rows[:-1]).all())
        on_gpu = self.pinned and str(device).startswith('cuda')
        ahead, self._ahead = self._ahead, None
        if run and ahead is not None and ahead[:2] == (int(rows[0]), n):
            torch.cuda.current_stream(device).wait_event(ahead[3])
            out = ahead[2]
        elif run:
            if ahead is not None:
                ahead[3].synchronize()
            out = self._copy_run(int(rows[0]), n, device)
        else:
            if ahead is not None:
                ahead[3].synchronize()
            out = {}
            for key, src in self.tensors.items():
                dst = torch.empty((n, *src.shape[1:]), dtype=src.dtype, device=device)
                if n:
                    dst.copy_(src.index_select(0, rows))
                out[key] = dst
        if run and on_gpu and self.prefetch:
            follow = (int(rows[-1]) + 1) % self.resident
            if follow + n <= self.resident:
                self._prefetch(follow, n, device)
        return out


class _Span:
    """An event that is open: `end(tag)` stamps its duration and tag into the profile."""

    def __init__(self, name: str):
        self.event = EventManager.record_event(name)

    def end(self, tag: Optional[str] = None):
        if tag is not None:
            self.event.tag = tag
        EventManager.record_event('', self.event)
        return self.event


class _GlobalBatchLedger:
    """Sample ranges of the global batch in progress.

    Three regimes decide when the distributor hears that samples are done:
      * no accumulation, or accumulation with a checkpoint per micro-batch (the accumulated gradient survives a
        cut): every finished micro-batch is final at once;
      * a train mode that never kills a batch: likewise;
      * accumulation WITHOUT checkpoints in a mode that kills batches: nothing is final until the micro-batch
        that steps has finished -- a cut anywhere rolls the whole global batch back, so the ranges are kept
        and reported together at the end."""

    def __init__(self, accumulate: bool, checkpoint: bool):
        self.accumulate, self.checkpoint = accumulate, checkpoint
        self.done: List[RangeVec] = []
        self.current: Optional[RangeVec] = None

    def _final_at_once(self) -> bool:
        return (not self.accumulate) or self.checkpoint or not _C.get_colocate_train_mode().is_kill_batch()

    def open(self, range_vec: RangeVec):
        self.current = range_vec

    def micro_batch_finished(self, batch: Batch):
        self.done.append(self.current)
        if self._final_at_once():
            _Distributor.finish_batch(batch.get_range(), batch.should_update_param())
        self.current = None

    def global_batch_finished(self):
        if not self._final_at_once():
            for k, range_vec in enumerate(self.done):
                _Distributor.finish_batch(range_vec, k == len(self.done) - 1)
        self.done = []
        _Distributor.next_global_batch()

    def micro_batch_cut(self, batch: Batch) -> int:
        """Returns how many samples went back beyond the cut micro-batch itself (a rollback)."""
        rolled_back = 0
        if self.accumulate and not self.checkpoint:
            for range_vec in self.done:
                rolled_back += _num_sample_of_batch_range_vec(range_vec)
                _Distributor.abort_batch(range_vec, False)
            rolled_back += _num_sample_of_batch_range_vec(self.current)
            self.done = []
        _Distributor.abort_batch(self.current, batch.should_update_param())
        self.current = None
        return rolled_back

    @property
    def rolls_back(self) -> bool:
        return self.accumulate and not self.checkpoint


class MicroBatchManager:
    """dynamic_batch.py:87-310"""
    _micro_batch_manager: Optional[MicroBatchManager] = None

    def __init__(self, dynamic_dataset: DynamicBatchDataset, enable_grad_accumulate: bool = False,
                 checkpoint_micro_batch: bool = False):
        assert MicroBatchManager._micro_batch_manager is None
        MicroBatchManager._micro_batch_manager = self
        self._dynamic_dataset = dynamic_dataset
        self._enable_grad_accumulate = enable_grad_accumulate
        self._checkpoint_micro_batch = checkpoint_micro_batch
        self._ledger = _GlobalBatchLedger(enable_grad_accumulate, checkpoint_micro_batch)
        self._batch_span: Optional[_Span] = None
        self._global_span: Optional[_Span] = None

    # ---- loss scaling: a micro-batch contributes its share of the global batch's mean ----
    def loss_scale(self, batch: Batch) -> float:
        """The factor `scale_loss` applies, for engines that fold it into the loss kernel."""
        if not self._enable_grad_accumulate:
            return 1.0
        return self._dynamic_dataset.get_batch_size(batch) / _Distributor.get_global_batch_size()

    def scale_loss(self, batch: Batch, loss):
        """loss /= global_batch_size / batch_size  (dynamic_batch.py:112-120)"""
        return loss * self.loss_scale(batch) if self._enable_grad_accumulate else loss

    # ---- the optimizer step, never cut ----
    def optimizer_step(self, batch: Batch, optimizer, amp_scaler=None, grad_accumulator=None):
        """dynamic_batch.py:122-153.  With a checkpoint per micro-batch the gradients are accumulated every time
        and the step runs on the micro-batch that closes the global batch; otherwise the engine steps on its own
        gradient buffer whenever parameters are due."""
        checkpointing = self._should_checkpoint_micro_batch()
        if not checkpointing and self._enable_grad_accumulate and not batch.should_update_param():
            return
        if checkpointing:
            assert grad_accumulator is not None
        with get_colocate_ctrl().steps_no_interrupt():
            span = _Span('optimizer_step')
            if checkpointing:
                grad_accumulator.accumulate()
                stepping = batch.should_update_param()
                if stepping:
                    grad_accumulator.step(optimizer, amp_scaler)
                span.end('global' if stepping else 'local')
            else:
                optimizer.optimizer_step(use_global=False)
                optimizer.zero_grad()
                span.end()

    @contextlib.contextmanager
    def ddp_sync_context(self, model, batch: Batch):
        """One GPU: there is no gradient exchange to hold back (dynamic_batch.py:155-167)."""
        yield

    # ---- life of a micro-batch ----
    def begin_batch(self, epoch_idx: int, batch_idx: int, batch: Batch, batch_range_vec):
        self._ledger.open(batch_range_vec)
        size = len(batch)
        self._batch_span = _Span(f'batch_{epoch_idx:02d}_{batch_idx:03d}_{size:02d}')
        if self._enable_grad_accumulate and self._global_span is None:
            self._global_span = _Span(
                f'global_batch_{epoch_idx:02d}_{batch_idx:03d}_{_Distributor.get_global_batch_size():02d}')

    def finish_batch(self, epoch_idx: int, batch_idx: int, batch: Batch):
        # what still sits in a software launch queue is not on the stream yet: queues first, then the stream
        _C.SyncAllStreams()
        if torch.cuda.is_available():
            torch.cuda.current_stream().synchronize()
        self._serve_adjust_l2(batch)
        event = self._batch_span.end(_BATCH_FINISH_TAG)
        self._batch_span = None
        if _C.get_train_rank() == 0:
            _PerfModel.record_thpt(len(batch), event.duration)
        self._ledger.micro_batch_finished(batch)
        if batch.should_update_param():
            if self._global_span is not None:
                self._global_span.end(_BATCH_FINISH_TAG)
                self._global_span = None
            self._ledger.global_batch_finished()
        self._dynamic_dataset._next_batch()

    def _serve_adjust_l2(self, batch: Batch):
        """colocate-l2 answers at the end of a micro-batch, when nothing is in flight."""
        ctrl = get_colocate_ctrl()
        if ctrl.train_mode != TrainMode.COLOCATE_L2 or ctrl._stub.cmd != CtrlEvent.kColocateAdjustL2:
            return
        if _C.get_train_world_size() == 1:
            ctrl.release_and_reply(False)
            if not batch.should_update_param():   # the rest of the global batch is re-split at the new size
                _Distributor.distribute_batch(True, True, False)
        elif batch.should_update_param():
            dist.wait_barrier()
            ctrl.release_and_reply(False)

    def abort_batch(self, epoch_idx: int, batch_idx: int, batch: Batch):
        self._batch_span.end(_BATCH_CANCEL_TAG)
        self._batch_span = None
        if self._ledger.rolls_back and self._global_span is not None:
            self._global_span.end(_BATCH_CANCEL_TAG)
            self._global_span = None
        rolled_back = self._ledger.micro_batch_cut(batch)
        if rolled_back:
            from .trainer import Trainer
            stat = Trainer._trainer._cur_epoch_stat if Trainer._trainer is not None else None
            if stat is not None:
                stat.num_rollback_batch += rolled_back

    def vote_finish_last_micro_batch(self) -> bool:
        return _Distributor.vote_finish_last_micro_batch()

    def vote_abort_last_micro_batch(self):
        _Distributor.vote_abort_last_micro_batch()

    def reset_last_micro_batch_finish_vote(self):
        _Distributor.reset_last_micro_batch_finish_vote()

    def _should_checkpoint_micro_batch(self):
        return bool(self._enable_grad_accumulate and self._checkpoint_micro_batch)


# ----------------------------------------------------------------------------------------------------------------
class DynamicBatchDataset:
    """dynamic_batch.py:313-538.  Iterating yields `Batch` objects until the distributor has seen every global
    batch of the epoch; the size of each is whatever the controller's target allows at that moment."""
    _dynamic_batch_dataset: Optional[DynamicBatchDataset] = None

    def __init__(self, ds_type: DatasetType, ds_size: int, colocate_ctrl,
                 vision_dataset_config: Optional[VisionDatasetConfig] = None,
                 text_dataset_config: Optional[TextDatasetConfig] = None,
                 empty_cache_at_larger_batch_size: bool = False, fake_data=False, device=None, seed=0,
                 num_distinct_samples: Optional[int] = None):
        assert DynamicBatchDataset._dynamic_batch_dataset is None
        DynamicBatchDataset._dynamic_batch_dataset = self
        self.ds_type, self.ds_size, self.col_ctrl = ds_type, ds_size, colocate_ctrl
        self.vision_dataset_config, self.text_dataset_config = vision_dataset_config, text_dataset_config
        self._empty_cache_at_larger_batch_size = empty_cache_at_larger_batch_size
        self._state = DatasetState.INIT
        self._last_batch = None
        self.device = device if device is not None else f'cuda:{_C.get_train_rank()}'
        if not fake_data:
            # the reference reads workload_data/cifar10/*.npy, which is not shipped
            print('Warning: fake_data is forced to be True (no dataset files)', file=sys.stderr)
        resident = ds_size if num_distinct_samples is None else min(ds_size, num_distinct_samples)
        gen = torch.Generator().manual_seed(seed)
        if ds_type == DatasetType.VISION:
            cfg = vision_dataset_config
            tensors = {'images': torch.randn(resident, *cfg.input_shape, generator=gen),
                       'labels': torch.randint(0, cfg.num_class, (resident,), generator=gen)}
        elif ds_type == DatasetType.TEXT_GEN:
            ids = torch.randint(100, 30000, (resident, text_dataset_config.seq_len), generator=gen)
            tensors = {'input_ids': ids, 'labels': ids}
        else:
            raise Exception(f"Unsupported dataset type: {ds_type}")
        self._samples = _HostSamples(tensors, pinned=torch.cuda.is_available() and str(self.device).startswith('cuda'))
        self.all_inputs = self._samples.tensors
        self._size_key = 'images' if ds_type == DatasetType.VISION else 'input_ids'

    def get_target_batch_size(self):
        return self.col_ctrl.target_batch_size

    def get_next_batch_size(self):
        return _Distributor.query_next_batch_size(self.get_target_batch_size())

    def get_batch_size(self, batch: Batch):
        return len(batch[self._size_key])

    def _next_batch(self):
        assert self._state == DatasetState.ITER
        self._state = DatasetState.NEXT

    def _wait_valid_batch_size(self):
        """A target of zero means inference holds everything for now: keep answering its requests and wait."""
        size = self.get_next_batch_size()
        while size <= 0 and self.col_ctrl.train_mode.is_colocate():
            _C.update_current_batch_size(size)
            if self.col_ctrl._stub.cmd in (CtrlEvent.kColocateAdjustL1, CtrlEvent.kColocateAdjustL2):
                self.col_ctrl.release_and_reply()
            time.sleep(1e-3)
            size = self.get_next_batch_size()
        return size

    def _get_batch(self) -> Batch:
        with EventManager.record_duration_event('wait_valid_batch'):
            asked = self._wait_valid_batch_size()
        range_vec, closes_global_batch = _Distributor.get_batch(asked)
        batch = Batch(self._samples.to_device(range_vec, self.device))
        got = self.get_batch_size(batch)
        if _Distributor._lazy_distributing:
            assert 1 <= got <= asked, (f"batch size mismatch: 1 <= {got} <= {asked}, "
                                       f"check lazy batch distributing implementation.")
        else:
            assert got == asked, (f"batch size mismatch: {got} != {asked}, "
                                  f"check batch distirbutor and dataset implementation.")
        batch['do_step'] = bool(closes_global_batch)
        batch['range'] = range_vec
        return batch

    def __iter__(self) -> Iterator[Batch]:
        per_epoch = _Distributor.get_num_global_batch_per_epoch()
        _Distributor.next_epoch()
        _Distributor.next_global_batch()
        while _Distributor.get_num_proced_global_batch() < per_epoch:
            batch = self._get_batch()
            size = self.get_batch_size(batch)
            grew = self._state != DatasetState.INIT and self.get_batch_size(self._last_batch) < size
            if grew and self._empty_cache_at_larger_batch_size and _C.is_enable_shared_tensor():
                MemoryPool.empty_cache()
            self._state, self._last_batch = DatasetState.ITER, batch
            if self.col_ctrl is not None:
                self.col_ctrl.report_batch_size(size)
                _C.update_current_batch_size(size)
            yield batch


def init_dynamic_batch(dataset_size: int, dataset_type: DatasetType,
                       dataset_config: Union[VisionDatasetConfig, TextDatasetConfig], batch_size: int,
                       global_batch_size: Optional[int] = None, enable_grad_accumulate: bool = False,
                       checkpoint_micro_batch: bool = False, empty_cache_at_larger_batch_size: bool = False,
                       batch_distribute_policy: BatchDistributePolicy = BatchDistributePolicy.FIX,
                       lazy_batch_distributing: bool = False, fake_data: bool = False, **dataset_kwargs
                       ) -> Tuple[DynamicBatchDataset, MicroBatchManager]:
    """dynamic_batch.py:541-613: dataset, distributor, manager and throughput model, in that order."""
    assert _C.is_configured(), "torch_col is not initialized"
    assert CtrlBase._colocate_ctrl is not None, "colocate control must be initialized before dynamic batch dataset."
    colocated = _C.get_colocate_train_mode().is_colocate()
    assert enable_grad_accumulate or not colocated, "enable grad accumulate when colocate training."
    assert enable_grad_accumulate or global_batch_size is None, "enable grad accumulate when global batch size is set."
    if global_batch_size is None:
        global_batch_size = batch_size * _C.get_train_world_size()
    if checkpoint_micro_batch and not enable_grad_accumulate:
        print(f'torch_col: Warning: should not accumulate grad (global_batch_size {global_batch_size}, '
              f'batch_size {batch_size}), checkpoint_micro_batch will be False.', file=sys.stderr)
        checkpoint_micro_batch = False
    if not colocated and batch_distribute_policy != BatchDistributePolicy.FIX:
        print(f'torch_col: Warning: batch_distribute_policy will be {BatchDistributePolicy.FIX} '
              f'when not colocate with inference.', file=sys.stderr)
        batch_distribute_policy = BatchDistributePolicy.FIX

    dataset = DynamicBatchDataset(
        ds_type=dataset_type, ds_size=dataset_size, colocate_ctrl=CtrlBase._colocate_ctrl,
        vision_dataset_config=dataset_config if dataset_type == DatasetType.VISION else None,
        text_dataset_config=dataset_config if dataset_type == DatasetType.TEXT_GEN else None,
        empty_cache_at_larger_batch_size=empty_cache_at_larger_batch_size, fake_data=fake_data, **dataset_kwargs)
    dist.init_dynamic_batch_distributor(dataset_size, batch_size, global_batch_size, lazy_batch_distributing,
                                        batch_distribute_policy.value)
    manager = MicroBatchManager(dynamic_dataset=dataset, enable_grad_accumulate=enable_grad_accumulate,
                                checkpoint_micro_batch=checkpoint_micro_batch)
    dist.init_train_performance_model()
    return dataset, manager


def get_dynamic_dataset() -> DynamicBatchDataset:
    assert DynamicBatchDataset._dynamic_batch_dataset is not None
    return DynamicBatchDataset._dynamic_batch_dataset


def get_micro_batch_manager() -> MicroBatchManager:
    assert MicroBatchManager._micro_batch_manager is not None
    return MicroBatchManager._micro_batch_manager


def _reset_singletons():
    """One process may set the object graph up again (tests)."""
    DynamicBatchDataset._dynamic_batch_dataset = None
    MicroBatchManager._micro_batch_manager = None
