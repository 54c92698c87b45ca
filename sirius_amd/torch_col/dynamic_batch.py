"""Dynamic-batch dataset and micro-batch bookkeeping
(pytorch/torch_col/dynamic_batch.py:27-625).  Sample ranges, `do_step`, the finish / abort /
rollback rules, event names and tags follow the reference; the optimizer step goes to the
engine's fused kernels instead of torch.optim."""
from __future__ import annotations

import contextlib
import dataclasses
import sys
import time
from enum import Enum, IntEnum
from typing import Iterator, List, Optional, Tuple, Union

import numpy as np
import torch

from . import _C, dist
from ._C import CtrlEvent, TrainMode
from .colocate_ctrl import ColocateCtrl, CtrlBase, DummyCtrl, SwitchCtrl, get_colocate_ctrl
from .dist import _DynamicBatchDistirbutor, _PerfModel
from .util import EventManager, MemoryPool

_BATCH_FINISH_TAG = 'finish'
_BATCH_CANCEL_TAG = 'cancel'


class BatchDistributePolicy(Enum):
    FIX = 'fix'
    SIMPLE = 'simple'
    BY_PERFORMANCE = 'by_performance'


def _num_sample_of_batch_range_vec(batch_range_vec: List[Tuple[int, int]]) -> int:
    return sum(j - i for i, j in batch_range_vec)


def _num_sample_of_batch_range(batch_range) -> int:
    # the reference passes a whole range vector here (dynamic_batch.py:278-286)
    if batch_range and isinstance(batch_range[0], (tuple, list)):
        return _num_sample_of_batch_range_vec(batch_range)
    return batch_range[1] - batch_range[0]


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


class Batch(dict):
    def __init__(self, inputs: Optional[dict] = None):
        super().__init__()
        for k, v in (inputs or {}).items():
            self[k] = v

    def should_update_param(self):
        return self.get('do_step', True)

    def get_range(self) -> List[Tuple[int, int]]:
        return self['range']

    def __len__(self) -> int:
        return DynamicBatchDataset._dynamic_batch_dataset.get_batch_size(self)


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
        self._last_batch = None
        self._batch_event = None
        self._global_batch_event = None
        self._past_micro_batch_range_vecs_in_global_batch = []
        self._last_batch_range_vec = None

    def loss_scale(self, batch: Batch) -> float:
        """The factor scale_loss multiplies by, for engines that fold it into the loss kernel."""
        if not self._enable_grad_accumulate:
            return 1.0
        return self._dynamic_dataset.get_batch_size(batch) / _DynamicBatchDistirbutor.get_global_batch_size()

    def scale_loss(self, batch: Batch, loss):
        """loss /= global_batch_size / batch_size  (dynamic_batch.py:112-120)"""
        if self._enable_grad_accumulate:
            scale_factor = (_DynamicBatchDistirbutor.get_global_batch_size()
                            / self._dynamic_dataset.get_batch_size(batch))
            loss /= scale_factor
        return loss

    def optimizer_step(self, batch: Batch, optimizer, amp_scaler=None, grad_accumulator=None):
        """dynamic_batch.py:122-153.  `optimizer` is the engine (its fused SGD is the step)."""
        if self._should_checkpoint_micro_batch():
            assert grad_accumulator is not None
            with get_colocate_ctrl().steps_no_interrupt():
                step_event = EventManager.record_event('optimizer_step')
                grad_accumulator.accumulate()
                if batch.should_update_param():
                    grad_accumulator.step(optimizer, amp_scaler)
                    step_event.tag = 'global'
                else:
                    step_event.tag = 'local'
                EventManager.record_event('', step_event)
        elif not self._enable_grad_accumulate or batch.should_update_param():
            with get_colocate_ctrl().steps_no_interrupt():
                step_event = EventManager.record_event('optimizer_step')
                optimizer.optimizer_step(use_global=False)
                optimizer.zero_grad()
                EventManager.record_event('', step_event)

    @contextlib.contextmanager
    def ddp_sync_context(self, model, batch: Batch):
        """dynamic_batch.py:155-167: one GPU, there is no gradient exchange to suppress."""
        yield

    def begin_batch(self, epoch_idx: int, batch_idx: int, batch: Batch, batch_range_vec):
        self._last_batch_range_vec = batch_range_vec
        self._last_batch = batch
        self._record_batch_event(epoch_idx, batch_idx, len(batch))

    def finish_batch(self, epoch_idx: int, batch_idx: int, batch: Batch):
        # launches still in a software queue are not yet on the stream: drain the queues first
        _C.SyncAllStreams()
        if torch.cuda.is_available():
            torch.cuda.current_stream().synchronize()
        col_ctrl = get_colocate_ctrl()
        if col_ctrl.train_mode == TrainMode.COLOCATE_L2:
            if col_ctrl._stub.cmd == CtrlEvent.kColocateAdjustL2:
                if _C.get_train_world_size() == 1:
                    col_ctrl.release_and_reply(False)
                    if not batch.should_update_param():
                        _DynamicBatchDistirbutor.distribute_batch(True, True, False)
                elif batch.should_update_param():
                    dist.wait_barrier()
                    col_ctrl.release_and_reply(False)

        self._complete_batch_event(_BATCH_FINISH_TAG, batch)
        self._past_micro_batch_range_vecs_in_global_batch.append(self._last_batch_range_vec)

        if (not self._enable_grad_accumulate
                or not _C.get_colocate_train_mode().is_kill_batch()
                or self._should_checkpoint_micro_batch()):
            _DynamicBatchDistirbutor.finish_batch(batch.get_range(), batch.should_update_param())

        if batch.should_update_param():  # the micro-batch that steps ends the global batch
            self._next_global_batch()

        self._last_batch = None
        self._last_batch_range_vec = None
        self._dynamic_dataset._next_batch()

    def abort_batch(self, epoch_idx: int, batch_idx: int, batch: Batch):
        self._complete_batch_event(_BATCH_CANCEL_TAG, batch)
        if self._enable_grad_accumulate and not self._checkpoint_micro_batch:
            self._rollback_micro_batch()
        else:
            _DynamicBatchDistirbutor.abort_batch(self._last_batch_range_vec, batch.should_update_param())
        self._last_batch = None
        self._last_batch_range_vec = None

    def vote_finish_last_micro_batch(self) -> bool:
        return _DynamicBatchDistirbutor.vote_finish_last_micro_batch()

    def vote_abort_last_micro_batch(self):
        _DynamicBatchDistirbutor.vote_abort_last_micro_batch()

    def reset_last_micro_batch_finish_vote(self):
        _DynamicBatchDistirbutor.reset_last_micro_batch_finish_vote()

    def _record_batch_event(self, epoch_idx: int, batch_idx: int, batch_size: int):
        self._batch_event = EventManager.record_event(f'batch_{epoch_idx:02d}_{batch_idx:03d}_{batch_size:02d}')
        if self._enable_grad_accumulate and self._global_batch_event is None:
            global_batch_size = _DynamicBatchDistirbutor.get_global_batch_size()
            self._global_batch_event = EventManager.record_event(
                f'global_batch_{epoch_idx:02d}_{batch_idx:03d}_{global_batch_size:02d}')

    def _complete_batch_event(self, tag: str, batch: Batch):
        assert self._batch_event is not None
        self._batch_event.tag = tag
        EventManager.record_event('', self._batch_event)
        if _C.get_train_rank() == 0 and tag == _BATCH_FINISH_TAG:
            _PerfModel.record_thpt(len(batch), self._batch_event.duration)
        self._batch_event = None

    def _complate_global_batch_event(self, tag: str):
        assert self._global_batch_event is not None
        self._global_batch_event.tag = tag
        EventManager.record_event('', self._global_batch_event)
        self._global_batch_event = None

    def _should_checkpoint_micro_batch(self):
        return bool(self._enable_grad_accumulate and self._checkpoint_micro_batch)

    def _rollback_micro_batch(self):
        assert self._enable_grad_accumulate and not self._checkpoint_micro_batch, (
            "only used for accumulation without checkpoint")
        from .trainer import Trainer
        self._complate_global_batch_event(_BATCH_CANCEL_TAG)
        stat = Trainer._trainer._cur_epoch_stat if Trainer._trainer is not None else None
        for idx in self._past_micro_batch_range_vecs_in_global_batch:
            if stat is not None:
                stat.num_rollback_batch += _num_sample_of_batch_range(idx)
            _DynamicBatchDistirbutor.abort_batch(idx, False)
        _DynamicBatchDistirbutor.abort_batch(self._last_batch_range_vec, self._last_batch.should_update_param())
        if stat is not None:
            stat.num_rollback_batch += _num_sample_of_batch_range(self._last_batch_range_vec)
        self._past_micro_batch_range_vecs_in_global_batch = []
        self._last_batch_range_vec = None

    def _next_global_batch(self):
        if self._enable_grad_accumulate:
            self._complate_global_batch_event(_BATCH_FINISH_TAG)
        if (self._enable_grad_accumulate and _C.get_colocate_train_mode().is_kill_batch()
                and not self._checkpoint_micro_batch):
            num_micro_batch = len(self._past_micro_batch_range_vecs_in_global_batch)
            for i, batch_range in enumerate(self._past_micro_batch_range_vecs_in_global_batch):
                _DynamicBatchDistirbutor.finish_batch(batch_range, i == num_micro_batch - 1)
        self._past_micro_batch_range_vecs_in_global_batch = []
        _DynamicBatchDistirbutor.next_global_batch()


class DynamicBatchDataset:
    """dynamic_batch.py:313-538: holds the (synthetic) samples in pinned host memory and yields
    `Batch` dicts sized by the current target batch size."""
    _dynamic_batch_dataset: Optional[DynamicBatchDataset] = None

    def __init__(self, ds_type: DatasetType, ds_size: int, colocate_ctrl,
                 vision_dataset_config: Optional[VisionDatasetConfig] = None,
                 text_dataset_config: Optional[TextDatasetConfig] = None,
                 empty_cache_at_larger_batch_size: bool = False, fake_data=False, device=None, seed=0,
                 num_distinct_samples: Optional[int] = None):
        assert DynamicBatchDataset._dynamic_batch_dataset is None
        DynamicBatchDataset._dynamic_batch_dataset = self
        self.ds_type = ds_type
        self.ds_size = ds_size
        self.col_ctrl = colocate_ctrl
        self.vision_dataset_config = vision_dataset_config
        self.text_dataset_config = text_dataset_config
        self._empty_cache_at_larger_batch_size = empty_cache_at_larger_batch_size
        self._state = DatasetState.INIT
        self._last_batch = None
        self._ds_ring_repeat = True
        self.device = device if device is not None else f'cuda:{_C.get_train_rank()}'
        if not fake_data:
            # the reference's real data (workload_data/cifar10/*.npy) is not shipped
            print('Warning: fake_data is forced to be True (no dataset files)', file=sys.stderr)
        # the ring-repeat rule of the reference (dynamic_batch.py:449-454) lets a small resident
        # set stand for a larger dataset: sample i is row i % num_distinct_samples
        n = ds_size if num_distinct_samples is None else min(ds_size, num_distinct_samples)
        pin = torch.cuda.is_available() and str(self.device).startswith('cuda')
        g = torch.Generator().manual_seed(seed)

        def host(t):
            return t.pin_memory() if pin else t
        if ds_type == DatasetType.VISION:
            self.all_inputs = {
                'images': host(torch.randn(n, *vision_dataset_config.input_shape, generator=g)),
                'labels': host(torch.randint(0, vision_dataset_config.num_class, (n,), generator=g)),
            }
        elif ds_type == DatasetType.TEXT_GEN:
            ids = host(torch.randint(100, 30000, (n, text_dataset_config.seq_len), generator=g))
            self.all_inputs = {'input_ids': ids, 'labels': ids}
        else:
            raise Exception(f"Unsupported dataset type: {ds_type}")

    def get_target_batch_size(self):
        return self.col_ctrl.target_batch_size

    def get_next_batch_size(self):
        return _DynamicBatchDistirbutor.query_next_batch_size(self.get_target_batch_size())

    def get_batch_size(self, batch: Batch):
        if self.ds_type == DatasetType.VISION:
            return len(batch['images'])
        if self.ds_type == DatasetType.TEXT_GEN:
            return len(batch['input_ids'])
        raise Exception(f"Unsupported dataset type: {self.ds_type}")

    def _next_batch(self):
        assert self._state == DatasetState.ITER
        self._state = DatasetState.NEXT

    def _retrieve_batch(self, batch_range_vec) -> dict:
        batch = {}
        batch_size = _num_sample_of_batch_range_vec(batch_range_vec)
        for k, src in self.all_inputs.items():
            out = torch.empty([batch_size, *src.shape[1:]], dtype=src.dtype, device=self.device)
            off = 0
            for i, j in batch_range_vec:
                l = j - i
                if self._ds_ring_repeat and i >= len(src):
                    i = i % len(src)
                    j = i + l
                if j <= len(src):
                    out[off:off + l].copy_(src[i:j], non_blocking=True)
                else:  # the range wraps round the resident set
                    head = len(src) - i
                    out[off:off + head].copy_(src[i:], non_blocking=True)
                    idx = torch.arange(head, l) % len(src)
                    out[off + head:off + l].copy_(src[idx], non_blocking=True)
                off += l
            batch[k] = out
        return batch

    def _wait_valid_batch_size(self):
        batch_size = self.get_next_batch_size()
        if self.col_ctrl.train_mode.is_colocate():
            while batch_size <= 0:
                _C.update_current_batch_size(batch_size)
                if self.col_ctrl._stub.cmd in (CtrlEvent.kColocateAdjustL1, CtrlEvent.kColocateAdjustL2):
                    self.col_ctrl.release_and_reply()
                time.sleep(1e-3)
                batch_size = self.get_next_batch_size()
        return batch_size

    def _get_batch(self) -> Batch:
        with EventManager.record_duration_event('wait_valid_batch'):
            _batch_size = self._wait_valid_batch_size()
        batch_range_vec, last_micro_batch = _DynamicBatchDistirbutor.get_batch(_batch_size)
        batch = Batch(self._retrieve_batch(batch_range_vec))
        batch_size = self.get_batch_size(batch)
        if not _DynamicBatchDistirbutor._lazy_distributing:
            assert batch_size == _batch_size, (
                f"batch size mismatch: {batch_size} != {_batch_size}, "
                f"check batch distirbutor and dataset implementation.")
        else:
            assert 1 <= batch_size <= _batch_size, (
                f"batch size mismatch: 1 <= {batch_size} <= {_batch_size}, "
                f"check lazy batch distributing implementation.")
        batch['do_step'] = bool(last_micro_batch)
        batch['range'] = batch_range_vec
        return batch

    def __iter__(self) -> Iterator[Batch]:
        num_global_batch_per_epoch = _DynamicBatchDistirbutor.get_num_global_batch_per_epoch()
        _DynamicBatchDistirbutor.next_epoch()
        _DynamicBatchDistirbutor.next_global_batch()
        while _DynamicBatchDistirbutor.get_num_proced_global_batch() < num_global_batch_per_epoch:
            batch = self._get_batch()
            batch_size = self.get_batch_size(batch)
            if (self._state != DatasetState.INIT and _C.is_enable_shared_tensor()
                    and self._empty_cache_at_larger_batch_size
                    and self.get_batch_size(self._last_batch) < batch_size):
                MemoryPool.empty_cache()
            self._state = DatasetState.ITER
            self._last_batch = batch
            if self.col_ctrl is not None:
                self.col_ctrl.report_batch_size(batch_size)
                _C.update_current_batch_size(batch_size)
            yield batch


def init_dynamic_batch(dataset_size: int, dataset_type: DatasetType,
                       dataset_config: Union[VisionDatasetConfig, TextDatasetConfig], batch_size: int,
                       global_batch_size: Optional[int] = None, enable_grad_accumulate: bool = False,
                       checkpoint_micro_batch: bool = False, empty_cache_at_larger_batch_size: bool = False,
                       batch_distribute_policy: BatchDistributePolicy = BatchDistributePolicy.FIX,
                       lazy_batch_distributing: bool = False, fake_data: bool = False, **dataset_kwargs
                       ) -> Tuple[DynamicBatchDataset, MicroBatchManager]:
    """dynamic_batch.py:541-613"""
    assert _C.is_configured(), "torch_col is not initialized"
    assert CtrlBase._colocate_ctrl is not None, "colocate control must be initialized before dynamic batch dataset."
    assert not (_C.get_colocate_train_mode().is_colocate() and not enable_grad_accumulate), (
        "enable grad accumulate when colocate training.")
    assert not (global_batch_size is not None and not enable_grad_accumulate), (
        "enable grad accumulate when global batch size is set.")
    if global_batch_size is None:
        global_batch_size = batch_size * _C.get_train_world_size()
    if not enable_grad_accumulate and checkpoint_micro_batch:
        print(f'torch_col: Warning: should not accumulate grad (global_batch_size {global_batch_size}, '
              f'batch_size {batch_size}), checkpoint_micro_batch will be False.', file=sys.stderr)
        checkpoint_micro_batch = False
    if not _C.get_colocate_train_mode().is_colocate() and batch_distribute_policy != BatchDistributePolicy.FIX:
        print(f'torch_col: Warning: batch_distribute_policy will be {BatchDistributePolicy.FIX} '
              f'when not colocate with inference.', file=sys.stderr)
        batch_distribute_policy = BatchDistributePolicy.FIX

    vision_ds_config = dataset_config if dataset_type == DatasetType.VISION else None
    text_ds_config = dataset_config if dataset_type == DatasetType.TEXT_GEN else None
    dynamic_dataset = DynamicBatchDataset(
        ds_type=dataset_type, ds_size=dataset_size, colocate_ctrl=CtrlBase._colocate_ctrl,
        vision_dataset_config=vision_ds_config, text_dataset_config=text_ds_config,
        empty_cache_at_larger_batch_size=empty_cache_at_larger_batch_size, fake_data=fake_data, **dataset_kwargs)
    dist.init_dynamic_batch_distributor(dataset_size, batch_size, global_batch_size, lazy_batch_distributing,
                                        batch_distribute_policy.value)
    micro_batch_manager = MicroBatchManager(dynamic_dataset=dynamic_dataset,
                                            enable_grad_accumulate=enable_grad_accumulate,
                                            checkpoint_micro_batch=checkpoint_micro_batch)
    dist.init_train_performance_model()
    return dynamic_dataset, micro_batch_manager


def get_dynamic_dataset() -> DynamicBatchDataset:
    assert DynamicBatchDataset._dynamic_batch_dataset is not None
    return DynamicBatchDataset._dynamic_batch_dataset


def get_micro_batch_manager() -> MicroBatchManager:
    assert MicroBatchManager._micro_batch_manager is not None
    return MicroBatchManager._micro_batch_manager


def _reset_singletons():
    """Lets one process set the object graph up again (tests)."""
    DynamicBatchDataset._dynamic_batch_dataset = None
    MicroBatchManager._micro_batch_manager = None
