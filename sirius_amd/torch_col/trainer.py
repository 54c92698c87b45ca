"""The epoch loop and what happens when a micro-batch is cut: abort -> give memory back and answer -> re-split the
samples -> (task switch: wait for the resume).  Names, statistics, event names (`epoch_EE_SIZE`,
`batch_exception_...`, `batch_restart_...`) and printed lines are the reference's
(pytorch/torch_col/trainer.py:24-272).

A cut arrives as one of three exceptions out of `iter_train_fn`: raised by a checkpoint between launch segments
(ColocateAdjustL1Exception, SwitchL1Exception) or by the engine itself when the control thread has already
killed its launches (EngineColocateAdjustL1Exception).  The recovery is a fixed list of phases, each a method
below; `handle_abort_batch` only sequences them.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Any, Callable, Optional

from . import _C, dist, xsched
from .colocate_ctrl import (ColocateAdjustL1Exception, EngineColocateAdjustL1Exception, SwitchCtrl,
                            SwitchL1Exception)
from .dist import _DynamicBatchDistirbutor
from .dynamic_batch import Batch, get_dynamic_dataset, get_micro_batch_manager
from .util import Event, EventManager, MemoryPool

_CUT = (ColocateAdjustL1Exception, SwitchL1Exception, EngineColocateAdjustL1Exception)


@dataclass
class TrainStat:
    killed_batch: int = 0
    finished_batch: int = 0
    tried_batch: int = 0


@dataclass
class EpochStat:
    killed_batch: int = 0
    finished_batch: int = 0
    tried_batch: int = 0
    finished_sample: int = 0
    num_rollback_batch: int = 0
    killed_time: float = 0.0
    finished_time: float = 0.0


class Trainer:
    _trainer: Optional[Trainer] = None

    def __init__(self, model, iter_train_fn: Callable[[Any], float]):
        Trainer._trainer = self
        self.rank = _C.get_train_rank()
        self.model = model
        self.iter_train_fn = iter_train_fn
        self.dynamic_dataset = get_dynamic_dataset()
        self.batch_manager = get_micro_batch_manager()
        self.data_loader = self.dynamic_dataset   # the reference's DataLoader(batch_size=None) is plain iteration
        self.overall_stat = TrainStat()
        self.epoch_stats, self.epoch_events = [], []
        self._cur_epoch_stat: Optional[EpochStat] = None
        # largest batch seen since the last cut: growing past it means cached blocks of the smaller plan are
        # in the way and go back to the pool first
        self._last_max_batch_size_from_last_kill: Optional[int] = None

    # ------------------------------------------------------------------ statistics
    def _count(self, field: str, n: int = 1):
        setattr(self._cur_epoch_stat, field, getattr(self._cur_epoch_stat, field) + n)
        if hasattr(self.overall_stat, field):
            setattr(self.overall_stat, field, getattr(self.overall_stat, field) + n)

    def get_overall_stat(self) -> TrainStat:
        return self.overall_stat

    def get_last_epoch_stat(self) -> Optional[EpochStat]:
        return self.epoch_stats[-1] if self.epoch_stats else None

    def get_last_epoch_event(self) -> Optional[Event]:
        return self.epoch_events[-1] if self.epoch_events else None

    def get_last_epoch_duration(self) -> Optional[float]:
        event = self.get_last_epoch_event()
        return event.duration if event is not None else None

    # ------------------------------------------------------------------ the loop
    def _make_room_for(self, size: int):
        seen = self._last_max_batch_size_from_last_kill
        if seen is not None and size > seen:
            MemoryPool.empty_cache()
            print(f'empty cache due to greater batch size {seen} -> {size}')
        if seen is None or size > seen:
            self._last_max_batch_size_from_last_kill = size

    def train_one_epoch(self, epoch_idx: int) -> Optional[float]:
        epoch_event = EventManager.record_event(f'epoch_{epoch_idx:02d}_{self.dynamic_dataset.ds_size}')
        self._cur_epoch_stat = EpochStat()
        loss_sum = 0
        for batch_idx, batch in enumerate(self.data_loader):
            self._count('tried_batch')
            self._make_room_for(len(batch))
            self.batch_manager.begin_batch(epoch_idx, batch_idx, batch, batch['range'])
            try:
                loss = self.iter_train_fn(batch)
            except _CUT as cut:
                self.handle_abort_batch(epoch_idx, batch_idx, batch, cut)
                continue
            self.batch_manager.finish_batch(epoch_idx, batch_idx, batch)
            if epoch_idx == 0 and batch_idx == 0:
                self._default_first_batch_callback()
            loss_sum += loss
            self._count('finished_batch')
            self._count('finished_sample', self.dynamic_dataset.get_batch_size(batch))
        EventManager.record_event('', epoch_event)
        self.epoch_stats.append(self._cur_epoch_stat)
        self.epoch_events.append(epoch_event)
        self._cur_epoch_stat = None
        return loss_sum / self.dynamic_dataset.ds_size

    # ------------------------------------------------------------------ a cut micro-batch
    def handle_abort_batch(self, epoch_idx: int, batch_idx: int, batch: Batch, exception: Exception):
        """trainer.py:160-250"""
        if epoch_idx == 0 and batch_idx == 0:
            raise RuntimeError("first micro batch could not be interrupted, please increase the delay time")
        ctrl = self.dynamic_dataset.col_ctrl
        size = self.dynamic_dataset.get_batch_size(batch)
        self._abort(epoch_idx, batch_idx, batch, exception, ctrl)
        with EventManager.record_duration_event(f'batch_exception_{epoch_idx:02d}_{batch_idx:03d}_{size:02d}'):
            ctrl.release_and_reply(True)
            print(f'[Rank {_C.get_train_rank()} | {exception}] batch_size: {size} -> '
                  f'{ctrl.unpub_target_batch_size}.')
        self._count('killed_batch')
        with EventManager.record_duration_event(f'batch_restart_{epoch_idx:02d}_{batch_idx:03d}'):
            self._reconfigure(ctrl)
        if _C.get_colocate_train_mode().is_taskswitch():
            self._wait_for_resume(ctrl)
        self._last_max_batch_size_from_last_kill = None

    def _abort(self, epoch_idx, batch_idx, batch, exception, ctrl):
        """Every rank has stopped; the samples of the cut micro-batch go back to the distributor; its gradients
        are partial and are dropped (accumulated ones stay)."""
        dist.wait_barrier()
        if isinstance(exception, EngineColocateAdjustL1Exception):
            xsched.kill_batch()     # the control thread cut the queue; this clears what the training thread added since
        self.batch_manager.abort_batch(epoch_idx, batch_idx, batch)
        self.model.discard_partial_grads()
        if isinstance(ctrl, SwitchCtrl):
            if _C.is_train_master():
                ctrl._stub.set_global_has_batch_killed(True)
            dist.wait_barrier()

    def _reconfigure(self, ctrl):
        """Launches are accepted again and the rest of the global batch is split for the new batch size."""
        master, colocated = _C.get_train_rank() == 0, _C.get_colocate_train_mode().is_colocate()
        if master:
            self.batch_manager.reset_last_micro_batch_finish_vote()
        dist.wait_barrier()
        if colocated:
            ctrl.set_killed_batch_recover()
        if master:
            _DynamicBatchDistirbutor.distribute_batch(True, True, False)
            if colocated:
                ctrl.set_killed_batch_reconfiged()
        dist.wait_barrier()

    def _wait_for_resume(self, ctrl):
        while not ctrl._stub.prepare_resume():
            time.sleep(1e-3)
        dist.wait_barrier()

    # ------------------------------------------------------------------ first batch
    def _default_first_batch_callback(self):
        """After the first micro-batch everything allocated so far is model state: tagging ends, and the launch
        queue starts counting from an empty state."""
        if _C.is_enable_shared_tensor():
            _C.tag_model_end()
        if _C.is_enable_xsched():
            if xsched.is_guess_nccl_begined():
                xsched.guess_nccl_end()
            _C.SyncAllStreams()
            xsched.initial_kill_batch(0, 0)

    def _default_first_epoch_callback(self):
        pass

    def _is_ddp_training(self):
        return False
