"""Epoch loop with abort -> release -> reconfigure (pytorch/torch_col/trainer.py:24-272)."""
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
        self.dynamic_dataset = get_dynamic_dataset()
        self.batch_manager = get_micro_batch_manager()
        # the reference wraps the dataset in a DataLoader(batch_size=None, num_workers=0),
        # which is plain iteration
        self.data_loader = self.dynamic_dataset
        self.iter_train_fn = iter_train_fn
        self.overall_stat = TrainStat(0, 0, 0)
        self.epoch_stats = []
        self.epoch_events = []
        self._cur_epoch_stat = None
        self._last_max_batch_size_from_last_kill = None

    def train_one_epoch(self, epoch_idx: int) -> Optional[float]:
        epoch_event = EventManager.record_event(f'epoch_{epoch_idx:02d}_{self.dynamic_dataset.ds_size}')
        self._cur_epoch_stat = EpochStat()
        running_loss = 0

        for batch_idx, batch in enumerate(self.data_loader):
            self._cur_epoch_stat.tried_batch += 1
            self.overall_stat.tried_batch += 1

            if self._last_max_batch_size_from_last_kill is None:
                self._last_max_batch_size_from_last_kill = len(batch)
            elif len(batch) > self._last_max_batch_size_from_last_kill:
                MemoryPool.empty_cache()
                print(f'empty cache due to greater batch size '
                      f'{self._last_max_batch_size_from_last_kill} -> {len(batch)}')
                self._last_max_batch_size_from_last_kill = len(batch)

            self.batch_manager.begin_batch(epoch_idx, batch_idx, batch, batch['range'])
            try:
                _running_loss = self.iter_train_fn(batch)
            except (ColocateAdjustL1Exception, SwitchL1Exception, EngineColocateAdjustL1Exception) as exception:
                self.handle_abort_batch(epoch_idx, batch_idx, batch, exception)
            else:
                self.batch_manager.finish_batch(epoch_idx, batch_idx, batch)
                if epoch_idx == 0 and batch_idx == 0:
                    self._default_first_batch_callback()
                running_loss += _running_loss
                self._cur_epoch_stat.finished_batch += 1
                self._cur_epoch_stat.finished_sample += self.dynamic_dataset.get_batch_size(batch)
                self.overall_stat.finished_batch += 1

        EventManager.record_event('', epoch_event)
        self.epoch_stats.append(self._cur_epoch_stat)
        self.epoch_events.append(epoch_event)
        self._cur_epoch_stat = None
        return running_loss / self.dynamic_dataset.ds_size

    def get_overall_stat(self) -> TrainStat:
        return self.overall_stat

    def get_last_epoch_stat(self) -> Optional[EpochStat]:
        return self.epoch_stats[-1] if self.epoch_stats else None

    def get_last_epoch_event(self) -> Optional[Event]:
        return self.epoch_events[-1] if self.epoch_events else None

    def get_last_epoch_duration(self) -> Optional[float]:
        e = self.get_last_epoch_event()
        return None if e is None else e.duration

    def handle_abort_batch(self, epoch_idx: int, batch_idx: int, batch: Batch, exception: Exception):
        """trainer.py:160-250"""
        if epoch_idx == 0 and batch_idx == 0:
            raise RuntimeError("first micro batch could not be interrupted, please increase the delay time")

        # first, finish aborting the batch
        dist.wait_barrier()
        if isinstance(exception, EngineColocateAdjustL1Exception):
            xsched.kill_batch()
        self.batch_manager.abort_batch(epoch_idx, batch_idx, batch)
        # gradients of the killed micro-batch are partial: drop them (the accumulated ones stay)
        self.model.discard_partial_grads()
        col_ctrl = self.dynamic_dataset.col_ctrl
        if isinstance(col_ctrl, SwitchCtrl):
            if _C.is_train_master():
                col_ctrl._stub.set_global_has_batch_killed(True)
            dist.wait_barrier()

        # second, release memory and reply to inference
        batch_size = self.dynamic_dataset.get_batch_size(batch)
        with EventManager.record_duration_event(f'batch_exception_{epoch_idx:02d}_{batch_idx:03d}_{batch_size:02d}'):
            col_ctrl.release_and_reply(True)
            print(f'[Rank {_C.get_train_rank()} | {exception}] batch_size: {batch_size} -> '
                  f'{col_ctrl.unpub_target_batch_size}.')
        self._cur_epoch_stat.killed_batch += 1
        self.overall_stat.killed_batch += 1

        # third, re-configure training and restart
        with EventManager.record_duration_event(f'batch_restart_{epoch_idx:02d}_{batch_idx:03d}'):
            if _C.get_train_rank() == 0:
                self.batch_manager.reset_last_micro_batch_finish_vote()
            dist.wait_barrier()
            if _C.get_colocate_train_mode().is_colocate():
                col_ctrl.set_killed_batch_recover()  # launches are accepted again
            if _C.get_train_rank() == 0:
                _DynamicBatchDistirbutor.distribute_batch(True, True, False)
                if _C.get_colocate_train_mode().is_colocate():
                    col_ctrl.set_killed_batch_reconfiged()
            dist.wait_barrier()

        # [task switch] fourth, wait for resume
        if _C.get_colocate_train_mode().is_taskswitch():
            while not col_ctrl._stub.prepare_resume():
                time.sleep(1e-3)
            dist.wait_barrier()
        self._last_max_batch_size_from_last_kill = None

    def _default_first_batch_callback(self):
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
