"""The inference server's side of the adjust protocol, for a stand-in peer that behaves like the real one: the
controller that numbers and sends the commands (server/control/controller.cc:75-150, 207-327, 377-386) and the
resource manager that decides how much memory is free (server/resource_manager.cc:22-87).

Controller          owns the shared segment like DebugServer does, follows training's status from the messages
                    it sends back, and sends adjust commands the way the server's controller does:
                      * every call takes the next command id, also when nothing is sent;
                      * nothing is sent while training is idle;
                      * ColocateAdjust is skipped (id 0) when no rank's unpublished target lies below its
                        published one, i.e. the last shrink has already been taken up;
                      * WaitColocateAdjustDone returns once training's reply carries an id >= the command's.
ResourceManager     free memory for inference and memory training may use, from the pool's size, the two tenants'
                    usage and the adjuster's prediction for training.
"""
import threading
import time
from enum import Enum
from typing import List, Optional, Sequence

from . import _C
from ._C import CtrlEvent
from .train_adjuster import TrainAdjuster


class TrainStatus(Enum):
    kIdle = 0
    kRunning = 1
    kInterrupted = 2


class Controller:
    def __init__(self, train_world_size: int = 1, colocate_level: int = 1, verbose: bool = False):
        assert colocate_level in (1, 2)
        self._comm = _C.PyInfTraCommunicator(True, True, train_world_size)
        self._world = train_world_size
        self._event = CtrlEvent.kColocateAdjustL1 if colocate_level == 1 else CtrlEvent.kColocateAdjustL2
        self._verbose = verbose
        self._lock = threading.Condition()
        self._adjust_cmd_id = 1               # Controller::adjust_cmd_id starts at 1
        self._interrupt_cmd_id = 0
        self.train_status = TrainStatus.kIdle
        self.adjust_done_ids = [0] * train_world_size
        self.task_switch_done_id = 0
        self.reported_batch_size = None
        self.target_batch_size = None         # TrainLauncher's target: set on kTrainStart from the board
        self.received = []
        self.sent = []
        self._running = True
        self._thread = threading.Thread(target=self._train_monitor, name="controller-monitor", daemon=True)
        self._thread.start()

    # ---- Controller::TrainMonitor (controller.cc:84-150)
    def _train_monitor(self):
        while self._running:
            for rank in range(self._world):
                msg = self._comm.timed_get_tra2inf(5, rank)
                if msg is None:
                    continue
                with self._lock:
                    self.received.append((_C.get_unix_timestamp_us(), rank, msg))
                    ev = msg.event
                    if ev == CtrlEvent.kTrainStart:
                        assert self.train_status == TrainStatus.kIdle
                        self.train_status = TrainStatus.kRunning
                        self.target_batch_size = _C.get_train_info(0, "init_batch_size")
                    elif ev == CtrlEvent.kInterruptTrainDone:
                        self.train_status = TrainStatus.kInterrupted
                        self.task_switch_done_id = msg.id
                    elif ev == CtrlEvent.kResumeTrainDone:
                        assert self.train_status in (TrainStatus.kInterrupted, TrainStatus.kRunning)
                        self.train_status = TrainStatus.kRunning
                    elif ev in (CtrlEvent.kColocateAdjustL1Done, CtrlEvent.kColocateAdjustL2Done):
                        self.adjust_done_ids[rank] = msg.id
                    elif ev == CtrlEvent.kTrainEnd:
                        assert self.train_status in (TrainStatus.kRunning, TrainStatus.kIdle)
                        self.train_status = TrainStatus.kIdle
                    elif ev == CtrlEvent.kReportBatchSize:
                        assert self.train_status != TrainStatus.kIdle
                        self.reported_batch_size = msg.value
                    self._lock.notify_all()
                if self._verbose and msg.event != CtrlEvent.kReportBatchSize:
                    print(f'[Controller] MonitorTrain: {msg}')

    def is_train_idle(self) -> bool:
        return self.train_status == TrainStatus.kIdle

    def _next_adjust_id(self) -> int:
        with self._lock:
            cmd_id = self._adjust_cmd_id
            self._adjust_cmd_id += 1
            return cmd_id

    def _put_all(self, cmd_id: int, event: CtrlEvent, values: Sequence[int]):
        for rank, value in enumerate(values):
            self._comm.put_inf2tra(_C.PyCtrlMsgEntry(cmd_id, event, int(value)), rank)
            self.sent.append((_C.get_unix_timestamp_us(), rank, cmd_id, event, int(value)))

    # ---- Controller::ColocateAdjust (controller.cc:207-262)
    def colocate_adjust(self, batch_size: int) -> int:
        """Inference needs the room of `batch_size` samples.  Returns the command's id; 0 when the request is
        already satisfied (every rank still has a shrink it has not taken up: unpublished target < target)."""
        cmd_id = self._next_adjust_id()
        if self.is_train_idle():
            return cmd_id
        target = [_C.get_train_info(r, "target_batch_size") for r in range(self._world)]
        unpub = [_C.get_train_info(r, "target_batch_size_unpublished") for r in range(self._world)]
        if not any(u < t for u, t in zip(unpub, target)):
            # the reference's rule, literally: without an unpublished shrink on some rank the adjust is "satisfied"
            return 0
        self.target_batch_size -= batch_size
        self._put_all(cmd_id, self._event, [self.target_batch_size] * self._world)
        return cmd_id

    # ---- Controller::ColocateInferRequireAdjust / ColocateInferReleaseAdjust (controller.cc:264-327)
    def colocate_infer_require_adjust(self, plans: Sequence[int]) -> int:
        """plans: the new batch size of every training rank (TrainAdjuster::AdjustPlan::batch_size); the plan's
        author has already written them on the board as unpublished targets."""
        assert len(plans) == self._world and plans
        cmd_id = self._next_adjust_id()
        if not self.is_train_idle():
            self._put_all(cmd_id, self._event, plans)
        return cmd_id

    def colocate_infer_release_adjust(self, plans: Sequence[int]) -> int:
        assert len(plans) == self._world
        cmd_id = self._next_adjust_id()
        if not self.is_train_idle():
            self._put_all(cmd_id, CtrlEvent.kInferExit, plans)
        return cmd_id

    # ---- Controller::WaitColocateAdjustDone (controller.cc:377-386)
    def wait_colocate_adjust_done(self, cmd_id: int, rank: int = 0, timeout_s: Optional[float] = None) -> bool:
        if self.is_train_idle():
            return True
        with self._lock:
            return self._lock.wait_for(lambda: self.adjust_done_ids[rank] >= cmd_id, timeout_s)

    # ---- task switching (controller.cc:152-205)
    def interrupt_train(self) -> int:
        self._interrupt_cmd_id += 1
        if not self.is_train_idle():
            self._put_all(self._interrupt_cmd_id, CtrlEvent.kInterruptTrain, [0] * self._world)
        return self._interrupt_cmd_id

    def resume_train(self) -> int:
        self._interrupt_cmd_id += 1
        if not self.is_train_idle():
            self._put_all(self._interrupt_cmd_id, CtrlEvent.kResumeTrain, [0] * self._world)
        return self._interrupt_cmd_id

    def wait_train_status(self, status: TrainStatus, timeout_s: float = 10.0) -> bool:
        with self._lock:
            return self._lock.wait_for(lambda: self.train_status == status, timeout_s)

    # ---- the two requests an inference model makes, with the adjuster's arithmetic in between
    def infer_require_memory_mb(self, required_mem_mb: float, adjuster: Optional[TrainAdjuster] = None) -> int:
        """TrainAdjuster::GetInferRequireMemAdjustPlan + ColocateInferRequireAdjust: write the new target on the
        board as unpublished, send it.  Returns the command id (0: nothing to do)."""
        adjuster = adjuster or TrainAdjuster()
        target = adjuster.infer_require_mem_adjust_plan(required_mem_mb)
        if target is None:
            return 0
        from .._lib import lib
        lib().tch_train_info_set_field(0, 6, int(target))
        self.target_batch_size = target
        return self.colocate_infer_require_adjust([target] * self._world)

    def infer_release_memory_mb(self, avail_mem_mb: float, adjuster: Optional[TrainAdjuster] = None) -> int:
        adjuster = adjuster or TrainAdjuster()
        target = adjuster.infer_release_mem_adjust_plan(avail_mem_mb)
        from .._lib import lib
        lib().tch_train_info_set_field(0, 6, int(target))
        self.target_batch_size = target
        return self.colocate_infer_release_adjust([target] * self._world)

    def stop(self):
        self._running = False
        self._thread.join()


class ResourceManager:
    """server/resource_manager.cc:22-87 in shared-tensor mode (the pool is the whole budget)."""

    def __init__(self, adjuster: Optional[TrainAdjuster] = None, train_memory_over_predict_mb: float = 0.0, device: int = 0):
        self.adjuster = adjuster or TrainAdjuster()
        self.over_predict_mb = train_memory_over_predict_mb
        self.device = device

    @staticmethod
    def _mb(nbytes: int) -> float:
        return nbytes / 1024.0 / 1024.0

    def infer_memory_mb(self) -> float:
        return self._mb(_C.cuda_memory_pool_infer_usage(self.device))

    def train_memory_mb(self) -> float:
        return self._mb(_C.cuda_memory_pool_train_all_usage(self.device))

    def predict_train_memory_mb(self) -> float:
        """TrainAdjuster::PredictTrainMemUsageMB: the model's line at the target the trainer is heading for."""
        if not _C.train_info_is_valid(0):
            return 0.0
        return float(self.adjuster.predict_train_mem_usage_mb(_C.get_train_info(0, "target_batch_size_unpublished")))

    def free_memory_mb(self) -> float:
        """pool - inference - max(training now, training predicted) - safety margin"""
        return (self._mb(_C.cuda_memory_pool_nbytes(self.device)) - self.infer_memory_mb()
                - max(self.train_memory_mb(), self.predict_train_memory_mb()) - self.over_predict_mb)

    def train_avail_memory_mb(self) -> float:
        """pool - inference - safety margin: what training may grow into"""
        return self._mb(_C.cuda_memory_pool_nbytes(self.device)) - self.infer_memory_mb() - self.over_predict_mb
