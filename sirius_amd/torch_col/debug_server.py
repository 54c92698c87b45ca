"""Minimal stand-in for the inference server that sends adjust commands by hand
(pytorch/torch_col/debug_server.py:5-61)."""
import threading

from . import _C
from ._C import CtrlEvent


class DebugServer:
    def __init__(self, train_world_size, verbose=True):
        self._cmd_ids = {}
        self._inf_tra_comm = _C.PyInfTraCommunicator(True, True, train_world_size)
        self._verbose = verbose
        self.received = []
        self._running = True
        self._thread = threading.Thread(target=self._recv_from_train, daemon=True)
        self._thread.start()

    def _send(self, event, batch_size):
        cmd_id = self._cmd_ids[event] = self._cmd_ids.get(event, 0) + 1
        # the real server writes the new target on the information board before it sends the
        # command (server/train_adjuster.cc FillAdjustPlan); the trainer publishes it when it
        # redistributes the batch
        from .._lib import lib
        if lib().tch_train_info_is_valid(0):
            lib().tch_train_info_set_field(0, 6, int(batch_size))
        self._inf_tra_comm.put_inf2tra(_C.PyCtrlMsgEntry(cmd_id, event, batch_size), 0)
        return cmd_id

    def colocate_l1(self, batch_size: int):
        return self._send(CtrlEvent.kColocateAdjustL1, batch_size)

    def colocate_l2(self, batch_size: int):
        return self._send(CtrlEvent.kColocateAdjustL2, batch_size)

    def infer_exit(self, batch_size: int):
        return self._send(CtrlEvent.kInferExit, batch_size)

    # -- compute units the inference side wants for itself (SMPartitioner::SetInferRequiredTpcNum)
    def set_infer_required_cus(self, n: int, device: int = 0):
        _C.set_infer_required_cus(n, device)

    # -- task switching (the controller's pair of commands, server/control/controller.cc:207-260)
    def interrupt_train(self):
        cmd_id = self._cmd_ids[CtrlEvent.kInterruptTrain] = self._cmd_ids.get(CtrlEvent.kInterruptTrain, 0) + 1
        self._inf_tra_comm.put_inf2tra(_C.PyCtrlMsgEntry(cmd_id, CtrlEvent.kInterruptTrain, 0), 0)
        return cmd_id

    def resume_train(self):
        cmd_id = self._cmd_ids[CtrlEvent.kResumeTrain] = self._cmd_ids.get(CtrlEvent.kResumeTrain, 0) + 1
        self._inf_tra_comm.put_inf2tra(_C.PyCtrlMsgEntry(cmd_id, CtrlEvent.kResumeTrain, 0), 0)
        return cmd_id

    # -- requests in megabytes, through the server's own arithmetic (server/train_adjuster.cc)
    def require_memory_mb(self, required_mem_mb: float, adjuster=None):
        """Inference needs required_mem_mb more: shrink training by ceil(MB / slope) samples."""
        from .train_adjuster import TrainAdjuster
        adjuster = adjuster or TrainAdjuster()
        target = adjuster.infer_require_mem_adjust_plan(required_mem_mb)
        if target is None:
            return None
        self.colocate_l1(target)
        return target

    def release_memory_mb(self, avail_mem_mb: float, adjuster=None):
        """Inference left avail_mem_mb to training: grow to what fits (at most the initial size)."""
        from .train_adjuster import TrainAdjuster
        adjuster = adjuster or TrainAdjuster()
        target = adjuster.infer_release_mem_adjust_plan(avail_mem_mb)
        self.infer_exit(target)
        return target

    def _recv_from_train(self):
        while self._running:
            msg = self._inf_tra_comm.timed_get_tra2inf(10, 0)
            if msg is None:
                continue
            self.received.append((_C.get_unix_timestamp_us(), msg))
            if self._verbose and msg.event != CtrlEvent.kReportBatchSize:
                print(f'timestamp {_C.get_unix_timestamp()}: {msg}')

    def stop(self):
        self._running = False
        self._thread.join()
