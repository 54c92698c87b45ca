"""Python half of the inference<->training handover (pytorch/torch_col/colocate_ctrl.py:30-572).

The reference hangs forward / backward hooks on every leaf nn.Module; the step here is a recorded
launch program cut into one segment per layer, and the same hook bodies run between segments
(`engine.set_checkpoint_hook`).  Class names, the exceptions and where they are raised, the stage
timings of the adjust line and the event names follow the reference.
"""
import abc
import contextlib
import os
import time
from typing import List, Optional, Union

from . import _C, xsched
from ._C import ColocateCtrlHookMode, CtrlEvent, TrainMode
from .util import EventManager, MemoryPool


def register_saved_tensor_hook():
    """colocate_ctrl.py:18-27 tags every tensor autograd saves; activations here belong to the
    engine's plan, which registers itself as their owner when it is hooked."""
    return None


class CtrlBase(abc.ABC):
    _colocate_ctrl = None

    def __init__(self, train_mode: TrainMode, hook_mode: ColocateCtrlHookMode, num_epoch: int, batch_size: int):
        if CtrlBase._colocate_ctrl is not None:
            raise RuntimeError("Only one instance of Colocate Ctrl can be created.")
        CtrlBase._colocate_ctrl = self
        self.train_mode = train_mode
        self.hook_mode = hook_mode
        self.input_batch_size = batch_size
        self.num_epoch = num_epoch
        self._stub = None
        self._grad_fn = None

    @classmethod
    def _reset_singleton(cls):
        """Lets one process build a second controller after the first was stopped (tests)."""
        CtrlBase._colocate_ctrl = None

    @abc.abstractmethod
    def steps_no_interrupt(self):
        ...

    @abc.abstractmethod
    def register_pytorch_hook(self, module_list):
        ...

    def release_and_reply(self, barrier: Optional[bool] = None):
        if self.train_mode.is_colocate():
            return self.adjust()
        if self.train_mode.is_taskswitch():
            assert barrier is not None
            return self.switch(barrier)

    @abc.abstractmethod
    def report_batch_size(self, batch_size):
        ...

    @property
    @abc.abstractmethod
    def target_batch_size(self):
        ...

    @property
    @abc.abstractmethod
    def unpub_target_batch_size(self):
        ...

    def train_start(self):
        self._stub.train_start()

    def train_end(self):
        if _C.is_enable_shared_tensor():
            MemoryPool.empty_cache()
        return self._stub.train_end()

    def stop(self):
        self._stub.stop()

    def can_exit_after_infer_worklaod_done(self):
        return self._stub.can_exit_after_infer_worklaod_done()

    def set_train_first_epoch_done(self):
        self._stub.set_train_first_epoch_done()

    @classmethod
    def register_fbward_hook(cls, module, fwd_hook, bwd_hook):
        """colocate_ctrl.py:101-110: leaves get the hooks.  An engine is one leaf whose segments
        call back with ('fwd' | 'bwd', layer name)."""
        if not _C.is_enable_fbward_hook():
            return
        if hasattr(module, "set_checkpoint_hook"):
            def hook(phase, name):
                if phase == 'fwd':
                    fwd_hook(module, name, None)
                else:
                    bwd_hook(module, name, None)
            module.set_checkpoint_hook(hook)
            _C.register_interm_memory_owner(module.release_activations)


class SwitchL1Exception(Exception):
    pass


class ColocateAdjustL1Exception(Exception):
    pass


class EngineColocateAdjustL1Exception(Exception):
    pass


def _used_gb():
    return MemoryPool.get_memory_usage(), MemoryPool.get_allocated_memory()


class SwitchCtrl(CtrlBase):
    """colocate_ctrl.py:117-301"""

    def __init__(self, train_mode, hook_mode, num_epoch, batch_size):
        assert train_mode in {TrainMode.TASKSWITCH_L1, TrainMode.TASKSWITCH_L0}
        super().__init__(train_mode, hook_mode, num_epoch, batch_size)
        self._stub = _C.PySwitchStub()
        self._grad_fn = []

    def _interrupted(self):
        return self._stub.cmd == CtrlEvent.kInterruptTrain

    @contextlib.contextmanager
    def steps_no_interrupt(self):
        if self.train_mode == TrainMode.TASKSWITCH_L0:
            yield
            return
        if self.hook_mode.use_xsched():
            while xsched.get_xqueue_size() != 0:
                if self._interrupted():
                    xsched.kill_batch()
                    raise SwitchL1Exception('before_critical_section')
        _C.SyncAllStreams()
        if self._interrupted():
            raise SwitchL1Exception('before_critical_section')
        self._stub.StepsNoInteruptBegin()
        if self._interrupted():
            self._stub.StepsNoInteruptEnd()
            raise SwitchL1Exception('before_critical_section')
        yield
        _C.SyncAllStreams()
        self._stub.StepsNoInteruptEnd()
        if _C.get_train_world_size() == 1 and self._interrupted():
            self.switch(barrier=False)

    def register_pytorch_hook(self, module_list):
        if self.train_mode == TrainMode.TASKSWITCH_L0:
            return
        if self.hook_mode == ColocateCtrlHookMode.XSCHED_SYNC2:
            self._stub.EnableTorchColEngine()
        for module in module_list:
            CtrlBase.register_fbward_hook(module, self.get_fwd_hook(), self.get_bwd_hook())

    def _hook(self, where):
        sync = self.hook_mode == ColocateCtrlHookMode.SYNC
        if not sync and not self.hook_mode.use_xsched():
            raise RuntimeError(f"Unsupported hook_mode: {self.hook_mode.name}")

        def hook(module, input, output):
            if sync:
                _C.SyncAllStreams()
            if self._interrupted():
                if not sync:
                    xsched.kill_batch()
                raise SwitchL1Exception(f"[Task Switch {where}]")
        return hook

    def get_fwd_hook(self):
        return self._hook("FWD")

    def get_bwd_hook(self):
        return self._hook("BWD")

    def switch(self, barrier: bool):
        if self.train_mode == TrainMode.TASKSWITCH_L1:
            return self.switch_l1(barrier)
        raise RuntimeError(f"Unsupported train_mode: {self.train_mode.name}")

    def switch_l1(self, barrier: bool):
        t0 = time.time()
        _C.release_interm_memory()
        old_gpu_mem = MemoryPool.get_memory_usage()
        MemoryPool.empty_cache()
        cur_gpu_mem = MemoryPool.get_memory_usage()
        succ = self.try_reply_interrupt(barrier)
        t1 = time.time()
        if succ:
            print(f'[Switch L1 {(t1-t0)*1e3:.1f} ms] target batch_size: {self.target_batch_size}, '
                  f'memory usage: {old_gpu_mem:.2f}GB -> {cur_gpu_mem:.2f}GB.', flush=True)
        return succ

    def try_reply_interrupt(self, barrier):
        return self._stub.try_interrupt_train_done(barrier)

    @property
    def target_batch_size(self):
        return self.input_batch_size

    @property
    def unpub_target_batch_size(self):
        return self.input_batch_size

    def report_batch_size(self, batch_size):
        self._stub.report_batch_size(batch_size)

    def set_killed_batch_recover(self):
        self._stub.set_killed_batch_recover()


class ColocateCtrl(CtrlBase):
    """colocate_ctrl.py:310-503"""

    def __init__(self, train_mode, hook_mode, num_epoch, batch_size):
        assert train_mode in (TrainMode.COLOCATE_L1, TrainMode.COLOCATE_L2)
        super().__init__(train_mode, hook_mode, num_epoch, batch_size)
        self._stub = _C.PyColocateStub(batch_size)
        self._grad_fn = []
        self.last_adjust = None  # stage timings (ms) and bytes of the most recent adjust

    def _adjust_l1_pending(self):
        return self._stub.cmd == CtrlEvent.kColocateAdjustL1

    @contextlib.contextmanager
    def steps_no_interrupt(self):
        if self.train_mode == TrainMode.COLOCATE_L1:
            # drain the launch queue first so that the critical section starts with nothing pending
            if self.hook_mode.use_xsched():
                while xsched.get_xqueue_size() != 0:
                    if self._adjust_l1_pending():
                        xsched.kill_batch()
                        raise ColocateAdjustL1Exception('before_critical_section')
            _C.SyncAllStreams()
            if self._adjust_l1_pending():
                raise ColocateAdjustL1Exception('before_critical_section')
            self._stub.StepsNoInteruptBegin()
            if self._adjust_l1_pending():
                self._stub.StepsNoInteruptEnd()
                raise ColocateAdjustL1Exception('before_critical_section')
            yield
            _C.SyncAllStreams()
            self._stub.StepsNoInteruptEnd()
            # a request that arrived during the step is served right after it: nothing is in flight
            if _C.get_train_world_size() == 1 and self._adjust_l1_pending():
                with EventManager.record_duration_event('adjust_after_step'):
                    self.adjust()
        else:
            self._stub.StepsNoInteruptBegin()
            yield
            self._stub.StepsNoInteruptEnd()

    def register_pytorch_hook(self, module_list):
        if self.train_mode != TrainMode.COLOCATE_L1:
            return
        if self.hook_mode == ColocateCtrlHookMode.SYNC:
            def fwd_hook(module, input, output):
                with EventManager.record_duration_event('sync_fwd'):
                    _C.SyncAllStreams()
                    if self._adjust_l1_pending():
                        raise ColocateAdjustL1Exception('[Adjust SYNC FWD]')

            def bwd_hook(module, grad_input, grad_output):
                with EventManager.record_duration_event('sync_bwd'):
                    _C.SyncAllStreams()
                    if self._adjust_l1_pending():
                        raise ColocateAdjustL1Exception('[Adjust SYNC BWD]')
        elif self.hook_mode == ColocateCtrlHookMode.XSCHED_SYNC2:
            # the control thread kills on receipt; the engine notices the rejected launches
            print("SetUpTorchColEngine")
            self._stub.EnableTorchColEngine()
            for module in module_list:
                if hasattr(module, "set_cut_exception"):
                    module.set_cut_exception(EngineColocateAdjustL1Exception)
                    _C.register_interm_memory_owner(module.release_activations)
            return
        elif self.hook_mode.use_xsched():
            # one event per layer would swamp the log at 310 segments a step: the checks are silent
            def fwd_hook(module, input, output):
                if self._adjust_l1_pending():
                    xsched.kill_batch()
                    raise ColocateAdjustL1Exception('[Adjust XSCHED_SYNC FWD]')

            def bwd_hook(module, grad_input, grad_output):
                if self._adjust_l1_pending():
                    xsched.kill_batch()
                    raise ColocateAdjustL1Exception('[Adjust XSCHED_SYNC BWD]')
        else:
            raise RuntimeError(f"Unsupported hook_mode: {self.hook_mode.name}")
        for module in module_list:
            CtrlBase.register_fbward_hook(module, fwd_hook, bwd_hook)

    def adjust(self):
        if self.train_mode == TrainMode.COLOCATE_L1:
            return self.adjust_l1()
        if self.train_mode == TrainMode.COLOCATE_L2:
            return self.adjust_l2()
        raise RuntimeError(f"Unsupported train_mode: {self.train_mode.name}")

    def adjust_l1(self):
        """colocate_ctrl.py:413-445: release activations | return whole pages | reply | read usage."""
        t0 = time.time()
        with EventManager.record_duration_event('adjust_l1'):
            old_cached, old_alloc = _used_gb()
            released = _C.release_interm_memory()
            t1 = time.time()
            freed = MemoryPool.empty_cache()
            t2 = time.time()
            self._stub.adjust_l1_done()
            t3 = time.time()
            cur_cached, cur_alloc = _used_gb()
        t4 = time.time()
        self.last_adjust = {"release_ms": (t1 - t0) * 1e3, "empty_cache_ms": (t2 - t1) * 1e3,
                            "reply_ms": (t3 - t2) * 1e3, "stat_ms": (t4 - t3) * 1e3,
                            "released_bytes": released, "pool_bytes_returned": freed}
        print(f'[Rank {_C.get_train_rank()} | PID {os.getpid()} | {_C.get_unix_timestamp_us()/1000}]'
              f' [Adjust L1 {(t1-t0)*1e3:.1f} | {(t2-t1)*1e3:.1f} | {(t3-t2)*1e3:.1f} | {(t4-t3)*1e3:.1f} ms]'
              f' target batch_size: {self.target_batch_size},'
              f' memory cached: {old_cached:.2f}GB -> {cur_cached:.2f}GB,'
              f' memory allocated: {old_alloc:.2f}GB -> {cur_alloc:.2f}GB.', flush=True)

    def adjust_l2(self):
        """colocate_ctrl.py:448-469"""
        t0 = time.time()
        with EventManager.record_duration_event('adjust_l2'):
            old_cached, old_alloc = _used_gb()
            freed = MemoryPool.empty_cache()
            self._stub.adjust_l2_done()
            cur_cached, cur_alloc = _used_gb()
        t1 = time.time()
        self.last_adjust = {"empty_cache_ms": (t1 - t0) * 1e3, "pool_bytes_returned": freed}
        print(f'[{_C.get_unix_timestamp_us()/1000}] [Adjust L2 {(t1-t0)*1e3:.1f} ms]'
              f' target batch_size: {self.target_batch_size},'
              f' memory cached: {old_cached:.2f}GB -> {cur_cached:.2f}GB,'
              f' memory allocated: {old_alloc:.2f}GB -> {cur_alloc:.2f}GB.', flush=True)

    def report_batch_size(self, batch_size):
        self._stub.report_batch_size(batch_size)

    @property
    def target_batch_size(self):
        return self._stub.target_batch_size

    @property
    def unpub_target_batch_size(self):
        return self._stub.unpub_target_batch_size

    def set_killed_batch_recover(self):
        self._stub.set_killed_batch_recover()

    def set_killed_batch_reconfiged(self):
        self._stub.set_killed_batch_reconfiged()


class DummyCtrl(CtrlBase):
    """colocate_ctrl.py:506-553"""

    def __init__(self, train_mode, hook_mode, num_epoch, batch_size):
        super().__init__(train_mode, hook_mode, num_epoch, batch_size)
        self._stub = _C.PyDummyStub()
        assert hook_mode == ColocateCtrlHookMode.NONE

    @contextlib.contextmanager
    def steps_no_interrupt(self):
        yield

    def check_async_killed_batch(self):
        pass

    def register_pytorch_hook(self, module_list):
        pass

    def report_batch_size(self, batch_size):
        pass

    @property
    def target_batch_size(self):
        return self.input_batch_size

    @property
    def unpub_target_batch_size(self):
        return self.input_batch_size

    def train_end(self):
        self._stub.train_end()


def create_colocate_ctrl(train_mode: TrainMode, hook_mode: ColocateCtrlHookMode, num_epoch: int,
                         batch_size: int) -> Union[DummyCtrl, ColocateCtrl, SwitchCtrl]:
    if train_mode == TrainMode.NORMAL:
        return DummyCtrl(train_mode, hook_mode, num_epoch, batch_size)
    if train_mode.is_colocate():
        return ColocateCtrl(train_mode, hook_mode, num_epoch, batch_size)
    if train_mode.is_taskswitch() or train_mode == TrainMode.TASKSWITCH_L0:
        return SwitchCtrl(train_mode, hook_mode, num_epoch, batch_size)
    raise RuntimeError(f"Unsupported train_mode: {train_mode}")


def get_colocate_ctrl() -> Union[DummyCtrl, ColocateCtrl, SwitchCtrl]:
    assert CtrlBase._colocate_ctrl is not None
    return CtrlBase._colocate_ctrl
