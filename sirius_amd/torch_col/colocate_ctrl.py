"""Training's side of the handover protocol: when may a micro-batch be cut, what happens to the memory, what is
answered.  Public names, exception types, event names and the `[Adjust L1 ...]` report line are those of the
reference's controllers (pytorch/torch_col/colocate_ctrl.py:30-572); the bodies are written for this engine.

The engine's step is a recorded program of launches with a checkpoint after every layer.  A controller is
therefore three small things:

  * a *pending test*: "is the command that interrupts training set on the stub?"
    (kColocateAdjustL1 for colocation, kInterruptTrain for task switching);
  * a *checkpoint callback* the engine calls between launch segments, chosen by hook mode from one table
    (_CHECKPOINT_STYLES): synchronise then look, look then kill the queued launches, or nothing at all because
    the control thread kills on receipt and the engine raises when its launches are rejected;
  * a *critical section* around the optimizer step (`steps_no_interrupt`), the same sequence for both
    controllers: drain the launch queue, synchronise, announce the section to the stub, look once more -- and
    after the section serve a command that arrived meanwhile, when nothing is in flight.
"""
import abc
import contextlib
import os
import time
from typing import Callable, Optional, Union

from . import _C, xsched
from ._C import ColocateCtrlHookMode, CtrlEvent, TrainMode
from .util import EventManager, MemoryPool


class SwitchL1Exception(Exception):
    pass


class ColocateAdjustL1Exception(Exception):
    pass


class EngineColocateAdjustL1Exception(Exception):
    pass


def register_saved_tensor_hook():
    """The reference tags every tensor autograd saves (colocate_ctrl.py:18-27); here a plan owns its
    activations and the engine is registered as their owner when it is hooked."""
    return None


# hook mode -> (synchronise before looking, kill the queued launches when the command is there)
_CHECKPOINT_STYLES = {
    ColocateCtrlHookMode.SYNC: (True, False),
    ColocateCtrlHookMode.XSCHED_SYNC: (False, True),
    ColocateCtrlHookMode.XSCHED_SYNC2: (False, True),
}


class CtrlBase(abc.ABC):
    _colocate_ctrl = None

    #: what a cut raises and the first word of its message ("[Adjust XSCHED_SYNC FWD]" / "[Task Switch FWD]")
    interrupt_exception = RuntimeError
    interrupt_label = ""

    def __init__(self, train_mode: TrainMode, hook_mode: ColocateCtrlHookMode, num_epoch: int, batch_size: int):
        if CtrlBase._colocate_ctrl is not None:
            raise RuntimeError("Only one instance of Colocate Ctrl can be created.")
        CtrlBase._colocate_ctrl = self
        self.train_mode, self.hook_mode = train_mode, hook_mode
        self.num_epoch, self.input_batch_size = num_epoch, batch_size
        self._stub = None
        self._grad_fn = None

    @classmethod
    def _reset_singleton(cls):
        """One process may build a second controller after the first was stopped (tests)."""
        CtrlBase._colocate_ctrl = None

    # ---- what differs between the controllers ----
    def _pending(self) -> bool:
        """The command that interrupts training is waiting on the stub."""
        return False

    def _interruptible(self) -> bool:
        """This train mode cuts micro-batches at all."""
        return False

    def _serve_after_step(self):
        """A command arrived during the optimizer step; nothing is in flight now."""

    # ---- the critical section around the optimizer step ----
    @contextlib.contextmanager
    def steps_no_interrupt(self):
        if not self._interruptible():
            self._begin_plain_section()
            yield
            self._end_plain_section()
            return
        where = 'before_critical_section'
        if self.hook_mode.use_xsched():
            # what is still queued in software has not started: it can be dropped instead of waited for
            while xsched.get_xqueue_size() != 0:
                if self._pending():
                    xsched.kill_batch()
                    raise self.interrupt_exception(where)
        _C.SyncAllStreams()
        if self._pending():
            raise self.interrupt_exception(where)
        self._stub.StepsNoInteruptBegin()
        if self._pending():      # set between the look and the announcement
            self._stub.StepsNoInteruptEnd()
            raise self.interrupt_exception(where)
        yield
        _C.SyncAllStreams()
        self._stub.StepsNoInteruptEnd()
        if _C.get_train_world_size() == 1 and self._pending():
            self._serve_after_step()

    def _begin_plain_section(self):
        pass

    def _end_plain_section(self):
        pass

    # ---- checkpoints between the launch segments of the engines ----
    def _checkpoint(self) -> Callable[[str, str], None]:
        """fn(phase, layer): runs after every layer of a forward / backward replay."""
        style = _CHECKPOINT_STYLES.get(self.hook_mode)
        if style is None:
            raise RuntimeError(f"Unsupported hook_mode: {self.hook_mode.name}")
        sync_first, kill_queue = style
        mode = self.hook_mode.name if self.interrupt_label == "Adjust" else ""

        def checkpoint(phase, layer):
            if sync_first:
                with EventManager.record_duration_event('sync_fwd' if phase == 'fwd' else 'sync_bwd'):
                    _C.SyncAllStreams()
            if not self._pending():
                return
            if kill_queue:
                xsched.kill_batch()
            tag = " ".join(w for w in (self.interrupt_label, mode, phase.upper()[:3]) if w)
            raise self.interrupt_exception(f"[{tag}]")
        return checkpoint

    def get_fwd_hook(self):
        cp = self._checkpoint()
        return lambda module, input, output: cp('fwd', getattr(module, '__name__', ''))

    def get_bwd_hook(self):
        cp = self._checkpoint()
        return lambda module, grad_input, grad_output: cp('bwd', getattr(module, '__name__', ''))

    @classmethod
    def register_fbward_hook(cls, module, fwd_hook, bwd_hook):
        """The reference hangs the pair on every leaf module (colocate_ctrl.py:101-110); an engine is one leaf
        that calls back per layer with ('fwd' | 'bwd', layer name)."""
        if not _C.is_enable_fbward_hook() or not hasattr(module, "set_checkpoint_hook"):
            return
        module.set_checkpoint_hook(lambda phase, name: (fwd_hook if phase == 'fwd' else bwd_hook)(module, name, None))
        _C.register_interm_memory_owner(module.release_activations)

    def register_pytorch_hook(self, module_list):
        if not self._interruptible():
            return
        if self.hook_mode == ColocateCtrlHookMode.XSCHED_SYNC2:
            self._stub.EnableTorchColEngine()
        if self.hook_mode == ColocateCtrlHookMode.XSCHED_SYNC2 and self.interrupt_label == "Adjust":
            # the control thread kills on receipt; the engine notices its rejected launches and raises
            print("SetUpTorchColEngine")
            for engine in module_list:
                if hasattr(engine, "set_cut_exception"):
                    engine.set_cut_exception(EngineColocateAdjustL1Exception)
                    _C.register_interm_memory_owner(engine.release_activations)
            return
        checkpoint = self._checkpoint()
        if not _C.is_enable_fbward_hook():
            return
        for engine in module_list:
            if hasattr(engine, "set_checkpoint_hook"):
                engine.set_checkpoint_hook(checkpoint)
                _C.register_interm_memory_owner(engine.release_activations)

    # ---- release and reply ----
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

    # ---- life cycle ----
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


def _give_memory_back():
    """The memory half of every reply: the plans' activations go back to the allocator, whole pages go back to
    the pool (unmapped from this process unless the pool runs in lazy mode).  Returns
    (activation bytes released, pool bytes returned, ms for the first, ms for the second)."""
    t0 = time.time()
    from .dynamic_batch import DynamicBatchDataset      # the micro-batch copied ahead of time is memory too
    if DynamicBatchDataset._dynamic_batch_dataset is not None:
        DynamicBatchDataset._dynamic_batch_dataset._samples.drop_prefetched()
    released = _C.release_interm_memory()
    t1 = time.time()
    returned = MemoryPool.empty_cache()
    t2 = time.time()
    return released, returned, (t1 - t0) * 1e3, (t2 - t1) * 1e3


def _used_gb():
    return MemoryPool.get_memory_usage(), MemoryPool.get_allocated_memory()


class SwitchCtrl(CtrlBase):
    """Task switching: inference interrupts training altogether and resumes it later
    (colocate_ctrl.py:117-301)."""
    interrupt_exception = SwitchL1Exception
    interrupt_label = "Task Switch"

    def __init__(self, train_mode, hook_mode, num_epoch, batch_size):
        assert train_mode in {TrainMode.TASKSWITCH_L1, TrainMode.TASKSWITCH_L0}
        super().__init__(train_mode, hook_mode, num_epoch, batch_size)
        self._stub = _C.PySwitchStub()
        self._grad_fn = []

    def _pending(self):
        return self._stub.cmd == CtrlEvent.kInterruptTrain

    def _interruptible(self):
        return self.train_mode != TrainMode.TASKSWITCH_L0

    def _serve_after_step(self):
        self.switch(barrier=False)

    def switch(self, barrier: bool):
        if self.train_mode != TrainMode.TASKSWITCH_L1:
            raise RuntimeError(f"Unsupported train_mode: {self.train_mode.name}")
        return self.switch_l1(barrier)

    def switch_l1(self, barrier: bool):
        began = time.time()
        before = MemoryPool.get_memory_usage()
        _give_memory_back()
        after = MemoryPool.get_memory_usage()
        acknowledged = self.try_reply_interrupt(barrier)
        if acknowledged:
            print(f'[Switch L1 {(time.time() - began) * 1e3:.1f} ms] target batch_size: {self.target_batch_size}, '
                  f'memory usage: {before:.2f}GB -> {after:.2f}GB.', flush=True)
        return acknowledged

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
    """Colocation: inference asks for memory, training shrinks its batch (L1: at once, killing the micro-batch
    in flight; L2: at the end of it) and grows back when told (colocate_ctrl.py:310-503)."""
    interrupt_exception = ColocateAdjustL1Exception
    interrupt_label = "Adjust"

    def __init__(self, train_mode, hook_mode, num_epoch, batch_size):
        assert train_mode in (TrainMode.COLOCATE_L1, TrainMode.COLOCATE_L2)
        super().__init__(train_mode, hook_mode, num_epoch, batch_size)
        self._stub = _C.PyColocateStub(batch_size)
        self._grad_fn = []
        #: the most recent adjust: stage timings in ms, bytes released / returned, stale mappings left
        self.last_adjust = None

    def _pending(self):
        return self._stub.cmd == CtrlEvent.kColocateAdjustL1

    def _interruptible(self):
        return self.train_mode == TrainMode.COLOCATE_L1

    def _serve_after_step(self):
        with EventManager.record_duration_event('adjust_after_step'):
            self.adjust()

    # L2 never cuts a micro-batch: its section only tells the stub that a step is running
    def _begin_plain_section(self):
        self._stub.StepsNoInteruptBegin()

    def _end_plain_section(self):
        self._stub.StepsNoInteruptEnd()

    def adjust(self):
        if self.train_mode == TrainMode.COLOCATE_L1:
            return self.adjust_l1()
        if self.train_mode == TrainMode.COLOCATE_L2:
            return self.adjust_l2()
        raise RuntimeError(f"Unsupported train_mode: {self.train_mode.name}")

    def adjust_l1(self):
        """Release | return pages | reply | read usage: the four stage times of the report line
        (colocate_ctrl.py:413-445)."""
        with EventManager.record_duration_event('adjust_l1'):
            cached0, alloc0 = _used_gb()
            released, returned, release_ms, pages_ms = _give_memory_back()
            t = time.time()
            self._stub.adjust_l1_done()
            reply_ms = (time.time() - t) * 1e3
            t = time.time()
            cached1, alloc1 = _used_gb()
        stat_ms = (time.time() - t) * 1e3
        # lazy pools answer first and take the mappings of the pages they gave away down afterwards (a peer that
        # has claimed such a page waits for its flag in the page table before it maps it)
        t = time.time()
        trimmed = MemoryPool.trim_stale_mappings()
        trim_ms = (time.time() - t) * 1e3
        self.last_adjust = {"release_ms": release_ms, "empty_cache_ms": pages_ms, "reply_ms": reply_ms,
                            "stat_ms": stat_ms, "released_bytes": released, "pool_bytes_returned": returned,
                            "trimmed_after_reply": trimmed, "trim_after_reply_ms": trim_ms,
                            "stale_pages_after": MemoryPool.stale_pages()}
        print(f'[Rank {_C.get_train_rank()} | PID {os.getpid()} | {_C.get_unix_timestamp_us()/1000}]'
              f' [Adjust L1 {release_ms:.1f} | {pages_ms:.1f} | {reply_ms:.1f} | {stat_ms:.1f} ms]'
              f' target batch_size: {self.target_batch_size},'
              f' memory cached: {cached0:.2f}GB -> {cached1:.2f}GB,'
              f' memory allocated: {alloc0:.2f}GB -> {alloc1:.2f}GB.', flush=True)

    def adjust_l2(self):
        """colocate_ctrl.py:448-469: nothing is in flight at the end of a micro-batch; cached pages go back."""
        began = time.time()
        with EventManager.record_duration_event('adjust_l2'):
            cached0, alloc0 = _used_gb()
            returned = MemoryPool.empty_cache()
            self._stub.adjust_l2_done()
            cached1, alloc1 = _used_gb()
        took_ms = (time.time() - began) * 1e3
        self.last_adjust = {"empty_cache_ms": took_ms, "pool_bytes_returned": returned}
        print(f'[{_C.get_unix_timestamp_us()/1000}] [Adjust L2 {took_ms:.1f} ms]'
              f' target batch_size: {self.target_batch_size},'
              f' memory cached: {cached0:.2f}GB -> {cached1:.2f}GB,'
              f' memory allocated: {alloc0:.2f}GB -> {alloc1:.2f}GB.', flush=True)

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
    """Training alone on the GPU: nobody interrupts (colocate_ctrl.py:506-553)."""

    def __init__(self, train_mode, hook_mode, num_epoch, batch_size):
        super().__init__(train_mode, hook_mode, num_epoch, batch_size)
        self._stub = _C.PyDummyStub()
        assert hook_mode == ColocateCtrlHookMode.NONE

    def check_async_killed_batch(self):
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
        kind = DummyCtrl
    elif train_mode.is_colocate():
        kind = ColocateCtrl
    elif train_mode.is_taskswitch() or train_mode == TrainMode.TASKSWITCH_L0:
        kind = SwitchCtrl
    else:
        raise RuntimeError(f"Unsupported train_mode: {train_mode}")
    return kind(train_mode, hook_mode, num_epoch, batch_size)


def get_colocate_ctrl() -> Union[DummyCtrl, ColocateCtrl, SwitchCtrl]:
    assert CtrlBase._colocate_ctrl is not None
    return CtrlBase._colocate_ctrl
