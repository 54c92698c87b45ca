"""Python-visible names of the reference's compiled module `torch_col._C._main`
(pytorch/torch_col/cython/main.pyx, ctrl_stub.pxi, util_cls.pxi), bound to the flat C ABI of
libtorch_col_hip.so.  Names, argument meaning and return values follow the .pyx; where the
reference aborts the process on a native failure this module raises TorchColHipError.
"""
import ctypes
import enum
import os
import sys
import threading
import time
import weakref

from .._lib import CtrlMsg, TorchColHipError, check, check_host, lib

# ---------------------------------------------------------------------------------- enums


class ColocateCtrlHookMode(enum.Enum):
    """cython/util_cls.pxi:7-16"""
    NONE = 'none'
    SYNC = 'sync'
    XSCHED_SYNC = 'xsched-sync'
    XSCHED_SYNC2 = 'xsched-sync2'

    def use_xsched(self):
        return self in {ColocateCtrlHookMode.XSCHED_SYNC, ColocateCtrlHookMode.XSCHED_SYNC2}


class TrainMode(enum.Enum):
    """cython/util_cls.pxi:19-39"""
    NORMAL = 'normal'
    COLOCATE_L1 = 'colocate-l1'
    COLOCATE_L2 = 'colocate-l2'
    TASKSWITCH_L0 = 'taskswitch-l0'
    TASKSWITCH_L1 = 'taskswitch-l1'
    TASKSWITCH_L2 = 'taskswitch-l2'
    TASKSWITCH_L3 = 'taskswitch-l3'

    def is_normal(self):
        return self == TrainMode.NORMAL

    def is_colocate(self):
        return self in {TrainMode.COLOCATE_L1, TrainMode.COLOCATE_L2}

    def is_kill_batch(self):
        return self in {TrainMode.COLOCATE_L1, TrainMode.TASKSWITCH_L1}

    def is_taskswitch(self):
        return self in {TrainMode.TASKSWITCH_L1, TrainMode.TASKSWITCH_L2, TrainMode.TASKSWITCH_L3}


class CtrlEvent(enum.IntEnum):
    """common/inf_tra_comm/message_queue.h:18-40; cython/main.pyx:347-368.  Values 0..12."""
    kTrainStart = 0
    kTrainEnd = 1
    kInterruptTrainDone = 2
    kResumeTrainDone = 3
    kColocateAdjustL1Done = 4
    kColocateAdjustL2Done = 5
    kReportBatchSize = 6
    kInterruptTrain = 7
    kResumeTrain = 8
    kColocateAdjustL1 = 9
    kColocateAdjustL2 = 10
    kInferExit = 11
    kInferenceWorkloadDone = 12
    kNumEvent = 13


_INF2TRA, _TRA2INF = 0, 1

# ---------------------------------------------------------------------------------- init / config


def torch_col_init(train_rank=0, train_world_size=1, use_gpu=None):
    """main.pyx:140-143 -> TorchColInit (csrc/init.cc:17-41).  use_gpu=False builds the CPU model
    of the HBM pool (tests without a device); None picks by whether a GPU is visible."""
    if use_gpu is None:
        import torch
        use_gpu = torch.cuda.is_available()
    check_host(lib().tch_TorchColInit(train_rank, train_world_size, 1 if use_gpu else 0), "torch_col_init")


def torch_col_shutdown():
    lib().tch_TorchColShutdown()


def is_configured():
    return bool(lib().tch_TorchColConfig_IsConfigured())


def is_enable_shared_tensor():
    return bool(lib().tch_TorchColConfig_IsEnableSharedTensor())


def is_enable_dynamic_sm_partition():
    return bool(lib().tch_TorchColConfig_IsEnableDynamicSmPartition())


def is_enable_xsched():
    return bool(lib().tch_TorchColConfig_IsEnableXsched())


def kill_batch_on_recv():
    return bool(lib().tch_TorchColConfig_KillBatchOnRecv())


def get_colocate_ctrl_hook_mode():
    return ColocateCtrlHookMode(lib().tch_TorchColConfig_GetColocateCtrlHookMode().decode())


def get_colocate_train_mode():
    return TrainMode(lib().tch_TorchColConfig_GetColocateTrainMode().decode())


def is_release_interm_memory_v1():
    return bool(lib().tch_TorchColConfig_IsReleaseIntermMemoryByGradFn())


def is_release_interm_memory_v2():
    return bool(lib().tch_TorchColConfig_IsReleaseIntermMemoryByTagging())


def disable_release_interm_memory():
    lib().tch_TorchColConfig_SetReleaseIntermMemoryByGradFn(0)
    lib().tch_TorchColConfig_SetReleaseIntermMemoryByTagging(0)


_fbward_hook_disabled = False


def disable_fbward_hook():
    global _fbward_hook_disabled
    _fbward_hook_disabled = True


def is_enable_fbward_hook():
    return bool(lib().tch_TorchColConfig_IsEnableFbwardHook()) and not _fbward_hook_disabled


def is_train_master():
    return bool(lib().tch_TorchColConfig_IsTrainMaster())


def get_train_rank():
    return int(lib().tch_TorchColConfig_GetTrainRank())


def set_train_rank(rank):
    lib().tch_TorchColConfig_SetTrainRank(int(rank))


def get_train_world_size():
    return int(lib().tch_TorchColConfig_GetTrainWorldSize())


def set_train_world_size(world_size):
    lib().tch_TorchColConfig_SetTrainWorldSize(int(world_size))


def set_train_rank_world_size(rank, world_size):
    set_train_rank(rank)
    set_train_world_size(world_size)


def has_colocated_infer_server():
    return bool(lib().tch_TorchColConfig_HasColocatedInferServer())


def get_train_profile_log_path():
    return lib().tch_TorchColConfig_GetTrainProfileLogPath().decode()


def get_shared_tensor_pool_gb():
    return float(lib().tch_TorchColConfig_GetSharedTensorPoolGb())


# ---------------------------------------------------------------------------------- memory


def cuda_memory_pool_infer_usage(device_id):
    return int(lib().tch_cuda_memory_pool_infer_usage(device_id))


def cuda_memory_pool_train_usage(device_id):
    return int(lib().tch_cuda_memory_pool_train_usage(device_id))


def cuda_memory_pool_train_peak_usage(device_id):
    return int(lib().tch_cuda_memory_pool_train_peak_usage(device_id))


def cuda_memory_pool_train_all_usage(device_id):
    return int(lib().tch_cuda_memory_pool_train_all_usage(device_id))


def cuda_memory_pool_free_train_local(device_id):
    return int(lib().tch_cuda_memory_pool_free_train_local(device_id))


def pool_counters(device_id):
    c = (ctypes.c_uint64 * 6)()
    lib().tch_pool_counters(device_id, c)
    out = dict(zip(("allocs", "frees", "maps", "unmaps", "revives", "stale"), (int(v) for v in c)))
    out["unmap_calls"] = int(lib().tch_pool_unmap_calls(device_id))
    return out


def pool_trim(device_id, max_pages=1 << 30):
    return int(lib().tch_pool_trim(device_id, max_pages))


def cuda_memory_pool_num_free_pages(device_id):
    return int(lib().tch_cuda_memory_pool_num_free_pages(device_id))


def cuda_memory_pool_nbytes(device_id):
    return int(lib().tch_cuda_memory_pool_nbytes(device_id))


class _PoolBlock:
    """Owner of one block of the HBM pool, exported through the CUDA array interface so that
    torch wraps the memory without copying; the block returns to the pool when the last
    tensor viewing it is gone."""

    def __init__(self, device, nbytes, stream):
        self.device, self.nbytes = device, nbytes
        self.generation = lib().tch_pool_generation(device)
        self.ptr = lib().tch_pool_malloc(nbytes, device, stream)
        if not self.ptr:
            raise TorchColHipError(f"pool allocation of {nbytes} bytes failed: "
                                   f"{(lib().tch_host_last_error() or b'').decode()}")
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (self.ptr, False),
                                         "version": 2, "strides": None}

        _live_blocks[self.ptr] = weakref.ref(self)

    def release(self):
        """Give the block back now, whoever still holds a tensor over it (the holder must not
        touch it again): ReleaseUnderlyingStorage of the reference (csrc/util.cc)."""
        if self.ptr:
            _live_blocks.pop(self.ptr, None)
            # a block of a pool that has been shut down meanwhile went away with that pool
            if lib().tch_pool_generation(self.device) == self.generation:
                lib().tch_pool_free(self.ptr, self.nbytes, self.device, None)
            self.ptr = None
            return self.nbytes
        return 0

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


_live_blocks = {}


def pool_release(tensor):
    """Free the pool block under `tensor` at once (no-op for a tensor that is not the start of a
    live pool block).  Returns the bytes released."""
    ref = _live_blocks.get(tensor.data_ptr())
    blk = ref() if ref is not None else None
    return blk.release() if blk is not None else 0


def pool_empty(shape, dtype, device=None):
    """An uninitialised tensor whose storage is a block of the shared HBM pool (the path
    torch.empty takes through CUDAColAllocator::allocate in the reference,
    csrc/torch_allocator_plugin.cc:84-139)."""
    import math
    import torch
    if device is None:
        device = get_train_rank()
    if isinstance(shape, int):
        shape = (shape,)
    itemsize = torch.empty(0, dtype=dtype).element_size()
    n = int(math.prod(shape))
    if n == 0:
        return torch.empty(shape, dtype=dtype, device=f"cuda:{device}")
    stream = torch.cuda.current_stream(device).cuda_stream
    blk = _PoolBlock(device, n * itemsize, stream)
    flat = torch.as_tensor(blk, device=f"cuda:{device}")
    return flat.view(dtype).view(shape)


pool_empty.release = pool_release  # allocator protocol of the engines: allocator(shape, dtype), allocator.release(t)


def install_pluggable_allocator():
    """Route every torch device allocation through the pool (the reference installs its
    CUDAColAllocator before the first allocation, csrc/torch_allocator_plugin.cc:31-58).
    Must run before torch allocates on the device."""
    import torch
    alloc = pluggable_allocator()
    torch.cuda.memory.change_current_allocator(alloc)
    return alloc


_pluggable = None


def pluggable_allocator():
    """torch's view of the pool's allocator hook (tch_pool_malloc / tch_pool_free)."""
    global _pluggable
    if _pluggable is None:
        import torch
        from .._lib import LIB_PATH
        _pluggable = torch.cuda.memory.CUDAPluggableAllocator(LIB_PATH, "tch_pool_malloc", "tch_pool_free")
    return _pluggable


def torch_mem_pool():
    """A torch.cuda.MemPool on the pool's allocator: inside `with torch.cuda.use_mem_pool(p):`
    every torch allocation of this thread is a pool block, without replacing torch's allocator
    for the whole process."""
    import torch
    return torch.cuda.MemPool(pluggable_allocator().allocator())


# memory that is not model state and is dropped on a handover: engines register a callable that
# releases their activations (the role of grad_fn / tagged saved tensors in the reference)
_interm_releasers = []


def register_interm_memory_owner(fn):
    ref = weakref.WeakMethod(fn) if hasattr(fn, "__self__") else (lambda: fn)
    _interm_releasers.append(ref)


def tag_model_start():
    lib().tch_tag_model_start(get_train_rank())


def tag_model_end():
    lib().tch_tag_model_end(get_train_rank())


def tag_interm_memory(tensor):
    return bool(lib().tch_tag_interm_memory(get_train_rank(), tensor.data_ptr()))


def release_interm_memory():
    """ReleaseIntermMemory (csrc/mem_tagging.cc / torch_allocator_plugin.cc:343-369): every
    registered owner drops its activations, then any explicitly tagged block is freed."""
    released = 0
    alive = []
    for ref in _interm_releasers:
        fn = ref()
        if fn is not None:
            alive.append(ref)
            released += int(fn() or 0)
    _interm_releasers[:] = alive
    released += int(lib().tch_release_interm_memory(get_train_rank()))
    return released


def untag_interm_memory():
    lib().tch_untag_interm_memory(get_train_rank())


def release_grad_fn_saved_tensor(grad_fn):
    """main.pyx:247-250.  There is no autograd graph on this path; an owner registered with
    register_interm_memory_owner stands where the grad_fn stood."""
    if callable(grad_fn):
        grad_fn()


def release_underlying_storage(tensor):
    tensor.set_(tensor.new_empty(0).untyped_storage(), 0, (0,))


def rearrange_memory():
    """main.pyx:278-280: a no-op hint here, empty_cache already returns whole pages."""
    return None


# ---------------------------------------------------------------------------------- queue control


def RegisterStream(stream):
    h = lib().tch_RegisterStream(int(stream))
    if h == 0:
        raise TorchColHipError("RegisterStream failed: " + (lib().tch_last_error() or b"").decode())
    return h


def UnRegisterStream(stream):
    lib().tch_UnRegisterStream(int(stream))


def UnRegisterAllStreams():
    lib().tch_UnRegisterAllStreams()


def GetXQueueSize(stream):
    return int(lib().tch_GetXQueueSize(int(stream)))


def GetXQueueSizeAllStreams():
    return int(lib().tch_GetXQueueSizeAllStreams())


def GetTotalXQueueSize():
    return int(lib().tch_GetTotalXQueueSize())


def AbortStream(stream):
    return int(lib().tch_AbortStream(int(stream)))


def AbortAllStreams():
    return int(lib().tch_AbortAllStreams())


def SyncStream(stream):
    return int(lib().tch_SyncStream(int(stream)))


def SyncAllStreams():
    return int(lib().tch_SyncAllStreams())


def SetRejectCudaCalls(reject):
    lib().tch_SetRejectCudaCalls(1 if reject else 0)


_guess_nccl = False


def GuessNcclBegin():
    global _guess_nccl
    _guess_nccl = True


def GuessNcclEnd():
    global _guess_nccl
    _guess_nccl = False


def IsGuessNcclBegined():
    return _guess_nccl


def GetNcclStreams():
    """One GPU, no collective streams to discover."""
    return []


_cu_partition = {"on": False}


def SMPartitionInit(stream=None, min_train_cus=8, max_train_cus=0, total_cus=0):
    """csrc/init.cc:43-71: from now on the training launches are confined to the compute units the inference
    side leaves (its demand sits on the shared board, common/sm_partition.cc:60-76).  Compute units take the
    place of the reference's TPCs; the confinement is a CU-masked stream per share instead of a mask per launch.
    `stream` is accepted for the reference's call shape (the engines' contexts pick the masked streams)."""
    check(lib().tch_cu_partition_init(int(total_cus), int(min_train_cus), int(max_train_cus)), "tch_cu_partition_init")
    _cu_partition["on"] = True


def sm_partition_enabled():
    return _cu_partition["on"]


def sm_partition_total():
    return int(lib().tch_cu_partition_total())


def set_infer_required_cus(n, device=0):
    """SMPartitioner::SetInferRequiredTpcNum (the inference side's call; the stand-in peer uses it)."""
    check_host(lib().tch_infer_required_cus_set(int(device), int(n)), "tch_infer_required_cus_set")


def get_train_avail_cus(device=0):
    """SMPartitioner::GetTrainAvailTpcNum: what training may use right now."""
    required = lib().tch_infer_required_cus_get(int(device))
    return int(lib().tch_cu_partition_train_avail(max(0, int(required))))


def monitor_sm_partition(interval):
    """The reference starts a thread that logs the partition every `interval` seconds (csrc/init.cc:60-70);
    here: one line with the state of the moment."""
    if _cu_partition["on"]:
        info(f"[CU partition] total {sm_partition_total()} train may use {get_train_avail_cus()}")
    return None


# ---------------------------------------------------------------------------------- comm


class PyCtrlMsgEntry:
    """main.pyx:413-434"""

    def __init__(self, id, cmd, value):
        self._c = CtrlMsg(int(id), int(cmd), int(value))

    @property
    def event(self):
        return CtrlEvent(self._c.event)

    @property
    def id(self):
        return int(self._c.id)

    @property
    def value(self):
        return int(self._c.value)

    def __repr__(self):
        return f"CtrlMsgEntry(id={self.id}, event={self.event.name}, value={self.value})"


def _msg_from_c(c):
    return PyCtrlMsgEntry(c.id, c.event, c.value)


class PyInfTraCommunicator:
    """main.pyx:436-483.  With all arguments None the already initialised communicator is used."""

    def __init__(self, is_server=None, cleanup=None, train_world_size=None):
        if is_server is None and cleanup is None and train_world_size is None:
            if not lib().tch_InfTraCommunicator_IsInitialized():
                raise TorchColHipError("InfTraCommunicator is not initialized")
        else:
            check_host(lib().tch_InfTraCommunicator_Init(int(bool(is_server)), int(bool(cleanup)),
                                                         int(train_world_size)), "InfTraCommunicator.Init")

    def put_inf2tra(self, entry, id):
        check_host(lib().tch_mq_put(_INF2TRA, id, ctypes.byref(entry._c)), "put")

    def put_all_inf2tra(self, entry):
        check_host(lib().tch_mq_put_all(_INF2TRA, ctypes.byref(entry._c)), "put_all")

    def put_tra2inf(self, entry, id):
        check_host(lib().tch_mq_put(_TRA2INF, id, ctypes.byref(entry._c)), "put")

    def _block_get(self, direction, id):
        out = CtrlMsg()
        check_host(lib().tch_mq_block_get(direction, id, ctypes.byref(out)), "block_get")
        return _msg_from_c(out)

    def block_get_inf2tra(self, id):
        return self._block_get(_INF2TRA, id)

    def block_get_tra2inf(self, id):
        return self._block_get(_TRA2INF, id)

    def _timed_get(self, direction, timeout_ms, id):
        out = CtrlMsg()
        rc = check_host(lib().tch_mq_timed_get(direction, id, int(timeout_ms), ctypes.byref(out)), "timed_get")
        return _msg_from_c(out) if rc == 1 else None

    def timed_get_inf2tra(self, timeout_ms, id):
        return self._timed_get(_INF2TRA, timeout_ms, id)

    def timed_get_tra2inf(self, timeout_ms, id):
        return self._timed_get(_TRA2INF, timeout_ms, id)

    def timed_get_tra2inf_from_any(self, timeout_ms):
        out, who = CtrlMsg(), ctypes.c_int(-1)
        rc = check_host(lib().tch_mq_timed_get_from_any(_TRA2INF, int(timeout_ms), ctypes.byref(who),
                                                        ctypes.byref(out)), "timed_get_from_any")
        return (who.value, _msg_from_c(out)) if rc == 1 else None

    def clear(self):
        lib().tch_mq_clear()

    @staticmethod
    def shutdown():
        lib().tch_InfTraCommunicator_Shutdown()


_TRAIN_INFO_FIELDS = {"pid": 0, "rank": 1, "world_size": 2, "init_batch_size": 3, "current_batch_size": 4,
                      "target_batch_size": 5, "target_batch_size_unpublished": 6, "first_epoch_done": 7}


def init_train_info(init_batch_size, current_batch_size, model_name=None, pid=None):
    """main.pyx:485-515: publish this rank's row of the information board (no-op without a
    colocated inference server)."""
    if not lib().tch_InfTraCommunicator_IsInitialized():
        return
    name = model_name.encode() if model_name is not None else None
    check_host(lib().tch_init_train_info(int(init_batch_size), int(current_batch_size), name), "init_train_info")
    if pid is not None:
        lib().tch_train_info_set_field(get_train_rank(), 0, int(pid))


def update_current_batch_size(current_batch_size):
    """main.pyx:518-528"""
    if not lib().tch_InfTraCommunicator_IsInitialized():
        return
    check_host(lib().tch_update_current_batch_size(int(current_batch_size)), "update_current_batch_size")


def get_train_info(id, field):
    return int(lib().tch_train_info_get_field(int(id), _TRAIN_INFO_FIELDS[field]))


def train_info_is_valid(id):
    return bool(lib().tch_train_info_is_valid(int(id)))


def get_train_info_model_name(id):
    buf = ctypes.create_string_buffer(256)
    lib().tch_train_info_model_name(int(id), buf, 256)
    return buf.value.decode()


# ---------------------------------------------------------------------------------- stubs


class _StubBase:
    _KIND = 0

    def __init__(self, batch_size=0):
        self._h = lib().tch_stub_create(self._KIND, int(batch_size))
        if not self._h:
            raise TorchColHipError("stub create failed: " + (lib().tch_host_last_error() or b"").decode())

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().tch_stub_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def train_start(self):
        lib().tch_stub_train_start(self._h)

    def train_end(self):
        lib().tch_stub_train_end(self._h)

    def stop(self):
        lib().tch_stub_stop(self._h)

    def can_exit_after_infer_worklaod_done(self):
        return bool(lib().tch_stub_can_exit_after_infer_worklaod_done(self._h))

    def set_train_first_epoch_done(self):
        lib().tch_stub_set_train_first_epoch_done(self._h)

    def report_batch_size(self, batch_size):
        lib().tch_stub_report_batch_size(self._h, int(batch_size))

    def StepsNoInteruptBegin(self):
        lib().tch_stub_StepsNoInteruptBegin(self._h)

    def StepsNoInteruptEnd(self):
        lib().tch_stub_StepsNoInteruptEnd(self._h)

    def EnableTorchColEngine(self):
        """ctrl_stub.pxi: switches the reference's autograd engine to the checkpointing one; the
        recorded launch program already checks between segments, nothing to switch here."""
        return None

    @property
    def cmd(self):
        c = int(lib().tch_stub_cmd(self._h))
        return None if c < 0 else CtrlEvent(c)

    @cmd.setter
    def cmd(self, value):
        lib().tch_stub_set_cmd(self._h, -1 if value is None else int(value))

    def last_error(self):
        return (lib().tch_stub_last_error(self._h) or b"").decode()

    def process_msg(self, entry):
        """Deliver one message synchronously (what the control thread does on receipt)."""
        return int(lib().tch_stub_process_msg(self._h, ctypes.byref(entry._c)))


class PyDummyStub(_StubBase):
    """ctrl_stub.pxi:69-86"""
    _KIND = 0


class PySwitchStub(_StubBase):
    """ctrl_stub.pxi:88-140"""
    _KIND = 1

    def try_interrupt_train_done(self, barrier=False):
        return bool(lib().tch_stub_try_interrupt_train_done(self._h, int(bool(barrier))))

    def train_resume_done(self):
        lib().tch_stub_train_resume_done(self._h)

    def prepare_resume(self):
        return bool(lib().tch_stub_prepare_resume(self._h))

    def set_killed_batch_recover(self):
        lib().tch_stub_set_killed_batch_recover(self._h)

    def set_global_interrupt_flag(self, flag):
        lib().tch_stub_set_global_interrupt_flag(self._h, int(bool(flag)))

    def get_global_interrupt_flag(self):
        return bool(lib().tch_stub_get_global_interrupt_flag(self._h))

    def set_global_has_batch_killed(self, flag):
        lib().tch_stub_set_global_has_batch_killed(self._h, int(bool(flag)))

    def get_global_has_batch_killed(self):
        return bool(lib().tch_stub_get_global_has_batch_killed(self._h))


class PyColocateStub(_StubBase):
    """ctrl_stub.pxi:142-231"""
    _KIND = 2

    def __init__(self, batch_size):
        super().__init__(batch_size)

    @property
    def target_batch_size(self):
        return int(lib().tch_stub_target_batch_size(self._h))

    @property
    def unpub_target_batch_size(self):
        return int(lib().tch_stub_unpub_target_batch_size(self._h))

    def adjust_l1_done(self):
        lib().tch_stub_adjust_l1_done(self._h)

    def adjust_l2_done(self):
        lib().tch_stub_adjust_l2_done(self._h)

    def passed_time_from_set_cmd(self):
        return float(lib().tch_stub_passed_time_from_set_cmd(self._h))

    def set_killed_batch_recover(self):
        lib().tch_stub_set_killed_batch_recover(self._h)

    def set_killed_batch_reconfiged(self):
        lib().tch_stub_set_killed_batch_reconfiged(self._h)


def _time_stamps(fn):
    cap = 1 << 16
    buf = (ctypes.c_int64 * cap)()
    n = fn(buf, cap)
    return [int(buf[i]) for i in range(min(n, cap))]


def get_adjust_request_time_stamp():
    return _time_stamps(lib().tch_get_adjust_request_time_stamp)


def get_adjust_done_time_stamp():
    return _time_stamps(lib().tch_get_adjust_done_time_stamp)


# ---------------------------------------------------------------------------------- util


def get_unix_timestamp():
    return int(lib().tch_get_unix_timestamp())


def get_unix_timestamp_us():
    return int(lib().tch_get_unix_timestamp_us())


def _glog(level, msg, file, line):
    if isinstance(msg, bytes):
        msg = msg.decode()
    if isinstance(file, bytes):
        file = file.decode()
    t = time.time()
    stamp = time.strftime("%m%d %H:%M:%S", time.localtime(t)) + f".{int((t % 1) * 1e6):06d}"
    print(f"{level}{stamp} {threading.get_native_id()} {os.path.basename(file)}:{line}] {msg}", file=sys.stderr,
          flush=True)


def CallGLOG_INFO(log_str, file, line):
    _glog("I", log_str, file, line)


def CallGLOG_DINFO(log_str, file, line):
    if os.environ.get("COLTRAIN_LOG_ALL") == "1" or os.environ.get("GLOG_v"):
        _glog("I", log_str, file, line)


class PyTensorWeakRef:
    """main.pyx:550-567"""

    def __init__(self, tensor):
        self._ref = weakref.ref(tensor)

    def _t(self):
        return self._ref()

    def nbytes(self):
        t = self._t()
        return 0 if t is None else t.numel() * t.element_size()

    def storage_nbytes(self):
        t = self._t()
        return 0 if t is None else t.untyped_storage().nbytes()

    def data_ptr(self):
        t = self._t()
        return 0 if t is None else t.data_ptr()
