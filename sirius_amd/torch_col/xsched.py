"""Stream registration and batch killing on top of the preemptible launch queue
(pytorch/torch_col/xsched.py:69-156)."""
from typing import Optional, Union

from . import _C


def _handle(stream):
    return stream if isinstance(stream, int) else stream.cuda_stream


def register_stream(stream, is_enable_dynamic_sm_partition: bool = True):
    stream = _handle(stream)
    _C.RegisterStream(stream)
    if (_C.has_colocated_infer_server() and _C.is_enable_dynamic_sm_partition()
            and is_enable_dynamic_sm_partition):
        _C.SMPartitionInit(stream)


def unregister_stream(stream):
    _C.UnRegisterStream(_handle(stream))


def unregister_all_streams():
    _C.UnRegisterAllStreams()


def get_xqueue_size(stream=None) -> int:
    if stream is None:
        return _C.GetXQueueSizeAllStreams()
    return _C.GetXQueueSize(_handle(stream))


def _abort_and_sync(stream):
    if stream is None:
        num_cmds = _C.AbortAllStreams()
        _C.SyncAllStreams()
    else:
        stream = _handle(stream)
        num_cmds = _C.AbortStream(stream)
        _C.SyncStream(stream)
    return num_cmds


def initial_kill_batch(epoch, batch, stream=None):
    """xsched.py:102-118: one abort after the very first batch so that the first real kill
    does not pay for lazily created queue state."""
    if epoch == 0 and batch == 0:
        t1 = _C.get_unix_timestamp()
        num_cmds = _abort_and_sync(stream)
        t2 = _C.get_unix_timestamp()
        print(f'initial_kill_batch cost {t2 - t1} ms, num_cmds={num_cmds}')


def kill_batch(stream=None):
    """xsched.py:121-135: drop every launch not yet handed to the hardware queue, wait for
    the at most `queue length` launches in flight."""
    t1 = _C.get_unix_timestamp()
    num_cmds = _abort_and_sync(stream)
    t2 = _C.get_unix_timestamp()
    print(f'kill batch cost {t2 - t1} ms, num_cmds={num_cmds} '
          f'total_queue_size={_C.GetTotalXQueueSize()}')
    return num_cmds


def suspend_all_streams(sync_hw: bool = False):
    """Training's queues stop handing launches to the hardware until resume_all_streams()."""
    _C.lib().tch_SuspendAllStreams(int(sync_hw))


def resume_all_streams(drop_commands: bool = False):
    _C.lib().tch_ResumeAllStreams(int(drop_commands))


def set_reject_cuda_calls(reject: bool):
    _C.SetRejectCudaCalls(reject)


def guess_nccl_begin():
    _C.GuessNcclBegin()


def guess_nccl_end():
    _C.GuessNcclEnd()


def is_guess_nccl_begined():
    return _C.IsGuessNcclBegined()


def get_nccl_streams():
    return _C.GetNcclStreams()
