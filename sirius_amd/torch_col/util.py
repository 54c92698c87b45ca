"""Logging, pool usage figures, and the event log the reference's profiling tools consume
(pytorch/torch_col/util.py:16-191)."""
import contextlib
import csv
import glob
import inspect
import io
import os
from dataclasses import dataclass
from typing import Optional

from . import _C, dist
from ._C import TrainMode


def _join(args):
    if len(args) == 1:
        msg = args[0]
    else:
        msg = ' '.join(f'{a}' for a in args)
    return msg if isinstance(msg, str) else f'{msg}'


def info(*args):
    _C.CallGLOG_INFO(_join(args), 'torch_col', 0)


def info_with_frame(*args):
    caller = inspect.getframeinfo(inspect.stack()[1][0])
    _C.CallGLOG_INFO(_join(args), caller.filename, caller.lineno)


def dinfo(*args):
    caller = inspect.getframeinfo(inspect.stack()[1][0])
    _C.CallGLOG_DINFO(_join(args), caller.filename, caller.lineno)


def cleanup_previous_shm():
    """util.py:56-61: remove the segments a crashed run left behind."""
    for pat in ("/dev/shm/colserve_shm_*", "/dev/shm/sem.colserve_shm_*"):
        for f in glob.glob(pat):
            try:
                os.unlink(f)
            except OSError:
                pass


_GB = 1024 ** 3


def _device_used_gb():
    import torch
    free, total = torch.cuda.mem_get_info(_C.get_train_rank())
    return (total - free) / _GB


class MemoryPool:
    """util.py:64-97.  Figures in GB."""

    @classmethod
    def get_memory_usage(cls):
        if _C.is_enable_shared_tensor():
            return _C.cuda_memory_pool_train_all_usage(_C.get_train_rank()) / _GB
        return _device_used_gb()

    @classmethod
    def get_memory_peak_usage(cls):
        if _C.is_enable_shared_tensor():
            return _C.cuda_memory_pool_train_peak_usage(_C.get_train_rank()) / _GB
        return _device_used_gb()

    @classmethod
    def get_allocated_memory(cls):
        if _C.is_enable_shared_tensor():
            return _C.cuda_memory_pool_train_usage(_C.get_train_rank()) / _GB
        return _device_used_gb()

    @classmethod
    def empty_cache(cls):
        if _C.is_enable_shared_tensor():
            return _C.cuda_memory_pool_free_train_local(_C.get_train_rank())
        import torch
        if torch.cuda.is_available():
            torch.cuda.empty_cache()
        return 0

    @classmethod
    def stale_pages(cls):
        """Mappings this process still holds over pages it gave back (lazy pools only; 0 otherwise)."""
        if not _C.is_enable_shared_tensor():
            return 0
        return _C.pool_counters(_C.get_train_rank())["stale"]

    @classmethod
    def trim_stale_mappings(cls):
        """Remove those mappings; returns how many.  A pool in eager mode has none."""
        if not _C.is_enable_shared_tensor():
            return 0
        return _C.pool_trim(_C.get_train_rank())


@dataclass
class Event:
    timestamp: int
    name: str
    loc: str
    duration: float
    tag: str

    def __str__(self) -> str:
        return f'{self.timestamp} {self.loc} {self.name} {self.duration} {self.tag}'


_CSV_FIELDS = ("timestamp", "name", "loc", "duration", "tag", "rank")


class EventManager:
    """util.py:113-179.  Timestamps are kept in microseconds; the dump writes milliseconds with
    two decimals, columns timestamp,name,loc,duration,tag,rank -- the schema of the reference's
    train-profile.csv."""
    _event_list: list = []
    _default_event_log_path = 'train-profile.csv'

    @classmethod
    def set_log_path(cls, path: str):
        cls._event_log_path = path

    @classmethod
    def reset(cls):
        cls._event_list = []

    @classmethod
    def record_event(cls, name: str, prev_event: Optional[Event] = None, record_loc: bool = False):
        timestamp = _C.get_unix_timestamp_us()
        if record_loc:
            caller = inspect.getframeinfo(inspect.stack()[1][0])
            loc = f'{caller.filename}:{caller.lineno}'
        else:
            loc = 'none'
        if prev_event is not None:
            prev_event.duration = (timestamp - prev_event.timestamp) / 1000
        if len(name) > 0:
            event = Event(timestamp, name, loc, 0, '')
            cls._event_list.append(event)
            return event

    @classmethod
    @contextlib.contextmanager
    def record_duration_event(cls, name: str):
        timestamp = _C.get_unix_timestamp_us()
        event = Event(timestamp, name, 'none', 0, '')
        cls._event_list.append(event)
        yield event
        event.duration = (_C.get_unix_timestamp_us() - timestamp) / 1000

    @classmethod
    def _to_csv(cls, header: bool) -> str:
        out = io.StringIO()
        w = csv.writer(out, lineterminator='\n')
        if header:
            w.writerow(_CSV_FIELDS)
        rank = _C.get_train_rank()
        for e in cls._event_list:
            w.writerow([f'{e.timestamp / 1000:.2f}', e.name, e.loc, f'{float(e.duration):.2f}', e.tag, rank])
        return out.getvalue()

    @classmethod
    def dump(cls, path: Optional[str] = None, train_mode: Optional[TrainMode] = None):
        if path is None:
            path = _C.get_train_profile_log_path() or getattr(cls, "_event_log_path", cls._default_event_log_path)
        if train_mode is not None and train_mode.is_colocate():
            for ts in _C.get_adjust_request_time_stamp():
                cls._event_list.append(Event(ts, 'recv_adjust', 'none', 0, ''))
            for ts in _C.get_adjust_done_time_stamp():
                cls._event_list.append(Event(ts, 'adjust_done', 'none', 0, ''))
        if _C.get_train_rank() == 0:
            text = cls._to_csv(header=True) + '\n'
            for i in range(1, _C.get_train_world_size()):
                text += dist.recv_msg(i) + '\n'
            with open(path, 'w') as f:
                f.write(text)
            info(f'[EventMananger] dump train event to {path}')
        else:
            dist.send_msg(0, cls._to_csv(header=False))
        dist.wait_barrier()
        return path


def initialize_sgd_optimizer(model, optimizer=None):
    """util.py:182-191 pre-creates zero gradients and momentum buffers so that memory is stable
    from the first step; the engine allocates its flat gradient and optimizer-state buffers when it is
    built, so this only checks that they exist."""
    state = [getattr(model, n, None) for n in ("momentum_buf", "exp_avg")]
    assert model.grads is not None and any(t is not None for t in state)
