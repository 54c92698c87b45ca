"""Logging, pool usage figures, and the event log the reference's profiling tools consume
(pytorch/torch_col/util.py:16-191)."""
import contextlib
import csv
import glob
import inspect
import io
import os
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


class Event:
    """One row of the training profile: a name, when it began (microseconds since the epoch), how long it took
    (milliseconds, filled in when the span closes), where it was recorded and a free-form tag.  The field names are
    the columns of the reference's train-profile.csv (pytorch/torch_col/util.py:100-110)."""
    __slots__ = ("timestamp", "name", "loc", "duration", "tag")

    def __init__(self, timestamp: int, name: str, loc: str = 'none', duration: float = 0, tag: str = ''):
        self.timestamp, self.name, self.loc, self.duration, self.tag = timestamp, name, loc, duration, tag

    def close(self, now_us: int):
        """The span ends now: duration in milliseconds from the two microsecond stamps."""
        self.duration = (now_us - self.timestamp) / 1000

    def __eq__(self, other):
        return isinstance(other, Event) and all(getattr(self, f) == getattr(other, f) for f in self.__slots__)

    def __repr__(self) -> str:
        return f'Event({self.timestamp}, {self.name!r}, {self.loc!r}, {self.duration}, {self.tag!r})'

    def __str__(self) -> str:
        return f'{self.timestamp} {self.loc} {self.name} {self.duration} {self.tag}'


_CSV_FIELDS = ("timestamp", "name", "loc", "duration", "tag", "rank")


def _call_site(depth: int) -> str:
    """file:line of the frame `depth` levels above the caller of this function."""
    frame = inspect.currentframe()
    for _ in range(depth + 1):
        frame = frame.f_back
    return f'{frame.f_code.co_filename}:{frame.f_lineno}'


class EventManager:
    """The training profile (pytorch/torch_col/util.py:113-179): a list of spans in the order they began.
    Timestamps are kept in microseconds so that two events do not collide; durations are milliseconds; the dump
    writes milliseconds with two decimals, columns timestamp,name,loc,duration,tag,rank -- the schema of the
    reference's train-profile.csv."""
    _event_list: list = []
    _default_event_log_path = 'train-profile.csv'

    @classmethod
    def set_log_path(cls, path: str):
        cls._event_log_path = path

    @classmethod
    def reset(cls):
        cls._event_list = []

    @classmethod
    def _open(cls, name: str, now_us: int, loc: str = 'none') -> Event:
        span = Event(now_us, name, loc)
        cls._event_list.append(span)
        return span

    @classmethod
    def record_event(cls, name: str, prev_event: Optional[Event] = None, record_loc: bool = False):
        """Close `prev_event` (if any) and open a span called `name` at the same instant; an empty name only closes.
        Returns the new span, or None."""
        now = _C.get_unix_timestamp_us()
        if prev_event is not None:
            prev_event.close(now)
        if not name:
            return None
        return cls._open(name, now, _call_site(1) if record_loc else 'none')

    @classmethod
    @contextlib.contextmanager
    def record_duration_event(cls, name: str):
        """A span around the body of a `with` block.  A body that raises (a micro-batch that is cut short) leaves
        its span open, duration 0, as in the reference."""
        span = cls._open(name, _C.get_unix_timestamp_us())
        yield span
        span.close(_C.get_unix_timestamp_us())

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
