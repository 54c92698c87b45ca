"""Python-visible names of the reference's compiled module `torch_col._C._dist`
(pytorch/torch_col/cython/dist.pyx:25-193): intra-train barrier and string messages, the
dynamic batch distributor and the throughput model."""
import ctypes

from .._lib import TorchColHipError, check_host, lib

_MAX_RANGES = 4096


def wait_barrier():
    lib().tch_wait_barrier()


def send_msg(dst_rank, msg):
    data = msg.encode() if isinstance(msg, str) else bytes(msg)
    check_host(lib().tch_send_msg(int(dst_rank), data, len(data)), "send_msg")


def recv_msg(src_rank):
    cap = 1 << 16
    while True:
        buf = ctypes.create_string_buffer(cap)
        n = lib().tch_recv_msg(int(src_rank), buf, cap)
        if n >= 0:
            return buf.raw[:n].decode()
        if -n <= cap:
            raise TorchColHipError("recv_msg failed: " + (lib().tch_host_last_error() or b"").decode())
        cap = -n


def _pack(ranges):
    flat = []
    for lo, hi in ranges:
        flat += [int(lo), int(hi)]
    return (ctypes.c_int * max(1, len(flat)))(*flat), len(ranges)


def _unpack(buf, n):
    return [(int(buf[2 * i]), int(buf[2 * i + 1])) for i in range(n)]


def init_dynamic_batch_distributor(dataset_size, input_batch_size, global_batch_size, lazy_distributing=False,
                                   distribute_policy="fix"):
    """dist.pyx:72-87 -> DynamicBatchDistirbutor::Init (csrc/dynamic_batch.cc:40-65)."""
    check_host(lib().tch_init_dynamic_batch_distributor(int(dataset_size), int(input_batch_size),
                                                        int(global_batch_size), int(bool(lazy_distributing)),
                                                        str(distribute_policy).encode()),
               "init_dynamic_batch_distributor")
    _DynamicBatchDistirbutor._lazy_distributing = bool(lazy_distributing)


def shutdown_dynamic_batch_distributor():
    lib().tch_shutdown_dynamic_batch_distributor()


class _DynamicBatchDistirbutor:  # the reference's spelling
    """dist.pyx:90-166: static facade over the process-wide distributor."""
    _lazy_distributing = False

    @staticmethod
    def get_batch(batch_size):
        buf = (ctypes.c_int * (2 * _MAX_RANGES))()
        last = ctypes.c_int(0)
        n = check_host(lib().tch_distributor_get_batch(int(batch_size), buf, _MAX_RANGES, ctypes.byref(last)),
                       "get_batch")
        return _unpack(buf, n), bool(last.value)

    @staticmethod
    def query_next_batch_size(batch_size):
        return int(lib().tch_distributor_query_next_batch_size(int(batch_size)))

    @staticmethod
    def finish_batch(batch_range_vec, end_of_global_batch):
        buf, n = _pack(batch_range_vec)
        check_host(lib().tch_distributor_finish_batch(buf, n, int(bool(end_of_global_batch))), "finish_batch")

    @staticmethod
    def abort_batch(batch_range_vec, end_of_global_batch):
        buf, n = _pack(batch_range_vec)
        check_host(lib().tch_distributor_abort_batch(buf, n, int(bool(end_of_global_batch))), "abort_batch")

    @staticmethod
    def vote_finish_last_micro_batch():
        return bool(check_host(lib().tch_distributor_vote_finish_last_micro_batch(), "vote_finish"))

    @staticmethod
    def vote_abort_last_micro_batch():
        lib().tch_distributor_vote_abort_last_micro_batch()

    @staticmethod
    def reset_last_micro_batch_finish_vote():
        lib().tch_distributor_reset_last_micro_batch_finish_vote()

    @staticmethod
    def distribute_batch(check_num_unproced_samples, distribute_to_all, at_global_batch_begin):
        lib().tch_distributor_distribute_batch(int(bool(check_num_unproced_samples)), int(bool(distribute_to_all)),
                                               int(bool(at_global_batch_begin)))

    @staticmethod
    def next_epoch():
        return int(check_host(lib().tch_distributor_next_epoch(), "next_epoch"))

    @staticmethod
    def next_global_batch():
        lib().tch_distributor_next_global_batch()

    @staticmethod
    def get_global_batch_size():
        return int(lib().tch_distributor_get_global_batch_size())

    @staticmethod
    def get_num_global_batch_per_epoch():
        return int(lib().tch_distributor_get_num_global_batch_per_epoch())

    @staticmethod
    def get_num_proced_global_batch():
        return int(lib().tch_distributor_get_num_proced_global_batch())

    # -- inspection used by tests and the debug tooling
    @staticmethod
    def snapshot(which):
        """which: 'unproc' | 'procing' | 'proced' -> the ordered ranges of that set, all ranks merged."""
        code = {"unproc": 0, "procing": 1, "proced": 2}[which]
        buf = (ctypes.c_int * (2 * _MAX_RANGES))()
        n = check_host(lib().tch_distributor_snapshot(code, buf, _MAX_RANGES), "snapshot")
        return _unpack(buf, n)

    @staticmethod
    def counters():
        buf = (ctypes.c_int * 64)()
        n = lib().tch_distributor_counters(buf, 64)
        return [int(buf[i]) for i in range(n)]


def init_train_performance_model():
    """dist.pyx:169-171: the model lives in the intra-train shared segment and exists once that
    segment does."""
    return None


class _PerfModel:
    """dist.pyx:174-193 -> csrc/perf_model.cc:25-94"""

    @staticmethod
    def record_thpt(batch_size, batch_time_ms):
        lib().tch_perf_model_record_thpt(int(batch_size), float(batch_time_ms))

    @staticmethod
    def get_thpt(batch_size):
        return float(lib().tch_perf_model_get_thpt(int(batch_size)))

    @staticmethod
    def get_thpt_vec(batch_sizes):
        n = len(batch_sizes)
        inp = (ctypes.c_int * max(1, n))(*[int(b) for b in batch_sizes])
        out = (ctypes.c_double * max(1, n))()
        lib().tch_perf_model_get_thpt_vec(inp, n, out)
        return [float(out[i]) for i in range(n)]

    @staticmethod
    def clear():
        lib().tch_perf_model_clear()
