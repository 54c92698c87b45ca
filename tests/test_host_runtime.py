"""Host runtime behind the C ABI, on the CPU: configuration, message queues and information
board, intra-train sync, batch distributor, throughput model, control stubs, HBM pool model.

What pins each part (none of them has stored expectations in the reference's tests):
  distributor  invariants + an independent Python enumeration of the reference's rules
               (csrc/dynamic_batch.cc:254-398,576-671) on small datasets
  perf model   the closed form of csrc/perf_model.cc:25-94 evaluated by hand
  queues       FIFO per (direction, rank), timed get semantics
  info board   field rules of common/inf_tra_comm/shared_info.cc:54-108
  stubs        the state machine of csrc/control_stub.cc:402-640 driven message by message
  pool         configuration constants (common/cuda_allocator.cc:61-85) + determinism of offsets
"""
import ctypes
import json
import multiprocessing as mp
import os
import random
import subprocess
import sys
import time

import pytest

from sirius_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
from sirius_amd._lib import CtrlMsg, lib

_PORT = [20000 + (os.getpid() % 5000) * 7]


@pytest.fixture()
def fresh(monkeypatch):
    """A clean runtime on its own shared-memory namespace."""
    _PORT[0] += 1
    monkeypatch.setenv("SIRIUS_PORT", str(_PORT[0]))
    for k in list(os.environ):
        if k.startswith("COLTRAIN_"):
            monkeypatch.delenv(k)
    L = lib()
    L.tch_TorchColShutdown()
    yield L
    L.tch_TorchColShutdown()
    for f in os.listdir("/dev/shm"):
        if f.startswith(f"colserve_shm_{os.getuid()}_p{_PORT[0]}"):
            os.unlink(os.path.join("/dev/shm", f))


# ------------------------------------------------------------------ ABI surface

def test_every_declared_symbol_is_exported():
    sig = _lib.declared_symbols()
    assert len(sig) >= 160
    handle = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in sig if not hasattr(handle, n)]
    assert not missing, missing


def test_header_parser_types():
    sig = _lib.declared_symbols()
    assert sig["tch_pool_malloc"] == (ctypes.c_void_p, [ctypes.c_ssize_t, ctypes.c_int, ctypes.c_void_p])
    assert sig["tch_perf_model_get_thpt"] == (ctypes.c_double, [ctypes.c_int])
    assert sig["tch_host_last_error"] == (ctypes.c_char_p, [])
    assert sig["tch_get_unix_timestamp_us"][0] is ctypes.c_int64


# ------------------------------------------------------------------ config

def test_config_defaults_and_env(fresh, monkeypatch):
    L = fresh
    assert L.tch_TorchColInit(0, 1, 0) == 0
    assert L.tch_TorchColConfig_IsConfigured() == 1
    assert L.tch_TorchColConfig_GetColocateTrainMode() == b"normal"
    assert L.tch_TorchColConfig_GetColocateCtrlHookMode() == b"none"
    assert L.tch_TorchColConfig_IsEnableSharedTensor() == 0
    assert L.tch_TorchColConfig_HasColocatedInferServer() == 0
    assert L.tch_TorchColConfig_IsTrainMaster() == 1
    monkeypatch.setenv("COLTRAIN_MODE", "colocate-l1")
    monkeypatch.setenv("COLTRAIN_HOOK_MODE", "xsched-sync")
    monkeypatch.setenv("COLTRAIN_USE_XSCHED", "1")
    monkeypatch.setenv("COLTRAIN_DYNAMIC_SM_PARTITION", "1")
    monkeypatch.setenv("COLTRAIN_PROFILE_LOG_PATH", "/tmp/x.csv")
    monkeypatch.setenv("COLTRAIN_SHARED_TENSOR_POOL_GB", "2.5")
    L.tch_TorchColConfig_Reload(0, 1)
    assert L.tch_TorchColConfig_GetColocateTrainMode() == b"colocate-l1"
    assert L.tch_TorchColConfig_GetColocateCtrlHookMode() == b"xsched-sync"
    assert L.tch_TorchColConfig_IsEnableXsched() == 1
    assert L.tch_TorchColConfig_IsEnableDynamicSmPartition() == 1
    assert L.tch_TorchColConfig_GetTrainProfileLogPath() == b"/tmp/x.csv"
    assert L.tch_TorchColConfig_GetSharedTensorPoolGb() == 2.5
    # dynamic partitioning needs the launch queue (csrc/config.cc:76-79)
    monkeypatch.setenv("COLTRAIN_USE_XSCHED", "0")
    L.tch_TorchColConfig_Reload(0, 1)
    assert L.tch_TorchColConfig_IsEnableDynamicSmPartition() == 0


def test_init_rejects_bad_rank(fresh):
    assert fresh.tch_TorchColInit(2, 2, 0) < 0
    assert b"rank" in fresh.tch_host_last_error()


# ------------------------------------------------------------------ queues + info board

def _msg(i, e, v):
    return CtrlMsg(i, e, v)


def test_message_queue_fifo_and_timed_get(fresh):
    L = fresh
    assert L.tch_InfTraCommunicator_Init(1, 1, 2) == 0
    for i in range(5):
        assert L.tch_mq_put(0, 0, ctypes.byref(_msg(i, 9, 10 * i))) == 0
    assert L.tch_mq_put(0, 1, ctypes.byref(_msg(77, 11, 64))) == 0
    out = CtrlMsg()
    for i in range(5):  # FIFO per (direction, rank)
        assert L.tch_mq_try_get(0, 0, ctypes.byref(out)) == 1
        assert (out.id, out.event, out.value) == (i, 9, 10 * i)
    assert L.tch_mq_try_get(0, 0, ctypes.byref(out)) == 0
    assert L.tch_mq_try_get(1, 1, ctypes.byref(out)) == 0  # the other direction is separate
    assert L.tch_mq_try_get(0, 1, ctypes.byref(out)) == 1 and out.id == 77
    t0 = time.time()
    assert L.tch_mq_timed_get(1, 0, 50, ctypes.byref(out)) == 0
    assert 0.04 <= time.time() - t0 < 1.0
    # put_all reaches every rank
    assert L.tch_mq_put_all(0, ctypes.byref(_msg(5, 12, 0))) == 0
    for r in range(2):
        assert L.tch_mq_try_get(0, r, ctypes.byref(out)) == 1 and out.event == 12
    who = ctypes.c_int(-1)
    assert L.tch_mq_put(1, 1, ctypes.byref(_msg(8, 4, 0))) == 0
    assert L.tch_mq_timed_get_from_any(1, 50, ctypes.byref(who), ctypes.byref(out)) == 1
    assert who.value == 1 and out.id == 8
    assert L.tch_mq_put(0, 5, ctypes.byref(_msg(0, 0, 0))) < 0  # rank out of range


def test_message_queue_blocking_get_wakes(fresh):
    import threading
    L = fresh
    assert L.tch_InfTraCommunicator_Init(1, 1, 1) == 0
    got = []

    def waiter():
        out = CtrlMsg()
        L.tch_mq_block_get(0, 0, ctypes.byref(out))
        got.append((out.id, time.time()))
    th = threading.Thread(target=waiter)
    th.start()
    time.sleep(0.05)
    t_put = time.time()
    L.tch_mq_put(0, 0, ctypes.byref(_msg(42, 9, 1)))
    th.join(2)
    assert got and got[0][0] == 42 and got[0][1] - t_put < 0.05  # condvar wake, not a poll interval


def test_info_board(fresh, monkeypatch):
    L = fresh
    monkeypatch.setenv("COLTRAIN_HAS_INFER_SERVER", "1")
    assert L.tch_InfTraCommunicator_Init(1, 1, 1) == 0
    assert L.tch_TorchColInit(0, 1, 0) == 0
    assert L.tch_train_info_is_valid(0) == 0
    assert L.tch_init_train_info(64, 64, b"resnet152") == 0
    assert L.tch_train_info_is_valid(0) == 1
    f = lambda k: L.tch_train_info_get_field(0, k)
    assert f(0) == os.getpid() and f(1) == 0 and f(2) == 1 and f(3) == 64 and f(4) == 64
    # target batch size starts at the initial one (shared_info.cc:54-75)
    assert f(5) == 64 and f(6) == 64
    buf = ctypes.create_string_buffer(256)
    L.tch_train_info_model_name(0, buf, 256)
    assert buf.value == b"resnet152"
    assert L.tch_update_current_batch_size(16) == 0
    assert f(4) == 16 and f(3) == 64
    assert L.tch_train_info_set_field(0, 7, 1) == 0 and f(7) == 1


# ------------------------------------------------------------------ perf model (closed form)

def test_perf_model_closed_form(fresh):
    L = fresh
    assert L.tch_TorchColInit(0, 1, 0) == 0
    L.tch_perf_model_clear()
    g = L.tch_perf_model_get_thpt
    assert g(8) == -1.0                                # empty model
    L.tch_perf_model_record_thpt(16, 100.0)            # 0.16 samples / ms
    assert g(0) == 0.0 and g(-3) == 0.0
    assert g(16) == pytest.approx(0.16)
    assert g(8) == pytest.approx(0.08)                 # below the smallest key: proportional
    assert g(32) == pytest.approx(0.32)                # above the largest key: proportional
    L.tch_perf_model_record_thpt(64, 200.0)            # 0.32
    assert g(40) == pytest.approx(0.16 + (0.32 - 0.16) / 48 * 24)   # linear interpolation
    assert g(128) == pytest.approx(0.32 / 64 * 128)
    L.tch_perf_model_record_thpt(16, 50.0)             # running mean of 0.16 and 0.32
    assert g(16) == pytest.approx(0.24)
    L.tch_perf_model_record_thpt(16, 0.0)              # ignored: no time
    L.tch_perf_model_record_thpt(0, 10.0)              # ignored: no samples
    assert g(16) == pytest.approx(0.24)
    inp = (ctypes.c_int * 3)(8, 16, 40)
    out = (ctypes.c_double * 3)()
    L.tch_perf_model_get_thpt_vec(inp, 3, out)
    assert list(out) == [g(8), g(16), g(40)]


# ------------------------------------------------------------------ distributor

def _ranges(L, bs):
    buf = (ctypes.c_int * 256)()
    last = ctypes.c_int(0)
    n = L.tch_distributor_get_batch(bs, buf, 128, ctypes.byref(last))
    assert n >= 0, L.tch_host_last_error()
    return [(buf[2 * i], buf[2 * i + 1]) for i in range(n)], bool(last.value)


def _pack(r):
    flat = [v for lo_hi in r for v in lo_hi]
    return (ctypes.c_int * max(1, len(flat)))(*flat), len(r)


def _snap(L, which):
    buf = (ctypes.c_int * 512)()
    n = L.tch_distributor_snapshot(which, buf, 256)
    return [(buf[2 * i], buf[2 * i + 1]) for i in range(n)]


def _start(L, ds, bs, gbs, lazy=0, policy=b"fix"):
    assert L.tch_TorchColInit(0, 1, 0) == 0
    assert L.tch_init_dynamic_batch_distributor(ds, bs, gbs, lazy, policy) == 0, L.tch_host_last_error()
    assert L.tch_distributor_next_epoch() == 0
    L.tch_distributor_next_global_batch()


def test_distributor_handover_case(fresh):
    """Global batch 64: target 64 -> one range that steps; target 16 -> four ranges, the last
    one steps; an aborted range goes back to the unprocessed set and is issued first again."""
    L = fresh
    _start(L, 128, 64, 64)
    assert L.tch_distributor_get_global_batch_size() == 64
    assert L.tch_distributor_get_num_global_batch_per_epoch() == 2
    r, last = _ranges(L, 64)
    assert r == [(0, 64)] and last
    buf, n = _pack(r)
    assert L.tch_distributor_finish_batch(buf, n, 1) == 0
    L.tch_distributor_next_global_batch()
    assert L.tch_distributor_get_num_proced_global_batch() == 1
    seen = []
    r0, last = _ranges(L, 16)
    assert r0 == [(64, 80)] and not last
    buf, n = _pack(r0)
    L.tch_distributor_finish_batch(buf, n, 0)
    r1, last = _ranges(L, 16)
    assert r1 == [(80, 96)] and not last
    buf, n = _pack(r1)
    assert L.tch_distributor_abort_batch(buf, n, 0) == 0       # killed micro-batch
    assert _snap(L, 0) == [(80, 96), (96, 128)]                 # back in order, kept as its own range
    r1b, last = _ranges(L, 16)
    assert r1b == [(80, 96)] and not last                       # re-issued first
    buf, n = _pack(r1b)
    L.tch_distributor_finish_batch(buf, n, 0)
    r2, last = _ranges(L, 16)
    assert r2 == [(96, 112)] and not last
    buf, n = _pack(r2)
    L.tch_distributor_finish_batch(buf, n, 0)
    r3, last = _ranges(L, 16)
    assert r3 == [(112, 128)] and last                          # do_step exactly here
    buf, n = _pack(r3)
    L.tch_distributor_finish_batch(buf, n, 1)
    L.tch_distributor_next_global_batch()
    assert L.tch_distributor_get_num_proced_global_batch() == 2


def test_distributor_truncates_last_global_batch(fresh):
    L = fresh
    _start(L, 100, 32, 64)
    assert L.tch_distributor_get_num_global_batch_per_epoch() == 2      # ceil(100 / 64)
    total = 0
    for gb in range(2):
        while True:
            r, last = _ranges(L, 32)
            total += sum(b - a for a, b in r)
            buf, n = _pack(r)
            L.tch_distributor_finish_batch(buf, n, int(last))
            if last:
                break
        L.tch_distributor_next_global_batch()
    assert total == 100                                                  # second global batch is 36
    assert L.tch_distributor_get_num_proced_global_batch() == 2


from oracle.host import DistributorModel as _Model  # noqa: E402  (the independent restatement)
from oracle.host import PerfModelOracle, split_global_batch  # noqa: E402


def test_perf_model_against_restatement(fresh):
    L = fresh
    assert L.tch_TorchColInit(0, 1, 0) == 0
    L.tch_perf_model_clear()
    rng, ref = random.Random(9), PerfModelOracle()
    for _ in range(40):
        bs, ms = rng.choice([4, 8, 16, 24, 64]), rng.uniform(5, 200)
        L.tch_perf_model_record_thpt(bs, ms)
        ref.record(bs, ms)
    for bs in range(-2, 100):
        assert L.tch_perf_model_get_thpt(bs) == pytest.approx(ref.get(bs), rel=1e-12, abs=1e-15)


def test_adjust_arithmetic_of_the_peer():
    """server/train_adjuster.cc:69-145,521-538 by hand: ResNet-152, (base, slope) = (1150, 85)."""
    from oracle import host
    base, slope = host.MODEL_MEM_PARAM_SHARED["resnet152"]
    assert host.predict_train_mem_usage_mb(base, slope, 64) == 1150 + 85 * 64
    assert host.predict_train_mem_usage_mb(base, slope, 0) == 1150
    assert host.delta_batch_size(slope, 4080) == 48          # 4080 / 85 = 48 exactly
    assert host.delta_batch_size(slope, 4081) == 49          # ceil
    assert host.predict_target_batch_size(base, slope, 1150 + 85 * 16 + 84, 64) == 16   # floor
    assert host.predict_target_batch_size(base, slope, 100, 64) == 0
    assert host.predict_target_batch_size(base, slope, 1e6, 64) == 64
    assert host.infer_require_mem_target(64, 4080, slope) == 16
    assert host.infer_require_mem_target(0, 4080, slope) is None
    assert host.infer_require_mem_target(64, 0, slope) is None
    assert host.infer_require_mem_target(8, 4080, slope, min_train_bs=1, num_gpus=2) == 1
    assert split_global_batch(21, 2) == [11, 10]
    assert split_global_batch(21, 2, "by_performance", [1.0, 1.0]) == [11, 10]
    assert sum(split_global_batch(64, 3, "by_performance", [3.0, 1.0, 0.01])) == 64


@pytest.mark.parametrize("seed", range(6))
def test_distributor_random_walk_against_enumeration(fresh, seed):
    rng = random.Random(seed)
    ds, gbs = rng.choice([(24, 8), (32, 16), (30, 12), (17, 17)])
    L = fresh
    _start(L, ds, gbs, gbs)
    done = 0
    for gb in range((ds + gbs - 1) // gbs):
        size = min(gbs, ds - done)
        m = _Model(done, done + size)
        steps = 0
        while True:
            bs = rng.randint(1, gbs)
            q = L.tch_distributor_query_next_batch_size(bs)
            r, last = _ranges(L, bs)
            er, elast = m.get(bs)
            assert r == er and last == elast
            assert q == sum(b - a for a, b in r)
            buf, n = _pack(r)
            if rng.random() < 0.35:
                L.tch_distributor_abort_batch(buf, n, int(last))
                m.abort(er)
            else:
                L.tch_distributor_finish_batch(buf, n, int(last))
                m.finish(er)
                steps += int(last)
            # invariants: the three sets partition the global batch
            un, pr, pd = _snap(L, 0), _snap(L, 1), _snap(L, 2)
            assert un == m.unproc and pd == m.proced and sorted(pr) == sorted(m.procing)
            c = (ctypes.c_int * 8)()
            L.tch_distributor_counters(c, 8)
            assert c[0] + c[1] + c[2] == size
            assert c[0] == sum(b - a for a, b in un) and c[2] == sum(b - a for a, b in pd)
            if not m.unproc and not m.procing:
                break
        assert steps == 1                       # do_step exactly once per global batch
        assert m.proced[0][0] == done and m.proced[-1][1] == done + size
        assert all(b == c for (_, b), (c, _) in zip(m.proced, m.proced[1:]))
        L.tch_distributor_next_global_batch()
        done += size
    assert L.tch_distributor_get_num_proced_global_batch() == (ds + gbs - 1) // gbs


def _rank_main(rank, world, port, policy, q):
    os.environ["SIRIUS_PORT"] = str(port)
    for k in list(os.environ):
        if k.startswith("COLTRAIN_"):
            del os.environ[k]
    L = lib()
    try:
        assert L.tch_TorchColInit(rank, world, 0) == 0, L.tch_host_last_error()
        L.tch_wait_barrier()
        # string messages, including lengths that are multiples of the 256-byte chunk and empty
        if rank == 1:
            for n in (0, 1, 255, 256, 257, 512, 5000):
                s = bytes((65 + i % 26) for i in range(n))
                assert L.tch_send_msg(0, s, n) == 0
        else:
            for n in (0, 1, 255, 256, 257, 512, 5000):
                buf = ctypes.create_string_buffer(8192)
                got = L.tch_recv_msg(1, buf, 8192)
                assert got == n and buf.raw[:n] == bytes((65 + i % 26) for i in range(n)), (n, got)
        L.tch_wait_barrier()
        if rank == 0 and policy == b"by_performance":
            L.tch_perf_model_clear()
            L.tch_perf_model_record_thpt(8, 100.0)
        L.tch_wait_barrier()
        assert L.tch_init_dynamic_batch_distributor(40, 8, 21, 0, policy) == 0, L.tch_host_last_error()
        L.tch_wait_barrier()
        e = L.tch_distributor_next_epoch()
        L.tch_distributor_next_global_batch()
        L.tch_wait_barrier()
        mine = []
        while True:
            buf = (ctypes.c_int * 64)()
            last = ctypes.c_int(0)
            n = L.tch_distributor_get_batch(8, buf, 32, ctypes.byref(last))
            if n <= 0:
                break
            r = [(buf[2 * i], buf[2 * i + 1]) for i in range(n)]
            mine += r
            pb, pn = _pack(r)
            L.tch_distributor_finish_batch(pb, pn, last.value)
            if last.value:
                break
        L.tch_wait_barrier()
        q.put((rank, e, mine, None))
    except Exception as ex:  # report instead of hanging the parent
        q.put((rank, -1, [], repr(ex)))
    finally:
        L.tch_wait_barrier() if False else None


@pytest.mark.parametrize("policy", [b"fix", b"by_performance"])
def test_two_ranks_share_a_global_batch(policy):
    """World size 2 in two processes: barrier, chunked string messages, and the split of a
    global batch of 21 samples: q = 21 // 2 = 10, the first 21 % 2 ranks get one more
    (csrc/dynamic_batch.cc:262-275); by-performance with equal throughput gives the same sizes."""
    port = 30000 + os.getpid() % 20000
    ctx = mp.get_context("spawn")
    q = ctx.Queue()
    ps = [ctx.Process(target=_rank_main, args=(r, 2, port, policy, q)) for r in range(2)]
    for p in ps:
        p.start()
    res = {}
    for _ in range(2):
        rank, e, mine, err = q.get(timeout=60)
        assert err is None, err
        res[rank] = mine
    for p in ps:
        p.join(20)
        assert p.exitcode == 0
    n0 = sum(b - a for a, b in res[0])
    n1 = sum(b - a for a, b in res[1])
    assert (n0, n1) == (11, 10)
    cover = sorted(res[0] + res[1])
    assert cover[0][0] == 0 and cover[-1][1] == 21
    for (a, b), (c, d) in zip(cover, cover[1:]):
        assert b == c                                # disjoint and contiguous
    for f in os.listdir("/dev/shm"):
        if f.startswith(f"colserve_shm_{os.getuid()}_p{port}"):
            os.unlink(os.path.join("/dev/shm", f))


# ------------------------------------------------------------------ stubs

def _colocate_setup(L, monkeypatch, world=1, hook="xsched-sync"):
    monkeypatch.setenv("COLTRAIN_HAS_INFER_SERVER", "1")
    monkeypatch.setenv("COLTRAIN_MODE", "colocate-l1")
    monkeypatch.setenv("COLTRAIN_HOOK_MODE", hook)
    monkeypatch.setenv("COLTRAIN_USE_XSCHED", "1")
    assert L.tch_InfTraCommunicator_Init(1, 1, world) == 0
    assert L.tch_TorchColInit(0, world, 0) == 0
    assert L.tch_init_train_info(64, 64, b"resnet152") == 0


def _drain(L, direction=1, rank=0):
    out, got = CtrlMsg(), []
    while L.tch_mq_try_get(direction, rank, ctypes.byref(out)) == 1:
        got.append((out.id, out.event, out.value))
    return got


def test_colocate_stub_adjust_flow(fresh, monkeypatch):
    L = fresh
    _colocate_setup(L, monkeypatch)
    assert L.tch_init_dynamic_batch_distributor(128, 64, 64, 0, b"fix") == 0
    s = L.tch_stub_create(2, 64)
    assert s
    try:
        assert L.tch_stub_cmd(s) == -1
        assert L.tch_stub_target_batch_size(s) == 64
        L.tch_stub_train_start(s)
        assert _drain(L)[-1][1] == 0                                   # kTrainStart
        # the peer writes the unpublished target on the board, then sends the request
        # (server/train_adjuster.cc FillAdjustPlan -> controller); the control thread picks it up
        assert L.tch_train_info_set_field(0, 6, 16) == 0
        L.tch_mq_put(0, 0, ctypes.byref(_msg(7, 9, 16)))               # kColocateAdjustL1 -> 16
        for _ in range(200):
            if L.tch_stub_cmd(s) == 9:
                break
            time.sleep(0.005)
        assert L.tch_stub_cmd(s) == 9
        # unpublished target changes at once, the published one when the adjust is done
        assert L.tch_stub_unpub_target_batch_size(s) == 16
        assert L.tch_stub_target_batch_size(s) == 64
        assert L.tch_stub_passed_time_from_set_cmd(s) >= 0.0
        L.tch_stub_adjust_l1_done(s)
        assert L.tch_stub_cmd(s) == -1
        assert (7, 4, 0) in [(i, e, 0) for i, e, v in _drain(L)]       # kColocateAdjustL1Done, same id
        # the trainer publishes the new target when it redistributes the batch
        # (csrc/dynamic_batch.cc:236-254), as Trainer.handle_abort_batch does after the reply
        assert L.tch_stub_target_batch_size(s) == 64
        L.tch_stub_set_killed_batch_recover(s)
        L.tch_distributor_distribute_batch(1, 1, 0)
        L.tch_stub_set_killed_batch_reconfiged(s)
        assert L.tch_stub_target_batch_size(s) == 16
        # inference leaves: the master redistributes by itself, no reply is sent
        assert L.tch_train_info_set_field(0, 6, 64) == 0
        assert L.tch_stub_process_msg(s, ctypes.byref(_msg(8, 11, 64))) == 0
        assert L.tch_stub_target_batch_size(s) == 64
        n_req, n_done = (ctypes.c_int64 * 8)(), (ctypes.c_int64 * 8)()
        assert L.tch_get_adjust_request_time_stamp(n_req, 8) >= 1
        assert L.tch_get_adjust_done_time_stamp(n_done, 8) >= 1
        assert n_done[0] >= n_req[0] > 0
        # workload done lets training exit
        assert L.tch_stub_can_exit_after_infer_worklaod_done(s) == 0
        L.tch_stub_process_msg(s, ctypes.byref(_msg(9, 12, 0)))
        L.tch_stub_report_batch_size(s, 32)
        assert (0, 6, 32) in [(0, e, v) for i, e, v in _drain(L)]      # kReportBatchSize
        L.tch_stub_train_end(s)
        assert _drain(L)[-1][1] == 1                                   # kTrainEnd
    finally:
        L.tch_stub_stop(s)
        L.tch_stub_destroy(s)


def test_colocate_stub_step_mutex_defers_the_kill(fresh, monkeypatch):
    """While the trainer is inside StepsNoInterupt the control thread must not run the kill
    (control_stub.cc:486-510 takes step_mutex_): the command becomes visible only after End."""
    L = fresh
    _colocate_setup(L, monkeypatch, hook="xsched-sync2")  # the mode in which the control thread kills on receipt
    s = L.tch_stub_create(2, 64)
    try:
        L.tch_stub_StepsNoInteruptBegin(s)
        L.tch_mq_put(0, 0, ctypes.byref(_msg(1, 9, 8)))
        time.sleep(0.1)
        assert L.tch_stub_cmd(s) == -1
        L.tch_stub_StepsNoInteruptEnd(s)
        for _ in range(200):
            if L.tch_stub_cmd(s) == 9:
                break
            time.sleep(0.005)
        assert L.tch_stub_cmd(s) == 9
        L.tch_stub_adjust_l1_done(s)
    finally:
        L.tch_stub_stop(s)
        L.tch_stub_destroy(s)


def test_unknown_event_is_reported_not_fatal(fresh, monkeypatch):
    L = fresh
    _colocate_setup(L, monkeypatch)
    s = L.tch_stub_create(2, 64)
    try:
        assert L.tch_stub_process_msg(s, ctypes.byref(_msg(1, 7, 0))) < 0     # kInterruptTrain to a colocate stub
        assert L.tch_stub_last_error(s)
    finally:
        L.tch_stub_stop(s)
        L.tch_stub_destroy(s)


def test_switch_stub_interrupt_resume(fresh, monkeypatch):
    L = fresh
    monkeypatch.setenv("COLTRAIN_HAS_INFER_SERVER", "1")
    monkeypatch.setenv("COLTRAIN_MODE", "taskswitch-l1")
    assert L.tch_InfTraCommunicator_Init(1, 1, 1) == 0
    assert L.tch_TorchColInit(0, 1, 0) == 0
    s = L.tch_stub_create(1, 0)
    try:
        assert L.tch_stub_process_msg(s, ctypes.byref(_msg(3, 7, 0))) == 0    # kInterruptTrain
        assert L.tch_stub_cmd(s) == 7
        assert L.tch_stub_try_interrupt_train_done(s, 0) == 1
        assert (3, 2) in [(i, e) for i, e, v in _drain(L)]                    # kInterruptTrainDone
        assert L.tch_stub_try_interrupt_train_done(s, 0) == 0                 # one reply per command id
        assert L.tch_stub_prepare_resume(s) == 0
        assert L.tch_stub_process_msg(s, ctypes.byref(_msg(4, 8, 0))) == 0    # kResumeTrain
        assert L.tch_stub_prepare_resume(s) == 1
        # kResumeTrainDone carries id 0 (control_stub.cc:377-382)
        assert (0, 3) in [(i, e) for i, e, v in _drain(L)]
    finally:
        L.tch_stub_stop(s)
        L.tch_stub_destroy(s)


# ------------------------------------------------------------------ pool model

MB = 1 << 20


def test_pool_constants_and_accounting(fresh):
    L = fresh
    assert L.tch_pool_init(0, 512 * MB, 0) == 0
    try:
        assert L.tch_cuda_memory_pool_nbytes(0) == 512 * MB
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 16            # 32 MB pages
        assert L.tch_pool_malloc(0, 0, None) is None                     # zero bytes -> null
        a = L.tch_pool_malloc(1000, 0, None)
        assert a and a % 1024 == 0                                       # 1 KB alignment
        assert L.tch_cuda_memory_pool_train_usage(0) == 1024
        assert L.tch_cuda_memory_pool_train_all_usage(0) == 32 * MB      # one page mapped
        b = L.tch_pool_malloc(2 * MB, 0, None)                           # 2 MB goes to the large segment
        assert L.tch_pool_offset_of(0, b) - L.tch_pool_offset_of(0, a) >= 512 * MB
        c = L.tch_pool_malloc(2 * MB - 1024, 0, None)                    # just below the threshold: small segment
        assert L.tch_pool_offset_of(0, c) == 1024
        L.tch_pool_free(a, 1000, 0, None)
        L.tch_pool_free(c, 0, 0, None)
        assert L.tch_cuda_memory_pool_train_usage(0) == 2 * MB
        assert L.tch_cuda_memory_pool_train_peak_usage(0) == 1024 + 2 * MB + 2 * MB - 1024
        assert L.tch_cuda_memory_pool_train_all_usage(0) == 64 * MB      # freed blocks keep their pages
        assert L.tch_cuda_memory_pool_free_train_local(0) == 32 * MB     # small segment's page goes back
        assert L.tch_cuda_memory_pool_train_all_usage(0) == 32 * MB
        # inference takes free pages, training cannot grow past what is left
        assert L.tch_pool_infer_claim_pages(0, 100) == 15
        assert L.tch_cuda_memory_pool_infer_usage(0) == 15 * 32 * MB
        assert L.tch_pool_malloc(64 * MB, 0, None) is None
        assert b"page" in L.tch_host_last_error() or b"memory" in L.tch_host_last_error()
        assert L.tch_pool_infer_release_pages(0, 15) == 15
        d = L.tch_pool_malloc(64 * MB, 0, None)
        assert d
        L.tch_pool_free(d, 0, 0, None)
        L.tch_pool_free(b, 0, 0, None)
        assert L.tch_cuda_memory_pool_train_usage(0) == 0
        L.tch_cuda_memory_pool_free_train_local(0)
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 16
    finally:
        L.tch_pool_shutdown(0)


def _trace(L, seed, n=400):
    """A seeded alloc / free / empty_cache trace; returns the offsets it produced."""
    rng = random.Random(seed)
    live, offs = [], []
    for _ in range(n):
        r = rng.random()
        if r < 0.55 or not live:
            size = rng.choice([512, 4096, 100_000, MB, 3 * MB, 20 * MB, 40 * MB])
            p = L.tch_pool_malloc(size, 0, None)
            if p:
                live.append(p)
                offs.append(L.tch_pool_offset_of(0, p))
            else:
                offs.append(-1)
        elif r < 0.95:
            L.tch_pool_free(live.pop(rng.randrange(len(live))), 0, 0, None)
        else:
            offs.append(("ec", L.tch_cuda_memory_pool_free_train_local(0)))
    for p in live:
        L.tch_pool_free(p, 0, 0, None)
    return offs


def test_pool_offsets_are_a_function_of_the_trace(fresh):
    L = fresh
    runs = []
    for _ in range(2):
        assert L.tch_pool_init(0, 1024 * MB, 0) == 0
        runs.append(_trace(L, 5))
        L.tch_pool_shutdown(0)
    assert runs[0] == runs[1]
    assert sum(1 for o in runs[0] if o == -1) < len(runs[0]) // 2


def test_pool_no_overlap_and_best_fit(fresh):
    L = fresh
    assert L.tch_pool_init(0, 1024 * MB, 0) == 0
    try:
        rng = random.Random(1)
        live = {}
        for _ in range(600):
            if rng.random() < 0.6 or not live:
                size = rng.choice([1024, 10_000, MB, 5 * MB, 33 * MB])
                p = L.tch_pool_malloc(size, 0, None)
                if p:
                    off = L.tch_pool_offset_of(0, p)
                    for o, (s, _) in live.items():
                        assert off + size <= o or o + s <= off, "blocks overlap"
                    live[off] = (size, p)
            else:
                off = rng.choice(list(live))
                L.tch_pool_free(live.pop(off)[1], 0, 0, None)
        for s, p in live.values():
            L.tch_pool_free(p, 0, 0, None)
        # best fit: with holes of 3 MB and 5 MB (in that address order reversed) a 3 MB request
        # takes the 3 MB hole
        L.tch_cuda_memory_pool_free_train_local(0)
        a = L.tch_pool_malloc(5 * MB, 0, None)
        g1 = L.tch_pool_malloc(2 * MB, 0, None)
        b = L.tch_pool_malloc(3 * MB, 0, None)
        g2 = L.tch_pool_malloc(2 * MB, 0, None)
        ob = L.tch_pool_offset_of(0, b)
        L.tch_pool_free(a, 0, 0, None)
        L.tch_pool_free(b, 0, 0, None)
        c = L.tch_pool_malloc(3 * MB, 0, None)
        assert L.tch_pool_offset_of(0, c) == ob
        for p in (c, g1, g2):
            L.tch_pool_free(p, 0, 0, None)
    finally:
        L.tch_pool_shutdown(0)


@pytest.mark.parametrize("pool_mb,page_mb,lazy", [(1024, 32, 0), (1024, 32, 1), (512, 64, 0), (2048, 128, 1)])
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_pool_placement_follows_the_independent_model(fresh, seed, pool_mb, page_mb, lazy):
    """oracle.host.PoolModel states the placement policy with lists and linear scans; the C++ pool (ordered maps,
    a size index, a shared page table) must agree with it after EVERY operation of a random walk: the offset of
    each block, which requests are refused, the bytes empty_cache returns, the owner of every physical page and
    the slot it is mapped at -- in eager and lazy unmapping, at three page sizes, with the other tenant taking
    and returning pages in between.  (The reference's own allocator, mpool, is not in its tree: what is pinned is
    that the pool follows the policy this build states, not mpool's tie-breaking.)"""
    from pool_walk import walk_against_model
    ok, refused = walk_against_model(fresh, seed, pool_mb, page_mb, lazy, use_gpu=False)
    assert ok > 150, "the walk must allocate"
    if pool_mb <= 1024:
        assert refused > 0, "and must run out of pages now and then (the refusal path is part of the policy)"


def test_pool_model_by_hand():
    """The model itself, on cases small enough to follow on paper (so that the two sides cannot agree on nonsense)."""
    from oracle.host import PoolModel
    m = PoolModel(512 * MB)                          # 16 pages of 32 MB, range 4 GB, small segment 512 MB
    assert m.alloc(0) is None
    a = m.alloc(1000)                                # rounded to 1024, small segment, page 0 at slot 0
    assert a == 0 and m.train_usage == 1024 and m.owner[0] == m.TRAIN and m.slot_page == {0: 0}
    b = m.alloc(2 * MB)                              # the threshold itself goes to the large segment
    assert b == 512 * MB and m.slot_page[16] == 1    # slot = 512 MB / 32 MB, next free page
    c = m.alloc(2 * MB - 1024)                       # just below: small segment, right behind a
    assert c == 1024
    m.free(a)
    d = m.alloc(512)                                 # best fit: the 1024-byte hole, not the tail of the page
    assert d == 0
    m.free(c)
    m.free(d)                                        # a + c + the rest of the page merge into one free block
    assert m.segs[0]["blocks"] == [[0, 32 * MB, False]]
    assert m.empty_cache() == 32 * MB and m.owner[0] == m.FREE and 0 not in m.slot_page
    assert m.empty_cache() == 0                      # b is live: its page stays
    assert m.infer_claim(100) == 15 and m.alloc(64 * MB) is None and m.segs[1]["blocks"][-1][2] is False
    assert m.infer_release(2) == 2 and m.owner[14:] == [m.FREE, m.FREE]
    e = m.alloc(40 * MB)                             # grows over the refused request's free tail block: 514 .. 554 MB
    assert e == b + 2 * MB and m.slot_page == {16: 1, 17: 14}   # slot 16 is live already, slot 17 takes the lowest free page
    # lazy mode: the mapping stays, and the same range gets the same pages back without a map
    z = PoolModel(128 * MB, lazy_unmap=True)
    p = z.alloc(64 * MB)
    z.free(p)
    assert z.empty_cache() == 64 * MB and z.maps == 2 and z.unmaps == 0 and len(z.slot_page) == 2
    assert z.alloc(64 * MB) == p and z.maps == 2 and z.revives == 2


def _counters(L):
    c = (ctypes.c_uint64 * 6)()
    L.tch_pool_counters(0, c)
    return dict(zip(("allocs", "frees", "maps", "unmaps", "revives", "stale"), (int(v) for v in c)))


def test_pool_lazy_mode_hands_pages_back_without_unmapping(fresh):
    """Lazy mode: returning pages is bookkeeping, no driver unmap on the handover path; the mapping is reused
    when the page is still free at regrowth, and replaced when inference has taken the page."""
    L = fresh
    assert L.tch_pool_init_ex(0, 128 * MB, 0, 32 * MB, 1) == 0            # 4 pages, lazy unmapping
    try:
        a = L.tch_pool_malloc(64 * MB, 0, None)
        assert _counters(L)["maps"] == 2
        L.tch_pool_free(a, 0, 0, None)
        assert L.tch_cuda_memory_pool_free_train_local(0) == 64 * MB
        c = _counters(L)
        assert c["unmaps"] == 0 and c["stale"] == 2
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 4 and L.tch_cuda_memory_pool_train_all_usage(0) == 0
        # 64 -> 16 -> 64: the same range grows back over pages that are still free
        a2 = L.tch_pool_malloc(64 * MB, 0, None)
        assert a2 == a
        c = _counters(L)
        assert c["maps"] == 2 and c["unmaps"] == 0 and c["revives"] == 2 and c["stale"] == 0
        L.tch_pool_free(a2, 0, 0, None)
        L.tch_cuda_memory_pool_free_train_local(0)
        # inference takes three of the four pages, among them the two with stale mappings
        assert L.tch_pool_infer_claim_pages(0, 3) == 3
        b = L.tch_pool_malloc(32 * MB, 0, None)            # slot 0 again: its old page is gone
        assert b == a
        c = _counters(L)
        assert c["unmaps"] == 1 and c["maps"] == 3 and c["stale"] == 1
        assert L.tch_pool_malloc(64 * MB, 0, None) is None  # nothing left
        assert L.tch_pool_trim(0, 100) == 1 and _counters(L)["stale"] == 0
        L.tch_pool_free(b, 0, 0, None)
        assert L.tch_pool_infer_release_pages(0, 3) == 3
    finally:
        L.tch_pool_shutdown(0)


def test_pool_eager_mode_unmaps_what_it_hands_back(fresh):
    """The default: a page the table calls FREE is mapped nowhere in the training process.  Neighbouring slots
    go in one driver call; growing back maps again (no revival), and the offsets are the same as in lazy mode."""
    L = fresh
    assert L.tch_pool_init(0, 256 * MB, 0) == 0             # 8 pages of 32 MB, eager
    try:
        assert L.tch_pool_page_bytes(0) == 32 * MB
        a = L.tch_pool_malloc(96 * MB, 0, None)
        keep = L.tch_pool_malloc(32 * MB, 0, None)
        b = L.tch_pool_malloc(64 * MB, 0, None)
        assert _counters(L)["maps"] == 6
        L.tch_pool_free(a, 0, 0, None)
        L.tch_pool_free(b, 0, 0, None)
        assert L.tch_cuda_memory_pool_free_train_local(0) == 160 * MB
        c = _counters(L)
        assert c["unmaps"] == 5 and c["stale"] == 0
        assert L.tch_pool_unmap_calls(0) == 2                # two runs: slots 0-2 and slots 4-5
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 7 and L.tch_cuda_memory_pool_train_all_usage(0) == 32 * MB
        a2 = L.tch_pool_malloc(96 * MB, 0, None)
        assert a2 == a
        c = _counters(L)
        assert c["maps"] == 9 and c["revives"] == 0
        assert L.tch_pool_trim(0, 100) == 0
        L.tch_pool_free(a2, 0, 0, None)
        L.tch_pool_free(keep, 0, 0, None)
    finally:
        L.tch_pool_shutdown(0)


def test_pool_offsets_do_not_depend_on_the_unmapping_mode_and_scale_to_the_whole_part(fresh):
    """The same trace gives the same offsets eager or lazy; a pool of 256 GB (the part has 288) follows it too,
    and runs with 128 MB pages as well (a segment grows in whole pages, so placement then differs)."""
    L = fresh
    runs = {}
    for name, (size, page, lazy) in {"eager": (1024 * MB, 32 * MB, 0), "lazy": (1024 * MB, 32 * MB, 1),
                                     "big": (256 * 1024 * MB, 32 * MB, 0), "big128": (256 * 1024 * MB, 128 * MB, 0)}.items():
        assert L.tch_pool_init_ex(0, size, 0, page, lazy) == 0, L.tch_host_last_error()
        assert L.tch_cuda_memory_pool_num_free_pages(0) == size // page
        runs[name] = _trace(L, 5)
        L.tch_pool_shutdown(0)
    assert runs["eager"] == runs["lazy"]
    big_base = 256 * 1024 * MB          # start of the large segment: one eighth of 8 x 256 GB
    small_base = 1024 * MB
    rebased = [o if not isinstance(o, int) or o < small_base else o - small_base + big_base for o in runs["eager"]]
    # the 1 GB pool runs out of pages where the big pool does not: compare up to the first failure
    upto = next((i for i, o in enumerate(runs["eager"]) if o == -1), len(rebased))
    def offsets_only(r):
        return [o for o in r if isinstance(o, int)]
    assert offsets_only(runs["big"][:upto]) == offsets_only(rebased[:upto])
    assert -1 not in runs["big"] and -1 not in runs["big128"]
    assert all(o % 1024 == 0 for o in offsets_only(runs["big128"]))
    assert L.tch_pool_init_ex(0, 1024 * 1024 * MB, 0, 32 * MB, 0) < 0      # more pages than the table holds
    assert b"page table" in L.tch_host_last_error()


_PEER_CHILD = r"""
import ctypes, json, os, sys
sys.path.insert(0, sys.argv[1])
from sirius_amd._lib import lib
L = lib()
out = {}
assert L.tch_pool_peer_attach(0) == 0, L.tch_host_last_error()
out["pages"], out["page_bytes"], out["free"] = L.tch_pool_peer_num_pages(0), L.tch_pool_peer_page_bytes(0), L.tch_pool_peer_free_pages(0)
got = (ctypes.c_int * 16)()
out["claimed"] = L.tch_pool_peer_claim(0, 5, got)
out["indices"] = list(got)[:out["claimed"]]
out["map"] = L.tch_pool_peer_map(0, got[0])
out["map_error"] = L.tch_host_last_error().decode()
print(json.dumps(out), flush=True)
sys.stdin.readline()                      # the parent looks at the table, then lets us go on
back = (ctypes.c_int * 2)(got[0], got[1])
rel = L.tch_pool_peer_release(0, back, 2)
print(json.dumps({"released": rel, "free": L.tch_pool_peer_free_pages(0)}), flush=True)
sys.stdin.readline()
os._exit(0)                               # dies holding three pages: detach never runs
"""


def test_pool_page_table_is_shared_with_another_process(fresh, tmp_path):
    """The page table lives in shared memory: a separate process attaches, sees the same pages, claims FREE
    ones (the trainer then cannot grow over them), gives some back, and the pages of a peer that died are
    there to be taken back.  (CPU model: there is no device memory to map; the GPU test maps and writes.)"""
    L = fresh
    assert L.tch_pool_init(0, 256 * MB, 0) == 0              # 8 pages
    child = None
    try:
        a = L.tch_pool_malloc(64 * MB, 0, None)              # pages 0, 1 -> training
        child = subprocess.Popen([sys.executable, "-c", _PEER_CHILD, ROOT], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                                 env=dict(os.environ), text=True)
        first = json.loads(child.stdout.readline())
        assert first["pages"] == 8 and first["page_bytes"] == 32 * MB and first["free"] == 6
        assert first["claimed"] == 5 and first["indices"] == [2, 3, 4, 5, 6]
        assert not first["map"] and "CPU model" in first["map_error"]
        assert L.tch_cuda_memory_pool_infer_usage(0) == 5 * 32 * MB
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 1
        assert L.tch_pool_malloc(64 * MB, 0, None) is None    # one page left: training cannot grow by two
        child.stdin.write("\n")
        child.stdin.flush()
        second = json.loads(child.stdout.readline())
        assert second == {"released": 2, "free": 3}
        b = L.tch_pool_malloc(64 * MB, 0, None)               # now it can
        assert b
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 1
        child.stdin.write("\n")
        child.stdin.flush()
        child.wait(timeout=20)
        # the in-process stand-in only ever gives back its own pages, not the dead peer's ...
        assert L.tch_pool_infer_release_pages(0, 8) == 0
        # ... but a process that no longer exists owns nothing: its three pages come back on the next look
        assert L.tch_cuda_memory_pool_infer_usage(0) == 0
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 4
        L.tch_pool_free(a, 0, 0, None)
        L.tch_pool_free(b, 0, 0, None)
    finally:
        if child is not None and child.poll() is None:
            child.kill()
        L.tch_pool_shutdown(0)
    # a second pool of the same name can be made once the first is gone; a live one is not taken over
    assert L.tch_pool_init(0, 64 * MB, 0) == 0
    L.tch_pool_shutdown(0)


_HOLDER_CHILD = r"""
import ctypes, sys, time
sys.path.insert(0, sys.argv[1])
from sirius_amd._lib import lib
L = lib()
assert L.tch_pool_peer_attach(0) == 0, L.tch_host_last_error()
got = (ctypes.c_int * 8)()
print(L.tch_pool_peer_claim(0, 6, got), flush=True)
time.sleep(600)                           # killed by the parent while it holds the pages
"""


def test_lazy_pool_flags_pages_until_their_old_mapping_is_gone(fresh):
    """Lazy mode hands pages back before it unmaps them: the pages are FREE and claimable at once, flagged in the
    shared table while the creator still maps them, and a peer's map waits for the flag (here: gives up after the
    time it was given, then succeeds -- as far as the CPU model can -- once trim() has removed the mappings)."""
    L = fresh
    assert L.tch_pool_init_ex(0, 256 * MB, 0, 32 * MB, 1) == 0        # 8 pages, lazy
    try:
        a = L.tch_pool_malloc(96 * MB, 0, None)
        L.tch_pool_free(a, 0, 0, None)
        assert L.tch_cuda_memory_pool_free_train_local(0) == 96 * MB     # relabelled, still mapped
        assert L.tch_pool_peer_attach(0) == 0, L.tch_host_last_error()
        got = (ctypes.c_int * 8)()
        assert L.tch_pool_peer_claim(0, 5, got) == 5 and list(got)[:5] == [0, 1, 2, 3, 4]
        assert L.tch_pool_peer_still_mapped(0, got, 5) == 3              # pages 0-2 carried the block
        t0 = time.time()
        assert not L.tch_pool_peer_map_wait(0, 0, 30)
        assert time.time() - t0 >= 0.03 and b"still mapped" in L.tch_host_last_error()
        assert not L.tch_pool_peer_map_wait(0, 3, 30)                    # never mapped by the creator: no wait
        assert b"CPU model" in L.tch_host_last_error()
        assert L.tch_pool_trim(0, 2) == 2
        assert L.tch_pool_peer_still_mapped(0, got, 5) == 1
        assert L.tch_pool_trim(0, 100) == 1
        assert L.tch_pool_peer_still_mapped(0, got, 5) == 0
        assert not L.tch_pool_peer_map_wait(0, 0, 30) and b"CPU model" in L.tch_host_last_error()
        # a page that training takes back itself (revived) is not waited for by anybody
        back = (ctypes.c_int * 5)(*list(got)[:5])
        assert L.tch_pool_peer_release(0, back, 5) == 5
        b = L.tch_pool_malloc(32 * MB, 0, None)
        L.tch_pool_free(b, 0, 0, None)
        L.tch_cuda_memory_pool_free_train_local(0)
        c = L.tch_pool_malloc(32 * MB, 0, None)                          # same slot, same page, revived
        assert c == b
        one = (ctypes.c_int * 1)(0)
        assert L.tch_pool_peer_still_mapped(0, one, 1) == 0
        L.tch_pool_free(c, 0, 0, None)
    finally:
        L.tch_pool_peer_detach(0)
        L.tch_pool_shutdown(0)


def test_pool_takes_back_the_pages_of_a_killed_peer(fresh):
    """An inference process that is killed (SIGKILL: no destructor, no detach) while it owns pages must not keep
    them for good: training's next request that finds too few free pages looks for owners that no longer exist."""
    L = fresh
    assert L.tch_pool_init(0, 256 * MB, 0) == 0              # 8 pages
    child = subprocess.Popen([sys.executable, "-c", _HOLDER_CHILD, ROOT], stdout=subprocess.PIPE, env=dict(os.environ),
                             text=True)
    try:
        assert int(child.stdout.readline()) == 6
        assert L.tch_cuda_memory_pool_num_free_pages(0) == 2
        assert L.tch_pool_malloc(4 * 32 * MB, 0, None) is None          # the peer is alive: its pages are its own
        assert b"out of pool memory" in L.tch_host_last_error()
        child.kill()
        child.wait(timeout=20)
        a = L.tch_pool_malloc(4 * 32 * MB, 0, None)                     # the request itself takes them back
        assert a, L.tch_host_last_error()
        assert L.tch_cuda_memory_pool_infer_usage(0) == 0 and L.tch_cuda_memory_pool_num_free_pages(0) == 4
        L.tch_pool_free(a, 0, 0, None)
    finally:
        if child.poll() is None:
            child.kill()
        L.tch_pool_shutdown(0)


def test_pool_quiesces_before_pages_change_hands_and_outside_its_locks(fresh):
    """FreeTrainLocals first lets a runtime drain what it has queued (the hook), then waits for the device, and only
    then takes its locks: the hook below calls back into the pool (it would deadlock under the locks) and sees the
    pages still in training's hands."""
    L = fresh
    assert L.tch_pool_init(0, 256 * MB, 0) == 0
    seen = []
    HOOK = ctypes.CFUNCTYPE(None, ctypes.c_void_p)

    def hook(_):
        seen.append((L.tch_cuda_memory_pool_train_all_usage(0), L.tch_pool_null_backend_probe(0, 1)))
    cb = HOOK(hook)
    try:
        a = L.tch_pool_malloc(64 * MB, 0, None)
        L.tch_pool_free(a, 0, 0, None)
        L.tch_pool_set_quiesce_hook(0, ctypes.cast(cb, ctypes.c_void_p), None)
        assert L.tch_cuda_memory_pool_free_train_local(0) == 64 * MB
        assert seen == [(64 * MB, 0)], seen            # called once, before the backend's quiesce, pages still mapped
        assert L.tch_pool_null_backend_probe(0, 1) >= 1
        L.tch_pool_set_quiesce_hook(0, None, None)
        b = L.tch_pool_malloc(32 * MB, 0, None)
        L.tch_pool_free(b, 0, 0, None)
        L.tch_cuda_memory_pool_free_train_local(0)
        assert len(seen) == 1
    finally:
        L.tch_pool_shutdown(0)


def test_pool_mapping_failure_leaves_no_slot_without_access(fresh):
    """The driver refuses the second of three mappings: the request fails, the slot mapped before the failure
    keeps its page AND has access rights, and the next request over it works."""
    L = fresh
    assert L.tch_pool_init(0, 256 * MB, 0) == 0
    try:
        L.tch_pool_null_backend_fail_map_in(0, 2)
        assert L.tch_pool_malloc(96 * MB, 0, None) is None
        assert b"refuse" in L.tch_host_last_error()
        assert L.tch_pool_null_backend_probe(0, 0) == 0, "a mapped slot was left without access rights"
        assert L.tch_cuda_memory_pool_train_usage(0) == 0
        assert L.tch_cuda_memory_pool_train_all_usage(0) == 32 * MB     # the first slot stays mapped under a free block
        a = L.tch_pool_malloc(96 * MB, 0, None)
        assert a and L.tch_pool_null_backend_probe(0, 0) == 0
        assert L.tch_cuda_memory_pool_train_all_usage(0) == 96 * MB
        L.tch_pool_free(a, 0, 0, None)
        assert L.tch_cuda_memory_pool_free_train_local(0) == 96 * MB
    finally:
        L.tch_pool_shutdown(0)


def test_pool_cross_stream_free_is_deferred(fresh):
    """A block used on another stream is only reusable once that stream's event has finished
    (csrc/torch_allocator_plugin.cc:141-178,383-412); recording the block's own stream is
    ignored (:223-226)."""
    L = fresh
    assert L.tch_pool_init(0, 256 * MB, 0) == 0
    try:
        s1, s2 = ctypes.c_void_p(0x10), ctypes.c_void_p(0x20)
        p = L.tch_pool_malloc(4 * MB, 0, s1)
        L.tch_pool_record_stream(p, 0, s1)                     # own stream: ignored
        L.tch_pool_free(p, 0, 0, s1)
        assert L.tch_cuda_memory_pool_train_usage(0) == 0      # freed at once
        p = L.tch_pool_malloc(4 * MB, 0, s1)
        L.tch_pool_record_stream(p, 0, s2)
        L.tch_pool_free(p, 0, 0, s1)
        assert L.tch_cuda_memory_pool_train_usage(0) == 4 * MB  # still held
        assert L.tch_pool_process_events(0) == 0
        L.tch_pool_null_backend_complete_events(0, 1 << 30)
        assert L.tch_pool_process_events(0) == 1
        assert L.tch_cuda_memory_pool_train_usage(0) == 0
    finally:
        L.tch_pool_shutdown(0)


def test_pool_tagging_releases_only_intermediates(fresh):
    L = fresh
    assert L.tch_pool_init(0, 256 * MB, 0) == 0
    try:
        L.tch_tag_model_start(0)
        w = L.tch_pool_malloc(8 * MB, 0, None)
        L.tch_tag_model_end(0)
        x = L.tch_pool_malloc(4 * MB, 0, None)
        y = L.tch_pool_malloc(4 * MB, 0, None)
        assert L.tch_tag_interm_memory(0, w) == 0              # parameters are never tagged
        assert L.tch_tag_interm_memory(0, x) == 1
        assert L.tch_tag_interm_memory(0, y) == 1
        L.tch_pool_free(y, 0, 0, None)                          # already gone when the release runs
        assert L.tch_release_interm_memory(0) == 4 * MB
        assert L.tch_cuda_memory_pool_train_usage(0) == 8 * MB
        L.tch_pool_free(w, 0, 0, None)
    finally:
        L.tch_pool_shutdown(0)
