"""The Python surface (sirius_amd.torch_col) end to end on the CPU: the object graph
create_colocate_ctrl -> init_dynamic_batch -> Trainer(model, iter_train_fn) of the reference's
train scripts (train/swin_b.py:26-138), driven by an in-process peer that sends
kColocateAdjustL1(16) and later kInferExit(64).  The engine is a stand-in that owns pool blocks
and calls the checkpoint hook once per layer; no arithmetic runs here, the step itself is
covered by the GPU tests."""
import csv
import os

import pytest
import torch

from sirius_amd._lib import lib

MB = 1 << 20


class StandInEngine:
    """Engine-shaped object: activations are blocks of the (CPU model of the) HBM pool."""

    def __init__(self, layers=12):
        self.layers = layers
        self.grads = self.momentum_buf = object()
        self._hook = None
        self._blocks = []
        self.steps = self.accumulated = 0
        self.forward_calls = []
        self.before_layer = None

    def set_checkpoint_hook(self, fn):
        self._hook = fn

    def _alloc(self, nbytes):
        p = lib().tch_pool_malloc(nbytes, 0, None)
        assert p
        self._blocks.append(p)

    def release_activations(self):
        n = len(self._blocks)
        for p in self._blocks:
            lib().tch_pool_free(p, 0, 0, None)
        self._blocks = []
        return n * 4 * MB

    def forward_backward(self, batch_size):
        self.release_activations()
        self.forward_calls.append(batch_size)
        for phase in ("fwd", "bwd"):
            for i in range(self.layers):
                if self.before_layer:
                    self.before_layer(phase, i)
                if phase == "fwd":
                    self._alloc(4 * MB)
                if self._hook:
                    self._hook(phase, f"layer{i}")
        return 1.0

    def ensure_global_grads(self):
        pass

    def accumulate(self):
        self.accumulated += 1

    def optimizer_step(self, use_global=False, zero_global=True):
        self.steps += 1

    def zero_grad(self):
        pass

    def discard_partial_grads(self):
        pass


@pytest.fixture()
def colocate_env(monkeypatch, tmp_path):
    port = 40000 + os.getpid() % 10000
    env = {"SIRIUS_PORT": str(port), "COLTRAIN_MODE": "colocate-l1", "COLTRAIN_HOOK_MODE": "xsched-sync",
           "COLTRAIN_USE_XSCHED": "1", "COLTRAIN_HAS_INFER_SERVER": "1", "COLTRAIN_USE_SHARED_TENSOR": "1",
           "COLTRAIN_HAS_SHARED_TENSOR_SERVER": "0", "COLTRAIN_SHARED_TENSOR_POOL_GB": "0.5",
           "COLTRAIN_PROFILE_LOG_PATH": str(tmp_path / "train-profile.csv")}
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    import sirius_amd.torch_col as torch_col
    torch_col.torch_col_shutdown()
    torch_col.reset_for_tests()
    yield torch_col
    torch_col.reset_for_tests()
    torch_col.torch_col_shutdown()
    for f in os.listdir("/dev/shm"):
        if f.startswith(f"colserve_shm_{os.getuid()}_p{port}"):
            os.unlink(os.path.join("/dev/shm", f))


def test_names_of_the_reference_surface_exist():
    import sirius_amd.torch_col as tc
    names = """torch_col_init is_configured is_enable_shared_tensor is_enable_dynamic_sm_partition is_enable_xsched
    get_colocate_ctrl_hook_mode get_colocate_train_mode is_release_interm_memory_v1 is_release_interm_memory_v2
    disable_release_interm_memory disable_fbward_hook is_enable_fbward_hook is_train_master get_train_rank
    set_train_rank get_train_world_size set_train_world_size set_train_rank_world_size has_colocated_infer_server
    get_train_profile_log_path cuda_memory_pool_infer_usage cuda_memory_pool_train_usage
    cuda_memory_pool_train_peak_usage cuda_memory_pool_train_all_usage cuda_memory_pool_free_train_local
    release_grad_fn_saved_tensor release_underlying_storage tag_model_start tag_model_end tag_interm_memory
    release_interm_memory untag_interm_memory rearrange_memory RegisterStream UnRegisterStream UnRegisterAllStreams
    GetXQueueSize GetXQueueSizeAllStreams GetTotalXQueueSize AbortStream AbortAllStreams SyncStream SyncAllStreams
    SetRejectCudaCalls GuessNcclBegin GuessNcclEnd IsGuessNcclBegined GetNcclStreams SMPartitionInit
    monitor_sm_partition CtrlEvent PyCtrlMsgEntry PyInfTraCommunicator init_train_info update_current_batch_size
    PyDummyStub PySwitchStub PyColocateStub get_adjust_request_time_stamp get_adjust_done_time_stamp
    get_unix_timestamp get_unix_timestamp_us CallGLOG_INFO CallGLOG_DINFO PyTensorWeakRef TrainMode
    ColocateCtrlHookMode MemoryPool EventManager info dinfo info_with_frame GradAccumulator
    register_saved_tensor_hook create_colocate_ctrl DummyCtrl SwitchCtrl SwitchL1Exception ColocateCtrl
    ColocateAdjustL1Exception EngineColocateAdjustL1Exception Trainer DynamicBatchDataset MicroBatchManager
    get_dynamic_dataset get_micro_batch_manager init_dynamic_batch BatchDistributePolicy get_colocate_ctrl
    DebugServer setup_colocate_training cleanup_colocate_training dist xsched util""".split()
    missing = [n for n in names if not hasattr(tc, n)]
    assert not missing, missing
    for n in """wait_barrier send_msg recv_msg init_dynamic_batch_distributor _DynamicBatchDistirbutor
             init_train_performance_model _PerfModel""".split():
        assert hasattr(tc.dist, n), n
    assert [e.value for e in tc.CtrlEvent] == list(range(14))
    assert tc.TrainMode.COLOCATE_L1.is_kill_batch() and not tc.TrainMode.COLOCATE_L2.is_kill_batch()
    assert tc.ColocateCtrlHookMode.XSCHED_SYNC.use_xsched() and not tc.ColocateCtrlHookMode.SYNC.use_xsched()


def test_handover_64_16_64(colocate_env, capsys):
    tc = colocate_env
    server = tc.DebugServer(1, verbose=False)          # the peer owns the shared segment
    try:
        tc.torch_col_init(0, 1, use_gpu=False)
        tc.init_train_info(64, 64, model_name="resnet152")
        train_mode, hook_mode = tc.get_colocate_train_mode(), tc.get_colocate_ctrl_hook_mode()
        assert train_mode == tc.TrainMode.COLOCATE_L1 and hook_mode == tc.ColocateCtrlHookMode.XSCHED_SYNC
        tc.tag_model_start()
        engine = StandInEngine()
        weights = lib().tch_pool_malloc(40 * MB, 0, None)
        ctrl = tc.create_colocate_ctrl(train_mode, hook_mode, 1, 64)
        ctrl.register_pytorch_hook([engine])
        ds, mgr = tc.init_dynamic_batch(
            dataset_size=64 * 6, dataset_type=tc.dynamic_batch.DatasetType.VISION,
            dataset_config=tc.dynamic_batch.VisionDatasetConfig((3, 4, 4), 10), batch_size=64,
            global_batch_size=64, enable_grad_accumulate=True, checkpoint_micro_batch=True,
            fake_data=True, device="cpu")
        ctrl.train_start()
        acc = tc.GradAccumulator(engine)
        sizes, scales = [], []
        state = {"n": 0}

        def before_layer(phase, i):
            # global batch 2 (third call), in the middle of backward: inference asks for memory
            if state["n"] == 3 and phase == "bwd" and i == 5 and not state.get("sent"):
                state["sent"] = True
                # 4080 MB at 85 MB per sample (server/train_adjuster.cc:535-538,658) = 48 samples less
                assert server.require_memory_mb(4080) == 16
                for _ in range(2000):
                    if ctrl._stub.cmd == tc.CtrlEvent.kColocateAdjustL1:
                        break
                    import time
                    time.sleep(0.001)
        engine.before_layer = before_layer

        def iter_train_fn(batch):
            state["n"] += 1
            if state["n"] == 9:                        # later: inference leaves
                assert server.release_memory_mb(1150 + 85 * 64 + 10) == 64
            sizes.append(len(batch))
            scales.append(mgr.loss_scale(batch))
            loss = engine.forward_backward(len(batch))
            mgr.optimizer_step(batch, engine, grad_accumulator=acc)
            return loss * len(batch)

        trainer = tc.Trainer(engine, iter_train_fn)
        trainer.train_one_epoch(0)
        stat = trainer.get_last_epoch_stat()

        # 64, 64, 64 (killed), then the killed global batch again as 4 x 16, ...
        assert sizes[:3] == [64, 64, 64]
        assert sizes[3:7] == [16, 16, 16, 16]
        assert scales[0] == 1.0 and scales[3] == 0.25          # loss /= 64 / 16
        assert 64 in sizes[8:]                                  # back at 64 after kInferExit
        assert stat.killed_batch == 1 and stat.finished_sample == 64 * 6
        assert engine.steps == 6                                # one optimizer step per global batch
        assert engine.accumulated == stat.finished_batch
        # the reply went out with the request's id, after the activations had gone back to the pool
        done = [m for _, m in server.received if m.event == tc.CtrlEvent.kColocateAdjustL1Done]
        assert len(done) == 1 and done[0].id == 1
        a = ctrl.last_adjust
        assert a["released_bytes"] > 0 and a["pool_bytes_returned"] >= 32 * MB
        req, fin = tc.get_adjust_request_time_stamp(), tc.get_adjust_done_time_stamp()
        assert len(req) == 1 and len(fin) == 1 and 0 <= fin[0] - req[0] < 50_000   # < 50 ms
        out = capsys.readouterr().out
        assert "[Adjust L1" in out and "batch_size: 64 -> 16" in out
        # event log: names and tags of the reference's train-profile.csv
        ctrl.train_end()
        ctrl.stop()
        path = tc.EventManager.dump(None, train_mode)
        rows = list(csv.DictReader(open(path)))
        assert list(rows[0].keys()) == ["timestamp", "name", "loc", "duration", "tag", "rank"]
        names = [r["name"] for r in rows]
        assert "epoch_00_384" in names and "recv_adjust" in names and "adjust_done" in names
        assert any(n.startswith("batch_exception_00_002_64") for n in names)
        assert any(n.startswith("batch_restart_00_002") for n in names)
        assert "adjust_l1" in names and "wait_valid_batch" in names
        tags = {r["name"]: r["tag"] for r in rows}
        assert tags["batch_00_002_64"] == "cancel" and tags["batch_00_000_64"] == "finish"
        assert tags["global_batch_00_000_64"] == "finish"
        assert {r["tag"] for r in rows if r["name"] == "optimizer_step"} == {"global", "local"}
        lib().tch_pool_free(weights, 0, 0, None)
    finally:
        server.stop()


def test_controller_command_ids_skip_rule_and_free_memory(colocate_env):
    """The server's controller and resource manager as the stand-in peer restates them
    (server/control/controller.cc:84-150,207-327,377-386; server/resource_manager.cc:22-87): command ids count
    every call, nothing is sent to an idle trainer, a ColocateAdjust that finds no rank with an unpublished shrink
    is skipped with id 0, the wait returns on a reply with an id >= the command's; free memory = pool - inference
    - max(training now, training predicted) - margin."""
    import time
    tc = colocate_env
    ctl = tc.Controller(1, colocate_level=1)
    stub = None
    try:
        tc.torch_col_init(0, 1, use_gpu=False)
        tc.init_train_info(64, 64, model_name="resnet152")
        # idle trainer: ids are taken, nothing is sent
        assert ctl.is_train_idle()
        assert ctl.colocate_infer_require_adjust([48]) == 1 and ctl.colocate_adjust(8) == 2 and not ctl.sent
        assert ctl.wait_colocate_adjust_done(2) is True          # idle: nothing to wait for
        stub = tc.PyColocateStub(64)
        stub.train_start()
        assert ctl.wait_train_status(tc.TrainStatus.kRunning, 5.0)
        assert ctl.target_batch_size == 64
        # board: target 64, unpublished 64 -> no rank has a shrink pending: skipped, id 0, but the id is used up
        assert ctl.colocate_adjust(8) == 0 and not ctl.sent
        # inference asks for 4080 MB: 48 samples at 85 MB (server/train_adjuster.cc:535-538) -> target 16, id 4
        cmd = ctl.infer_require_memory_mb(4080)
        assert cmd == 4 and tc._C.get_train_info(0, "target_batch_size_unpublished") == 16
        assert [(r, i, e, v) for _, r, i, e, v in ctl.sent] == [(0, 4, tc.CtrlEvent.kColocateAdjustL1, 16)]
        for _ in range(2000):
            if stub.cmd == tc.CtrlEvent.kColocateAdjustL1:
                break
            time.sleep(0.001)
        assert stub.cmd == tc.CtrlEvent.kColocateAdjustL1 and stub.unpub_target_batch_size == 16 and stub.target_batch_size == 64
        # now a shrink is pending (unpublished 16 < published 64): ColocateAdjust goes out, value = launcher target - 8
        assert ctl.wait_colocate_adjust_done(cmd, timeout_s=0.05) is False
        assert ctl.colocate_adjust(8) == 5 and ctl.sent[-1][2:] == (5, tc.CtrlEvent.kColocateAdjustL1, 8)
        stub.adjust_l1_done()
        assert ctl.wait_colocate_adjust_done(cmd, timeout_s=5.0) is True and ctl.adjust_done_ids[0] >= cmd
        # resource manager on the pool of this environment (0.5 GB): training predicted at its new target
        rm = tc.ResourceManager(train_memory_over_predict_mb=10.0)
        pool_mb = tc._C.cuda_memory_pool_nbytes(0) / 1024 / 1024
        assert pool_mb == 512.0
        target = tc._C.get_train_info(0, "target_batch_size_unpublished")
        assert rm.predict_train_memory_mb() == 1150 + 85 * target
        blk = lib().tch_pool_malloc(96 * MB, 0, None)
        assert rm.train_memory_mb() >= 96.0 and rm.infer_memory_mb() == 0.0
        assert rm.free_memory_mb() == pool_mb - 0.0 - max(rm.train_memory_mb(), rm.predict_train_memory_mb()) - 10.0
        assert rm.train_avail_memory_mb() == pool_mb - 10.0
        lib().tch_pool_free(blk, 0, 0, None)
        # inference leaves 1150 + 85 * 64 + 10 MB to training: back to the initial size, as kInferExit
        cmd = ctl.infer_release_memory_mb(1150 + 85 * 64 + 10)
        assert ctl.sent[-1][2:] == (cmd, tc.CtrlEvent.kInferExit, 64)
        stub.train_end()
        assert ctl.wait_train_status(tc.TrainStatus.kIdle, 5.0)
    finally:
        if stub is not None:
            stub.stop()
        ctl.stop()
