"""The one event log the reference holds (train-profile.csv: dataset 1000, global batch 500, micro-batch 32) as a
golden vector for the batch distributor, the micro-batch manager and the event log: the same run replayed through
this package's object graph writes the same rows (names, tags, order); and the throughput post-processing
(util/profile/throughput.py, collect_train_thpt.py) on that log gives the figures its columns fix.
tests/golden/train_profile_reference.csv holds the first two epochs of the reference's file (copied by
tests/golden/make_profile_fixture.py)."""
import csv
import os

import pytest

from sirius_amd._lib import lib

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURE = os.path.join(HERE, "golden", "train_profile_reference.csv")


class CountingEngine:
    """Engine-shaped object that counts what the training loop asks of it."""

    def __init__(self):
        self.grads = self.momentum_buf = object()
        self.steps = self.zeroed = 0

    def set_checkpoint_hook(self, fn):
        pass

    def release_activations(self):
        return 0

    def optimizer_step(self, use_global=False, zero_global=True):
        self.steps += 1

    def zero_grad(self):
        self.zeroed += 1

    def ensure_global_grads(self):
        pass

    def discard_partial_grads(self):
        pass


@pytest.fixture()
def plain_env(monkeypatch, tmp_path):
    port = 41000 + os.getpid() % 10000
    for k in list(os.environ):
        if k.startswith("COLTRAIN_"):
            monkeypatch.delenv(k)
    monkeypatch.setenv("SIRIUS_PORT", str(port))
    monkeypatch.setenv("COLTRAIN_MODE", "normal")
    monkeypatch.setenv("COLTRAIN_PROFILE_LOG_PATH", str(tmp_path / "train-profile.csv"))
    import sirius_amd.torch_col as torch_col
    torch_col.torch_col_shutdown()
    torch_col.reset_for_tests()
    yield torch_col
    torch_col.reset_for_tests()
    torch_col.torch_col_shutdown()
    for f in os.listdir("/dev/shm"):
        if f.startswith(f"colserve_shm_{os.getuid()}_p{port}"):
            os.unlink(os.path.join("/dev/shm", f))


def _reference_rows():
    return [r for r in csv.DictReader(open(FIXTURE)) if r["name"]]


def test_replay_writes_the_rows_of_the_reference_log(plain_env):
    tc = plain_env
    tc.torch_col_init(0, 1, use_gpu=False)
    tc.init_train_info(32, 32, model_name="resnet152")
    train_mode, hook_mode = tc.get_colocate_train_mode(), tc.get_colocate_ctrl_hook_mode()
    assert train_mode == tc.TrainMode.NORMAL
    engine = CountingEngine()
    ctrl = tc.create_colocate_ctrl(train_mode, hook_mode, 2, 32)
    ctrl.register_pytorch_hook([engine])
    # train/resnet152.py:44-60 with --batch-size 32 --global-batch-size 500: gradients accumulate over the
    # micro-batches of a global batch, no checkpoint per micro-batch outside the colocation modes
    ds, mgr = tc.init_dynamic_batch(
        dataset_size=1000, dataset_type=tc.dynamic_batch.DatasetType.VISION,
        dataset_config=tc.dynamic_batch.VisionDatasetConfig((3, 2, 2), 10), batch_size=32, global_batch_size=500,
        enable_grad_accumulate=True, checkpoint_micro_batch=False, fake_data=True, device="cpu")
    ctrl.train_start()
    sizes, updates = [], []

    def iter_train_fn(batch):
        sizes.append(len(batch))
        updates.append(batch.should_update_param())
        assert abs(mgr.loss_scale(batch) - len(batch) / 500) < 1e-12      # loss /= global / micro
        mgr.optimizer_step(batch, engine)
        return 0.0

    trainer = tc.Trainer(engine, iter_train_fn)
    for epoch in range(2):
        trainer.train_one_epoch(epoch)
    ctrl.train_end()
    ctrl.stop()
    path = tc.EventManager.dump(None, train_mode)
    mine = [r for r in csv.DictReader(open(path)) if r["name"]]
    ref = _reference_rows()
    assert list(mine[0].keys()) == ["timestamp", "name", "loc", "duration", "tag", "rank"]
    key = lambda r: (r["name"], r["loc"], r["tag"], r["rank"])   # noqa: E731
    assert [key(r) for r in mine] == [key(r) for r in ref]
    # what the names say: 15 x 32 + 20 per global batch, the step on the closing micro-batch only
    per_global = [32] * 15 + [20]
    assert sizes == per_global * 4
    assert updates == ([False] * 15 + [True]) * 4
    assert engine.steps == 4 and engine.zeroed == 4
    stat = trainer.get_last_epoch_stat()
    assert stat.finished_batch == 32 and stat.finished_sample == 1000 and stat.killed_batch == 0
    # starts are ordered as logged, every micro-batch lies inside its global batch, every global batch in its epoch
    ts = [float(r["timestamp"]) for r in mine]
    assert ts == sorted(ts)


def test_throughput_figures_of_the_reference_log(tmp_path):
    from sirius_amd.torch_col import profile_thpt as P
    (t,) = P.read_train_profile(FIXTURE)
    assert [len(t[k]) for k in ("epoch", "global_batch", "batch", "batch_restart", "wait_valid_batch")] == [2, 4, 64, 0, 64]
    assert [e["epoch_size"] for e in t["epoch"]] == [1000, 1000]
    assert {g["batch_size"] for g in t["global_batch"]} == {500} and all(g["finished"] for g in t["global_batch"])
    assert [b["batch"] for b in t["batch"][:17]] == list(range(17)) and t["batch"][15]["batch_size"] == 20
    begin, end = t["batch"][0]["start_time"], t["batch"][-1]["end_time"]
    ideal, real, avg_t, avg_sz, n_done, n_cancel, waste, restart_waste = P.eval_throughput(
        t["batch"], begin, end, t["batch_restart"], t["wait_valid_batch"])
    # the same sums taken with awk over the fixture's columns: 64 micro-batches, 2000 samples, 11019.19 ms of
    # micro-batch time, 11032.17 ms from the first start to the last end
    assert (n_done, n_cancel) == (64, 0) and waste == 0 and restart_waste == -1
    # (end - start is taken of sums with a 1.7e12 timestamp, as in the reference: good to about 1e-4 ms per row)
    assert abs(ideal - 2000 / 11019.19 * 1000) < 1e-3 and abs(ideal - 181.501544) < 1e-3
    assert abs(real - 2000 / 11032.17 * 1000) < 1e-4
    assert abs(avg_t - 172.174844) < 1e-5 and avg_sz == 31.25
    # a window that cuts the first epoch off: only the micro-batches that lie inside count
    second = t["epoch"][1]
    _, _, _, _, n2, _, _, _ = P.eval_throughput(t["batch"], second["start_time"], end)
    assert n2 == 32
    # a cancelled micro-batch is waste, not throughput
    cut = [dict(b) for b in t["batch"]]
    cut[3]["finished"], cut[3]["tag"] = False, "cancel"
    i3, r3, _, _, n3, c3, w3, _ = P.eval_throughput(cut, begin, end)
    assert (n3, c3) == (63, 1) and abs(w3 - cut[3]["duration"] / 11032.17 * 100) < 1e-6
    assert abs(r3 - (2000 - 32) / 11032.17 * 1000) < 1e-4
    # per epoch: 1000 samples in 5877.10 and 5156.01 ms
    avg, e2e, secs = P.eval_throughput_by_epoch(t["epoch"], t["epoch"][0]["start_time"], t["epoch"][1]["end_time"])
    assert abs(avg - (1000 / 5877.10 + 1000 / 5156.01) / 2 * 1000) < 1e-6
    assert abs(secs - (5877.10 + 5156.01) / 2 / 1000) < 1e-9
    assert abs(e2e - 2000 / (1736345215640.28 + 5156.01 - 1736345209763.13) * 1000) < 1e-4
    assert P.eval_throughput([], 0, 1) == (-1,) * 8 and P.eval_throughput_by_epoch([], 0, 1) == (-1,) * 3
    # collect_train_thpt: start, end, size of every finished micro-batch
    out = tmp_path / "thpt.csv"
    assert P.collect_train_thpt(FIXTURE, str(out)) == 64
    rows = list(csv.DictReader(open(out)))
    assert list(rows[0].keys()) == ["start_timestamp", "end_timestamp", "batch_size"]
    assert float(rows[0]["start_timestamp"]) == 1736345209764.06 and rows[15]["batch_size"] == "20"
    assert abs(float(rows[0]["end_timestamp"]) - (1736345209764.06 + 875.95)) < 1e-6
