import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # Tests that need a second process next to a GPU process (a peer of the shared pool) get it from
    # multiprocessing's fork server.  It is started here, before any test can have initialised the GPU: its
    # children are forked from a process that never touched the device, and the test process itself never
    # forks or execs once it has.
    import multiprocessing as mp
    try:
        mp.get_context("forkserver")
        from multiprocessing import forkserver
        forkserver.ensure_running()
    except Exception:     # a platform without a fork server: those tests skip themselves
        pass


@pytest.fixture(scope="session")
def ctx():
    import torch
    from sirius_amd import ops
    assert torch.cuda.is_available(), "gpu tests need a GPU"
    return ops.Context(torch.cuda.current_stream())
