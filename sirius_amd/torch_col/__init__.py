"""The training-side plugin surface of the reference (pytorch/torch_col/__init__.py:1-78) on top
of libtorch_col_hip.so.  `import sirius_amd.torch_col as torch_col` gives the same names the
reference's train scripts use."""
from . import xsched
from ._C import *  # noqa: F401,F403
from ._C import (ColocateCtrlHookMode, CtrlEvent, PyColocateStub, PyCtrlMsgEntry, PyDummyStub,  # noqa: F401
                 PyInfTraCommunicator, PySwitchStub, PyTensorWeakRef, TrainMode)
from . import dist  # noqa: F401
from . import util  # noqa: F401
from .util import MemoryPool, EventManager, info, dinfo, info_with_frame  # noqa: F401
from .accumulate import GradAccumulator  # noqa: F401
from . import colocate_ctrl  # noqa: F401
from .colocate_ctrl import (register_saved_tensor_hook, create_colocate_ctrl, DummyCtrl, SwitchCtrl,  # noqa: F401
                            SwitchL1Exception, ColocateCtrl, ColocateAdjustL1Exception,
                            EngineColocateAdjustL1Exception, get_colocate_ctrl)
from . import dynamic_batch  # noqa: F401
from .dynamic_batch import (DynamicBatchDataset, MicroBatchManager, get_dynamic_dataset,  # noqa: F401
                            get_micro_batch_manager, init_dynamic_batch, BatchDistributePolicy)
from .trainer import Trainer  # noqa: F401
from .debug_server import DebugServer  # noqa: F401
from .controller import Controller, ResourceManager, TrainStatus  # noqa: F401


def setup_colocate_training(rank: int, world_size: int, will_use_nccl_comm: bool, init_nccl_process_group: bool):
    """__init__.py:31-66.  Returns the training stream (default priority), which is also made
    torch's current stream; with COLTRAIN_USE_XSCHED it is registered for preemption."""
    import torch
    if init_nccl_process_group and not will_use_nccl_comm:
        raise ValueError('init_nccl_process_group is True but will_use_nccl_comm is False')
    if world_size != 1 or will_use_nccl_comm or init_nccl_process_group:
        raise ValueError('this build trains on one GPU: world_size must be 1 and no collective group is created')
    torch_col_init(rank, world_size)
    torch.cuda.set_device(rank)
    stream = torch.cuda.Stream(device=rank)
    if is_enable_xsched():
        xsched.register_stream(stream)
        info(f'xsched register stream {stream.cuda_stream}')
    else:
        info(f'skip xsched register stream {stream.cuda_stream}')
    torch.cuda.set_stream(stream)
    return stream


def cleanup_colocate_training(destory_nccl_process_group: bool = False):
    """__init__.py:69-77"""
    if is_enable_xsched():
        xsched.unregister_all_streams()


def reset_for_tests():
    """Forget the per-process singletons (controller, dataset, manager, trainer, event log)."""
    colocate_ctrl.CtrlBase._reset_singleton()
    dynamic_batch._reset_singletons()
    Trainer._trainer = None
    EventManager.reset()
