"""ResNet-152 training under the colocation protocol: the flow of the reference's train scripts
(train/swin_b.py:14-138 for the object graph, train/resnet152.py:17-153 for model, optimizer and
dataset shape) on the HIP engine.

    python -m sirius_amd.train.resnet152 --batch-size 64 --num-epoch 1

The environment contract is the launcher's (server/train_launcher.cc:205-305): COLTRAIN_MODE,
COLTRAIN_HOOK_MODE, COLTRAIN_USE_XSCHED, COLTRAIN_HAS_INFER_SERVER, COLTRAIN_USE_SHARED_TENSOR,
COLTRAIN_SHARED_TENSOR_POOL_GB, COLTRAIN_PROFILE_LOG_PATH.  `--peer-script` runs an in-process
stand-in for the inference server that sends adjust commands at given micro-batch indices.
"""
import argparse
import os
import sys
from typing import Optional

import torch

from .. import torch_col
from ..resnet import ResNetEngine
from ..torch_col import MemoryPool, dynamic_batch
from .common import PeerScript, attach_cu_partition, autotune_requested, cleanup, run_epochs, setup  # noqa: F401  (PeerScript is part of this module's interface)


def train(num_epoch: int, batch_size: int, global_batch_size: Optional[int] = None, dataset_size: int = 1000,
          dtype=torch.bfloat16, depths=(3, 8, 36, 3), width=64, num_classes=1000, image_size=224,
          peer: Optional[PeerScript] = None, num_distinct_samples: Optional[int] = 256, seed=0):
    stream = setup()
    torch_col.init_train_info(batch_size, batch_size, model_name='resnet152')
    train_mode = torch_col.get_colocate_train_mode()
    hook_mode = torch_col.get_colocate_ctrl_hook_mode()

    if torch_col.is_enable_shared_tensor():
        torch_col.tag_model_start()
    allocator = torch_col.pool_empty if torch_col.is_enable_shared_tensor() else None
    model = ResNetEngine(depths=depths, width=width, num_classes=num_classes, dtype=dtype, image_size=image_size,
                         lr=0.1, momentum=0.9, weight_decay=1e-4, stream=stream, allocator=allocator,
                         autotune=autotune_requested())
    model.init_kaiming(seed)
    print(f"Train params memory usage: {MemoryPool.get_memory_usage() * 1024:.2f}M")

    col_ctrl = torch_col.create_colocate_ctrl(train_mode, hook_mode, num_epoch, batch_size)
    col_ctrl.register_pytorch_hook([model])
    attach_cu_partition(model)
    enable_grad_accumulator = global_batch_size is not None or col_ctrl.train_mode.is_colocate()
    checkpoint_micro_batch = col_ctrl.train_mode.is_kill_batch()
    train_dataset, batch_manager = torch_col.init_dynamic_batch(
        dataset_size=dataset_size, dataset_type=dynamic_batch.DatasetType.VISION,
        dataset_config=dynamic_batch.VisionDatasetConfig((3, image_size, image_size), num_classes),
        batch_size=batch_size, global_batch_size=global_batch_size,
        enable_grad_accumulate=enable_grad_accumulator, checkpoint_micro_batch=checkpoint_micro_batch,
        lazy_batch_distributing=False, fake_data=True,
        batch_distribute_policy=dynamic_batch.BatchDistributePolicy.BY_PERFORMANCE,
        num_distinct_samples=num_distinct_samples, seed=seed)

    col_ctrl.train_start()
    torch_col.util.initialize_sgd_optimizer(model)
    grad_accumulator = torch_col.GradAccumulator(model) if batch_manager._checkpoint_micro_batch else None
    print(f'resnet152 after initialize, allocated {MemoryPool.get_allocated_memory()} '
          f'cached {MemoryPool.get_memory_usage()}', flush=True, file=sys.stderr)

    counter = {"n": 0}

    def iter_train_fn(batch: dynamic_batch.Batch):
        if peer is not None:
            peer.on_batch(counter["n"])
        counter["n"] += 1
        images, targets = batch['images'], batch['labels']
        # loss /= global_batch_size / batch_size is folded into the loss kernel
        plan, _ = model.forward_backward(images, targets, loss_scale=batch_manager.loss_scale(batch))
        batch_manager.optimizer_step(batch, model, grad_accumulator=grad_accumulator)
        # the loss stays on the GPU (no read-back per micro-batch): the epoch line reads the last one
        return 0.0

    return run_epochs("ResNet", model, iter_train_fn, col_ctrl, train_mode, num_epoch, batch_size, global_batch_size)


def main():
    parser = argparse.ArgumentParser('Train Resnet')
    parser.add_argument('--batch-size', type=int, default=64)
    parser.add_argument('--global-batch-size', type=int, default=None)
    parser.add_argument('--num-epoch', type=int, default=1)
    parser.add_argument('--dataset-size', type=int, default=1000)
    parser.add_argument('--fp32', action='store_true')
    parser.add_argument('--peer-script', type=str, default='',
                        help="e.g. '10:l1:16,20:exit:64' = at micro-batch 10 send AdjustL1 to 16, at 20 InferExit to 64")
    args = parser.parse_args()
    peer = None
    if args.peer_script:
        at = {}
        for item in args.peer_script.split(','):
            idx, kind, bs = item.split(':')
            at[int(idx)] = (kind, int(bs))
        os.environ.setdefault("COLTRAIN_HAS_INFER_SERVER", "1")
        peer = PeerScript(at, verbose=True)
    print(f"ResNet152 training, batch-size={args.batch_size}, num-epoch={args.num_epoch}")
    try:
        train(args.num_epoch, args.batch_size, global_batch_size=args.global_batch_size,
              dataset_size=args.dataset_size, dtype=torch.float32 if args.fp32 else torch.bfloat16, peer=peer)
    finally:
        if peer is not None:
            peer.stop()


if __name__ == '__main__':
    main()
