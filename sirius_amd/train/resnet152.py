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
import threading
import time
from typing import Optional

import torch

from .. import torch_col
from ..resnet import ResNetEngine
from ..torch_col import EventManager, MemoryPool, dynamic_batch


def setup():
    torch_col.info(f'[Train PID {os.getpid()}] setup')
    return torch_col.setup_colocate_training(0, 1, False, False)


def cleanup():
    torch_col.cleanup_colocate_training(False)


class PeerScript:
    """Stand-in inference server: `at` maps a micro-batch index to ('l1' | 'l2' | 'exit', batch size).
    The command is sent from a side thread `delay_ms` after the micro-batch began, so that it lands
    while kernels are queued, as a real request would."""

    def __init__(self, at, delay_ms=5.0, verbose=False):
        self.server = torch_col.DebugServer(1, verbose=verbose)
        self.at = dict(at)
        self.delay_ms = delay_ms
        self.sent = []

    def on_batch(self, idx):
        cmd = self.at.pop(idx, None)
        if cmd is None:
            return
        kind, bs = cmd

        def fire():
            time.sleep(self.delay_ms / 1e3)
            t = torch_col.get_unix_timestamp_us()
            {"l1": self.server.colocate_l1, "l2": self.server.colocate_l2,
             "exit": self.server.infer_exit}[kind](bs)
            self.sent.append((t, kind, bs))
        threading.Thread(target=fire, daemon=True).start()

    def stop(self):
        self.server.stop()


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
                         lr=0.1, momentum=0.9, weight_decay=1e-4, stream=stream, allocator=allocator)
    model.init_kaiming(seed)
    print(f"Train params memory usage: {MemoryPool.get_memory_usage() * 1024:.2f}M")

    col_ctrl = torch_col.create_colocate_ctrl(train_mode, hook_mode, num_epoch, batch_size)
    col_ctrl.register_pytorch_hook([model])
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

    trainer = torch_col.Trainer(model, iter_train_fn)
    for epoch in range(num_epoch):
        trainer.train_one_epoch(epoch)
        model.synchronize()
        running_loss = model.last_loss()
        epoch_stat = trainer.get_last_epoch_stat()
        epoch_duration = trainer.get_last_epoch_duration()
        mem_info = f'mem {MemoryPool.get_memory_usage():.2f}Gb'
        batch_info = (f'batch cnt {epoch_stat.finished_batch} '
                      f'avg {epoch_duration / max(1, epoch_stat.finished_batch):.1f}ms')
        if train_mode.is_kill_batch():
            batch_info += (f' | try {epoch_stat.tried_batch} kill {epoch_stat.killed_batch}, '
                           f'{epoch_stat.killed_time*1e3:.1f}ms finish {epoch_stat.finished_batch}, '
                           f'{epoch_stat.finished_time*1e3:.1f}ms')
        if global_batch_size is not None:
            batch_info += f' | num_rollback_sampels {epoch_stat.num_rollback_batch}'
        print(f'[ResNet epoch {epoch}] {epoch_duration / 1e3:.3f}s | {batch_info} | batch-size {batch_size} '
              f'| {mem_info} | thpt {epoch_stat.finished_sample / (epoch_duration / 1e3):.3f} '
              f'| loss {running_loss:.6f}', flush=True)
        if col_ctrl.can_exit_after_infer_worklaod_done():
            print('[hook] inference workload done, will exit training', flush=True)
            break

    if train_mode.is_kill_batch():
        overall_stat = trainer.get_overall_stat()
        print("[ResNet] Epoch x Batch {} | Batch Total Tried {} Killed {} Finished {}".format(
            num_epoch * batch_size, overall_stat.tried_batch, overall_stat.killed_batch,
            overall_stat.finished_batch), flush=True)
    col_ctrl.train_end()
    col_ctrl.stop()
    path = EventManager.dump(None, train_mode)
    cleanup()
    return {"trainer": trainer, "model": model, "ctrl": col_ctrl, "profile": path}


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
