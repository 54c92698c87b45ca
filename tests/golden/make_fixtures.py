"""Writes the golden vectors in this folder.  Run from the repository root:

    python tests/golden/make_fixtures.py

The reference commits no vectors for this path (its training arithmetic lives in PyTorch /
torchvision, its tests compare GPU with CPU on unseeded inputs), so the vectors are produced here,
from seeded inputs, by routines that share no code with what they check:

  ops_small.npz     operator outputs by brute force in float64 (oracle/brute.py: seven-loop
                    convolution and its two gradients, two-pass batch statistics and the textbook
                    BatchNorm gradient, first-maximum pooling index, logsumexp cross-entropy, the
                    scalar SGD recurrence).  Checked against: the torch-CPU oracle and the HIP kernels.
  resnet_tiny.npz   one training step of a 14-convolution Bottleneck ResNet (depths 1,1,1,1, width 8,
                    8 classes, 32x32 images, batch 4) run by torch on the CPU in float64: weights,
                    batch, loss, every gradient, weights after the SGD step.  Checked against: the
                    fp32 oracle step and the HIP engine.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
HERE = os.path.dirname(os.path.abspath(__file__))

from oracle import brute  # noqa: E402
from oracle import resnet as oracle_resnet  # noqa: E402

TINY = dict(depths=(1, 1, 1, 1), num_classes=8, width=8)


def ops_small():
    rng = np.random.default_rng(1234)
    out = {}
    # convolutions: (N, H, W, C, K, R, stride, pad)
    for i, (N, H, W, C, K, R, s, p) in enumerate([(2, 6, 6, 8, 8, 3, 1, 1), (1, 7, 5, 8, 16, 1, 2, 0),
                                                  (2, 9, 9, 8, 8, 3, 2, 1), (1, 8, 8, 4, 8, 7, 2, 3)]):
        x = rng.standard_normal((N, H, W, C))
        w = rng.standard_normal((K, R, R, C)) / np.sqrt(C * R * R)
        y = brute.conv2d_fwd(x, w, s, p)
        dy = rng.standard_normal(y.shape)
        out[f"conv{i}_cfg"] = np.array([N, H, W, C, K, R, s, p])
        out[f"conv{i}_x"], out[f"conv{i}_w"], out[f"conv{i}_y"], out[f"conv{i}_dy"] = x, w, y, dy
        out[f"conv{i}_dx"] = brute.conv2d_dgrad(dy, w, x.shape, s, p)
        out[f"conv{i}_dw"] = brute.conv2d_wgrad(x, dy, w.shape, s, p)
    # BatchNorm, training mode
    for i, (rows, C) in enumerate([(24, 8), (130, 16)]):
        x = rng.standard_normal((rows, C)) * 2 + 0.5
        g, b = rng.uniform(0.5, 1.5, C), rng.standard_normal(C)
        y, mean, var, var_unbiased = brute.bn_train(x, g, b, 1e-5)
        dy = rng.standard_normal((rows, C))
        dx, dg, db = brute.bn_bwd(dy, x, g, 1e-5)
        for k, v in dict(x=x, gamma=g, beta=b, y=y, mean=mean, var=var, var_unbiased=var_unbiased, dy=dy, dx=dx,
                         dgamma=dg, dbeta=db).items():
            out[f"bn{i}_{k}"] = v
    # max pooling 3x3 stride 2 pad 1 with ties (quantised values): integer indices
    x = np.round(rng.standard_normal((2, 9, 9, 8)) * 2) / 2
    y, idx = brute.maxpool_first_max(x, 3, 2, 1)
    out["pool_x"], out["pool_y"], out["pool_idx"] = x, y, idx.astype(np.int64)
    # cross-entropy
    z = rng.standard_normal((6, 16)) * 3
    lab = rng.integers(0, 16, 6)
    rows, mean, dz = brute.cross_entropy(z, lab)
    out["ce_logits"], out["ce_labels"], out["ce_rows"], out["ce_mean"], out["ce_dlogits"] = z, lab, rows, mean, dz
    # SGD with momentum and weight decay, three steps from a zero buffer
    p, g = rng.standard_normal(32), rng.standard_normal(32)
    ps = np.array([brute.sgd_scalar(float(a), float(b), 0.1, 0.9, 1e-4, 3)[0] for a, b in zip(p, g)])
    out["sgd_p"], out["sgd_g"], out["sgd_p3"] = p, g, ps
    np.savez_compressed(os.path.join(HERE, "ops_small.npz"), **out)
    return len(out)


def resnet_tiny():
    model = oracle_resnet.make_model(seed=7, **TINY).double()
    x, y = oracle_resnet.make_batch(4, size=32, num_classes=8, seed=7)
    x = x.double()
    out = {"x": x.numpy().astype(np.float32), "y": y.numpy()}
    for k, v in model.state_dict().items():
        if "num_batches_tracked" not in k:
            out["w0/" + k] = v.numpy().astype(np.float32)  # exact: the weights were drawn in fp32
    hist = oracle_resnet.train_steps(model, x, y, 1, lr=0.1, momentum=0.9, weight_decay=1e-4)
    losses, grads = hist[0]
    out["loss"] = np.array(losses)
    for k, v in grads.items():
        out["grad/" + k] = v.numpy().astype(np.float32)
    for k, v in model.state_dict().items():
        if "num_batches_tracked" not in k:
            out["w1/" + k] = v.numpy().astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "resnet_tiny.npz"), **out)
    return len(out)


if __name__ == "__main__":
    print("ops_small.npz:", ops_small(), "arrays")
    print("resnet_tiny.npz:", resnet_tiny(), "arrays")
