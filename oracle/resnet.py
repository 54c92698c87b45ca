"""Plain torch.nn ResNet (Bottleneck, stride on the 3x3) and the reference's training
step on CPU.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The reference builds ``torchvision.models.resnet152`` (train/resnet152.py:22); torchvision
is not part of this image, so the architecture is written out here: conv7x7/2 - BN - ReLU -
maxpool3x3/2 - Bottleneck stages [3, 8, 36, 3] with widths 64/128/256/512 (x4 expansion,
stride on the 3x3 conv, 1x1/stride downsample + BN on the first block of a stage) - global
average pool - Linear(2048, classes).  Parameter names follow torchvision's state dict so
weights can be exchanged by name.  Pinned by: parameter count 60,192,808 for [3, 8, 36, 3]
with 1000 classes, output shape, and the per-operator pins in tests/test_oracle_pins.py.

The step restates train/resnet152.py:84-91 with the loss scaling of
pytorch/torch_col/dynamic_batch.py:112-120 and the accumulator of
pytorch/torch_col/accumulate.py:20-47.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F


class Bottleneck(nn.Module):
    expansion = 4

    def __init__(self, inplanes, planes, stride, downsample):
        super().__init__()
        self.conv1 = nn.Conv2d(inplanes, planes, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(planes)
        self.conv2 = nn.Conv2d(planes, planes, 3, stride=stride, padding=1, bias=False)
        self.bn2 = nn.BatchNorm2d(planes)
        self.conv3 = nn.Conv2d(planes, planes * 4, 1, bias=False)
        self.bn3 = nn.BatchNorm2d(planes * 4)
        self.downsample = downsample

    def forward(self, x):
        out = F.relu(self.bn1(self.conv1(x)))
        out = F.relu(self.bn2(self.conv2(out)))
        out = self.bn3(self.conv3(out))
        idn = x if self.downsample is None else self.downsample(x)
        return F.relu(out + idn)


class ResNet(nn.Module):
    def __init__(self, depths=(3, 8, 36, 3), num_classes=1000, width=64):
        super().__init__()
        self.conv1 = nn.Conv2d(3, width, 7, stride=2, padding=3, bias=False)
        self.bn1 = nn.BatchNorm2d(width)
        inplanes = width
        for i, depth in enumerate(depths):
            planes = width * (2 ** i)
            stride = 1 if i == 0 else 2
            blocks = []
            for b in range(depth):
                s = stride if b == 0 else 1
                ds = None
                if b == 0 and (s != 1 or inplanes != planes * 4):
                    ds = nn.Sequential(nn.Conv2d(inplanes, planes * 4, 1, stride=s, bias=False),
                                       nn.BatchNorm2d(planes * 4))
                blocks.append(Bottleneck(inplanes, planes, s, ds))
                inplanes = planes * 4
            setattr(self, f"layer{i + 1}", nn.Sequential(*blocks))
        self.num_stages = len(depths)
        self.fc = nn.Linear(inplanes, num_classes)
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode="fan_out", nonlinearity="relu")

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.bn1(self.conv1(x))), 3, 2, 1)
        for i in range(self.num_stages):
            x = getattr(self, f"layer{i + 1}")(x)
        return self.fc(torch.flatten(F.adaptive_avg_pool2d(x, 1), 1))


def make_model(depths=(3, 8, 36, 3), num_classes=1000, width=64, seed=0):
    """Kaiming-normal (fan_out, relu) convolutions, BN gamma 1 / beta 0, nn.Linear default init."""
    torch.manual_seed(seed)
    return ResNet(depths, num_classes, width)


def make_batch(batch, size=224, num_classes=1000, seed=0):
    g = torch.Generator()
    g.manual_seed(seed + 1)
    x = torch.randn(batch, 3, size, size, generator=g)
    y = torch.randint(0, num_classes, (batch,), generator=g)
    return x, y


def train_steps(model, x, y, steps, lr=0.1, momentum=0.9, weight_decay=1e-4, micro_batches=1, autocast_bf16=False):
    """Run `steps` optimizer steps on the global batch (x, y), each split into `micro_batches`
    equal micro-batches whose losses are scaled by micro/global and whose gradients are
    accumulated, exactly one optimizer step per global batch.  Returns per-step
    (losses of every micro-batch, gradients at the optimizer step)."""
    model.train()
    opt = torch.optim.SGD(model.parameters(), lr=lr, momentum=momentum, weight_decay=weight_decay)
    n = x.shape[0]
    assert n % micro_batches == 0
    mb = n // micro_batches
    history = []
    for _ in range(steps):
        opt.zero_grad(set_to_none=True)
        losses = []
        for i in range(micro_batches):
            xs, ys = x[i * mb:(i + 1) * mb], y[i * mb:(i + 1) * mb]
            if autocast_bf16:
                with torch.autocast("cpu", dtype=torch.bfloat16):
                    loss = F.cross_entropy(model(xs), ys)
            else:
                loss = F.cross_entropy(model(xs), ys)
            losses.append(loss.item())
            (loss / (n / mb)).backward()
        grads = {k: p.grad.detach().clone() for k, p in model.named_parameters()}
        opt.step()
        history.append((losses, grads))
    return history
