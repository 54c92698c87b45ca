"""NHWC operator oracle on CPU fp32 (test infrastructure only; see oracle/__init__.py).

Each function is the PyTorch CPU routine the reference's training step ends up
in (reference call sites: train/resnet152.py:22-29,84-91), wrapped so that it
takes and returns the NHWC / KRSC layouts the HIP kernels use.
"""
import torch
import torch.nn.functional as F


def _nchw(x):
    return x.permute(0, 3, 1, 2).contiguous()


def _nhwc(x):
    return x.permute(0, 2, 3, 1).contiguous()


def _oihw(w_krsc):
    return w_krsc.permute(0, 3, 1, 2).contiguous()


def conv2d_fwd(x, w, stride, pad, bias=None):
    """x [N,H,W,C], w [K,R,S,C] -> y [N,Ho,Wo,K]  (F.conv2d)."""
    return _nhwc(F.conv2d(_nchw(x.float()), _oihw(w.float()), bias, stride=stride, padding=pad))


def conv2d_dgrad(dy, w, x_shape, stride, pad):
    """Gradient of conv2d_fwd w.r.t. x, by autograd through F.conv2d."""
    x = torch.zeros(x_shape, dtype=torch.float32).permute(0, 3, 1, 2).contiguous().requires_grad_(True)
    y = F.conv2d(x, _oihw(w.float()), None, stride=stride, padding=pad)
    (gx,) = torch.autograd.grad(y, x, _nchw(dy.float()))
    return _nhwc(gx)


def conv2d_wgrad(x, dy, w_shape, stride, pad):
    """Gradient of conv2d_fwd w.r.t. w [K,R,S,C], by autograd through F.conv2d."""
    K, R, S, C = w_shape
    w = torch.zeros(K, C, R, S, dtype=torch.float32, requires_grad=True)
    y = F.conv2d(_nchw(x.float()), w, None, stride=stride, padding=pad)
    (gw,) = torch.autograd.grad(y, w, _nchw(dy.float()))
    return gw.permute(0, 2, 3, 1).contiguous()


def bn_fwd_train(x, gamma, beta, running_mean, running_var, momentum=0.1, eps=1e-5, residual=None, relu=False):
    """Training-mode BatchNorm over the last dim of NHWC x; returns (y, mean, invstd) and
    updates the running statistics in place (F.batch_norm)."""
    C = x.shape[-1]
    x2 = x.float().reshape(-1, C)
    y = F.batch_norm(x2, running_mean, running_var, gamma, beta, True, momentum, eps)
    mean = x2.mean(0)
    var = x2.var(0, unbiased=False)
    y = y.reshape(x.shape)
    if residual is not None:
        y = y + residual.float()
    if relu:
        y = torch.relu(y)
    return y, mean, 1.0 / torch.sqrt(var + eps)


def bn_bwd(dy, x, gamma, eps=1e-5, relu_mask=None):
    """(dx, dgamma, dbeta) of training-mode BatchNorm, by autograd; dy is gated by relu_mask > 0."""
    C = x.shape[-1]
    g = dy.float()
    if relu_mask is not None:
        g = g * (relu_mask.float() > 0)
    x2 = x.float().reshape(-1, C).clone().requires_grad_(True)
    gm = gamma.clone().requires_grad_(True)
    bt = torch.zeros(C, requires_grad=True)
    y = F.batch_norm(x2, None, None, gm, bt, True, 0.1, eps)
    gx, gg, gb = torch.autograd.grad(y, (x2, gm, bt), g.reshape(-1, C))
    return gx.reshape(x.shape), gg, gb


def maxpool_fwd(x, ksize, stride, pad):
    """(y, index) with index = h*W + w of the chosen element (F.max_pool2d, return_indices)."""
    y, idx = F.max_pool2d(_nchw(x.float()), ksize, stride, pad, return_indices=True)
    return _nhwc(y), _nhwc(idx)


def maxpool_bwd(dy, x, ksize, stride, pad):
    xc = _nchw(x.float()).requires_grad_(True)
    y = F.max_pool2d(xc, ksize, stride, pad)
    (gx,) = torch.autograd.grad(y, xc, _nchw(dy.float()))
    return _nhwc(gx)


def avgpool_fwd(x):
    return x.float().mean(dim=(1, 2))


def avgpool_bwd(dy, x_shape):
    N, H, W, C = x_shape
    return (dy.float() / (H * W)).reshape(N, 1, 1, C).expand(N, H, W, C).contiguous()


def softmax_ce(logits, labels, loss_scale=1.0):
    """(loss_rows, loss_mean, dlogits of loss_mean*loss_scale) -- nn.CrossEntropyLoss(mean)."""
    z = logits.float().clone().requires_grad_(True)
    rows = F.cross_entropy(z, labels, reduction="none")
    mean = rows.mean()
    (g,) = torch.autograd.grad(mean * loss_scale, z)
    return rows.detach(), mean.detach(), g


def sgd_momentum(params, grads, bufs, lr, momentum, weight_decay, steps=1):
    """torch.optim.SGD on one flat parameter with a pre-zeroed momentum buffer
    (the reference pre-creates the buffers: pytorch/torch_col/util.py:182-191)."""
    p = params.clone().requires_grad_(True)
    opt = torch.optim.SGD([p], lr=lr, momentum=momentum, weight_decay=weight_decay)
    opt.state[p]["momentum_buffer"] = bufs.clone()
    for _ in range(steps):
        p.grad = grads.clone()
        opt.step()
    return p.detach(), opt.state[p]["momentum_buffer"]
