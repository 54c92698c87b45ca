"""Closed forms and brute force on tiny inputs (numpy / pure Python), used to PIN the operator
oracle in oracle/nn_ops.py.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Each function states the mathematics directly, with no shared code path with torch, so that a
dropped term, a wrong sign or index or a transposed operand in nn_ops fails a comparison.
"""
import math

import numpy as np


def conv2d_fwd(x, w, stride, pad):
    """7-loop convolution.  x [N,H,W,C], w [K,R,S,C] -> y [N,Ho,Wo,K] (float64)."""
    N, H, W, C = x.shape
    K, R, S, _ = w.shape
    Ho, Wo = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    y = np.zeros((N, Ho, Wo, K))
    for n in range(N):
        for ho in range(Ho):
            for wo in range(Wo):
                for k in range(K):
                    acc = 0.0
                    for r in range(R):
                        for s in range(S):
                            hi, wi = ho * stride - pad + r, wo * stride - pad + s
                            if 0 <= hi < H and 0 <= wi < W:
                                for c in range(C):
                                    acc += float(x[n, hi, wi, c]) * float(w[k, r, s, c])
                    y[n, ho, wo, k] = acc
    return y


def conv2d_dgrad(dy, w, x_shape, stride, pad):
    """Scatter form of the data gradient: every product of the forward sum sends dy*w back to x."""
    N, H, W, C = x_shape
    K, R, S, _ = w.shape
    _, Ho, Wo, _ = dy.shape
    dx = np.zeros(x_shape)
    for n in range(N):
        for ho in range(Ho):
            for wo in range(Wo):
                for r in range(R):
                    for s in range(S):
                        hi, wi = ho * stride - pad + r, wo * stride - pad + s
                        if 0 <= hi < H and 0 <= wi < W:
                            for k in range(K):
                                dx[n, hi, wi, :] += float(dy[n, ho, wo, k]) * w[k, r, s, :].astype(np.float64)
    return dx


def conv2d_wgrad(x, dy, w_shape, stride, pad):
    N, H, W, C = x.shape
    K, R, S, _ = w_shape
    _, Ho, Wo, _ = dy.shape
    dw = np.zeros(w_shape)
    for n in range(N):
        for ho in range(Ho):
            for wo in range(Wo):
                for r in range(R):
                    for s in range(S):
                        hi, wi = ho * stride - pad + r, wo * stride - pad + s
                        if 0 <= hi < H and 0 <= wi < W:
                            dw[:, r, s, :] += np.outer(dy[n, ho, wo, :].astype(np.float64),
                                                       x[n, hi, wi, :].astype(np.float64))
    return dw


def bn_train(x, gamma, beta, eps):
    """fp64 batch statistics over all but the last dim: (y, mean, biased var, unbiased var)."""
    x2 = x.reshape(-1, x.shape[-1]).astype(np.float64)
    n = x2.shape[0]
    mean = x2.sum(0) / n
    var = ((x2 - mean) ** 2).sum(0) / n
    y = (x2 - mean) / np.sqrt(var + eps) * gamma + beta
    return y.reshape(x.shape), mean, var, var * n / max(n - 1, 1)


def bn_bwd(dy, x, gamma, eps):
    """Closed form: dx = gamma*invstd*(g - mean(g) - xhat*mean(g*xhat)), dgamma = sum g*xhat, dbeta = sum g."""
    x2 = x.reshape(-1, x.shape[-1]).astype(np.float64)
    g = dy.reshape(-1, x.shape[-1]).astype(np.float64)
    n = x2.shape[0]
    mean = x2.mean(0)
    invstd = 1.0 / np.sqrt(((x2 - mean) ** 2).mean(0) + eps)
    xhat = (x2 - mean) * invstd
    dbeta, dgamma = g.sum(0), (g * xhat).sum(0)
    dx = gamma * invstd * (g - dbeta / n - xhat * dgamma / n)
    return dx.reshape(x.shape), dgamma, dbeta


def maxpool_first_max(x, ksize, stride, pad):
    """(y, index): row-major window scan, a later element wins only if strictly greater or NaN,
    index = h*W + w in the input plane; the start index is the first in-range element."""
    N, H, W, C = x.shape
    Ho, Wo = (H + 2 * pad - ksize) // stride + 1, (W + 2 * pad - ksize) // stride + 1
    y = np.zeros((N, Ho, Wo, C), dtype=x.dtype)
    idx = np.zeros((N, Ho, Wo, C), dtype=np.int64)
    for n in range(N):
        for ho in range(Ho):
            for wo in range(Wo):
                h0, w0 = max(ho * stride - pad, 0), max(wo * stride - pad, 0)
                h1, w1 = min(ho * stride - pad + ksize, H), min(wo * stride - pad + ksize, W)
                for c in range(C):
                    best, arg = -math.inf, h0 * W + w0
                    for h in range(h0, h1):
                        for w in range(w0, w1):
                            v = float(x[n, h, w, c])
                            if v > best or math.isnan(v):
                                best, arg = v, h * W + w
                    y[n, ho, wo, c], idx[n, ho, wo, c] = best, arg
    return y, idx


def cross_entropy(logits, labels):
    """rows of logsumexp(z) - z[label], their mean, and d(mean)/dz = (softmax - onehot)/rows."""
    z = logits.astype(np.float64)
    m = z.max(1, keepdims=True)
    lse = m[:, 0] + np.log(np.exp(z - m).sum(1))
    rows = lse - z[np.arange(len(labels)), labels]
    sm = np.exp(z - lse[:, None])
    sm[np.arange(len(labels)), labels] -= 1.0
    return rows, rows.mean(), sm / len(labels)


def sgd_scalar(p, g, lr, momentum, wd, steps):
    """Scalar recurrence with a pre-zeroed buffer: g' = g + wd*p; buf = mu*buf + g'; p -= lr*buf."""
    buf = 0.0
    for _ in range(steps):
        gp = g + wd * p
        buf = momentum * buf + gp
        p = p - lr * buf
    return p, buf
