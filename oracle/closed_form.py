"""Float64 numpy forward/backward from the explicit formulas (no autograd).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  For small shapes: the
N x V matrices are materialised.

    u = X W                         (X, W already dequantised)
    t = tanh(u / cap),  z = cap t   tiny/train.py:742
    lse_i = log sum_v exp(z_iv)
    loss_i = sum_k w_k [valid_ik] (lse_i - z[i, y_{i+k}])      tiny/cuda_kernels.py:226-240
    dz_iv = g_i ( (sum_k w_k [valid_ik]) p_iv - sum_k w_k [valid_ik][v = y_{i+k}] )
    du = dz (1 - t^2);  dX = du W^T;  dW = X^T du              tiny/cuda_kernels.py:388-412

valid_ik <=> i+k < N and y_{i+k} != -1.  With a single weight 1 this is plain
cross entropy with ignore_index = -1 (tiny/train.py:743).  'mean' divides by the
number of valid rows.
"""
import numpy as np

IGNORE_INDEX = -1


def forward(X, W, y, cap, mtp_weights=(1.0,)):
    X = np.asarray(X, np.float64)
    W = np.asarray(W, np.float64)
    y = np.asarray(y, np.int64)
    N = X.shape[0]
    u = X @ W
    t = np.tanh(u / cap)
    z = cap * t
    m = z.max(axis=1, keepdims=True)
    lse = (m + np.log(np.exp(z - m).sum(axis=1, keepdims=True)))[:, 0]
    losses = np.zeros(N)
    for k, wk in enumerate(mtp_weights):
        for i in range(N - k):
            tgt = y[i + k]
            if tgt != IGNORE_INDEX:
                losses[i] += wk * (lse[i] - z[i, tgt])
    return dict(u=u, t=t, z=z, lse=lse, losses=losses, argmax=u.argmax(axis=1))


def backward(X, W, y, cap, g, mtp_weights=(1.0,)):
    """g: (N,) upstream gradient of each per-row loss."""
    X = np.asarray(X, np.float64)
    W = np.asarray(W, np.float64)
    y = np.asarray(y, np.int64)
    g = np.asarray(g, np.float64)
    N = X.shape[0]
    f = forward(X, W, y, cap, mtp_weights)
    p = np.exp(f["z"] - f["lse"][:, None])
    dz = np.zeros_like(p)
    for i in range(N):
        sw = 0.0
        for k, wk in enumerate(mtp_weights):
            if i + k < N and y[i + k] != IGNORE_INDEX:
                sw += wk
                dz[i, y[i + k]] -= wk
        dz[i] += sw * p[i]
        dz[i] *= g[i]
    du = dz * (1.0 - f["t"] ** 2)
    return dict(dz=dz, du=du, dx=du @ W.T, dw=X.T @ du, **f)


def mean_loss_and_grads(X, W, y, cap):
    """reduction='mean' over valid rows with upstream gradient 1."""
    y = np.asarray(y, np.int64)
    valid = y != IGNORE_INDEX
    nv = int(valid.sum())
    g = np.where(valid, 1.0 / max(nv, 1), 0.0)
    b = backward(X, W, y, cap, g)
    loss = b["losses"].sum() / nv if nv > 0 else float("nan")
    return loss, b
