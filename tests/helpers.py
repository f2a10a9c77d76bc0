"""Shared helpers of the test-suite: seeded inputs and error measures."""
import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def softmax(x, axis=-1):
    x = x - x.max(axis=axis, keepdims=True)
    e = np.exp(x)
    return e / e.sum(axis=axis, keepdims=True)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def delta_inputs(seed, N, H, L, E, M, dtype=np.float64, w0=False):
    g = rng(seed)
    q = softmax(g.standard_normal((N, H, L, E))).astype(dtype)
    k = softmax(g.standard_normal((N, H, L, E))).astype(dtype)
    v = g.standard_normal((N, H, L, M)).astype(dtype)
    beta = sigmoid(g.standard_normal((N, H, L, 1))).astype(dtype)
    W0 = (g.standard_normal((N, H, E, M)) * (0.5 if w0 else 0.0)).astype(dtype)
    go = g.standard_normal((N, H, L, M)).astype(dtype)
    return q, k, v, beta, W0, go


def rnn_inputs(seed, N, H, L, D, dtype=np.float64, w0=False):
    g = rng(seed)
    z = g.standard_normal((N, H, L, D)).astype(dtype)
    k = softmax(g.standard_normal((N, H, L, D))).astype(dtype)
    v = g.standard_normal((N, H, L, D)).astype(dtype)
    beta = sigmoid(g.standard_normal((N, H, L, 1))).astype(dtype)
    W0 = (g.standard_normal((N, H, D, D)) * (0.5 if w0 else 0.0)).astype(dtype)
    h0 = (g.standard_normal((N, H, 1, D)) * (1.0 if w0 else 0.0)).astype(dtype)
    go = g.standard_normal((N, H, L, D)).astype(dtype)
    return z, k, v, W0, beta, h0, go


def rec_inputs(seed, N, H, L, D, dtype=np.float64, w0=False, rscale=None):
    g = rng(seed)
    qx, kx, vx = (g.standard_normal((N, H, L, D)).astype(dtype) for _ in range(3))
    bx = g.standard_normal((N, H, L, 1)).astype(dtype)
    sc = (1.0 / np.sqrt(D)) if rscale is None else rscale
    R_q, R_k, R_v = ((g.standard_normal((1, H, D, D)) * sc).astype(dtype) for _ in range(3))
    r_b = (g.standard_normal((1, H, 1, D)) * sc).astype(dtype)
    W0 = (g.standard_normal((N, H, D, D)) * (0.5 if w0 else 0.0)).astype(dtype)
    h0 = (g.standard_normal((N, H, 1, D)) * (1.0 if w0 else 0.0)).astype(dtype)
    go = g.standard_normal((N, H, L, D)).astype(dtype)
    return qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0, go


def lstm_inputs(seed, N, H, L, D, dtype=np.float64, w0=False):
    """Delta LSTM v4: (Zs, Ks, Vs, Bs, Ws, h0, c0, go), the first five as (i, u, o) triples."""
    g = rng(seed)
    Zs = [g.standard_normal((N, H, L, D)).astype(dtype) for _ in range(3)]
    Ks = [softmax(g.standard_normal((N, H, L, D))).astype(dtype) for _ in range(3)]
    Vs = [g.standard_normal((N, H, L, D)).astype(dtype) for _ in range(3)]
    Bs = [sigmoid(g.standard_normal((N, H, L, 1))).astype(dtype) for _ in range(3)]
    Ws = [(g.standard_normal((N, H, D, D)) * (0.5 if w0 else 0.0)).astype(dtype) for _ in range(3)]
    h0 = (g.standard_normal((N, H, 1, D)) * (1.0 if w0 else 0.0)).astype(dtype)
    c0 = (g.standard_normal((N, H, 1, D)) * (1.0 if w0 else 0.0)).astype(dtype)
    go = g.standard_normal((N, H, L, D)).astype(dtype)
    return Zs, Ks, Vs, Bs, Ws, h0, c0, go


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)))) if np.size(a) else 0.0


def within(a, b, atol, rtol):
    """|a-b| <= atol + rtol*|b| elementwise (b is the trusted side)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return bool(np.all(np.abs(a - b) <= atol + rtol * np.abs(b)))


def fd_grad(f, x, idx, eps=1e-6):
    """Central difference of scalar f() w.r.t. x.flat[idx] (x is modified in place and restored)."""
    flat = x.reshape(-1)
    old = flat[idx]
    flat[idx] = old + eps
    fp = f()
    flat[idx] = old - eps
    fm = f()
    flat[idx] = old
    return (fp - fm) / (2 * eps)
