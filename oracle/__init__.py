"""TEST INFRASTRUCTURE ONLY: CPU oracle of the fast-weight update operators.

Only ``tests/``, ``__graft_entry__.smoke()`` and the CPU-baseline leg of
``bench.py`` may import this package.  The product (the HIP library and the
``autograd.Function`` wrappers over it) never does.

Two restatements of the reference's ground truth live here:

* ``libfwp_oracle.so`` (``fwp_oracle.c``): plain C, float and double, forward and
  reverse-mode backward, reached through the numpy functions below.
* ``torch_loop.py``: the PyTorch step loops of the reference's self tests, whose
  autograd gives an independent gradient to check the C backward against and
  whose run time is the reference's CPU path.

Parity status: every function below is pinned by closed forms, brute force,
finite differences and autograd in ``tests/test_oracle_*.py``; none is
"parity unpinned".
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfwp_oracle.so")
_lib = None


def build(force=False):
    """Compile the C oracle with the Makefile next to this file."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libfwp_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.fwp_oracle_threads.restype = ctypes.c_int
    return _lib


def threads():
    return int(lib().fwp_oracle_threads())


def set_threads(n):
    lib().fwp_oracle_set_threads(ctypes.c_int(int(n)))


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "_f32"
    if dtype == np.float64:
        return "_f64"
    raise TypeError("oracle supports float32 and float64 only")


def _c(a, dtype):
    return np.ascontiguousarray(np.asarray(a), dtype=dtype)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _call(name, dtype, ptr_args, int_args):
    fn = getattr(lib(), name + _sfx(dtype))
    fn.restype = None
    fn(*[(_p(a) if a is not None else ctypes.c_void_p(0)) for a in ptr_args],
       *[ctypes.c_int(int(i)) for i in int_args])


# --------------------------------------------------------------------- delta

def delta_fwd(q, k, v, beta, W0):
    """out[N,H,L,M], W_L[N,H,E,M] of the delta rule; q,k [N,H,L,E], v [N,H,L,M],
    beta [N,H,L,1], W0 [N,H,E,M]."""
    dt = np.asarray(q).dtype
    q, k, v, beta = _c(q, dt), _c(k, dt), _c(v, dt), _c(beta, dt)
    N, H, L, E = q.shape
    M = v.shape[-1]
    assert k.shape == (N, H, L, E) and v.shape == (N, H, L, M)
    assert beta.shape == (N, H, L, 1) and np.shape(W0) == (N, H, E, M)
    W = _c(W0, dt).copy()
    out = np.empty((N, H, L, M), dt)
    _call("fwp_oracle_delta_fwd", dt, [q, k, v, beta, W, out], [N, H, L, E, M])
    return out, W


def delta_bwd(q, k, v, beta, W0, go):
    """(gq, gk, gv, gbeta, gW0) for upstream gradient go[N,H,L,M]."""
    dt = np.asarray(q).dtype
    q, k, v, beta, W0, go = (_c(x, dt) for x in (q, k, v, beta, W0, go))
    N, H, L, E = q.shape
    M = v.shape[-1]
    gq, gk, gv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    gb, gW0 = np.empty_like(beta), np.empty_like(W0)
    _call("fwp_oracle_delta_bwd", dt, [q, k, v, beta, W0, go, gq, gk, gv, gb, gW0],
          [N, H, L, E, M])
    return gq, gk, gv, gb, gW0


# ------------------------------------------------------------------ sum rule

def sum_fwd(q, k, v, W0):
    """out[N,H,L,M], W_L of the sum update rule W += k (x) v, out = W^T q."""
    dt = np.asarray(q).dtype
    q, k, v = _c(q, dt), _c(k, dt), _c(v, dt)
    N, H, L, E = q.shape
    M = v.shape[-1]
    assert k.shape == (N, H, L, E) and v.shape == (N, H, L, M) and np.shape(W0) == (N, H, E, M)
    W = _c(W0, dt).copy()
    out = np.empty((N, H, L, M), dt)
    _call("fwp_oracle_sum_fwd", dt, [q, k, v, W, out], [N, H, L, E, M])
    return out, W


def sum_bwd(q, k, v, W0, go, through_state=False):
    """(gq, gk, gv).  ``through_state=False`` is what the reference computes: its grad_Q
    leaves out the carried-in state W0; ``True`` is the gradient of the loop as written."""
    dt = np.asarray(q).dtype
    q, k, v, W0, go = (_c(x, dt) for x in (q, k, v, W0, go))
    N, H, L, E = q.shape
    M = v.shape[-1]
    gq, gk, gv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    _call("fwp_oracle_sum_bwd", dt, [q, k, v, W0, go, gq, gk, gv],
          [N, H, L, E, M, int(bool(through_state))])
    return gq, gk, gv


# -------------------------------------------------------------- Delta RNN v2

def rnn_fwd(z, k, v, W0, beta, h0):
    """Argument order of the reference op: (Z, K, V, W, beta, h0).
    Returns out[N,H,L,D], W_L, h_L[N,H,1,D]."""
    dt = np.asarray(z).dtype
    z, k, v, beta = _c(z, dt), _c(k, dt), _c(v, dt), _c(beta, dt)
    N, H, L, D = z.shape
    assert k.shape == v.shape == (N, H, L, D) and beta.shape == (N, H, L, 1)
    assert np.shape(W0) == (N, H, D, D) and np.shape(h0) == (N, H, 1, D)
    W, h = _c(W0, dt).copy(), _c(h0, dt).copy()
    out = np.empty((N, H, L, D), dt)
    _call("fwp_oracle_rnn_fwd", dt, [z, k, v, beta, W, h, out], [N, H, L, D])
    return out, W, h


def rnn_bwd(z, k, v, W0, beta, h0, go):
    """(gz, gk, gv, gbeta)."""
    dt = np.asarray(z).dtype
    z, k, v, beta, W0, h0, go = (_c(x, dt) for x in (z, k, v, beta, W0, h0, go))
    N, H, L, D = z.shape
    gz, gk, gv, gb = (np.empty_like(z), np.empty_like(k), np.empty_like(v),
                      np.empty_like(beta))
    _call("fwp_oracle_rnn_bwd", dt, [z, k, v, beta, W0, h0, go, gz, gk, gv, gb],
          [N, H, L, D])
    return gz, gk, gv, gb


# ------------------------------------------------------------- Delta LSTM v4

def _stack3(gates, dt):
    return np.ascontiguousarray(np.stack([np.asarray(g, dt) for g in gates]))


def lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0):
    """Delta LSTM v4.  ``Zs, Ks, Vs, Bs, Ws`` are triples in gate order (i, u, o):
    z, k, v ``[N,H,L,D]``, beta ``[N,H,L,1]``, W ``[N,H,D,D]``; h0, c0 ``[N,H,1,D]``.
    Returns (out, cell_out, [W_i, W_u, W_o] after L steps, h_L, c_L)."""
    dt = np.asarray(Zs[0]).dtype
    Z, K, V, B, W = (_stack3(x, dt) for x in (Zs, Ks, Vs, Bs, Ws))
    _, N, H, L, D = Z.shape
    assert K.shape == V.shape == Z.shape and B.shape == (3, N, H, L, 1) and W.shape == (3, N, H, D, D)
    assert np.shape(h0) == np.shape(c0) == (N, H, 1, D)
    h, c = _c(h0, dt).copy(), _c(c0, dt).copy()
    out, cell = np.empty((N, H, L, D), dt), np.empty((N, H, L, D), dt)
    _call("fwp_oracle_lstm_fwd", dt, [Z, K, V, B, W, h, c, out, cell], [N, H, L, D])
    return out, cell, [W[0], W[1], W[2]], h, c


def lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go):
    """Gradients for an upstream gradient on ``out`` only (the reference ignores the one on
    the cell output): (gZ, gK, gV, gB), each a list in gate order (i, u, o)."""
    dt = np.asarray(Zs[0]).dtype
    Z, K, V, B, W = (_stack3(x, dt) for x in (Zs, Ks, Vs, Bs, Ws))
    _, N, H, L, D = Z.shape
    h0, c0, go = _c(h0, dt), _c(c0, dt), _c(go, dt)
    gZ, gK, gV, gB = np.empty_like(Z), np.empty_like(K), np.empty_like(V), np.empty_like(B)
    _call("fwp_oracle_lstm_bwd", dt, [Z, K, V, B, W, h0, c0, go, gZ, gK, gV, gB], [N, H, L, D])
    return tuple([g[0], g[1], g[2]] for g in (gZ, gK, gV, gB))


# ------------------------------------------------------- Recurrent Delta Net

def rec_fwd(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0):
    """R_* [1,H,D,D], r_b [1,H,1,D].  Returns out, W_L, h_L."""
    dt = np.asarray(qx).dtype
    qx, kx, vx, bx = _c(qx, dt), _c(kx, dt), _c(vx, dt), _c(bx, dt)
    R_q, R_k, R_v, r_b = _c(R_q, dt), _c(R_k, dt), _c(R_v, dt), _c(r_b, dt)
    N, H, L, D = qx.shape
    assert R_q.shape == R_k.shape == R_v.shape == (1, H, D, D)
    assert r_b.shape == (1, H, 1, D) and bx.shape == (N, H, L, 1)
    assert np.shape(W0) == (N, H, D, D) and np.shape(h0) == (N, H, 1, D)
    W, h = _c(W0, dt).copy(), _c(h0, dt).copy()
    out = np.empty((N, H, L, D), dt)
    _call("fwp_oracle_rec_fwd", dt, [qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h, out],
          [N, H, L, D])
    return out, W, h


def rec_bwd(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0, go):
    """(gqx, gkx, gvx, gbx, gR_q, gR_k, gR_v, gr_b)."""
    dt = np.asarray(qx).dtype
    (qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0, go) = (
        _c(x, dt) for x in (qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0, go))
    N, H, L, D = qx.shape
    gqx, gkx, gvx, gbx = (np.empty_like(qx), np.empty_like(kx), np.empty_like(vx),
                          np.empty_like(bx))
    gRq, gRk, gRv, grb = (np.empty_like(R_q), np.empty_like(R_k), np.empty_like(R_v),
                          np.empty_like(r_b))
    _call("fwp_oracle_rec_bwd", dt,
          [qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0, go, gqx, gkx, gvx, gbx,
           gRq, gRk, gRv, grb], [N, H, L, D])
    return gqx, gkx, gvx, gbx, gRq, gRk, gRv, grb
