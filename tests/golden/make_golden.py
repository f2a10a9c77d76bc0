"""Writes the golden fixtures of this directory from the CPU oracle.

The reference ships no golden vectors for the fast-weight operators, so these
freeze seeded inputs (float32) and the float64 oracle's outputs and gradients on
them.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle  # noqa: E402
from helpers import delta_inputs, lstm_inputs, rec_inputs, rnn_inputs  # noqa: E402


def f32(arrays):
    return [a.astype(np.float32) for a in arrays]


def f64(arrays):
    return [a.astype(np.float64) for a in arrays]


def main():
    # the CPU-runnable benchmark configuration: B=2,H=2,T=64,D=16, W0=0, seed 0
    q, k, v, beta, W0, go = f32(delta_inputs(0, 2, 2, 64, 16, 16))
    out, W = oracle.delta_fwd(*f64([q, k, v, beta, W0]))
    gq, gk, gv, gb, _ = oracle.delta_bwd(*f64([q, k, v, beta, W0, go]))
    np.savez_compressed(os.path.join(HERE, "delta_b2h2t64d16.npz"), q=q, k=k, v=v, beta=beta, W0=W0, go=go,
                        out=out, W=W, gq=gq, gk=gk, gv=gv, gbeta=gb)

    z, k, v, W0, beta, h0, go = f32(rnn_inputs(1, 1, 2, 32, 32, w0=True))
    out, W, h = oracle.rnn_fwd(*f64([z, k, v, W0, beta, h0]))
    gz, gk, gv, gb = oracle.rnn_bwd(*f64([z, k, v, W0, beta, h0, go]))
    np.savez_compressed(os.path.join(HERE, "rnn_b1h2t32d32.npz"), z=z, k=k, v=v, W0=W0, beta=beta, h0=h0, go=go,
                        out=out, W=W, h=h, gz=gz, gk=gk, gv=gv, gbeta=gb)

    x = f32(rec_inputs(2, 1, 2, 32, 32, w0=True))
    names = "qx kx vx bx R_q R_k R_v r_b W0 h0 go".split()
    out, W, h = oracle.rec_fwd(*f64(x[:10]))
    grads = oracle.rec_bwd(*f64(x))
    gnames = ["g" + n for n in names[:8]]
    np.savez_compressed(os.path.join(HERE, "rec_b1h2t32d32.npz"), **dict(zip(names, x)), out=out, W=W, h=h,
                        **dict(zip(gnames, grads)))

    # sum rule at the shape of the reference's self test (E != M), carried-in state; both gradient conventions
    q, k, v, _, W0, go = f32(delta_inputs(3, 3, 5, 7, 11, 4, w0=True))
    out, W = oracle.sum_fwd(*f64([q, k, v, W0]))
    gq, gk, gv = oracle.sum_bwd(*f64([q, k, v, W0, go]))
    gq_exact = oracle.sum_bwd(*f64([q, k, v, W0, go]), through_state=True)[0]
    np.savez_compressed(os.path.join(HERE, "sum_b3h5t7e11m4.npz"), q=q, k=k, v=v, W0=W0, go=go, out=out, W=W,
                        gq=gq, gk=gk, gv=gv, gq_exact=gq_exact)

    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(4, 1, 2, 24, 16, dtype=np.float32, w0=True)
    out, cell, Wn, h, c = oracle.lstm_fwd(f64(Zs), f64(Ks), f64(Vs), f64(Bs), f64(Ws), h0.astype(np.float64),
                                          c0.astype(np.float64))
    gZ, gK, gV, gB = oracle.lstm_bwd(f64(Zs), f64(Ks), f64(Vs), f64(Bs), f64(Ws), h0.astype(np.float64),
                                     c0.astype(np.float64), go.astype(np.float64))
    stack = lambda xs: np.stack(xs)
    np.savez_compressed(os.path.join(HERE, "lstm_b1h2t24d16.npz"), Z=stack(Zs), K=stack(Ks), V=stack(Vs),
                        B=stack(Bs), W0=stack(Ws), h0=h0, c0=c0, go=go, out=out, cell=cell, W=stack(Wn), h=h,
                        c=c, gZ=stack(gZ), gK=stack(gK), gV=stack(gV), gB=stack(gB))


if __name__ == "__main__":
    main()
