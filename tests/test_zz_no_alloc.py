"""The entry point that allocates nothing (fwp_rec_bwd_static) against fwp_rec_bwd, through the C ABI:
the same bits, on two calls in a row, the second one smaller (so that what the first left in the
library's scratch array would show if it were read), and its size limit.  fwp_rec_bwd itself is held
to the float64 oracle in test_gpu_parity.py and test_gpu_baseline_sizes.py; here the static entry
point's gradients are compared with the oracle's directly as well
(|hip - oracle| <= 1e-4 + 1e-3 |oracle| elementwise)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, rec_inputs, within

pytestmark = pytest.mark.gpu


def forward(L_, lib, arrays, chunk):
    qx, kx, vx, bx, Rq, Rk, Rv, rb, W0, h0, go = (torch.from_numpy(a).cuda() for a in arrays)
    N, H, T, D = qx.shape
    view = lambda t: L_.View(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))
    W, h = W0.clone(), h0.clone()
    f32 = dict(device="cuda", dtype=torch.float32)
    out, q_act, k_act, vdiff = (torch.empty((N, H, T, D), **f32) for _ in range(4))
    beta_act = torch.empty((N, H, T), **f32)
    ckpt = torch.empty((N, H, (T + chunk - 1) // chunk, D, D), **f32)
    stream = L_.stream_of(qx)
    L_.check(lib.fwp_rec_fwd(view(qx), view(kx), view(vx), view(bx), L_.ptr(Rq), L_.ptr(Rk), L_.ptr(Rv),
                             L_.ptr(rb), L_.ptr(W), L_.ptr(h), L_.ptr(out), L_.ptr(q_act), L_.ptr(k_act),
                             L_.ptr(beta_act), L_.ptr(vdiff), L_.ptr(ckpt), N, H, T, D, chunk, stream), "fwd")
    return dict(N=N, H=H, T=T, D=D, view=view, go=go, h0=h0, Rq=Rq, Rk=Rk, Rv=Rv, rb=rb, out=out, q_act=q_act,
                k_act=k_act, beta_act=beta_act, vdiff=vdiff, ckpt=ckpt, stream=stream)


def backward(L_, lib, s, chunk, static):
    N, H, T, D = s["N"], s["H"], s["T"], s["D"]
    f32 = dict(device="cuda", dtype=torch.float32)
    # NaN-filled: every element has to be written by the call
    grads = [torch.full((N, H, T, D), float("nan"), **f32) for _ in range(3)] + \
            [torch.full((N, H, T, 1), float("nan"), **f32)] + \
            [torch.full((1, H, D, D), float("nan"), **f32) for _ in range(3)] + \
            [torch.full((1, H, 1, D), float("nan"), **f32)]
    head = [L_.ptr(s[n]) for n in ("q_act", "k_act", "beta_act", "vdiff", "out", "h0")] + [s["view"](s["go"])] + \
           [L_.ptr(s[n]) for n in ("Rq", "Rk", "Rv", "rb", "ckpt")] + [L_.ptr(g) for g in grads]
    tail = [N, H, T, D, chunk, s["stream"]]
    if static:
        rc = lib.fwp_rec_bwd_static(*head, *tail)
    else:
        ws = torch.empty((N, H, 3 * D * D + D), **f32)
        rc = lib.fwp_rec_bwd(*head, L_.ptr(ws), *tail)
    L_.check(rc, "bwd")
    torch.cuda.synchronize()
    return [g.cpu().numpy() for g in grads]


def test_static_scratch_entry_point_matches_the_allocating_one(fwp):
    L_ = fwp._lib
    lib = L_.lib()
    chunk = L_.query(L_.Q_DEFAULT_CHUNK)
    names = ("gqx", "gkx", "gvx", "gbx", "gRq", "gRk", "gRv", "grb")
    # two calls in a row on one stream, the second smaller in every dimension that sizes the scratch
    for seed, (N, H, T, D) in ((31, (5, 4, 80, 32)), (32, (2, 3, 40, 16))):
        print(f"fwp_rec_bwd_static seed={seed} N={N} H={H} T={T} D={D}", flush=True)
        arrays = rec_inputs(seed, N, H, T, D, dtype=np.float32, w0=True)
        saved = forward(L_, lib, arrays, chunk)
        want = backward(L_, lib, saved, chunk, static=False)
        got = backward(L_, lib, saved, chunk, static=True)
        for name, g, w in zip(names, got, want):
            assert np.isfinite(w).all(), name
            assert np.array_equal(g, w), f"{name} differs between fwp_rec_bwd_static and fwp_rec_bwd"
        exact = oracle.rec_bwd(*(np.asarray(a, np.float64) for a in arrays))
        for name, g, w in zip(names, got, exact):
            assert g.shape == w.shape, (name, g.shape, w.shape)
            assert within(g, w, 1e-4, 1e-3), f"{name} of fwp_rec_bwd_static: max abs err {max_abs(g, w):.3e} against the oracle"


def test_static_scratch_limit_is_enforced_before_any_launch(fwp):
    L_ = fwp._lib
    lib = L_.lib()
    limit = L_.query(L_.Q_STATIC_SCRATCH_FLOATS)
    assert limit == 2 << 20
    D, H = 32, 8
    per = 3 * D * D + D
    N = limit // (H * per) + 1                   # one batch entry too many
    p = ctypes.c_void_p(4096)
    v = L_.View(4096, H * 64 * D, 64 * D, D)
    args = [p] * 6 + [v] + [p] * 13
    rc = lib.fwp_rec_bwd_static(*args, N, H, 64, D, 64, None)
    assert rc == -6 and "scratch" in L_.strerror(rc)
    torch.cuda.synchronize()
