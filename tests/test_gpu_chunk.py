"""GPU parity of the delta rule through the C ABI with checkpoint distances other than the
default: every kernel kind has to place and find its checkpoints (and the forward kind and the
backward kind may differ, since a caller may change the setting between the two calls)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import delta_inputs, within, max_abs

pytestmark = pytest.mark.gpu
ATOL, RTOL = 1e-4, 1e-3
KINDS = ("scan", "chunked", "split", "phase")


def run(fwp, arrays, chunk, fwd_kind, bwd_kind):
    L_ = fwp._lib
    lib = L_.lib()
    code = {"scan": L_.DELTA_SCAN, "chunked": L_.DELTA_CHUNKED, "split": L_.DELTA_SPLIT, "phase": L_.DELTA_PHASE}
    q, k, v, beta, W0, go = (torch.from_numpy(a).cuda() for a in arrays)
    N, H, T, E = q.shape
    M = v.shape[-1]
    view = lambda t: L_.View(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))
    W = W0.clone()
    out, vdiff = torch.empty_like(v), torch.empty_like(v)
    # what a caching allocator may hand back after a blocked forward of the same shape: a header that
    # says "per-block matrices follow" and stale matrices; every forward kind has to set it right
    ckpt = torch.ones(L_.delta_ckpt_floats(N, H, T, E, M, chunk), device="cuda", dtype=torch.float32)
    gq, gk, gv, gb = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(beta)
    stream = L_.stream_of(q)
    try:
        L_.config(L_.CFG_DELTA_KERNELS, code[fwd_kind])
        L_.check(lib.fwp_delta_fwd(view(q), view(k), view(v), view(beta), L_.ptr(W), L_.ptr(out), L_.ptr(vdiff),
                                   L_.ptr(ckpt), N, H, T, E, M, chunk, stream), "fwd")
        L_.config(L_.CFG_DELTA_KERNELS, code[bwd_kind])
        L_.check(lib.fwp_delta_bwd(view(q), view(k), view(beta), L_.ptr(vdiff), view(go), L_.ptr(ckpt), L_.ptr(gq),
                                   L_.ptr(gk), L_.ptr(gv), L_.ptr(gb), N, H, T, E, M, chunk, stream), "bwd")
    finally:
        L_.config(L_.CFG_DELTA_KERNELS, L_.DELTA_AUTO)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (out, W, gq, gk, gv, gb)]


@pytest.mark.parametrize("chunk", [32, 96, 128])
@pytest.mark.parametrize("D", [16, 32])
@pytest.mark.parametrize("kind", KINDS)
def test_checkpoint_distance(fwp, kind, D, chunk):
    N, H, T = 2, 3, 160       # ten blocks of 16: the last chunk is a partial one for every distance here
    arrays = delta_inputs(11, N, H, T, D, D, dtype=np.float32, w0=True)
    q, k, v, beta, W0, go = (a.astype(np.float64) for a in arrays)
    want = [*oracle.delta_fwd(q, k, v, beta, W0), *oracle.delta_bwd(q, k, v, beta, W0, go)]
    got = run(fwp, arrays, chunk, kind, kind)
    for name, g, w in zip(("out", "W", "gq", "gk", "gv", "gbeta"), got, want):
        assert within(g, w, ATOL, RTOL), f"{name}: max abs err {max_abs(g, w):.3e}"


@pytest.mark.parametrize("fwd_kind,bwd_kind", [(a, b) for a in KINDS for b in KINDS if a != b])
def test_forward_and_backward_of_different_kinds(fwp, fwd_kind, bwd_kind):
    N, H, T, D = 2, 2, 96, 16
    arrays = delta_inputs(12, N, H, T, D, D, dtype=np.float32, w0=True)
    q, k, v, beta, W0, go = (a.astype(np.float64) for a in arrays)
    want = [*oracle.delta_fwd(q, k, v, beta, W0), *oracle.delta_bwd(q, k, v, beta, W0, go)]
    got = run(fwp, arrays, 64, fwd_kind, bwd_kind)
    for name, g, w in zip(("out", "W", "gq", "gk", "gv", "gbeta"), got, want):
        assert within(g, w, ATOL, RTOL), f"{fwd_kind}->{bwd_kind} {name}: max abs err {max_abs(g, w):.3e}"


@pytest.mark.parametrize("D", [16, 32])
def test_long_sequence_kinds_agree(fwp, D):
    """2048 steps (128 blocks, 32 chunks): the three kernel kinds against the oracle and each other."""
    N, H, T = 1, 3, 2048
    arrays = delta_inputs(13, N, H, T, D, D, dtype=np.float32, w0=True)
    q, k, v, beta, W0, go = (a.astype(np.float64) for a in arrays)
    want = [*oracle.delta_fwd(q, k, v, beta, W0), *oracle.delta_bwd(q, k, v, beta, W0, go)]
    for kind in KINDS:
        got = run(fwp, arrays, 64, kind, kind)
        for name, g, w in zip(("out", "W", "gq", "gk", "gv", "gbeta"), got, want):
            assert within(g, w, ATOL, RTOL), f"{kind} {name}: max abs err {max_abs(g, w):.3e}"
