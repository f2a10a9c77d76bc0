"""GPU parity of the sum update rule (fast_weight_sum, through the C ABI) against the
float64 CPU oracle.  Tolerance: |hip - oracle| <= 1e-4 + 1e-3 * |oracle| elementwise."""
import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, rng, within

pytestmark = pytest.mark.gpu
ATOL, RTOL = 1e-4, 1e-3


def dev(x, grad=False):
    t = torch.from_numpy(np.asarray(x, np.float32)).to("cuda")
    return t.requires_grad_(True) if grad else t


def check(name, got, want):
    got = got.detach().cpu().numpy()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert np.all(np.isfinite(got)), name
    assert within(got, want, ATOL, RTOL), f"{name}: max abs err {max_abs(got, want):.3e}"


def inputs(seed, N, H, L, E, M, w0):
    g = rng(seed)
    q, k = g.random((N, H, L, E)), g.random((N, H, L, E))
    q, k = q / q.sum(-1, keepdims=True), k / k.sum(-1, keepdims=True)
    v = g.standard_normal((N, H, L, M))
    W0 = g.standard_normal((N, H, E, M)) * 0.5 if w0 else np.zeros((N, H, E, M))
    return q, k, v, W0, g.standard_normal((N, H, L, M))


SHAPES = [
    (3, 5, 7, 11, 4, False),      # the reference's self test
    (2, 2, 47, 16, 16, True),     # around the 16-step block boundaries of the blocked kernels
    (1, 2, 33, 32, 32, True),
    (2, 2, 64, 16, 16, False),
    (2, 3, 130, 16, 16, True),    # ragged tail chunk, carried-in state
    (2, 2, 256, 32, 32, True),
    (1, 2, 1, 32, 32, True),
    (2, 2, 40, 32, 128, True),    # fast-net layers: d_head x fast_ff_d_head and back
    (2, 2, 40, 128, 32, False),
    (1, 2, 70, 16, 128, True),
    (2, 1, 33, 128, 16, True),
    (1, 2, 200, 32, 128, True),   # longer than one chunk of the state checkpoints
    (1, 1, 150, 128, 32, True),
    (1, 1, 20, 5, 3, True),
    # rectangular and larger states on the matrix cores (feature maps that widen the keys; d_head 64)
    (2, 2, 40, 96, 16, True),
    (1, 2, 48, 64, 64, True),
    (2, 1, 37, 16, 64, False),
    (1, 2, 64, 64, 32, True),
    (1, 1, 33, 32, 64, True),
    (1, 2, 20, 96, 32, False),
    (1, 2, 50, 64, 16, True),
    (1, 1, 17, 16, 32, True),
    (1, 1, 31, 32, 16, False),
    # keys of 192 features whole; by slices of value columns and with zero padded keys
    (2, 2, 40, 192, 16, True),
    (1, 2, 50, 192, 32, True),   # 192 x 32, 64 x 128, 128 x 64: whole, on several waves whatever the setting
    (2, 1, 40, 64, 128, True),
    (1, 2, 70, 128, 64, False),
    (1, 1, 40, 128, 128, True),  # two slices of 128 x 64
    (2, 1, 33, 96, 64, True),    # two slices of 96 x 32
    (1, 2, 33, 48, 24, True),
    (1, 1, 70, 160, 40, False),
    (2, 2, 1, 64, 128, True),
]


@pytest.mark.parametrize("mode", ["reference", "exact"])
@pytest.mark.parametrize("N,H,L,E,M,w0", SHAPES)
def test_sum(fwp, delta_kernels, N, H, L, E, M, w0, mode):
    q, k, v, W0, go = inputs(200 + L + E, N, H, L, E, M, w0)
    tq, tk, tv = (dev(x, True) for x in (q, k, v))
    W = dev(W0)
    fwp.FastWeightSum.state_gradient = mode
    try:
        out = fwp.fast_weight_sum(tq, tk, tv, W)
        ref_out, ref_W = oracle.sum_fwd(q, k, v, W0)
        check("out", out, ref_out)
        check("W", W, ref_W)
        out.backward(dev(go))
    finally:
        fwp.FastWeightSum.state_gradient = "reference"
    refs = oracle.sum_bwd(q, k, v, W0, go, through_state=(mode == "exact"))
    for name, t, r in zip("q k v".split(), (tq, tk, tv), refs):
        check("grad_" + name, t.grad, r)
    check("W after backward", W, ref_W)


def test_sum_strided_views_segments_and_no_grad(fwp, delta_kernels):
    N, H, L, D = 2, 3, 48, 16
    q, k, v, W0, go = inputs(9, N, H, L, D, D, True)
    lnh = lambda x: dev(np.ascontiguousarray(x.transpose(2, 0, 1, 3))).permute(1, 2, 0, 3)
    tq, tk, tv, tgo = lnh(q), lnh(k), lnh(v), lnh(go)
    for t in (tq, tk, tv):
        t.requires_grad_(True)
    W = dev(W0)
    a, b = slice(0, 20), slice(20, L)
    o1 = fwp.fast_weight_sum(tq[:, :, a], tk[:, :, a], tv[:, :, a], W)
    o2 = fwp.fast_weight_sum(tq[:, :, b], tk[:, :, b], tv[:, :, b], W)
    ref_out, ref_W = oracle.sum_fwd(q, k, v, W0)
    check("out", torch.cat([o1, o2], dim=2), ref_out)
    check("W", W, ref_W)
    o1.backward(tgo[:, :, a])
    refs = oracle.sum_bwd(q[:, :, a], k[:, :, a], v[:, :, a], W0, go[:, :, a])
    check("grad_q", tq.grad[:, :, a], refs[0])
    check("grad_k", tk.grad[:, :, a], refs[1])
    check("grad_v", tv.grad[:, :, a], refs[2])
    with torch.no_grad():
        W = dev(W0)
        check("out (no grad)", fwp.fast_weight_sum(dev(q), dev(k), dev(v), W), ref_out)


def test_sum_equals_delta_rule_on_orthonormal_keys(fwp):
    # beta = 1 and mutually orthonormal keys: v_old = 0 at every step, the two rules coincide
    N, H, D = 2, 2, 16
    g = rng(5)
    basis = np.linalg.qr(g.standard_normal((N, H, D, D)))[0]          # rows of basis^T are orthonormal
    k = np.swapaxes(basis, -1, -2)                                     # L = D steps
    q, v = g.standard_normal((N, H, D, D)), g.standard_normal((N, H, D, D))
    W1, W2 = dev(np.zeros((N, H, D, D))), dev(np.zeros((N, H, D, D)))
    a = fwp.fast_weight_sum(dev(q), dev(k), dev(v), W1)
    b = fwp.fast_weight_delta(dev(q), dev(k), dev(v), dev(np.ones((N, H, D, 1))), W2)
    assert torch.allclose(a, b, atol=2e-5, rtol=1e-4)
    assert torch.allclose(W1, W2, atol=2e-5, rtol=1e-4)


def test_sum_by_slices_checks_the_state_it_is_given(fwp):
    """A state shape that runs by slices of value columns makes the checks of the whole-state path on the
    caller's W before anything runs, and leaves W alone when it raises."""
    q, k, v, W0, _ = inputs(9, 1, 2, 20, 128, 128, True)
    tq, tk, tv, W = dev(q), dev(k), dev(v), dev(W0)
    assert fwp.fast_transformers.sum_plan(128, 128) is not None
    with pytest.raises(fwp._lib.FwpError, match="W must be"):
        fwp.fast_weight_sum(tq, tk, tv, W.transpose(2, 3))
    with pytest.raises(fwp._lib.FwpError, match="W must be"):
        fwp.fast_weight_sum(tq, tk, tv, W[:, :, :64])
    with pytest.raises(fwp._lib.FwpError, match="shape mismatch"):
        fwp.fast_weight_sum(tq, tk[:, :, :-1], tv, W)
    assert torch.equal(W, dev(W0))
