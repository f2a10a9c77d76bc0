"""Pins the CPU oracle of the sum update rule (oracle.sum_fwd / sum_bwd).

The reference's self test compares its kernel with a PyTorch loop on random inputs and
holds no vectors (algorithmic/fast_transformers/__init__.py:87-200).  What fixes the
answer: the sum rule is causal linear attention, out = W0^T q + tril(Q K^T) V, whose
gradients are masked matrix products as well; none of the checks below uses a recurrence.
"""
import numpy as np
import torch

import oracle
from oracle import torch_loop
from helpers import max_abs, rng


def inputs(seed, N, H, L, E, M, w0=True):
    g = rng(seed)
    q, k = g.random((N, H, L, E)), g.random((N, H, L, E))
    q, k = q / q.sum(-1, keepdims=True), k / k.sum(-1, keepdims=True)     # as the reference's test draws them
    v = g.standard_normal((N, H, L, M))
    W0 = g.standard_normal((N, H, E, M)) * 0.5 if w0 else np.zeros((N, H, E, M))
    go = g.standard_normal((N, H, L, M))
    return q, k, v, W0, go


def masked(a):
    """Keep s <= t of a[..., t, s]."""
    return np.tril(a)


def test_forward_is_masked_attention():
    q, k, v, W0, _ = inputs(0, 2, 3, 9, 5, 4)
    out, W = oracle.sum_fwd(q, k, v, W0)
    att = masked(np.einsum("nhte,nhse->nhts", q, k))
    want = np.einsum("nhts,nhsm->nhtm", att, v) + np.einsum("nhem,nhte->nhtm", W0, q)
    assert max_abs(out, want) < 1e-13
    assert max_abs(W, W0 + np.einsum("nhse,nhsm->nhem", k, v)) < 1e-13


def test_backward_is_masked_products():
    q, k, v, W0, go = inputs(1, 2, 2, 8, 6, 3)
    for through in (False, True):
        gq, gk, gv = oracle.sum_bwd(q, k, v, W0, go, through_state=through)
        gatt = masked(np.einsum("nhtm,nhsm->nhts", go, v))                  # d out / d (q_t . k_s)
        want_q = np.einsum("nhts,nhse->nhte", gatt, k)
        if through:
            want_q = want_q + np.einsum("nhem,nhtm->nhte", W0, go)
        att = masked(np.einsum("nhte,nhse->nhts", q, k))
        assert max_abs(gq, want_q) < 1e-13
        assert max_abs(gk, np.einsum("nhts,nhte->nhse", gatt, q)) < 1e-13
        assert max_abs(gv, np.einsum("nhts,nhtm->nhsm", att, go)) < 1e-13


def test_reference_gradient_differs_from_the_exact_one_only_through_the_carried_state():
    q, k, v, W0, go = inputs(2, 1, 2, 7, 4, 4)
    ref = oracle.sum_bwd(q, k, v, W0, go)
    exact = oracle.sum_bwd(q, k, v, W0, go, through_state=True)
    assert max_abs(ref[1], exact[1]) == 0 and max_abs(ref[2], exact[2]) == 0
    assert max_abs(exact[0] - ref[0], np.einsum("nhem,nhtm->nhte", W0, go)) < 1e-13
    zero = np.zeros_like(W0)
    assert max_abs(oracle.sum_bwd(q, k, v, zero, go)[0],
                   oracle.sum_bwd(q, k, v, zero, go, through_state=True)[0]) == 0


def test_autograd_of_the_step_loop_agrees_with_the_exact_gradient():
    q, k, v, W0, go = inputs(3, 2, 2, 10, 5, 7)
    ts = [torch.from_numpy(a).requires_grad_(True) for a in (q, k, v)]
    out, W = torch_loop.sum_loop(*ts, torch.from_numpy(W0))
    want_out, want_W = oracle.sum_fwd(q, k, v, W0)
    assert max_abs(out.detach().numpy(), want_out) < 1e-13
    assert max_abs(W.detach().numpy(), want_W) < 1e-13
    grads = torch.autograd.grad(out, ts, torch.from_numpy(go))
    for got, want in zip(grads, oracle.sum_bwd(q, k, v, W0, go, through_state=True)):
        assert max_abs(got.numpy(), want) < 1e-12


def test_float32_build_and_segment_split():
    q, k, v, W0, go = inputs(4, 2, 2, 33, 16, 16)
    out64, W64 = oracle.sum_fwd(q, k, v, W0)
    f = lambda a: a.astype(np.float32)
    out32, W32 = oracle.sum_fwd(f(q), f(k), f(v), f(W0))
    assert out32.dtype == np.float32 and max_abs(out32, out64) < 1e-5
    a, Wa = oracle.sum_fwd(q[:, :, :12], k[:, :, :12], v[:, :, :12], W0)
    b, Wb = oracle.sum_fwd(q[:, :, 12:], k[:, :, 12:], v[:, :, 12:], Wa)
    assert max_abs(np.concatenate((a, b), 2), out64) < 1e-13 and max_abs(Wb, W64) < 1e-13
