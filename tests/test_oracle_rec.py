"""Pins the CPU oracle of the Recurrent Delta Net op (oracle.rec_fwd / rec_bwd).

Reference ground truth: the PyTorch loop of
algorithmic/rec_update_fwm_tanh/__init__.py:263-302 (tanh of the previous output
feeds q, k, v and beta through R_q, R_k, R_v, r_b; softmax on q and k, sigmoid on
beta, all inside the op).  No golden vectors exist upstream.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_loop
from helpers import fd_grad, max_abs, rec_inputs, rng, sigmoid, softmax


def _activations(x, out):
    qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0 = x
    y = np.tanh(np.concatenate([h0, out[:, :, :-1]], axis=2))          # [N,H,L,D]
    q = softmax(qx + np.einsum("nhle,hem->nhlm", y, R_q[0]))
    k = softmax(kx + np.einsum("nhle,hem->nhlm", y, R_k[0]))
    v = vx + np.einsum("nhle,hem->nhlm", y, R_v[0])
    b = sigmoid(bx + np.einsum("nhle,he->nhl", y, r_b[0, :, 0])[..., None])
    return y, q, k, v, b


def test_without_feedback_it_is_the_activated_delta_rule():
    *x, go = rec_inputs(1, 2, 3, 9, 6, w0=True, rscale=0.0)
    qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0 = x
    out, W, h = oracle.rec_fwd(*x)
    q, k, b = softmax(qx), softmax(kx), sigmoid(bx)
    d_out, d_W = oracle.delta_fwd(q, k, vx, b, W0)
    assert max_abs(out, d_out) < 1e-14 and max_abs(W, d_W) < 1e-14
    gq, gk, gv, gb, _ = oracle.delta_bwd(q, k, vx, b, W0, go)
    gqx, gkx, gvx, gbx, gRq, gRk, gRv, grb = oracle.rec_bwd(*x, go)
    assert max_abs(gqx, q * (gq - (gq * q).sum(-1, keepdims=True))) < 1e-13
    assert max_abs(gkx, k * (gk - (gk * k).sum(-1, keepdims=True))) < 1e-13
    assert max_abs(gvx, gv) < 1e-13 and max_abs(gbx, gb * b * (1 - b)) < 1e-13
    # with R=0 the R-gradients are still the outer products with tanh of the delayed output
    y = np.tanh(np.concatenate([h0, out[:, :, :-1]], axis=2))
    assert max_abs(gRq[0], np.einsum("nhle,nhlm->hem", y, gqx)) < 1e-12
    assert max_abs(gRk[0], np.einsum("nhle,nhlm->hem", y, gkx)) < 1e-12
    assert max_abs(gRv[0], np.einsum("nhle,nhlm->hem", y, gvx)) < 1e-12
    assert max_abs(grb[0, :, 0], np.einsum("nhle,nhl->he", y, gbx[..., 0])) < 1e-12


def test_is_the_delta_rule_on_activations_of_its_own_output():
    *x, go = rec_inputs(2, 2, 2, 12, 8, w0=True)
    out, W, h = oracle.rec_fwd(*x)
    y, q, k, v, b = _activations(x, out)
    d_out, d_W = oracle.delta_fwd(q, k, v, b, x[8])
    assert max_abs(out, d_out) < 1e-13 and max_abs(W, d_W) < 1e-13
    assert max_abs(h, out[:, :, -1:]) == 0.0


def test_softmax_gradients_sum_to_zero():
    *x, go = rec_inputs(3, 2, 2, 10, 8, w0=True)
    gqx, gkx = oracle.rec_bwd(*x, go)[:2]
    assert np.abs(gqx.sum(-1)).max() < 1e-13 and np.abs(gkx.sum(-1)).max() < 1e-13


def test_segment_split_with_carried_state():
    *x, go = rec_inputs(4, 2, 2, 11, 4, w0=True)
    qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0 = x
    out, W, h = oracle.rec_fwd(*x)
    a, b = slice(0, 6), slice(6, 11)
    o1, W1, h1 = oracle.rec_fwd(qx[:, :, a], kx[:, :, a], vx[:, :, a], bx[:, :, a], R_q, R_k, R_v, r_b, W0, h0)
    o2, W2, h2 = oracle.rec_fwd(qx[:, :, b], kx[:, :, b], vx[:, :, b], bx[:, :, b], R_q, R_k, R_v, r_b, W1, h1)
    assert max_abs(np.concatenate([o1, o2], 2), out) == 0.0
    assert max_abs(W2, W) == 0.0 and max_abs(h2, h) == 0.0


def test_backward_against_finite_differences():
    *x, go = rec_inputs(5, 2, 2, 6, 5, w0=True)
    an = oracle.rec_bwd(*x, go)

    def loss():
        return float((oracle.rec_fwd(*x)[0] * go).sum())

    g = rng(0)
    for xi, gx in zip(x[:8], an):
        for idx in g.choice(xi.size, size=min(10, xi.size), replace=False):
            num = fd_grad(loss, xi, int(idx))
            assert abs(num - gx.reshape(-1)[idx]) < 2e-7 * (1 + abs(num))


@pytest.mark.parametrize("shape,rscale", [((2, 3, 13, 8), None), ((3, 5, 11, 32), 0.5)])
def test_backward_against_autograd_of_the_torch_loop(shape, rscale):
    *x, go = rec_inputs(6, *shape, w0=True, rscale=rscale)
    tin = [torch.from_numpy(a) for a in x]
    out_t, g_t = torch_loop.grads(torch_loop.rec_update_loop, tin, list(range(8)), torch.from_numpy(go))
    out, W, h = oracle.rec_fwd(*x)
    _, W_t, h_t = torch_loop.rec_update_loop(*tin)
    assert max_abs(out, out_t.numpy()) < 1e-12
    assert max_abs(W, W_t.numpy()) < 1e-12 and max_abs(h, h_t.numpy()) < 1e-12
    for a, b in zip(oracle.rec_bwd(*x, go), g_t):
        assert max_abs(a, b.numpy()) < 1e-10


def test_float32_tracks_float64_over_256_steps():
    *x, go = rec_inputs(7, 2, 2, 256, 32)
    ref = oracle.rec_fwd(*x)[0]
    x32 = [a.astype(np.float32) for a in x]
    assert np.all(np.abs(oracle.rec_fwd(*x32)[0] - ref) <= 1e-4 + 1e-3 * np.abs(ref))
    for a, b in zip(oracle.rec_bwd(*x32, go.astype(np.float32)), oracle.rec_bwd(*x, go)):
        assert np.all(np.abs(a - b) <= 1e-4 + 1e-3 * np.abs(b))
