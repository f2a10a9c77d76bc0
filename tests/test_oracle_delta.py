"""Pins the CPU oracle of the delta rule (oracle.delta_fwd / delta_bwd).

The reference holds no golden vectors for this op (its only test compares the
kernel with a PyTorch loop, algorithmic/fast_weight/__init__.py:99-253), so the
oracle is pinned by what the mathematics fixes: closed forms, an explicit
matrix-product brute force, invariances, finite differences and autograd.
None of these re-types the oracle's own recurrence.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_loop
from helpers import delta_inputs, fd_grad, max_abs, rng


def test_single_step_closed_form():
    # T=1, W0=0: out = beta * v * (k.q)
    q, k, v, beta, W0, _ = delta_inputs(1, 2, 3, 1, 5, 7)
    out, W = oracle.delta_fwd(q, k, v, beta, W0)
    kq = (q * k).sum(-1, keepdims=True)
    assert max_abs(out, beta * v * kq) < 1e-14
    assert max_abs(W, k[:, :, 0, :, None] * (beta * v)[:, :, 0, None, :]) < 1e-14


def test_beta_zero_reads_initial_state():
    q, k, v, beta, W0, go = delta_inputs(2, 2, 2, 6, 4, 3, w0=True)
    beta = np.zeros_like(beta)
    out, W = oracle.delta_fwd(q, k, v, beta, W0)
    assert max_abs(out, np.einsum("nhem,nhle->nhlm", W0, q)) < 1e-14
    assert max_abs(W, W0) == 0.0
    gq, gk, gv, gb, gW0 = oracle.delta_bwd(q, k, v, beta, W0, go)
    assert max_abs(gv, 0 * gv) == 0.0
    assert max_abs(gq, np.einsum("nhem,nhlm->nhle", W0, go)) < 1e-14
    assert max_abs(gW0, np.einsum("nhle,nhlm->nhem", q, go)) < 1e-13


def test_one_hot_keys_are_a_key_value_store():
    # beta=1, one-hot keys: the memory returns exactly the last value written under a key.
    N, H, E, M = 1, 2, 4, 3
    slots = [0, 2, 1, 2, 0, 3]
    L = len(slots)
    g = rng(3)
    k = np.zeros((N, H, L, E))
    for t, s in enumerate(slots):
        k[:, :, t, s] = 1.0
    v = g.standard_normal((N, H, L, M))
    beta = np.ones((N, H, L, 1))
    W0 = np.zeros((N, H, E, M))
    out, W = oracle.delta_fwd(k.copy(), k, v, beta, W0)   # query = the key just written
    assert max_abs(out, v) < 1e-15
    last = {s: t for t, s in enumerate(slots)}
    for s, t in last.items():
        assert max_abs(W[:, :, s, :], v[:, :, t, :]) < 1e-15


def test_orthonormal_keys_equal_causal_linear_attention():
    # beta=1, W0=0, mutually orthonormal keys: v_old=0 at every step, so the delta rule
    # equals the sum rule out_t = sum_{j<=t} v_j (k_j . q_t), computed here as a masked matmul.
    N, H, L, E, M = 2, 2, 6, 8, 5
    g = rng(4)
    k = np.stack([np.linalg.qr(g.standard_normal((E, E)))[0][:L] for _ in range(N * H)])
    k = k.reshape(N, H, L, E)
    q = g.standard_normal((N, H, L, E))
    v = g.standard_normal((N, H, L, M))
    out, _ = oracle.delta_fwd(q, k, v, np.ones((N, H, L, 1)), np.zeros((N, H, E, M)))
    att = np.tril(np.einsum("nhte,nhje->nhtj", q, k))
    assert max_abs(out, att @ v) < 1e-13


def test_brute_force_matrix_product():
    # W_t^T (as M x E) = W_{t-1}^T (I - b k k^T) + b v k^T, expanded as an explicit product.
    q, k, v, beta, W0, _ = delta_inputs(5, 1, 2, 7, 4, 3, w0=True)
    out, W = oracle.delta_fwd(q, k, v, beta, W0)
    for h in range(2):
        A = W0[0, h].T.copy()                       # [M,E]
        P = [np.eye(4) - beta[0, h, t, 0] * np.outer(k[0, h, t], k[0, h, t]) for t in range(7)]
        for t in range(7):
            acc = W0[0, h].T.copy()
            for i in range(t + 1):
                acc = acc @ P[i]
            for j in range(t + 1):
                term = beta[0, h, j, 0] * np.outer(v[0, h, j], k[0, h, j])
                for i in range(j + 1, t + 1):
                    term = term @ P[i]
                acc = acc + term
            assert max_abs(out[0, h, t], acc @ q[0, h, t]) < 1e-13
            A = acc
        assert max_abs(W[0, h], A.T) < 1e-13


def test_read_back_identity():
    # after writing at step t:  W_t^T k_t = v_old + beta (v - v_old) |k|^2
    q, k, v, beta, W0, _ = delta_inputs(6, 1, 1, 5, 6, 4, w0=True)
    W = W0
    for t in range(5):
        sl = slice(t, t + 1)
        v_old = np.einsum("nhem,nhe->nhm", W, k[:, :, t])
        out, W = oracle.delta_fwd(k[:, :, sl], k[:, :, sl], v[:, :, sl], beta[:, :, sl], W)
        k2 = (k[:, :, t] ** 2).sum(-1, keepdims=True)
        assert max_abs(out[:, :, 0], v_old + beta[:, :, t] * (v[:, :, t] - v_old) * k2) < 1e-14


def test_linear_in_values_and_state():
    q, k, v1, beta, W1, _ = delta_inputs(7, 2, 2, 9, 5, 6, w0=True)
    _, _, v2, _, W2, _ = delta_inputs(8, 2, 2, 9, 5, 6, w0=True)
    o1, Wa = oracle.delta_fwd(q, k, v1, beta, W1)
    o2, Wb = oracle.delta_fwd(q, k, v2, beta, W2)
    o3, Wc = oracle.delta_fwd(q, k, 2 * v1 - 3 * v2, beta, 2 * W1 - 3 * W2)
    assert max_abs(o3, 2 * o1 - 3 * o2) < 1e-12
    assert max_abs(Wc, 2 * Wa - 3 * Wb) < 1e-12


def test_segment_split_and_permutation():
    q, k, v, beta, W0, _ = delta_inputs(9, 3, 2, 12, 4, 6, w0=True)
    out, W = oracle.delta_fwd(q, k, v, beta, W0)
    a = slice(0, 5)
    b = slice(5, 12)
    o1, W1 = oracle.delta_fwd(q[:, :, a], k[:, :, a], v[:, :, a], beta[:, :, a], W0)
    o2, W2 = oracle.delta_fwd(q[:, :, b], k[:, :, b], v[:, :, b], beta[:, :, b], W1)
    assert max_abs(np.concatenate([o1, o2], 2), out) == 0.0 and max_abs(W2, W) == 0.0
    perm = [2, 0, 1]
    op, Wp = oracle.delta_fwd(q[perm], k[perm], v[perm], beta[perm], W0[perm])
    assert max_abs(op, out[perm]) == 0.0 and max_abs(Wp, W[perm]) == 0.0


@pytest.mark.parametrize("E,M", [(4, 4), (3, 6), (7, 2)])
def test_backward_against_finite_differences(E, M):
    q, k, v, beta, W0, go = delta_inputs(10 + E, 2, 2, 6, E, M, w0=True)
    an = oracle.delta_bwd(q, k, v, beta, W0, go)

    def loss():
        return float((oracle.delta_fwd(q, k, v, beta, W0)[0] * go).sum())

    g = rng(0)
    for x, gx in zip((q, k, v, beta, W0), an):
        for idx in g.choice(x.size, size=min(12, x.size), replace=False):
            num = fd_grad(loss, x, int(idx))
            assert abs(num - gx.reshape(-1)[idx]) < 1e-7 * (1 + abs(num))


@pytest.mark.parametrize("shape", [(2, 3, 17, 8, 8), (1, 2, 9, 5, 11)])
def test_backward_against_autograd_of_the_torch_loop(shape):
    N, H, L, E, M = shape
    q, k, v, beta, W0, go = delta_inputs(20, N, H, L, E, M, w0=True)
    tin = [torch.from_numpy(x) for x in (q, k, v, beta, W0)]
    out_t, g_t = torch_loop.grads(torch_loop.delta_loop, tin, [0, 1, 2, 3, 4], torch.from_numpy(go))
    out, W = oracle.delta_fwd(q, k, v, beta, W0)
    assert max_abs(out, out_t.numpy()) < 1e-12
    assert max_abs(W, torch_loop.delta_loop(*tin)[1].numpy()) < 1e-12
    for a, b in zip(oracle.delta_bwd(q, k, v, beta, W0, go), g_t):
        assert max_abs(a, b.numpy()) < 1e-11


def test_float32_tracks_float64_over_256_steps():
    # the fp32 oracle at the benchmark's sequence length stays inside the parity budget
    q, k, v, beta, W0, go = delta_inputs(30, 2, 2, 256, 16, 16)
    ref = oracle.delta_fwd(q, k, v, beta, W0)[0]
    f32 = [x.astype(np.float32) for x in (q, k, v, beta, W0, go)]
    out32 = oracle.delta_fwd(*f32[:5])[0]
    assert out32.dtype == np.float32
    assert max_abs(out32, ref) < 1e-4
    g64 = oracle.delta_bwd(q, k, v, beta, W0, go)
    g32 = oracle.delta_bwd(*f32)
    for a, b in zip(g32[:4], g64[:4]):
        assert np.all(np.abs(a - b) <= 1e-4 + 1e-3 * np.abs(b))


def test_random_positive_inputs_like_the_reference_self_test():
    # shapes and input recipe of algorithmic/fast_weight/__init__.py:117-127 (uniform, sum-normalised)
    g = rng(111)
    N, H, L, D = 3, 5, 11, 64
    q = g.random((N, H, L, D)); k = g.random((N, H, L, D)); v = g.random((N, H, L, D))
    q /= q.sum(-1, keepdims=True); k /= k.sum(-1, keepdims=True)
    beta = 1 / (1 + np.exp(-g.random((N, H, L, 1))))
    W0 = np.zeros((N, H, D, D))
    tin = [torch.from_numpy(x) for x in (q, k, v, beta, W0)]
    out_t, g_t = torch_loop.grads(torch_loop.delta_loop, tin, [0, 1, 2, 3], torch.ones(N, H, L, D, dtype=torch.float64))
    assert max_abs(oracle.delta_fwd(q, k, v, beta, W0)[0], out_t.numpy()) < 1e-12
    for a, b in zip(oracle.delta_bwd(q, k, v, beta, W0, np.ones((N, H, L, D))), g_t):
        assert max_abs(a, b.numpy()) < 1e-10
