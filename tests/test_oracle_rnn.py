"""Pins the CPU oracle of the Delta RNN v2 op (oracle.rnn_fwd / rnn_bwd).

Reference ground truth: the PyTorch loop of
algorithmic/fast_weight_rnn_v2/__init__.py:205-217 (exact softmax of the previous
output, no epsilon in the denominator).  No golden vectors exist upstream.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_loop
from helpers import fd_grad, max_abs, rng, rnn_inputs, softmax


def test_no_writes_passes_z_through():
    z, k, v, W0, beta, h0, _ = rnn_inputs(1, 2, 2, 7, 5)
    out, W, h = oracle.rnn_fwd(z, k, v, W0, 0 * beta, h0)
    assert max_abs(out, z) == 0.0 and max_abs(W, 0 * W) == 0.0
    assert max_abs(h[:, :, 0], z[:, :, -1]) == 0.0


def test_width_one_is_a_scalar_recurrence():
    g = rng(2)
    L = 9
    z, k, v = g.standard_normal((3, L))
    beta = 1 / (1 + np.exp(-g.standard_normal(L)))
    w, ref = 0.3, []
    for t in range(L):
        w = w + k[t] * beta[t] * (v[t] - w * k[t])
        ref.append(w * 1.0 + z[t])          # softmax of a single number is 1
    sh = (1, 1, L, 1)
    out, W, h = oracle.rnn_fwd(z.reshape(sh), k.reshape(sh), v.reshape(sh), np.full((1, 1, 1, 1), 0.3),
                               beta.reshape(sh), np.full((1, 1, 1, 1), -1.7))
    assert max_abs(out.reshape(-1), np.array(ref)) < 1e-14 and abs(W.item() - w) < 1e-14


def test_is_the_delta_rule_queried_with_softmax_of_its_own_output():
    z, k, v, W0, beta, h0, _ = rnn_inputs(3, 2, 3, 10, 6, w0=True)
    out, W, h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    s = softmax(np.concatenate([h0, out[:, :, :-1]], axis=2))
    d_out, d_W = oracle.delta_fwd(s, k, v, beta, W0)
    assert max_abs(out, d_out + z) < 1e-13 and max_abs(W, d_W) == 0.0
    assert max_abs(h, out[:, :, -1:]) == 0.0


def test_segment_split_with_carried_state():
    z, k, v, W0, beta, h0, _ = rnn_inputs(4, 2, 2, 11, 4, w0=True)
    out, W, h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    a, b = slice(0, 4), slice(4, 11)
    o1, W1, h1 = oracle.rnn_fwd(z[:, :, a], k[:, :, a], v[:, :, a], W0, beta[:, :, a], h0)
    o2, W2, h2 = oracle.rnn_fwd(z[:, :, b], k[:, :, b], v[:, :, b], W1, beta[:, :, b], h1)
    assert max_abs(np.concatenate([o1, o2], 2), out) == 0.0
    assert max_abs(W2, W) == 0.0 and max_abs(h2, h) == 0.0


def test_backward_against_finite_differences():
    z, k, v, W0, beta, h0, go = rnn_inputs(5, 2, 2, 6, 5, w0=True)
    an = oracle.rnn_bwd(z, k, v, W0, beta, h0, go)

    def loss():
        return float((oracle.rnn_fwd(z, k, v, W0, beta, h0)[0] * go).sum())

    g = rng(0)
    for x, gx in zip((z, k, v, beta), an):
        for idx in g.choice(x.size, size=12, replace=False):
            num = fd_grad(loss, x, int(idx))
            assert abs(num - gx.reshape(-1)[idx]) < 1e-7 * (1 + abs(num))


@pytest.mark.parametrize("shape", [(2, 3, 13, 8), (3, 5, 11, 64)])
def test_backward_against_autograd_of_the_torch_loop(shape):
    z, k, v, W0, beta, h0, go = rnn_inputs(6, *shape, w0=True)
    tin = [torch.from_numpy(x) for x in (z, k, v, W0, beta, h0)]
    out_t, g_t = torch_loop.grads(torch_loop.rnn_v2_loop, tin, [0, 1, 2, 4], torch.from_numpy(go))
    out, W, h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    _, W_t, h_t = torch_loop.rnn_v2_loop(*tin)
    assert max_abs(out, out_t.numpy()) < 1e-12
    assert max_abs(W, W_t.numpy()) < 1e-12 and max_abs(h, h_t.numpy()) < 1e-12
    for a, b in zip(oracle.rnn_bwd(z, k, v, W0, beta, h0, go), g_t):
        assert max_abs(a, b.numpy()) < 1e-11


def test_float32_tracks_float64_over_256_steps():
    z, k, v, W0, beta, h0, go = rnn_inputs(7, 2, 2, 256, 32)
    ref = oracle.rnn_fwd(z, k, v, W0, beta, h0)[0]
    f32 = [x.astype(np.float32) for x in (z, k, v, W0, beta, h0, go)]
    assert np.all(np.abs(oracle.rnn_fwd(*f32[:6])[0] - ref) <= 1e-4 + 1e-3 * np.abs(ref))
    for a, b in zip(oracle.rnn_bwd(*f32), oracle.rnn_bwd(z, k, v, W0, beta, h0, go)):
        assert np.all(np.abs(a - b) <= 1e-4 + 1e-3 * np.abs(b))
