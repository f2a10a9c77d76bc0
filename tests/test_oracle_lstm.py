"""Pins the CPU oracle of the Delta LSTM v4 (oracle.lstm_fwd / lstm_bwd).

The reference's only check is kernel-vs-loop on random inputs (fast_lstm_v4/__init__.py:
218-560).  The oracle is pinned by special cases that reduce to already pinned operators
or to closed forms, by autograd through the restated loop and by finite differences."""
import numpy as np
import torch

import oracle
from oracle import torch_loop
from helpers import fd_grad, lstm_inputs, max_abs, sigmoid, softmax


def test_single_step_closed_form():
    Zs, Ks, Vs, Bs, Ws, h0, c0, _ = lstm_inputs(0, 2, 3, 1, 5, w0=True)
    out, cell, Wn, h, c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    s = softmax(h0[:, :, 0])
    pre = []
    for g in range(3):
        k, v, b = Ks[g][:, :, 0], Vs[g][:, :, 0], Bs[g][:, :, 0]
        v_old = np.einsum("nhem,nhe->nhm", Ws[g], k)
        W1 = Ws[g] + k[..., None] * (b * (v - v_old))[..., None, :]
        assert max_abs(Wn[g], W1) < 1e-14
        pre.append(np.einsum("nhem,nhe->nhm", W1, s) + Zs[g][:, :, 0])
    i, u, o = sigmoid(pre[0]), pre[1], sigmoid(pre[2])
    c1 = i * u + (1 - i) * c0[:, :, 0]
    assert max_abs(cell[:, :, 0], c1) < 1e-14
    assert max_abs(out[:, :, 0], o * c1) < 1e-14
    assert max_abs(h[:, :, 0], o * c1) < 1e-14 and max_abs(c[:, :, 0], c1) < 1e-14


def test_open_gates_reduce_to_the_delta_rnn():
    # z_i, z_o -> +40: i = o = 1 in double precision, so c = u, h = u = W_u^T softmax(h) + z_u
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(1, 2, 2, 9, 6, w0=True)
    Zs[0] = np.full_like(Zs[0], 40.0)
    Zs[2] = np.full_like(Zs[2], 40.0)
    out, cell, Wn, h, c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    rnn_out, rnn_W, rnn_h = oracle.rnn_fwd(Zs[1], Ks[1], Vs[1], Ws[1], Bs[1], h0)
    assert max_abs(out, rnn_out) < 1e-12 and max_abs(cell, rnn_out) < 1e-12
    assert max_abs(Wn[1], rnn_W) < 1e-13 and max_abs(h, rnn_h) < 1e-12
    gZ, gK, gV, gB = oracle.lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go)
    rz, rk, rv, rb = oracle.rnn_bwd(Zs[1], Ks[1], Vs[1], Ws[1], Bs[1], h0, go)
    for got, want in ((gZ[1], rz), (gK[1], rk), (gV[1], rv), (gB[1], rb)):
        assert max_abs(got, want) < 1e-11


def test_closed_input_gate_keeps_the_cell():
    # z_i -> -40: the cell never changes; h_t = o_t c_0
    Zs, Ks, Vs, Bs, Ws, h0, c0, _ = lstm_inputs(2, 1, 2, 7, 4, w0=True)
    Zs[0] = np.full_like(Zs[0], -40.0)
    out, cell, *_ = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    assert max_abs(cell, np.broadcast_to(c0, cell.shape)) < 1e-12
    assert np.all(np.abs(out) <= np.abs(np.broadcast_to(c0, out.shape)) + 1e-12)


def test_memories_of_the_three_gates_are_independent_delta_rules():
    Zs, Ks, Vs, Bs, Ws, h0, c0, _ = lstm_inputs(3, 2, 2, 12, 5, w0=True)
    *_, Wn, _, _ = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    for g in range(3):
        _, W = oracle.delta_fwd(Ks[g], Ks[g], Vs[g], Bs[g], Ws[g])
        assert max_abs(Wn[g], W) < 1e-13


def _torch_args(Zs, Ks, Vs, Bs, Ws, h0, c0, grad=True):
    ts = []
    for g in range(3):
        for x in (Zs[g], Ks[g], Vs[g], Bs[g]):
            ts.append(torch.from_numpy(x).requires_grad_(grad))
        ts.append(torch.from_numpy(Ws[g]))
    return ts + [torch.from_numpy(h0), torch.from_numpy(c0)]


def test_autograd_of_the_step_loop():
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(4, 2, 3, 11, 6, w0=True)
    args = _torch_args(Zs, Ks, Vs, Bs, Ws, h0, c0)
    out, cell, Wn, h, c = torch_loop.lstm_v4_loop(*args)
    o_out, o_cell, o_W, o_h, o_c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    assert max_abs(out.detach().numpy(), o_out) < 1e-12
    assert max_abs(cell.detach().numpy(), o_cell) < 1e-12
    assert max_abs(h.detach().numpy(), o_h) < 1e-12 and max_abs(c.detach().numpy(), o_c) < 1e-12
    for g in range(3):
        assert max_abs(Wn[g].detach().numpy(), o_W[g]) < 1e-12
    out.backward(torch.from_numpy(go))
    gZ, gK, gV, gB = oracle.lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go)
    for g in range(3):
        z, k, v, b = args[5 * g:5 * g + 4]
        for got, want in ((gZ[g], z), (gK[g], k), (gV[g], v), (gB[g], b)):
            assert max_abs(got, want.grad.numpy()) < 1e-11


def test_finite_differences():
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(5, 1, 2, 6, 4, w0=True)
    gZ, gK, gV, gB = oracle.lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go)
    loss = lambda: float((oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)[0] * go).sum())
    for pack, grads, name in ((Zs, gZ, "z"), (Ks, gK, "k"), (Vs, gV, "v"), (Bs, gB, "beta")):
        for g in range(3):
            x = pack[g]
            for idx in (0, x.size // 2 + 1, x.size - 1):
                num = fd_grad(loss, x, idx)
                assert abs(num - grads[g].reshape(-1)[idx]) < 2e-7, (name, g, idx)
