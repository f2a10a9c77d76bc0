"""GPU parity of the Delta LSTM v4 (fast_lstm_v4, through the C ABI) against the float64
CPU oracle.  Tolerance: |hip - oracle| <= 1e-4 + 1e-3 * |oracle| elementwise."""
import numpy as np
import pytest
import torch

import oracle
from helpers import lstm_inputs, max_abs, within

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


def op_args(Zs, Ks, Vs, Bs, Ws, h0, c0, grad=True, wrap=dev):
    args, diff, states = [], [], []
    for a in range(3):
        gate = [wrap(x, grad) for x in (Zs[a], Ks[a], Vs[a], Bs[a])]
        W = wrap(Ws[a])
        args += gate + [W]
        diff.append(gate)
        states.append(W)
    h, c = wrap(h0), wrap(c0)
    return args + [h, c], diff, states, h, c


SHAPES = [
    (3, 5, 11, 18, False),     # the reference's self test
    (2, 2, 64, 16, False),
    (2, 3, 130, 32, True),     # ragged tail chunk, carried-in states
    (1, 2, 1, 32, True),       # single step
    (2, 2, 70, 8, True),
    (1, 1, 19, 5, True),
    (2, 2, 40, 24, True),      # 18, 8, 5 and 24 run padded to 16 or 32
    (1, 2, 20, 40, True),      # wider than any register kernel: the kernels that keep the state in LDS
]


@pytest.mark.parametrize("N,H,L,D,w0", SHAPES)
def test_lstm(fwp, N, H, L, D, w0):
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(300 + L + D, N, H, L, D, w0=w0)
    args, diff, states, h, c = op_args(Zs, Ks, Vs, Bs, Ws, h0, c0)
    out, cell = fwp.fast_lstm_v4(*args)
    r_out, r_cell, r_W, r_h, r_c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    check("out", out, r_out)
    check("cell", cell, r_cell)
    check("h", h, r_h)
    check("c", c, r_c)
    for a in range(3):
        check(f"W[{a}]", states[a], r_W[a])
    assert not cell.requires_grad
    out.backward(dev(go))
    grads = oracle.lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go)
    for a, gate in enumerate("iuo"):
        for j, name in enumerate("z k v beta".split()):
            check(f"grad_{name}_{gate}", diff[a][j].grad, grads[j][a])


def test_lstm_strided_views_segments_and_no_grad(fwp):
    N, H, L, D = 2, 3, 40, 16
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(11, N, H, L, D, w0=True)
    lnh = lambda x, grad=False: dev(np.ascontiguousarray(np.asarray(x).transpose(2, 0, 1, 3))).permute(1, 2, 0, 3) \
        if np.ndim(x) == 4 and np.shape(x)[2] == L else dev(x)
    args, _, states, h, c = op_args(Zs, Ks, Vs, Bs, Ws, h0, c0, grad=False, wrap=lnh)
    seg = lambda sl: [t[:, :, sl] if (t.dim() == 4 and t.shape[2] == L) else t for t in args]
    with torch.no_grad():
        o1, c1 = fwp.fast_lstm_v4(*seg(slice(0, 17)))
        o2, c2 = fwp.fast_lstm_v4(*seg(slice(17, L)))
    r_out, r_cell, r_W, r_h, r_c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    check("out", torch.cat([o1, o2], 2), r_out)
    check("cell", torch.cat([c1, c2], 2), r_cell)
    check("h", h, r_h)
    check("c", c, r_c)
    for a in range(3):
        check(f"W[{a}]", states[a], r_W[a])


def test_lstm_gradient_from_the_cell_output_is_ignored(fwp):
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(12, 1, 2, 9, 16)
    args, diff, *_ = op_args(Zs, Ks, Vs, Bs, Ws, h0, c0)
    out, cell = fwp.fast_lstm_v4(*args)
    (out * dev(go)).sum().backward()
    want = oracle.lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go)
    check("grad_z_u", diff[1][0].grad, want[0][1])


@pytest.mark.parametrize("D,T", [(32, 45), (16, 70)])
def test_lstm_backward_one_and_four_waves_per_sequence(fwp, D, T):
    """Below 1024 sequences the backward pass puts four waves on a sequence, from there on one:
    1100 sequences in one call against the same sequences in calls of 600 and 500.
    Tolerance: |a - b| <= 1e-4 + 1e-3 |b|."""
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(21, 1100, 1, T, D, dtype=np.float32, w0=True)
    tens = [dev(x) for x in (*Zs, *Ks, *Vs, *Bs)]
    Wd, hd, cd, god = [dev(w) for w in Ws], dev(h0), dev(c0), dev(go)

    def grads(sl):
        ts = [t[sl].clone().requires_grad_(True) for t in tens]
        args = []
        for a in range(3):
            args += [ts[a], ts[3 + a], ts[6 + a], ts[9 + a], Wd[a][sl].clone()]
        out, _ = fwp.fast_lstm_v4(*args, hd[sl].clone(), cd[sl].clone())
        return torch.autograd.grad(out, ts, god[sl])

    whole = grads(slice(0, 1100))
    parts = [grads(slice(0, 600)), grads(slice(600, 1100))]
    for i, w in enumerate(whole):
        got = torch.cat([parts[0][i], parts[1][i]], 0)
        assert torch.isfinite(got).all()
        assert torch.allclose(got, w, atol=1e-4, rtol=1e-3), (i, float((got - w).abs().max()))


@pytest.mark.parametrize("N,H,L,D", [(2, 3, 30, 32), (1, 2, 40, 16), (70, 8, 12, 32)])
def test_lstm_softmax_of_entries_far_apart(fwp, N, H, L, D):
    """The first entry of the output far below the others at every step (its candidate value is -80
    and its input and output gates are open): the kernels shift the softmax by the first entry and
    take the exact maximum only when an entry lies far above it, as here.  The last shape has more
    than 512 sequences: one wave per sequence forward."""
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(31 + D, N, H, L, D, w0=True)
    Zs[0][..., 0], Zs[1][..., 0], Zs[2][..., 0] = 10.0, -80.0, 10.0
    h0[..., 0], c0[..., 0] = -80.0, -80.0
    args, diff, states, h, c = op_args(Zs, Ks, Vs, Bs, Ws, h0, c0)
    out, cell = fwp.fast_lstm_v4(*args)
    ref = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    check("out", out, ref[0])
    check("cell", cell, ref[1])
    out.backward(dev(go))
    grads = oracle.lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go)
    for a, gate in enumerate("iuo"):
        for j, name in enumerate("z k v beta".split()):
            check(f"grad_{name}_{gate}", diff[a][j].grad, grads[j][a])
