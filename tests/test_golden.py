"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the float64
oracle): the oracle must keep reproducing them, and the HIP operators must match them."""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, within

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLD, name)))


def d(*xs):
    return [x.astype(np.float64) for x in xs]


def test_oracle_reproduces_delta_fixture():
    g = load("delta_b2h2t64d16.npz")
    out, W = oracle.delta_fwd(*d(g["q"], g["k"], g["v"], g["beta"], g["W0"]))
    assert max_abs(out, g["out"]) < 1e-12 and max_abs(W, g["W"]) < 1e-12
    grads = oracle.delta_bwd(*d(g["q"], g["k"], g["v"], g["beta"], g["W0"], g["go"]))
    for a, n in zip(grads, ("gq", "gk", "gv", "gbeta")):
        assert max_abs(a, g[n]) < 1e-11


def test_oracle_reproduces_rnn_and_rec_fixtures():
    g = load("rnn_b1h2t32d32.npz")
    out, W, h = oracle.rnn_fwd(*d(g["z"], g["k"], g["v"], g["W0"], g["beta"], g["h0"]))
    assert max_abs(out, g["out"]) < 1e-12 and max_abs(W, g["W"]) < 1e-12 and max_abs(h, g["h"]) < 1e-12
    g = load("rec_b1h2t32d32.npz")
    names = "qx kx vx bx R_q R_k R_v r_b W0 h0".split()
    out, W, h = oracle.rec_fwd(*d(*[g[n] for n in names]))
    assert max_abs(out, g["out"]) < 1e-12 and max_abs(W, g["W"]) < 1e-12
    grads = oracle.rec_bwd(*d(*[g[n] for n in names], g["go"]))
    for a, n in zip(grads, names[:8]):
        assert max_abs(a, g["g" + n]) < 1e-10


def test_oracle_reproduces_sum_and_lstm_fixtures():
    g = load("sum_b3h5t7e11m4.npz")
    out, W = oracle.sum_fwd(*d(g["q"], g["k"], g["v"], g["W0"]))
    assert max_abs(out, g["out"]) < 1e-12 and max_abs(W, g["W"]) < 1e-12
    gq, gk, gv = oracle.sum_bwd(*d(g["q"], g["k"], g["v"], g["W0"], g["go"]))
    assert max(max_abs(gq, g["gq"]), max_abs(gk, g["gk"]), max_abs(gv, g["gv"])) < 1e-12
    assert max_abs(oracle.sum_bwd(*d(g["q"], g["k"], g["v"], g["W0"], g["go"]), through_state=True)[0],
                   g["gq_exact"]) < 1e-12
    g = load("lstm_b1h2t24d16.npz")
    gates = [list(d(*g[n])) for n in ("Z", "K", "V", "B", "W0")]
    out, cell, Wn, h, c = oracle.lstm_fwd(*gates, *d(g["h0"], g["c0"]))
    assert max_abs(out, g["out"]) < 1e-12 and max_abs(cell, g["cell"]) < 1e-12
    assert max_abs(np.stack(Wn), g["W"]) < 1e-12 and max_abs(h, g["h"]) < 1e-12 and max_abs(c, g["c"]) < 1e-12
    grads = oracle.lstm_bwd(*gates, *d(g["h0"], g["c0"], g["go"]))
    for got, n in zip(grads, ("gZ", "gK", "gV", "gB")):
        assert max_abs(np.stack(got), g[n]) < 1e-10


def test_float32_oracle_is_inside_the_parity_budget_on_the_fixtures():
    g = load("delta_b2h2t64d16.npz")
    out, _ = oracle.delta_fwd(g["q"], g["k"], g["v"], g["beta"], g["W0"])
    assert out.dtype == np.float32 and within(out, g["out"], 1e-4, 1e-3)


def _dev(x, grad=False):
    t = torch.from_numpy(np.asarray(x, np.float32)).to("cuda")
    return t.requires_grad_(True) if grad else t


def _check(name, got, want):
    got = got.detach().cpu().numpy()
    assert within(got, want, 1e-4, 1e-3), f"{name}: max abs err {max_abs(got, want):.3e}"


@pytest.mark.gpu
def test_hip_delta_matches_fixture(fwp):
    g = load("delta_b2h2t64d16.npz")
    ts = [_dev(g[n], True) for n in ("q", "k", "v", "beta")]
    W = _dev(g["W0"])
    out = fwp.fast_weight_delta(*ts, W)
    out.backward(_dev(g["go"]))
    _check("out", out, g["out"])
    _check("W", W, g["W"])
    for t, n in zip(ts, ("gq", "gk", "gv", "gbeta")):
        _check(n, t.grad, g[n])


@pytest.mark.gpu
def test_hip_rnn_matches_fixture(fwp):
    g = load("rnn_b1h2t32d32.npz")
    ts = [_dev(g[n], True) for n in ("z", "k", "v", "beta")]
    W, h = _dev(g["W0"]), _dev(g["h0"])
    out = fwp.fast_rnn_v2(ts[0], ts[1], ts[2], W, ts[3], h)
    out.backward(_dev(g["go"]))
    _check("out", out, g["out"])
    _check("W", W, g["W"])
    _check("h", h, g["h"])
    for t, n in zip(ts, ("gz", "gk", "gv", "gbeta")):
        _check(n, t.grad, g[n])


@pytest.mark.gpu
def test_hip_rec_matches_fixture(fwp):
    g = load("rec_b1h2t32d32.npz")
    names = "qx kx vx bx R_q R_k R_v r_b".split()
    ts = [_dev(g[n], True) for n in names]
    W, h = _dev(g["W0"]), _dev(g["h0"])
    out = fwp.rec_update_fwm_tanh(*ts, W, h)
    out.backward(_dev(g["go"]))
    _check("out", out, g["out"])
    _check("W", W, g["W"])
    _check("h", h, g["h"])
    for t, n in zip(ts, names):
        _check("g" + n, t.grad, g["g" + n])


@pytest.mark.gpu
@pytest.mark.parametrize("mode,key", [("reference", "gq"), ("exact", "gq_exact")])
def test_hip_sum_matches_fixture(fwp, mode, key):
    g = load("sum_b3h5t7e11m4.npz")
    ts = [_dev(g[n], True) for n in ("q", "k", "v")]
    W = _dev(g["W0"])
    fwp.FastWeightSum.state_gradient = mode
    try:
        out = fwp.fast_weight_sum(*ts, W)
        out.backward(_dev(g["go"]))
    finally:
        fwp.FastWeightSum.state_gradient = "reference"
    _check("out", out, g["out"])
    _check("W", W, g["W"])
    for t, n in zip(ts, (key, "gk", "gv")):
        _check(n, t.grad, g[n])


@pytest.mark.gpu
def test_hip_lstm_matches_fixture(fwp):
    g = load("lstm_b1h2t24d16.npz")
    diff = [[_dev(g[n][a], True) for n in ("Z", "K", "V", "B")] for a in range(3)]
    Ws = [_dev(g["W0"][a]) for a in range(3)]
    h, c = _dev(g["h0"]), _dev(g["c0"])
    args = []
    for a in range(3):
        args += diff[a] + [Ws[a]]
    out, cell = fwp.fast_lstm_v4(*args, h, c)
    out.backward(_dev(g["go"]))
    _check("out", out, g["out"])
    _check("cell", cell, g["cell"])
    _check("h", h, g["h"])
    _check("c", c, g["c"])
    for a in range(3):
        _check(f"W[{a}]", Ws[a], g["W"][a])
        for j, n in enumerate(("gZ", "gK", "gV", "gB")):
            _check(f"{n}[{a}]", diff[a][j].grad, g[n][a])
