"""Stepwise inference: one call per time step (L = 1, no gradient), the state carried from call to call in W, h
and c as an actor or a decoder does (reference: the inference loop of
reinforcement_learning/torchbeast/polybeast_learner.py:376-393 calling torchbeast/layer.py:173,256-260,342 with T = 1; language_modeling/src/utils/cuda_fast_weight_layer.py:149-185 with carried `mems`).  Such calls
take kernels of their own; the results of a run of them are held to the float64 oracle's run over the whole
sequence, and to the kernels written for sequences.

Tolerance: |hip - oracle| <= 1e-4 + 1e-3 |oracle| elementwise."""
import numpy as np
import pytest
import torch

import oracle
from helpers import delta_inputs, lstm_inputs, max_abs, rec_inputs, rnn_inputs, within

pytestmark = pytest.mark.gpu
ATOL, RTOL = 1e-4, 1e-3
STEPS = 7


def dev(x):
    return torch.from_numpy(np.asarray(x, np.float32)).to("cuda")


def check(name, got, want):
    got = got.detach().cpu().numpy()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert np.all(np.isfinite(got)), name
    assert within(got, want, ATOL, RTOL), f"{name}: max abs err {max_abs(got, want):.3e}"


def step_of(t, i):
    return t[:, :, i:i + 1]


@pytest.fixture(params=["step kernels", "sequence kernels"])
def kernels(request, fwp):
    L_ = fwp._lib
    on = request.param == "step kernels"
    L_.config(L_.CFG_STEP_KERNELS, int(on))
    yield on
    L_.config(L_.CFG_STEP_KERNELS, 1)


def counted(fwp, on, calls, before, what):
    """Every call went to the single-step kernels, or none did."""
    took = fwp._lib.step_launches() - before
    assert took == (calls if on else 0), f"{what}: {took} of {calls} calls on the single-step kernels"


DELTA_STEP_SHAPES = [(2, 3, 16, 16), (4, 2, 32, 32), (1, 2, 64, 32), (2, 1, 96, 16), (1, 2, 128, 128), (2, 2, 16, 128),
                     (1, 3, 32, 64), (3, 1, 128, 16)]


@pytest.mark.parametrize("N,H,E,M", DELTA_STEP_SHAPES)
@pytest.mark.parametrize("time_major", [False, True])
def test_delta_rule_step_by_step(fwp, kernels, N, H, E, M, time_major):
    q, k, v, beta, W0, _ = delta_inputs(300 + E + M, N, H, STEPS, E, M, w0=True)
    want_out, want_W = oracle.delta_fwd(q, k, v, beta, W0)
    if time_major:      # [L,N,H,.] storage seen as [N,H,L,.], as the reference's layers hand it over
        tq, tk, tv, tb = (dev(np.ascontiguousarray(x.transpose(2, 0, 1, 3))).permute(1, 2, 0, 3) for x in (q, k, v, beta))
    else:
        tq, tk, tv, tb = (dev(x) for x in (q, k, v, beta))
    W = dev(W0)
    before = fwp._lib.step_launches()
    with torch.no_grad():
        outs = [fwp.fast_weight_delta(*(step_of(t, i) for t in (tq, tk, tv, tb)), W) for i in range(STEPS)]
    counted(fwp, kernels, STEPS, before, "delta rule")
    assert all(o.shape == (N, H, 1, M) for o in outs)
    check("out", torch.cat(outs, 2), want_out)
    check("W", W, want_W)


def test_delta_rule_steps_of_a_width_run_in_slices(fwp, kernels):
    """M = 3 D + 1 (the Delta-Delta layer's value width): the operator cuts the value columns into slices."""
    N, H, E, M = 2, 2, 32, 97
    q, k, v, beta, W0, _ = delta_inputs(41, N, H, STEPS, E, M, w0=True)
    want_out, want_W = oracle.delta_fwd(q, k, v, beta, W0)
    tq, tk, tv, tb = (dev(x) for x in (q, k, v, beta))
    W = dev(W0)
    with torch.no_grad():
        outs = [fwp.fast_weight_delta(*(step_of(t, i) for t in (tq, tk, tv, tb)), W) for i in range(STEPS)]
    check("out", torch.cat(outs, 2), want_out)
    check("W", W, want_W)


def test_a_differentiated_single_step_stays_on_the_sequence_kernels(fwp):
    """With gradients wanted the call saves for backward, which the single-step kernels do not."""
    q, k, v, beta, W0, go = delta_inputs(43, 2, 2, 1, 32, 32, w0=True)
    ts = [dev(x).requires_grad_(True) for x in (q, k, v, beta)]
    W = dev(W0)
    before = fwp._lib.step_launches()
    out = fwp.fast_weight_delta(*ts, W)
    out.backward(dev(go))
    assert fwp._lib.step_launches() == before
    check("out", out, oracle.delta_fwd(q, k, v, beta, W0)[0])
    for name, t, want in zip("q k v beta".split(), ts, oracle.delta_bwd(q, k, v, beta, W0, go)):
        check("grad_" + name, t.grad, want)


@pytest.mark.parametrize("N,H,E,M", [(2, 3, 16, 16), (1, 2, 32, 32), (2, 1, 32, 128), (1, 2, 128, 16), (1, 1, 96, 64)])
def test_sum_rule_step_by_step(fwp, kernels, N, H, E, M):
    q, k, v, _, W0, _ = delta_inputs(500 + E + M, N, H, STEPS, E, M, w0=True)
    want_out, want_W = oracle.sum_fwd(q, k, v, W0)
    tq, tk, tv = (dev(x) for x in (q, k, v))
    W = dev(W0)
    before = fwp._lib.step_launches()
    with torch.no_grad():
        outs = [fwp.fast_weight_sum(*(step_of(t, i) for t in (tq, tk, tv)), W) for i in range(STEPS)]
    counted(fwp, kernels, STEPS, before, "sum rule")
    check("out", torch.cat(outs, 2), want_out)
    check("W", W, want_W)


@pytest.mark.parametrize("N,H,D", [(2, 3, 16), (5, 2, 32), (64, 8, 32)])
def test_delta_rnn_step_by_step(fwp, kernels, N, H, D):
    z, k, v, W0, beta, h0, _ = rnn_inputs(600 + D, N, H, STEPS, D, w0=True)
    want_out, want_W, want_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    tz, tk, tv, tb = (dev(x) for x in (z, k, v, beta))
    W, h = dev(W0), dev(h0)
    before = fwp._lib.step_launches()
    with torch.no_grad():
        outs = [fwp.fast_rnn_v2(step_of(tz, i), step_of(tk, i), step_of(tv, i), W, step_of(tb, i), h) for i in range(STEPS)]
    counted(fwp, kernels, STEPS, before, "Delta RNN")
    check("out", torch.cat(outs, 2), want_out)
    check("W", W, want_W)
    check("h", h, want_h)


@pytest.mark.parametrize("N,H,D", [(2, 3, 16), (5, 2, 32), (64, 8, 32)])
def test_recurrent_delta_net_step_by_step(fwp, kernels, N, H, D):
    *x, _ = rec_inputs(700 + D, N, H, STEPS, D, w0=True)
    want_out, want_W, want_h = oracle.rec_fwd(*x)
    ts = [dev(a) for a in x]
    W, h = ts[8], ts[9]
    before = fwp._lib.step_launches()
    with torch.no_grad():
        outs = [fwp.rec_update_fwm_tanh(*(step_of(t, i) for t in ts[:4]), *ts[4:8], W, h) for i in range(STEPS)]
    counted(fwp, kernels, STEPS, before, "Recurrent Delta Net")
    check("out", torch.cat(outs, 2), want_out)
    check("W", W, want_W)
    check("h", h, want_h)


@pytest.mark.parametrize("N,H,D", [(2, 3, 16), (5, 2, 32), (64, 8, 32)])
def test_delta_lstm_step_by_step(fwp, kernels, N, H, D):
    Zs, Ks, Vs, Bs, Ws, h0, c0, _ = lstm_inputs(800 + D, N, H, STEPS, D, w0=True)
    want_out, want_cell, want_W, want_h, want_c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    tz, tk, tv, tb = ([dev(a) for a in xs] for xs in (Zs, Ks, Vs, Bs))
    tw = [dev(a) for a in Ws]
    h, c = dev(h0), dev(c0)
    before = fwp._lib.step_launches()
    outs, cells = [], []
    with torch.no_grad():
        for i in range(STEPS):
            args = []
            for a in range(3):
                args += [step_of(tz[a], i), step_of(tk[a], i), step_of(tv[a], i), step_of(tb[a], i), tw[a]]
            o, cl = fwp.fast_lstm_v4(*args, h, c)
            outs.append(o)
            cells.append(cl)
    counted(fwp, kernels, STEPS, before, "Delta LSTM")
    check("out", torch.cat(outs, 2), want_out)
    check("cell", torch.cat(cells, 2), want_cell)
    for a, gate in enumerate("iuo"):
        check("W_" + gate, tw[a], want_W[a])
    check("h", h, want_h)
    check("c", c, want_c)


def test_softmax_of_entries_far_apart_in_a_single_step(fwp, kernels):
    """States and pre-activations of very different magnitude: the softmaxes shift by the exact maximum."""
    N, H, D = 2, 2, 32
    z, k, v, W0, beta, h0, _ = rnn_inputs(77, N, H, 3, D, w0=True)
    h0 = h0 * 60.0
    z = z * 30.0
    want_out, want_W, want_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    tz, tk, tv, tb = (dev(x) for x in (z, k, v, beta))
    W, h = dev(W0), dev(h0)
    with torch.no_grad():
        outs = [fwp.fast_rnn_v2(step_of(tz, i), step_of(tk, i), step_of(tv, i), W, step_of(tb, i), h) for i in range(3)]
    check("out", torch.cat(outs, 2), want_out)
    check("h", h, want_h)


# Beyond 2048 sequences the single-step kernels put four waves (four sequences) into a workgroup; a count
# that is not a multiple of four leaves the last workgroup partly filled.
MANY = 2081


@pytest.mark.parametrize("N,H,E,M", [(MANY, 1, 16, 16), (2053, 1, 32, 64), (2052 // 4 + 1, 4, 128, 128)])
def test_delta_rule_steps_of_many_sequences(fwp, kernels, N, H, E, M):
    steps = 3
    q, k, v, beta, W0, _ = delta_inputs(900 + E + M, N, H, steps, E, M, w0=True)
    want_out, want_W = oracle.delta_fwd(q, k, v, beta, W0)
    tq, tk, tv, tb = (dev(x) for x in (q, k, v, beta))
    W = dev(W0)
    before = fwp._lib.step_launches()
    with torch.no_grad():
        outs = [fwp.fast_weight_delta(*(step_of(t, i) for t in (tq, tk, tv, tb)), W) for i in range(steps)]
    counted(fwp, kernels, steps, before, "delta rule")
    check("out", torch.cat(outs, 2), want_out)
    check("W", W, want_W)


@pytest.mark.parametrize("D", [16, 32])
def test_recurrent_operators_steps_of_many_sequences(fwp, kernels, D):
    steps, N, H = 3, MANY, 1
    L_ = fwp._lib
    before = L_.step_launches()
    with torch.no_grad():
        z, k, v, W0, beta, h0, _ = rnn_inputs(910 + D, N, H, steps, D, w0=True)
        want_out, want_W, want_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
        tz, tk, tv, tb = (dev(x) for x in (z, k, v, beta))
        W, h = dev(W0), dev(h0)
        outs = [fwp.fast_rnn_v2(step_of(tz, i), step_of(tk, i), step_of(tv, i), W, step_of(tb, i), h) for i in range(steps)]
        check("rnn out", torch.cat(outs, 2), want_out)
        check("rnn W", W, want_W)
        check("rnn h", h, want_h)

        *x, _ = rec_inputs(920 + D, N, 2, steps, D, w0=True)       # two heads: R is indexed by the head
        want_out, want_W, want_h = oracle.rec_fwd(*x)
        ts = [dev(a) for a in x]
        outs = [fwp.rec_update_fwm_tanh(*(step_of(t, i) for t in ts[:4]), *ts[4:8], ts[8], ts[9]) for i in range(steps)]
        check("rec out", torch.cat(outs, 2), want_out)
        check("rec W", ts[8], want_W)
        check("rec h", ts[9], want_h)

        Zs, Ks, Vs, Bs, Ws, h0, c0, _ = lstm_inputs(930 + D, N, H, steps, D, w0=True)
        want_out, want_cell, want_W, want_h, want_c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
        tz, tk, tv, tb = ([dev(a) for a in xs] for xs in (Zs, Ks, Vs, Bs))
        tw = [dev(a) for a in Ws]
        h, c = dev(h0), dev(c0)
        outs = []
        for i in range(steps):
            args = []
            for a in range(3):
                args += [step_of(tz[a], i), step_of(tk[a], i), step_of(tv[a], i), step_of(tb[a], i), tw[a]]
            outs.append(fwp.fast_lstm_v4(*args, h, c)[0])
        check("lstm out", torch.cat(outs, 2), want_out)
        for a, gate in enumerate("iuo"):
            check("lstm W_" + gate, tw[a], want_W[a])
        check("lstm h", h, want_h)
        check("lstm c", c, want_c)
    counted(fwp, kernels, 3 * steps, before, "recurrent operators")
