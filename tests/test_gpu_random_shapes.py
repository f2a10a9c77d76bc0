"""Seeded random shapes, layouts and gradient needs for the delta and the sum rule against the float64
oracle: key widths 1..200 and value widths 1..140 cross every way a state is run (whole, by slices of value
columns, with zero padded keys, several waves per sequence or one, on the LDS-state kernels), lengths 1..70
cross the 16-step block boundaries, inputs come contiguous or as permuted views of [L,N,H,D] storage, and
a random subset of the inputs asks for a gradient.  Tolerance: |hip - oracle| <= 1e-4 + 1e-3 |oracle|."""
import numpy as np
import pytest
import torch

import oracle
from helpers import delta_inputs, max_abs, rng, within

pytestmark = pytest.mark.gpu
ATOL, RTOL = 1e-4, 1e-3
WIDTHS = [16, 32, 64, 96, 128, 192]


def check(name, got, want):
    got = got.detach().cpu().numpy()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert np.all(np.isfinite(got)), name
    assert within(got, want, ATOL, RTOL), f"{name}: max abs err {max_abs(got, want):.3e}"


def draw(seed):
    g = rng(1000 + seed)
    pick = lambda hi: int(g.choice(WIDTHS)) if g.random() < 0.4 else int(g.integers(1, hi + 1))
    E, M = pick(200), pick(140)
    while E * M > 16384:        # the largest state the library accepts
        M = max(1, M // 2)
    N, H, L = int(g.integers(1, 4)), int(g.integers(1, 4)), int(g.integers(1, 71))
    time_major = bool(g.random() < 0.5)
    needs = [bool(g.random() < 0.8) for _ in range(4)]
    if not any(needs):
        needs[int(g.integers(0, 4))] = True
    return N, H, L, E, M, bool(g.random() < 0.7), time_major, needs


def on_device(a, time_major, grad):
    t = torch.from_numpy(np.asarray(a, np.float32)).cuda()
    if time_major:      # the same values as a permuted view of [L,N,H,D] storage
        t = t.permute(2, 0, 1, 3).contiguous().permute(1, 2, 0, 3)
    return t.requires_grad_(True) if grad else t


@pytest.mark.parametrize("seed", range(40))
def test_delta_rule_random_case(fwp, seed):
    N, H, L, E, M, w0, time_major, needs = draw(seed)
    print(f"delta seed={seed} N={N} H={H} L={L} E={E} M={M} w0={w0} time_major={time_major} needs={needs}", flush=True)
    q, k, v, beta, W0, go = delta_inputs(seed, N, H, L, E, M, w0=w0)
    ts = [on_device(a, time_major, n) for a, n in zip((q, k, v, beta), needs)]
    W = torch.from_numpy(W0.astype(np.float32)).cuda()
    out = fwp.fast_weight_delta(*ts, W)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(torch.from_numpy(go.astype(np.float32)).cuda())
    for name, t, n, r in zip("q k v beta".split(), ts, needs, oracle.delta_bwd(q, k, v, beta, W0, go)):
        if n:
            check("grad_" + name, t.grad, r)
        else:
            assert t.grad is None


@pytest.mark.parametrize("seed", range(40, 70))
def test_sum_rule_random_case(fwp, seed):
    N, H, L, E, M, w0, time_major, needs = draw(seed)
    needs = needs[:3] if any(needs[:3]) else [True, False, False]
    print(f"sum seed={seed} N={N} H={H} L={L} E={E} M={M} w0={w0} time_major={time_major} needs={needs}", flush=True)
    q, k, v, _, W0, go = delta_inputs(seed, N, H, L, E, M, w0=w0)
    ts = [on_device(a, time_major, n) for a, n in zip((q, k, v), needs)]
    W = torch.from_numpy(W0.astype(np.float32)).cuda()
    out = fwp.fast_weight_sum(*ts, W)
    ref_out, ref_W = oracle.sum_fwd(q, k, v, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(torch.from_numpy(go.astype(np.float32)).cuda())
    for name, t, n, r in zip("q k v".split(), ts, needs, oracle.sum_bwd(q, k, v, W0, go, through_state=False)):
        if n:
            check("grad_" + name, t.grad, r)
        else:
            assert t.grad is None


def draw_recurrent(seed):
    g = rng(5000 + seed)
    D = int(g.choice([16, 32])) if g.random() < 0.25 else int(g.integers(1, 41))     # up to 32 padded, beyond in LDS
    return int(g.integers(1, 4)), int(g.integers(1, 4)), int(g.integers(1, 50)), D, bool(g.random() < 0.7)


@pytest.mark.parametrize("seed", range(70, 90))
def test_delta_rnn_random_case(fwp, seed):
    from helpers import rnn_inputs
    N, H, L, D, w0 = draw_recurrent(seed)
    print(f"rnn seed={seed} N={N} H={H} L={L} D={D} w0={w0}", flush=True)
    z, k, v, W0, beta, h0, go = rnn_inputs(seed, N, H, L, D, w0=w0)
    tz, tk, tv, tb = (on_device(a, False, True) for a in (z, k, v, beta))
    W, h = on_device(W0, False, False), on_device(h0, False, False)
    out = fwp.fast_rnn_v2(tz, tk, tv, W, tb, h)
    ref_out, ref_W, ref_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    check("h", h, ref_h)
    out.backward(on_device(go, False, False))
    for name, t, r in zip("z k v beta".split(), (tz, tk, tv, tb), oracle.rnn_bwd(z, k, v, W0, beta, h0, go)):
        check("grad_" + name, t.grad, r)


@pytest.mark.parametrize("seed", range(90, 110))
def test_recurrent_delta_net_random_case(fwp, seed):
    from helpers import rec_inputs
    N, H, L, D, w0 = draw_recurrent(seed)
    print(f"rec seed={seed} N={N} H={H} L={L} D={D} w0={w0}", flush=True)
    *x, go = rec_inputs(seed, N, H, L, D, w0=w0)
    ts = [on_device(a, False, True) for a in x[:8]]
    W, h = on_device(x[8], False, False), on_device(x[9], False, False)
    out = fwp.rec_update_fwm_tanh(*ts, W, h)
    ref_out, ref_W, ref_h = oracle.rec_fwd(*x)
    check("out", out, ref_out)
    check("W", W, ref_W)
    check("h", h, ref_h)
    out.backward(on_device(go, False, False))
    for name, t, r in zip("qx kx vx bx R_q R_k R_v r_b".split(), ts, oracle.rec_bwd(*x, go)):
        check("grad_" + name, t.grad, r)


@pytest.mark.parametrize("seed", range(110, 125))
def test_delta_lstm_random_case(fwp, seed):
    from helpers import lstm_inputs
    N, H, L, D, w0 = draw_recurrent(seed)
    print(f"lstm seed={seed} N={N} H={H} L={L} D={D} w0={w0}", flush=True)
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(seed, N, H, L, D, w0=w0)
    args, diff, states = [], [], []
    for a in range(3):
        gate = [on_device(x, False, True) for x in (Zs[a], Ks[a], Vs[a], Bs[a])]
        W = on_device(Ws[a], False, False)
        args += gate + [W]
        diff += gate
        states.append(W)
    h, c = on_device(h0, False, False), on_device(c0, False, False)
    out, cell = fwp.fast_lstm_v4(*args, h, c)
    r_out, r_cell, r_W, r_h, r_c = oracle.lstm_fwd(Zs, Ks, Vs, Bs, Ws, h0, c0)
    check("out", out, r_out)
    check("cell", cell, r_cell)
    check("h", h, r_h)
    check("c", c, r_c)
    for a in range(3):
        check(f"W[{a}]", states[a], r_W[a])
    out.backward(on_device(go, False, False))
    grads = oracle.lstm_bwd(Zs, Ks, Vs, Bs, Ws, h0, c0, go)
    flat = [g for gate in zip(*grads) for g in gate] if len(grads) == 4 else None
    assert flat is not None and len(flat) == len(diff)
    for i, (t, r) in enumerate(zip(diff, flat)):
        check(f"grad[{i}]", t.grad, r)
