"""GPU parity: the HIP operators (through the autograd Functions, i.e. through the
C ABI) against the float64 CPU oracle on the same seeded inputs.

Tolerance (fp32, stated by the task): |hip - oracle| <= 1e-4 + 1e-3 * |oracle|
elementwise, for outputs, final states and every gradient.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import delta_inputs, rec_inputs, rnn_inputs, within, max_abs

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


DELTA_SHAPES = [
    (2, 2, 64, 16, 16, False),    # the CPU-runnable configuration of the benchmark list
    (3, 5, 11, 64, 64, False),    # shape of the reference self test
    (2, 3, 130, 16, 16, True),    # ragged tail chunk, carried-in state
    (2, 2, 256, 32, 32, True),
    (1, 2, 1, 16, 16, True),      # single step (RL-style stepping)
    (2, 2, 37, 32, 97, True),     # E != M (Delta-Delta layer: M = 3D+1): slices of 64, 32 and a padded 1 value columns
    (2, 2, 70, 32, 128, True),    # Delta-MLP layer, wide side as values: two slices of 64 value columns
    (2, 2, 70, 128, 32, True),    # ... as keys: eight key tiles on the several-wave kernels
    (1, 2, 50, 128, 64, True),    # ... two slices of 32 value columns
    (1, 3, 40, 128, 16, True),    # Performer with 64 random features
    (1, 2, 50, 96, 48, True),     # 96 keys take values of 16 or 32: slices of 32 and 16
    (1, 2, 40, 192, 32, True),    # DPFP with nu = 3 at D = 32 (E = 2 nu D): twelve key tiles, two slices of 16 value columns
    (2, 1, 50, 160, 16, True),    # Performer with 80 random features: keys zero padded to 192
    (1, 2, 33, 200, 24, True),    # keys beyond 192: state in LDS
    (1, 1, 33, 256, 64, True),    # the largest state the library accepts (16384 floats)
    (1, 3, 70, 24, 8, False),     # E != M, M smaller
    (1, 1, 20, 5, 3, True),       # odd sizes
]


@pytest.mark.parametrize("N,H,L,E,M,w0", DELTA_SHAPES)
def test_delta(fwp, delta_kernels, N, H, L, E, M, w0):
    q, k, v, beta, W0, go = delta_inputs(100 + L + E, N, H, L, E, M, w0=w0)
    tq, tk, tv, tb = (dev(x, True) for x in (q, k, v, beta))
    W = dev(W0)
    out = fwp.fast_weight_delta(tq, tk, tv, tb, W)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(dev(go))
    for name, t, r in zip("q k v beta".split(), (tq, tk, tv, tb), oracle.delta_bwd(q, k, v, beta, W0, go)):
        check("grad_" + name, t.grad, r)
    check("W after backward", W, ref_W)     # backward does not rewind the caller's state


# every state shape E x M (multiples of 16) that the kernels with several waves per sequence are built for
RECTANGULAR = [(16, 16), (16, 32), (16, 64), (32, 16), (32, 32), (32, 64), (64, 16), (64, 32), (64, 64),
               (96, 16), (96, 32), (128, 16), (128, 32), (192, 16)]


@pytest.mark.parametrize("E,M", RECTANGULAR)
@pytest.mark.parametrize("L", [16, 80])
def test_delta_rectangular_states(fwp, E, M, L):
    """E != M and D = 64 (feature maps that widen the keys, values wider than keys): whole blocks go to
    the matrix-core kernels, other lengths (checked once below) to the LDS kernels."""
    N, H = 2, 3
    q, k, v, beta, W0, go = delta_inputs(700 + E + M + L, N, H, L, E, M, w0=True)
    tq, tk, tv, tb = (dev(x, True) for x in (q, k, v, beta))
    W = dev(W0)
    out = fwp.fast_weight_delta(tq, tk, tv, tb, W)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(dev(go))
    for name, t, r in zip("q k v beta".split(), (tq, tk, tv, tb), oracle.delta_bwd(q, k, v, beta, W0, go)):
        check("grad_" + name, t.grad, r)


def test_delta_rectangular_states_views_and_segments(fwp):
    # permuted views of [L,N,H,*] storage, a carried state over two segments (80 = 48 + 32), E = 96, M = 16
    N, H, L, E, M = 2, 2, 80, 96, 16
    q, k, v, beta, W0, go = delta_inputs(77, N, H, L, E, M, w0=True)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    ref_g = oracle.delta_bwd(q, k, v, beta, W0, go)
    lead = [dev(np.ascontiguousarray(np.transpose(x, (2, 0, 1, 3))), True) for x in (q, k, v, beta)]
    tq, tk, tv, tb = (t.permute(1, 2, 0, 3) for t in lead)
    W = dev(W0)
    outs = []
    for a, b in ((0, 48), (48, 80)):
        outs.append(fwp.fast_weight_delta(tq[:, :, a:b], tk[:, :, a:b], tv[:, :, a:b], tb[:, :, a:b], W))
        W = W.clone()           # the state an earlier segment's backward reads must stay as it was
    out = torch.cat(outs, 2)
    check("out", out, ref_out)
    check("W", W, ref_W)
    # gradients of the two segments on their own (the state is not differentiated through, as in the reference)
    out.backward(dev(go))
    first = oracle.delta_bwd(q[:, :, :48], k[:, :, :48], v[:, :, :48], beta[:, :, :48], W0, go[:, :, :48])
    mid_W = oracle.delta_fwd(q[:, :, :48], k[:, :, :48], v[:, :, :48], beta[:, :, :48], W0)[1]
    second = oracle.delta_bwd(q[:, :, 48:], k[:, :, 48:], v[:, :, 48:], beta[:, :, 48:], mid_W, go[:, :, 48:])
    for name, t, a, b in zip("q k v beta".split(), lead, first, second):
        check("grad_" + name, t.grad.permute(1, 2, 0, 3), np.concatenate((a, b), 2))


@pytest.mark.parametrize("L", [15, 16, 17, 31, 33, 47, 48, 100])
@pytest.mark.parametrize("D", [16, 32])
def test_delta_block_edges(fwp, delta_kernels, L, D):
    # lengths around the 16-step block and 32-step prefetch boundaries of the blocked kernel
    q, k, v, beta, W0, go = delta_inputs(500 + L + D, 2, 2, L, D, D, w0=True)
    tq, tk, tv, tb = (dev(x, True) for x in (q, k, v, beta))
    W = dev(W0)
    out = fwp.fast_weight_delta(tq, tk, tv, tb, W)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(dev(go))
    for name, t, r in zip("q k v beta".split(), (tq, tk, tv, tb), oracle.delta_bwd(q, k, v, beta, W0, go)):
        check("grad_" + name, t.grad, r)


@pytest.mark.parametrize("D", [16, 32])
def test_delta_write_strengths_zero_tiny_negative_and_above_one(fwp, delta_kernels, D):
    # write strengths as the operator admits them (any real number, not only sigmoid outputs): exact
    # zeros (the step writes nothing, v - v_old still is saved for backward), denormals, tiny values,
    # negative values and values above one, spread so that some blocks of 16 steps have none of them
    q, k, v, beta, W0, go = delta_inputs(900 + D, 2, 3, 100, D, D, w0=True)
    beta = beta.copy()
    beta[:, :, 5] = 0.0
    beta[:, :, 17:20] = 0.0
    beta[0, :, 40] = 1e-42          # denormal
    beta[1, :, 41] = 1e-33
    beta[:, :, 50] = -0.7
    beta[:, :, 66] = 1.9
    beta[:, :, 99] = 0.0            # in the last, partial block
    tq, tk, tv, tb = (dev(x, True) for x in (q, k, v, beta))
    W = dev(W0)
    out = fwp.fast_weight_delta(tq, tk, tv, tb, W)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(dev(go))
    for name, t, r in zip("q k v beta".split(), (tq, tk, tv, tb), oracle.delta_bwd(q, k, v, beta, W0, go)):
        check("grad_" + name, t.grad, r)


def test_delta_strided_views_and_segments(fwp, delta_kernels):
    # inputs as the layers pass them: [L,N,H,*] storage permuted to [N,H,L,*], and a carried state
    N, H, L, D = 2, 3, 48, 16
    q, k, v, beta, W0, go = delta_inputs(7, N, H, L, D, D, w0=True)
    def lnh(x):
        return dev(np.ascontiguousarray(x.transpose(2, 0, 1, 3))).permute(1, 2, 0, 3)
    tq, tk, tv, tb, tgo = lnh(q), lnh(k), lnh(v), lnh(beta), lnh(go)
    for t in (tq, tk, tv, tb):
        t.requires_grad_(True)
    assert not tq.is_contiguous()
    W = dev(W0)
    a, b = slice(0, 20), slice(20, L)
    o1 = fwp.fast_weight_delta(tq[:, :, a], tk[:, :, a], tv[:, :, a], tb[:, :, a], W)
    o2 = fwp.fast_weight_delta(tq[:, :, b], tk[:, :, b], tv[:, :, b], tb[:, :, b], W)
    out = torch.cat([o1, o2], dim=2)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    # gradients of the first segment alone (the carried state is detached, as in the reference)
    o1.backward(tgo[:, :, a])
    refs = oracle.delta_bwd(q[:, :, a], k[:, :, a], v[:, :, a], beta[:, :, a], W0, go[:, :, a])
    check("grad_q", tq.grad[:, :, a], refs[0])
    check("grad_beta", tb.grad[:, :, a], refs[3])


@pytest.mark.parametrize("E,M,L", [(16, 16, 40), (32, 32, 100), (96, 16, 50), (16, 64, 33)])
def test_delta_no_grad_path(fwp, delta_kernels, E, M, L):
    # nothing is saved for backward: no vdiff, no checkpoints, no per-block inverses
    q, k, v, beta, W0, _ = delta_inputs(8, 2, 2, L, E, M, w0=True)
    with torch.no_grad():
        W = dev(W0)
        out = fwp.fast_weight_delta(dev(q), dev(k), dev(v), dev(beta), W)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    check("out", out, ref_out)
    check("W", W, ref_W)


RNN_SHAPES = [(2, 2, 64, 16, False), (3, 5, 11, 64, False), (2, 2, 256, 32, True), (1, 2, 1, 32, True),
              (3, 5, 40, 32, True), (1, 3, 100, 16, True),
              (2, 3, 77, 8, True), (1, 1, 19, 5, True),
              (2, 2, 50, 24, True), (1, 2, 1, 18, True)]     # head sizes that run padded to 16 or 32: these four


@pytest.mark.parametrize("N,H,L,D,w0", RNN_SHAPES)
def test_rnn(fwp, N, H, L, D, w0):
    z, k, v, W0, beta, h0, go = rnn_inputs(200 + L + D, N, H, L, D, w0=w0)
    tz, tk, tv, tb = (dev(x, True) for x in (z, k, v, beta))
    W, h = dev(W0), dev(h0)
    out = fwp.fast_rnn_v2(tz, tk, tv, W, tb, h)
    ref_out, ref_W, ref_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    check("h", h, ref_h)
    out.backward(dev(go))
    for name, t, r in zip("z k v beta".split(), (tz, tk, tv, tb), oracle.rnn_bwd(z, k, v, W0, beta, h0, go)):
        check("grad_" + name, t.grad, r)


REC_SHAPES = [(2, 2, 64, 16, False), (3, 5, 11, 32, False), (2, 2, 256, 32, True), (1, 2, 1, 32, True),
              (1, 3, 100, 16, True),
              (2, 3, 77, 8, True), (1, 1, 19, 5, True), (1, 2, 30, 64, False),
              (2, 2, 50, 24, True), (1, 2, 1, 18, True)]     # 8, 5, 24 and 18 run padded to 16 or 32


@pytest.mark.parametrize("N,H,L,D,w0", REC_SHAPES)
def test_rec(fwp, N, H, L, D, w0):
    *x, go = rec_inputs(300 + L + D, N, H, L, D, w0=w0)
    ts = [dev(a, True) for a in x[:8]]
    W, h = dev(x[8]), dev(x[9])
    out = fwp.rec_update_fwm_tanh(*ts, W, h)
    ref_out, ref_W, ref_h = oracle.rec_fwd(*x)
    check("out", out, ref_out)
    check("W", W, ref_W)
    check("h", h, ref_h)
    out.backward(dev(go))
    names = "qx kx vx bx R_q R_k R_v r_b".split()
    for name, t, r in zip(names, ts, oracle.rec_bwd(*x, go)):
        check("grad_" + name, t.grad, r)


def test_lds_state_kernels_of_the_recurrent_operators_at_a_small_head_size(fwp):
    """The operators pad head sizes below 32; the autograd Functions under them do not, and send D = 5 to
    the kernels that keep the state in LDS."""
    N, H, L, D = 1, 2, 19, 5
    z, k, v, W0, beta, h0, go = rnn_inputs(5, N, H, L, D, w0=True)
    tz, tk, tv, tb = (dev(x, True) for x in (z, k, v, beta))
    W, h = dev(W0), dev(h0)
    out = fwp.FastRNNv2.apply(tz, tk, tv, W, tb, h)
    ref_out, ref_W, ref_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    check("rnn out", out, ref_out)
    check("rnn W", W, ref_W)
    out.backward(dev(go))
    for name, t, r in zip("z k v beta".split(), (tz, tk, tv, tb), oracle.rnn_bwd(z, k, v, W0, beta, h0, go)):
        check("rnn grad_" + name, t.grad, r)
    *x, go = rec_inputs(6, N, H, L, D, w0=True)
    ts = [dev(a, True) for a in x[:8]]
    W, h = dev(x[8]), dev(x[9])
    out = fwp.FastWeightRecUpdateTanh.apply(*ts, W, h)
    ref_out, ref_W, ref_h = oracle.rec_fwd(*x)
    check("rec out", out, ref_out)
    check("rec h", h, ref_h)
    out.backward(dev(go))
    for name, t, r in zip("qx kx vx bx R_q R_k R_v r_b".split(), ts, oracle.rec_bwd(*x, go)):
        check("rec grad_" + name, t.grad, r)


@pytest.mark.parametrize("D", [24, 9])
def test_padded_head_sizes_carry_their_states_and_keep_the_operators_errors(fwp, D):
    """Head sizes that run padded: two calls with W and h carried over equal the oracle's whole run (the
    states that come back are the narrow ones), outputs that differ by hundreds do not reach the padding,
    and a state the operator refuses is refused with the operator's own message, W and h untouched."""
    N, H, L = 2, 3, 44
    z, k, v, W0, beta, h0, go = rnn_inputs(31 + D, N, H, L, D, w0=True)
    z, h0 = z * 60.0, h0 * 60.0
    ref_out, ref_W, ref_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    W, h = dev(W0), dev(h0)
    a, b = slice(0, 20), slice(20, L)
    outs = [fwp.fast_rnn_v2(dev(z[:, :, s]), dev(k[:, :, s]), dev(v[:, :, s]), W, dev(beta[:, :, s]), h) for s in (a, b)]
    assert W.shape == (N, H, D, D) and h.shape == (N, H, 1, D)
    check("out", torch.cat(outs, 2), ref_out)
    check("W", W, ref_W)
    check("h", h, ref_h)
    before = W.clone()
    with pytest.raises(fwp._lib.FwpError, match="contiguous"):
        fwp.fast_rnn_v2(dev(z), dev(k), dev(v), W.transpose(2, 3), dev(beta), h)
    with pytest.raises(AssertionError):
        fwp.fast_rnn_v2(dev(z), dev(k[:, :, :-1]), dev(v), W, dev(beta), h)
    assert torch.equal(W, before)


@pytest.mark.parametrize("N,H,L,D", [(2, 3, 40, 32), (1, 2, 50, 16), (130, 8, 20, 32)])
def test_rnn_softmax_of_entries_far_apart(fwp, N, H, L, D):
    """Outputs that differ by hundreds across the D entries: the kernels shift the softmax by the
    first entry and take the exact maximum only when an entry lies far above it, which these inputs
    make happen at most steps (the last shape has more than 1024 sequences: one wave per sequence)."""
    z, k, v, W0, beta, h0, go = rnn_inputs(77 + D, N, H, L, D, w0=True)
    z, h0 = z * 60.0, h0 * 60.0
    tz, tk, tv, tb = (dev(x, True) for x in (z, k, v, beta))
    W, h = dev(W0), dev(h0)
    out = fwp.fast_rnn_v2(tz, tk, tv, W, tb, h)
    ref_out, ref_W, ref_h = oracle.rnn_fwd(z, k, v, W0, beta, h0)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(dev(go))
    for name, t, r in zip("z k v beta".split(), (tz, tk, tv, tb), oracle.rnn_bwd(z, k, v, W0, beta, h0, go)):
        check("grad_" + name, t.grad, r)


@pytest.mark.parametrize("N,H,L,D", [(2, 3, 40, 32), (1, 2, 50, 16)])
def test_rec_softmax_of_entries_far_apart(fwp, N, H, L, D):
    """The same for the Recurrent Delta Net: query and key inputs that differ by hundreds."""
    *x, go = rec_inputs(78 + D, N, H, L, D, w0=True)
    x[0], x[1] = x[0] * 60.0, x[1] * 60.0
    ts = [dev(a, True) for a in x[:8]]
    W, h = dev(x[8]), dev(x[9])
    out = fwp.rec_update_fwm_tanh(*ts, W, h)
    ref_out, ref_W, ref_h = oracle.rec_fwd(*x)
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.backward(dev(go))
    names = "qx kx vx bx R_q R_k R_v r_b".split()
    for name, t, r in zip(names, ts, oracle.rec_bwd(*x, go)):
        check("grad_" + name, t.grad, r)


def test_rnn_and_rec_take_strided_views(fwp):
    # inputs as the layers pass them: [L,N,H,*] storage permuted to [N,H,L,*]
    def lnh(x):
        return dev(np.ascontiguousarray(x.transpose(2, 0, 1, 3))).permute(1, 2, 0, 3)
    z, k, v, W0, beta, h0, go = rnn_inputs(11, 2, 3, 40, 32, w0=True)
    ts = [lnh(a).requires_grad_(True) for a in (z, k, v, beta)]
    out = fwp.fast_rnn_v2(ts[0], ts[1], ts[2], dev(W0), ts[3], dev(h0))
    out.backward(lnh(go))
    check("rnn out", out, oracle.rnn_fwd(z, k, v, W0, beta, h0)[0])
    for t, r in zip(ts, oracle.rnn_bwd(z, k, v, W0, beta, h0, go)):
        check("rnn grad", t.grad, r)
    *x, go = rec_inputs(12, 2, 3, 40, 32, w0=True)
    ts = [lnh(a).requires_grad_(True) for a in x[:4]] + [dev(a, True) for a in x[4:8]]
    out = fwp.rec_update_fwm_tanh(*ts, dev(x[8]), dev(x[9]))
    out.backward(lnh(go))
    check("rec out", out, oracle.rec_fwd(*x)[0])
    for t, r in zip(ts, oracle.rec_bwd(*x, go)):
        check("rec grad", t.grad, r)


def test_deterministic(fwp):
    *x, go = rec_inputs(9, 4, 2, 50, 32)
    res = []
    for _ in range(2):
        ts = [dev(a, True) for a in x[:8]]
        out = fwp.rec_update_fwm_tanh(*ts, dev(x[8]), dev(x[9]))
        out.backward(dev(go))
        res.append([out.detach().clone()] + [t.grad.clone() for t in ts])
    for a, b in zip(*res):
        assert torch.equal(a, b)


def test_rejects_cpu_tensors_and_bad_shapes(fwp):
    q, k, v, beta, W0, _ = delta_inputs(1, 1, 1, 4, 4, 4)
    cpu = [torch.from_numpy(a.astype(np.float32)) for a in (q, k, v, beta, W0)]
    with pytest.raises(RuntimeError):
        fwp.fast_weight_delta(*cpu)
    with pytest.raises(RuntimeError):
        fwp.fast_weight_delta(dev(q), dev(k[:, :, :3]), dev(v), dev(beta), dev(W0))
    with pytest.raises(AssertionError):
        fwp.fast_rnn_v2(dev(v), dev(k), dev(v), dev(W0), dev(beta), dev(v[:, :, :1, :3]))


def test_sliced_value_columns_check_w_like_the_whole_state_path(fwp):
    """A call that runs by slices of value columns (E = 32, M = 128) refuses a W that the whole-state
    path refuses - wrong shape, not contiguous, not fp32 - with the same error, before anything runs:
    the caller's W is untouched afterwards."""
    q, k, v, beta, W0, _ = delta_inputs(77, 2, 2, 40, 32, 128, w0=True)
    args = [dev(x) for x in (q, k, v, beta)]
    wide = dev(np.concatenate([W0, W0], -1))
    for bad in (wide[..., ::2], dev(W0).double(), dev(W0)[..., :64], dev(W0)[:1]):
        before = bad.clone()
        with pytest.raises(fwp._lib.FwpError, match="W must be a contiguous fp32"):
            fwp.fast_weight_delta(*args, bad)
        assert torch.equal(bad, before)


# ------------------------------------------------------------------ output layout

TIME_MAJOR_SHAPES = [
    (2, 3, 130, 16, 16),     # blocked kernels, ragged last block
    (2, 2, 256, 32, 32),
    (1, 2, 1, 16, 16),       # single step: scan kernels
    (2, 3, 20, 16, 16),      # short: scan kernels
    (2, 2, 37, 32, 97),      # LDS-state kernels, rows of 97 floats
    (1, 1, 20, 5, 3),
    (2, 3, 80, 96, 16),      # rectangular state on the several-wave kernels
]


@pytest.mark.parametrize("N,H,L,E,M", TIME_MAJOR_SHAPES)
def test_delta_output_with_steps_outermost(fwp, delta_kernels, N, H, L, E, M):
    """The operator writes its [N,H,L,M] result into [L,N,H,M] storage on request, and by itself when Q
    is a view of storage laid out that way (the reference's layers: cuda_fast_weight_layer.py:108-116
    hand over permuted views and reshape the result to [L,N,H*M], :158-163)."""
    q, k, v, beta, W0, go = delta_inputs(900 + L + E + M, N, H, L, E, M, w0=True)
    ref_out, ref_W = oracle.delta_fwd(q, k, v, beta, W0)
    ref_g = oracle.delta_bwd(q, k, v, beta, W0, go)
    # asked for
    ts = [dev(x, True) for x in (q, k, v, beta)]
    W = dev(W0)
    out = fwp.fast_weight_delta(*ts, W, True)
    assert out.shape == (N, H, L, M) and out.permute(2, 0, 1, 3).is_contiguous()
    check("out", out, ref_out)
    check("W", W, ref_W)
    out.permute(2, 0, 1, 3).reshape(L, N, H * M).backward(
        dev(np.ascontiguousarray(np.transpose(go, (2, 0, 1, 3))).reshape(L, N, H * M)))
    for name, t, r in zip("q k v beta".split(), ts, ref_g):
        check("grad_" + name, t.grad, r)
    # following Q: views of [L,N,H,*] storage in, a view of [L,N,H,M] storage out; contiguous in, contiguous out
    lead = [dev(np.ascontiguousarray(np.transpose(x, (2, 0, 1, 3)))) for x in (q, k, v, beta)]
    out2 = fwp.fast_weight_delta(*(t.permute(1, 2, 0, 3) for t in lead), dev(W0))
    if L > 1 and N * H > 1:
        assert out2.permute(2, 0, 1, 3).is_contiguous()
    check("out (views in)", out2, ref_out)
    out3 = fwp.fast_weight_delta(*(dev(x) for x in (q, k, v, beta)), dev(W0))
    assert out3.is_contiguous()
    out4 = fwp.fast_weight_delta(*(t.permute(1, 2, 0, 3) for t in lead), dev(W0), False)
    assert out4.is_contiguous()
    check("out (views in, contiguous out)", out4, ref_out)


@pytest.mark.parametrize("N,H,L,D", [(2, 3, 100, 16), (2, 2, 70, 32), (1, 2, 9, 32), (2, 2, 40, 24)])
def test_delta_forward_through_the_c_abi_into_a_wider_buffer(fwp, delta_kernels, N, H, L, D):
    """fwp_delta_fwd_strided: rows of the result land inside a wider [N,H,L,D+16] buffer whose other
    columns stay as they were."""
    L_ = fwp._lib
    lib = L_.lib()
    q, k, v, beta, W0, _ = delta_inputs(950 + L + D, N, H, L, D, D, dtype=np.float32, w0=True)
    want, want_W = oracle.delta_fwd(*(a.astype(np.float64) for a in (q, k, v, beta, W0)))
    tq, tk, tv, tb, W = (torch.from_numpy(a).cuda() for a in (q, k, v, beta, W0))
    wide = torch.full((N, H, L, D + 16), -7.0, device="cuda")
    view = lambda t: L_.View(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))
    window = wide[..., 8:8 + D]          # 32-byte offset: rows stay 16-byte aligned
    ov = L_.OutView(window.data_ptr(), window.stride(0), window.stride(1), window.stride(2))
    L_.check(lib.fwp_delta_fwd_strided(view(tq), view(tk), view(tv), view(tb), L_.ptr(W), ov, None, None,
                                       N, H, L, D, D, L_.query(L_.Q_DEFAULT_CHUNK), L_.stream_of(tq)), "fwd")
    torch.cuda.synchronize()
    check("out", window, want)
    check("W", W, want_W)
    assert bool((wide[..., :8] == -7.0).all()) and bool((wide[..., 8 + D:] == -7.0).all())
