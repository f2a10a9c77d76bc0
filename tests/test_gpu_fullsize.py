"""Benchmark-size checks through properties that do not need an oracle run of that size:
carried-state segment splits, linearity in the values, batch/head permutation, determinism."""
import numpy as np
import pytest
import torch

from helpers import delta_inputs, rec_inputs, rnn_inputs

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.asarray(a, np.float32)).cuda()


def grads_of(fn, inputs, go):
    ts = [t.clone().requires_grad_(True) for t in inputs]
    out = fn(ts)
    return out.detach(), torch.autograd.grad(out, ts, go)


def test_delta_full_size_properties(fwp):
    # LM-small shape of the benchmark: B=96,H=8,T=256,D=16
    q, k, v, beta, W0, go = (dev(a) for a in delta_inputs(0, 96, 8, 256, 16, 16, dtype=np.float32))

    def run(qq, kk, vv, bb, w0):
        W = w0.clone()
        return fwp.fast_weight_delta(qq, kk, vv, bb, W), W

    out, W = run(q, k, v, beta, W0)
    assert torch.isfinite(out).all()
    # a split at a position that is not a block boundary, state carried over (the blocked kernels
    # regroup the arithmetic at the split, so equality is to rounding, not bitwise)
    a, b = slice(0, 100), slice(100, 256)
    o1, W1 = run(q[:, :, a], k[:, :, a], v[:, :, a], beta[:, :, a], W0)
    o2, W2 = run(q[:, :, b], k[:, :, b], v[:, :, b], beta[:, :, b], W1)
    assert torch.allclose(torch.cat([o1, o2], 2), out, atol=5e-6, rtol=1e-5)
    assert torch.allclose(W2, W, atol=5e-6, rtol=1e-5)
    # a split on a block boundary is bitwise the same computation
    a, b = slice(0, 96), slice(96, 256)
    o1, W1 = run(q[:, :, a], k[:, :, a], v[:, :, a], beta[:, :, a], W0)
    o2, W2 = run(q[:, :, b], k[:, :, b], v[:, :, b], beta[:, :, b], W1)
    assert torch.equal(torch.cat([o1, o2], 2), out) and torch.equal(W2, W)
    # linear in (v, W0)
    v2 = torch.randn_like(v)
    o_b, _ = run(q, k, v2, beta, W0)
    o_c, _ = run(q, k, 2 * v - 3 * v2, beta, W0)
    assert torch.allclose(o_c, 2 * out - 3 * o_b, atol=2e-4, rtol=1e-3)
    # batch permutation
    perm = torch.randperm(96, device="cuda")
    o_p, W_p = run(q[perm], k[perm], v[perm], beta[perm], W0[perm])
    assert torch.equal(o_p, out[perm]) and torch.equal(W_p, W[perm])
    # gradients: deterministic, and the gradient of sum(out * go) w.r.t. v is linear in go
    _, g1 = grads_of(lambda t: fwp.fast_weight_delta(*t, W0.clone()), [q, k, v, beta], go)
    _, g2 = grads_of(lambda t: fwp.fast_weight_delta(*t, W0.clone()), [q, k, v, beta], go)
    for x, y in zip(g1, g2):
        assert torch.isfinite(x).all() and torch.equal(x, y)
    _, g3 = grads_of(lambda t: fwp.fast_weight_delta(*t, W0.clone()), [q, k, v, beta], 2 * go)
    assert torch.allclose(g3[2], 2 * g1[2], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("shape", [(96, 8, 256, 16), (32, 8, 1024, 32), (160, 8, 250, 16), (64, 8, 128, 32), (40, 8, 100, 16),
                                   (41, 25, 40, 16), (129, 9, 50, 32)])
@pytest.mark.parametrize("op", ["delta", "sum"])
def test_blocked_kernels_against_scan_kernels_at_full_occupancy(fwp, op, shape):
    """The blocked kernels (matrix cores, buffer-resource loads and stores) against the step-by-step
    kernels (another code path altogether) at sizes that put several waves on every SIMD: what only
    goes wrong when waves share a SIMD or the memory pipeline is busy shows here, not at the sizes
    the oracle is run at.  Tolerance as for the oracle parity: |a - b| <= 1e-4 + 1e-3 |b|."""
    B, H, T, D = shape
    q, k, v, beta, W0, go = (dev(a) for a in delta_inputs(1, B, H, T, D, D, dtype=np.float32))
    L_ = fwp._lib
    res = {}
    try:
        for kind in ("scan", "chunked", "split", "auto"):
            L_.config(L_.CFG_DELTA_KERNELS, {"scan": L_.DELTA_SCAN, "chunked": L_.DELTA_CHUNKED,
                                             "split": L_.DELTA_SPLIT, "auto": L_.DELTA_AUTO}[kind])
            W = W0.clone()
            if op == "delta":
                out, g = grads_of(lambda t: fwp.fast_weight_delta(*t, W), [q, k, v, beta], go)
            else:
                out, g = grads_of(lambda t: fwp.fast_weight_sum(*t, W), [q, k, v], go)
            res[kind] = (out, W, *g)
    finally:
        L_.config(L_.CFG_DELTA_KERNELS, L_.DELTA_AUTO)
    for kind in ("chunked", "split", "auto"):
        for i, (x, y) in enumerate(zip(res[kind], res["scan"])):
            assert torch.isfinite(x).all()
            assert torch.allclose(x, y, atol=1e-4, rtol=1e-3), (kind, i, float((x - y).abs().max()))


def off_by_one_float(t):
    """The same values at an address that is not a multiple of 16 bytes: the blocked and the
    step-by-step kernels refuse such a view and the generic kernels take the call."""
    buf = torch.empty(t.numel() + 1, device=t.device, dtype=t.dtype)
    buf[1:].copy_(t.reshape(-1))
    return buf[1:].view(t.shape)


@pytest.mark.parametrize("B,H,T,E,M", [(96, 8, 100, 32, 128), (96, 8, 100, 128, 32), (64, 4, 130, 16, 128),
                                       (33, 9, 47, 128, 16), (40, 8, 100, 192, 16),
                                       # up to 512 sequences: several waves per sequence (key tiles x value tiles)
                                       (40, 8, 100, 32, 128), (40, 8, 100, 128, 32), (32, 8, 130, 64, 64),
                                       (64, 8, 70, 16, 128), (50, 8, 90, 96, 32), (32, 16, 50, 32, 64),
                                       # only the several-wave form takes these, at any number of sequences
                                       (40, 8, 60, 192, 32), (96, 8, 40, 64, 128), (24, 8, 70, 128, 64)])
def test_sum_widest_states_blocked_against_generic_kernels(fwp, B, H, T, E, M):
    """The fast-net layers' memories (d_head x 4 d_head and back) at hundreds of sequences: the
    blocked kernels (one wave per sequence beyond 512 sequences, several up to there) against the generic
    ones, which a misaligned q selects.  Tolerance as for the oracle parity: |a - b| <= 1e-4 + 1e-3 |b|."""
    q, k, v, _, W0, go = (dev(a) for a in delta_inputs(5, B, H, T, E, M, dtype=np.float32, w0=True))
    res = []
    for misaligned in (False, True):
        W = W0.clone()
        ts = [t.clone().requires_grad_(True) for t in (q, k, v)]
        if misaligned:
            ts[0] = off_by_one_float(q).requires_grad_(True)
            assert ts[0].data_ptr() % 16 == 4
        out = fwp.fast_weight_sum(*ts, W)
        res.append((out.detach(), W, *torch.autograd.grad(out, ts, go)))
    for i, (x, y) in enumerate(zip(*res)):
        assert torch.isfinite(x).all()
        assert torch.allclose(x, y, atol=1e-4, rtol=1e-3), (i, float((x - y).abs().max()))


@pytest.mark.parametrize("E,M", [(64, 32), (96, 16), (16, 64), (64, 64), (32, 64), (96, 32)])
def test_delta_rectangular_states_at_full_occupancy(fwp, E, M):
    """1024 sequences (several waves on every SIMD) of the rectangular state shapes: a split on a
    block boundary with the state carried over is the same computation bit for bit, two runs give
    the same bits, and a sample of the sequences agrees with the float64 oracle."""
    import oracle
    arrays = delta_inputs(3, 128, 8, 128, E, M, dtype=np.float32)
    q, k, v, beta, W0, go = (dev(a) for a in arrays)

    def run(qq, kk, vv, bb, w0):
        W = w0.clone()
        return fwp.fast_weight_delta(qq, kk, vv, bb, W), W

    out, W = run(q, k, v, beta, W0)
    a, b = slice(0, 64), slice(64, 128)
    o1, W1 = run(q[:, :, a], k[:, :, a], v[:, :, a], beta[:, :, a], W0)
    o2, W2 = run(q[:, :, b], k[:, :, b], v[:, :, b], beta[:, :, b], W1)
    assert torch.equal(torch.cat([o1, o2], 2), out) and torch.equal(W2, W)
    _, g1 = grads_of(lambda t: fwp.fast_weight_delta(*t, W0.clone()), [q, k, v, beta], go)
    _, g2 = grads_of(lambda t: fwp.fast_weight_delta(*t, W0.clone()), [q, k, v, beta], go)
    for x, y in zip(g1, g2):
        assert torch.isfinite(x).all() and torch.equal(x, y)
    pick = [5, 77, 127]        # batch entries from the first, a middle and the last workgroups
    sub = [x[pick] for x in arrays]
    ref_out, ref_W = oracle.delta_fwd(*sub[:5])
    ref_g = oracle.delta_bwd(*sub)
    idx = torch.tensor(pick, device="cuda")
    for got, want in zip((out, W, *g1), (ref_out, ref_W, *ref_g)):
        got = got[idx].cpu().numpy()
        assert np.all(np.abs(got - want) <= 1e-4 + 1e-3 * np.abs(want)), float(np.abs(got - want).max())


@pytest.mark.parametrize("shape", [(1, 2, 20000, 16), (1, 1, 70001, 32)])
def test_delta_long_sequences_blocked_against_scan(fwp, shape):
    """Thousands of blocks and checkpoints per sequence (32-bit block offsets, the chunk index
    arithmetic, groups of four blocks with a partial last group): blocked kernels against the
    step-by-step kernels, outputs, final state and gradients."""
    N, H, T, D = shape
    q, k, v, beta, W0, go = (dev(a) for a in delta_inputs(5, N, H, T, D, D, dtype=np.float32))
    L_ = fwp._lib
    res = {}
    try:
        for kind in ("scan", "chunked", "split"):
            L_.config(L_.CFG_DELTA_KERNELS, {"scan": L_.DELTA_SCAN, "chunked": L_.DELTA_CHUNKED,
                                             "split": L_.DELTA_SPLIT}[kind])
            W = W0.clone()
            out, g = grads_of(lambda t: fwp.fast_weight_delta(*t, W), [q, k, v, beta], go)
            res[kind] = (out, W, *g)
    finally:
        L_.config(L_.CFG_DELTA_KERNELS, L_.DELTA_AUTO)
    for kind in ("chunked", "split"):
        for i, (x, y) in enumerate(zip(res[kind], res["scan"])):
            assert torch.isfinite(x).all()
            assert torch.allclose(x, y, atol=1e-4, rtol=1e-3), (kind, i, float((x - y).abs().max()))


def test_rnn_full_size_properties(fwp):
    z, k, v, W0, beta, h0, go = (dev(a) for a in rnn_inputs(1, 64, 8, 256, 32, dtype=np.float32))

    def run(sl, w0, hh):
        W, h = w0.clone(), hh.clone()
        out = fwp.fast_rnn_v2(z[:, :, sl], k[:, :, sl], v[:, :, sl], W, beta[:, :, sl], h)
        return out, W, h

    out, W, h = run(slice(0, 256), W0, h0)
    assert torch.isfinite(out).all() and torch.equal(h[:, :, 0], out[:, :, -1])
    o1, W1, h1 = run(slice(0, 70), W0, h0)
    o2, W2, h2 = run(slice(70, 256), W1, h1)
    assert torch.equal(torch.cat([o1, o2], 2), out) and torch.equal(W2, W) and torch.equal(h2, h)
    _, g1 = grads_of(lambda t: fwp.fast_rnn_v2(t[0], t[1], t[2], W0.clone(), t[3], h0.clone()), [z, k, v, beta], go)
    _, g2 = grads_of(lambda t: fwp.fast_rnn_v2(t[0], t[1], t[2], W0.clone(), t[3], h0.clone()), [z, k, v, beta], go)
    for x, y in zip(g1, g2):
        assert torch.isfinite(x).all() and torch.equal(x, y)
    assert torch.equal(g1[0][:, :, -1], go[:, :, -1])      # grad_z of the last step is the upstream gradient


@pytest.mark.parametrize("D,T", [(32, 100), (16, 70)])
def test_rnn_one_two_and_three_waves_per_sequence(fwp, D, T):
    """The Delta RNN puts several waves on a sequence: forward two up to 1024 sequences (two sequences
    to a workgroup up to 512, then four), one beyond; backward three up to 512, two beyond.  1100 sequences in
    one call against the same sequences in calls of 600 and 500 and of 511 (an odd count leaves a
    workgroup with one sequence) and 589.  Tolerance: |a - b| <= 1e-4 + 1e-3 |b|."""
    NS = 1100
    z, k, v, W0, beta, h0, go = (dev(a) for a in rnn_inputs(7, NS, 1, T, D, dtype=np.float32, w0=True))

    def run(sl):
        ts = [x[sl].clone().requires_grad_(True) for x in (z, k, v, beta)]
        out = fwp.fast_rnn_v2(ts[0], ts[1], ts[2], W0[sl].clone(), ts[3], h0[sl].clone())
        return (out.detach(), *torch.autograd.grad(out, ts, go[sl]))

    whole = run(slice(0, NS))
    for cut in (600, 511):
        parts = [run(slice(0, cut)), run(slice(cut, NS))]
        for i, w in enumerate(whole):
            got = torch.cat([parts[0][i], parts[1][i]], 0)
            assert torch.isfinite(got).all()
            assert torch.allclose(got, w, atol=1e-4, rtol=1e-3), (cut, i, float((got - w).abs().max()))


@pytest.mark.parametrize("D,T", [(32, 70), (16, 50)])
def test_rec_workgroups_of_two_and_of_four_sequences(fwp, D, T):
    """The Recurrent Delta Net's kernels put two sequences in a workgroup up to 512 sequences and four
    beyond (forward: from 513 to 1024): 1100 sequences in one call against the same sequences in
    calls of 600 and 500 and of 511 (an odd count leaves a workgroup with spare waves) and 589.  The
    gradients of the recurrent weights are sums over the sequences, so the parts' are added.
    Tolerance: |a - b| <= 1e-4 + 1e-3 |b| (1e-3 + 1e-3 |b| on those sums of 1100 terms)."""
    NS = 1100
    *x, go = (dev(a) for a in rec_inputs(9, NS, 1, T, D, dtype=np.float32, w0=True))
    qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0 = x

    def run(sl):
        ts = [t[sl].clone().requires_grad_(True) for t in (qx, kx, vx, bx)]
        rs = [t.clone().requires_grad_(True) for t in (R_q, R_k, R_v, r_b)]
        out = fwp.rec_update_fwm_tanh(*ts, *rs, W0[sl].clone(), h0[sl].clone())
        g = torch.autograd.grad(out, [*ts, *rs], go[sl])
        return (out.detach(), *g[:4]), g[4:]

    whole, whole_r = run(slice(0, NS))
    for cut in (600, 511):
        (a, ar), (b, br) = run(slice(0, cut)), run(slice(cut, NS))
        for i, w in enumerate(whole):
            got = torch.cat([a[i], b[i]], 0)
            assert torch.isfinite(got).all()
            assert torch.allclose(got, w, atol=1e-4, rtol=1e-3), (cut, i, float((got - w).abs().max()))
        for i, w in enumerate(whole_r):
            got = ar[i] + br[i]
            assert torch.allclose(got, w, atol=1e-3, rtol=1e-3), (cut, "R", i, float((got - w).abs().max()))


def test_rec_full_size_properties(fwp):
    *x, go = (dev(a) for a in rec_inputs(2, 64, 8, 256, 32, dtype=np.float32))
    qx, kx, vx, bx, R_q, R_k, R_v, r_b, W0, h0 = x

    def run(sl, w0, hh):
        W, h = w0.clone(), hh.clone()
        out = fwp.rec_update_fwm_tanh(qx[:, :, sl], kx[:, :, sl], vx[:, :, sl], bx[:, :, sl], R_q, R_k, R_v, r_b, W, h)
        return out, W, h

    out, W, h = run(slice(0, 256), W0, h0)
    assert torch.isfinite(out).all()
    o1, W1, h1 = run(slice(0, 130), W0, h0)
    o2, W2, h2 = run(slice(130, 256), W1, h1)
    assert torch.equal(torch.cat([o1, o2], 2), out) and torch.equal(W2, W) and torch.equal(h2, h)
    fn = lambda t: fwp.rec_update_fwm_tanh(*t, W0.clone(), h0.clone())
    _, g1 = grads_of(fn, x[:8], go)
    _, g2 = grads_of(fn, x[:8], go)
    for a, b in zip(g1, g2):
        assert torch.isfinite(a).all() and torch.equal(a, b)
    # the softmax Jacobian annihilates constants: grad_qx and grad_kx sum to zero over D
    scale = g1[0].abs().max().item()
    assert g1[0].sum(-1).abs().max().item() <= 1e-4 * max(scale, 1.0)
    assert g1[1].sum(-1).abs().max().item() <= 1e-4 * max(g1[1].abs().max().item(), 1.0)
