"""The C++ autograd binding of the delta rule (csrc/fwp_torch.cpp) against the Python
autograd.Function over the same C ABI: same results bit for bit, same errors, same treatment
of views and of inputs that need no gradient."""
import importlib

import numpy as np
import pytest
import torch

from helpers import delta_inputs


def native(fwp):
    mod = fwp.fast_weight._fwp_torch
    if mod is None:
        pytest.fail("recurrent-fwp_amd/_fwp_torch.so has not been built (csrc/build_torch.sh)")
    return mod


def test_binding_is_built_and_is_the_default(fwp):
    fw = importlib.import_module(fwp.__name__ + ".fast_weight")
    assert fw._operator is native(fwp).fast_weight_delta


def test_binding_refuses_what_the_python_function_refuses(fwp):
    f = native(fwp).fast_weight_delta
    q = torch.zeros(1, 1, 2, 4)
    with pytest.raises(fwp._lib.FwpError, match="MI355X"):
        f(q, q, q, q[..., :1], torch.zeros(1, 1, 4, 4))


@pytest.mark.gpu
@pytest.mark.parametrize("N,H,L,E,M", [(2, 2, 64, 16, 16), (2, 3, 130, 32, 32), (1, 2, 37, 200, 8), (1, 2, 1, 16, 16)])
@pytest.mark.parametrize("time_major", [None, True, False])
def test_same_as_python_function(fwp, N, H, L, E, M, time_major):
    q, k, v, beta, W0, go = (torch.from_numpy(a).cuda() for a in delta_inputs(3, N, H, L, E, M, dtype=np.float32))
    results = []
    for f in (native(fwp).fast_weight_delta, fwp.DeltaFastWeight.apply):
        ins = [t.clone().requires_grad_(True) for t in (q, k, v, beta)]
        W = W0.clone()
        out = f(*ins, W) if time_major is None else f(*ins, W, time_major)
        grads = torch.autograd.grad(out, ins, go)
        results.append([out, W, *grads])
    for a, b in zip(*results):
        assert torch.equal(a, b) and a.stride() == b.stride()


@pytest.mark.gpu
def test_views_no_grad_and_shape_errors(fwp):
    f = native(fwp).fast_weight_delta
    N, H, L, D = 2, 2, 48, 16
    q, k, v, beta, W0, go = (torch.from_numpy(a).cuda() for a in delta_inputs(5, N, H, L, D, D, dtype=np.float32))
    # [L,N,H,3D+1] storage as the Delta-Net layer hands it over: permuted views, v with unaligned rows
    packed = torch.cat((q, k, v, beta), -1).permute(2, 0, 1, 3).contiguous()
    qs, ks, vs, bs = (t.permute(1, 2, 0, 3) for t in packed.split((D, D, D, 1), -1))
    W1, W2 = W0.clone(), W0.clone()
    assert torch.equal(f(qs, ks, vs, bs, W1), fwp.DeltaFastWeight.apply(q, k, v, beta, W2))
    assert torch.equal(W1, W2)
    # only v wants a gradient
    vr = v.clone().requires_grad_(True)
    out = f(q, k, vr, beta, W0.clone())
    (gv,) = torch.autograd.grad(out, vr, go)
    vr2 = v.clone().requires_grad_(True)
    (gv2,) = torch.autograd.grad(fwp.DeltaFastWeight.apply(q, k, vr2, beta, W0.clone()), vr2, go)
    assert torch.equal(gv, gv2)
    with torch.no_grad():
        assert not f(q.requires_grad_(True), k, v, beta, W0.clone()).requires_grad
    with pytest.raises(fwp._lib.FwpError, match="shape mismatch"):
        f(q, k[:, :, :-1], v, beta, W0.clone())
    with pytest.raises(fwp._lib.FwpError, match="W must be"):
        f(q, k, v, beta, W0.clone().transpose(2, 3))


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["reference", "exact"])
@pytest.mark.parametrize("N,H,L,E,M", [(2, 2, 64, 16, 16), (3, 5, 11, 200, 7), (1, 2, 130, 32, 32)])
def test_sum_rule_same_as_python_function(fwp, mode, N, H, L, E, M):
    q, k, v, _, W0, go = (torch.from_numpy(a).cuda() for a in delta_inputs(7, N, H, L, E, M, dtype=np.float32))
    assert fwp.fast_weight_sum is not fwp.FastWeightSum.apply
    fwp.FastWeightSum.state_gradient = mode
    try:
        results = []
        for f in (fwp.fast_weight_sum, fwp.FastWeightSum.apply):
            ins = [t.clone().requires_grad_(True) for t in (q, k, v)]
            W = W0.clone()
            out = f(*ins, W)
            results.append([out, W, *torch.autograd.grad(out, ins, go)])
        for a, b in zip(*results):
            assert torch.equal(a, b)
        fwp.FastWeightSum.state_gradient = "something else"
        with pytest.raises(fwp._lib.FwpError, match="state_gradient"):
            fwp.fast_weight_sum(q, k, v, W0.clone())
    finally:
        fwp.FastWeightSum.state_gradient = "reference"


@pytest.mark.gpu
@pytest.mark.parametrize("N,H,L,D", [(2, 2, 64, 32), (1, 3, 37, 16), (2, 1, 1, 32), (1, 2, 20, 40)])
def test_delta_rnn_same_as_python_function(fwp, N, H, L, D):
    from helpers import rnn_inputs
    z, k, v, W0, beta, h0, go = (torch.from_numpy(a).cuda() for a in rnn_inputs(21, N, H, L, D, dtype=np.float32, w0=True))
    assert importlib.import_module(fwp.__name__ + ".fast_weight_rnn_v2")._operator is native(fwp).fast_rnn_v2
    results = []
    for f in (fwp.fast_rnn_v2, fwp.FastRNNv2.apply):
        ins = [t.clone().requires_grad_(True) for t in (z, k, v, beta)]
        W, h = W0.clone(), h0.clone()
        out = f(ins[0], ins[1], ins[2], W, ins[3], h)
        results.append([out, W, h, *torch.autograd.grad(out, ins, go)])
    for a, b in zip(*results):
        assert torch.equal(a, b)
    with pytest.raises(AssertionError):
        fwp.fast_rnn_v2(z, k[:, :, :-1], v, W0.clone(), beta, h0.clone())


@pytest.mark.gpu
@pytest.mark.parametrize("N,H,L,D", [(2, 2, 64, 32), (1, 3, 37, 16), (2, 1, 1, 32), (1, 2, 20, 40)])
def test_recurrent_delta_net_same_as_python_function(fwp, N, H, L, D):
    from helpers import rec_inputs
    arrays = [torch.from_numpy(a).cuda() for a in rec_inputs(22, N, H, L, D, dtype=np.float32, w0=True)]
    diff, W0, h0, go = arrays[:8], arrays[8], arrays[9], arrays[10]
    assert importlib.import_module(fwp.__name__ + ".rec_update_fwm_tanh")._operator is native(fwp).rec_update_fwm_tanh
    results = []
    for f in (fwp.rec_update_fwm_tanh, fwp.FastWeightRecUpdateTanh.apply):
        ins = [t.clone().requires_grad_(True) for t in diff]
        W, h = W0.clone(), h0.clone()
        out = f(*ins, W, h)
        results.append([out, W, h, *torch.autograd.grad(out, ins, go)])
    for a, b in zip(*results):
        assert torch.equal(a, b)
    with pytest.raises(AssertionError, match="Reshape"):
        fwp.rec_update_fwm_tanh(*diff[:4], diff[4][0], *diff[5:], W0.clone(), h0.clone())


@pytest.mark.gpu
@pytest.mark.parametrize("N,H,L,D", [(2, 2, 64, 32), (1, 2, 24, 16), (2, 1, 1, 32), (1, 2, 11, 36)])
def test_delta_lstm_same_as_python_function(fwp, N, H, L, D):
    from helpers import lstm_inputs
    Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(23, N, H, L, D, dtype=np.float32, w0=True)
    cu = lambda a: torch.from_numpy(a).cuda()
    assert importlib.import_module(fwp.__name__ + ".fast_lstm_v4")._operator is native(fwp).fast_lstm_v4
    results = []
    for f in (fwp.fast_lstm_v4, fwp.FastLSTMv4.apply):
        ins, args, states = [], [], []
        for g in range(3):
            quad = [cu(x[g]).requires_grad_(True) for x in (Zs, Ks, Vs, Bs)]
            W = cu(Ws[g]).clone()
            ins += quad
            states.append(W)
            args += [*quad, W]
        h, c = cu(h0).clone(), cu(c0).clone()
        out, cell = f(*args, h, c)
        assert not cell.requires_grad
        results.append([out, cell, h, c, *states, *torch.autograd.grad(out, ins, cu(go))])
    for a, b in zip(*results):
        assert torch.equal(a, b)
    with pytest.raises(fwp._lib.FwpError, match="h0 and c0"):
        fwp.fast_lstm_v4(*args, h[:, :, 0], c)


@pytest.mark.gpu
@pytest.mark.parametrize("N,H,L,E,M", [(2, 2, 37, 32, 97), (2, 2, 70, 32, 128), (1, 2, 50, 128, 64), (1, 2, 1, 32, 97)])
@pytest.mark.parametrize("time_major", [None, True])
def test_slices_of_value_columns_cut_in_cpp_and_in_python_agree(fwp, N, H, L, E, M, time_major):
    """Value widths that no kernel takes whole: the C++ function cuts them into slices inside one graph node,
    the Python path (what runs without the C++ function) makes one call of the autograd Function per slice.
    Same kernels on the same slices; the sums over the slices (gradients of Q, K, beta) may be taken in
    another order, so those are held to 1e-6 relative to the tensor's scale instead of bit for bit."""
    fw = importlib.import_module(fwp.__name__ + ".fast_weight")
    q, k, v, beta, W0, go = (torch.from_numpy(a).cuda() for a in delta_inputs(9, N, H, L, E, M, dtype=np.float32, w0=True))
    results = []
    for f in (native(fwp).fast_weight_delta, fw.fast_weight_delta_sliced):
        ins = [t.clone().requires_grad_(True) for t in (q, k, v, beta)]
        W = W0.clone()
        out = f(*ins, W) if time_major is None else f(*ins, W, time_major)
        grads = torch.autograd.grad(out, ins, go)
        results.append([out, W, *grads])
    names = ("out", "W", "gq", "gk", "gv", "gbeta")
    for name, a, b in zip(names, *results):
        assert a.shape == b.shape, name
        if name in ("out", "W", "gv"):
            assert torch.equal(a, b), name
        else:
            assert float((a - b).abs().max()) <= 1e-6 * float(b.abs().max()), name
    a, b = results[0][0], results[1][0]      # the same memory order (a stride of an axis of one element says nothing)
    assert [s for s, n in zip(a.stride(), a.shape) if n > 1] == [s for s, n in zip(b.stride(), b.shape) if n > 1]
