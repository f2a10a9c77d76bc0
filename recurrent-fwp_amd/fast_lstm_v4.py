"""Delta LSTM v4 (three recurrent fast weight memories gating an LSTM cell): drop-in for the
reference's ``fast_lstm_v4`` package (language_modeling/src/utils/fast_lstm_v4/__init__.py:36-208)."""
import ctypes

import torch

from . import _lib, _padding
from .fast_weight import _fwp_torch, _nchunk


def _views(ts):
    return (_lib.View * 3)(*[t[1] for t in ts])


class FastLSTMv4(torch.autograd.Function):
    """``rnn_out, cell_out = fast_lstm_v4(Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0)``.

    Per gate g in (i, u, o): Z, K, V ``[N,H,L,D]``, beta ``[N,H,L,1]``, W ``[N,H,D,D]``;
    h0, c0 ``[N,H,1,D]``.  The W, h0 and c0 are in/out: on return they hold the memories,
    the output and the cell after the last step.  Per step every memory takes a delta-rule
    write of its (K, V, beta), then with ``s = softmax(h_{t-1})``:
    ``i = sigmoid(W_i^T s + z_i)``, ``u = W_u^T s + z_u``, ``o = sigmoid(W_o^T s + z_o)``,
    ``c_t = i u + (1 - i) c_{t-1}``, ``h_t = o c_t``.
    Gradients flow to the twelve Z, K, V, beta from ``rnn_out`` only; a gradient arriving
    on ``cell_out`` is ignored, as in the reference (:128).
    """

    @staticmethod
    def forward(ctx, Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0):
        _lib.require_device(Zi)
        _lib.same_device(Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0)
        N, H, L, _ = Zi.shape
        D = Vi.shape[-1]
        Zs, Ks, Vs, Bs, Ws = (Zi, Zu, Zo), (Ki, Ku, Ko), (Vi, Vu, Vo), (bi, bu, bo), (Wi, Wu, Wo)
        for a in range(3):
            if not (Zs[a].shape == Ks[a].shape == Vs[a].shape == (N, H, L, D)
                    and Bs[a].shape == (N, H, L, 1) and Ws[a].shape == (N, H, D, D)):
                raise _lib.FwpError("shape mismatch between the gates' Z, K, V [N,H,L,D], beta "
                                    "[N,H,L,1] and W [N,H,D,D]")
        if h0.shape != (N, H, 1, D) or c0.shape != (N, H, 1, D):
            raise _lib.FwpError("h0 and c0 must be [N,H,1,D]")
        for name, t in (("Wi", Wi), ("Wu", Wu), ("Wo", Wo), ("h0", h0), ("c0", c0)):
            if not t.is_contiguous() or t.dtype != torch.float32:
                raise _lib.FwpError(f"{name} must be a contiguous fp32 tensor")
        Zr, Kr, Vr, Br = ([_lib.rows(t) for t in ts] for ts in (Zs, Ks, Vs, Bs))
        need_grad = any(ctx.needs_input_grad)
        chunk = _lib.query(_lib.Q_DEFAULT_CHUNK)
        dev = Zi.device
        f32 = dict(device=dev, dtype=torch.float32)
        out = torch.empty((N, H, L, D), **f32)
        cell = torch.empty((N, H, L, D), **f32)
        gates = vdiff = ckpt = h_init = c_init = None
        if need_grad:
            h_init, c_init = h0.detach().clone(), c0.detach().clone()
            gates = torch.empty((3, N, H, L, D), **f32)
            vdiff = torch.empty((3, N, H, L, D), **f32)
            ckpt = torch.empty((3, N, H, _nchunk(L, chunk), D, D), **f32)
        Wp = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in Ws])
        with _lib.on_device(dev):
            rc = _lib.lib().fwp_lstm_fwd(
                _views(Zr), _views(Kr), _views(Vr), _views(Br), Wp, _lib.ptr(h0), _lib.ptr(c0),
                _lib.ptr(out), _lib.ptr(cell), _lib.ptr(gates) if need_grad else None,
                _lib.ptr(vdiff) if need_grad else None, _lib.ptr(ckpt) if need_grad else None,
                N, H, L, D, chunk, _lib.stream_of(Zi))
        _lib.check(rc, "fwp_lstm_fwd")
        if need_grad:
            ctx.save_for_backward(*[t[0] for t in Kr], *[t[0] for t in Br], vdiff, gates, out, cell,
                                  h_init, c_init, ckpt)
            ctx.dims = (N, H, L, D, chunk)
        ctx.mark_non_differentiable(cell)
        ctx.set_materialize_grads(False)
        return out, cell

    @staticmethod
    def backward(ctx, grad_out, grad_cell):
        if grad_out is None:
            return (None,) * 17
        (Ki, Ku, Ko, bi, bu, bo, vdiff, gates, out, cell, h_init, c_init, ckpt) = ctx.saved_tensors
        N, H, L, D, chunk = ctx.dims
        Kr = [_lib.rows(t) for t in (Ki, Ku, Ko)]
        Br = [_lib.rows(t) for t in (bi, bu, bo)]
        grad_out, gov = _lib.rows(grad_out)
        f32 = dict(device=out.device, dtype=torch.float32)
        gz, gk, gv = (torch.empty((3, N, H, L, D), **f32) for _ in range(3))
        gb = torch.empty((3, N, H, L, 1), **f32)
        with _lib.on_device(out.device):
            rc = _lib.lib().fwp_lstm_bwd(
                _views(Kr), _views(Br), _lib.ptr(vdiff), _lib.ptr(gates), _lib.ptr(out),
                _lib.ptr(cell), _lib.ptr(h_init), _lib.ptr(c_init), gov, _lib.ptr(ckpt),
                _lib.ptr(gz), _lib.ptr(gk), _lib.ptr(gv), _lib.ptr(gb), N, H, L, D, chunk,
                _lib.stream_of(out))
        _lib.check(rc, "fwp_lstm_bwd")
        res = []
        for a in range(3):
            res += [gz[a], gk[a], gv[a], gb[a], None]
        return (*res, None, None)


# the same operator as a C++ autograd function (csrc/fwp_torch.cpp) when that has been built
_operator = _fwp_torch.fast_lstm_v4 if _fwp_torch is not None else FastLSTMv4.apply


def fast_lstm_v4(Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0):
    """``rnn_out, cell_out = fast_lstm_v4(Zi, Ki, Vi, bi, Wi, Zu, ..., Wo, h0, c0)``, the reference's
    operator (language_modeling/src/utils/fast_lstm_v4/__init__.py:208).  A head size below 32 that is
    not 16 runs on the kernels of the next of the two.  The padded entries of h must be -BIG for the
    softmax to give them exactly zero (see _padding.py): h0 is padded with -BIG, Zi and Zo with +BIG (both
    gates exactly one) and Zu with -BIG, so that every later c = i u + (1 - i) c and h = o c of a padded
    entry is -BIG again; K, V, W and c0 are padded with zeros.  The states come back in W, h0, c0."""
    args = (Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0)
    D = Vi.shape[-1] if Vi.dim() == 4 else 0
    width = _padding.padded_width(D)
    if width is None or Zi.dim() != 4:
        return _operator(*args)
    N, H, L, _ = Zi.shape
    gates = ((Zi, Ki, Vi, bi, Wi), (Zu, Ku, Vu, bu, Wu), (Zo, Ko, Vo, bo, Wo))
    for Z, K, V, b, W in gates:
        if not (Z.shape == K.shape == V.shape == (N, H, L, D) and b.shape == (N, H, L, 1)
                and _padding.state_ok(W, (N, H, D, D))):
            return _operator(*args)      # raises what the operator raises for these
    if not (_padding.state_ok(h0, (N, H, 1, D)) and _padding.state_ok(c0, (N, H, 1, D))):
        return _operator(*args)
    n = width - D
    padded, states = [], []
    for (Z, K, V, b, W), z_fill in zip(gates, (_padding.BIG, -_padding.BIG, _padding.BIG)):
        Wp = _padding.square(W.detach(), n)
        states.append(Wp)
        padded += [_padding.last(Z, n, z_fill), _padding.last(K, n), _padding.last(V, n), b, Wp]
    hp, cp = _padding.last(h0.detach(), n, -_padding.BIG), _padding.last(c0.detach(), n)
    out, cell = _operator(*padded, hp, cp)
    with torch.no_grad():
        for (_, _, _, _, W), Wp in zip(gates, states):
            W.copy_(Wp[:, :, :D, :D])
        h0.copy_(hp[..., :D])
        c0.copy_(cp[..., :D])
    return out[..., :D], cell[..., :D]
