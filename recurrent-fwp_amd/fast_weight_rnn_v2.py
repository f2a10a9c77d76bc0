"""Delta RNN v2 (recurrent fast weight): drop-in for the reference's
``fast_weight_rnn_v2`` package (algorithmic/fast_weight_rnn_v2/__init__.py:29-121)."""
import torch

from . import _lib, _padding
from .fast_weight import _fwp_torch, _nchunk


class FastRNNv2(torch.autograd.Function):
    """``rnn_out = fast_rnn_v2(Z, K, V, W, beta, h0)`` -- note the argument order.

    Z, K, V ``[N,H,L,D]``; beta ``[N,H,L,1]``; W ``[N,H,D,D]`` and h0 ``[N,H,1,D]`` are
    in/out: on return they hold the state and the output after the last step.
    Per step: W takes a delta-rule write of (K, V, beta), then
    ``h_t = W_t^T softmax(h_{t-1}) + z_t``.  Gradients flow to Z, K, V and beta.
    """

    @staticmethod
    def forward(ctx, Z, K, V, W, beta, h0):
        _lib.require_device(Z)
        _lib.same_device(Z, K, V, W, beta, h0)
        N, H, L, _ = Z.shape
        D = V.shape[-1]
        # same preconditions as the reference (:54-57)
        assert Z.shape == (N, H, L, D)
        assert K.shape == (N, H, L, D)
        assert V.shape == (N, H, L, D)
        assert beta.shape == (N, H, L, 1)
        assert h0.shape == (N, H, 1, D)
        assert W.shape == (N, H, D, D)
        for name, t in (("W", W), ("h0", h0)):
            if not t.is_contiguous() or t.dtype != torch.float32:
                raise _lib.FwpError(f"{name} must be a contiguous fp32 tensor")
        Z, zv = _lib.rows(Z)
        K, kv = _lib.rows(K)
        V, vv = _lib.rows(V)
        beta, bv = _lib.rows(beta)
        need_grad = any(ctx.needs_input_grad)
        chunk = _lib.query(_lib.Q_DEFAULT_CHUNK)
        dev = Z.device
        out = torch.empty((N, H, L, D), device=dev, dtype=torch.float32)
        vdiff = ckpt = h_init = None
        if need_grad:
            h_init = h0.detach().clone()
            vdiff = torch.empty((N, H, L, D), device=dev, dtype=torch.float32)
            ckpt = torch.empty((N, H, _nchunk(L, chunk), D, D), device=dev, dtype=torch.float32)
        with _lib.on_device(dev):
            rc = _lib.lib().fwp_rnn_fwd(
                zv, kv, vv, bv, _lib.ptr(W), _lib.ptr(h0), _lib.ptr(out),
                _lib.ptr(vdiff) if need_grad else None, _lib.ptr(ckpt) if need_grad else None,
                N, H, L, D, chunk, _lib.stream_of(Z))
        _lib.check(rc, "fwp_rnn_fwd")
        if need_grad:
            ctx.save_for_backward(K, beta, vdiff, out, h_init, ckpt)
            ctx.dims = (N, H, L, D, chunk)
        ctx.set_materialize_grads(False)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        if grad_out is None:
            return None, None, None, None, None, None
        K, beta, vdiff, out, h_init, ckpt = ctx.saved_tensors
        N, H, L, D, chunk = ctx.dims
        _, kv = _lib.rows(K)
        _, bv = _lib.rows(beta)
        grad_out, gv_ = _lib.rows(grad_out)
        dev = K.device
        grad_Z, grad_K, grad_V = (torch.empty((N, H, L, D), device=dev, dtype=torch.float32)
                                  for _ in range(3))
        grad_beta = torch.empty((N, H, L, 1), device=dev, dtype=torch.float32)
        with _lib.on_device(dev):
            rc = _lib.lib().fwp_rnn_bwd(
                kv, bv, _lib.ptr(vdiff), _lib.ptr(out), _lib.ptr(h_init), gv_, _lib.ptr(ckpt),
                _lib.ptr(grad_Z), _lib.ptr(grad_K), _lib.ptr(grad_V), _lib.ptr(grad_beta),
                N, H, L, D, chunk, _lib.stream_of(K))
        _lib.check(rc, "fwp_rnn_bwd")
        return grad_Z, grad_K, grad_V, None, grad_beta, None


# the same operator as a C++ autograd function (csrc/fwp_torch.cpp) when that has been built
_operator = _fwp_torch.fast_rnn_v2 if _fwp_torch is not None else FastRNNv2.apply


def fast_rnn_v2(Z, K, V, W, beta, h0):
    """``rnn_out = fast_rnn_v2(Z, K, V, W, beta, h0)``, the reference's operator
    (algorithmic/fast_weight_rnn_v2/__init__.py:121).  A head size below 32 that is not 16 runs on the
    kernels of the next of the two: K, V and W zero padded, Z and h0 padded with -BIG, so that the padded
    entries of softmax(h) are exactly zero (see _padding.py); W and h0 take the states back."""
    D = V.shape[-1] if V.dim() == 4 else 0
    width = _padding.padded_width(D)
    if width is None or Z.dim() != 4:
        return _operator(Z, K, V, W, beta, h0)
    N, H, L, _ = Z.shape
    if not (Z.shape == K.shape == V.shape and beta.shape == (N, H, L, 1) and _padding.state_ok(W, (N, H, D, D))
            and _padding.state_ok(h0, (N, H, 1, D))):
        return _operator(Z, K, V, W, beta, h0)      # raises what the operator raises for these
    n = width - D
    Wp, hp = _padding.square(W.detach(), n), _padding.last(h0.detach(), n, -_padding.BIG)
    out = _operator(_padding.last(Z, n, -_padding.BIG), _padding.last(K, n), _padding.last(V, n), Wp, beta, hp)
    with torch.no_grad():
        W.copy_(Wp[:, :, :D, :D])
        h0.copy_(hp[..., :D])
    return out[..., :D]
