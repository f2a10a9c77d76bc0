"""Recurrent Delta Net update with tanh feedback: drop-in for the reference's
``rec_update_fwm_tanh`` package (algorithmic/rec_update_fwm_tanh/__init__.py:31-139)."""
import torch

from . import _lib, _padding
from .fast_weight import _fwp_torch, _nchunk


class FastWeightRecUpdateTanh(torch.autograd.Function):
    """``out = rec_update_fwm_tanh(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0)``.

    qx, kx, vx ``[N,H,L,D]`` and bx ``[N,H,L,1]`` are pre-activation; R_q, R_k, R_v
    ``[1,H,D,D]`` (indexed ``[e_in][m_out]``) and r_b ``[1,H,1,D]`` feed
    ``tanh(out_{t-1})`` back into them; softmax on q and k and sigmoid on beta are
    applied inside.  W ``[N,H,D,D]`` and h0 ``[N,H,1,D]`` are in/out states.
    Gradients flow to the first eight arguments.
    """

    @staticmethod
    def forward(ctx, qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0):
        _lib.require_device(qx)
        _lib.same_device(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0)
        N, H, L, E = qx.shape
        M = vx.shape[-1]
        # same preconditions as the reference (:52-56)
        assert E == M, "Current kernel only support this case."
        assert R_q.shape == (1, H, M, M), "Reshape/unsqueeze if needed."
        assert R_k.shape == (1, H, M, M), "Reshape/unsqueeze if needed."
        assert R_v.shape == (1, H, M, M), "Reshape/unsqueeze if needed."
        assert r_b.shape == (1, H, 1, M), "Reshape/unsqueeze if needed."
        assert kx.shape == (N, H, L, M) and vx.shape == (N, H, L, M) and bx.shape == (N, H, L, 1)
        assert W.shape == (N, H, M, M) and h0.shape == (N, H, 1, M)
        for name, t in (("W", W), ("h0", h0)):
            if not t.is_contiguous() or t.dtype != torch.float32:
                raise _lib.FwpError(f"{name} must be a contiguous fp32 tensor")
        D = M
        qx, qv = _lib.rows(qx)
        kx, kv = _lib.rows(kx)
        vx, vv = _lib.rows(vx)
        bx, bv = _lib.rows(bx)
        Rq, Rk, Rv, rb = (t.detach().contiguous().float() for t in (R_q, R_k, R_v, r_b))
        need_grad = any(ctx.needs_input_grad)
        chunk = _lib.query(_lib.Q_DEFAULT_CHUNK)
        dev = qx.device
        out = torch.empty((N, H, L, D), device=dev, dtype=torch.float32)
        saved = [None] * 5
        h_init = None
        if need_grad:
            h_init = h0.detach().clone()
            saved = [torch.empty((N, H, L, D), device=dev, dtype=torch.float32),   # q after softmax
                     torch.empty((N, H, L, D), device=dev, dtype=torch.float32),   # k after softmax
                     torch.empty((N, H, L), device=dev, dtype=torch.float32),      # beta after sigmoid
                     torch.empty((N, H, L, D), device=dev, dtype=torch.float32),   # v - v_old
                     torch.empty((N, H, _nchunk(L, chunk), D, D), device=dev, dtype=torch.float32)]
        with _lib.on_device(dev):
            rc = _lib.lib().fwp_rec_fwd(
                qv, kv, vv, bv, _lib.ptr(Rq), _lib.ptr(Rk), _lib.ptr(Rv), _lib.ptr(rb),
                _lib.ptr(W), _lib.ptr(h0), _lib.ptr(out),
                *[(_lib.ptr(t) if t is not None else None) for t in saved],
                N, H, L, D, chunk, _lib.stream_of(qx))
        _lib.check(rc, "fwp_rec_fwd")
        if need_grad:
            ctx.save_for_backward(out, h_init, Rq, Rk, Rv, rb, *saved)
            ctx.dims = (N, H, L, D, chunk)
        ctx.set_materialize_grads(False)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        if grad_out is None:
            return (None,) * 10
        out, h_init, Rq, Rk, Rv, rb, q_act, k_act, beta_act, vdiff, ckpt = ctx.saved_tensors
        N, H, L, D, chunk = ctx.dims
        grad_out, gv_ = _lib.rows(grad_out)
        dev = out.device
        grad_qx, grad_kx, grad_vx = (torch.empty((N, H, L, D), device=dev, dtype=torch.float32)
                                     for _ in range(3))
        grad_bx = torch.empty((N, H, L, 1), device=dev, dtype=torch.float32)
        grad_R_q, grad_R_k, grad_R_v = (torch.empty((1, H, D, D), device=dev, dtype=torch.float32)
                                        for _ in range(3))
        grad_r_b = torch.empty((1, H, 1, D), device=dev, dtype=torch.float32)
        workspace = torch.empty((N, H, 3 * D * D + D), device=dev, dtype=torch.float32)
        with _lib.on_device(dev):
            rc = _lib.lib().fwp_rec_bwd(
                _lib.ptr(q_act), _lib.ptr(k_act), _lib.ptr(beta_act), _lib.ptr(vdiff),
                _lib.ptr(out), _lib.ptr(h_init), gv_, _lib.ptr(Rq), _lib.ptr(Rk), _lib.ptr(Rv),
                _lib.ptr(rb), _lib.ptr(ckpt), _lib.ptr(grad_qx), _lib.ptr(grad_kx),
                _lib.ptr(grad_vx), _lib.ptr(grad_bx), _lib.ptr(grad_R_q), _lib.ptr(grad_R_k),
                _lib.ptr(grad_R_v), _lib.ptr(grad_r_b), _lib.ptr(workspace),
                N, H, L, D, chunk, _lib.stream_of(out))
        _lib.check(rc, "fwp_rec_bwd")
        return (grad_qx, grad_kx, grad_vx, grad_bx,
                grad_R_q, grad_R_k, grad_R_v, grad_r_b, None, None)


# the same operator as a C++ autograd function (csrc/fwp_torch.cpp) when that has been built
_operator = _fwp_torch.rec_update_fwm_tanh if _fwp_torch is not None else FastWeightRecUpdateTanh.apply


def rec_update_fwm_tanh(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0):
    """``out = rec_update_fwm_tanh(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0)``, the reference's operator
    (algorithmic/rec_update_fwm_tanh/__init__.py:139).  A head size below 32 that is not 16 runs on the
    kernels of the next of the two: qx and kx padded with -BIG, so that the padded entries of the two
    softmaxes are exactly zero (see _padding.py), everything else with zeros; W and h0 take the states back."""
    args = (qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0)
    D = vx.shape[-1] if vx.dim() == 4 else 0
    width = _padding.padded_width(D)
    if width is None or qx.dim() != 4:
        return _operator(*args)
    N, H, L, _ = qx.shape
    if not (qx.shape == kx.shape == vx.shape == (N, H, L, D) and bx.shape == (N, H, L, 1)
            and R_q.shape == R_k.shape == R_v.shape == (1, H, D, D) and r_b.shape == (1, H, 1, D)
            and _padding.state_ok(W, (N, H, D, D)) and _padding.state_ok(h0, (N, H, 1, D))):
        return _operator(*args)      # raises what the operator raises for these
    n = width - D
    Wp, hp = _padding.square(W.detach(), n), _padding.last(h0.detach(), n)
    out = _operator(_padding.last(qx, n, -_padding.BIG), _padding.last(kx, n, -_padding.BIG), _padding.last(vx, n),
                    bx, _padding.square(R_q, n), _padding.square(R_k, n), _padding.square(R_v, n),
                    _padding.last(r_b, n), Wp, hp)
    with torch.no_grad():
        W.copy_(Wp[:, :, :D, :D])
        h0.copy_(hp[..., :D])
    return out[..., :D]
