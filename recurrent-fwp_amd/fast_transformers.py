"""Sum update rule (causal linear attention): drop-in for the reference's
``fast_transformers`` package (algorithmic/fast_transformers/__init__.py:25-84; the
language-modelling and RL copies are identical)."""
import torch

from . import _lib
from .fast_weight import _fwp_torch, _nchunk


class FastWeightSum(torch.autograd.Function):
    """``out = fast_weight_sum(Q, K, V, W)``: per step ``W += k (x) v``, ``out = W^T q``.

    Q, K ``[N,H,L,E]``; V ``[N,H,L,M]``; W ``[N,H,E,M]`` is the carried-in state on entry
    and the state after the last step on return.  Gradients flow to Q, K and V.

    ``state_gradient`` selects what grad_Q makes of a non-zero carried-in state:
    ``"reference"`` (default) leaves it out, as the reference's backward does
    (causal_product_cuda.cu:385 starts its accumulator at zero); ``"exact"`` is the
    gradient of the recurrence as written.  They agree whenever W enters as zeros.
    """

    state_gradient = "reference"

    @staticmethod
    def forward(ctx, Q, K, V, W):
        _lib.require_device(Q)
        _lib.same_device(Q, K, V, W)
        N, H, L, E = Q.shape
        M = V.shape[-1]
        if K.shape != (N, H, L, E) or V.shape != (N, H, L, M):
            raise _lib.FwpError(f"shape mismatch: Q{tuple(Q.shape)} K{tuple(K.shape)} V{tuple(V.shape)}")
        if W.shape != (N, H, E, M) or not W.is_contiguous() or W.dtype != torch.float32:
            raise _lib.FwpError("W must be a contiguous fp32 [N,H,E,M] tensor")
        if FastWeightSum.state_gradient not in ("reference", "exact"):
            raise _lib.FwpError("FastWeightSum.state_gradient must be 'reference' or 'exact'")
        Q, qv = _lib.rows(Q)
        K, kv = _lib.rows(K)
        V, vv = _lib.rows(V)
        need_grad = any(ctx.needs_input_grad[:3])
        chunk = _lib.query(_lib.Q_DEFAULT_CHUNK)
        out = torch.empty((N, H, L, M), device=Q.device, dtype=torch.float32)
        ckpt = W_init = None
        if need_grad:
            ckpt = torch.empty((N, H, _nchunk(L, chunk), E, M), device=Q.device, dtype=torch.float32)
            if FastWeightSum.state_gradient == "reference":
                W_init = W.clone()
        with _lib.on_device(Q):
            rc = _lib.lib().fwp_sum_fwd(qv, kv, vv, _lib.ptr(W), _lib.ptr(out),
                                        _lib.ptr(ckpt) if need_grad else None,
                                        N, H, L, E, M, chunk, _lib.stream_of(Q))
        _lib.check(rc, "fwp_sum_fwd")
        if need_grad:
            ctx.save_for_backward(Q, K, V, ckpt, *([W_init] if W_init is not None else []))
            ctx.dims = (N, H, L, E, M, chunk)
        ctx.set_materialize_grads(False)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        if grad_out is None:
            return None, None, None, None
        Q, K, V, ckpt, *rest = ctx.saved_tensors
        N, H, L, E, M, chunk = ctx.dims
        _, qv = _lib.rows(Q)
        _, kv = _lib.rows(K)
        _, vv = _lib.rows(V)
        grad_out, gv_ = _lib.rows(grad_out)
        grad_Q = torch.empty((N, H, L, E), device=Q.device, dtype=torch.float32)
        grad_K = torch.empty((N, H, L, E), device=Q.device, dtype=torch.float32)
        grad_V = torch.empty((N, H, L, M), device=Q.device, dtype=torch.float32)
        with _lib.on_device(Q):
            rc = _lib.lib().fwp_sum_bwd(qv, kv, vv, gv_, _lib.ptr(ckpt),
                                        _lib.ptr(rest[0]) if rest else None, _lib.ptr(grad_Q),
                                        _lib.ptr(grad_K), _lib.ptr(grad_V), N, H, L, E, M, chunk,
                                        _lib.stream_of(Q))
        _lib.check(rc, "fwp_sum_bwd")
        return grad_Q, grad_K, grad_V, None


def _native_sum(Q, K, V, W):
    """The same operator as a C++ autograd function (csrc/fwp_torch.cpp)."""
    mode = FastWeightSum.state_gradient
    if mode != "reference" and mode != "exact":
        raise _lib.FwpError("FastWeightSum.state_gradient must be 'reference' or 'exact'")
    return _fwp_torch.fast_weight_sum(Q, K, V, W, mode == "exact")


fast_weight_sum = _native_sum if _fwp_torch is not None else FastWeightSum.apply
