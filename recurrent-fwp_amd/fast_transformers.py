"""Sum update rule (causal linear attention): drop-in for the reference's
``fast_transformers`` package (algorithmic/fast_transformers/__init__.py:25-84; the
language-modelling and RL copies are identical)."""
import torch

from . import _lib
from .fast_weight import _fwp_torch, _nchunk, pick_width


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


_operator = _native_sum if _fwp_torch is not None else FastWeightSum.apply

# Value widths the blocked kernels take for a given key width, and those the single-step kernels take.
_FAST_WIDTHS = {16: (16, 32, 64, 128), 32: (16, 32, 64, 128), 64: (16, 32, 64, 128), 96: (16, 32),
                128: (16, 32, 64), 192: (16, 32)}
_STEP_WIDTHS = (16, 32, 64, 128)
_plans = {}


def sum_plan(E, M):
    """How a state of E x M is run when no fast kernel takes it whole: ``None`` (as it is), or
    ``(keys, slices)``: the keys zero padded to ``keys`` features and value columns [first, last) run as a
    state of keys x width for every ``(first, last, width)`` of ``slices``.  Both are exact for the sum rule:
    a column of ``W += k (x) v`` and of ``out = W^T q`` depends on that column of V and W only
    (causal_product_cuda.cu:15-96), the gradients of Q and K are sums over the columns, and a key feature
    that is zero in q and k adds nothing to any of them."""
    key = (E, M)
    if key not in _plans:
        keys = next((w for w in sorted(_FAST_WIDTHS) if w >= E), None)
        plan = None
        if keys is not None and not (keys == E and M in _FAST_WIDTHS[keys]):
            widths, slices, first = _FAST_WIDTHS[keys], [], 0
            while first < M:
                left = M - first
                width = pick_width(widths, left)
                last = min(M, first + width)
                slices.append((first, last, width))
                first = last
            plan = (keys, slices)
        _plans[key] = plan
    return _plans[key]


def fast_weight_sum(Q, K, V, W):
    """``out = fast_weight_sum(Q, K, V, W)``, the reference's operator
    (algorithmic/fast_transformers/__init__.py:84).  State shapes no blocked kernel takes whole (keys and values of 128, values of
    64 with keys of 96, widths that are not multiples of 16)
    run on them by slices of value columns with zero padded keys, see :func:`sum_plan`."""
    try:        # the common case first: a width pair seen before
        plan = _plans[(Q.size(-1), V.size(-1))]
    except (KeyError, IndexError):
        plan = sum_plan(Q.shape[-1], V.shape[-1]) if Q.dim() == 4 and V.dim() == 4 else None
    if plan is not None and Q.shape[2] == 1 and Q.shape[-1] in _FAST_WIDTHS and Q.shape[-1] <= 128 and \
            V.shape[-1] in _STEP_WIDTHS and not (torch.is_grad_enabled() and any(t.requires_grad for t in (Q, K, V))):
        plan = None     # a single step that saves nothing: the single-step kernels take these widths whole
    if plan is None:
        return _operator(Q, K, V, W)
    N, H, L, E = Q.shape
    M = V.shape[-1]
    # the checks the whole-state path makes on the caller's W, which the slices would hide from it
    if K.shape != Q.shape or V.shape[:3] != Q.shape[:3]:
        raise _lib.FwpError(f"shape mismatch: Q{tuple(Q.shape)} K{tuple(K.shape)} V{tuple(V.shape)}")
    if W.shape != (N, H, E, M) or not W.is_contiguous() or W.dtype != torch.float32:
        raise _lib.FwpError("W must be a contiguous fp32 [N,H,E,M] tensor")
    _lib.same_device(Q, K, V, W)
    keys, slices = plan
    pad = torch.nn.functional.pad
    if keys > E:
        Q, K = pad(Q, (0, keys - E)), pad(K, (0, keys - E))
    outs, states = [], []
    for first, last, width in slices:
        extra = width - (last - first)
        Vs = V[..., first:last]
        Ws = pad(W.detach()[..., first:last], (0, extra, 0, keys - E))      # a copy, contiguous
        if extra:
            Vs = pad(Vs, (0, extra))
        out = _operator(Q, K, Vs, Ws)
        states.append(Ws)
        outs.append(out[..., :last - first] if extra else out)
    # the state after the last step, in place, once every slice has run: a rejected slice leaves W as it was
    with torch.no_grad():
        for (first, last, _), Ws in zip(slices, states):
            W[..., first:last] = Ws[:, :, :E, :last - first]
    return torch.cat(outs, -1) if len(outs) > 1 else outs[0]
