"""Delta-rule fast weight memory: drop-in for the reference's ``fast_weight``
package (algorithmic/fast_weight/__init__.py:26-96; the language-modelling copy
is ``utils.fast_fast_weight``)."""
import torch

from . import _lib


def _nchunk(L, chunk):
    return (L + chunk - 1) // chunk


def rows_lead(t):
    """Is this 4-D [N,H,L,D] tensor a view of storage laid out [L,N,H,...] (the steps outermost), as
    the reference's layers hand their inputs over (permuted views of a [len, bsz, ...] projection)?"""
    N, H, L, _ = t.shape
    sN, sH, sL, _ = t.stride()
    others = ([sN] if N > 1 else []) + ([sH] if H > 1 else [])
    return L > 1 and bool(others) and all(sL > s for s in others)


class DeltaFastWeight(torch.autograd.Function):
    """``out = fast_weight_delta(Q, K, V, beta, W)``.

    Q, K ``[N,H,L,E]``; V ``[N,H,L,M]``; beta ``[N,H,L,1]``; W ``[N,H,E,M]`` is the
    initial state on entry and the state after the last step on return (in place).
    Gradients flow to Q, K, V and beta; W gets none, as in the reference (:92).
    Unlike the reference, backward leaves W untouched.

    ``out`` has the reference's shape ``[N,H,L,M]``; its memory follows Q's: when Q is a permuted
    view of ``[L,N,H,E]`` storage, as in the reference's layers, out is a permuted view of
    ``[L,N,H,M]`` storage, so that their ``transpose(1, 2).reshape(bsz, slen, H * D).transpose(0, 1)``
    right after the call (cuda_fast_weight_layer.py:158-163) is a view and not a copy.  A sixth
    argument forces either layout (``True``: steps outermost, ``False``: contiguous ``[N,H,L,M]``).
    """

    @staticmethod
    def forward(ctx, Q, K, V, beta, W, time_major=None):
        _lib.require_device(Q)
        _lib.same_device(Q, K, V, beta, W)
        N, H, L, E = Q.shape
        M = V.shape[-1]
        if K.shape != (N, H, L, E) or V.shape != (N, H, L, M) or beta.shape != (N, H, L, 1):
            raise _lib.FwpError(f"shape mismatch: Q{tuple(Q.shape)} K{tuple(K.shape)} "
                                f"V{tuple(V.shape)} beta{tuple(beta.shape)}")
        if W.shape != (N, H, E, M) or not W.is_contiguous() or W.dtype != torch.float32:
            raise _lib.FwpError("W must be a contiguous fp32 [N,H,E,M] tensor")
        need_grad = any(ctx.needs_input_grad[:4])
        chunk = _lib.query(_lib.Q_DEFAULT_CHUNK)
        if time_major is None:
            time_major = rows_lead(Q)
        Q, qv = _lib.rows(Q)
        K, kv = _lib.rows(K)
        V, vv = _lib.rows(V)
        beta, bv = _lib.rows(beta)
        if time_major:
            out = torch.empty((L, N, H, M), device=Q.device, dtype=torch.float32).permute(1, 2, 0, 3)
        else:
            out = torch.empty((N, H, L, M), device=Q.device, dtype=torch.float32)
        ov = _lib.OutView(out.data_ptr(), out.stride(0), out.stride(1), out.stride(2))
        saved = vdiff = ckpt = None
        if need_grad:
            # v - v_old [N,H,L,M] and the checkpoints behind it, one allocation (L*M is a multiple
            # of 4 floats whenever the kernels need 16-byte alignment of either)
            n_vdiff = N * H * L * M
            saved = torch.empty(n_vdiff + _lib.delta_ckpt_floats(N, H, L, E, M, chunk), device=Q.device,
                                dtype=torch.float32)
            vdiff = saved.data_ptr()
            ckpt = vdiff + 4 * n_vdiff
        with _lib.on_device(Q):
            rc = _lib.lib().fwp_delta_fwd_strided(qv, kv, vv, bv, _lib.ptr(W), ov, vdiff, ckpt,
                                                  N, H, L, E, M, chunk, _lib.stream_of(Q))
        if rc:
            _lib.check(rc, "fwp_delta_fwd_strided")
        if need_grad:
            ctx.save_for_backward(Q, K, beta, saved)
            ctx.dims = (N, H, L, E, M, chunk)
            ctx.views = (qv, kv, bv)        # of the saved tensors, which keep the memory alive
        ctx.set_materialize_grads(False)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        if grad_out is None:
            return None, None, None, None, None, None
        Q, K, beta, saved = ctx.saved_tensors
        N, H, L, E, M, chunk = ctx.dims
        vdiff = saved.data_ptr()
        ckpt = vdiff + 4 * N * H * L * M
        qv, kv, bv = ctx.views
        _lib.same_device(Q, grad_out)
        grad_out, gv_ = _lib.rows(grad_out)
        grad_Q = torch.empty((N, H, L, E), device=Q.device, dtype=torch.float32)
        grad_K = torch.empty((N, H, L, E), device=Q.device, dtype=torch.float32)
        grad_V = torch.empty((N, H, L, M), device=Q.device, dtype=torch.float32)
        grad_beta = torch.empty((N, H, L, 1), device=Q.device, dtype=torch.float32)
        with _lib.on_device(Q):
            rc = _lib.lib().fwp_delta_bwd(
                qv, kv, bv, vdiff, gv_, ckpt, _lib.ptr(grad_Q),
                _lib.ptr(grad_K), _lib.ptr(grad_V), _lib.ptr(grad_beta), N, H, L, E, M, chunk,
                _lib.stream_of(Q))
        if rc:
            _lib.check(rc, "fwp_delta_bwd")
        return grad_Q, grad_K, grad_V, grad_beta, None, None


def _native():
    """The same operator as a C++ autograd function (csrc/fwp_torch.cpp), when it has been built:
    a forward + backward pair costs about 35 us less interpreter time through it."""
    try:
        from . import _fwp_torch
    except ImportError:
        return None
    _fwp_torch.set_error_class(_lib.FwpError)
    return _fwp_torch


_fwp_torch = _native()
_operator = _fwp_torch.fast_weight_delta if _fwp_torch is not None else DeltaFastWeight.apply

# Value widths the blocked kernels take for a given key width (fwp_delta_kind names the kernels).
_FAST_WIDTHS = {16: (16, 32, 64), 32: (16, 32, 64), 64: (16, 32, 64), 96: (16, 32), 128: (16, 32),
                192: (16,)}
# Value widths the single-step kernels take (with any of the key widths above up to 128).
_STEP_WIDTHS = (16, 32, 64, 128)
_plans = {}


def pick_width(widths, left):
    """The width of the next slice when ``left`` value columns remain: the narrowest that holds them all when
    at most a third of it is padding (one launch instead of two), else the widest that fits, else the
    narrowest, padded."""
    holds = [w for w in widths if w >= left and 2 * (w - left) <= left]
    if holds:
        return min(holds)
    fits = [w for w in widths if w <= left]
    return max(fits) if fits else min(widths)


def column_plan(E, M):
    """How a state of E x M is run when no fast kernel takes it whole: ``None`` (run it as it is) or a
    list of ``(first, last, width)``: value columns [first, last) run as a state of E x width, zero
    padded when width > last - first.  The columns of the delta rule's state never mix -
    v_old[m], the written value, W[:, m] and out[m] depend on column m and on the shared q, k, beta
    only (fast_weight_cuda.cu:101-143) - so the operator on a slice of V, W is exact, the gradients of
    Q, K, beta are the sums over the slices, and a padded column (v = 0, W = 0) stays zero."""
    key = (E, M)
    if key not in _plans:
        widths = _FAST_WIDTHS.get(E)
        plan = None
        if widths is not None and not (M in widths):
            plan, first = [], 0
            while first < M:
                left = M - first
                width = pick_width(widths, left)
                last = min(M, first + width)
                plan.append((first, last, width))
                first = last
        _plans[key] = plan
    return _plans[key]


def fast_weight_delta(Q, K, V, beta, W, time_major=None):
    """``out = fast_weight_delta(Q, K, V, beta, W)``, the reference's operator
    (algorithmic/fast_weight/__init__.py:96).  Key widths of 16, 32, 64, 96 and 128 with value widths
    the blocked kernels do not take whole (M = 3 D + 1 of the Delta-Delta layer, M = 128 of the
    Delta-MLP layer: cuda_fast_weight_layer.py:1474-1492,1605-1610) run on them by slices of value
    columns, see :func:`column_plan`: inside the C++ autograd function when it is built (one graph node,
    results written in place), by :func:`fast_weight_delta_sliced` otherwise."""
    if _fwp_torch is not None:      # the C++ function cuts the value columns itself (csrc/fwp_torch.cpp column_plan)
        return _operator(Q, K, V, beta, W) if time_major is None else _operator(Q, K, V, beta, W, time_major)
    return fast_weight_delta_sliced(Q, K, V, beta, W, time_major)


def fast_weight_delta_sliced(Q, K, V, beta, W, time_major=None, operator=DeltaFastWeight.apply):
    """The operator with the slices of value columns cut here, one call of the autograd Function per
    slice (what runs when the C++ function has not been built)."""
    try:        # the common case first: a width pair seen before (two size() calls and one dictionary lookup)
        plan = _plans[(Q.size(-1), V.size(-1))]
    except (KeyError, IndexError):
        plan = column_plan(Q.shape[-1], V.shape[-1]) if Q.dim() == 4 and V.dim() == 4 else None
    if plan is not None and Q.shape[2] == 1 and Q.shape[-1] <= 128 and V.shape[-1] in _STEP_WIDTHS and not (
            torch.is_grad_enabled() and any(t.requires_grad for t in (Q, K, V, beta))):
        plan = None     # a single step that saves nothing: the single-step kernels take these widths whole
    if plan is None:
        return operator(Q, K, V, beta, W) if time_major is None else operator(Q, K, V, beta, W, time_major)
    if Q.dim() != 4 or V.dim() != 4:
        raise _lib.FwpError(f"expected 4-D [N,H,L,D] tensors, got {Q.dim()}-D and {V.dim()}-D")
    # the same checks on W as the whole-state path makes (there the slices would hide the caller's W from them)
    N, H, L, E = Q.shape
    M = V.shape[-1]
    if W.shape != (N, H, E, M) or not W.is_contiguous() or W.dtype != torch.float32:
        raise _lib.FwpError("W must be a contiguous fp32 [N,H,E,M] tensor")
    _lib.same_device(Q, K, V, beta, W)
    outs, states = [], []
    for first, last, width in plan:
        pad = width - (last - first)
        Vs, Ws = V[..., first:last], W.detach()[..., first:last]
        if pad:
            Vs, Ws = torch.nn.functional.pad(Vs, (0, pad)), torch.nn.functional.pad(Ws, (0, pad))
        else:
            Ws = Ws.contiguous()
        out = operator(Q, K, Vs, beta, Ws, False)
        states.append(Ws)
        outs.append(out[..., :last - first] if pad else out)
    # the state after the last step, in place, once every slice has run: a rejected slice leaves W as it was
    with torch.no_grad():
        for (first, last, _), Ws in zip(plan, states):
            W[..., first:last] = Ws[..., :last - first]
    out = torch.cat(outs, -1)
    if time_major or (time_major is None and rows_lead(Q)):
        out = out.permute(2, 0, 1, 3).contiguous().permute(1, 2, 0, 3)
    return out
