"""ctypes binding of libfwp_hip.so (the C ABI declared in include/fwp_hip.h).

There is no fallback: if the shared library is missing or a call is rejected the
caller gets an exception.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "libfwp_hip.so")

_F = ctypes.POINTER(ctypes.c_float)


class View(ctypes.Structure):
    """struct fwp_view: device pointer + element strides of the N, H, L axes."""
    _fields_ = [("ptr", ctypes.c_void_p), ("sN", ctypes.c_int64), ("sH", ctypes.c_int64),
                ("sL", ctypes.c_int64)]


class OutView(ctypes.Structure):
    """struct fwp_out_view: a strided [N,H,L,M] output."""
    _fields_ = [("ptr", ctypes.c_void_p), ("sN", ctypes.c_int64), ("sH", ctypes.c_int64),
                ("sL", ctypes.c_int64)]


class FwpError(RuntimeError):
    pass


_P, _I, _V = ctypes.c_void_p, ctypes.c_int, View
_VP = ctypes.POINTER(View)          # host array of views (one per gate)
_SIGNATURES = {
    "fwp_delta_fwd": [_V] * 4 + [_P] * 4 + [_I] * 6 + [_P],
    "fwp_delta_bwd": [_V] * 3 + [_P, _V, _P] + [_P] * 4 + [_I] * 6 + [_P],
    "fwp_sum_fwd": [_V] * 3 + [_P] * 3 + [_I] * 6 + [_P],
    "fwp_sum_bwd": [_V] * 4 + [_P] * 5 + [_I] * 6 + [_P],
    "fwp_rnn_fwd": [_V] * 4 + [_P] * 5 + [_I] * 5 + [_P],
    "fwp_rnn_bwd": [_V, _V, _P, _P, _P, _V, _P] + [_P] * 4 + [_I] * 5 + [_P],
    "fwp_lstm_fwd": [_VP] * 4 + [_P] * 8 + [_I] * 5 + [_P],
    "fwp_lstm_bwd": [_VP] * 2 + [_P] * 6 + [_V] + [_P] * 5 + [_I] * 5 + [_P],
    "fwp_deltanet_prep_fwd": [_P] * 5 + [_I] * 4 + [ctypes.c_float, _P],
    "fwp_deltanet_prep_bwd": [_P] * 6 + [_I] * 4 + [ctypes.c_float, _P],
    "fwp_delta_fwd_strided": [_V] * 4 + [_P, OutView] + [_P] * 2 + [_I] * 6 + [_P],
    "fwp_rec_fwd": [_V] * 4 + [_P] * 12 + [_I] * 5 + [_P],
    "fwp_rec_bwd": [_P] * 6 + [_V] + [_P] * 14 + [_I] * 5 + [_P],
    "fwp_rec_bwd_static": [_P] * 6 + [_V] + [_P] * 13 + [_I] * 5 + [_P],
}
EXPORTS = sorted(list(_SIGNATURES) + ["fwp_strerror", "fwp_query", "fwp_check_device", "fwp_config",
                                       "fwp_delta_ckpt_floats", "fwp_delta_kind", "fwp_delta_fwd_kind"])
KIND_LDS, KIND_SCAN, KIND_CHUNKED, KIND_SPLIT, KIND_PHASE, KIND_STEP = 0, 1, 2, 3, 4, 5
CFG_DELTA_KERNELS, DELTA_AUTO, DELTA_SCAN, DELTA_CHUNKED, DELTA_SPLIT, DELTA_PHASE = 0, 0, 1, 2, 3, 4
CFG_STEP_KERNELS = 1

_lib = None
_checked_devices = set()


def lib():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise FwpError(
                f"{SO_PATH} is missing: build it with recurrent-fwp_amd/csrc/build.sh "
                "(there is no CPU or PyTorch fallback for the fast-weight operators)")
        handle = ctypes.CDLL(SO_PATH)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        handle.fwp_strerror.argtypes = [ctypes.c_int]
        handle.fwp_strerror.restype = ctypes.c_char_p
        handle.fwp_query.argtypes = [ctypes.c_int]
        handle.fwp_query.restype = ctypes.c_int
        handle.fwp_check_device.restype = ctypes.c_int
        handle.fwp_delta_ckpt_floats.argtypes = [ctypes.c_int] * 6
        handle.fwp_delta_ckpt_floats.restype = ctypes.c_longlong
        handle.fwp_delta_kind.argtypes = [_I] + [_V] * 4 + [_I] * 5
        handle.fwp_delta_kind.restype = ctypes.c_int
        handle.fwp_delta_fwd_kind.argtypes = [_V] * 4 + [OutView] + [_I] * 6
        handle.fwp_delta_fwd_kind.restype = ctypes.c_int
        handle.fwp_config.argtypes = [ctypes.c_int, ctypes.c_int]
        handle.fwp_config.restype = ctypes.c_int
        _lib = handle
    return _lib


_query_cache = {}


def query(what):
    if what not in _query_cache:
        _query_cache[what] = int(lib().fwp_query(int(what)))
    return _query_cache[what]


Q_VERSION, Q_CHUNK_QUANTUM, Q_DEFAULT_CHUNK, Q_MAX_STATE_FLOATS = 0, 1, 2, 3
Q_MAX_D_RNN, Q_MAX_D_REC, Q_MAX_D_LSTM, Q_STATIC_SCRATCH_FLOATS = 4, 5, 6, 7
Q_STEP_LAUNCHES = 8


def step_launches():
    """Calls so far that went to the single-step kernels (a running count, never cached)."""
    return int(lib().fwp_query(Q_STEP_LAUNCHES))


_ckpt_floats_cache = {}


def delta_ckpt_floats(N, H, L, E, M, chunk):
    key = (N, H, L, E, M, chunk)
    n = _ckpt_floats_cache.get(key)
    if n is None:
        n = int(lib().fwp_delta_ckpt_floats(N, H, L, E, M, chunk))
        if n < 0:
            raise FwpError(f"invalid dimensions N={N} H={H} L={L} E={E} M={M} chunk={chunk}")
        if len(_ckpt_floats_cache) > 1024:
            _ckpt_floats_cache.clear()
        _ckpt_floats_cache[key] = n
    return n


def config(key, value):
    check(lib().fwp_config(int(key), int(value)), "fwp_config")


def strerror(code):
    return lib().fwp_strerror(int(code)).decode()


def check(code, what):
    if code != 0:
        raise FwpError(f"{what} failed: {strerror(code)} (code {code})")


def require_device(t):
    """The operators exist for fp32 tensors on a gfx950 GPU only."""
    dev = t.device
    if dev in _checked_devices:
        return
    if dev.type != "cuda":
        raise FwpError(f"fast-weight operators need tensors on an MI355X GPU, got device '{dev}'")
    with torch.cuda.device(dev):
        check(lib().fwp_check_device(), "device check")
    _checked_devices.add(dev)


def same_device(ref, *others):
    """Every tensor of a call lives on the first one's GPU: the kernels get raw addresses, and an
    address of host memory or of another GPU would be a memory fault there, not an exception."""
    dev = ref.device
    for t in others:
        if t.device != dev:
            raise FwpError(f"all tensors of a call must be on the same device: got '{t.device}' beside '{dev}'")


def rows(t):
    """A view argument for a 4-D fp32 tensor.

    Permuted views are passed as they are.  A copy is made when the last axis is strided,
    and when rows of a multiple of 4 floats are not 16-byte aligned (a slice of a wider
    buffer, such as v inside a fused q|k|v|beta projection): one elementwise pass costs far
    less than giving up the kernels that read rows with 16-byte loads.
    """
    if t.dtype is not torch.float32:
        raise FwpError(f"fast-weight operators are fp32 only, got {t.dtype}")
    if t.dim() != 4:
        raise FwpError(f"expected a 4-D [N,H,L,D] tensor, got {t.dim()}-D")
    if t.is_contiguous():            # the common case, kept short: this runs eight times per step
        p = t.data_ptr()
        _, h, l, d = t.shape
        if d % 4 or p % 16 == 0:
            ld = l * d
            return t, View(p, h * ld, ld, d)
        t = t.clone()
        return t, View(t.data_ptr(), h * l * d, l * d, d)
    d = t.shape[-1]
    sn, sh, sl, sd = t.stride()
    if d != 1 and sd != 1:
        t = t.contiguous()
    elif d % 4 == 0 and (t.data_ptr() % 16 or sn % 4 or sh % 4 or sl % 4):
        t = t.contiguous()
    return t, View(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def ptr(t):
    """Device address of a tensor as ctypes takes it for a void* parameter."""
    return t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(t):
    """The current HIP stream of the tensor's device, as the C ABI takes it."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()
_single_gpu = None


def on_device(t):
    """Context that makes the tensor's GPU current for the launch; free when it already is."""
    global _single_gpu
    if _single_gpu is None:
        _single_gpu = torch.cuda.device_count() == 1
    if _single_gpu:
        return _NO_GUARD
    idx = (t if isinstance(t, torch.device) else t.device).index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(idx)
