"""Host-side checks that need no GPU: the shared library loads, exports every symbol the
header declares, and rejects bad calls before touching a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "fwp_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fwp_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(fwp):
    lib = fwp._lib.lib()
    names = declared_symbols()
    assert "fwp_delta_fwd" in names and "fwp_rec_bwd" in names and len(names) >= 9
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(fwp._lib.EXPORTS) == names


def test_query_and_error_strings(fwp):
    L = fwp._lib
    assert L.query(L.Q_VERSION) >= 1
    quantum, default = L.query(L.Q_CHUNK_QUANTUM), L.query(L.Q_DEFAULT_CHUNK)
    assert quantum > 0 and default % quantum == 0
    assert L.query(L.Q_MAX_STATE_FLOATS) >= 64 * 64
    assert L.strerror(0) == "ok"
    for code in (-1, -2, -3, -4, -5):
        assert L.strerror(code) not in ("ok", "unknown error")


def test_bad_arguments_are_rejected_without_a_device(fwp):
    L = fwp._lib
    lib = L.lib()
    v = L.View(4096, 64, 32, 16)
    null = L.View(0, 0, 0, 0)
    p = ctypes.c_void_p(4096)
    assert lib.fwp_delta_fwd(null, v, v, v, p, p, p, p, 1, 1, 4, 16, 16, 64, None) == -1      # FWP_E_NULL
    assert lib.fwp_delta_fwd(v, v, v, v, p, p, p, None, 1, 1, 4, 16, 16, 64, None) == -1      # vdiff without ckpt
    assert lib.fwp_delta_fwd(v, v, v, v, p, p, p, p, 0, 1, 4, 16, 16, 64, None) == -2         # FWP_E_SHAPE
    assert lib.fwp_delta_fwd(v, v, v, v, p, p, p, p, 1, 1, 4, 16, 16, 24, None) == -3         # FWP_E_CHUNK
    assert lib.fwp_delta_fwd(v, v, v, v, p, p, p, p, 1, 1, 4, 512, 512, 64, None) == -4       # FWP_E_TOO_LARGE
    assert lib.fwp_rnn_fwd(v, v, v, v, p, None, p, p, p, 1, 1, 4, 16, 64, None) == -1


def test_operators_refuse_cpu_tensors(fwp):
    import torch
    q = torch.zeros(1, 1, 2, 4)
    with pytest.raises(fwp._lib.FwpError):
        fwp.fast_weight_delta(q, q, q, q[..., :1], torch.zeros(1, 1, 4, 4))
