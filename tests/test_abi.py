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


def test_ckpt_size_and_config_entry_points(fwp):
    L = fwp._lib
    lib = L.lib()
    chunk = L.query(L.Q_DEFAULT_CHUNK)
    # states only when the blocked kernels do not apply, states + header + one 16x16 matrix per 16 steps otherwise
    assert L.delta_ckpt_floats(2, 3, 100, 24, 8, chunk) == 2 * 3 * 2 * 24 * 8
    n16 = L.delta_ckpt_floats(2, 3, 100, 16, 16, chunk)
    assert n16 > 2 * 3 * 2 * 256 and (n16 - 2 * 3 * 2 * 256 - 2 * 3 * 7 * 256) in range(0, 65)
    assert lib.fwp_delta_ckpt_floats(0, 3, 100, 16, 16, chunk) == -1
    with pytest.raises(L.FwpError):
        L.delta_ckpt_floats(1, 1, 8, 16, 16, chunk + 1)
    for value in (L.DELTA_SCAN, L.DELTA_CHUNKED, L.DELTA_AUTO):
        L.config(L.CFG_DELTA_KERNELS, value)
    assert lib.fwp_config(L.CFG_DELTA_KERNELS, 7) != 0 and lib.fwp_config(99, 0) != 0
    # Delta LSTM and sum rule: NULL checks come before any launch
    null3 = (L.View * 3)()
    assert lib.fwp_lstm_fwd(null3, null3, null3, null3, None, None, None, None, None, None, None, None,
                            1, 1, 4, 16, chunk, None) == -1
    v = L.View(4096, 64, 32, 16)
    p = ctypes.c_void_p(4096)
    assert lib.fwp_sum_fwd(v, v, v, None, p, p, 1, 1, 4, 16, 16, chunk, None) == -1
    assert lib.fwp_sum_bwd(v, v, v, v, p, None, p, p, p, 1, 1, 4, 16, 16, 24, None) == -3


def test_delta_dispatch_keeps_32_bit_kernels_off_views_beyond_their_range(fwp):
    """fwp_delta_kind is the dispatch of fwp_delta_fwd / fwp_delta_bwd as a pure function.  Views into
    [T, B, H*D] storage with T = 8192 and B*H*D = 65536 pass 2 GiB along the sequence axis: the
    kernels that address a sequence with 32-bit offsets must not get them, forward or backward."""
    L = fwp._lib
    lib = L.lib()
    N, H, T, D = 128, 32, 8192, 16
    small = L.View(4096, H * T * D, T * D, D)
    huge = L.View(4096, H * D, D, N * H * D)          # permuted [T,N,H,D]: 256 KiB between steps
    beta = L.View(4096, H * T, T, 1)
    offsets32 = (L.KIND_CHUNKED, L.KIND_SPLIT, L.KIND_PHASE)
    for setting in (L.DELTA_AUTO, L.DELTA_CHUNKED, L.DELTA_SPLIT):
        L.config(L.CFG_DELTA_KERNELS, setting)
        try:
            for backward in (0, 1):
                assert lib.fwp_delta_kind(backward, small, small, small, beta, 4, 8, 256, D, D) in offsets32
                for views in ((huge, small, small), (small, huge, small), (small, small, huge)):
                    kind = lib.fwp_delta_kind(backward, *views, beta, N, H, T, D, D)
                    assert kind == L.KIND_SCAN, (setting, backward, kind)
        finally:
            L.config(L.CFG_DELTA_KERNELS, L.DELTA_AUTO)
    # short sequences stay on the scan kernels, shapes without a fast kernel on the LDS kernels
    assert lib.fwp_delta_kind(0, small, small, small, beta, 4, 8, 8, D, D) == L.KIND_SCAN
    # several waves per sequence while the chip holds every sequence's workgroup at once, one wave beyond
    for D_, most in ((16, 1024), (32, 512)):
        rows = L.View(4096, 8 * 256 * D_, 256 * D_, D_)
        for backward in (0, 1):
            assert lib.fwp_delta_kind(backward, rows, rows, rows, beta, most // 8, 8, 256, D_, D_) == L.KIND_SPLIT
            assert lib.fwp_delta_kind(backward, rows, rows, rows, beta, most // 8 + 1, 8, 256, D_, D_) == L.KIND_CHUNKED
    odd = L.View(4096, 8 * 64 * 24, 64 * 24, 24)
    assert lib.fwp_delta_kind(1, odd, odd, odd, beta, 4, 8, 64, 24, 24) == L.KIND_LDS
    assert lib.fwp_delta_kind(0, small, small, small, beta, 0, 8, 64, D, D) == -2


def test_forward_dispatch_knows_the_output_view_and_single_steps(fwp):
    """fwp_delta_fwd_kind is fwp_delta_fwd_strided's choice of kernels as a pure function: the output view
    counts like an input read 16 bytes at a time, and a single step that saves nothing has kernels of its own."""
    L = fwp._lib
    lib = L.lib()
    N, H, T, D = 128, 32, 8192, 16
    small = L.View(4096, 8 * 256 * D, 256 * D, D)
    beta = L.View(4096, 8 * 256, 256, 1)
    out_small = L.OutView(4096, 8 * 256 * D, 256 * D, D)
    assert lib.fwp_delta_fwd_kind(small, small, small, beta, out_small, 1, 4, 8, 256, D, D) == L.KIND_SPLIT
    # a time-major output whose rows pass 2 GiB: 64-bit scan kernels, not the LDS-state ones
    big_in = L.View(4096, H * T * D, T * D, D)
    big_beta = L.View(4096, H * T, T, 1)
    out_huge = L.OutView(4096, H * D, D, N * H * D)
    assert lib.fwp_delta_fwd_kind(big_in, big_in, big_in, big_beta, out_huge, 1, N, H, T, D, D) == L.KIND_SCAN
    assert lib.fwp_delta_kind(0, big_in, big_in, big_in, big_beta, N, H, T, D, D) == L.KIND_CHUNKED
    # output rows that are not 16-byte aligned: only the LDS-state kernels write those
    out_odd = L.OutView(4100, 8 * 256 * D, 256 * D, D)
    assert lib.fwp_delta_fwd_kind(small, small, small, beta, out_odd, 1, 4, 8, 256, D, D) == L.KIND_LDS
    # one step: kernels of its own when nothing is saved, the scan kernels when the call saves for backward
    one = L.View(4096, 8 * D, D, D)
    one_beta = L.View(4096, 8, 1, 1)
    out_one = L.OutView(4096, 8 * D, D, D)
    assert lib.fwp_delta_fwd_kind(one, one, one, one_beta, out_one, 0, 4, 8, 1, D, D) == L.KIND_STEP
    assert lib.fwp_delta_fwd_kind(one, one, one, one_beta, out_one, 1, 4, 8, 1, D, D) == L.KIND_SCAN
    L.config(L.CFG_STEP_KERNELS, 0)
    try:
        assert lib.fwp_delta_fwd_kind(one, one, one, one_beta, out_one, 0, 4, 8, 1, D, D) == L.KIND_SCAN
    finally:
        L.config(L.CFG_STEP_KERNELS, 1)
    assert lib.fwp_delta_fwd_kind(one, one, one, one_beta, out_one, 0, 0, 8, 1, D, D) == -2


def test_a_call_is_dispatched_under_one_setting_while_another_thread_changes_it(fwp):
    """Every entry point reads the FWP_CFG_DELTA_KERNELS switch once.  While a second thread flips it between
    SCAN and SPLIT, every answer of fwp_delta_kind must be one that a single setting gives (SCAN or SPLIT for
    16 x 16 states at L = 256): a call that saw SCAN where the several-wave kernels are chosen and SPLIT where
    the one-wave blocks are would answer CHUNKED, which neither setting does."""
    import threading
    L = fwp._lib
    lib = L.lib()
    D = 16
    view = L.View(4096, 8 * 256 * D, 256 * D, D)
    beta = L.View(4096, 8 * 256, 256, 1)
    single = {}
    for setting in (L.DELTA_SCAN, L.DELTA_SPLIT):
        L.config(L.CFG_DELTA_KERNELS, setting)
        single[setting] = lib.fwp_delta_kind(0, view, view, view, beta, 96, 8, 256, D, D)
    assert single == {L.DELTA_SCAN: L.KIND_SCAN, L.DELTA_SPLIT: L.KIND_SPLIT}
    stop = threading.Event()

    def flip():
        while not stop.is_set():
            lib.fwp_config(L.CFG_DELTA_KERNELS, L.DELTA_SCAN)
            lib.fwp_config(L.CFG_DELTA_KERNELS, L.DELTA_SPLIT)

    t = threading.Thread(target=flip)
    t.start()
    try:
        seen = set()
        for _ in range(50000):
            for backward in (0, 1):
                seen.add(lib.fwp_delta_kind(backward, view, view, view, beta, 96, 8, 256, D, D))
    finally:
        stop.set()
        t.join()
        L.config(L.CFG_DELTA_KERNELS, L.DELTA_AUTO)
    assert seen <= set(single.values()), seen


def test_value_columns_are_sliced_onto_the_blocked_kernels(fwp):
    """Shapes of the reference's call sites that no kernel takes whole are run by slices of value
    columns, every slice a state shape the blocked kernels take (checked against fwp_delta_kind)."""
    import importlib
    fw = importlib.import_module(fwp.__name__ + ".fast_weight")
    L = fwp._lib
    lib = L.lib()
    assert fw.column_plan(32, 32) is None and fw.column_plan(96, 16) is None and fw.column_plan(128, 16) is None
    assert fw.column_plan(128, 32) is None
    assert fw.column_plan(24, 8) is None and fw.column_plan(5, 3) is None          # no fast kernel for these keys
    assert fw.column_plan(32, 97) == [(0, 64, 64), (64, 96, 32), (96, 97, 16)]
    assert fw.column_plan(32, 128) == [(0, 64, 64), (64, 128, 64)]
    assert fw.column_plan(128, 64) == [(0, 32, 32), (32, 64, 32)]
    assert fw.column_plan(96, 48) == [(0, 32, 32), (32, 48, 16)]
    # one padded launch where at most a third of it is padding: 3 D + 1 at D = 16, and 24 or 48 columns
    assert fw.column_plan(16, 49) == [(0, 49, 64)] and fw.column_plan(32, 24) == [(0, 24, 32)]
    assert fw.column_plan(64, 48) == [(0, 48, 64)] and fw.column_plan(64, 40) == [(0, 32, 32), (32, 40, 16)]
    assert fw.column_plan(192, 24) == [(0, 16, 16), (16, 24, 16)]
    # the sum rule: its own table of widths, keys padded as well
    ft = fwp.fast_transformers
    assert ft.sum_plan(32, 128) is None and ft.sum_plan(192, 16) is None and ft.sum_plan(200, 16) is None
    assert ft.sum_plan(192, 32) is None and ft.sum_plan(64, 128) is None and ft.sum_plan(128, 64) is None
    assert ft.sum_plan(128, 128) == (128, [(0, 64, 64), (64, 128, 64)])
    assert ft.sum_plan(96, 64) == (96, [(0, 32, 32), (32, 64, 32)])
    assert ft.sum_plan(48, 24) == (64, [(0, 24, 32)]) and ft.sum_plan(11, 4) == (16, [(0, 4, 16)])
    for E, M in ((32, 97), (32, 128), (128, 64), (96, 48), (64, 100), (16, 1), (16, 49), (64, 48)):
        plan = fw.column_plan(E, M)
        assert plan[0][0] == 0 and plan[-1][1] == M and all(a[1] == b[0] for a, b in zip(plan, plan[1:]))
        for first, last, width in plan:
            assert 0 < last - first <= width
            qv = L.View(4096, 8 * 64 * E, 64 * E, E)
            vv = L.View(4096, 8 * 64 * width, 64 * width, width)
            bv = L.View(4096, 8 * 64, 64, 1)
            for backward in (0, 1):
                assert lib.fwp_delta_kind(backward, qv, qv, vv, bv, 4, 8, 64, E, width) in (L.KIND_SPLIT, L.KIND_CHUNKED)


def test_largest_state_of_a_differentiated_call_is_published(fwp):
    L = fwp._lib
    rnn, rec, lstm = (L.query(q) for q in (L.Q_MAX_D_RNN, L.Q_MAX_D_REC, L.Q_MAX_D_LSTM))
    assert 64 <= lstm <= rec <= rnn <= 128


def test_operators_refuse_tensors_on_different_devices(fwp):
    """Only the first tensor being on the GPU is not enough: the others are passed by address."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("needs a machine without a GPU (the check itself is device independent)")
    L = fwp._lib
    meta = torch.zeros(1, 1, 2, 4, device="meta")
    cpu = torch.zeros(1, 1, 2, 4)
    with pytest.raises(L.FwpError, match="same device"):
        L.same_device(meta, meta, cpu)
    L.same_device(cpu, cpu, cpu)


def test_operators_refuse_cpu_tensors(fwp):
    import torch
    q = torch.zeros(1, 1, 2, 4)
    with pytest.raises(fwp._lib.FwpError):
        fwp.fast_weight_delta(q, q, q, q[..., :1], torch.zeros(1, 1, 4, 4))
