#!/usr/bin/env python3
"""Benchmark of the fast-weight update operators on one MI355X.

A step is one forward + backward of the operator (through its autograd
Function, allocations included) over one synthetic batch that is already
resident in HBM.  Default workload: the delta rule at the LM-small shape
B=96, H=8, T=256, D=16 (fp32).  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload delta|rnn|rec]
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

METRIC = "fast-weight update tokens/s (fwd+bwd), % of FP32-VALU roofline, 1 GPU"
PEAK_VALU = 157.3e12     # MI355X fp32 vector peak (packed), FLOP/s
PEAK_HBM = 8.0e12        # MI355X HBM3E, B/s

# HBM bytes per launch of the forward / backward kernel, measured with rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch; FETCH_SIZE scaled x2.0 and WRITE_SIZE x1.0 by what the same counters read
# for a 2 GiB device-to-device copy, `--copy-calibration`).  They live in profiles/hbm_traffic.txt, which
# `bench.py --workload W --traffic-from FETCH_DIR WRITE_DIR` rewrites from the output directories of the
# two counter runs; a workload without an entry there reports traffic null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0


def measured_traffic():
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f)["bytes_per_launch"]
    except (OSError, ValueError, KeyError):
        return {}


def update_traffic(workload, fetch_dir, write_dir):
    """Average FETCH_SIZE / WRITE_SIZE per dispatch of the library's forward and backward kernels in the
    two rocprofv3 output directories -> bytes per launch of that workload in profiles/hbm_traffic.txt."""
    import glob
    import sqlite3

    def per_kernel(directory, counter):
        dbs = glob.glob(os.path.join(directory, "**", "*.db"), recursive=True)
        if not dbs:
            sys.exit(f"bench.py: no rocprofv3 database under {directory}")
        con = sqlite3.connect(dbs[0])
        tables = [r[0] for r in con.execute("select name from sqlite_master where type in ('table','view')")]
        table = [t for t in tables if t.startswith("counters_collection")][0]
        rows = con.execute(f"select kernel_name, avg(value) from {table} where counter_name = ? "
                           "group by kernel_name", (counter,)).fetchall()
        out = {}
        for kernel, kib in rows:
            if "fwp" not in kernel or "reduce_param" in kernel or "prep" in kernel:
                continue
            out["fwd" if "fwd" in kernel else "bwd"] = kib * 1024.0
        return out

    fetch, write = per_kernel(fetch_dir, "FETCH_SIZE"), per_kernel(write_dir, "WRITE_SIZE")
    entry = {d: round(fetch[d] * FETCH_SCALE + write[d] * WRITE_SCALE, -5) for d in ("fwd", "bwd")}
    table = measured_traffic()
    table[workload] = entry
    with open(TRAFFIC_FILE, "w") as f:
        json.dump({"what": "HBM bytes per launch of the forward / backward kernel of a bench.py workload: "
                           "rocprofv3 FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 (KiB per dispatch; the factors are "
                           "what the counters read for a 2 GiB copy, bench.py --copy-calibration)",
                   "rewritten_by": "python3 bench.py --workload W --traffic-from FETCH_DIR WRITE_DIR",
                   "bytes_per_launch": table}, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps({workload: entry}))


# name -> (B, H, T, D, algorithmic flops per token-head = c*D^2, fwd bytes, bwd bytes per token-head)
WORKLOADS = {
    "delta": dict(B=96, H=8, T=256, D=16, flop_c=20, fwd_bytes=lambda D: (4 * D + 1) * 4,
                  bwd_bytes=lambda D: (7 * D + 2) * 4,
                  label="delta-rule fast_weight fwd+bwd, B=96 H=8 T=256 D=16, fp32"),
    "delta_lm": dict(B=32, H=8, T=1024, D=32, flop_c=20, fwd_bytes=lambda D: (4 * D + 1) * 4,
                     bwd_bytes=lambda D: (7 * D + 2) * 4,
                     label="delta-rule fast_weight fwd+bwd at the shape one layer of the 16-layer LM gives it, "
                           "B=32 H=8 T=1024 D=32, fp32"),
    "sum": dict(B=96, H=8, T=256, D=16, flop_c=12, fwd_bytes=lambda D: 4 * D * 4,
                bwd_bytes=lambda D: 7 * D * 4,
                label="sum-rule fast_weight_sum (causal linear attention) fwd+bwd, B=96 H=8 T=256 D=16, fp32"),
    "rnn": dict(B=64, H=8, T=256, D=32, flop_c=20, fwd_bytes=lambda D: (4 * D + 1) * 4,
                bwd_bytes=lambda D: (8 * D + 2) * 4,
                label="Delta RNN fast_rnn_v2 fwd+bwd, B=64 H=8 T=256 D=32, fp32"),
    "lstm": dict(B=64, H=8, T=256, D=32, flop_c=60, fwd_bytes=lambda D: (18 * D + 3) * 4,
                 bwd_bytes=lambda D: (23 * D + 6) * 4,
                 label="Delta LSTM fast_lstm_v4 fwd+bwd, B=64 H=8 T=256 D=32, fp32"),
    "rec": dict(B=64, H=8, T=256, D=32, flop_c=38, fwd_bytes=lambda D: (4 * D + 1) * 4,
                bwd_bytes=lambda D: (8 * D + 2) * 4,
                label="Recurrent Delta Net rec_update_fwm_tanh fwd+bwd, B=64 H=8 T=256 D=32, fp32"),
}


def make_inputs(name, w):
    import numpy as np
    from helpers import delta_inputs, lstm_inputs, rec_inputs, rnn_inputs
    B, H, T, D = w["B"], w["H"], w["T"], w["D"]
    if name.startswith("delta") or name == "sum":
        return delta_inputs(0, B, H, T, w.get("E", D), w.get("M", D), dtype=np.float32)
    if name == "rnn":
        return rnn_inputs(0, B, H, T, D, dtype=np.float32)
    if name == "lstm":
        Zs, Ks, Vs, Bs, Ws, h0, c0, go = lstm_inputs(0, B, H, T, D, dtype=np.float32)
        return [*Zs, *Ks, *Vs, *Bs, *Ws, h0, c0, go]
    return rec_inputs(0, B, H, T, D, dtype=np.float32)


def gpu_step_fn(name, pkg, arrays):
    """Returns (step, n_diff) where step() runs one fwd+bwd on the GPU."""
    import torch
    dev = [torch.from_numpy(a).to("cuda:0") for a in arrays]
    go = dev[-1]
    if name.startswith("delta"):
        q, k, v, beta, W0 = dev[:5]
        diff = [t.requires_grad_(True) for t in (q, k, v, beta)]
        W = W0.clone()

        def step():
            W.zero_()                     # W0 = 0 for every step of the benchmark
            out = pkg.fast_weight_delta(*diff, W)
            torch.autograd.grad(out, diff, go)
            return out
    elif name == "sum":
        q, k, v, _, W0 = dev[:5]
        diff = [t.requires_grad_(True) for t in (q, k, v)]
        W = W0.clone()

        def step():
            W.zero_()
            out = pkg.fast_weight_sum(*diff, W)
            torch.autograd.grad(out, diff, go)
            return out
    elif name == "lstm":
        Zs, Ks, Vs, Bs, Ws = (dev[3 * i:3 * i + 3] for i in range(5))
        h, c = dev[15].clone(), dev[16].clone()
        diff = [t.requires_grad_(True) for t in (*Zs, *Ks, *Vs, *Bs)]
        Ws = [w.clone() for w in Ws]

        def step():
            for t in (*Ws, h, c):
                t.zero_()
            args = []
            for a in range(3):
                args += [Zs[a], Ks[a], Vs[a], Bs[a], Ws[a]]
            out, _ = pkg.fast_lstm_v4(*args, h, c)
            torch.autograd.grad(out, diff, go)
            return out
    elif name == "rnn":
        z, k, v, W0, beta, h0 = dev[:6]
        diff = [t.requires_grad_(True) for t in (z, k, v, beta)]
        W, h = W0.clone(), h0.clone()

        def step():
            W.zero_()
            h.zero_()
            out = pkg.fast_rnn_v2(diff[0], diff[1], diff[2], W, diff[3], h)
            torch.autograd.grad(out, diff, go)
            return out
    else:
        diff = [t.requires_grad_(True) for t in dev[:8]]
        W0, h0 = dev[8], dev[9]
        W, h = W0.clone(), h0.clone()

        def step():
            W.zero_()
            h.zero_()
            out = pkg.rec_update_fwm_tanh(*diff, W, h)
            torch.autograd.grad(out, diff, go)
            return out
    return step, diff


def stream_floor(name):
    """What the step's algorithmic HBM bytes cost at this size when nothing is computed: copies of one
    [B,H,T,D] array into another (each launch reads and writes B*H*T*D*4 bytes), back to back between two
    events like the kernel timings; forward and backward floors = their algorithmic bytes at that rate."""
    import torch
    w = WORKLOADS[name]
    B, H, T, D = w["B"], w["H"], w["T"], w["D"]
    n = B * H * T * D
    src = [torch.randn(n, device="cuda:0") for _ in range(4)]
    dst = [torch.empty(n, device="cuda:0") for _ in range(4)]

    def sweep():
        for a, b in zip(src, dst):
            b.copy_(a)
    for _ in range(20):
        sweep()
    torch.cuda.synchronize()
    reps = 200
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        sweep()
    e1.record()
    torch.cuda.synchronize()
    per_copy_s = e0.elapsed_time(e1) * 1e-3 / (reps * 4)
    rate = 2 * n * 4 / per_copy_s
    token_heads = B * H * T
    fwd_b, bwd_b = w["fwd_bytes"](D) * token_heads, w["bwd_bytes"](D) * token_heads
    return {"workload": w["label"], "copy_bytes": 2 * n * 4, "copy_us": per_copy_s * 1e6, "copy_GBps": rate / 1e9,
            "fwd_floor_us": fwd_b / rate * 1e6, "bwd_floor_us": bwd_b / rate * 1e6,
            "step_floor_us": (fwd_b + bwd_b) / rate * 1e6}


def kernel_times(name, pkg, arrays, iters):
    """Average duration (s) of the forward and of the backward launch, timed with HIP
    events on the stream the kernels are launched on (direct C-ABI calls, buffers preallocated)."""
    import torch
    L = pkg._lib
    lib = L.lib()
    dev = [torch.from_numpy(a).to("cuda:0") for a in arrays]
    go = dev[-1]
    stream_of = lambda: L.stream_of(go)      # evaluated per launch: the current stream may be a capturing one
    chunk = L.query(L.Q_DEFAULT_CHUNK)
    f32 = dict(device="cuda:0", dtype=torch.float32)

    def view(t):
        return L.View(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))

    if name.startswith("delta"):
        q, k, v, beta, W0 = dev[:5]
        N, H, T, E = q.shape
        M = v.shape[-1]
        nch = (T + chunk - 1) // chunk
        W = W0.clone()
        out, vdiff = torch.empty_like(v), torch.empty_like(v)
        ckpt = torch.empty(L.delta_ckpt_floats(N, H, T, E, M, chunk), **f32)
        gq, gk, gv, gb = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(beta)

        def fwd():
            return lib.fwp_delta_fwd(view(q), view(k), view(v), view(beta), L.ptr(W), L.ptr(out), L.ptr(vdiff),
                                     L.ptr(ckpt), N, H, T, E, M, chunk, stream_of())

        def bwd():
            return lib.fwp_delta_bwd(view(q), view(k), view(beta), L.ptr(vdiff), view(go), L.ptr(ckpt), L.ptr(gq),
                                     L.ptr(gk), L.ptr(gv), L.ptr(gb), N, H, T, E, M, chunk, stream_of())
        reset = lambda: W.copy_(W0)
    elif name == "sum":
        q, k, v, _, W0 = dev[:5]
        N, H, T, E = q.shape
        M = v.shape[-1]
        nch = (T + chunk - 1) // chunk
        W = W0.clone()
        out = torch.empty_like(v)
        ckpt = torch.empty((N, H, nch, E, M), **f32)
        gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

        def fwd():
            return lib.fwp_sum_fwd(view(q), view(k), view(v), L.ptr(W), L.ptr(out), L.ptr(ckpt), N, H, T, E, M,
                                   chunk, stream_of())

        def bwd():
            return lib.fwp_sum_bwd(view(q), view(k), view(v), view(go), L.ptr(ckpt), None, L.ptr(gq), L.ptr(gk),
                                   L.ptr(gv), N, H, T, E, M, chunk, stream_of())
        reset = lambda: W.copy_(W0)
    elif name == "lstm":
        import ctypes
        Zs, Ks, Vs, Bs, Ws0 = (dev[3 * i:3 * i + 3] for i in range(5))
        h0, c0 = dev[15], dev[16]
        N, H, T, D = Zs[0].shape
        nch = (T + chunk - 1) // chunk
        Ws = [w.clone() for w in Ws0]
        h, c = h0.clone(), c0.clone()
        out, cell = torch.empty_like(Zs[0]), torch.empty_like(Zs[0])
        gates, vdiff = torch.empty((3, N, H, T, D), **f32), torch.empty((3, N, H, T, D), **f32)
        ckpt = torch.empty((3, N, H, nch, D, D), **f32)
        gz, gk, gv = (torch.empty((3, N, H, T, D), **f32) for _ in range(3))
        gb = torch.empty((3, N, H, T, 1), **f32)
        views = lambda ts: (L.View * 3)(*[view(t) for t in ts])
        Wp = (ctypes.c_void_p * 3)(*[w.data_ptr() for w in Ws])

        def fwd():
            return lib.fwp_lstm_fwd(views(Zs), views(Ks), views(Vs), views(Bs), Wp, L.ptr(h), L.ptr(c), L.ptr(out),
                                    L.ptr(cell), L.ptr(gates), L.ptr(vdiff), L.ptr(ckpt), N, H, T, D, chunk,
                                    stream_of())

        def bwd():
            return lib.fwp_lstm_bwd(views(Ks), views(Bs), L.ptr(vdiff), L.ptr(gates), L.ptr(out), L.ptr(cell),
                                    L.ptr(h0), L.ptr(c0), view(go), L.ptr(ckpt), L.ptr(gz), L.ptr(gk), L.ptr(gv),
                                    L.ptr(gb), N, H, T, D, chunk, stream_of())

        W = Ws[0]

        def reset():
            for w, w0 in zip(Ws, Ws0):
                w.copy_(w0)
            h.copy_(h0)
            c.copy_(c0)
    elif name == "rnn":
        z, k, v, W0, beta, h0 = dev[:6]
        N, H, T, D = z.shape
        nch = (T + chunk - 1) // chunk
        W, h = W0.clone(), h0.clone()
        out, vdiff = torch.empty_like(v), torch.empty_like(v)
        ckpt = torch.empty((N, H, nch, D, D), **f32)
        gz, gk, gv, gb = torch.empty_like(z), torch.empty_like(k), torch.empty_like(v), torch.empty_like(beta)

        def fwd():
            return lib.fwp_rnn_fwd(view(z), view(k), view(v), view(beta), L.ptr(W), L.ptr(h), L.ptr(out),
                                   L.ptr(vdiff), L.ptr(ckpt), N, H, T, D, chunk, stream_of())

        def bwd():
            return lib.fwp_rnn_bwd(view(k), view(beta), L.ptr(vdiff), L.ptr(out), L.ptr(h0), view(go), L.ptr(ckpt),
                                   L.ptr(gz), L.ptr(gk), L.ptr(gv), L.ptr(gb), N, H, T, D, chunk, stream_of())

        def reset():
            W.copy_(W0)
            h.copy_(h0)
    else:
        qx, kx, vx, bx, Rq, Rk, Rv, rb, W0, h0 = dev[:10]
        N, H, T, D = qx.shape
        nch = (T + chunk - 1) // chunk
        W, h = W0.clone(), h0.clone()
        out, vdiff, qa, ka = (torch.empty_like(vx) for _ in range(4))
        ba = torch.empty((N, H, T), **f32)
        ckpt = torch.empty((N, H, nch, D, D), **f32)
        g = [torch.empty_like(t) for t in (qx, kx, vx, bx, Rq, Rk, Rv, rb)]
        ws = torch.empty((N, H, 3 * D * D + D), **f32)

        def fwd():
            return lib.fwp_rec_fwd(view(qx), view(kx), view(vx), view(bx), L.ptr(Rq), L.ptr(Rk), L.ptr(Rv),
                                   L.ptr(rb), L.ptr(W), L.ptr(h), L.ptr(out), L.ptr(qa), L.ptr(ka), L.ptr(ba),
                                   L.ptr(vdiff), L.ptr(ckpt), N, H, T, D, chunk, stream_of())

        def bwd():
            return lib.fwp_rec_bwd(L.ptr(qa), L.ptr(ka), L.ptr(ba), L.ptr(vdiff), L.ptr(out), L.ptr(h0), view(go),
                                   L.ptr(Rq), L.ptr(Rk), L.ptr(Rv), L.ptr(rb), L.ptr(ckpt), *[L.ptr(t) for t in g],
                                   L.ptr(ws), N, H, T, D, chunk, stream_of())

        def reset():
            W.copy_(W0)
            h.copy_(h0)

    def timed(fn):
        """Average duration of a launch: batches of `iters` back-to-back launches between two events on the
        launch stream, the median batch (the first launches after an idle spell run at lower clocks)."""
        for _ in range(50):
            L.check(fn(), "warm-up launch")
        torch.cuda.synchronize()
        batches = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                rc = fn()
            e1.record()
            L.check(rc, "timed launch")
            e1.synchronize()
            batches.append(e0.elapsed_time(e1) * 1e-3 / iters)
        return sorted(batches)[len(batches) // 2]

    t_f = timed(fwd)       # the state carries over between launches; the work per launch is the same
    reset()
    L.check(fwd(), "forward before backward timing")
    t_b = timed(bwd)

    def abi_step():
        """state reset + forward + backward, straight through the C ABI on preallocated buffers"""
        if name == "lstm":
            reset()
        else:
            W.zero_()
        if name in ("rnn", "rec"):
            h.zero_()
        L.check(fwd(), "forward")
        L.check(bwd(), "backward")

    return t_f, t_b, abi_step


def cpu_baseline(name, arrays, w, reps):
    """The reference's CPU path (its PyTorch step loop + autograd), restated, on the host cores."""
    import torch
    from oracle import torch_loop
    cores = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        cores = min(cores, int(env))
    torch.set_num_threads(cores)
    ts = [torch.from_numpy(a) for a in arrays]
    go = ts[-1]
    if name.startswith("delta"):
        loop, inputs, idx = torch_loop.delta_loop, ts[:5], [0, 1, 2, 3]
    elif name == "sum":
        loop, inputs, idx = torch_loop.sum_loop, [ts[0], ts[1], ts[2], ts[4]], [0, 1, 2]
    elif name == "lstm":
        order = []
        for a in range(3):                       # (Z, K, V, beta, W) per gate, then h0, c0
            order += [ts[a], ts[3 + a], ts[6 + a], ts[9 + a], ts[12 + a]]
        loop, inputs = torch_loop.lstm_v4_loop, order + [ts[15], ts[16]]
        idx = [5 * a + j for a in range(3) for j in range(4)]
    elif name == "rnn":
        loop, inputs, idx = torch_loop.rnn_v2_loop, ts[:6], [0, 1, 2, 4]
    else:
        loop, inputs, idx = torch_loop.rec_update_loop, ts[:10], list(range(8))
    torch_loop.grads(loop, inputs, idx, go)     # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        torch_loop.grads(loop, inputs, idx, go)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    tokens = w["B"] * w["T"]
    return {"value": tokens / med, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"full batch of the workload, PyTorch step loop fwd+bwd on the host, median of {reps} runs "
                      f"({med * 1e3:.0f} ms each)"}


LM_CONFIG = dict(n_token=32768, n_layer=16, n_head=8, d_model=256, d_head=32, d_inner=1024)
LM_BATCH, LM_LEN = 32, 1024


def zipf_tokens(n_token, shape, s=1.1, seed=0):
    """i.i.d. draws from Zipf(s) truncated to the vocabulary: P(rank r) ~ r^-s."""
    import numpy as np
    p = np.arange(1, n_token + 1, dtype=np.float64) ** -s
    cdf = np.cumsum(p / p.sum())
    u = np.random.default_rng(seed).random(shape)
    return np.minimum(np.searchsorted(cdf, u), n_token - 1).astype(np.int64)


def run_lm(args, pkg):
    """Forward + backward of the 16-layer Delta-Net language model (random init, Zipf tokens): the
    operator measured where the reference uses it.  Reports whole-model tokens/s and the share of the
    step spent in the fast-weight kernels (timed on their own at the shape the layers give them)."""
    import torch
    torch.manual_seed(0)
    model = pkg.DeltaNetLM(**LM_CONFIG).to("cuda:0")
    toks = torch.from_numpy(zipf_tokens(LM_CONFIG["n_token"], (LM_LEN + 1, LM_BATCH))).to("cuda:0")
    data, target = toks[:-1], toks[1:]
    params = [p for p in model.parameters()]
    torch.autograd.set_multithreading_enabled(False)

    def step():
        (loss,) = model(data, target)
        grads = torch.autograd.grad(loss.mean(), params)
        return loss, grads

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss, _ = step()
    torch.cuda.synchronize()
    step_s = (time.perf_counter() - t0) / args.steps
    tokens = LM_BATCH * LM_LEN

    w = WORKLOADS["delta_lm"]
    t_f, t_b, _ = kernel_times("delta_lm", pkg, make_inputs("delta_lm", w), 20)
    D, th = w["D"], w["B"] * w["H"] * w["T"]
    op_s = LM_CONFIG["n_layer"] * (t_f + t_b)
    dom_t, dom_bytes = (t_b, w["bwd_bytes"](D) * th) if t_b >= t_f else (t_f, w["fwd_bytes"](D) * th)
    result = {
        "metric": "Delta-Net LM training tokens/s (fwd+bwd), 1 GPU", "value": tokens / step_s, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": step_s * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (Zipf(1.1) tokens, random-init weights)",
        "config": {"workload": "16-layer Delta-Net LM fwd+bwd, d_model=256 H=8 D=32 FFN=1024 vocab=32768, "
                               "B=32 T=1024, fp32", **LM_CONFIG, "B": LM_BATCH, "T": LM_LEN},
        "loss": float(loss.mean()),
        "roofline": {"bound": "hbm", "kernel": "delta bwd at B=32 H=8 T=1024 D=32",
                     "achieved": dom_bytes / dom_t / 1e9, "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": dom_bytes / dom_t / PEAK_HBM, "traffic": None},
        "fast_weight_op": {"fwd_us": t_f * 1e6, "bwd_us": t_b * 1e6, "per_step_ms": op_s * 1e3,
                           "share_of_step": op_s / step_s},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = lm_cpu_baseline(pkg)
    return result


def lm_cpu_baseline(pkg):
    """The same model with the PyTorch step loop as operator on the host cores, on a slice of the batch."""
    import torch
    from oracle.torch_loop import delta_loop
    cores = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        cores = min(cores, int(env))
    torch.set_num_threads(cores)

    def loop_op(q, k, v, beta, W):
        out, W_end = delta_loop(q, k, v, beta, W.clone())
        W.copy_(W_end.detach())
        return out

    torch.manual_seed(0)
    model = pkg.DeltaNetLM(fast_weight_op=loop_op, **LM_CONFIG)
    B, T = 4, 128
    toks = torch.from_numpy(zipf_tokens(LM_CONFIG["n_token"], (T + 1, B)))
    params = list(model.parameters())
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        (loss,) = model(toks[:-1], toks[1:])
        torch.autograd.grad(loss.mean(), params)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times[1:])
    return {"value": B * T / med, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"the same 16-layer model, B={B} T={T} slice, PyTorch step loop as operator, fwd+bwd, "
                      f"median of 2 runs after a warm-up ({med:.1f} s each)"}


def run_single_steps(args, pkg):
    """Stepwise inference: one call per time step (T = 1, no gradient, state carried in W and h), as an
    actor or a decoder makes them.  Reported per operator: through the package's default entry point (the
    single-step kernels), the same with those kernels switched off (the kernels written for sequences), and
    through the Python autograd.Function."""
    import numpy as np
    import torch
    from helpers import delta_inputs, rec_inputs, rnn_inputs
    B, H, D = 32, 8, 32
    dev = lambda arrays: [torch.from_numpy(a).to("cuda:0") for a in arrays]
    q, k, v, beta, W0, _ = dev(delta_inputs(0, B, H, 1, D, D, dtype=np.float32))
    z, rk, rv, rW0, rbeta, rh0, _ = dev(rnn_inputs(0, B, H, 1, D, dtype=np.float32))
    rec = dev(rec_inputs(0, B, H, 1, D, dtype=np.float32))
    W, h = W0.clone(), rh0.clone()
    calls = {
        "fast_weight_delta": (lambda f: f(q, k, v, beta, W), pkg.fast_weight_delta, pkg.DeltaFastWeight.apply),
        "fast_rnn_v2": (lambda f: f(z, rk, rv, W, rbeta, h), pkg.fast_rnn_v2, pkg.FastRNNv2.apply),
        "rec_update_fwm_tanh": (lambda f: f(*rec[:8], W, h), pkg.rec_update_fwm_tanh,
                                pkg.FastWeightRecUpdateTanh.apply),
    }
    n = max(args.steps, 1) * 10
    out = {}
    with torch.no_grad():
        for name, (call, default, python) in calls.items():
            for label, f in (("default", default), ("sequence_kernels", default), ("python_function", python)):
                # "sequence_kernels": the same calls with the single-step kernels switched off
                pkg._lib.config(pkg._lib.CFG_STEP_KERNELS, int(label != "sequence_kernels"))
                for _ in range(args.warmup):
                    call(f)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(n):
                    call(f)
                torch.cuda.synchronize()
                out.setdefault(name, {})[label + "_us"] = (time.perf_counter() - t0) / n * 1e6
                if label != "python_function":
                    # what a caller that needs each step's result before the next sees: call + wait
                    m = max(n // 10, 1)
                    t0 = time.perf_counter()
                    for _ in range(m):
                        call(f)
                        torch.cuda.synchronize()
                    out[name][label + "_waited_us"] = (time.perf_counter() - t0) / m * 1e6
    lat = out["fast_weight_delta"]["default_us"] * 1e-6
    return {"metric": "stepwise inference tokens/s (one forward call per time step, no gradient), 1 GPU",
            "value": B / lat, "unit": "tokens/s", "n_gpus": 1, "steps": n, "warmup": args.warmup,
            "ms_per_step": lat * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32", "data": "synthetic",
            "config": {"workload": "single steps: fast_weight_delta forward, B=32 H=8 T=1 D=32, state carried",
                       "B": B, "H": H, "T": 1, "D": D},
            "roofline": None, "cpu_baseline": None, "latency_us_per_call": out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 2000; 200 for the language model)")
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps before them (default a tenth of --steps: a step takes ~50 us and "
                         "the first milliseconds on a cold GPU run 10 %% slower)")
    ap.add_argument("--workload", choices=sorted(WORKLOADS) + ["lm", "step"], default="delta")
    ap.add_argument("--cpu-reps", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--delta-kernels", choices=["auto", "scan", "chunked", "split", "phase"], default="auto",
                    help="delta-rule kernels for D=16/32: step-by-step register-state scan or 16-step blocks "
                         "on the matrix cores (default: the library's choice)")
    ap.add_argument("--lib", metavar="PATH",
                    help="take the kernel-timing leg's launches from this build of libfwp_hip.so (a variant built "
                         "for a measurement); the eager step still runs on the package's own library")
    ap.add_argument("--dims", nargs=5, type=int, metavar=("B", "H", "T", "E", "M"),
                    help="with --workload delta or sum and --kernel-leg-only: another batch and state shape (E key features, "
                         "M value columns) for the per-kernel leg, e.g. 32 8 512 64 64")
    ap.add_argument("--kernel-leg-only", action="store_true",
                    help="only the per-kernel leg (back-to-back launches through the C ABI): for profiles of a "
                         "build given with --lib, whose kernels must not mix with the package's own in a trace")
    ap.add_argument("--graph", action="store_true",
                    help="time a HIP graph replay of the step recorded through the C ABI instead of eager calls")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run five device-to-device copies of 2 GiB (a kernel of known traffic for "
                         "scaling rocprofv3's FETCH_SIZE / WRITE_SIZE) and exit")
    ap.add_argument("--stream-floor", action="store_true",
                    help="only time plain device-to-device copies of one of the workload's [B,H,T,D] arrays, back to "
                         "back like the kernels (what moving the step's algorithmic bytes costs at this size), and exit")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="rewrite this workload's entry of profiles/hbm_traffic.txt from the output directories "
                         "of `rocprofv3 --pmc FETCH_SIZE` and `rocprofv3 --pmc WRITE_SIZE` runs of it, and exit")
    args = ap.parse_args()
    if args.traffic_from:
        update_traffic(args.workload, *args.traffic_from)
        return
    if args.steps is None:
        args.steps = 200 if args.workload == "lm" else 2000
    if args.warmup is None:
        args.warmup = max(args.steps // 10, 1)
    if args.copy_calibration:
        import torch
        src = torch.ones(512 * 1024 * 1024, device="cuda:0")      # 2 GiB: far beyond every cache level
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": src.numel() * 4, "copy_bytes_written": src.numel() * 4}))
        return
    if args.stream_floor:
        print(json.dumps(stream_floor(args.workload if args.workload in WORKLOADS else "delta")))
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (sequences are independent; "
                 "more GPUs would just split the batch). Use --gpus 1.")

    import torch
    from __graft_entry__ import package
    pkg = package()
    if args.lib:
        # the C++ functions are linked against the package's own library and keep using it; the ctypes binding,
        # which the per-kernel leg and the C-ABI window go through, loads the given one
        pkg._lib.SO_PATH = os.path.abspath(args.lib)
    pkg._lib.lib()                       # fails loudly if the HIP library is not built
    pkg._lib.config(pkg._lib.CFG_DELTA_KERNELS, {"auto": 0, "scan": 1, "chunked": 2, "split": 3, "phase": 4}[args.delta_kernels])
    name = args.workload
    if name == "lm":
        print(json.dumps(run_lm(args, pkg)))
        return
    if name == "step":
        print(json.dumps(run_single_steps(args, pkg)))
        return
    w = WORKLOADS[name]
    if args.dims:
        if name not in ("delta", "sum") or not args.kernel_leg_only:
            sys.exit("bench.py: --dims goes with --workload delta or sum and --kernel-leg-only")
        B, H, T, E, M = args.dims
        w = dict(w, B=B, H=H, T=T, E=E, M=M, label=w["label"].split(",")[0] + f", B={B} H={H} T={T} E={E} M={M}, fp32")
    arrays = make_inputs(name, w)
    B, H, T, D = w["B"], w["H"], w["T"], w["D"]
    tokens = B * T
    token_heads = tokens * H

    # run backward on the calling thread: the hand-over to the autograd engine's device thread costs
    # more than the kernels of this step take
    torch.autograd.set_multithreading_enabled(False)
    step, _ = gpu_step_fn(name, pkg, arrays)

    def timed_steps(fn, warmup=None, steps=None):
        """(seconds per step, seconds of host time per step spent issuing) over `steps` steps after `warmup`
        untimed ones, a synchronisation on either side."""
        warmup = args.warmup if warmup is None else warmup
        steps = args.steps if steps is None else steps
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        t_issued = time.perf_counter()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps, (t_issued - t0) / steps

    # Three legs, in this order.  (1) The per-kernel leg: back-to-back launches through the C ABI.  (2) The
    # steady state of the eager step: 2000 steps after 200, as a training loop runs them.  (3) The window the
    # command line asks for: --warmup untimed steps, then exactly --steps timed ones; `value` is this one.
    # With the default command of a fresh box (20 steps after 5, one millisecond of work) leg (3) on its own
    # measured the process warming up - the first few hundred calls of the eager path issue 10-40 % slower
    # than later ones, and the GPU runs a 1 ms burst after an idle spell 10 % slower than sustained work -
    # so it comes last; legs (1) and (2) are reported beside it under "kernels" and "steady".
    t_f, t_b, abi_step = kernel_times(name, pkg, arrays, 100)
    if args.kernel_leg_only:
        th = B * H * T
        fwd_bytes, bwd_bytes = w["fwd_bytes"](D), w["bwd_bytes"](D)
        if args.dims:       # at E x M, per token-head: forward 2E + 2M (+ 1: beta) floats, backward 4E + 3M (+ 2)
            extra = name == "delta"
            fwd_bytes, bwd_bytes = (2 * w["E"] + 2 * w["M"] + extra) * 4, (4 * w["E"] + 3 * w["M"] + 2 * extra) * 4
        t_step, _ = timed_steps(abi_step, 20, 200)      # state reset + forward + backward, through the C ABI
        print(json.dumps({"workload": w["label"], "lib": pkg._lib.SO_PATH, "fwd_us": t_f * 1e6, "bwd_us": t_b * 1e6,
                          "fwd_GBps": fwd_bytes * th / t_f / 1e9, "bwd_GBps": bwd_bytes * th / t_b / 1e9,
                          "c_abi_step_us": t_step * 1e6}))
        return
    steady_steps = 2000 if w["T"] * w["B"] * w["H"] * w["D"] <= 96 * 8 * 256 * 16 * 2 else 300
    steady_s, steady_issue_s = timed_steps(step, steady_steps // 10, steady_steps)
    abi_s, _ = timed_steps(abi_step, 5, 20)
    eager_s, eager_issue_s = timed_steps(step)
    launch = "eager calls of the autograd Function"
    step_s = eager_s
    if args.graph:
        # The same three launches (state reset, forward, backward) recorded once into a HIP graph
        # through the C ABI on preallocated buffers and replayed: no Python or autograd-engine time
        # between the kernels.
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                abi_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            abi_step()
        step_s, _ = timed_steps(graph.replay)
        launch = "hipGraph replay of reset+forward+backward recorded through the C ABI"
    ms = step_s * 1e3
    value = tokens / step_s

    fwd_bytes = w["fwd_bytes"](D) * token_heads
    bwd_bytes = w["bwd_bytes"](D) * token_heads
    dom = "bwd" if t_b >= t_f else "fwd"
    dom_bytes, dom_t = (bwd_bytes, t_b) if dom == "bwd" else (fwd_bytes, t_f)
    flops = w["flop_c"] * D * D * token_heads
    kernel_s = t_f + t_b
    result = {
        "metric": METRIC, "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": w["label"], "B": B, "H": H, "T": T, "D": D, "launch": launch},
        "roofline": {"bound": "hbm", "kernel": f"{name} {dom}", "achieved": dom_bytes / dom_t / 1e9,
                     "peak": PEAK_HBM / 1e9, "unit": "GB/s", "frac": dom_bytes / dom_t / PEAK_HBM,
                     "traffic": measured_traffic().get(name, {}).get(dom)},
        "kernels": {"fwd_us": t_f * 1e6, "bwd_us": t_b * 1e6,
                    "fwd_GBps": fwd_bytes / t_f / 1e9, "bwd_GBps": bwd_bytes / t_b / 1e9,
                    "kernel_only_tokens_per_s": tokens / kernel_s,
                    "valu_frac_of_157.3TF": flops / kernel_s / PEAK_VALU,
                    "hbm_frac_of_8TBps": (fwd_bytes + bwd_bytes) / kernel_s / PEAK_HBM,
                    "step_valu_frac_of_157.3TF": flops / (ms * 1e-3) / PEAK_VALU,
                    "eager_tokens_per_s": tokens / eager_s, "eager_ms_per_step": eager_s * 1e3},
        # host time per step spent issuing the timed steps (the rest of a step's time the host waits for the GPU)
        "issue_ms_per_step": eager_issue_s * 1e3,
        # the same eager step in steady state, and reset + forward + backward straight through the C ABI on
        # preallocated buffers (no allocation, no autograd engine) in a window of 20 steps after 5
        "steady": {"steps": steady_steps, "ms_per_step": steady_s * 1e3, "tokens_per_s": tokens / steady_s,
                   "issue_ms_per_step": steady_issue_s * 1e3},
        "c_abi_step": {"steps": 20, "ms_per_step": abi_s * 1e3, "tokens_per_s": tokens / abi_s},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(name, arrays, w, args.cpu_reps)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
