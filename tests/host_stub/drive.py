"""Drives the host build of the C++ autograd functions (see build.sh) on host tensors: forward and backward
of every operator with the autograd engine's worker threads on and off, from the main thread and from
other Python threads at once, saved tensors freed early, graphs run twice, permuted and unaligned views.
Run as a script (python drive.py BUILD_DIR [python]; with "python" the package's Python autograd.Functions
over ctypes are driven instead of the C++ ones), normally by tests/test_binding_host.py; under AddressSanitizer
every read and write of the stand-in library is checked against the buffers the binding handed it.
Prints 'host stub drive ok' at the end."""
import gc
import importlib.util
import sys
import threading

import torch


def load(build_dir):
    spec = importlib.util.spec_from_file_location("_fwp_torch_host", build_dir + "/_fwp_torch_host.so")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


class PythonFunctions:
    """The package's Python autograd.Functions over ctypes with the stand-in library in place of the real
    one: host tensors pass the device check, the stream is NULL."""

    def __init__(self, build_dir):
        import os
        root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
        sys.path.insert(0, root)
        pkg = importlib.import_module("recurrent-fwp_amd")
        L_ = pkg._lib
        L_._lib = None
        L_.SO_PATH = build_dir + "/libfwp_hip.so"
        L_.require_device = lambda t: None
        L_.stream_of = lambda t: None
        L_.on_device = lambda t: L_._NO_GUARD
        L_._query_cache.clear()
        self.fast_weight_delta = lambda q, k, v, beta, W, tm: pkg.DeltaFastWeight.apply(q, k, v, beta, W, tm)
        self.fast_weight_sum = lambda q, k, v, W, exact: self._sum(pkg, q, k, v, W, exact)
        self.fast_rnn_v2 = pkg.FastRNNv2.apply
        self.rec_update_fwm_tanh = pkg.FastWeightRecUpdateTanh.apply
        self.fast_lstm_v4 = pkg.FastLSTMv4.apply

    @staticmethod
    def _sum(pkg, q, k, v, W, exact):
        pkg.FastWeightSum.state_gradient = "exact" if exact else "reference"
        return pkg.FastWeightSum.apply(q, k, v, W)


def rnd(*shape, grad=False):
    return torch.randn(*shape, requires_grad=grad)


def delta_case(m, N, H, L, E, M, time_major, views):
    if views:      # the reference's layers: permuted views of [L,N,H,.] storage; v a slice of a wider projection
        big = torch.randn(L, N, H, 2 * E + M + 1, requires_grad=True)
        q, k, v, beta = (big[..., :E].permute(1, 2, 0, 3), big[..., E:2 * E].permute(1, 2, 0, 3),
                         big[..., 2 * E:2 * E + M].permute(1, 2, 0, 3), big[..., -1:].permute(1, 2, 0, 3))
        leaves = [big]
    else:
        q, k, v, beta = rnd(N, H, L, E, grad=True), rnd(N, H, L, E, grad=True), rnd(N, H, L, M, grad=True), rnd(N, H, L, 1, grad=True)
        leaves = [q, k, v, beta]
    W = torch.zeros(N, H, E, M)
    out = m.fast_weight_delta(q, k, v, beta, W, time_major)
    assert out.shape == (N, H, L, M)
    assert bool((W == 1).all())
    go = torch.randn(N, H, L, M)
    grads = torch.autograd.grad(out, leaves, go, retain_graph=True)
    again = torch.autograd.grad(out, leaves, go)
    for a, b, leaf in zip(grads, again, leaves):
        assert a.shape == leaf.shape and torch.equal(a, b)
    try:
        torch.autograd.grad(out, leaves, go)
    except RuntimeError as e:
        assert "second time" in str(e) or "freed" in str(e), e
    else:
        raise AssertionError("a third backward through a freed graph must raise")
    # the result outlives everything it was computed from
    del q, k, v, beta, W, leaves, go
    gc.collect()
    return float(out.detach().sum()) + sum(float(g.sum()) for g in grads)


def others_case(m, N, H, L, D):
    total = 0.0
    q, k, v = (rnd(N, H, L, D, grad=True) for _ in range(3))
    W = torch.zeros(N, H, D, D)
    for exact in (False, True):
        out = m.fast_weight_sum(q, k, v, W, exact)
        total += sum(float(g.sum()) for g in torch.autograd.grad(out, [q, k, v], torch.randn(N, H, L, D)))
    beta = rnd(N, H, L, 1, grad=True)
    h0 = torch.zeros(N, H, 1, D)
    out = m.fast_rnn_v2(q, k, v, W, beta, h0)
    out.sum().backward()
    total += float(q.grad.sum())
    Rs = [rnd(1, H, D, D, grad=True) for _ in range(3)] + [rnd(1, H, 1, D, grad=True)]
    out = m.rec_update_fwm_tanh(q, k, v, beta, *Rs, W, h0)
    gs = torch.autograd.grad(out, [q, k, v, beta] + Rs, torch.randn(N, H, L, D))
    assert [g.shape for g in gs[4:]] == [R.shape for R in Rs]
    total += sum(float(g.sum()) for g in gs)
    args = []
    for _ in range(3):
        args += [rnd(N, H, L, D, grad=True), rnd(N, H, L, D, grad=True), rnd(N, H, L, D, grad=True),
                 rnd(N, H, L, 1, grad=True), torch.zeros(N, H, D, D)]
    out, cell = m.fast_lstm_v4(*args, torch.zeros(N, H, 1, D), torch.zeros(N, H, 1, D))
    diff = [a for a in args if a.requires_grad]
    gs = torch.autograd.grad(out, diff, torch.randn(N, H, L, D))
    total += sum(float(g.sum()) for g in gs)
    with torch.no_grad():
        m.fast_weight_delta(q, k, v, beta, W, None)
    return total


def worker(m, seed, results):
    torch.manual_seed(seed)
    acc = 0.0
    for rep in range(6):
        for tm in (None, True, False):
            for views in (False, True):
                acc += delta_case(m, 2 + rep % 2, 3, 33 + rep, 16, 16 + 16 * (rep % 2), tm, views)
        # value widths that run by slices of value columns: 3 D + 1 (a padded last slice, rows that are not
        # 16-byte aligned), 128 (two slices written in place), 128 keys with 64 values
        for E, M in ((32, 97), (32, 128), (128, 64)):
            acc += delta_case(m, 2, 2, 20 + rep, E, M, (None, True, False)[rep % 3], rep % 2 == 1)
        acc += others_case(m, 2, 2, 17 + rep, 16)
    results[seed] = acc


def main():
    m = PythonFunctions(sys.argv[1]) if "python" in sys.argv[2:] else load(sys.argv[1])
    for threaded in (True, False):
        torch.autograd.set_multithreading_enabled(threaded)
        results = {}
        worker(m, 0, results)
        threads = [threading.Thread(target=worker, args=(m, s, results)) for s in (1, 2, 3)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert len(results) == 4 and all(r == r for r in results.values()), results
    print("host stub drive ok")


if __name__ == "__main__":
    main()
