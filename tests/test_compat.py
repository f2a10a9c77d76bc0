"""The import lines of the reference's layer code resolve, unchanged, to this implementation once
`compat/` is first on sys.path (algorithmic/layers.py:7-10,
language_modeling/src/utils/cuda_fast_weight_layer.py:9-23, reinforcement_learning/torchbeast/layer.py:7-10)."""
import os
import subprocess
import sys
import textwrap

import numpy as np
import pytest

import oracle
from helpers import delta_inputs, within

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
COMPAT = os.path.join(ROOT, "compat")

ALGORITHMIC = """
from fast_transformers import fast_weight_sum
from fast_weight import fast_weight_delta
from fast_weight_rnn_v2 import fast_rnn_v2
from rec_update_fwm_tanh import rec_update_fwm_tanh
"""
LANGUAGE_MODELING = """
from utils.fast_fast_weight import fast_weight_delta
from utils.fast_transformers import fast_weight_sum

# Delta RNN variants
from utils.fast_weight_rnn import fast_rnn
from utils.fast_weight_rnn_v2 import fast_rnn_v2

# Delta LSTM variants
from utils.fast_lstm import fast_lstm
from utils.fast_lstm_v2 import fast_lstm_v2
from utils.fast_lstm_v3 import fast_lstm_v3
from utils.fast_lstm_v4 import fast_lstm_v4

# Recurrent Delta Net
from utils.rec_update_fwm_tanh import rec_update_fwm_tanh
"""
TORCHBEAST = """
from torchbeast.fast_weight import fast_weight_delta
from torchbeast.fast_transformers import fast_weight_sum
from torchbeast.rec_update_fwm_tanh import rec_update_fwm_tanh
from torchbeast.fast_weight_rnn_v2 import fast_rnn_v2
"""


def run_fresh(code, extra_dirs=()):
    """In a fresh interpreter: compat first on sys.path, then `extra_dirs` (stand-ins for the
    reference's own directories), then the code."""
    head = "import sys\n" + "".join(f"sys.path.insert(0, {d!r})\n" for d in reversed((COMPAT, *extra_dirs)))
    r = subprocess.run([sys.executable, "-c", head + textwrap.dedent(code)], capture_output=True, text=True,
                       cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    return r.stdout


@pytest.mark.parametrize("lines", [ALGORITHMIC, LANGUAGE_MODELING, TORCHBEAST])
def test_reference_import_lines_resolve_to_this_package(lines):
    out = run_fresh(lines + """
import importlib
pkg = importlib.import_module("recurrent-fwp_amd")
for name in ("fast_weight_delta", "fast_weight_sum", "fast_rnn_v2", "rec_update_fwm_tanh"):
    assert globals()[name] is getattr(pkg, name), name
if "fast_lstm_v4" in globals():
    assert fast_lstm_v4 is pkg.fast_lstm_v4
    for old in (fast_rnn, fast_lstm, fast_lstm_v2, fast_lstm_v3):     # not built: loud, not silent
        try:
            old()
        except NotImplementedError:
            pass
        else:
            raise AssertionError(old)
print("resolved")
""")
    assert "resolved" in out


def test_other_modules_of_the_namespace_packages_are_still_found(tmp_path):
    """`utils` and `torchbeast` stay namespace packages: a module that only the caller's own
    directory has (utils.performer_helper in the reference) is found there, the operators here."""
    (tmp_path / "utils").mkdir()
    (tmp_path / "utils" / "performer_helper.py").write_text("prime = 7\n")
    (tmp_path / "utils" / "fast_fast_weight").mkdir()
    (tmp_path / "utils" / "fast_fast_weight" / "__init__.py").write_text("raise ImportError('the CUDA one')\n")
    out = run_fresh("""
from utils.fast_fast_weight import fast_weight_delta
from utils.performer_helper import prime
print("prime", prime, fast_weight_delta.__module__ if hasattr(fast_weight_delta, "__module__") else "")
""", extra_dirs=(str(tmp_path),))
    assert "prime 7" in out


def test_launcher_puts_the_shims_ahead_of_the_scripts_directory(tmp_path):
    (tmp_path / "fast_weight").mkdir()
    (tmp_path / "fast_weight" / "__init__.py").write_text("raise ImportError('the CUDA one')\n")
    (tmp_path / "main.py").write_text("import sys\nfrom fast_weight import fast_weight_delta\n"
                                      "import helper_next_to_script\nprint('ran', sys.argv[1:])\n")
    (tmp_path / "helper_next_to_script.py").write_text("")
    r = subprocess.run([sys.executable, os.path.join(COMPAT, "run.py"), str(tmp_path / "main.py"), "--x", "1"],
                       capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0 and "ran ['--x', '1']" in r.stdout, r.stdout + r.stderr


@pytest.mark.gpu
def test_one_operator_through_every_shim_path():
    import importlib
    import torch
    if COMPAT not in sys.path:
        sys.path.insert(0, COMPAT)
    q, k, v, beta, W0, go = delta_inputs(41, 2, 2, 48, 16, 16, dtype=np.float32, w0=True)
    want = oracle.delta_fwd(*(a.astype(np.float64) for a in (q, k, v, beta, W0)))[0]
    for path in ("fast_weight", "utils.fast_fast_weight", "torchbeast.fast_weight"):
        fn = importlib.import_module(path).fast_weight_delta
        out = fn(*(torch.from_numpy(a).cuda() for a in (q, k, v, beta)), torch.from_numpy(W0).cuda())
        assert within(out.cpu().numpy(), want, 1e-4, 1e-3), path
    z = torch.from_numpy(v).cuda()
    for path in ("fast_weight_rnn_v2", "utils.fast_weight_rnn_v2", "torchbeast.fast_weight_rnn_v2"):
        fn = importlib.import_module(path).fast_rnn_v2
        h0 = torch.zeros(2, 2, 1, 16, device="cuda")
        out = fn(z, torch.from_numpy(k).cuda(), z, torch.from_numpy(W0).cuda(), torch.from_numpy(beta).cuda(), h0)
        assert torch.isfinite(out).all() and torch.equal(h0[:, :, 0], out[:, :, -1]), path
    for path in ("fast_transformers", "utils.fast_transformers", "torchbeast.fast_transformers",
                 "rec_update_fwm_tanh", "utils.rec_update_fwm_tanh", "torchbeast.rec_update_fwm_tanh",
                 "utils.fast_lstm_v4"):
        mod = importlib.import_module(path)
        assert callable(getattr(mod, path.split(".")[-1].replace("fast_transformers", "fast_weight_sum")))
