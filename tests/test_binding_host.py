"""The host side of the operators without a GPU: csrc/fwp_torch.cpp built with -DFWP_HOST_STUB (host tensors,
NULL stream) against a stand-in library that launches nothing but reads every input and writes every output
of a call on the host (tests/host_stub/).  tests/host_stub/drive.py runs forward and backward of every
operator through it, with the autograd engine's worker threads on and off and from several Python threads
at once; the Python autograd.Functions over ctypes are driven the same way.  What this pins: shapes, saved
tensors and their lifetimes, the one-allocation gradient views, errors for a graph run twice - the host
logic that a GPU test would only exercise through its results.

With FWP_HOST_ASAN=1 both libraries are built with -fsanitize=address and the driver runs with libasan
preloaded, so every access of the stand-in library is checked against the buffers the binding gave it
(about three minutes; off by default)."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
STUB = os.path.join(HERE, "host_stub")


@pytest.fixture(scope="module")
def build(tmp_path_factory):
    asan = os.environ.get("FWP_HOST_ASAN") == "1"
    out = str(tmp_path_factory.mktemp("host_stub"))
    subprocess.run(["bash", os.path.join(STUB, "build.sh"), out] + (["asan"] if asan else []), check=True,
                   capture_output=True, timeout=600)
    env = dict(os.environ)
    if asan:
        libs = [subprocess.run(["gcc", "-print-file-name=" + n], check=True, capture_output=True,
                               text=True).stdout.strip() for n in ("libasan.so", "libstdc++.so")]
        # the sanitizer's runtime has to come first; whatever is preloaded already stays behind it
        env["LD_PRELOAD"] = ":".join(libs + [p for p in env.get("LD_PRELOAD", "").split(":") if p])
        env["ASAN_OPTIONS"] = "detect_leaks=0:halt_on_error=1"
    return out, env


@pytest.mark.parametrize("functions", ["cpp", "python"])
def test_host_side_of_every_operator_against_the_stand_in_library(build, functions):
    out, env = build
    cmd = [sys.executable, os.path.join(STUB, "drive.py"), out] + (["python"] if functions == "python" else [])
    run = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=1500, cwd=out)
    assert run.returncode == 0 and "host stub drive ok" in run.stdout, run.stdout[-2000:] + run.stderr[-4000:]
