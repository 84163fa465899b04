"""The host side of the C-ABI library under AddressSanitizer + UBSan, without a GPU.

tests/host_stub builds every source of rstorch_amd/csrc for the host only (hipcc --cuda-host-only)
against a stand-in HIP runtime whose device memory is host memory and whose launches do nothing,
and runs a driver through the benchmark's call sequence at its real shapes (big model with a
recorded step graph, its destruction, the SGD-only runs, freshly built small models), two models and
operator-level calls sharing an engine, the layer-by-layer state machine, every route of the
contraction planner, the stager's slot accounting and the teardown.  It checks what a CPU can check:
status codes, allocation and graph lifetimes (double frees, launches of destroyed graphs, allocation
or synchronisation during stream capture abort the run), heap misuse and undefined behaviour in the
planners.  No numerical result comes out of it - kernels never run there."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host_stub")


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"),
                    reason="needs hipcc to compile the host side")
def test_host_logic_is_clean_under_asan_and_ubsan():
    build = subprocess.run(["make", "-C", HERE, "-j8", "-s"], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([os.path.join(HERE, "build", "host_logic_driver")], capture_output=True, text=True,
                         env=env, timeout=300)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert "host logic ok" in run.stdout
    assert "ERROR: AddressSanitizer" not in run.stderr and "runtime error" not in run.stderr
