"""The addressing of the contraction kernels, checked on the CPU before anything reaches a GPU.

tests/host_stub/address_sweep_driver.cpp plans a few thousand contractions (ragged extents, M = 2,
K not a multiple of 16, rows of 70000 doubles, leading dimensions just under and at 2^22 and 2^26,
misaligned and odd operands, every epilogue, every workspace mode, grouped and paired launches) with
the library's own planner; tests/host_stub/address_model.cpp walks every workgroup, wavefront and
lane of every planned grid through the index functions the kernels themselves use
(rstorch_amd/csrc/gemm_addressing.h) and aborts on the first read or write outside its operand, LDS
stage or workspace, on a K slice that is multiplied twice or never, and on an output element that is
stored twice or never.  The driver also fails when a kernel or a route of the planner is not reached."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host_stub")


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"),
                    reason="needs hipcc to compile the host side")
def test_every_planned_lane_stays_inside_its_operand():
    build = subprocess.run(["make", "-C", HERE, "-j8", "-s"], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    run = subprocess.run([os.path.join(HERE, "build", "address_sweep_driver")], capture_output=True, text=True,
                         timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert "address sweep ok" in run.stdout


MUTANTS = {
    # the tile DMA's last-row clamp, off by one
    "last_row_clamp": ("const int rr = o0 + row < ext ? row : ext - 1 - o0;",
                       "const int rr = o0 + row < ext ? row : ext - o0;"),
    # the last row of the contraction is not kept away from the tile DMA: the pair on the last column
    # of an odd, output-contiguous extent then reads one double behind the operand
    "last_k_row_not_kept_back": ("RST_HD int dma_whole_steps(int K, int k_reserve) { return (K - k_reserve) / BK; }",
                                 "RST_HD int dma_whole_steps(int K, int k_reserve) { return K / BK; }"),
}


@pytest.mark.parametrize("mutant", sorted(MUTANTS))
def test_the_model_catches_a_wrong_offset(tmp_path, mutant):
    """The checker is only worth something if it fails when the arithmetic is wrong: rebuild the
    model and the library's contraction source against a copy of the index header with one line
    changed, and the sweep must abort with a bounds message."""
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("needs hipcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    csrc = os.path.join(root, "rstorch_amd", "csrc")
    work = tmp_path / "mutant"
    shutil.copytree(os.path.join(root, "tests", "host_stub"), work / "tests" / "host_stub",
                    ignore=shutil.ignore_patterns("build"))
    shutil.copytree(csrc, work / "rstorch_amd" / "csrc")
    shutil.copytree(os.path.join(root, "include"), work / "include", ignore=shutil.ignore_patterns("__pycache__"))
    header = work / "rstorch_amd" / "csrc" / "gemm_addressing.h"
    text = header.read_text()
    good, wrong = MUTANTS[mutant]
    assert text.count(good) == 1
    header.write_text(text.replace(good, wrong))
    build = subprocess.run(["make", "-C", str(work / "tests" / "host_stub"), "-j8", "-s", "build/address_sweep_driver"],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    run = subprocess.run([str(work / "tests" / "host_stub" / "build" / "address_sweep_driver")],
                         capture_output=True, text=True, timeout=900)
    assert run.returncode != 0
    assert "address model:" in run.stderr and "outside the operand" in run.stderr
