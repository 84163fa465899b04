"""The C++ host mirror (rstorch_amd/cpp/rstorch.hpp): the reference's unit tests for the path and
the README training loop, compiled against the C ABI and run on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rstorch_amd", "cpp", "bin")


def _run(name, *args):
    exe = os.path.join(BIN, name)
    assert os.path.exists(exe), "build the C++ mirror first (__graft_entry__.build())"
    return subprocess.run([exe, *args], capture_output=True, text=True, timeout=120)


def test_reference_unit_tests_on_the_mirror():
    out = _run("test_mirror")
    assert out.returncode == 0, out.stdout + out.stderr
    assert "all mirror tests passed" in out.stdout


def test_readme_loop_trains():
    out = _run("readme_loop", "2", "300")
    assert out.returncode == 0, out.stdout + out.stderr
    lines = [l for l in out.stdout.splitlines() if l.startswith("EPOCH")]
    assert len(lines) == 2
    losses = [float(l.split("loss")[1].split("-")[0]) for l in lines]
    assert losses[1] < losses[0] < 2.5  # fits the fixed pool of batches: the loss goes down
    assert "Sequential { layers: [Identity, Linear(784, 100), ReLU, Linear(100, 100), ReLU, Linear(100, 10)] }" in out.stdout


def test_fresh_input_loops_agree_whichever_stream_generates():
    """train_loop: the single-call step on inputs regenerated every step, once with a second engine
    refilling the other of two buffers behind events, once with the generator on the training stream.
    Same generator streams, same steps: the last loss is the same number, which it is only if every
    step saw its own batch complete (a hand-over that lets a step start early, or a refill that
    overwrites a batch still being read, changes it)."""
    two = _run("train_loop", "C0", "600", "50", "loss")
    one = _run("train_loop", "C0", "600", "50", "loss", "one-stream")
    assert two.returncode == 0 and one.returncode == 0, two.stdout + two.stderr + one.stdout + one.stderr
    last = lambda out: out.stdout.split("last loss ")[1].split()[0]
    assert last(two) == last(one)
    assert 0.0 < float(last(two)) < 2.5
    big_two = _run("train_loop", "C1", "60", "10")
    big_one = _run("train_loop", "C1", "60", "10", "one-stream")
    assert big_two.returncode == 0 and big_one.returncode == 0, big_two.stderr + big_one.stderr
    assert last(big_two) == last(big_one)
