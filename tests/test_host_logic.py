"""Host-side logic that needs no GPU: the Sequential container, the builder, bench.py's flags."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_sequential_container_operations():
    """src/module/sequential.rs:16-60: new / push / insert / remove / len / is_empty."""
    import rstorch_amd as rs
    m = rs.Sequential.new([])
    assert m.is_empty() and m.len() == 0
    a, b, c = rs.Identity.new(), rs.ReLU.new(), rs.Identity.new()
    m.push(a); m.push(c); m.insert(1, b)
    assert m.layers == [a, b, c] and m.len() == 3 and not m.is_empty()
    assert m.remove(5) is None and m.len() == 3      # out of range -> None, as in the reference
    assert m.remove(0) is a and m.layers == [b, c]
    m.push_box(a); m.insert_box(0, c)
    assert m.len() == 4
    assert len(m.parameters()) == 0
    m.train(); m.eval()


def test_sequential_builder_spellings():
    import rstorch_amd as rs
    m = rs.sequential((rs.Identity,), rs.ReLU.new(), rs.ReLU)
    assert [type(l) for l in m.layers] == [rs.Identity, rs.ReLU, rs.ReLU]


def test_identity_passes_anything_through():
    import rstorch_amd as rs
    obj = object()
    assert rs.Identity.new().forward(obj) is obj and rs.Identity.new().backward(obj) is obj


def test_initialiser_sigmas():
    """he.rs:12, xavier.rs:12, sigma.rs:15-21."""
    import math
    import rstorch_amd as rs
    assert rs.KaimingNormal()._sigma(784, 100) == 1.0 / math.sqrt(784.0)
    assert rs.XavierNormal()._sigma(30, 20) == math.sqrt(2.0 / 50.0)
    assert rs.Normal.new(0.0, float("inf")) is None and rs.Normal.new_std(0.5).std == 0.5


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True)
    assert out.returncode != 0 and "ONE GPU" in out.stderr


def test_hip_flags_disable_packed_fp32_and_contraction():
    from rstorch_amd import _build
    flags = " ".join(_build.HIP_FLAGS)
    assert "-packed-fp32-ops" in flags and "-ffp-contract=off" in flags and "gfx950" in flags


def test_traffic_figure_belongs_to_the_current_kernel_sources():
    """bench.py reports roofline.traffic from a committed counter profile (profiles/c4_hbm_traffic.md);
    the figure is only valid for the kernel sources it was measured on.  When this fails, collect the
    profile again and update C4_TRAFFIC_BYTES_PER_LAUNCH and the digest in bench.py."""
    sys.path.insert(0, ROOT)
    import bench
    assert bench.kernel_sources_digest() == bench.C4_TRAFFIC_SOURCE["kernel_sources_sha16"]
