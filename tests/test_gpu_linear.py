"""Linear forward/backward on the GPU (through the C ABI) against the CPU oracle.

Tolerance: max|got-want| / max|want| <= 1e-10 per tensor (the bound BASELINE.json states for
logits and every dW/db); the contraction order differs from the oracle's, so results are not
bit-identical."""
import json
import os

import numpy as np
import pytest

from conftest import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-10
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")


def _linear(rs, w, b):
    return rs.Linear.new_with_kernel(w.shape[1], w.shape[0], rs.FromArrays(w, b))


SHAPES = [
    (1, 1, 1), (3, 2, 1), (2, 3, 10), (32, 784, 100), (32, 100, 100), (32, 100, 10),
    (37, 101, 13), (5, 7, 3), (129, 17, 130), (64, 64, 64), (100, 300, 33),
    (512, 256, 384), (1024, 128, 1000), (256, 1024, 1024), (2048, 100, 10),
    # >= 256 tiles of 128x128 with ragged edges: the direct-to-LDS kernels (K % 16 == 0) and the
    # register-staged kernel with a K tail, for each of the three operand layouts
    (2050, 64, 2046), (2064, 2046, 2046), (2050, 2046, 2048),
    # 256..511 tiles: one workgroup per CU on the direct-to-LDS kernels
    (2064, 2048, 2046),
    # 32..255 tiles with a long contraction: the direct-to-LDS kernels on up to eight K slices
    # (forward 128 tiles x 4 slices, input gradient 64 tiles x 8; ragged: 128 tiles x 4; weight
    # gradient with its bias gradient over 4 slices)
    (512, 2048, 4096), (498, 2048, 4094), (2048, 1024, 1000),
    # the same with a K remainder (a masked extra tile in slice 0), and K below one whole step
    (512, 2056, 4096), (2048, 1000, 4096), (2048, 10, 2048),
    # fewer than 256 tiles of 128x128 and a contraction of up to 1024: the 64x64 direct-to-LDS kernel -
    # forward unsplit with a K remainder, forward on two K slices, input gradient of a narrow layer
    # (128-wide tiles would be half empty) on four K slices, ragged edges
    (2048, 1000, 512), (1024, 1024, 512), (4096, 64, 2048), (2050, 1022, 510), (16384, 512, 64),
    # small outputs with a long contraction: the split-K path (with and without a K tail)
    (8192, 784, 100), (8192, 100, 10), (32, 4099, 24), (4100, 7, 9), (16384, 33, 65),
    # odd extents and leading dimensions on the direct-to-LDS kernels (8-byte aligned pairs; where an
    # output-contiguous operand has an odd extent the last row of the contraction goes with the tail):
    # 128x128 tiles unsliced and on K slices, a batch that is a multiple of 16 (the tail is then a
    # whole step), the 64x64 tiles, a single last column in a tile of its own (1025 = 8 x 128 + 1)
    (2047, 1023, 4095), (2048, 1023, 4095), (2049, 2047, 1025), (8192, 785, 101), (1031, 4097, 515),
    # forward products of 257..511 tiles of 128x128: K slices even out the compute units that would
    # otherwise get two tiles against one (288 tiles on two slices; 324 ragged tiles with a K remainder)
    (1024, 2048, 4608), (1030, 2056, 4600),
]


@pytest.mark.parametrize("batch,k,n", SHAPES)
@pytest.mark.parametrize("fuse_relu", [False, True])
def test_forward_matches_oracle(engine, oracle, batch, k, n, fuse_relu):
    import rstorch_amd as rs
    rng = np.random.default_rng(batch * 1000003 + k * 1009 + n)
    x = rng.standard_normal((batch, k))
    w = rng.standard_normal((n, k)) / np.sqrt(k)
    b = rng.standard_normal((1, n))
    lin = _linear(rs, w, b)
    got = lin._forward(x, fuse_relu).to_numpy()
    want = oracle.linear_forward(x, w, b)
    if fuse_relu:
        want = oracle.relu_forward(want)
    assert rel_err(got, want) <= TOL


@pytest.mark.parametrize("batch,k,n", SHAPES)
def test_backward_matches_oracle(engine, oracle, batch, k, n):
    import rstorch_amd as rs
    rng = np.random.default_rng(batch * 7919 + k * 31 + n)
    x = rng.standard_normal((batch, k))
    w = rng.standard_normal((n, k)) / np.sqrt(k)
    b = rng.standard_normal((1, n))
    g = rng.standard_normal((batch, n))
    lin = _linear(rs, w, b)
    lin.forward(x)
    gx = lin.backward(g).to_numpy()
    want_gw, want_gb, want_gx = oracle.linear_backward(g, x, w)
    params = list(lin.parameters())
    assert params[0].grad.shape == w.shape and params[1].grad.shape == b.shape
    assert rel_err(params[0].grad.to_numpy(), want_gw) <= TOL
    assert rel_err(params[1].grad.to_numpy(), want_gb) <= TOL
    assert rel_err(gx, want_gx) <= TOL


# 256..511 tiles with a very long contraction (K >= 24576): the direct-to-LDS kernels cut K in two
# halves - forward, input gradient, and weight gradient (+ bias gradient over slices) in turn
@pytest.mark.parametrize("batch,k,n", [(2048, 24576, 2046), (2064, 2048, 24576), (24576, 2048, 2046),
                                       (24577, 2047, 2045)])  # (the last: odd everywhere, 8-byte aligned pairs)
def test_two_way_k_split_matches_oracle(engine, oracle, batch, k, n):
    import rstorch_amd as rs
    rng = np.random.default_rng(batch + 3 * k + 7 * n)
    x = rng.standard_normal((batch, k))
    w = rng.standard_normal((n, k)) / np.sqrt(k)
    b = rng.standard_normal((1, n))
    g = rng.standard_normal((batch, n))
    lin = _linear(rs, w, b)
    out = lin._forward(x, True).to_numpy()
    gx = lin.backward(g).to_numpy()
    params = list(lin.parameters())
    oracle.set_threads(8)
    try:
        assert rel_err(out, oracle.relu_forward(oracle.linear_forward(x, w, b))) <= TOL
        want_gw, want_gb, want_gx = oracle.linear_backward(g, x, w)
    finally:
        oracle.set_threads(1)
    assert rel_err(params[0].grad.to_numpy(), want_gw) <= TOL
    assert rel_err(params[1].grad.to_numpy(), want_gb) <= TOL
    assert rel_err(gx, want_gx) <= TOL


@pytest.mark.parametrize("batch,k,n", [(32, 100, 10), (130, 66, 34), (512, 256, 128)])
def test_backward_with_fused_relu_mask(engine, oracle, batch, k, n):
    """grad_input * (input > 0) in the epilogue == Linear.backward then ReLU.backward."""
    import rstorch_amd as rs
    rng = np.random.default_rng(5 + batch)
    pre = rng.standard_normal((batch, k))
    x = oracle.relu_forward(pre)  # the layer's input is a ReLU output
    w = rng.standard_normal((n, k))
    g = rng.standard_normal((batch, n))
    lin = _linear(rs, w, np.zeros((1, n)))
    lin.forward(x)
    got = lin._backward(g, True).to_numpy()
    _, _, gx = oracle.linear_backward(g, x, w)
    want = oracle.relu_backward(gx, pre)
    assert rel_err(got, want) <= TOL
    assert np.all(got[pre <= 0] == 0.0)


def test_reference_known_answers(engine):
    """The reference's own Linear tests (src/module/linear.rs:97-131), exact small integers."""
    import rstorch_amd as rs
    kats = json.load(open(GOLDEN))
    f = kats["linear_forward"]
    lin = _linear(rs, np.array(f["weight"]), np.array(f["bias"]))
    np.testing.assert_array_equal(lin.forward(np.array(f["input"])).to_numpy(), np.array(f["output"]))
    b = kats["linear_backward"]
    lin = _linear(rs, np.array(b["weight"]), np.array(b["bias"]))
    lin.forward(np.array(b["input"]))
    gx = lin.backward(np.array(b["gradient"])).to_numpy()
    p = list(lin.parameters())
    np.testing.assert_array_equal(p[0].grad.to_numpy(), np.array(b["grad_weight"]))
    np.testing.assert_array_equal(p[1].grad.to_numpy(), np.array(b["grad_bias"]))
    np.testing.assert_array_equal(gx, np.array(b["grad_input"]))
    assert p[0].grad.shape == p[0].parm.shape and p[1].grad.shape == p[1].parm.shape


def test_identity_weight_copies_input(engine):
    """W = I reduces the contraction to a copy: bit-exact."""
    import rstorch_amd as rs
    rng = np.random.default_rng(3)
    x = rng.standard_normal((70, 48))
    lin = _linear(rs, np.eye(48), np.zeros((1, 48)))
    np.testing.assert_array_equal(lin.forward(x).to_numpy(), x)


def test_one_hot_input_selects_weight_rows(engine):
    """One-hot rows select columns of W (exact), and dW = G^T X / n scatters G rows (exact
    for a power-of-two batch)."""
    import rstorch_amd as rs
    rng = np.random.default_rng(4)
    k, n, batch = 24, 19, 16
    idx = rng.integers(0, k, size=batch)
    x = np.zeros((batch, k)); x[np.arange(batch), idx] = 1.0
    w = rng.standard_normal((n, k)); b = rng.standard_normal((1, n))
    lin = _linear(rs, w, b)
    np.testing.assert_array_equal(lin.forward(x).to_numpy(), w[:, idx].T + b)


# Small integers make every product and every partial sum exact, whatever the order of the
# additions, so the three results of Linear::backward can be compared with numpy BIT FOR BIT:
# dW = (G^T X) / batch with the division by the batch size (src/module/linear.rs:63-64; blocks
# inside the matrix multiply by the exact reciprocal when the batch is a power of two and divide
# otherwise, blocks on its edge always divide), db = colsum(G) / batch, dX = (G W) * [x > 0].
# The shapes mix interior and edge blocks of the 128x128, 64x64 and 32x32 kernels.
@pytest.mark.parametrize("batch,k,n", [(1024, 384, 300), (1000, 384, 300), (4096, 1024, 1280), (4000, 1024, 1280),
                                       (512, 4096, 4096), (96, 130, 70), (8192, 784, 100), (8200, 784, 100),
                                       (64, 32, 70000), (128, 70000, 64)])  # long rows: large lane offsets in the interior epilogue
def test_backward_on_integer_data_is_bit_exact(engine, batch, k, n):
    from rstorch_amd import _ffi
    rng = np.random.default_rng(batch + k + n)
    hx = rng.integers(-3, 4, size=(batch, k)).astype(np.float64)
    hw = rng.integers(-3, 4, size=(n, k)).astype(np.float64)
    hg = rng.integers(-3, 4, size=(batch, n)).astype(np.float64)
    x, w, g = engine.from_numpy(hx), engine.from_numpy(hw), engine.from_numpy(hg)
    gw, gb, gx = engine.empty(n, k), engine.empty(1, n), engine.empty(batch, k)
    _ffi.check(engine.lib.rst_linear_backward(engine.handle, g.ptr, x.ptr, w.ptr, gw.ptr, gb.ptr, gx.ptr, x.ptr,
                                              batch, k, n))
    np.testing.assert_array_equal(gw.to_numpy(), (hg.T @ hx) / batch)
    np.testing.assert_array_equal(gb.to_numpy(), hg.sum(axis=0, keepdims=True) / batch)
    np.testing.assert_array_equal(gx.to_numpy(), (hg @ hw) * (hx > 0))
    # forward with bias and ReLU on the same data
    hb = rng.integers(-50, 51, size=(1, n)).astype(np.float64)
    b, out = engine.from_numpy(hb), engine.empty(batch, n)
    _ffi.check(engine.lib.rst_linear_forward(engine.handle, x.ptr, w.ptr, b.ptr, out.ptr, batch, k, n, 1))
    np.testing.assert_array_equal(out.to_numpy(), np.maximum(hx @ hw.T + hb, 0.0))


def test_backward_twice_raises(engine):
    import rstorch_amd as rs
    lin = _linear(rs, np.ones((2, 3)), np.zeros((1, 2)))
    with pytest.raises(rs.StateError):
        lin.parameters()  # no gradient yet (reference: unwrap on None, linear.rs:72)
    lin.forward(np.ones((4, 3)))
    lin.backward(np.ones((4, 2)))
    with pytest.raises(rs.StateError):
        lin.backward(np.ones((4, 2)))  # cache consumed (linear.rs:61)
    with pytest.raises(rs.ShapeError):
        lin.forward(np.ones((4, 5)))


def _sweep_cases():
    rng = np.random.default_rng(12345)
    cases = []
    for _ in range(36):
        kind = int(rng.integers(0, 4))
        if kind == 0:    # hundreds of 128x128 tiles, dimensions a little off the tile grid
            b, k, n = (int(rng.integers(3, 36)) * 64 + int(rng.choice([0, 2, 6, 14])) for _ in range(3))
        elif kind == 1:  # few tiles and a long contraction (K slices), with and without a K remainder
            b = int(rng.integers(1, 8)) * 128 + int(rng.choice([0, 2, 30]))
            n = int(rng.integers(2, 20)) * 128 - int(rng.choice([0, 2, 100]))
            k = int(rng.integers(20, 300)) * 16 + int(rng.choice([0, 2, 8, 14]))
        elif kind == 2:  # odd sizes: nothing is aligned
            b, k, n = (int(rng.integers(1, 900)) for _ in range(3))
        else:            # long batch, narrow layers
            b = int(rng.integers(100, 5000)) * 2
            k = int(rng.integers(1, 60)) * 2
            n = int(rng.integers(1, 60)) * 2
        cases.append((b, k, n))
    rng = np.random.default_rng(54321)
    for _ in range(28):
        kind = int(rng.integers(0, 3))
        if kind == 0:    # the 64x64 direct-to-LDS band: a long batch, one narrow side, a contraction of a few hundred
            b = int(rng.integers(16, 130)) * 64 + int(rng.choice([0, 2, 10]))
            k, n = int(rng.integers(12, 70)) * 16 + int(rng.choice([0, 2, 8])), int(rng.integers(8, 130)) * 2
            if rng.integers(0, 2):
                k, n = n + 190, k
        elif kind == 1:  # whole tiles only: every block takes the interior epilogue; power-of-two and other batches
            b = int(rng.choice([256, 512, 768, 1024, 1536, 2048]))
            k, n = int(rng.integers(1, 12)) * 128, int(rng.integers(1, 12)) * 128
        else:            # one or two tiles of output over a very long batch (weight gradient in many K slices)
            b = int(rng.integers(40, 140)) * 128 + int(rng.choice([0, 8]))
            k, n = int(rng.integers(5, 130)) * 2, int(rng.integers(5, 130)) * 2
        cases.append((b, k, n))
    # odd extents on every direct-to-LDS route (8-byte aligned pairs, the last row of the contraction with
    # the tail where an output-contiguous operand has an odd extent)
    rng = np.random.default_rng(777)
    for _ in range(18):
        kind = int(rng.integers(0, 3))
        if kind == 0:    # hundreds of 128x128 tiles
            b, k, n = (2 * int(rng.integers(700, 1500)) + 1 for _ in range(3))
        elif kind == 1:  # few tiles and a long contraction: K slices
            b = int(rng.integers(1, 8)) * 128 + int(rng.choice([-1, 1, 31]))
            n = int(rng.integers(2, 20)) * 128 - int(rng.choice([1, 3, 101]))
            k = 2 * int(rng.integers(160, 2400)) + 1
        else:            # the 64x64 band
            b = int(rng.integers(16, 130)) * 64 + int(rng.choice([-1, 1, 9]))
            k, n = 2 * int(rng.integers(96, 560)) + 1, 2 * int(rng.integers(8, 130)) + 1
            if rng.integers(0, 2):
                k, n = n + 190, k
        cases.append((b, k, n))
    return cases


@pytest.mark.parametrize("batch,k,n", _sweep_cases())
def test_seeded_shape_sweep_matches_numpy(engine, batch, k, n):
    """Every kernel-selection path (tile sizes, K slices, K remainder, unaligned fallbacks) on seeded
    random shapes, forward with fused ReLU and backward with the fused mask, against numpy float64."""
    import rstorch_amd as rs
    rng = np.random.default_rng(batch * 31 + k * 17 + n)
    x = rng.standard_normal((batch, k))
    w = rng.standard_normal((n, k)) / np.sqrt(k)
    b = rng.standard_normal((1, n))
    g = rng.standard_normal((batch, n))
    lin = _linear(rs, w, b)
    out = lin._forward(x, True).to_numpy()
    gx = lin._backward(g, True).to_numpy()
    params = list(lin.parameters())
    assert rel_err(out, np.maximum(x @ w.T + b, 0.0)) <= TOL
    assert rel_err(gx, (g @ w) * (x > 0)) <= TOL
    assert rel_err(params[0].grad.to_numpy(), g.T @ x / batch) <= TOL
    assert rel_err(params[1].grad.to_numpy(), g.sum(0, keepdims=True) / batch) <= TOL
