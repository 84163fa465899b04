"""The device generator and the initialisers built on it (src/module/init/{mod,he,xavier,sigma}.rs).

The reference draws from an unseedable thread RNG, so there are no reference vectors: what the
reference fixes is the distribution (normal, sigma = 1/sqrt(in) for Kaiming, sqrt(2/(in+out)) for
Xavier, user (mean, std) for Normal), the weight shape (out, in) and the zero bias of shape (1, out).
The counter-based generator underneath is pinned three ways: the published splitmix64 test vector,
an independent pure-Python restatement of value(seed, stream, index), and bit-equality between the
device kernels and the CPU restatement for the uniform and one-hot fills (integer work + exact
scaling); the normal fill goes through the device's log/sqrt/cos and is compared within a few ulp,
then by its sample moments."""
import ctypes
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MASK = (1 << 64) - 1
SEED = 0x5EED


def _mix64(z):
    z = (z + 0x9E3779B97F4A7C15) & MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return z ^ (z >> 31)


def _draw(seed, stream, index):
    key = _mix64(_mix64(seed) ^ ((stream * 0xD1342543DE82EF95) & MASK))
    return _mix64((key + index * 0x9E3779B97F4A7C15) & MASK)


def _u01(r):
    return float(r >> 11) * 2.0 ** -53


def test_generator_known_answers(engine, oracle):
    # splitmix64 from state 0: the first output of Vigna's reference implementation
    assert _mix64(0) == 0xE220A8397B1DCDAF
    assert _mix64(0x9E3779B97F4A7C15) == 0x6E789E6AA1B965F4
    for seed, stream, index in [(0, 0, 0), (SEED, 7, 123456789), (MASK, MASK, MASK), (1, 2, 3)]:
        assert oracle.rng_u64(seed, stream, index) == _draw(seed, stream, index)
    got = engine.uniform(1, 5, SEED, 3).to_numpy().ravel()
    want = [_u01(_draw(SEED, 3, i)) for i in range(5)]
    assert got.tolist() == want


# n > 16384 * 256 = 4194304: the grid-stride loop of the fill kernels takes a second trip
@pytest.mark.parametrize("n", [1, 2, 255, 257, 65537, 16384 * 256 + 12345])
def test_uniform_fill_is_bit_identical(engine, oracle, n):
    for lo, hi in ((0.0, 1.0), (-0.75, 2.5)):
        got = engine.uniform(1, n, SEED, 11, lo, hi).to_numpy()
        want = oracle.fill_uniform((1, n), SEED, 11, lo, hi)
        np.testing.assert_array_equal(got, want)
        assert got.min() >= lo and got.max() < hi
    if n > 1000:  # another stream or seed is another sequence
        a = engine.uniform(1, n, SEED, 12).to_numpy()
        b = engine.uniform(1, n, SEED + 1, 11).to_numpy()
        base = oracle.fill_uniform((1, n), SEED, 11)
        assert np.mean(a == base) < 1e-3 and np.mean(b == base) < 1e-3


@pytest.mark.parametrize("rows,cols", [(1, 1), (1, 7), (33, 10), (1000, 37), (3, 32768),
                                       (4099, 1025)])
def test_one_hot_fill_is_bit_identical(engine, oracle, rows, cols):
    got = engine.one_hot(rows, cols, SEED, 21).to_numpy()
    want = oracle.fill_one_hot(rows, cols, SEED, 21)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got.sum(axis=1), np.ones(rows))
    labels = [_draw(SEED, 21, r) % cols for r in range(min(rows, 50))]
    assert got[:len(labels)].argmax(axis=1).tolist() == labels


def test_one_hot_labels_are_uniform(engine):
    rows, cols = 1 << 16, 10
    counts = engine.one_hot(rows, cols, SEED, 22).to_numpy().sum(axis=0)
    expect = rows / cols
    chi2 = float(((counts - expect) ** 2 / expect).sum())
    assert chi2 < 33.7  # 99.99th percentile of chi-square with 9 degrees of freedom


@pytest.mark.parametrize("n", [1, 3, 4097, 16384 * 256 + 77])
def test_normal_fill_matches_the_cpu_restatement(engine, oracle, n):
    mean, std = 0.25, 0.02
    got = engine.normal(1, n, SEED, 31, mean, std).to_numpy()
    want = oracle.fill_normal((1, n), SEED, 31, mean, std)
    # same uniforms, same formula; log, sqrt, cos come from two maths libraries.  cos(2 pi u) loses
    # relative accuracy near its zeros, so the bound is absolute in units of std
    assert np.max(np.abs(got - want)) <= 64 * np.finfo(np.float64).eps * std
    z = (got - mean) / std
    assert np.all(np.isfinite(z)) and np.max(np.abs(z)) < 8.6  # sqrt(-2 ln 2^-53) = 8.57


def test_normal_fill_moments(engine):
    n = 1 << 22
    z = engine.normal(1, n, SEED, 32).to_numpy().ravel()
    se_mean = 1.0 / math.sqrt(n)
    se_std = 1.0 / math.sqrt(2.0 * n)
    assert abs(z.mean()) < 4 * se_mean
    assert abs(z.std() - 1.0) < 4 * se_std
    assert abs(np.mean(z ** 3)) < 4 * math.sqrt(15.0 / n)        # skewness 0
    assert abs(np.mean(z ** 4) - 3.0) < 4 * math.sqrt(96.0 / n)  # kurtosis 3
    # one tail probability: P(|z| > 1.959964) = 0.05
    p = np.mean(np.abs(z) > 1.959964)
    assert abs(p - 0.05) < 4 * math.sqrt(0.05 * 0.95 / n)
    # consecutive draws are uncorrelated
    assert abs(np.mean(z[:-1] * z[1:])) < 4 * se_mean


def _sigma_check(w, sigma):
    n = w.size
    assert abs(w.mean()) < 4 * sigma / math.sqrt(n)
    assert abs(w.std() / sigma - 1.0) < 4 / math.sqrt(2.0 * n)


def test_linear_new_is_kaiming_with_zero_bias(engine):
    """Linear::new -> KaimingNormal (linear.rs:36-38): weight (out, in) ~ N(0, 1/sqrt(in)),
    bias zeros (1, out) (he.rs:9-15, init/mod.rs:15-17)."""
    import rstorch_amd as rs
    layer = rs.Linear.new(784, 300)
    assert layer.weight.shape == (300, 784) and layer.bias.shape == (1, 300)
    _sigma_check(layer.weight.to_numpy(), 1.0 / math.sqrt(784.0))
    np.testing.assert_array_equal(layer.bias.to_numpy(), np.zeros((1, 300)))
    other = rs.Linear.new(784, 300)  # the reference's thread RNG never repeats a layer either
    assert np.mean(other.weight.to_numpy() == layer.weight.to_numpy()) < 1e-3


def test_initialisers_sigma_and_shape(engine, oracle):
    import rstorch_amd as rs
    fan_in, fan_out = 512, 384
    w = rs.XavierNormal(seed=5).weight(fan_in, fan_out, engine)
    assert w.shape == (fan_out, fan_in)
    _sigma_check(w.to_numpy(), math.sqrt(2.0 / (fan_in + fan_out)))  # xavier.rs:12
    w = rs.KaimingNormal(seed=5).weight(fan_in, fan_out, engine)
    assert w.shape == (fan_out, fan_in)
    _sigma_check(w.to_numpy(), 1.0 / math.sqrt(fan_in))  # he.rs:12
    init = rs.Normal.new(1.5, 0.3)  # sigma.rs:15-22
    w = init.weight(fan_in, fan_out, engine).to_numpy()
    assert w.shape == (fan_out, fan_in)
    _sigma_check(w - 1.5, 0.3)
    assert rs.Normal.new(0.0, float("inf")) is None and rs.Normal.new(0.0, float("nan")) is None  # sigma.rs:16-19
    np.testing.assert_array_equal(init.bias(fan_in, fan_out, engine).to_numpy(), np.zeros((1, fan_out)))
    # a seeded initialiser is reproducible, and layers built with new_with_kernel take its values
    a = rs.KaimingNormal(seed=9)
    layer = rs.Linear.new_with_kernel(20, 30, a)
    assert layer.weight.shape == (30, 20) and layer.bias.shape == (1, 30)
    _sigma_check(layer.weight.to_numpy(), 1.0 / math.sqrt(20.0))


def test_model_init_kaiming_stream_numbering(engine, oracle):
    """rst_model_init_kaiming: tensor i (reference order: weight, bias per Linear) uses generator
    stream first_stream + i; weights N(0, 1/sqrt(in)), biases zero."""
    import rstorch_amd as rs
    spec = [("identity",), ("linear", 96, 40), ("relu",), ("linear", 40, 24), ("relu",), ("linear", 24, 7)]
    dm = rs.DeviceModel(spec, engine)
    first = 100
    dm.init_kaiming(SEED, first)
    params = dm.parameters()
    assert [p.shape for p, _ in params] == [(40, 96), (1, 40), (24, 40), (1, 24), (7, 24), (1, 7)]
    for i, (p, _) in enumerate(params):
        got = p.to_numpy()
        if i % 2 == 1:
            np.testing.assert_array_equal(got, np.zeros(p.shape))
            continue
        fan_in = p.shape[1]
        sigma = 1.0 / math.sqrt(float(fan_in))
        direct = engine.normal(p.shape[0], p.shape[1], SEED, first + i, 0.0, sigma).to_numpy()
        np.testing.assert_array_equal(got, direct)  # the same kernel on the documented stream
        want = oracle.fill_normal(p.shape, SEED, first + i, 0.0, sigma)
        assert np.max(np.abs(got - want)) <= 64 * np.finfo(np.float64).eps * sigma
    dm.close()
