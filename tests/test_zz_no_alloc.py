"""rst_cross_entropy_static (fixed scratch inside the library's device image, no allocation in the
call) against rst_cross_entropy: same loss bits and same gradient bits, on two calls in a row, the
second on a smaller input, so that what the first call left in the shared scratch is seen not to
leak into the second."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(engine, z, t):
    from rstorch_amd import _ffi
    rows, cols = z.shape
    dz, dt = engine.from_numpy(z), engine.from_numpy(t)
    out = []
    for name in ("rst_cross_entropy", "rst_cross_entropy_static"):
        g = engine.full(rows, cols, -7.0)
        loss = ctypes.c_double(-1.0)
        fn = getattr(engine.lib, name)
        if name == "rst_cross_entropy":
            status = fn(engine.handle, dz.ptr, dt.ptr, g.ptr, None, rows, cols, ctypes.byref(loss))
        else:
            status = fn(engine.handle, dz.ptr, dt.ptr, g.ptr, rows, cols, ctypes.byref(loss))
        out.append((status, loss.value, g.to_numpy()))
    return out


# (first call, second smaller call): register-resident rows finished by one workgroup, rows spread
# over several workgroups + the reduction launch, and the two-walk kernel for wide rows
@pytest.mark.parametrize("first,second", [((48, 10), (7, 10)), ((3000, 1000), (129, 1000)),
                                          ((300, 4100), (64, 37)), ((64, 32768), (5, 32768))])
def test_static_scratch_cross_entropy_matches_the_allocating_entry_point(engine, oracle, first, second):
    rng = np.random.default_rng(first[0] + second[0])
    for rows, cols in (first, second):
        z = rng.standard_normal((rows, cols)) * 3.0
        t = np.zeros((rows, cols))
        t[np.arange(rows), rng.integers(0, cols, rows)] = 1.0
        if rows > 2:
            t[1] = rng.random(cols)
            t[1] /= t[1].sum()  # one soft-label row
        (s0, l0, g0), (s1, l1, g1) = _both(engine, z, t)
        assert s0 == 0 and s1 == 0
        assert l1 == l0
        np.testing.assert_array_equal(g1, g0)
        want_loss, prob = oracle.cross_entropy_forward(z, t)
        assert abs(l1 - want_loss) <= 1e-10 * abs(want_loss)
        want_g = oracle.cross_entropy_backward(prob, t)
        assert np.max(np.abs(g1 - want_g)) <= 1e-10 * np.max(np.abs(want_g))


def test_static_scratch_nan_flag_does_not_stick(engine):
    """NaN logits give RST_ERR_NAN (softmax.rs:38 panics) and the next, clean call is clean again."""
    from rstorch_amd import _ffi
    rng = np.random.default_rng(3)
    z = rng.standard_normal((500, 300))
    t = np.eye(300)[rng.integers(0, 300, 500)]
    bad = z.copy()
    bad[77, 5] = np.nan
    (s0, _, _), (s1, _, _) = _both(engine, bad, t)
    assert s0 == _ffi.RST_ERR_NAN and s1 == _ffi.RST_ERR_NAN
    (s0, l0, g0), (s1, l1, g1) = _both(engine, z[:40], t[:40])
    assert s0 == 0 and s1 == 0 and l0 == l1
    np.testing.assert_array_equal(g0, g1)


def test_static_scratch_limit_is_an_error(engine):
    from rstorch_amd import _ffi
    rows = 65536 + 1
    z = engine.zeros(rows, 2)
    g = engine.empty(rows, 2)
    status = engine.lib.rst_cross_entropy_static(engine.handle, z.ptr, z.ptr, g.ptr, rows, 2, None)
    assert status == _ffi.RST_ERR_UNSUPPORTED
    assert b"65536" in engine.lib.rst_last_error()
    # the largest size it takes: uniform logits, one-hot truth -> loss = ln 2
    rows = 65536
    t = engine.one_hot(rows, 2, 1, 1)
    loss = ctypes.c_double()
    _ffi.check(engine.lib.rst_cross_entropy_static(engine.handle, z.ptr, t.ptr, g.ptr, rows, 2,
                                                   ctypes.byref(loss)))
    assert abs(loss.value - np.log(2.0)) < 1e-15
