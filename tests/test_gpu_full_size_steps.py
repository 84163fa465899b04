"""Whole training steps of the two large configurations at FULL size against the oracle, on the
model's own data: one default step (SGD inside the weight-gradient launches, paired gradient grids,
graph replay) compared on the loss, EVERY dW/db and EVERY updated parameter at 1e-10, then the
multi-step criterion (loss within 1e-8 relative) with fresh inputs every step.

The oracle runs on the host cores the GPU box grants (16 threads; its summation order does not
depend on the thread count): a C2 step takes about half a second, a C4 step about three."""
import os
import time

import numpy as np
import pytest

from conftest import rel_err

pytestmark = pytest.mark.gpu

C4_SPEC = [("linear", 4096, 4096), ("relu",)] * 8 + [("linear", 4096, 32768)]
C2_SPEC = [("linear", 1024, 4096), ("relu",), ("linear", 4096, 4096), ("relu",), ("linear", 4096, 1000)]
ORACLE_THREADS = 16
SEED = 0x5EED


def _twin(oracle, dm, spec):
    """An oracle model holding the device model's weights."""
    ref = oracle.Model(spec)
    for (p, _), (q, _) in zip(ref.parameters(), dm.parameters()):
        p[...] = q.to_numpy()
    return ref


def _batch(engine, oracle, batch, n_in, n_out, step):
    """Inputs N(0,1) and one-hot labels of step `step` from the counter generator (stream = step).
    x is generated on the device and downloaded (the normal fill agrees with the CPU restatement
    only to a few ulps); the one-hot rows are bit-identical on both sides, so the host copy of the
    dense truth matrix is generated in place instead of travelling over PCIe."""
    x = engine.normal(batch, n_in, SEED, 1000 + 2 * step)
    y = engine.one_hot(batch, n_out, SEED, 1001 + 2 * step)
    return x, y, x.to_numpy(), oracle.fill_one_hot(batch, n_out, SEED, 1001 + 2 * step)


@pytest.mark.parametrize("name,spec,batch", [("C2", C2_SPEC, 2048), ("C4", C4_SPEC, 1024)])
def test_one_default_step_matches_oracle_on_every_tensor(engine, oracle, name, spec, batch):
    import rstorch_amd as rs
    dm = rs.DeviceModel(spec)
    dm.init_kaiming(SEED, 0)
    ref = _twin(oracle, dm, spec)
    x, y, hx, hy = _batch(engine, oracle, batch, dm.in_width, dm.out_width, 0)
    assert np.array_equal(y.to_numpy(), hy)  # the two generators agree on the labels
    oracle.set_threads(ORACLE_THREADS)
    try:
        want = ref.train_step(hx, hy, 0.01)
    finally:
        oracle.set_threads(1)
    got = dm.train_step(x, y, 0.01)  # records the graph
    assert abs(got - want) <= 1e-10 * abs(want), (got, want)
    worst_g = worst_p = 0.0
    for i, ((p, g), (rp, rg)) in enumerate(zip(dm.parameters(), ref.parameters())):
        eg, ep = rel_err(g.to_numpy(), rg), rel_err(p.to_numpy(), rp)
        assert eg <= 1e-10, "gradient %d: %.3e" % (i, eg)
        assert ep <= 1e-10, "parameter %d: %.3e" % (i, ep)
        worst_g, worst_p = max(worst_g, eg), max(worst_p, ep)
    print("%s one step: loss rel %.2e, worst gradient %.2e, worst parameter %.2e"
          % (name, abs(got - want) / abs(want), worst_g, worst_p), flush=True)
    # a second step on the same buffers replays the graph: still the oracle's step
    oracle.set_threads(ORACLE_THREADS)
    try:
        want = ref.train_step(hx, hy, 0.01)
    finally:
        oracle.set_threads(1)
    got = dm.train_step(x, y, 0.01)
    assert abs(got - want) <= 1e-10 * abs(want), (got, want)
    for i, ((p, g), (rp, rg)) in enumerate(zip(dm.parameters(), ref.parameters())):
        assert rel_err(g.to_numpy(), rg) <= 1e-10, "gradient %d after the replay" % i
        assert rel_err(p.to_numpy(), rp) <= 1e-10, "parameter %d after the replay" % i
    dm.close()


def _heartbeat(line):
    """A long comparison prints nothing a test runner would show before it ends; a line appended to a
    file in the run-output directory beside the tests shows that it is alive."""
    try:
        out_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out")
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "full_size_steps_progress.txt"), "a") as f:
            f.write(line + "\n")
    except OSError:
        pass


def _many_steps(engine, oracle, name, spec, batch, max_steps, min_steps, budget_s):
    import rstorch_amd as rs
    dm = rs.DeviceModel(spec)
    dm.init_kaiming(SEED, 0)
    ref = _twin(oracle, dm, spec)
    t0 = time.time()
    done, worst = 0, 0.0
    oracle.set_threads(ORACLE_THREADS)
    try:
        for step in range(max_steps):
            x, y, hx, hy = _batch(engine, oracle, batch, dm.in_width, dm.out_width, step)
            got = dm.train_step(x, y, 0.01)
            want = ref.train_step(hx, hy, 0.01)
            err = abs(got - want) / abs(want)
            assert err <= 1e-8, "%s step %d: %.17g vs %.17g" % (name, step, got, want)
            worst = max(worst, err)
            done = step + 1
            _heartbeat("%s: %d steps, %.0f s, worst loss error %.2e" % (name, done, time.time() - t0, worst))
            if done % 10 == 0:
                print("%s: %d steps, %.0f s, worst loss error %.2e" % (name, done, time.time() - t0, worst),
                      flush=True)
            if done >= min_steps and time.time() - t0 > budget_s:
                break
    finally:
        oracle.set_threads(1)
    assert done >= min_steps
    # the parameters the run ends with
    for i, ((p, _), (rp, _)) in enumerate(zip(dm.parameters(), ref.parameters())):
        assert rel_err(p.to_numpy(), rp) <= 1e-8, "parameter %d after %d steps" % (i, done)
    print("%s: %d steps compared, worst loss error %.2e" % (name, done, worst), flush=True)
    dm.close()


def test_hundred_steps_at_c2_full_size(engine, oracle):
    """Loss within 1e-8 relative over 100 steps of the wide MLP at batch 2048, fresh inputs per step."""
    _many_steps(engine, oracle, "C2", C2_SPEC, 2048, 100, 100, 1e9)


def test_many_steps_at_c4_full_size(engine, oracle):
    """The same criterion on the deep MLP at batch 1024 for as many of 100 steps as the oracle
    finishes in about two minutes (a step is 1.6 TFLOP on the host: about 2.5 s on 16 threads), 25 at least."""
    _many_steps(engine, oracle, "C4", C4_SPEC, 1024, 100, 25, 110.0)
