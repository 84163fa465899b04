#!/usr/bin/env python3
"""Benchmark of the rstorch f64 training step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra] [--eager]

Workload (BASELINE.json configs[4], the one the target sentence is quoted on): the deep MLP
(Linear(4096,4096)+ReLU) x 8 -> Linear(4096,32768), f64, batch 1024, CrossEntropyLoss,
SGD lr=0.01; weights N(0, 1/fan_in), inputs N(0,1), one-hot labels uniform over 32768 classes,
all generated on the device by the counter-based generator.  One step = forward, loss,
backward, SGD through the C ABI (rst_model_train_step), inputs resident in HBM.

Prints ONE JSON line.  `roofline` is for the FP64-MFMA contraction kernel instantiation with the
largest share of the step; per-launch durations come from HIP events recorded on the engine's
stream around every launch of the timed steps.  `cpu_baseline` is the CPU restatement (oracle)
timed on this host, single thread like the reference: one whole C4 step at the full batch.
`other_configs` holds, for configs[0..2], the graph-replay rate (C0 and C1: fresh inputs every step,
two resident batches refilled in turn on a second stream; also with the scalar loss read every step),
a second pass with per-launch events (contraction TFLOP/s against the FP64 MFMA peak) and the oracle
timed on the same configuration; `readme_loop` is the reference's README loop (README.md:64-74: the
module interface, loss and accuracy read back every step) run by the C++ host mirror in child
processes on configs[0], [1], [2] and [4], next to the single-call step of the same configuration.
"""
import argparse
import hashlib
import json
import os
import re
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP64_MFMA_TFLOPS = 78.6
PEAK_HBM_GBPS = 8000.0

# HBM-side bytes per launch of the C4 contraction kernels, averaged over the launches of one step
# (8 hidden layers + the head).  Measured with rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE, with and without --no-pair)
# of this script, scaled by the same counters on a streaming kernel of known size
# (--calibration-copy: FETCH x 2.0, WRITE x 1.0); the summary is kept under profiles/.
# A launch = the contraction plus, for the one that is contracted as two K slices (the head's input
# gradient), the reduction of the two partial results (134.3 MB); the weight gradient carries the SGD
# update of its layer.
# The figures hold for the kernel sources they were measured on: kernel_sources_sha16 is the first 16
# hex digits of the SHA-256 over the files below, taken when the profile was collected.  When the
# files have changed since, `traffic` is reported as null (and tests/test_host_logic.py fails) until
# the profile is collected again and the digest updated.
C4_TRAFFIC_SOURCE = {"profile": "profiles/c4_hbm_traffic.md",
                     "kernel_sources": ["rstorch_amd/csrc/gemm_f64.hip", "rstorch_amd/csrc/gemm_addressing.h"],
                     "kernel_sources_sha16": "237284b084fa9419"}


def kernel_sources_digest():
    h = hashlib.sha256()
    for rel in C4_TRAFFIC_SOURCE["kernel_sources"]:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]



C4_TRAFFIC_BYTES_PER_LAUNCH = {
    "linear_forward": (8 * 436.4e6 + 3856.8e6) / 9,
    "grad_weight": (8 * 862.0e6 + 7544.6e6) / 9,
    "grad_input": (7 * 470.0e6 + 3336.4e6 + 134.3e6) / 8,
    # a layer's weight gradient + SGD and the next layer's input gradient in one grid (the default):
    # six pairs at the hidden width and the one that carries the head's weight gradient
    "grad_pair": (6 * 1525.6e6 + 8036.9e6) / 7,
}

C4_SPEC = [("linear", 4096, 4096), ("relu",)] * 8 + [("linear", 4096, 32768)]
C4_BATCH = 1024
C2_SPEC = [("linear", 1024, 4096), ("relu",), ("linear", 4096, 4096), ("relu",),
           ("linear", 4096, 1000)]
# configs[2] with every extent odd: nothing is 16-byte aligned from one row to the next
C2_ODD_SPEC = [("linear", 1023, 4095), ("relu",), ("linear", 4095, 4095), ("relu",), ("linear", 4095, 999)]
C01_SPEC = [("identity",), ("linear", 784, 100), ("relu",), ("linear", 100, 100), ("relu",),
            ("linear", 100, 10)]
LR = 0.01
SEED = 0x5EED


def log(msg):
    print(msg, file=sys.stderr, flush=True)


def make_model(rs, eng, spec, batch, normal_inputs):
    dm = rs.DeviceModel(spec, eng)
    dm.init_kaiming(SEED, 0)
    n_in, n_out = dm.in_width, dm.out_width
    x = eng.normal(batch, n_in, SEED, 1000) if normal_inputs else eng.uniform(batch, n_in, SEED, 1000)
    y = eng.one_hot(batch, n_out, SEED, 1001)
    return dm, x, y


def time_steps(eng, dm, x, y, steps, warmup, profile):
    for _ in range(warmup):
        dm.train_step(x, y, LR, want_loss=False)
    eng.synchronize()
    if profile:
        dm.profile_enable(True)
    # the profiled (headline) run also marks every step, for the median and minimum step time
    marks = [eng.event() for _ in range(steps + 1 if profile else 2)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        dm.train_step(x, y, LR, want_loss=False)
        if profile:
            marks[i + 1].record()
    if not profile:
        marks[1].record()
    eng.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = marks[0].elapsed_ms(marks[-1])
    if profile:
        time_steps.per_step_ms = sorted(marks[i].elapsed_ms(marks[i + 1]) for i in range(steps))
    loss = dm.last_loss()
    recs = dm.profile_read() if profile else []
    if profile:
        dm.profile_enable(False)
    return wall, dev_ms, loss, recs


def summarise(recs, steps):
    """Per kernel class: launches per step, mean launch ms, achieved rate vs its roof."""
    groups = {}
    for r in recs:
        g = groups.setdefault(r["kernel"], {"ms": 0.0, "flops": 0.0, "bytes": 0.0, "n": 0})
        g["ms"] += r["ms"]; g["flops"] += r["flops"]; g["bytes"] += r["bytes"]; g["n"] += 1
    out = {}
    for k, g in groups.items():
        e = {"launches_per_step": g["n"] / steps, "avg_launch_ms": g["ms"] / g["n"],
             "ms_per_step": g["ms"] / steps}
        if g["flops"] > 0:
            e["bound"] = "mfma"
            e["achieved_tflops"] = g["flops"] / (g["ms"] * 1e-3) / 1e12
            e["frac"] = e["achieved_tflops"] / PEAK_FP64_MFMA_TFLOPS
        else:
            e["bound"] = "hbm"
            e["achieved_gbps"] = g["bytes"] / (g["ms"] * 1e-3) / 1e9
            e["frac"] = e["achieved_gbps"] / PEAK_HBM_GBPS
        out[k] = e
    return out


def bench_relu(rs, eng, iters=20):
    """The standalone ReLU kernels (what the module API runs when a ReLU does not follow or precede a
    Linear layer) over 2^27 doubles: 16 B per element forward, 24 B per element backward."""
    from rstorch_amd import _ffi
    n = 1 << 27
    x = eng.normal(1, n, SEED, 3100)
    g = eng.normal(1, n, SEED, 3101)
    out = eng.empty(1, n)
    res = {"elements": n}
    for name, nbytes, call in (
            ("forward", 16 * n, lambda: _ffi.check(eng.lib.rst_relu_forward(eng.handle, x.ptr, out.ptr, n))),
            ("backward", 24 * n, lambda: _ffi.check(eng.lib.rst_relu_backward(eng.handle, g.ptr, x.ptr, out.ptr, n)))):
        for _ in range(3):
            call()
        eng.synchronize()
        ev0, ev1 = eng.event(), eng.event()
        ev0.record()
        for _ in range(iters):
            call()
        ev1.record()
        eng.synchronize()
        ms = ev0.elapsed_ms(ev1) / iters
        res[name] = {"ms": ms, "achieved_gbps": nbytes / (ms * 1e-3) / 1e9,
                     "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS}
    return res


def bench_sgd_c3(rs, eng, iters=20):
    """configs[3]: SGD::step alone over 64 x (Linear(2048,2048) weight + bias), ~268.6M params."""
    import ctypes
    from rstorch_amd import _ffi
    shapes = [(2048, 2048), (1, 2048)] * 64
    total = sum(r * c for r, c in shapes)
    parm = eng.normal(1, total, SEED, 2000, 0.0, 0.02)
    grad = eng.normal(1, total, SEED, 2001, 0.0, 1e-3)
    res = {"parameters": total, "bytes_per_step": 24 * total}
    # (a) one launch over the 128 tensors (descriptor table)
    n = len(shapes)
    offs, o = [], 0
    for r, c in shapes:
        offs.append(o); o += r * c
    pp = (ctypes.c_void_p * n)(*[parm.ptr + 8 * f for f in offs])
    gp = (ctypes.c_void_p * n)(*[grad.ptr + 8 * f for f in offs])
    cnt = (ctypes.c_size_t * n)(*[r * c for r, c in shapes])
    for name, call in (
            ("tensor_list", lambda: _ffi.check(eng.lib.rst_sgd_step(eng.handle, pp, gp, cnt, n, LR))),
            ("arena", lambda: _ffi.check(eng.lib.rst_sgd_step_flat(eng.handle, parm.ptr, grad.ptr, total, LR)))):
        for _ in range(3):
            call()
        eng.synchronize()
        ev0, ev1 = eng.event(), eng.event()
        ev0.record()
        for _ in range(iters):
            call()
        ev1.record()
        ms = ev0.elapsed_ms(ev1) / iters
        res[name] = {"ms_per_step": ms, "steps_per_s": 1e3 / ms,
                     "achieved_gbps": 24.0 * total / (ms * 1e-3) / 1e9,
                     "frac_of_hbm_peak": 24.0 * total / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS}
    return res


def run_streaming_kernels(rs, eng, iters=10):
    """The HBM-bound kernels on their own, for profiler runs (kernel trace, FETCH_SIZE / WRITE_SIZE):
    the unfused ReLU passes and the flat SGD pass over 2^27 doubles (the SGD pass, 2 GiB read and 1 GiB
    written per launch, is the known-size kernel the counters are scaled by), the cross entropy and the
    accuracy count at the logit shapes of configs[2] (2048 x 1000) and configs[4] (1024 x 32768).
    Prints event-timed rates on its own."""
    import ctypes
    from rstorch_amd import _ffi
    lib, h = eng.lib, eng.handle
    n = 1 << 27
    a, b, c = eng.normal(1, n, SEED, 3100), eng.normal(1, n, SEED, 3101, 0.0, 1e-3), eng.empty(1, n)
    runs = [
        ("relu_forward", 16.0 * n, lambda: lib.rst_relu_forward(h, a.ptr, c.ptr, n)),
        ("relu_backward", 24.0 * n, lambda: lib.rst_relu_backward(h, b.ptr, a.ptr, c.ptr, n)),
        ("sgd_flat", 24.0 * n, lambda: lib.rst_sgd_step_flat(h, a.ptr, b.ptr, n, LR)),
    ]
    keep = []
    for rows, cols in ((2048, 1000), (1024, 32768)):
        z, t, g = eng.normal(rows, cols, SEED, 3200), eng.one_hot(rows, cols, SEED, 3201), eng.empty(rows, cols)
        keep.append((z, t, g))
        acc = ctypes.c_double()
        runs.append(("cross_entropy_%dx%d" % (rows, cols), 24.0 * rows * cols + 8.0 * rows,
                     lambda z=z, t=t, g=g, rows=rows, cols=cols: lib.rst_cross_entropy(h, z.ptr, t.ptr, g.ptr, None, rows, cols, None)))
        runs.append(("accuracy_%dx%d" % (rows, cols), 16.0 * rows * cols,
                     lambda z=z, t=t, rows=rows, cols=cols, acc=acc: lib.rst_accuracy(h, z.ptr, t.ptr, rows, cols, ctypes.byref(acc))))
    out = {}
    for name, nbytes, call in runs:
        for _ in range(2):
            _ffi.check(call())
        eng.synchronize()
        ev0, ev1 = eng.event(), eng.event()
        ev0.record()
        for _ in range(iters):
            _ffi.check(call())
        ev1.record()
        eng.synchronize()
        ms = ev0.elapsed_ms(ev1) / iters
        out[name] = {"ms": ms, "algorithmic_bytes": nbytes, "achieved_gbps": nbytes / (ms * 1e-3) / 1e9,
                     "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS}
    return out


def run_route_sweep(rs, eng):
    """Times Linear::forward, the weight gradient alone and the whole Linear::backward over a grid of
    mid-size shapes (batch 128..16384, widths 64..4096, at least one product below 256 tiles of
    128x128) under whatever RSTORCH_DMA64 says (unset: the planner's rule; 0: never the 64x64
    direct-to-LDS kernel; 1: wherever it is eligible).  CSV on stdout: the table the routing rule in
    choose_route is fitted to."""
    import itertools
    from rstorch_amd import _ffi
    lib, h = eng.lib, eng.handle

    def timeit(fn, reps=30):
        for _ in range(3):
            fn()
        eng.synchronize()
        a, b = eng.event(), eng.event()
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        eng.synchronize()
        return a.elapsed_ms(b) / reps * 1e3

    tiles = lambda m, n: ((m + 127) // 128) * ((n + 127) // 128)
    print("B,K,N,forward_us,weight_gradient_us,backward_us", flush=True)
    for B, K, N in itertools.product([128, 256, 512, 1024, 2048, 4096, 8192, 16384],
                                     [64, 100, 128, 256, 512, 784, 1024, 2048, 4096],
                                     [64, 100, 256, 512, 1000, 2048, 4096]):
        flops = 2.0 * B * K * N
        if flops < 5e7 or flops > 2e10 or min(tiles(B, N), tiles(N, K), tiles(B, K)) >= 256:
            continue
        x, w, b, g = eng.normal(B, K, 1, 1), eng.normal(N, K, 1, 2), eng.normal(1, N, 1, 3), eng.normal(B, N, 1, 4)
        o, gw, gb, gx = eng.empty(B, N), eng.empty(N, K), eng.empty(1, N), eng.empty(B, K)
        f = timeit(lambda: _ffi.check(lib.rst_linear_forward(h, x.ptr, w.ptr, b.ptr, o.ptr, B, K, N, 1)))
        dw = timeit(lambda: _ffi.check(lib.rst_linear_backward(h, g.ptr, x.ptr, w.ptr, gw.ptr, gb.ptr, None, None, B, K, N)))
        both = timeit(lambda: _ffi.check(lib.rst_linear_backward(h, g.ptr, x.ptr, w.ptr, gw.ptr, gb.ptr, gx.ptr, x.ptr, B, K, N)))
        print("%d,%d,%d,%.2f,%.2f,%.2f" % (B, K, N, f, dw, both), flush=True)
        del x, w, b, g, o, gw, gb, gx


def contraction_summary(recs, steps):
    """Contraction launches of a profiled pass: rate against the FP64 MFMA peak, the class with the
    largest share, and the step's launch count."""
    kernels = summarise(recs, steps)
    kinds = [k for k in ("linear_forward", "grad_weight", "grad_input", "grad_pair") if k in kernels]
    ms = sum(kernels[k]["ms_per_step"] for k in kinds)
    flops = sum(r["flops"] for r in recs if r["kernel"] in kinds) / steps
    dominant = max(kinds, key=lambda k: kernels[k]["ms_per_step"])
    return kernels, {
        "tflops": flops / (ms * 1e-3) / 1e12, "frac": flops / (ms * 1e-3) / 1e12 / PEAK_FP64_MFMA_TFLOPS,
        "flops_per_step": flops, "ms_per_step": ms, "launches_per_step": len(recs) / steps,
        "dominant": dominant, "dominant_tflops": kernels[dominant]["achieved_tflops"],
        "dominant_frac": kernels[dominant]["frac"],
        "dominant_avg_launch_ms": kernels[dominant]["avg_launch_ms"],
        "first_layer_input_gradient": "skipped (the README loop discards it)"}


def time_fresh_steps(rs, eng, loader, dm, batch, normal, steps, warmup, read_loss):
    """Steps on fresh inputs: two resident batches; while the training engine works on one, a second
    engine (a second stream of the same GPU) refills the other from the counter generator, stream
    number = step.  Events hand the buffers back and forth; the host never waits inside the loop
    unless read_loss asks for the scalar loss of every step."""
    from rstorch_amd import _ffi
    n_in, n_out = dm.in_width, dm.out_width
    bufs = [(eng.empty(batch, n_in), eng.empty(batch, n_out)) for _ in range(2)]
    filled = [loader.event() for _ in range(2)]   # recorded by the loader when a buffer is ready
    used = [eng.event() for _ in range(2)]        # recorded by the trainer when it is done with it

    def refill(slot, step):
        x, y = bufs[slot]
        fill = loader.lib.rst_fill_normal if normal else loader.lib.rst_fill_uniform
        _ffi.check(fill(loader.handle, x.ptr, x.size, SEED, 1000 + 2 * step, 0.0, 1.0))
        _ffi.check(loader.lib.rst_fill_one_hot(loader.handle, y.ptr, batch, n_out, SEED, 1001 + 2 * step))
        filled[slot].record()

    def run(first, count):
        refill(first % 2, first)
        loss = None
        for k in range(first, first + count):
            slot = k % 2
            if k + 1 < first + count:
                if k >= first + 1:
                    loader.wait_event(used[1 - slot])  # the step that last read the other buffer
                refill(1 - slot, k + 1)
            eng.wait_event(filled[slot])
            loss = dm.train_step(bufs[slot][0], bufs[slot][1], LR, want_loss=read_loss)
            used[slot].record()
        eng.synchronize()
        loader.synchronize()
        return loss

    run(0, warmup)
    t0 = time.perf_counter()
    run(warmup, steps)
    wall = time.perf_counter() - t0
    return wall, dm.last_loss()


def time_generated_in_stream(eng, dm, batch, normal, steps, warmup):
    """Steps on fresh inputs without a second stream: the counter generator refills the one batch on
    the training stream ahead of every step, so its time is inside the step and no event is needed."""
    from rstorch_amd import _ffi
    x, y = eng.empty(batch, dm.in_width), eng.empty(batch, dm.out_width)
    fill = eng.lib.rst_fill_normal if normal else eng.lib.rst_fill_uniform

    def run(first, count):
        for k in range(first, first + count):
            _ffi.check(fill(eng.handle, x.ptr, x.size, SEED, 1000 + 2 * k, 0.0, 1.0))
            _ffi.check(eng.lib.rst_fill_one_hot(eng.handle, y.ptr, batch, dm.out_width, SEED, 1001 + 2 * k))
            dm.train_step(x, y, LR, want_loss=False)
        eng.synchronize()

    run(0, warmup)
    t0 = time.perf_counter()
    run(warmup, steps)
    wall = time.perf_counter() - t0
    return wall, dm.last_loss()


def bench_small(rs, eng, spec, batch, normal, steps, warmup, eager, profile_steps, fresh_inputs=False):
    """steps_per_s: the fused step as shipped (graph replay unless --eager).  `contractions`: a
    second pass with an event after every launch (plain launches, one weight gradient per layer)."""
    dm, x, y = make_model(rs, eng, spec, batch, normal)
    if eager:
        dm.graph_enable(False)
    out = {"batch": batch, "steps": steps,
           "launch_mode": "graph replay" if dm.graph_active() else "plain launches"}
    if fresh_inputs:
        loader = rs.Engine(eng.device)
        wall, loss = time_fresh_steps(rs, eng, loader, dm, batch, normal, steps, warmup, False)
        out["inputs"] = ("fresh every step: two resident batches, refilled in turn on a second stream by the "
                         "counter generator (stream number = step)")
        wall_read, loss_read = time_fresh_steps(rs, eng, loader, dm, batch, normal, steps, warmup, True)
        out["with_loss_read_every_step"] = {"ms_per_step": wall_read * 1e3 / steps, "steps_per_s": steps / wall_read,
                                            "final_loss": loss_read}
        wall_gen, loss_gen = time_generated_in_stream(eng, dm, batch, normal, steps, warmup)
        out["generator_on_the_training_stream"] = {
            "ms_per_step": wall_gen * 1e3 / steps, "steps_per_s": steps / wall_gen, "final_loss": loss_gen,
            "note": "no second stream and no events: the generator's launches run ahead of every step on the "
                    "training stream, their time inside the step; at these sizes the two event hand-overs of the "
                    "two-stream protocol cost more than the generator takes"}
        wall_one, _, loss_one, _ = time_steps(eng, dm, x, y, steps, warmup, False)
        out["one_resident_batch"] = {"ms_per_step": wall_one * 1e3 / steps, "steps_per_s": steps / wall_one,
                                     "final_loss": loss_one}
        # the same with the scalar loss read back after every step, as the reference's loop does
        t0 = time.perf_counter()
        for _ in range(steps):
            loss_each = dm.train_step(x, y, LR, want_loss=True)
        wall_each = time.perf_counter() - t0
        out["one_resident_batch"]["with_loss_read_every_step"] = {
            "ms_per_step": wall_each * 1e3 / steps, "steps_per_s": steps / wall_each, "final_loss": loss_each}
        loader.close()
    else:
        wall, _, loss, _ = time_steps(eng, dm, x, y, steps, warmup, False)
        out["inputs"] = "one resident batch"
    out.update({"ms_per_step": wall * 1e3 / steps, "steps_per_s": steps / wall,
                "samples_per_s": steps / wall * batch, "final_loss": loss})
    _, _, _, recs = time_steps(eng, dm, x, y, profile_steps, 2, True)
    kernels, out["contractions"] = contraction_summary(recs, profile_steps)
    out["kernels"] = {k: {"avg_launch_us": v["avg_launch_ms"] * 1e3, "launches_per_step": v["launches_per_step"],
                          "frac": v["frac"], "bound": v["bound"]} for k, v in kernels.items()}
    dm.close()
    return out


README_LOOP_RUNS = {  # configuration -> (batch, steps per epoch, epochs)
    "C0": (32, 1875, 3), "C1": (8192, 400, 3), "C2": (2048, 40, 3), "C4": (1024, 20, 3)}


def readme_loop_child(config, layer_by_layer=False):
    """The README loop (README.md:64-74) through the C++ mirror of the module interface, in a process
    of its own, started before this one touches the GPU.  The rate is that of the last epoch."""
    exe = os.path.join(ROOT, "rstorch_amd", "cpp", "bin", "readme_loop")
    if not os.path.exists(exe):
        return {"error": "rstorch_amd/cpp/bin/readme_loop is not built (__graft_entry__.build())"}
    batch, steps, epochs = README_LOOP_RUNS[config]
    cmd = [exe, str(epochs), str(steps), config] + (["layers"] if layer_by_layer else [])
    try:
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=180)
    except subprocess.TimeoutExpired:
        return {"error": "readme_loop did not finish in 180 s"}
    rates = [float(m) for m in re.findall(r"\(([0-9.]+) steps/s\)", proc.stdout)]
    losses = [float(m) for m in re.findall(r"Avarage loss ([0-9.]+)", proc.stdout)]
    if proc.returncode != 0 or not rates:
        return {"error": "readme_loop failed: %s" % (proc.stderr.strip() or proc.stdout.strip())[:200]}
    return {"batch": batch, "steps_per_epoch": steps, "epochs": len(rates), "steps_per_s": rates[-1],
            "ms_per_step": 1e3 / rates[-1], "samples_per_s": rates[-1] * batch, "steps_per_s_per_epoch": rates,
            "average_loss_per_epoch": losses}


def readme_loops():
    out = {"shape": "model.forward(x) -> loss.forward(pred.clone(), y.clone()) -> accuracy(pred, y) -> "
                    "model.backward(loss.backward()) -> optim.step(model) through the module interface of the C++ "
                    "mirror; the loss and the accuracy are read back every step.  compiled: the Sequential runs "
                    "as a device model (backward deferred to the optimiser step, SGD inside the weight-gradient "
                    "launches, the first layer's input gradient skipped because the loop drops it; on small "
                    "networks the upper layers' input gradients are launched behind the loss before the host "
                    "waits for it); "
                    "layer_by_layer: one call per layer, SGD as a pass of its own"}
    for config in ("C0", "C1", "C2", "C4"):
        log("README loop, %s ..." % config)
        out[config] = {"compiled": readme_loop_child(config)}
        if config in ("C0", "C1"):
            out[config]["layer_by_layer"] = readme_loop_child(config, True)
    return out


def bench_staged(rs, eng, spec, batch, normal, steps, warmup, in_place=False):
    """Same step, but every batch comes from host memory through the pinned double-buffered
    stager (x as f64, labels as u32 expanded to one-hot rows on the device): the PCIe-inclusive
    rate.  The host arrays are prepared once; the per-step host work is the copy into pinned
    memory that rst_stager_submit_labels does."""
    import numpy as np
    dm = rs.DeviceModel(spec, eng)
    dm.init_kaiming(SEED, 0)
    n_in, n_out = dm.in_width, dm.out_width
    rng = np.random.default_rng(SEED)
    pool = [((rng.standard_normal((batch, n_in)) if normal else rng.random((batch, n_in))),
             rng.integers(0, n_out, batch).astype(np.uint32)) for _ in range(2)]
    st = rs.BatchStager(batch, n_in, n_out, depth=2, engine=eng)

    def send(k):
        if in_place:   # the loader writes straight into pinned memory (already there: no copy)
            st.host_slot(batch)
            st.commit(batch)
        else:
            st.submit(pool[k % 2][0], labels=pool[k % 2][1])

    if in_place:       # fill both pinned slots once
        for k in range(2):
            hx, hl = st.host_slot(batch)
            hx[...] = pool[k][0]; hl[...] = pool[k][1]
            st.commit(batch); st.next()

    def run(n):
        send(0)
        for k in range(n):
            if k + 1 < n:
                send(k + 1)
            x, y = st.next()
            dm.train_step(x, y, LR, want_loss=False)
        eng.synchronize()

    run(warmup)
    t0 = time.perf_counter()
    run(steps)
    wall = time.perf_counter() - t0
    loss = dm.last_loss()
    st.close(); dm.close()
    return {"batch": batch, "steps": steps, "ms_per_step": wall * 1e3 / steps,
            "steps_per_s": steps / wall, "samples_per_s": steps / wall * batch,
            "host_bytes_per_step": batch * (8 * n_in + 4), "final_loss": loss}


def cpu_baseline_small(spec, batch, normal, steps):
    """The oracle, single thread, on one of the small configurations: `steps` whole steps timed."""
    import numpy as np
    import oracle
    oracle.build()
    oracle.set_threads(1)
    ref = oracle.Model(spec)
    for i, (p, _) in enumerate(ref.parameters()):
        if p.shape[0] > 1:
            p[...] = oracle.fill_normal(p.shape, SEED, i, 0.0, p.shape[1] ** -0.5)
    n_in = next(l[1] for l in spec if l[0] == "linear")
    n_out = [l[2] for l in spec if l[0] == "linear"][-1]
    x = oracle.fill_normal((batch, n_in), SEED, 1000) if normal else oracle.fill_uniform((batch, n_in), SEED, 1000)
    y = oracle.fill_one_hot(batch, n_out, SEED, 1001)
    ref.train_step(x, y, LR)  # allocates the activation buffers
    t0 = time.perf_counter()
    for _ in range(steps):
        ref.train_step(x, y, LR)
    dt = time.perf_counter() - t0
    return {"value": steps / dt, "unit": "steps/s", "cores": 1, "kind": "port",
            "sample": "%d whole steps of the oracle, single thread" % steps, "s_per_step": dt / steps}


def cpu_baseline_sgd_c3(calls=10):
    """configs[3] on the host: the oracle's SGD::step over 268.6 M parameters, single thread."""
    import numpy as np
    import oracle
    total = 64 * (2048 * 2048 + 2048)
    parm = np.full(total, 0.02)
    grad = np.full(total, 1e-3)
    L = oracle.lib()
    oracle.set_threads(1)
    L.rsto_sgd_step(oracle._ptr(parm), oracle._ptr(grad), total, LR)
    t0 = time.perf_counter()
    for _ in range(calls):
        L.rsto_sgd_step(oracle._ptr(parm), oracle._ptr(grad), total, LR)
    dt = (time.perf_counter() - t0) / calls
    return {"value": 1.0 / dt, "unit": "steps/s", "cores": 1, "kind": "port",
            "sample": "%d calls of the oracle's SGD::step over %d parameters" % (calls, total),
            "achieved_gbps": 24.0 * total / dt / 1e9}


def cpu_baseline(sample_batches=(64, 256)):
    """The oracle (CPU restatement of the reference) on the C4 network: one whole step at the full
    batch of 1024, single thread, is the baseline.  Beside it, as a cross-check and for the all-cores
    figure, two reduced batches: a step costs t(B) = a + b*B (a: SGD and operand packing, independent
    of the batch; b: the per-row contraction and loss work), so two timed steps give t(1024).
    The oracle's weights here are uniform with the variance of N(0, 1/fan_in) (cheaper to draw;
    the timing does not depend on the distribution)."""
    import numpy as np
    import oracle
    oracle.build()
    # the GPU box grants a share of the host's cores; OMP_NUM_THREADS carries it
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    ref = oracle.Model(C4_SPEC)
    for i, (p, _) in enumerate(ref.parameters()):
        if p.shape[0] > 1:
            a = np.sqrt(3.0 / p.shape[1])  # uniform with the variance of N(0, 1/fan_in)
            p[...] = oracle.fill_uniform(p.shape, SEED, i, -a, a)
    b_lo, b_hi = sample_batches
    data = {B: (oracle.fill_normal((B, 4096), SEED, 1000), oracle.fill_one_hot(B, 32768, SEED, 1001))
            for B in sample_batches}
    out = {}
    for label, threads in (("single", 1), ("all", cores)):
        oracle.set_threads(threads)
        ref.train_step(*data[b_lo], LR)  # allocates the activation buffers, warms the thread pool
        times = {}
        for B in (b_hi, b_lo):
            t0 = time.perf_counter(); ref.train_step(*data[B], LR); times[B] = time.perf_counter() - t0
        slope = (times[b_hi] - times[b_lo]) / float(b_hi - b_lo)
        fixed = max(times[b_lo] - slope * b_lo, 0.0)
        t_full = fixed + slope * C4_BATCH
        out[label] = {"threads": threads, "t_step_s": {str(B): times[B] for B in sample_batches},
                      "per_row_s": slope, "batch_independent_s": fixed, "t_full_step_s_fitted": t_full,
                      "steps_per_s_fitted": 1.0 / t_full}
    # the baseline proper: one whole step at the full batch, single thread
    oracle.set_threads(1)
    full = (oracle.fill_normal((C4_BATCH, 4096), SEED, 1000), oracle.fill_one_hot(C4_BATCH, 32768, SEED, 1001))
    t0 = time.perf_counter()
    ref.train_step(*full, LR)
    out["single"]["t_full_step_s"] = time.perf_counter() - t0
    out["single"]["steps_per_s"] = 1.0 / out["single"]["t_full_step_s"]
    del ref, full
    return out, sample_batches, cores


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other configurations")
    ap.add_argument("--eager", action="store_true",
                    help="plain kernel launches instead of graph replay")
    ap.add_argument("--only", choices=["C0", "C1", "C2", "C2_odd"],
                    help="run one of the small configurations alone (for profiler runs)")
    ap.add_argument("--sgd-only", action="store_true",
                    help="time only SGD::step over the configs[3] parameter set (for profiler runs)")
    ap.add_argument("--no-pair", action="store_true",
                    help="launch every weight gradient and input gradient of C4 on its own (profiles that "
                         "attribute counters to one product at a time)")
    ap.add_argument("--streaming-kernels", action="store_true",
                    help="run only the HBM-bound kernels (ReLU, SGD, cross entropy, accuracy) on their own, "
                         "for profiler runs")
    ap.add_argument("--route-sweep", action="store_true",
                    help="time the three products of a Linear layer over the grid of mid-size shapes the "
                         "routing rule is fitted to; CSV on stdout")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one streaming ReLU over 1 GiB (reads 1 GiB, writes 1 GiB): the "
                         "known-size kernel that rocprofv3 FETCH_SIZE / WRITE_SIZE are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs the training step on ONE GPU; --gpus %d is not "
                 "supported (no collectives are part of this build)" % args.gpus)

    # a child process that uses the GPU runs before this process opens it
    readme_loop = None
    if not (args.no_extra or args.sgd_only or args.only or args.streaming_kernels or args.route_sweep):
        readme_loop = readme_loops()

    import rstorch_amd as rs
    eng = rs.default_engine()
    info = eng.device_info()
    log("device: %s, %d CUs" % (info["name"], info["compute_units"]))

    if args.sgd_only:
        print(json.dumps({"sgd_c3": bench_sgd_c3(rs, eng)}), flush=True)
        return
    if args.streaming_kernels:
        print(json.dumps({"streaming_kernels": run_streaming_kernels(rs, eng)}), flush=True)
        return
    if args.route_sweep:
        run_route_sweep(rs, eng)
        return

    # (name, layers, batch, N(0,1) inputs, timed steps, warm-up, profiled steps, fresh inputs every step)
    small = {"C0": ("C0_readme_b32", C01_SPEC, 32, False, 2000, 100, 200, True),
             "C1": ("C1_readme_b8192", C01_SPEC, 8192, False, 200, 20, 50, True),
             "C2": ("C2_wide_b2048", C2_SPEC, 2048, True, 20, 3, 10, False),
             "C2_odd": ("C2_odd_b2047", C2_ODD_SPEC, 2047, True, 20, 3, 10, False)}
    if args.only:
        name, spec, batch, normal, steps, warmup, psteps, fresh = small[args.only]
        print(json.dumps({name: bench_small(rs, eng, spec, batch, normal, steps, warmup, args.eager, psteps, fresh)}),
              flush=True)
        return

    if args.calibration_copy:
        from rstorch_amd import _ffi
        n = 1 << 27  # doubles = 1 GiB
        src, dst = eng.normal(1, n, SEED, 3000), eng.empty(1, n)
        for _ in range(2):
            _ffi.check(eng.lib.rst_relu_forward(eng.handle, src.ptr, dst.ptr, n))
        eng.synchronize()
        del src, dst

    dm, x, y = make_model(rs, eng, C4_SPEC, C4_BATCH, True)
    if args.eager:
        dm.graph_enable(False)
    if args.no_pair:
        dm.pair_gradients(False)
    tensors, params = dm.parameter_count()
    wall, dev_ms, loss, recs = time_steps(eng, dm, x, y, args.steps, args.warmup, True)
    ms_per_step = wall * 1e3 / args.steps
    per_step = time_steps.per_step_ms
    kernels = summarise(recs, args.steps)
    dm.close()
    log("C4: %.3f ms/step, loss %.6f" % (ms_per_step, loss))

    gemm_kinds = [k for k in ("linear_forward", "grad_weight", "grad_input", "grad_pair") if k in kernels]
    dominant = max(gemm_kinds, key=lambda k: kernels[k]["ms_per_step"])
    d = kernels[dominant]
    traffic_current = kernel_sources_digest() == C4_TRAFFIC_SOURCE["kernel_sources_sha16"]
    if not traffic_current:
        log("WARNING: the contraction kernel sources have changed since profiles/c4_hbm_traffic.md was collected: "
            "roofline.traffic is reported as null until the counters are collected again")
    launches = [r for r in recs if r["kernel"] == dominant]
    flops_per_launch = sum(r["flops"] for r in launches) / len(launches)
    kernel_names = {"grad_pair": "gemm_f64_mfma_dma_pair (a layer's weight gradient + SGD and the next layer's "
                                 "input gradient in one grid)"}
    roofline = {"kernel": kernel_names.get(dominant, "gemm_f64_mfma_dma (" + dominant + ")"), "bound": "mfma",
                "achieved": d["achieved_tflops"], "peak": PEAK_FP64_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": d["frac"],
                "traffic": C4_TRAFFIC_BYTES_PER_LAUNCH.get(dominant) if traffic_current else None,
                # the counters need a profiler run of their own (rocprofv3 --pmc): the figure is the one
                # of the committed profile, valid while the kernel sources are the ones it was taken on
                "traffic_measured_in_run": False,
                "traffic_unit": "bytes per launch (L2 misses + write-backs, rocprofv3 FETCH_SIZE/WRITE_SIZE)",
                "traffic_source": dict(C4_TRAFFIC_SOURCE, kernel_sources_sha16_now=kernel_sources_digest()),
                "algorithmic_bytes_per_launch": sum(r["bytes"] for r in launches) / len(launches),
                "avg_launch_ms": d["avg_launch_ms"], "flops_per_launch": flops_per_launch}
    gemm_ms = sum(kernels[k]["ms_per_step"] for k in gemm_kinds)
    gemm_flops = sum(r["flops"] for r in recs if r["kernel"] in gemm_kinds) / args.steps
    all_gemm = {"tflops": gemm_flops / (gemm_ms * 1e-3) / 1e12,
                "frac": gemm_flops / (gemm_ms * 1e-3) / 1e12 / PEAK_FP64_MFMA_TFLOPS,
                "flops_per_step": gemm_flops, "ms_per_step": gemm_ms,
                "first_layer_input_gradient": "skipped (the README loop discards it)"}

    result = {
        "metric": "training_steps_per_s", "value": args.steps / wall, "unit": "steps/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": "C4 deep MLP: (Linear(4096,4096)+ReLU)x8 -> Linear(4096,32768), "
                               "batch 1024, CrossEntropyLoss, SGD lr=0.01 (BASELINE.json configs[4])",
                   "batch": C4_BATCH, "parameters": params, "samples_per_s": args.steps / wall * C4_BATCH,
                   "device": info["name"], "device_ms_per_step": dev_ms / args.steps,
                   "device_ms_per_step_median": per_step[len(per_step) // 2],
                   "device_ms_per_step_min": per_step[0],
                   "final_loss": loss, "per_launch_events": True,
                   "paired_gradient_launches": not args.no_pair,
                   # the loss is computed on the device every step but the host does not read it inside
                   # the timed loop (one read after the last step); the README loop, which reads the
                   # loss and the accuracy every step, is reported as readme_loop
                   "per_step_loss_read": False},
        "roofline": roofline,
        "contractions": all_gemm,
        "kernels": kernels,
    }

    if not args.no_extra:
        log("SGD alone (configs[3]) ...")
        result["sgd_c3"] = bench_sgd_c3(rs, eng)
        result["relu_standalone"] = bench_relu(rs, eng)
        log("other configurations ...")
        result["other_configs"] = {
            name: bench_small(rs, eng, spec, batch, normal, steps, warmup, args.eager, psteps, fresh)
            for name, spec, batch, normal, steps, warmup, psteps, fresh in small.values()}
        result["readme_loop"] = readme_loop
        for config, name in (("C0", "C0_readme_b32"), ("C1", "C1_readme_b8192"), ("C2", "C2_wide_b2048")):
            # (the single-call step on one resident batch: the README loop also walks a small resident pool;
            # where measured, beside it the fraction of that step with the loss read every step, which is
            # what the loop does as well)
            other = result["other_configs"][name]
            resident = other.get("one_resident_batch", other)
            loop = readme_loop.get(config, {}).get("compiled", {})
            if "steps_per_s" in loop:
                loop["fraction_of_single_call_step"] = loop["steps_per_s"] / resident["steps_per_s"]
                if "with_loss_read_every_step" in resident:
                    loop["fraction_of_single_call_step_with_loss_read"] = \
                        loop["steps_per_s"] / resident["with_loss_read_every_step"]["steps_per_s"]
        if "steps_per_s" in readme_loop.get("C4", {}).get("compiled", {}):
            readme_loop["C4"]["compiled"]["fraction_of_single_call_step"] = \
                readme_loop["C4"]["compiled"]["steps_per_s"] / (args.steps / wall)
        log("host-fed (PCIe-inclusive) runs ...")
        result["host_fed"] = {
            "C1_readme_b8192": bench_staged(rs, eng, C01_SPEC, 8192, False, 100, 10),
            "C1_readme_b8192_pinned_in_place": bench_staged(rs, eng, C01_SPEC, 8192, False, 100, 10, True),
            "C4_deep_b1024": bench_staged(rs, eng, C4_SPEC, C4_BATCH, True, 10, 3),
        }

    if not args.no_cpu:
        log("CPU baseline (oracle) ...")
        cpu, sample_batches, cores = cpu_baseline()
        result["cpu_baseline"] = {
            "value": cpu["single"]["steps_per_s"], "unit": "steps/s", "cores": 1, "kind": "port",
            "sample": "oracle (C restatement of the reference, single thread like the reference) on "
                      "the same C4 network: ONE whole step at the full batch of 1024, timed; beside it "
                      "(detail) steps at batch %d and %d with t(B) = a + b*B fitted and evaluated at "
                      "1024 as a cross-check" % tuple(sample_batches),
            "detail": cpu["single"],
        }
        result["cpu_baseline_all_cores"] = {
            "value": cpu["all"]["steps_per_s_fitted"], "unit": "steps/s", "cores": cores, "kind": "port",
            "sample": "steps at batch %d and %d, OpenMP over the oracle's contraction blocks, "
                      "t(B) = a + b*B fitted and evaluated at 1024" % tuple(sample_batches),
            "detail": cpu["all"],
        }
        if not args.no_extra:
            log("CPU baselines of the other configurations ...")
            oc = result["other_configs"]
            oc["C0_readme_b32"]["cpu_baseline"] = cpu_baseline_small(C01_SPEC, 32, False, 1875)
            oc["C1_readme_b8192"]["cpu_baseline"] = cpu_baseline_small(C01_SPEC, 8192, False, 20)
            oc["C2_wide_b2048"]["cpu_baseline"] = cpu_baseline_small(C2_SPEC, 2048, True, 3)
            result["sgd_c3"]["cpu_baseline"] = cpu_baseline_sgd_c3()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
