"""Benchmark of the DVM hot path on one MI355X.

Headline (BASELINE.json configs[1]): fused batch-norm forward with training statistics, fp32 NCHW
[32,256,56,56], one launch of the vector VM. `value` is algorithmic GB/s: the tensor is read once
and written once (2 x 102 760 448 B + 2 KB parameters = 205 522 944 B per step) over the wall time
of K steps with inputs resident in HBM. The same JSON line carries the roofline figure of the kernel
(HIP events on the launch stream), a CPU baseline (the C oracle on this box's host, one core) and,
under "configs", the other BASELINE configs (latency / JIT microseconds / GB/s).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes one launch of the headline kernel moves come from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs of
# `bench.py --traffic-probe`, each scaled by the same counter's reading for a plain copy of known size. A counter
# cannot be read from inside this script, so the figure is read from the committed summary of those runs, which
# also records a hash of the sources that decide the kernel's schedule (tests/test_host.py fails when they changed
# since the measurement).
TRAFFIC_SUMMARY = os.path.join("profiles", "vec_rx_batchnorm_hbm_traffic.txt")
SCHEDULE_SOURCES = ["dvm_amd/csrc/device/vm_vector.hip", "dvm_amd/csrc/device/vm_vector_sweep.hip", "dvm_amd/csrc/device/vec_common.h",
                    "dvm_amd/csrc/isa_gfx950.h", "dvm_amd/csrc/host/schedule.cc", "dvm_amd/csrc/host/emit_vector.cc",
                    "dvm_amd/csrc/host/peephole.cc"]


def schedule_sources_hash():
    import hashlib
    h = hashlib.sha256()
    for rel in SCHEDULE_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def headline_traffic():
    """(bytes per launch or None, where the figure comes from) out of the committed counter summary."""
    import re
    path = os.path.join(ROOT, TRAFFIC_SUMMARY)
    try:
        text = open(path).read()
    except OSError:
        return None, "no counter summary (%s)" % TRAFFIC_SUMMARY
    m = re.search(r"traffic_bytes_per_launch = (\d+)", text)
    h = re.search(r"schedule_sources_sha256 = (\w+)", text)
    if not m:
        return None, "%s holds no traffic_bytes_per_launch line" % TRAFFIC_SUMMARY
    fresh = h is not None and h.group(1) == schedule_sources_hash()
    return int(m.group(1)), "%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy; %s)" % (
        TRAFFIC_SUMMARY, "measured on these sources" if fresh else "measured on an EARLIER version of the schedule sources")
METRIC = "fused-op HBM GB/s (% roofline) + matmul TFLOPS (% MFMA peak); JIT us/shape"


def bn_graph(t, x, g, b, n_red, eps):
    """mean / biased variance over N,H,W in one sweep (sum x, sum x^2, fp64 accumulation), then
    y = x * scale + shift with per-channel scale = gamma / sqrt(var + eps), shift = beta - mean * scale."""
    inv = 1.0 / n_red
    mean = t.mul(t.sum(x, (0, 2, 3), True), inv)
    ex2 = t.mul(t.sum(t.mul(x, x), (0, 2, 3), True), inv)
    var = t.sub(ex2, t.mul(mean, mean))
    scale = t.div(g, t.sqrt(t.add(var, eps)))
    shift = t.sub(b, t.mul(mean, scale))
    return t.add(t.mul(x, scale), shift)


def bn_graph_two_pass(t, x, g, b, n_red, eps):
    """The graph of the reference's own example (examples/02_batchnorm.py:27-42, with eps): the variance from the
    centred values, i.e. a second statistics sweep over x - mean (robust where |mean| >> sigma; one more pass over x)."""
    inv = 1.0 / n_red
    mean = t.mul(t.sum(x, (0, 2, 3), True), inv)
    xc = t.sub(x, mean)
    var = t.mul(t.sum(t.mul(xc, xc), (0, 2, 3), True), inv)
    return t.add(t.mul(t.div(xc, t.sqrt(t.add(var, eps))), g), b)


def vector_kernel_name(das_text):
    """Name of the vector VM kernel a one-launch program runs on, from its disassembly header."""
    head = das_text.split("\n")[1]
    if "sched=reduce-x" in head:
        return "dvm_vm_vec_rx_sw" if " sweeps" in head else "dvm_vm_vec_rx"
    return "dvm_vm_vec_ry" if "sched=reduce-y" in head else "dvm_vm_vec_pw"


def bench_batchnorm_two_pass(x, g, b, iters=20):
    """The two-pass form of the headline graph at the headline shape: time, launches, parity against float64."""
    from dvm_amd.tester import Tester
    n, c, h, w = x.shape
    t = Tester("split:dyn")
    lx, lg, lb = t.load(x), t.load(g), t.load(b)
    out = t.store(bn_graph_two_pass(t, lx, lg, lb, n * h * w, 1e-5))
    t.codegen()
    t.run()
    got = t.output(out)
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean((0, 2, 3), keepdims=True)) / np.sqrt(x64.var((0, 2, 3), keepdims=True) + 1e-5) * g + b
    if not np.allclose(got, want, rtol=1e-5, atol=1e-5):
        raise RuntimeError("two-pass batch-norm result differs from the NumPy golden")
    smp = sorted(t.perf_samples(warmup=3, iters=iters))
    med = smp[len(smp) // 2]
    alg = 2 * x.nbytes + g.nbytes + b.nbytes
    return {"graph": "sum(x) -> x - mean -> sum(sq) -> normalise (examples/02_batchnorm.py:27-42 with eps)", "launches": t.num_launches(),
            "kernel": vector_kernel_name(t.das()), "kernel_us_median": round(med, 2), "kernel_us_min": round(smp[0], 2),
            "kernel_us_mean": round(sum(smp) / len(smp), 2), "algorithmic_GBps": round(alg / med / 1e3, 1),
            "frac_of_8TBps": round(alg / med / 1e3 / HBM_PEAK_GBS, 4), "parity_max_abs_err_vs_numpy_f64": float(np.max(np.abs(got - want)))}


def bench_batchnorm(steps, warmup):
    from dvm_amd.tester import Tester
    n, c, h, w = 32, 256, 56, 56
    rng = np.random.default_rng(1002)
    x = rng.standard_normal([n, c, h, w], dtype=np.float32)
    g = rng.uniform(0.5, 1.5, [1, c, 1, 1]).astype(np.float32)
    b = rng.normal(0, 0.1, [1, c, 1, 1]).astype(np.float32)
    t = Tester("split:dyn")
    lx, lg, lb = t.load(x), t.load(g), t.load(b)
    out = t.store(bn_graph(t, lx, lg, lb, n * h * w, 1e-5))
    t.codegen()
    kernel_name = vector_kernel_name(t.das())
    jit_cold = t.jit_us()
    t.codegen()
    jit_warm = t.jit_us()
    launches = t.num_launches()
    for _ in range(warmup):
        t.bare_run()
    # K timed steps: asynchronous launches, one synchronisation at the end
    from dvm_amd import _core
    t0 = time.perf_counter()
    for _ in range(steps - 1):
        _core.PyKernel.run(t, sync=False)
    _core.PyKernel.run(t, sync=True)
    wall = time.perf_counter() - t0
    ms_per_step = wall / steps * 1e3
    samples = sorted(t.perf_samples(warmup=3, iters=max(20, steps)))
    ev_min, ev_mean, ev_median = samples[0], sum(samples) / len(samples), samples[len(samples) // 2]
    got = t.output(out)
    alg_bytes = 2 * x.nbytes + g.nbytes + b.nbytes
    # parity gate before any number counts
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean((0, 2, 3), keepdims=True)) / np.sqrt(x64.var((0, 2, 3), keepdims=True) + 1e-5) * g + b
    err = float(np.max(np.abs(got - want) / (np.abs(want) + 1.0)))
    if not np.allclose(got, want, rtol=1e-5, atol=1e-5):
        raise RuntimeError("batch-norm result differs from the NumPy golden: max rel err %g" % err)
    return {
        "x": x, "g": g, "b": b, "alg_bytes": alg_bytes, "ms_per_step": ms_per_step, "kernel_us_mean": ev_mean,
        "kernel_us_min": ev_min, "kernel_us_median": ev_median, "jit_us_cold": jit_cold, "jit_us_warm": jit_warm, "launches": launches, "max_rel_err": err,
        "kernel": kernel_name,
    }


def _numpy_batchnorm(x, g, b):
    """The NumPy golden of the reference's example (examples/02_batchnorm.py:19-24, with eps): float64 statistics."""
    x64 = x.astype(np.float64)
    mean = x64.mean((0, 2, 3), keepdims=True)
    var = x64.var((0, 2, 3), keepdims=True)
    return ((x64 - mean) / np.sqrt(var + 1e-5) * g + b).astype(np.float32)


def _blas_threads():
    try:
        from threadpoolctl import threadpool_info
        return [{"api": i.get("internal_api"), "threads": i.get("num_threads")} for i in threadpool_info()]
    except Exception:  # noqa: BLE001
        return os.environ.get("OMP_NUM_THREADS", "unknown")


def cpu_baseline_batchnorm(x, g, b, alg_bytes):
    """The CPU reference beside the GPU number: the reference has no CPU execution path for this backend, so the
    baseline is the NumPy golden itself (3 warm-ups on a slice, median of >= 5 runs, about 15 s of CPU work on a
    quarter of the batch, scaled to the full tensor's bytes); the scalar C port of the oracle is timed as well."""
    from oracle import oracle as ora
    part = x[:8]  # a bounded sample: 8 of the 32 images, same channel count and image size
    part_bytes = 2 * part.nbytes + g.nbytes + b.nbytes
    for _ in range(3):
        _numpy_batchnorm(part[:1], g, b)
    times = []
    t_all = time.perf_counter()
    while len(times) < 5 or (time.perf_counter() - t_all < 12.0 and len(times) < 40):
        t0 = time.perf_counter()
        _numpy_batchnorm(part, g, b)
        times.append(time.perf_counter() - t0)
    times.sort()
    np_med = times[len(times) // 2]
    ora.batchnorm_nchw(x[:2], g, b, 1e-5)
    ctimes = []
    for _ in range(5):
        t0 = time.perf_counter()
        ora.batchnorm_nchw(part, g, b, 1e-5)
        ctimes.append(time.perf_counter() - t0)
    ctimes.sort()
    return {"value": round(part_bytes / np_med / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "NumPy golden (float64 formula of examples/02_batchnorm.py with eps) on images 0..7 of the [32,256,56,56] tensor "
                      "(51.4 MB of algorithmic traffic per run), median of %d runs of %.2f s; elementwise NumPy runs on one thread" % (len(times), np_med),
            "host_cpu_count": os.cpu_count(), "blas": _blas_threads(),
            "c_port": {"value": round(part_bytes / ctimes[len(ctimes) // 2] / 1e9, 3), "unit": "GB/s", "cores": 1,
                       "sample": "scalar C oracle (oracle/dvm_oracle.c ora_batchnorm_nchw) on the same 8 images, median of 5 runs"}}


def bench_add():
    """configs[0]: fp32 [32,32] add; launch latency and JIT microseconds (a plumbing check)."""
    from dvm_amd.tester import Tester
    x, y = np.full([32, 32], 0.1, np.float32), np.full([32, 32], 0.3, np.float32)
    t = Tester("split:dyn")
    out = t.store(t.add(t.load(x), t.load(y)))
    t.codegen()
    cold = t.jit_us()
    t.codegen()
    warm = t.jit_us()
    t.run()
    assert np.array_equal(t.output(out), x + y)
    mn, _, mean = t.perf(warmup=3, iters=50)
    return {"kernel_us_mean": round(mean, 2), "kernel_us_min": round(mn, 2), "jit_us_cold": round(cold, 2), "jit_us_warm": round(warm, 2)}


def bench_rmsnorm(calls=200):
    """configs[2]: bf16 residual-add + RMSNorm + cast, R ~ U{1..8192} per call, 200 seeded calls."""
    from dvm_amd.tester import Tester
    rng = np.random.default_rng(1003)
    rows = rng.integers(1, 8193, calls)
    rmax = int(rows.max())
    xs = Tester.convert_to_bf16(rng.standard_normal([rmax, 4096], dtype=np.float32))
    rs = Tester.convert_to_bf16(rng.standard_normal([rmax, 4096], dtype=np.float32))
    wv = rng.uniform(0.9, 1.1, [4096]).astype(np.float32)
    t = Tester("split:dyn")
    x, r, w = t.load([1, 4096], "bfloat16"), t.load([1, 4096], "bfloat16"), t.load([4096], "float32")
    x_shape, r_shape = t.load_shape(x), t.load_shape(r)
    hf = t.cast(t.add(x, r), "float32")
    ss = t.sum(t.mul(hf, hf), (1,), True)
    rstd = t.div(1.0, t.sqrt(t.add(t.mul(ss, 1.0 / 4096), 1e-6)))
    out = t.store(t.cast(t.mul(t.mul(hf, rstd), w), "bfloat16"))
    t.input(w, wv)
    # the inputs live on the device once, at their largest extent; a call only changes the shape behind the loads (the
    # dynamic-shape interface, src/pybind_api.cc IntArrayRef) and generates code again, as a serving loop would
    t.input(x, xs)
    t.input(r, rs)
    jit, gbs, big_gbs, big_frac = [], [], [], []
    total_bytes = 0
    total_us = 0.0
    checked = 0
    for i, R in enumerate(rows):
        R = int(R)
        x_shape.update([R, 4096])
        r_shape.update([R, 4096])
        t.codegen()
        jit.append(t.jit_us())
        mn, _, mean = t.perf(warmup=1, iters=5)
        nbytes = 24576 * R + 16384
        total_bytes += nbytes
        total_us += mean
        gbs.append(nbytes / mean / 1e3)
        if R >= 512:
            big_gbs.append(nbytes / mean / 1e3)
        if i % 40 == 0:  # parity spot checks against the NumPy golden (1e-2)
            got = Tester.convert_from_bf16(t.output(out))
            hh = Tester.convert_from_bf16(Tester.convert_to_bf16(Tester.convert_from_bf16(xs[:R]) + Tester.convert_from_bf16(rs[:R]))).astype(np.float64)
            want = hh / np.sqrt((hh * hh).mean(1, keepdims=True) + 1e-6) * wv
            if not np.allclose(got, want, rtol=1e-2, atol=1e-2):
                raise RuntimeError("RMSNorm result differs from the NumPy golden at R=%d" % R)
            checked += 1
    jit_sorted = sorted(jit[1:])
    # the same 200 shapes again with nothing between the code generations (no launches, no copies): how the
    # reference's emitter was timed (Normalize + CodeGen in a loop), i.e. with warm caches
    back = []
    for R in rows:
        x_shape.update([int(R), 4096])
        r_shape.update([int(R), 4096])
        t.codegen()
        back.append(t.jit_us())
    back.sort()
    return {
        "calls": calls, "sum_alg_GB": round(total_bytes / 1e9, 3), "aggregate_GBps": round(total_bytes / total_us / 1e3, 1),
        "aggregate_frac_of_8TBps": round(total_bytes / total_us / 1e3 / HBM_PEAK_GBS, 4),
        "R>=512_median_GBps": round(float(np.median(big_gbs)), 1), "R>=512_median_frac": round(float(np.median(big_gbs)) / HBM_PEAK_GBS, 4),
        "jit_us_first": round(jit[0], 2), "jit_us_median": round(jit_sorted[len(jit_sorted) // 2], 2), "jit_us_max": round(jit_sorted[-1], 2),
        "jit_us_back_to_back_median": round(back[len(back) // 2], 2), "jit_us_back_to_back_min": round(back[0], 2),
        "launches_per_call": t.num_launches(), "parity_checked_calls": checked,
    }


def bench_matmul(m=8192, n=4096, k=4096, iters=20):
    """configs[4]: bf16 A[m,k] x B[k,n], fp32 accumulate, epilogue bias add + SiLU + cast to bf16, one launch."""
    from dvm_amd.tester import Tester
    rng = np.random.default_rng(1005)
    a = Tester.convert_to_bf16((rng.standard_normal([m, k], dtype=np.float32) / 8.0))
    b = Tester.convert_to_bf16((rng.standard_normal([k, n], dtype=np.float32) / 8.0))
    bias = (rng.standard_normal([n], dtype=np.float32) * np.float32(np.sqrt(0.1)))
    t = Tester("mix")
    x, y, bb = t.load(a.shape, "bfloat16"), t.load(b.shape, "bfloat16"), t.load(bias)
    t.input(x, a)
    t.input(y, b)
    h = t.add(t.cast(t.matmul(x, y, False, False), "float32"), bb)
    out = t.store(t.cast(t.div(h, t.add(t.exp(t.mul(h, -1.0)), 1.0)), "bfloat16"))
    t.codegen()
    cold = t.jit_us()
    t.run()
    got = Tester.convert_from_bf16(t.output(out))
    # parity on sampled rows against the NumPy golden (bf16 tolerance 1e-2)
    rows = rng.integers(0, m, 16)
    af, bf = Tester.convert_from_bf16(a[rows]).astype(np.float64), Tester.convert_from_bf16(b).astype(np.float64)
    hh = Tester.convert_from_bf16(Tester.convert_to_bf16((af @ bf).astype(np.float32))).astype(np.float64) + bias
    want = hh / (1.0 + np.exp(-hh))
    if not np.allclose(got[rows], want, rtol=1e-2, atol=1e-2):
        raise RuntimeError("matmul epilogue result differs from the NumPy golden")
    smp = sorted(t.perf_samples(warmup=3, iters=iters))
    mn, mean, med = smp[0], sum(smp) / len(smp), smp[len(smp) // 2]
    flops = 2.0 * m * n * k
    return {"shape": [m, n, k], "kernel_us_mean": round(mean, 2), "kernel_us_min": round(mn, 2), "kernel_us_median": round(med, 2), "TFLOPs": round(flops / mean / 1e6, 1),
            "frac_of_2.5PFLOPs": round(flops / mean / 1e6 / 2500.0, 4), "launches": t.num_launches(), "jit_us_cold": round(cold, 2),
            "parity_rows_checked": len(rows)}


def bench_attention(b=8, h=32, s=2048, d=128, iters=10):
    """configs[3]: fused attention softmax(Q K^T / sqrt(d)) V, fp16, one launch; FLOPs = 4*b*h*s*s*d."""
    import math
    from dvm_amd.tester import Tester
    rng = np.random.default_rng(1004)
    q, k, v = (rng.standard_normal((b, h, s, d), dtype=np.float32).astype(np.float16) for _ in range(3))
    t = Tester("mix")
    sc = t.mul(t.matmul(t.load(q), t.load(k), False, True), 1.0 / math.sqrt(d))
    x = t.cast(sc, "float32")
    x = t.sub(x, t.max(x, (3,), True))
    e = t.exp(x)
    p = t.cast(t.div(e, t.sum(e, (3,), True)), "float16")
    out = t.store(t.matmul(p, t.load(v), False, False))
    t.codegen()
    cold = t.jit_us()
    t.run()
    got = t.output(out)
    for bi, hi in ((0, 0), (b - 1, h - 1)):  # parity on two heads against the NumPy golden (1e-2)
        sm = (q[bi, hi].astype(np.float64) @ k[bi, hi].astype(np.float64).T) / math.sqrt(d)
        sm = np.exp(sm - sm.max(-1, keepdims=True))
        want = (sm / sm.sum(-1, keepdims=True)) @ v[bi, hi].astype(np.float64)
        if not np.allclose(got[bi, hi], want, rtol=1e-2, atol=1e-2):
            raise RuntimeError("attention result differs from the NumPy golden")
    smp = sorted(t.perf_samples(warmup=2, iters=iters))
    mn, mean, med = smp[0], sum(smp) / len(smp), smp[len(smp) // 2]
    flops = 4.0 * b * h * s * s * d
    return {"shape": [b, h, s, d], "kernel_us_mean": round(mean, 2), "kernel_us_min": round(mn, 2), "kernel_us_median": round(med, 2), "TFLOPs": round(flops / mean / 1e6, 1),
            "frac_of_2.5PFLOPs": round(flops / mean / 1e6 / 2500.0, 4), "launches": t.num_launches(), "jit_us_cold": round(cold, 2),
            "parity_heads_checked": 2}


TORCH_ANCHOR = r"""
import json, sys, torch
dev = "cuda:0"
def timeit(f, warm, iters):
    for _ in range(warm): f()
    torch.cuda.synchronize()
    ts = []
    for _ in range(iters):
        a = torch.cuda.Event(enable_timing=True); b = torch.cuda.Event(enable_timing=True)
        a.record(); f(); b.record(); b.synchronize(); ts.append(a.elapsed_time(b) * 1e3)
    ts.sort(); return ts[0], ts[len(ts) // 2], sum(ts) / len(ts)
g = torch.Generator(device=dev).manual_seed(1)
out = {}
if "matmul" in sys.argv:
    A = (torch.randn(8192, 4096, device=dev, generator=g) / 8).bfloat16(); B = (torch.randn(4096, 4096, device=dev, generator=g) / 8).bfloat16()
    mn, med, mean = timeit(lambda: torch.matmul(A, B), 10, 30)
    out["matmul"] = {"op": "torch.matmul bf16 8192x4096x4096 (plain product, no epilogue)", "us_min": round(mn, 1), "us_median": round(med, 1),
                     "us_mean": round(mean, 1), "TFLOPs_median": round(2 * 8192 * 4096 * 4096 / med / 1e6, 1)}
if "attention" in sys.argv:
    q, k, v = (torch.randn(8, 32, 2048, 128, device=dev, generator=g).half() for _ in range(3))
    mn, med, mean = timeit(lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v), 5, 20)
    out["attention"] = {"op": "torch.nn.functional.scaled_dot_product_attention fp16 [8,32,2048,128]", "us_min": round(mn, 1), "us_median": round(med, 1),
                        "us_mean": round(mean, 1), "TFLOPs_median": round(4 * 8 * 32 * 2048 * 2048 * 128 / med / 1e6, 1)}
print("ANCHOR " + json.dumps(out))
"""


def torch_anchors(which):
    """The vendor libraries on the same box, in a process of their own that imports torch first: torch.matmul
    (hipBLASLt) and scaled_dot_product_attention at the shapes of configs[4] and configs[3], timed with events on
    torch's stream. A stated ceiling of what this box sustains, not a target and never part of the product path."""
    import subprocess
    try:
        r = subprocess.run([sys.executable, "-c", TORCH_ANCHOR] + list(which), capture_output=True, text=True, timeout=420)
        for line in r.stdout.splitlines():
            if line.startswith("ANCHOR "):
                return json.loads(line[7:])
        return {"error": (r.stderr or "no output").strip().splitlines()[-1][:200]}
    except Exception as e:  # noqa: BLE001  (no torch, no time: the bench line goes out without the anchors)
        return {"error": str(e)[:200]}


def traffic_probe():
    """For the counter runs (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE): five launches of the headline kernel
    and five launches of a plain copy of the same tensor through the pointwise VM kernel, whose traffic is
    known (102 760 448 B read, as many written); the copy calibrates the counters' unit."""
    from dvm_amd.tester import Tester
    bn = bench_batchnorm(5, 2)
    t = Tester("split")
    out = t.store(t.copy(t.load(bn["x"])))
    t.codegen()
    for _ in range(5):
        t.bare_run()
    t.run()
    assert np.array_equal(t.output(out), bn["x"])
    print(json.dumps({"probe": "traffic", "copy_bytes_each_way": int(bn["x"].nbytes)}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline leg")
    ap.add_argument("--only-headline", action="store_true", help="omit the other BASELINE configs")
    ap.add_argument("--skip-torch-anchor", action="store_true", help="do not time torch.matmul / SDPA beside the two MFMA configs")
    ap.add_argument("--configs", default="add,rmsnorm,attention,matmul", help="which of the other BASELINE configs to run (comma separated)")
    ap.add_argument("--traffic-probe", action="store_true", help="launch the headline kernel and a plain copy only (for counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the DVM hot path is a single-device operator JIT (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import dvm_amd as dvm
    if not dvm.Device.available():
        print("bench.py needs an MI355X and the built HIP device layer (dvm_amd/lib/libdvm_hip.so)", file=sys.stderr)
        sys.exit(1)
    if args.traffic_probe:
        traffic_probe()
        return
    bn = bench_batchnorm(args.steps, args.warmup)
    value = bn["alg_bytes"] / (bn["ms_per_step"] * 1e-3) / 1e9
    achieved = bn["alg_bytes"] / (bn["kernel_us_mean"] * 1e-6) / 1e9
    traffic, traffic_source = headline_traffic()
    line = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(bn["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: fused batch-norm forward (training statistics), fp32 NCHW [32,256,56,56], eps=1e-5, one launch",
                   "algorithmic_bytes_per_step": bn["alg_bytes"], "launches_per_step": bn["launches"],
                   "jit_us_cold": round(bn["jit_us_cold"], 2), "jit_us_warm": round(bn["jit_us_warm"], 2),
                   "parity_max_rel_err_vs_numpy_f64": bn["max_rel_err"]},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": bn["kernel"], "kernel_us_mean": round(bn["kernel_us_mean"], 2), "kernel_us_median": round(bn["kernel_us_median"], 2),
                     "kernel_us_min": round(bn["kernel_us_min"], 2)},
    }
    if not args.skip_cpu:
        line["cpu_baseline"] = cpu_baseline_batchnorm(bn["x"], bn["g"], bn["b"], bn["alg_bytes"])
    if not args.only_headline:
        others = {"add": ("add_fp32_32x32", bench_add), "rmsnorm": ("residual_rmsnorm_bf16_dynamic", bench_rmsnorm),
                  "attention": ("attention_fp16_b8_h32_s2048_d128", bench_attention),
                  "matmul": ("matmul_bias_silu_bf16_8192x4096x4096", bench_matmul)}
        line["configs"] = {others[c][0]: others[c][1]() for c in args.configs.split(",") if c in others}
        line["configs"]["batchnorm_two_pass_fp32_32x256x56x56"] = bench_batchnorm_two_pass(bn["x"], bn["g"], bn["b"])
        wanted = [c for c in ("matmul", "attention") if c in args.configs.split(",")]
        if wanted and not args.skip_torch_anchor:
            anchors = torch_anchors(wanted)
            for c in wanted:
                line["configs"][others[c][0]]["same_box_vendor_library"] = anchors.get(c, anchors)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
