#!/usr/bin/env python3
"""Benchmark of the TC HIP backend on one MI355X.

One "step" = one launch of the compiled TC over one batch of synthetic, seeded inputs that are
already resident in HBM.  The headline workload is the HBM-bound tensordot
O(n,c1,c3,h,w) +=! I0(n,c1,r_c2,h,w) * I1(n,r_c2,c3,h,w) at N=32, C1=512, C2=8, C3=2, H=W=28;
`--config` selects another of the five workloads; the other four are always measured too and
reported under "others" (kernel time, roofline, traffic); `--suite` appends the reference's other
benchmark programs at their default sizes under "suite".  Prints ONE JSON line.

Before the W warm-up steps of a workload the kernel is launched back to back for a fixed time
(--spin-ms, 150 ms): the kernels here run for 3 to 90 us, a handful of launches end before the
device has left its idle clocks, and what is measured is the steady state.  The spin is not part
of the warm-up or of the K timed steps.

Device memory comes from the library's own thin HIP layer (tensorcomprehensions_amd.DeviceBuffer):
PyTorch is not loaded, so the kernels are compiled by the hipRTC of the ROCm installation and
launched through its runtime (PyTorch bundles older copies of both).  Only `--suite`, which times
PyTorch's own GPU routines next to the comprehensions, loads PyTorch, first, for the whole process;
the ATen CPU baseline runs in a child process.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
FP32_PEAK_TFLOPS = 157.3       # MI355X fp32 matrix/vector, published
FP16_PEAK_TFLOPS = 2500.0      # MI355X dense fp16 matrix, published


def flops(name, shapes):
    if "tensordot" in name:
        n, c1, c2, h, w = shapes[0]
        c3 = shapes[1][2]
        return 2 * n * c1 * c2 * c3 * h * w
    if "batch_matmul" in name:
        b, n, m = shapes[0]
        return 2 * b * n * m * shapes[1][2]
    if "group_convolution" in name:
        n, g, c, h, w = shapes[0]
        _, f, _, kh, kw = shapes[1]
        oh, ow = h - kh + 1, w - kw + 1
        return n * g * f * oh * ow * (2 * c * kh * kw + 1)
    m, n = shapes[0]
    return 6 * m * n


SPIN_MS = 150.0
# Options cache written by the autotuner (`--tune ... --save-cache`), compcache wire format; the
# backend adds ".hip" to the name (HipBackend::makeDeviceFilename).
OPTIONS_CACHE = os.path.join(ROOT, "tensorcomprehensions_amd", "tuned", "benchmark_configs")
MIN_BURST = 200                # launches per timed burst of the workloads beside the headline one


def stored_options(name, ins):
    """The mapping options a workload is timed under: the best entry the autotuner recorded for
    this TC and these input sizes in the committed options cache; the tuner's base mapping of
    tests/workloads.py when the cache has none.  Returns (options text, where they came from)."""
    import tensorcomprehensions_amd as tc
    from tests import workloads as W
    src, entry = W.CONFIGS[name][0], W.CONFIGS[name][1]
    best = tc.load_from_cache(src, entry, ins, OPTIONS_CACHE, 1)
    if best:
        return best[0].to_text(), "autotuner's options cache " + os.path.relpath(OPTIONS_CACHE + ".hip", ROOT)
    return W.TUNED[name], "tests/workloads.py:TUNED (no entry in the options cache)"


def spin(ex, ins, outs, ms):
    """Back-to-back launches for about `ms` milliseconds of device time."""
    import tensorcomprehensions_amd as tc
    spent = 0.0
    while spent < ms * 1e3:
        spent += tc.profile_repeated(ex, ins, outs, 200)


def algorithmic_bytes(src, entry, ins):
    """Every input read once and every output written once."""
    import numpy as np
    import tensorcomprehensions_amd as tc
    n = sum(t.numel() * t.element_size() for t in ins)
    for dtype, shape, _ in tc.infer_output_tensor_info(src, entry, ins):
        count = 1
        for e in shape:
            count *= e
        n += count * np.dtype(dtype).itemsize
    return n


def to_device(array):
    """numpy -> device memory: a torch tensor when PyTorch is loaded (--suite), else a DeviceBuffer."""
    import tensorcomprehensions_amd as tc
    torch = sys.modules.get("torch")
    if torch is not None:
        return torch.from_numpy(array).cuda()
    return tc.DeviceBuffer.from_numpy(array)


def device_sync():
    torch = sys.modules.get("torch")
    if torch is not None:
        torch.cuda.synchronize()          # (profile_repeated has synchronised the stream already)


def measure(name, steps, warmup, options=None, bursts=1):
    import tensorcomprehensions_amd as tc
    from tests import workloads as W

    src, entry, shapes, _, _ = W.CONFIGS[name]
    ins = [to_device(a) for a in W.make_inputs(name)]
    opts, opts_from = (options, "command line or this run's tuning") if options else stored_options(name, ins)
    ex = tc.compile(src, entry, ins, opts)
    outs = tc.prepare_outputs(src, entry, ins)
    spin(ex, ins, outs, SPIN_MS)
    if warmup > 0:
        tc.profile_repeated(ex, ins, outs, warmup)      # W untimed steps; returns once they have finished
    # timed region: K steps issued back to back inside the library, bracketed by HIP events on the
    # launch stream (device time) and by the host clock around the synchronised whole
    t0 = time.perf_counter()
    device_us = tc.profile_repeated(ex, ins, outs, steps)
    device_sync()
    wall = time.perf_counter() - t0
    kernel_ms = device_us / 1e3 / steps
    if bursts > 1:
        # (the workloads beside the headline one: the median of several bursts of at least MIN_BURST
        # launches each, since K launches of a kernel of a few microseconds are over before the
        # figure has settled)
        n = max(steps, MIN_BURST)
        more = [tc.profile_repeated(ex, ins, outs, n) / n for _ in range(bursts)]
        kernel_ms = sorted(more)[len(more) // 2] / 1e3
    nbytes = algorithmic_bytes(src, entry, ins)
    return {
        "name": name, "options": opts, "options_from": opts_from, "wall_s": wall, "kernel_ms": kernel_ms, "bytes": nbytes,
        "flops": flops(name, shapes), "launch": [ex.launch_bounds(k) for k in range(ex.num_kernels)],
        "ins": ins, "outs": outs,
    }


COPY_TC = "def copy(float(N) I) -> (O) { O(i) = I(i) }"
COPY_ELEMS = 64 * 1024 * 1024           # 256 MiB read + 256 MiB written per launch


def calibrate_copy(steps):
    """A plain copy through the same backend: what FETCH_SIZE / WRITE_SIZE read for a kernel whose
    HBM traffic is known (268 435 456 B each way) scales the counters of the measured kernel."""
    import numpy as np
    import tensorcomprehensions_amd as tc
    src = to_device(np.ones(COPY_ELEMS, dtype=np.float32))
    ex = tc.compile(COPY_TC, "copy", [src], "naive;tile=4096;mapToThreads=256;mapToBlocks=16384;vectorWidth=4;unroll=16")
    (dst,) = tc.prepare_outputs(COPY_TC, "copy", [src])
    us = tc.profile_repeated(ex, [src], [dst], steps) / steps
    sys.stderr.write(f"copy calibration: {2 * 4 * COPY_ELEMS / us / 1e3:.1f} GB/s, {us:.1f} us per launch\n")


def launch_floor(steps, all_shapes=True):
    """Per-launch time of copy kernels that do next to nothing, issued back to back like the
    workloads (one wavefront; 64 and 500 blocks of 256 threads, 4 KiB each): what a launch costs
    on this device whatever the kernel does.  The 3 us workloads are to be read against it."""
    import numpy as np
    import tensorcomprehensions_amd as tc
    out = {}
    for label, n, opts in [("copy_1_block_of_64", 64, "naive;mapToThreads=64;mapToBlocks=1;tile=64"),
                           ("copy_64_blocks_of_256", 64 * 1024, "naive;mapToThreads=256;mapToBlocks=64;tile=1024;vectorWidth=4"),
                           ("copy_500_blocks_of_256", 500 * 1024, "naive;mapToThreads=256;mapToBlocks=500;tile=1024;vectorWidth=4")]:
        if not all_shapes and label != "copy_500_blocks_of_256":
            continue
        src = to_device(np.ones(n, dtype=np.float32))
        ex = tc.compile(COPY_TC, "copy", [src], opts)
        (dst,) = tc.prepare_outputs(COPY_TC, "copy", [src])
        spin(ex, [src], [dst], SPIN_MS)
        us = sorted(tc.profile_repeated(ex, [src], [dst], steps) / steps for _ in range(5))[2]
        out[label] = {"us_per_launch": round(us, 3), "kernel": ex.kernel_name(), "launch": ex.launch_bounds()}
    return out


ADD4_TC = "def add4(float(N) A, float(N) B, float(N) C, float(N) D) -> (O) { O(i) = A(i) + B(i) + C(i) + D(i) }"
STREAM_PROBES = [
    # name, TC, entry, input shapes, mapping options (each the best of a sweep over block shapes), bytes per launch
    ("copy 1:1", COPY_TC, "copy", [(COPY_ELEMS,)],
     "naive;tile=1024;mapToThreads=128;mapToBlocks=2097152;vectorWidth=2;unroll=8;useReadOnlyCache=1", 2 * 4 * COPY_ELEMS),
    # four reads to one write, 25 690 112 floats each: the mix and the volume of the large tensordot
    ("add4 4:1", ADD4_TC, "add4", [(25690112,)] * 4,
     "naive;tile=3136;mapToThreads=784;mapToBlocks=1000000;vectorWidth=2;unroll=128;useReadOnlyCache=1", 5 * 4 * 25690112),
    # the same with the tensordot's block: 196 threads in lanes of four
    ("add4 4:1, 196 threads x 4 lanes", ADD4_TC, "add4", [(25690112,)] * 4,
     "naive;tile=3136;mapToThreads=196;mapToBlocks=1000000;vectorWidth=4;unroll=128;useReadOnlyCache=1", 5 * 4 * 25690112),
    # reads only, the shape of the moments workload: one row per block
    ("rowsum 1:0", "def rowsum(float(M, N) X) -> (s) { s(m) +=! X(m, n) }", "rowsum", [(1024, 32768)],
     "naive;tile=1;mapToThreads=512;mapToBlocks=1024;matchLibraryCalls=1;unroll=8;vectorWidth=4;useReadOnlyCache=1",
     4 * (1024 * 32768 + 1024)),
]


def stream_probes(steps):
    """Kernels that do nothing but move data, through the same backend and launched like the
    workloads: what the memory system delivers for a read:write mix of 1:1, of 4:1 (the large
    tensordot's) and for reads alone (the moments').  Block shape matters: over thread counts, lane
    widths and elements per block the 4:1 stream measures 4.7 to 7.1 TB/s (blocks whose share is a
    power of two of 8 KiB or more are the slow ones), so each probe runs at the best shape found.
    The workloads' fractions of the 8 TB/s peak are to be read against these."""
    import numpy as np
    import tensorcomprehensions_amd as tc
    out = {}
    for label, src, entry, shapes, opts, nbytes in STREAM_PROBES:
        ins = [to_device(np.ones(shape, dtype=np.float32)) for shape in shapes]
        ex = tc.compile(src, entry, ins, opts)
        outs = tc.prepare_outputs(src, entry, ins)
        spin(ex, ins, outs, SPIN_MS)
        us = sorted(tc.profile_repeated(ex, ins, outs, steps) / steps for _ in range(5))[2]
        out[label] = {"us_per_launch": round(us, 2), "bytes": nbytes, "gb_per_s": round(nbytes / us / 1e3, 1),
                      "kernel": ex.kernel_name(), "launch": ex.launch_bounds()}
        del ins, outs
    return out


def measured_traffic(name, options):
    """HBM bytes per launch from the committed counter summary of this workload, if there is one
    and it was taken under the options being timed."""
    short = {"c2_tensordot": "tensordot_c2", "c3_batch_matmul": "batch_matmul_c3",
             "c4_group_convolution": "group_convolution_c4", "c5_moments": "moments_c5"}.get(name)
    path = os.path.join(ROOT, "profiles", f"{short}_hbm_traffic.txt")
    if not short or not os.path.exists(path):
        return None
    lines = open(path).read().splitlines()
    if f"options: {options}" not in lines:
        return None
    for line in lines:
        if line.startswith("traffic_bytes_per_launch:"):
            return int(line.split(":")[1])
    return None


def with_floor(roof, kernel_us, floor_us):
    """A kernel of a few microseconds next to what an empty launch costs on this device:
    floor_us = a near-empty copy kernel launched the same way, above_floor_us = the kernel's time
    minus that, frac_above_floor = the kernel's ideal time at the roofline / above_floor_us."""
    ideal_us = roof["frac"] * kernel_us
    above = kernel_us - floor_us
    roof["floor_us"] = round(floor_us, 3)
    roof["above_floor_us"] = round(above, 3)
    # (capped: a kernel whose time cannot be told from an empty launch's has hidden its work behind the launch)
    roof["frac_above_floor"] = round(min(1.0, ideal_us / above), 4) if above > 0 else 1.0
    return roof


def roofline(m):
    gbs = m["bytes"] / (m["kernel_ms"] * 1e-3) / 1e9
    tfl = m["flops"] / (m["kernel_ms"] * 1e-3) / 1e12
    if "group_convolution" in m["name"]:
        return {"bound": "mfma", "achieved": round(tfl, 3), "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tfl / FP32_PEAK_TFLOPS, 4), "traffic": measured_traffic(m["name"], m["options"])}
    return {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": measured_traffic(m["name"], m["options"])}


def cpu_baseline(name, nbytes, budget_s=15.0):
    """The oracle's sequential loop nest (-O3 -march=native, one core) on the same inputs."""
    from oracle import tc_oracle
    from tests import workloads as W
    src, entry, _, _, _ = W.CONFIGS[name]
    ins = W.make_inputs(name)
    tc_oracle.run(src, entry, ins, native=True)          # build + first touch
    times = []
    t_all = time.perf_counter()
    while len(times) < 5 and time.perf_counter() - t_all < budget_s:
        t0 = time.perf_counter()
        tc_oracle.run(src, entry, ins, native=True)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"full {name} workload, median of {len(times)} runs of the sequential loop nest, {med * 1e3:.1f} ms each"}


def aten_cpu_baseline(name, nbytes, budget_s=10.0):
    """aten_cpu_baseline_here in a child process (PyTorch stays out of the measuring process)."""
    import subprocess
    code = (f"import json, sys; sys.path.insert(0, {ROOT!r}); import bench; "
            f"print('ATEN_JSON' + json.dumps(bench.aten_cpu_baseline_here({name!r}, {nbytes}, {budget_s})))")
    try:
        out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=budget_s * 6 + 120)
        for text in out.stdout.splitlines():
            if text.startswith("ATEN_JSON"):
                return json.loads(text[len("ATEN_JSON"):])
    except subprocess.TimeoutExpired:
        pass
    return None


def aten_cpu_baseline_here(name, nbytes, budget_s=10.0):
    """The library routine the reference's own benchmarks compare with (at::einsum / bmm / conv2d / mean, var)
    on the host cores with torch's default intra-op threads; None for workloads without one."""
    import torch
    from tests import workloads as W
    ins = [torch.from_numpy(a) for a in W.make_inputs(name)]
    fn = {
        "c1_tensordot_small": lambda: torch.einsum("nachw,ncbhw->nabhw", ins[0], ins[1]),
        "c2_tensordot": lambda: torch.einsum("nachw,ncbhw->nabhw", ins[0], ins[1]),
        "c3_batch_matmul": lambda: torch.bmm(ins[0], ins[1]),
        "c4_group_convolution": lambda: torch.nn.functional.conv2d(
            ins[0].reshape(32, 512, 16, 16), ins[1].reshape(512, 16, 3, 3), ins[2].reshape(512), groups=32),
        "c5_moments": lambda: (ins[0].mean(1), ins[0].var(1, unbiased=False)),
    }.get(name)
    if fn is None:
        return None
    fn()
    times = []
    t_all = time.perf_counter()
    while len(times) < 5 and time.perf_counter() - t_all < budget_s:
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "threads": torch.get_num_threads(),
            "sample": f"ATen CPU routine on the full {name} workload, median of {len(times)} runs, {med * 1e3:.1f} ms each"}


def suite_library_routines():
    """What the reference's benchmark programs time next to each TC: the ATen routine(s), here on
    the same GPU through PyTorch (eager, one launch per operator)."""
    import torch
    import torch.nn.functional as F
    return {
        "tmm": lambda a, b: a @ b.t(),
        "half_tmm": lambda a, b: a @ b.t(),
        "half_matmul": lambda a, b: a @ b,
        "matmul": lambda a, b: a @ b,
        "convolution": lambda i, w, b: F.conv2d(i, w, b),
        "group_convolution": lambda i, w, b: F.conv2d(
            i.reshape(i.shape[0], -1, i.shape[3], i.shape[4]), w.reshape(-1, *w.shape[2:]), b.reshape(-1), groups=i.shape[1]),
        "2fcrelu": lambda i, w1, b1, w2, b2: F.relu(F.linear(F.relu(F.linear(i, w1, b1)), w2, b2)),
        "mlp1": lambda i, w1, b1: F.relu(i @ w1 + b1),
        "mlp3": lambda i, w2, b2, w3, b3, w4, b4: F.relu(F.linear(F.relu(F.linear(F.relu(F.linear(i, w2, b2)), w3, b3)), w4, b4)),
        "c3": lambda a, b: a @ b.t(),
        "lut": lambda t, i: t[i.long()].sum(1),
        "2lut": lambda t1, i1, t2, i2: (t1[i1.long()].sum(1), t2[i2.long()].sum(1)),
        "group_normalization": lambda i, g, b, mean, var: (
            g[None, :, :, None, None] * (i - mean[:, :, None, None, None]) * torch.rsqrt(var[:, :, None, None, None] + 1e-5)
            + b[None, :, :, None, None]),
        "moments2": lambda x: (x.mean(1), x.var(1, unbiased=False)),
        "sum": lambda x: x.sum(1),
        "mean": lambda x: x.mean(1),
        "sum_squares": lambda x: (x * x).sum(1),
        "var": lambda x, mean: (x * x).mean(1) - mean * mean,
        "sum_and_squares": lambda x: (x.sum(1), (x * x).sum(1)),
        "kronecker3_1": lambda w2, x: torch.einsum("mabc,kc->mabk", x, w2),
        "kronecker3_2": lambda w1, x: torch.einsum("mabk,jb->majk", x, w1),
        "kronecker3_3": lambda w0, x: torch.einsum("majk,ia->mijk", x, w0),
        "group_normalization_single_kernel": lambda i, g, b: F.group_norm(
            i.reshape(i.shape[0], -1, i.shape[3], i.shape[4]), i.shape[1], g.reshape(-1), b.reshape(-1), 1e-5),
        "kronecker3": lambda w0, w1, w2, x: torch.einsum("mabc,ia,jb,kc->mijk", x, w0, w1, w2),
    }


def measure_suite(steps, warmup, only=()):
    """Kernel time of every comprehension of tests/benchmark_tcs.py:REFERENCE_SIZES under its tuned
    options (sum over its kernels, HIP events around `steps` back-to-back runs), the bytes of all
    its inputs and outputs counted once (look-up tables: the gathered rows), and the library time."""
    import torch
    import tensorcomprehensions_amd as tc
    from tests import benchmark_tcs as B
    routines = suite_library_routines()
    out = {}
    cases = [(name, name, options, None) for name, options in B.TUNED_AT_REFERENCE_SIZES.items()]
    cases += [(name, case, options, k) for name, (case, _, options, k) in B.LARGE_CONTRACTIONS.items()]
    cases += [(name, case, options, 0) for name, (case, _, options, _k) in B.OTHER_REFERENCE_SIZES.items()]
    unknown = set(only) - {c[0] for c in cases}
    if unknown:
        sys.exit(f"--suite-cases: unknown comprehension(s) {sorted(unknown)}")
    for name, case, options, k in cases:
        if only and name not in only:
            continue
        src, entry, _, _ = B.CASES[case]
        arrays = B.make_inputs(name, reference_sizes=True) if name in B.REFERENCE_SIZES else B.make_large_inputs(name)
        ins = [torch.from_numpy(a).cuda() for a in arrays]
        ex = tc.compile(src, entry, ins, options)
        outs = tc.prepare_outputs(src, entry, ins)
        spin(ex, ins, outs, SPIN_MS / 3)
        for _ in range(warmup):
            tc.unchecked_run(ex, ins, outs)
        us = tc.profile_repeated(ex, ins, outs, steps) / steps
        nbytes = sum(t.numel() * t.element_size() for t in ins + outs)
        if name in ("lut", "2lut"):
            for table, index in zip(ins[0::2], ins[1::2]):
                nbytes += (index.numel() * table.shape[1] - table.numel()) * 4
        entry_out = {"kernel_us": round(us, 2), "kernels": ex.num_kernels, "bytes": nbytes,
                     "gb_per_s": round(nbytes / us / 1e3, 1),
                     "launch": [ex.launch_bounds(k) for k in range(ex.num_kernels)]}
        if k:
            # a contraction's matrix-core roofline: 2 flops per multiply-add over the 157.3 TFLOP/s fp32 peak
            flops = 2.0 * outs[0].numel() * k
            entry_out["tflops"] = round(flops / us * 1e-6, 1)
            if name.startswith("half_"):
                entry_out["frac_of_fp16_matrix_peak"] = round(flops / us * 1e-6 / FP16_PEAK_TFLOPS, 3)
            else:
                entry_out["frac_of_fp32_matrix_peak"] = round(flops / us * 1e-6 / FP32_PEAK_TFLOPS, 3)
        fn = routines.get(case)
        if fn is not None:
            for _ in range(warmup):
                fn(*ins)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                fn(*ins)
            e1.record()
            torch.cuda.synchronize()
            entry_out["library_us"] = round(e0.elapsed_time(e1) * 1e3 / steps, 2)
        out[name] = entry_out
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (defaults: the reference's benchmark protocol, benchmark_iterations / benchmark_warmup of
    # tc/core/flags.cc:59-66, overridable like its other flags from the environment)
    ap.add_argument("--steps", type=int, default=int(os.environ.get("TC_BENCHMARK_ITERATIONS", 100)))
    ap.add_argument("--warmup", type=int, default=int(os.environ.get("TC_BENCHMARK_WARMUP", 10)))
    ap.add_argument("--config", default="c2_tensordot")
    ap.add_argument("--options", default=None)
    ap.add_argument("--all", action="store_true", help="(kept for old command lines: the other workloads are always measured)")
    ap.add_argument("--only", action="store_true", help="measure the selected workload alone (profiling runs)")
    ap.add_argument("--spin-ms", type=float, default=SPIN_MS,
                    help="back-to-back launches for this long before the warm-up steps (device clocks)")
    ap.add_argument("--tune", default=None, metavar="GENERATIONSxPOPULATION",
                    help="autotune the workload from the naive options first (e.g. 5x40) and measure the best")
    ap.add_argument("--tune-base", default="naive", choices=["naive", "stored"],
                    help="base mapping of --tune: the naive options, or the base mapping of tests/workloads.py")
    ap.add_argument("--save-cache", action="store_true",
                    help="--tune reads and extends the committed options cache (tensorcomprehensions_amd/tuned/)")
    ap.add_argument("--tune-settings", default="", metavar="KEY=VALUE;...",
                    help="further tuner settings for --tune (seed_heuristics=0, refinement_rounds=0, seed=3, ...)")
    ap.add_argument("--suite", action="store_true",
                    help="also time the reference's other benchmark comprehensions at their default sizes")
    ap.add_argument("--suite-cases", default="", metavar="NAME,...",
                    help="restrict --suite to these comprehensions (profiling runs)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--floor", action="store_true",
                    help="also time near-empty copy kernels of 1, 64 and 500 blocks (the cost of a launch)")
    ap.add_argument("--stream", action="store_true",
                    help="also time kernels that only move data (copy, four reads to one write, reads alone)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain copy kernel of known size (reference point for HBM byte counters)")
    a = ap.parse_args()
    globals()["SPIN_MS"] = a.spin_ms
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this backend has no multi-GPU path (run with --gpus 1)")
    if a.suite:
        import torch  # noqa: F401  (first, so that the whole process runs on PyTorch's HIP runtime)
    import tensorcomprehensions_amd as tc
    from tests import workloads as W

    if a.calibrate:
        calibrate_copy(a.steps)
    tuned_in = None
    if a.tune:
        gens, pop = (int(x) for x in a.tune.lower().split("x"))
        src, entry = W.CONFIGS[a.config][0], W.CONFIGS[a.config][1]
        ins = [to_device(x) for x in W.make_inputs(a.config)]
        t0 = time.perf_counter()
        settings = {"generations": gens, "pop_size": pop, "threads": 16, "seed": 1, "top_k": 1}
        if a.save_cache:
            os.makedirs(os.path.dirname(OPTIONS_CACHE), exist_ok=True)
            settings["cache_file"] = OPTIONS_CACHE
        settings.update(kv.split("=", 1) for kv in a.tune_settings.split(";") if kv)
        best = tc.autotune(src, entry, ins, "naive" if a.tune_base == "naive" else W.TUNED[a.config], **settings)
        tuned_in = time.perf_counter() - t0
        if not best:
            sys.exit("the autotuner found no runnable candidate")
        a.options = best[0].to_text()
        del ins
    m = measure(a.config, a.steps, a.warmup, a.options)
    value = m["bytes"] * a.steps / m["wall_s"] / 1e9
    line = {
        "metric": "per-TC kernel GB/s or TFLOP/s on 1 MI355X and % of roofline",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(m["wall_s"] * 1e3 / a.steps, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": a.config, "shapes": [list(s) for s in W.CONFIGS[a.config][2]],
                   "options": m["options"], "launch": m["launch"], "algorithmic_bytes": m["bytes"]},
        "roofline": roofline(m),
        "device": tc.device_name(),
    }
    line["config"]["options_from"] = m["options_from"]
    if tuned_in is not None:
        line["config"]["options_from"] = (f"autotuned from the {a.tune_base} options, {a.tune} candidates, {tuned_in:.0f} s"
                                          + (f", {a.tune_settings}" if a.tune_settings else ""))
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(a.config, m["bytes"])
        line["cpu_baseline"]["host_cores"] = os.cpu_count()
        line["cpu_baseline"]["aten"] = aten_cpu_baseline(a.config, m["bytes"])
    # what a launch costs whatever the kernel does: part of every line, the workloads of a few
    # microseconds are read against it (--floor adds the one-wavefront and 64-block shapes)
    floor = launch_floor(max(a.steps, MIN_BURST), all_shapes=a.floor)
    line["launch_floor"] = floor
    floor_us = floor["copy_500_blocks_of_256"]["us_per_launch"]
    if not a.only:
        others = {}
        for name in W.CONFIGS:
            if name == a.config:
                continue
            o = measure(name, a.steps, a.warmup, bursts=7)
            roof = roofline(o)
            if o["kernel_ms"] * 1e3 < 4 * floor_us:
                roof = with_floor(roof, o["kernel_ms"] * 1e3, floor_us)
            others[name] = {"kernel_us": round(o["kernel_ms"] * 1e3, 3), "roofline": roof,
                            "gflops": round(o["flops"] / (o["kernel_ms"] * 1e-3) / 1e9, 1), "launch": o["launch"],
                            "options": o["options"], "options_from": o["options_from"]}
        line["others"] = others
    if a.stream:
        line["stream_probes"] = stream_probes(a.steps)
    if a.suite:
        line["suite"] = measure_suite(a.steps, a.warmup, [n for n in a.suite_cases.split(",") if n])
    print(json.dumps(line))


if __name__ == "__main__":
    main()
