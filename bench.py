#!/usr/bin/env python3
"""Benchmark of the sarek-hip hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-also]

Prints ONE JSON line.  A "step" is one pass of the workload's hot-path entry point over
one batch of synthetic input that is already resident in HBM.  The headline workload is
the bf16-in / f32-accumulate 8192^3 GEMM; the other configurations of the hot path
(fused triad+sum n=2^28, f32 GEMM 8192^3 and 1024^3, fp16 fused-epilogue GEMM) are
measured the same way and reported under "also", each with its own roofline object.

Timing mirrors the reference's benches (warmup, then timed iterations with the device
synchronised; benchmarks/bench_stream_triad.ml:76-116) with one difference: the K timed
steps are bracketed by one synchronise on each side, and the kernel time used for the
roofline comes from HIP events recorded on the launch stream.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
# MI355X peak engine clock: the published MFMA peaks are quoted at this clock
NOMINAL_CLOCK_MHZ = 2400.0
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch,
# FETCH_SIZE scaled by 2.0 and WRITE_SIZE by 1.0 after calibration against a plain 1 GiB copy).
MEASURED_TRAFFIC_BYTES = {
    "triad_sum_2p28": (1048600 * 2 + 1050630) * 1024,
    "gemm_bf16_8192": (793626 * 2 + 262153) * 1024,
    "gemm_f32_8192": (1695900 * 2 + 262153) * 1024,
    "gemm_f16_epilogue": (306687 * 2 + 176779) * 1024,
    "histogram_2p28": (524312 * 2 + 256) * 1024,
    "radix_scatter_5e7": (97880 * 2 + 215611) * 1024,
}
PEAK_MFMA_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="gemm_bf16_8192",
                    choices=["gemm_bf16_8192", "triad_sum_2p28", "gemm_f32_8192", "gemm_f32_1024",
                             "gemm_f16_epilogue", "copy_1gib", "vendor_gemm_bf16_8192", "histogram_2p28",
                             "radix_scatter_5e7"])
    ap.add_argument("--no-also", action="store_true", help="measure only the headline workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    return ap.parse_args()


class Events:
    """HIP events of the library, recorded on the stream the kernels are launched on."""

    def __init__(self, hip, stream):
        self.hip, self.stream = hip, stream
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        hip.check(hip.lib.sarek_hip_event_create(C.byref(self.e0)))
        hip.check(hip.lib.sarek_hip_event_create(C.byref(self.e1)))

    def start(self):
        self.hip.check(self.hip.lib.sarek_hip_event_record(self.e0, self.stream))

    def stop_ms(self):
        self.hip.check(self.hip.lib.sarek_hip_event_record(self.e1, self.stream))
        self.hip.check(self.hip.lib.sarek_hip_event_synchronize(self.e1))
        ms = C.c_float(0)
        self.hip.check(self.hip.lib.sarek_hip_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return float(ms.value)


def make_workload(name, torch, hip):
    """Returns (step_fn, info) with inputs resident on the GPU."""
    g = torch.Generator(device="cuda")
    if name == "copy_1gib":
        # plain device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters
        n = 1 << 28
        src = torch.rand(n, device="cuda", generator=g)
        dst = torch.empty_like(src)
        info = dict(metric="plain copy GB/s (counter calibration)", unit="GB/s", dtype="f32",
                    work=8.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="at::native copy kernel",
                    config={"workload": "dst.copy_(src), 1 GiB read + 1 GiB written", "n": n})
        return (lambda: dst.copy_(src)), info
    if name == "triad_sum_2p28":
        n = 1 << 28
        g.manual_seed(0xB)
        b = torch.rand(n, device="cuda", generator=g)
        g.manual_seed(0xC)
        c = torch.rand(n, device="cuda", generator=g)
        a = torch.empty_like(b)
        ws = hip.triad_sum_workspace(n)
        info = dict(metric="fused triad+sum GB/s", unit="GB/s", dtype="f32",
                    work=12.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="triad_kernel<true, true> (+ fold_kernel, 1 % of the time)",
                    config={"workload": "fused stream triad + sum, a=b+3c, sum(a)", "n": n,
                            "algorithmic_bytes": 12 * n})
        return (lambda: hip.triad_sum(b, c, 3.0, out=a, workspace=ws)), info
    if name in ("gemm_f32_8192", "gemm_f32_1024"):
        s = 8192 if name.endswith("8192") else 1024
        g.manual_seed(0xA11CE)
        a = torch.rand(s, s, device="cuda", generator=g) * 2 - 1
        g.manual_seed(0xB0B)
        b = torch.rand(s, s, device="cuda", generator=g) * 2 - 1
        c = torch.empty(s, s, device="cuda")
        info = dict(metric=f"f32 GEMM {s}^3 TFLOP/s", unit="TFLOP/s", dtype="f32",
                    work=2.0 * s ** 3, work_unit=1e12, bound="mfma", peak=PEAK_MFMA_TFLOPS["f32"],
                    kernel="gemm_f32_dma_kernel",
                    config={"workload": f"f32 GEMM C=A.B row-major, U[-1,1)", "m": s, "n": s, "k": s})
        return (lambda: hip.gemm_f32(a, b, out=c)), info
    if name == "gemm_bf16_8192":
        s = 8192
        g.manual_seed(0xA4)
        a = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
        g.manual_seed(0xB4)
        b = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
        c = torch.empty(s, s, device="cuda")
        info = dict(metric="GEMM TFLOP/s at 8192^3 (bf16-in, f32-accumulate)", unit="TFLOP/s",
                    dtype="bf16", work=2.0 * s ** 3, work_unit=1e12, bound="mfma",
                    peak=PEAK_MFMA_TFLOPS["bf16"], kernel="gemm16_dma_kernel<bf16, store, 64, 32, 2, 4, 2>",
                    config={"workload": "bf16-in f32-acc GEMM C=A.B row-major, N(0,0.02)",
                            "m": s, "n": s, "k": s})
        return (lambda: hip.gemm_bf16(a, b, out=c)), info
    if name == "vendor_gemm_bf16_8192":
        # the vendor library's GEMM (torch.matmul -> hipBLASLt) on the headline inputs, for
        # side-by-side profiles; it writes bf16 C where the kernel here writes f32
        s = 8192
        g.manual_seed(0xA4)
        a = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
        g.manual_seed(0xB4)
        b = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
        c = torch.empty(s, s, device="cuda", dtype=torch.bfloat16)
        info = dict(metric="vendor library GEMM TFLOP/s at 8192^3 (bf16 in, bf16 out)", unit="TFLOP/s",
                    dtype="bf16", work=2.0 * s ** 3, work_unit=1e12, bound="mfma",
                    peak=PEAK_MFMA_TFLOPS["bf16"], kernel="hipBLASLt (torch.matmul)",
                    config={"workload": "torch.matmul bf16, N(0,0.02)", "m": s, "n": s, "k": s})
        return (lambda: torch.matmul(a, b, out=c)), info
    if name == "histogram_2p28":
        n = 1 << 28
        g.manual_seed(0xC4)
        keys = torch.randint(0, 256, (n,), device="cuda", generator=g, dtype=torch.int32)
        hist = torch.zeros(256, device="cuda", dtype=torch.int32)
        info = dict(metric="256-bin histogram of int32 keys GB/s", unit="GB/s", dtype="i32",
                    work=4.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="histogram_kernel<ModPow2Bin>",
                    config={"workload": "histogram[key mod 256] += 1, uniform keys", "n": n,
                            "algorithmic_bytes": 4 * n})
        return (lambda: hip.histogram(keys, hist, 256)), info
    if name == "radix_scatter_5e7":
        n = 50_000_000
        g.manual_seed(0xC5)
        keys = torch.randint(0, 100000, (n,), device="cuda", generator=g, dtype=torch.int32)
        hist = torch.zeros(256, device="cuda", dtype=torch.int32)
        hip.radix_histogram(keys, hist, 0, 255)
        starts = (torch.cumsum(hist, 0) - hist).to(torch.int32)
        out = torch.empty(n, device="cuda", dtype=torch.int32)
        counters = torch.empty(256, device="cuda", dtype=torch.int32)
        info = dict(metric="radix-sort scatter pass (8-bit digit) GB/s", unit="GB/s", dtype="i32",
                    work=8.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="radix_scatter_kernel<1024, 16> (+ a 1 KiB copy that resets the counters)",
                    config={"workload": "out[counters[key & 255]++] = key, random keys below 100000", "n": n,
                            "algorithmic_bytes": 8 * n})

        def step():
            counters.copy_(starts)
            hip.radix_scatter(keys, out, counters, 0, 255)
        return step, info
    if name == "gemm_f16_epilogue":
        m, n, k = 4095, 11008, 4096
        g.manual_seed(0xA5)
        a = (torch.randn(m, k, device="cuda", generator=g) * 0.02).half()
        g.manual_seed(0xB5)
        b = (torch.randn(k, n, device="cuda", generator=g) * 0.02).half()
        bias = torch.rand(n, device="cuda", generator=g) * 0.2 - 0.1
        y = torch.empty(m, n, device="cuda")
        rs = torch.empty(m, device="cuda")
        info = dict(metric="fp16 GEMM + bias + ReLU + row-sum TFLOP/s", unit="TFLOP/s", dtype="f16",
                    work=2.0 * m * n * k, work_unit=1e12, bound="mfma",
                    peak=PEAK_MFMA_TFLOPS["f16"], kernel="gemm16_dma_kernel<f16, bias_relu_rowsum, 64, 32, 2, 4, 2>",
                    config={"workload": "fp16-in f32-acc Y=relu(A.B+bias), rowsum(Y)",
                            "m": m, "n": n, "k": k})
        return (lambda: hip.gemm_f16_bias_relu_rowsum(a, b, bias, out=y, rowsum=rs)), info
    raise ValueError(name)


def measure(name, torch, hip, steps, warmup):
    step, info = make_workload(name, torch, hip)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev = Events(hip, stream)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev.start()
    for _ in range(steps):
        step()
    gpu_ms = ev.stop_ms()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    # roofline: average launch duration from the HIP events around the timed region (the
    # launches run back to back there, as in a rocprofv3 kernel trace of this command);
    # for reference also the median of launches timed one at a time with a sync between
    # them, which run cooler and, under a power cap, faster
    kernel_ms = gpu_ms / steps
    per = []
    for _ in range(min(steps, 20)):
        ev.start()
        step()
        per.append(ev.stop_ms())
    per.sort()
    isolated_ms = per[len(per) // 2]
    ms_per_step = wall_ms / steps
    value = info["work"] / (ms_per_step * 1e-3) / info["work_unit"]
    achieved = info["work"] / (kernel_ms * 1e-3) / info["work_unit"]
    res = {
        "metric": info["metric"], "value": round(value, 2), "unit": info["unit"],
        "ms_per_step": round(ms_per_step, 5), "gpu_ms_per_step_events": round(gpu_ms / steps, 5),
        "dtype": info["dtype"], "config": info["config"],
        "roofline": {"bound": info["bound"], "achieved": round(achieved, 2), "peak": info["peak"],
                     "unit": "GB/s" if info["bound"] == "hbm" else "TFLOP/s",
                     "frac": round(achieved / info["peak"], 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(name),
                     "kernel": info["kernel"], "kernel_ms": round(kernel_ms, 5),
                     "isolated_launch_ms": round(isolated_ms, 5)},
    }
    if name == "triad_sum_2p28":
        res["roofline"]["probe_kernels_GBs"] = hbm_ceiling(torch, hip)
    if info["bound"] == "mfma":
        # shader clock the kernel actually ran at (in-kernel cycle counter against the
        # constant-rate wall clock), and the rate of those very launches against the peak
        # scaled to that clock
        with hip.clock_probe() as probe:
            pairs = []
            for _ in range(min(steps, 10)):
                probe.buf.zero_()
                ev.start()
                step()
                ms = ev.stop_ms()
                mhz = probe.mhz()
                if mhz:
                    pairs.append((ms, mhz))
        if pairs:
            pairs.sort()
            ms, mhz = pairs[len(pairs) // 2]
            res["roofline"]["shader_clock_mhz"] = round(mhz, 1)
            res["roofline"]["frac_of_peak_at_that_clock"] = round(
                info["work"] / (ms * 1e-3) / info["work_unit"] / (info["peak"] * mhz / NOMINAL_CLOCK_MHZ), 4)
    return res


HBM_PROBE_SRC = r"""
typedef float f4 __attribute__((ext_vector_type(4)));
#define LOADS(dst, src) _Pragma("unroll") for (int u = 0; u < 4; ++u) dst[u] = __builtin_nontemporal_load(src + base + u * 256)
extern "C" __global__ __launch_bounds__(256) void probe_read(const f4* r0, int n0, float* sink, int ns) {
  const long base = (long)blockIdx.x * 1024 + threadIdx.x;
  f4 v[4];
  LOADS(v, r0);
  const f4 s = v[0] + v[1] + v[2] + v[3];
  if (s.x + s.y + s.z + s.w == 12345.678f) sink[0] = 1.f;
}
extern "C" __global__ __launch_bounds__(256) void probe_write(f4* w, int nw) {
  const long base = (long)blockIdx.x * 1024 + threadIdx.x;
  const f4 v = {1.f, 2.f, 3.f, 4.f};
  _Pragma("unroll") for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(v, w + base + u * 256);
}
extern "C" __global__ __launch_bounds__(256) void probe_2r1w(f4* w, int nw, const f4* r0, int n0, const f4* r1, int n1) {
  const long base = (long)blockIdx.x * 1024 + threadIdx.x;
  f4 v[4], c[4];
  LOADS(v, r0);
  LOADS(c, r1);
  _Pragma("unroll") for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(v[u] + c[u], w + base + u * 256);
}
"""


def hbm_ceiling(torch, hip, n=1 << 28):
    """What this GPU's HBM delivers to the simplest kernels of three traffic shapes (one
    workgroup per 4096 floats, 128-bit non-temporal accesses), JIT-compiled through the
    plugin path: context for the triad's fraction of the nominal 8 TB/s."""
    a = torch.empty(n, device="cuda")
    b = torch.rand(n, device="cuda")
    c = torch.rand(n, device="cuda")
    sink = torch.zeros(1, device="cuda")
    grid = (n // 4096, 1, 1)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev = Events(hip, stream)
    out = {}
    for key, kern, items, nbytes in [
            ("read_only", "probe_read", [b, sink], 4 * n),
            ("write_only", "probe_write", [a], 4 * n),
            ("two_reads_one_write", "probe_2r1w", [a, b, c], 12 * n)]:
        times = []
        for i in range(12):
            ev.start()
            hip.run_source(HBM_PROBE_SRC, kern, (256, 1, 1), grid, items)
            ms = ev.stop_ms()
            if i >= 2:
                times.append(ms)
        times.sort()
        out[key] = round(nbytes / (times[len(times) // 2] * 1e-3) / 1e9, 1)
    return out


def cpu_baseline(name):
    """The CPU oracle (a C restatement of the reference's Native backend arithmetic) timed
    on this host's cores on a bounded sample of the same workload."""
    import numpy as np

    import oracle
    cores = os.cpu_count() or 1
    cores = min(cores, 16) if "GRAFT_REPO_ROOT" in os.environ else cores
    rng = np.random.default_rng(0)
    if name == "triad_sum_2p28":
        n = 1 << 28
        b = rng.random(n, dtype=np.float32)
        c = rng.random(n, dtype=np.float32)
        oracle.triad_sum(b[:1 << 20], c[:1 << 20], 3.0, threads=cores)
        passes = 40
        t0 = time.perf_counter()
        for _ in range(passes):
            oracle.triad_sum(b, c, 3.0, threads=cores)
        dt = (time.perf_counter() - t0) / passes
        return {"value": round(12.0 * n / dt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": f"the full n=2^28 workload (triad, block-256 tree sum, double fold), "
                          f"mean of {passes} passes, {dt * passes:.1f} s in total"}
    if name == "gemm_f16_epilogue":
        rows, n, k = 4095, 11008, 4096
    elif name == "gemm_f32_1024":
        rows, n, k = 1024, 1024, 1024
    else:
        rows, n, k = 4096, 8192, 8192
    a = rng.normal(0, 0.02, (rows, k)).astype(np.float32)
    b = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    idx = np.arange(rows, dtype=np.int32)
    oracle.gemm_rows(a[:8], b, idx[:8], threads=cores)
    t0 = time.perf_counter()
    oracle.gemm_rows(a, b, idx, threads=cores)
    dt = time.perf_counter() - t0
    return {"value": round(2.0 * rows * n * k / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores,
            "kind": "port",
            "sample": f"{rows} of the output rows (n={n}, k={k}), double accumulation in k order, {dt:.2f} s"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from spoc_amd import hip
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    head = measure(args.workload, torch, hip, args.steps, args.warmup)
    out = {
        "metric": head["metric"], "value": head["value"], "unit": head["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic", "config": head["config"], "roofline": head["roofline"],
        "gpu_ms_per_step_events": head["gpu_ms_per_step_events"],
    }
    if not args.no_cpu_baseline and args.workload not in ("copy_1gib", "vendor_gemm_bf16_8192"):
        out["cpu_baseline"] = cpu_baseline(args.workload)
    if not args.no_also:
        also = []
        for name in ["triad_sum_2p28", "gemm_f32_8192", "gemm_f16_epilogue", "gemm_f32_1024",
                     "gemm_bf16_8192", "histogram_2p28", "radix_scatter_5e7"]:
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            r = measure(name, torch, hip, args.steps, args.warmup)
            if not args.no_cpu_baseline and name == "triad_sum_2p28":
                r["cpu_baseline"] = cpu_baseline(name)
            also.append(r)
        out["also"] = also
    info = hip.device_info(0)
    out["device"] = {"name": info.name.decode(), "arch": info.gcn_arch.decode(),
                     "cus": info.multiprocessor_count, "clock_mhz": info.clock_rate_khz // 1000}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
