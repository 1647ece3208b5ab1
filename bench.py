#!/usr/bin/env python3
"""Benchmark of the sarek-hip hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--warmup-ms T] [--workload NAME] [--no-also]

Prints ONE JSON line.  A "step" is one pass of the workload's hot-path entry point over
one batch of synthetic input that is already resident in HBM.  The headline workload is
the bf16-in / f32-accumulate 8192^3 GEMM; the other configurations of the hot path
(fused triad+sum n=2^28, f32 GEMM 8192^3 and 1024^3, fp16 fused-epilogue GEMM) are
measured the same way and reported under "also", each with its own roofline object.

Every workload goes through the plugin boundary the way a Sarek program reaches it: the
reference benches' own kernels from their IR through Execute.run_vectors / run_pipeline, the
16-bit GEMMs and the fused epilogue as library kernel texts through Execute.run_source; the
record's "served_by" names the hand-written kernel that took the launch.

Timing mirrors the reference's benches (warmup, then timed iterations, each launched and
waited for; benchmarks/bench_stream_triad.ml:76-116): ms_per_step is the wall time of the K
timed iterations over K, ms_per_step_stats their min / median / avg / max.  The kernel time
used for the roofline comes from HIP events recorded round the dominant launch on the launch
stream, in a second round of K steps right after the timed ones (so that the handling of the events
is not part of ms_per_step); gpu_ms_per_step_back_to_back is the same step launched K times with one
wait at the end.
The warmup is W steps and at least --warmup-ms (60 ms) of them: after a pause the clocks of a
power-limited kernel need 30-40 ms of load to settle (--trace-launches shows the curve).
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
    "triad_sum_2p28": (1048600 * 2 + 1052680) * 1024,
    "map_sum_2p28": (1048590 * 2 + 1052710) * 1024,
    "gemm_bf16_8192": (788983 * 2 + 262171) * 1024,
    "gemm_f32_8192": (1572990 * 2 + 262144) * 1024,
    "gemm_f32_1024": (12345 * 2 + 4096) * 1024,
    "gemm_bf16_2048": (24690 * 2 + 16386) * 1024,
    "gemm_f16_epilogue": (287017 * 2 + 176780) * 1024,
    "histogram_2p28": (522398 * 2 + 256) * 1024,
    "radix_scatter_5e7": (97857 * 2 + 215917) * 1024,
}
PEAK_MFMA_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="gemm_bf16_8192",
                    choices=["gemm_bf16_8192", "gemm_f16_8192", "triad_sum_2p28", "gemm_f32_8192", "gemm_f32_1024",
                             "gemm_f16_epilogue", "gemm_f16_4095x11008x4096", "gemm_f16_shape", "gemm_bf16_shape", "gemm_bf16_2048", "gemm_f32_shape", "vendor_gemm_f32_shape", "copy_1gib",
                             "vendor_gemm_bf16_8192", "vendor_gemm_bf16_shape", "histogram_2p28",
                             "radix_scatter_5e7", "stencil_2d_shape", "conv2d_shape", "map_sum_2p28", "mfma_bf16_stream", "mfma_bf16_stream_32x32x16",
                             "l2_to_lds_stream", "radix_scatter_chain_probe", "triad_shape_probe", "fold_partials"])
    ap.add_argument("--fold", default="1048576,0", metavar="PARTIALS,TAKE_STAGES",
                    help="fold_partials: how many float32 partials, and 1 to give the library's sixteen fold stages "
                         "to other streams first, so that the measured fold runs without one")
    ap.add_argument("--warmup-ms", type=float, default=60.0,
                    help="warm up for at least this long (and at least --warmup steps): the clocks of a power-limited "
                         "kernel take 30-40 ms to settle after a pause")
    ap.add_argument("--trace-launches", action="store_true",
                    help="add the timed launches' kernel durations in launch order (kernel_us_by_launch)")
    ap.add_argument("--no-also", action="store_true", help="measure only the headline workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--shape", default="4096,11264,4096", metavar="M,N,K",
                    help="shape of the *_shape workloads (stencil_2d_shape, conv2d_shape: width,height,ignored)")
    ap.add_argument("--l2-stream", default="", metavar="WORKGROUPS,WINDOW_MIB",
                    help="shape of the l2_to_lds_stream workload (default 1024,2)")
    ap.add_argument("--triad-shape", default="256,4,0", metavar="THREADS,FLOAT4_PER_THREAD,PHASES",
                    help="triad_shape_probe: workgroup size, 128-bit pieces per thread and input, and whether a barrier "
                         "separates the workgroup's loads from its stores (1) or not (0)")
    ap.add_argument("--chain", default="0,1", metavar="PREDECESSORS,ROUNDS",
                    help="radix_scatter_chain_probe: status words of how many earlier tiles every tile reads, in how many "
                         "dependent rounds (0,1: no status traffic at all)")
    ap.add_argument("--zero-operands", action="store_true",
                    help="16-bit GEMM workloads: all-zero A and B (what the kernel does when the data costs no power)")
    ap.add_argument("--tunable", action="append", default=[], metavar="NAME=VALUE",
                    help="sarek_hip_set_tunable(NAME, VALUE) before measuring (kernel shape knobs; the measurement knobs "
                         "gemm16.ablate / ring / tj / mfma need --measure-build)")
    ap.add_argument("--measure-build", action="store_true",
                    help="load libsarek_hip_measure.so (make -C spoc_amd/csrc measure): the product's code plus the kernel "
                         "variants of the ablation studies, some of which compute wrong results on purpose")
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


def device_vector(sarek, hip, torch, tensor, kind=None, elem_size=None):
    """A Vector whose device buffer holds `tensor` (data made on the device by torch): created, given
    its buffer by Transfer.to_device, then filled device to device.  Location Both, as after an
    upload; the launches below never read the host block."""
    V = sarek.Vector
    v = V.create_custom(elem_size, tensor.numel()) if elem_size else V.create(kind, tensor.numel())
    sarek.Transfer.to_device(v)
    hip.check(hip.lib.sarek_hip_memcpy_dtod(v.device_ptr, tensor.data_ptr(), tensor.numel() * tensor.element_size()))
    return v


class Launch:
    """One prepared call through the plugin boundary: the ctypes argument block is built once."""

    def __init__(self, hip, fn, *args):
        self.hip, self.fn, self.args = hip, fn, args

    def __call__(self):
        rc = self.fn(*self.args)
        if rc != 0:
            self.hip.check(rc)


def dims(*d):
    return (C.c_int * 3)(*d)


ZERO_OPERANDS = False
FOLD = (1 << 20, 0)
CHAIN = (0, 1)
TRIAD_SHAPE = (256, 4, 0)
GEMM_SHAPE = (4096, 11264, 4096)
L2_STREAM_SHAPE = None


def make_workload(name, torch, hip):
    """Returns (main, tail, info, keep): main() launches the workload's dominant kernel through the plugin
    route named in info["route"], tail() (or None) the rest of the step; inputs are resident on the GPU."""
    from spoc_amd import reference_kernels as rk
    from spoc_amd import sarek
    E, V = sarek.Execute, sarek.Vector
    sarek.Device.init()
    lib = hip.lib
    g = torch.Generator(device="cuda")
    if name == "copy_1gib":
        # plain device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters
        n = 1 << 28
        src = torch.rand(n, device="cuda", generator=g)
        dst = torch.empty_like(src)
        info = dict(metric="plain copy GB/s (counter calibration)", unit="GB/s", dtype="f32",
                    work=8.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="at::native copy kernel", route="torch",
                    config={"workload": "dst.copy_(src), 1 GiB read + 1 GiB written", "n": n})
        return (lambda: dst.copy_(src)), None, info, None
    if name == "triad_sum_2p28":
        n = 1 << 28
        g.manual_seed(0xB)
        b = torch.rand(n, device="cuda", generator=g)
        vb = device_vector(sarek, hip, torch, b, V.float32)
        g.manual_seed(0xC)
        b.uniform_(0, 1, generator=g)
        vc = device_vector(sarek, hip, torch, b, V.float32)
        del b
        va, vout = V.create(V.float32, n), V.create(V.float32, n // 256)
        sarek.Transfer.to_device(va)
        sarek.Transfer.to_device(vout)
        total = torch.zeros(1, dtype=torch.float64, device="cuda")
        a0, n0 = E._args([E.Vec(va), E.Vec(vb), E.Vec(vc), E.Float32(3.0), E.Int32(n)])
        a1, n1 = E._args([E.Vec(va), E.Vec(vout), E.Int32(n)])
        ir0, ir1 = rk.stream_triad().encode(), rk.tree(False).encode()
        stages = (hip.PipelineStage * 2)()
        stages[0].ir_text, stages[0].block, stages[0].grid, stages[0].args, stages[0].n_args = \
            ir0, dims(256, 1, 1), dims(n // 256, 1, 1), a0, n0
        stages[1].ir_text, stages[1].block, stages[1].grid, stages[1].args, stages[1].n_args = \
            ir1, dims(256, 1, 1), dims(n // 256, 1, 1), a1, n1
        main = Launch(hip, lib.sarek_hip_execute_run_pipeline, stages, 2, None)
        tail = Launch(hip, lib.sarek_hip_fold_partials_f64, vout.device_ptr, n // 256, total.data_ptr(), None)
        info = dict(metric="fused triad+sum GB/s", unit="GB/s", dtype="f32",
                    work=12.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="triad_kernel<SUM_BLOCK256, nt> (then the fold of the 2^20 block sums: fold_onepass_kernel)",
                    route="Execute.run_pipeline [stream_triad IR; block-256 reduction IR], then sarek_hip_fold_partials_f64",
                    config={"workload": "fused stream triad + sum, a=b+3c, sum(a)", "n": n,
                            "algorithmic_bytes": 12 * n})
        return main, tail, info, (va, vb, vc, vout, total, a0, a1, ir0, ir1, stages)
    if name == "map_sum_2p28":
        # an element-wise kernel that is not one of the reference's benches (a = b - s * c), then the block-256 sum
        # of its output: recognised as a map, rebuilt from its own expression and fused with the sum
        n = 1 << 28
        g.manual_seed(0xB)
        b = torch.rand(n, device="cuda", generator=g)
        vb = device_vector(sarek, hip, torch, b, V.float32)
        g.manual_seed(0xC)
        b.uniform_(0, 1, generator=g)
        vc = device_vector(sarek, hip, torch, b, V.float32)
        del b
        va, vout = V.create(V.float32, n), V.create(V.float32, n // 256)
        sarek.Transfer.to_device(va)
        sarek.Transfer.to_device(vout)
        a0, n0 = E._args([E.Vec(va), E.Vec(vb), E.Vec(vc), E.Float32(3.0), E.Int32(n)])
        a1, n1 = E._args([E.Vec(va), E.Vec(vout), E.Int32(n)])
        ir0 = rk.stream_triad().replace("(add (read b", "(sub (read b").encode()
        ir1 = rk.tree(False).encode()
        stages = (hip.PipelineStage * 2)()
        stages[0].ir_text, stages[0].block, stages[0].grid, stages[0].args, stages[0].n_args = \
            ir0, dims(256, 1, 1), dims(n // 256, 1, 1), a0, n0
        stages[1].ir_text, stages[1].block, stages[1].grid, stages[1].args, stages[1].n_args = \
            ir1, dims(256, 1, 1), dims(n // 256, 1, 1), a1, n1
        main = Launch(hip, lib.sarek_hip_execute_run_pipeline, stages, 2, None)
        info = dict(metric="element-wise map + block-256 sum GB/s", unit="GB/s", dtype="f32",
                    work=12.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="sarek_map (the map's own expression in the stream kernels' shape, compiled at run time)",
                    route="Execute.run_pipeline [a = b - s c IR; block-256 reduction IR]",
                    config={"workload": "a = b - 3c, then the block-256 sums of a", "n": n,
                            "algorithmic_bytes": 12 * n})
        return main, None, info, (va, vb, vc, vout, a0, a1, ir0, ir1, stages)
    if name in ("gemm_f32_8192", "gemm_f32_1024"):
        s = 8192 if name.endswith("8192") else 1024
        g.manual_seed(0xA11CE)
        t = torch.rand(s, s, device="cuda", generator=g) * 2 - 1
        va = device_vector(sarek, hip, torch, t, V.float32)
        g.manual_seed(0xB0B)
        t = torch.rand(s, s, device="cuda", generator=g) * 2 - 1
        vb = device_vector(sarek, hip, torch, t, V.float32)
        del t
        vc = V.create(V.float32, s * s)
        sarek.Transfer.to_device(vc)
        a, n = E._args([E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(s), E.Int32(s), E.Int32(s)])
        ir = rk.matrix_mul_tiled().encode()
        main = Launch(hip, lib.sarek_hip_execute_run_vectors, ir, dims(16, 16, 1), dims(s // 16, s // 16, 1), 2048, a, n)
        info = dict(metric=f"f32 GEMM {s}^3 TFLOP/s", unit="TFLOP/s", dtype="f32",
                    work=2.0 * s ** 3, work_unit=1e12, bound="mfma", peak=PEAK_MFMA_TFLOPS["f32"],
                    kernel="gemm_f32_dma_kernel", route="Execute.run_vectors, matrix_mul_tiled IR (bench_matrix_mul_tiled.ml:55-95)",
                    config={"workload": "f32 GEMM C=A.B row-major, U[-1,1)", "m": s, "n": s, "k": s})
        return main, None, info, (va, vb, vc, a, ir)
    if name in ("gemm_bf16_8192", "gemm_f16_8192"):
        s = 8192
        bf16 = name == "gemm_bf16_8192"
        dt = torch.bfloat16 if bf16 else torch.float16
        g.manual_seed(0xA4)
        scale = 0.0 if ZERO_OPERANDS else 0.02
        t = (torch.randn(s, s, device="cuda", generator=g) * scale).to(dt)
        va = device_vector(sarek, hip, torch, t, elem_size=2)
        g.manual_seed(0xB4)
        t = (torch.randn(s, s, device="cuda", generator=g) * scale).to(dt)
        vb = device_vector(sarek, hip, torch, t, elem_size=2)
        del t
        vc = V.create(V.float32, s * s)
        sarek.Transfer.to_device(vc)
        lib_name = "gemm_bf16" if bf16 else "gemm_f16"
        src, entry = hip.library_kernel(lib_name)
        a, n = E._args([E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(s), E.Int32(s), E.Int32(s)])
        src_b, entry_b = src.encode(), entry.encode()
        main = Launch(hip, lib.sarek_hip_execute_run_source, src_b, hip.LANG_HIP, entry_b, dims(16, 16, 1),
                      dims(s // 16, s // 16, 1), 0, 1, a, n)
        tn = "bf16" if bf16 else "f16"
        info = dict(metric=f"GEMM TFLOP/s at 8192^3 ({tn}-in, f32-accumulate)", unit="TFLOP/s",
                    dtype=tn, work=2.0 * s ** 3, work_unit=1e12, bound="mfma",
                    peak=PEAK_MFMA_TFLOPS[tn], kernel=f"gemm16_m16_kernel<{tn}, store>",
                    route=f"Execute.run_source ~lang:HIP_Source, library kernel text '{lib_name}'",
                    config={"workload": f"{tn}-in f32-acc GEMM C=A.B row-major, N(0,0.02)",
                            "m": s, "n": s, "k": s})
        return main, None, info, (va, vb, vc, a, src_b, entry_b)
    if name in ("mfma_bf16_stream", "mfma_bf16_stream_32x32x16"):
        # The matrix pipes alone: the MFMA instructions of the 8192^3 product and nothing else (8 waves per CU,
        # N(0, 0.02)-like operands that stay in registers, no memory instruction in the loop), with the instruction
        # the GEMM kernel uses, v_mfma_f32_16x16x32_bf16 (32768 per wave), or with v_mfma_f32_32x32x16_bf16 (16384 per
        # wave).  What the package's power limit leaves of the published peak on such data.
        entry = "mfma_stream16" if name == "mfma_bf16_stream" else "mfma_stream"
        instr = "16x16x32" if name == "mfma_bf16_stream" else "32x32x16"
        out = torch.zeros(256 * 512, device="cuda")
        zero = 1 if ZERO_OPERANDS else 0
        items = [out, ("i32", 1024), ("i32", zero)]
        info = dict(metric="bf16 MFMA instruction stream TFLOP/s (no operand traffic)", unit="TFLOP/s", dtype="bf16",
                    work=256.0 * 8 * 1024 * 16 * 32768, work_unit=1e12, bound="mfma", peak=PEAK_MFMA_TFLOPS["bf16"],
                    kernel=f"{entry} (JIT)", route="Execute.run_source ~lang:HIP_Source, text in bench.py",
                    config={"workload": f"v_mfma_f32_{instr}_bf16 stream, 1.0995e12 flop over 2048 waves, register operands "
                                        + ("all zero" if zero else "N(0,0.02)-like")})
        return (lambda: hip.run_source(MFMA_STREAM_SRC, entry, (512, 1, 1), (256, 1, 1), items)), None, info, out
    if name == "l2_to_lds_stream":
        # The operand delivery of the 8192^3 16-bit GEMM and nothing else: 1024 workgroups of 8 waves each bring
        # 8 MiB (a 256 x 256 tile's A and B panels at K = 8192) into LDS with buffer_load_dwordx4 ... lds, 16 transfers
        # of 1 KiB in flight per wave, all from a 2 MiB window that the L2s hold: what the L2 -> LDS path delivers
        # when nothing else runs and nothing misses.  peak = 64 B per clock and CU at 2.4 GHz.
        src = torch.randint(0, 2 ** 31 - 1, ((16 << 20) // 4,), dtype=torch.int32, device="cuda", generator=g)
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        wgs, per_wg, window = 1024, 8 << 20, 2 << 20
        if L2_STREAM_SHAPE:       # --l2-stream WORKGROUPS,WINDOW_MIB (window a power of two, at most 16)
            wgs, window = L2_STREAM_SHAPE[0], L2_STREAM_SHAPE[1] << 20
        items = [src, sink, ("i32", per_wg // (512 * 16)), ("i32", (window // 16 - 1) & ~511), ("i32", (64 << 10) // 16)]
        info = dict(metric="L2 -> LDS transfer GB/s (no other work, every request an L2 hit)", unit="GB/s", dtype="u8",
                    work=float(wgs * per_wg), work_unit=1e9, bound="l2", peak=64.0 * 256 * NOMINAL_CLOCK_MHZ * 1e-3,
                    kernel="l2_to_lds (JIT)", route="Execute.run_source ~lang:HIP_Source, text in bench.py",
                    config={"workload": f"{wgs} workgroups x 8 MiB by buffer_load_dwordx4 ... lds from a {window >> 20} MiB window "
                                        "(the operand bytes of the 8192^3 16-bit GEMM with 256 x 256 tiles: 8.59 GB)"})
        return (lambda: hip.run_source(L2_STREAM_SRC, "l2_to_lds", (512, 1, 1), (wgs, 1, 1), items)), None, info, (src, sink)
    if name in ("gemm_f32_shape", "vendor_gemm_f32_shape"):
        # any --shape of the f32 GEMM through its C-ABI entry point (the IR route fixes 16 x 16 blocks that cover C), and
        # torch.matmul (no TF32) on the same inputs
        m, n, k = GEMM_SHAPE
        g.manual_seed(0xA11CE)
        a = torch.rand(m, k, device="cuda", generator=g) * 2 - 1
        g.manual_seed(0xB0B)
        b = torch.rand(k, n, device="cuda", generator=g) * 2 - 1
        c = torch.empty(m, n, device="cuda")
        vendor = name.startswith("vendor")
        info = dict(metric=("vendor library " if vendor else "") + f"f32 GEMM TFLOP/s at {m}x{n}x{k}", unit="TFLOP/s",
                    dtype="f32", work=2.0 * m * n * k, work_unit=1e12, bound="mfma", peak=PEAK_MFMA_TFLOPS["f32"],
                    kernel="hipBLASLt / rocBLAS (torch.matmul)" if vendor else "gemm_f32_dma_kernel",
                    route="torch.matmul" if vendor else "sarek_hip_gemm_f32 (C ABI)",
                    config={"workload": "f32 C=A.B row-major, U[-1,1)", "m": m, "n": n, "k": k,
                            "k_splits": 1 if vendor else hip.gemm_f32_k_splits(m, n, k)})
        if vendor:
            torch.backends.cuda.matmul.allow_tf32 = False
            return (lambda: torch.matmul(a, b, out=c)), None, info, None
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        main = Launch(hip, lib.sarek_hip_gemm_f32, C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()),
                      C.c_void_p(c.data_ptr()), m, n, k, stream)
        return main, None, info, (a, b, c)
    if name in ("vendor_gemm_bf16_8192", "vendor_gemm_bf16_shape"):
        # the vendor library's GEMM (torch.matmul -> hipBLASLt) on the headline inputs or on --shape, for
        # side-by-side profiles; it writes bf16 C where the kernel here writes f32
        m, n, k = (8192, 8192, 8192) if name == "vendor_gemm_bf16_8192" else GEMM_SHAPE
        g.manual_seed(0xA4)
        a = (torch.randn(m, k, device="cuda", generator=g) * 0.02).bfloat16()
        g.manual_seed(0xB4)
        b = (torch.randn(k, n, device="cuda", generator=g) * 0.02).bfloat16()
        c = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
        info = dict(metric=f"vendor library GEMM TFLOP/s at {m}x{n}x{k} (bf16 in, bf16 out)", unit="TFLOP/s",
                    dtype="bf16", work=2.0 * m * n * k, work_unit=1e12, bound="mfma",
                    peak=PEAK_MFMA_TFLOPS["bf16"], kernel="hipBLASLt (torch.matmul)", route="torch.matmul",
                    config={"workload": "torch.matmul bf16, N(0,0.02)", "m": m, "n": n, "k": k})
        return (lambda: torch.matmul(a, b, out=c)), None, info, None
    if name == "fold_partials":
        # the double fold of float32 partials (the host fold of bench_reduction.ml:154-160 kept on the device), with
        # one of the library's stages or, when other streams hold all sixteen, as one workgroup
        n, take = FOLD
        g.manual_seed(0xF0)
        parts = torch.rand(n, device="cuda", generator=g) * 4
        total = torch.zeros(1, dtype=torch.float64, device="cuda")
        held = []
        if take:
            seen = {}
            while len(seen) < 16:
                st = torch.cuda.Stream()
                seen[st.cuda_stream] = st
            small = torch.rand(1 << 17, device="cuda", generator=g)
            for st in seen.values():
                hip.check(lib.sarek_hip_fold_partials_f64(C.c_void_p(small.data_ptr()), small.numel(),
                                                          C.c_void_p(total.data_ptr()), C.c_void_p(st.cuda_stream)))
            torch.cuda.synchronize()
            held = [seen, small]
        main = Launch(hip, lib.sarek_hip_fold_partials_f64, C.c_void_p(parts.data_ptr()), n,
                      C.c_void_p(total.data_ptr()), C.c_void_p(torch.cuda.current_stream().cuda_stream))
        info = dict(metric="double fold of float32 partials GB/s", unit="GB/s", dtype="f64",
                    work=4.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="fold_pieces_kernel" if take else "fold_onepass_kernel",
                    route="sarek_hip_fold_partials_f64",
                    config={"workload": "sum of float32 partials in double, fixed order", "n": n,
                            "without_a_stage": bool(take), "algorithmic_bytes": 4 * n})
        return main, None, info, (parts, total, held)
    if name == "histogram_2p28":
        n = 1 << 28
        g.manual_seed(0xC4)
        t = torch.randint(0, 256, (n,), device="cuda", generator=g, dtype=torch.int32)
        vk = device_vector(sarek, hip, torch, t, V.int32)
        del t
        vh = V.create(V.int32, 256)
        vh.host[:] = 0
        sarek.Transfer.to_device(vh)
        a, na = E._args([E.Vec(vk), E.Vec(vh), E.Int32(n), E.Int32(256)])
        ir = rk.histogram().encode()
        main = Launch(hip, lib.sarek_hip_execute_run_vectors, ir, dims(256, 1, 1), dims(n // 256, 1, 1), 0, a, na)
        info = dict(metric="256-bin histogram of int32 keys GB/s", unit="GB/s", dtype="i32",
                    work=4.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="histogram_kernel<ModPow2Bin>", route="Execute.run_vectors, histogram IR (bench_histogram.ml:54-84)",
                    config={"workload": "histogram[key mod 256] += 1, uniform keys", "n": n,
                            "algorithmic_bytes": 4 * n})
        return main, None, info, (vk, vh, a, ir)
    if name in ("stencil_2d_shape", "conv2d_shape"):
        w, h = GEMM_SHAPE[0], GEMM_SHAPE[1]
        stencil = name[0] == "s"
        g.manual_seed(0xC6)
        t = torch.rand(w * h, device="cuda", generator=g) * 2 - 1
        vi = device_vector(sarek, hip, torch, t, V.float32)
        del t
        vo = V.create(V.float32, w * h)
        sarek.Transfer.to_device(vo)
        a, na = E._args([E.Vec(vi), E.Vec(vo), E.Int32(w), E.Int32(h)])
        if stencil:
            ir, block, grid = rk.stencil_2d().encode(), dims(16, 16, 1), dims((w + 15) // 16, (h + 15) // 16, 1)
        else:
            ir, block, grid = rk.conv2d().encode(), dims(256, 1, 1), dims((w * h + 255) // 256, 1, 1)
        main = Launch(hip, lib.sarek_hip_execute_run_vectors, ir, block, grid, 0, a, na)
        what = "five-point mean (bench_stencil_2d.ml:43-58)" if stencil else "3 x 3 box filter (bench_conv2d.ml:49-77)"
        info = dict(metric=("2-D five-point stencil" if stencil else "3 x 3 box filter") + " GB/s", unit="GB/s",
                    dtype="f64", work=8.0 * w * h, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="neighbourhood_kernel<%s>" % ("true" if not stencil else "false"),
                    route="Execute.run_vectors, " + what,
                    config={"workload": what + ", cells uniform[-1,1)", "width": w, "height": h,
                            "algorithmic_bytes": 8 * w * h})
        return main, None, info, (vi, vo, a, ir)
    if name == "radix_scatter_5e7":
        n = 50_000_000
        g.manual_seed(0xC5)
        keys = torch.randint(0, 100000, (n,), device="cuda", generator=g, dtype=torch.int32)
        hist = torch.zeros(256, device="cuda", dtype=torch.int32)
        hip.radix_histogram(keys, hist, 0, 255)
        starts = (torch.cumsum(hist, 0) - hist).to(torch.int32)
        vk = device_vector(sarek, hip, torch, keys, V.int32)
        del keys
        vo, vcnt = V.create(V.int32, n), V.create(V.int32, 256)
        sarek.Transfer.to_device(vo)
        sarek.Transfer.to_device(vcnt)
        a, na = E._args([E.Vec(vk), E.Vec(vo), E.Vec(vcnt), E.Int32(n), E.Int32(0), E.Int32(255)])
        ir = rk.radix_sort_scatter().encode()
        blocks = (n + 255) // 256
        reset = Launch(hip, lib.sarek_hip_memcpy_dtod, vcnt.device_ptr, starts.data_ptr(), 1024)
        scatter = Launch(hip, lib.sarek_hip_execute_run_vectors, ir, dims(256, 1, 1), dims(blocks, 1, 1), 0, a, na)

        def main():
            reset()
            scatter()
        info = dict(metric="radix-sort scatter pass (8-bit digit) GB/s", unit="GB/s", dtype="i32",
                    work=8.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="radix_scatter_kernel (+ a 1 KiB copy that resets the counters)",
                    route="Execute.run_vectors, radix-sort scatter IR (bench_radix_sort.ml:120-137)",
                    config={"workload": "out[counters[key & 255]++] = key, random keys below 100000", "n": n,
                            "algorithmic_bytes": 8 * n})
        return main, None, info, (vk, vo, vcnt, starts, a, ir)
    if name == "triad_shape_probe":
        # The plain triad (a = b + 3 c, the library kernel's arithmetic) in other launch shapes: THREADS x FLOAT4 pieces of
        # 16 bytes per workgroup and vector, all loads of a workgroup issued before its first store, optionally with a
        # barrier between the two phases so that a whole workgroup reads, then writes ("direction batching").
        threads, per_thread, phases = TRIAD_SHAPE
        n = 1 << 28
        b = torch.rand(n, device="cuda", generator=g)
        c = torch.rand(n, device="cuda", generator=g)
        a = torch.empty(n, device="cuda")
        src = TRIAD_SHAPE_SRC.replace("THREADS_N", str(threads)).replace("PIECES_N", str(per_thread)).replace("PHASES_N", str(phases))
        grid = n // 4 // (threads * per_thread)
        info = dict(metric="stream triad GB/s in a given launch shape", unit="GB/s", dtype="f32", work=12.0 * n, work_unit=1e9,
                    bound="hbm", peak=PEAK_HBM_GBS, kernel="triad_shape_probe (JIT)",
                    route="Execute.run_source ~lang:HIP_Source, text in bench.py",
                    config={"workload": f"a = b + 3c, {threads} threads x {per_thread} float4 per vector and workgroup"
                                        + (", loads | barrier | stores" if phases else ""), "n": n, "algorithmic_bytes": 12 * n})
        return (lambda: hip.run_source(src, "triad_shape_probe", (threads, 1, 1), (grid, 1, 1), [a, b, c])), None, info, (a, b, c)
    if name == "radix_scatter_chain_probe":
        # What a chained scan over the tiles (each tile publishes its 256 digit counts, later tiles add up what their
        # predecessors published) could cost at best in the scatter pass: the hand kernel's phases on 16384-key tiles with
        # the 256 returning atomics of a tile replaced by the scan's traffic alone -- 256 status words stored twice with
        # device scope, the words of CHAIN[0] earlier tiles loaded with device scope in CHAIN[1] dependent rounds -- and
        # no waiting for anybody (positions are wrong: timing only).  CHAIN = (0, 1): neither atomics nor status traffic.
        n = 3051 * 16384
        look, rounds = CHAIN
        g.manual_seed(0xC5)
        keys = torch.randint(0, 100000, (n,), device="cuda", generator=g, dtype=torch.int32)
        out = torch.empty_like(keys)
        counters = torch.zeros(256, device="cuda", dtype=torch.int32)
        status = torch.zeros(3051 * 256, device="cuda", dtype=torch.int32)
        src = SCATTER_CHAIN_SRC.replace("LOOK_N", str(look)).replace("ROUNDS_N", str(max(rounds, 1)))
        items = [out, keys, counters, status, ("i32", 0), ("i32", 255)]
        info = dict(metric="radix scatter pass with a chained scan's traffic in place of its atomics, GB/s (timing only)",
                    unit="GB/s", dtype="i32", work=8.0 * n, work_unit=1e9, bound="hbm", peak=PEAK_HBM_GBS,
                    kernel="scatter_chain_probe (JIT)", route="Execute.run_source ~lang:HIP_Source, text in bench.py",
                    config={"workload": f"16384-key tiles, every tile reads the status of {look} predecessors in {rounds} "
                                        "dependent rounds", "n": n, "algorithmic_bytes": 8 * n})
        return (lambda: hip.run_source(src, "scatter_chain_probe", (1024, 1, 1), (3051, 1, 1), items, shared_mem=65536)), \
            None, info, (keys, out, counters, status)
    if name in ("gemm_f16_4095x11008x4096", "gemm_f16_shape", "gemm_bf16_shape", "gemm_bf16_2048"):
        # the epilogue config's product without the epilogue (what the fused chain costs on top), any --shape, or
        # 2048^3: a product whose 256 x 256 tiles would occupy a quarter of the CUs (the 128 x 128 tile's case)
        m, n, k = {"gemm_f16_4095x11008x4096": (4095, 11008, 4096), "gemm_bf16_2048": (2048, 2048, 2048)}.get(name, GEMM_SHAPE)
        bf16 = name != "gemm_f16_4095x11008x4096" and name != "gemm_f16_shape"
        dt = torch.bfloat16 if bf16 else torch.float16
        g.manual_seed(0xA5)
        t = (torch.randn(m, k, device="cuda", generator=g) * 0.02).to(dt)
        va = device_vector(sarek, hip, torch, t, elem_size=2)
        g.manual_seed(0xB5)
        t = (torch.randn(k, n, device="cuda", generator=g) * 0.02).to(dt)
        vb = device_vector(sarek, hip, torch, t, elem_size=2)
        del t
        vy = V.create(V.float32, m * n)
        sarek.Transfer.to_device(vy)
        src, entry = hip.library_kernel("gemm_bf16" if bf16 else "gemm_f16")
        a, na = E._args([E.Vec(va), E.Vec(vb), E.Vec(vy), E.Int32(m), E.Int32(n), E.Int32(k)])
        src_b, entry_b = src.encode(), entry.encode()
        main = Launch(hip, lib.sarek_hip_execute_run_source, src_b, hip.LANG_HIP, entry_b, dims(16, 16, 1),
                      dims((n + 15) // 16, (m + 15) // 16, 1), 0, 1, a, na)
        tn = "bf16" if bf16 else "f16"
        tile = hip.gemm16_tile(m, n, k)
        kern = {256: "gemm16_m16_kernel", 128: "gemm16_m16_small_kernel"}.get(tile, "gemm16_staged_kernel")
        info = dict(metric=f"{tn} GEMM TFLOP/s at {m}x{n}x{k}", unit="TFLOP/s", dtype=tn,
                    work=2.0 * m * n * k, work_unit=1e12, bound="mfma",
                    peak=PEAK_MFMA_TFLOPS[tn], kernel=f"{kern}<{tn}, store>",
                    route=f"Execute.run_source ~lang:HIP_Source, library kernel text 'gemm_{tn}'",
                    config={"workload": f"{tn}-in f32-acc C=A.B, N(0,0.02)", "m": m, "n": n, "k": k,
                            "workgroup_tile": tile, "k_splits": hip.gemm16_k_splits(m, n, k)})
        return main, None, info, (va, vb, vy, a, src_b, entry_b)
    if name == "gemm_f16_epilogue":
        m, n, k = 4095, 11008, 4096
        g.manual_seed(0xA5)
        t = (torch.randn(m, k, device="cuda", generator=g) * 0.02).half()
        va = device_vector(sarek, hip, torch, t, elem_size=2)
        g.manual_seed(0xB5)
        t = (torch.randn(k, n, device="cuda", generator=g) * 0.02).half()
        vb = device_vector(sarek, hip, torch, t, elem_size=2)
        t = torch.rand(n, device="cuda", generator=g) * 0.2 - 0.1
        vbias = device_vector(sarek, hip, torch, t, V.float32)
        del t
        vy, vrs = V.create(V.float32, m * n), V.create(V.float32, m)
        sarek.Transfer.to_device(vy)
        sarek.Transfer.to_device(vrs)
        src, entry = hip.library_kernel("gemm_f16_bias_relu_rowsum")
        a, na = E._args([E.Vec(va), E.Vec(vb), E.Vec(vbias), E.Vec(vy), E.Vec(vrs), E.Int32(m), E.Int32(n), E.Int32(k)])
        src_b, entry_b = src.encode(), entry.encode()
        main = Launch(hip, lib.sarek_hip_execute_run_source, src_b, hip.LANG_HIP, entry_b, dims(256, 1, 1),
                      dims(1024, 1, 1), 0, 1, a, na)
        info = dict(metric="fp16 GEMM + bias + ReLU + row-sum TFLOP/s", unit="TFLOP/s", dtype="f16",
                    work=2.0 * m * n * k, work_unit=1e12, bound="mfma",
                    peak=PEAK_MFMA_TFLOPS["f16"], kernel="gemm16_m16_kernel<f16, bias_relu_rowsum>",
                    route="Execute.run_source ~lang:HIP_Source, library kernel text 'gemm_f16_bias_relu_rowsum'",
                    config={"workload": "fp16-in f32-acc Y=relu(A.B+bias), rowsum(Y)",
                            "m": m, "n": n, "k": k})
        return main, None, info, (va, vb, vbias, vy, vrs, a, src_b, entry_b)
    raise ValueError(name)


def stats(xs):
    xs = sorted(xs)
    return {"min": round(xs[0], 5), "median": round(xs[len(xs) // 2], 5), "avg": round(sum(xs) / len(xs), 5),
            "max": round(xs[-1], 5)}


WARMUP_MS = 60.0
TRACE_LAUNCHES = False


def measure(name, torch, hip, steps, warmup):
    """Warmup, then `steps` timed iterations, each launched and waited for, as the reference's benches do
    (benchmarks/bench_stream_triad.ml:98-115: time around launch + device synchronise, median reported).
    The dominant kernel's duration comes from HIP events recorded round its launch on the launch stream.
    The warmup is `warmup` steps and at least WARMUP_MS of them, launched and waited for like the timed ones: the
    package's power management needs 30-40 ms under a new load before the clocks settle (a power-limited kernel's
    third to sixth launch after a pause takes up to a third longer than its fiftieth)."""
    main, tail, info, keep = make_workload(name, torch, hip)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev = Events(hip, stream)
    sync = hip.lib.sarek_hip_device_synchronize
    path = None
    if info["route"].startswith("Execute"):
        main()                                   # alone, to read which code path served it
        path = hip.lib.sarek_hip_last_run_path().decode()
        sync()
    done, t_warm = 0, time.perf_counter()
    while done < warmup or (time.perf_counter() - t_warm) * 1e3 < WARMUP_MS:
        main()
        if tail:
            tail()
        sync()
        done += 1
    walls, kerns = [], []
    region = Events(hip, stream)                 # one pair of events round the whole timed region
    t0 = time.perf_counter()
    region.start()
    for _ in range(steps):
        w0 = time.perf_counter()
        main()
        if tail:
            tail()
        sync()
        walls.append((time.perf_counter() - w0) * 1e3)
    wall_ms = (time.perf_counter() - t0) * 1e3
    region_ms = region.stop_ms()
    # the dominant kernel's own duration: the same steps once more, HIP events round its launch
    for _ in range(steps):
        ev.start()
        main()
        hip.check(hip.lib.sarek_hip_event_record(ev.e1, stream))
        if tail:
            tail()
        sync()
        ms = C.c_float(0)
        hip.check(hip.lib.sarek_hip_event_elapsed_ms(ev.e0, ev.e1, C.byref(ms)))
        kerns.append(float(ms.value))
    kerns_in_order = list(kerns)
    ms_per_step = wall_ms / steps
    # second figure: the same launches back to back, one wait at the end (hotter: under the package power
    # limit the 16-bit GEMMs run slower this way)
    ev.start()
    for _ in range(steps):
        main()
        if tail:
            tail()
    back_to_back_ms = ev.stop_ms() / steps
    kernel_ms = sum(kerns) / len(kerns)
    value = info["work"] / (ms_per_step * 1e-3) / info["work_unit"]
    achieved = info["work"] / (kernel_ms * 1e-3) / info["work_unit"]
    res = {
        "metric": info["metric"], "value": round(value, 2), "unit": info["unit"],
        "ms_per_step": round(ms_per_step, 5), "ms_per_step_stats": stats(walls),
        "value_at_median": round(info["work"] / (stats(walls)["median"] * 1e-3) / info["work_unit"], 2),
        "gpu_ms_per_step_back_to_back": round(back_to_back_ms, 5),
        "dtype": info["dtype"], "config": info["config"], "route": info["route"], "served_by": path,
        "roofline": {"bound": info["bound"], "achieved": round(achieved, 2), "peak": info["peak"],
                     "unit": "GB/s" if info["bound"] in ("hbm", "l2") else "TFLOP/s",
                     "frac": round(achieved / info["peak"], 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(name),
                     "kernel": info["kernel"], "kernel_ms": round(kernel_ms, 5), "kernel_ms_stats": stats(kerns),
                     "timed_region_ms_per_step_by_events": round(region_ms / steps, 5),
                     "frac_back_to_back": round(info["work"] / (back_to_back_ms * 1e-3) / info["work_unit"] / info["peak"], 4)},
    }
    res["warmup_steps_done"] = done
    if TRACE_LAUNCHES:
        res["kernel_us_by_launch"] = [round(k * 1e3) for k in kerns_in_order]
    if name == "triad_sum_2p28":
        res["roofline"]["probe_kernels_GBs"] = hbm_ceiling(torch, hip)
    if name == "gemm_bf16_8192" and not ZERO_OPERANDS:
        # the same number of MFMA instructions per wave with nothing round them (register operands of the same
        # distribution, no memory instruction): what this box's power limit leaves of the peak on such data
        stream, stream32 = mfma_stream_rates(torch, hip)
        res["roofline"]["mfma_stream_only_TFLOPs"] = stream
        res["roofline"]["frac_of_mfma_stream_only"] = round(achieved / stream, 4)
        res["roofline"]["mfma_stream_only_32x32x16_TFLOPs"] = stream32
        # the vendor library on the same inputs, same protocol (torch.matmul -> hipBLASLt; it writes bf16 C)
        res["roofline"]["vendor_library_TFLOPs"] = vendor_gemm_rate(torch, hip)
    if info["bound"] == "mfma" and info["route"].startswith("Execute") and kernel_ms >= 0.2:
        # shader clock while the kernel runs: eight sleeping waves on a stream of their own count shader cycles against
        # the constant-rate clock over the first 70 % of the launch (nothing is added to the kernel itself), and the
        # rate of those very launches against the peak scaled to that clock
        sampler = hip.shader_clock_sampler()
        pairs = []
        for _ in range(min(steps, 10)):
            sampler.start(0.7 * kernel_ms)
            ev.start()
            main()
            ms = ev.stop_ms()
            mhz = sampler.mhz()
            if mhz:
                pairs.append((ms, mhz))
        sampler.close()
        if pairs:
            pairs.sort()
            ms, mhz = pairs[len(pairs) // 2]
            res["roofline"]["shader_clock_mhz"] = round(mhz, 1)
            res["roofline"]["frac_of_peak_at_that_clock"] = round(
                info["work"] / (ms * 1e-3) / info["work_unit"] / (info["peak"] * mhz / NOMINAL_CLOCK_MHZ), 4)
    del keep
    return res


MFMA_STREAM_SRC = r"""
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));
#define MF(ACC, A, B) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(ACC) : "v"(A), "v"(B))
__device__ inline float rnd(unsigned& s) {   // sum of four uniforms scaled to sigma = 0.02
  float acc = 0.f;
  for (int i = 0; i < 4; ++i) { s = s * 1664525u + 1013904223u; acc += (float)(s >> 8) * (1.0f / 16777216.0f) - 0.5f; }
  return acc * 0.0346f;
}
__device__ inline unsigned two_bf16(unsigned& s, int zero) {
  const float x = zero ? 0.f : rnd(s), y = zero ? 0.f : rnd(s);
  return (__float_as_uint(x) >> 16) | (__float_as_uint(y) & 0xffff0000u);
}
extern "C" __global__ __launch_bounds__(512) void mfma_stream(float* out, int n_out, int iters, int zero) {
  unsigned s = (blockIdx.x * 512 + threadIdx.x) * 2654435761u + 12345u;
  u4 A[2][4], B[2][2];
  _Pragma("unroll") for (int kk = 0; kk < 2; ++kk) {
    _Pragma("unroll") for (int i = 0; i < 4; ++i)
      _Pragma("unroll") for (int e = 0; e < 4; ++e) A[kk][i][e] = two_bf16(s, zero);
    _Pragma("unroll") for (int j = 0; j < 2; ++j)
      _Pragma("unroll") for (int e = 0; e < 4; ++e) B[kk][j][e] = two_bf16(s, zero);
  }
  f16v acc[4][2];
  _Pragma("unroll") for (int i = 0; i < 4; ++i)
    _Pragma("unroll") for (int j = 0; j < 2; ++j)
      _Pragma("unroll") for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it)
    _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)
      _Pragma("unroll") for (int i = 0; i < 4; ++i)
        _Pragma("unroll") for (int j = 0; j < 2; ++j) MF(acc[i][j], A[kk][i], B[kk][j]);
  float sum = 0.f;
  _Pragma("unroll") for (int i = 0; i < 4; ++i)
    _Pragma("unroll") for (int j = 0; j < 2; ++j) sum += acc[i][j][0] + acc[i][j][7];
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}
// the same flops per iteration with v_mfma_f32_16x16x32_bf16: 32 instructions on 16 accumulator tiles of 16 x 16
typedef float f4v __attribute__((ext_vector_type(4)));
#define MF16(ACC, A, B) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(ACC) : "v"(A), "v"(B))
extern "C" __global__ __launch_bounds__(512) void mfma_stream16(float* out, int n_out, int iters, int zero) {
  unsigned s = (blockIdx.x * 512 + threadIdx.x) * 2654435761u + 12345u;
  u4 A[2][4], B[2][4];
  _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)
    _Pragma("unroll") for (int i = 0; i < 4; ++i)
      _Pragma("unroll") for (int e = 0; e < 4; ++e) { A[kk][i][e] = two_bf16(s, zero); B[kk][i][e] = two_bf16(s, zero); }
  f4v acc[4][4];
  _Pragma("unroll") for (int i = 0; i < 4; ++i)
    _Pragma("unroll") for (int j = 0; j < 4; ++j)
      _Pragma("unroll") for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it)
    _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)
      _Pragma("unroll") for (int i = 0; i < 4; ++i)
        _Pragma("unroll") for (int j = 0; j < 4; ++j) MF16(acc[i][j], A[kk][i], B[kk][j]);
  float sum = 0.f;
  _Pragma("unroll") for (int i = 0; i < 4; ++i)
    _Pragma("unroll") for (int j = 0; j < 4; ++j) sum += acc[i][j][0] + acc[i][j][3];
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}
"""


L2_STREAM_SRC = r"""
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// every workgroup walks its own start in a window of (window_mask + 512) 16-byte pieces and brings 512 x 16 bytes per
// step into LDS; a wave keeps up to 16 transfers in flight
extern "C" __global__ __launch_bounds__(512) void l2_to_lds(const u32x4* __restrict__ src, int nsrc, unsigned* __restrict__ sink,
                                                           int nsink, int steps, int window_mask, int wg_stride) {
  __shared__ __attribute__((aligned(1024))) char stage[64 * 1024];
  const int wave = threadIdx.x >> 6;
  unsigned pos = (blockIdx.x * (unsigned)wg_stride) & window_mask;
  __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, nsrc * 4, 0x00020000);
  for (int i = 0; i < steps; i += 8) {
    _Pragma("unroll") for (int u = 0; u < 8; ++u) {
      const unsigned off = (((pos + u * 512) & window_mask) + threadIdx.x) << 4;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(stage + (u * 8 + wave) * 1024),
                                               16, (int)off, 0, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt((8 & 15) | ((8 >> 4) << 14) | (7 << 4) | (15 << 8));   // vmcnt <= 8
    pos = (pos + 8 * 512) & window_mask;
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (*(volatile unsigned*)(stage + threadIdx.x * 4) == 0x12345678u) sink[0] = 1;
}
"""


TRIAD_SHAPE_SRC = r"""
typedef float f4 __attribute__((ext_vector_type(4)));
#define THREADS THREADS_N
#define PIECES PIECES_N
__device__ inline float t1(float b, float c) { return (float)((double)b + (double)c * 3.0); }
extern "C" __global__ __launch_bounds__(THREADS) void triad_shape_probe(f4* __restrict__ a, int na, const f4* __restrict__ b, int nb,
                                                                       const f4* __restrict__ c, int nc) {
  const long base = (long)blockIdx.x * THREADS * PIECES + threadIdx.x;
  f4 bv[PIECES], cv[PIECES], r[PIECES];
  _Pragma("unroll") for (int u = 0; u < PIECES; ++u) bv[u] = __builtin_nontemporal_load(b + base + u * THREADS);
  _Pragma("unroll") for (int u = 0; u < PIECES; ++u) cv[u] = __builtin_nontemporal_load(c + base + u * THREADS);
  _Pragma("unroll") for (int u = 0; u < PIECES; ++u)
    r[u] = f4{t1(bv[u].x, cv[u].x), t1(bv[u].y, cv[u].y), t1(bv[u].z, cv[u].z), t1(bv[u].w, cv[u].w)};
  if (PHASES_N) __syncthreads();
  _Pragma("unroll") for (int u = 0; u < PIECES; ++u) __builtin_nontemporal_store(r[u], a + base + u * THREADS);
}
"""


SCATTER_CHAIN_SRC = r"""
typedef int i32x4 __attribute__((ext_vector_type(4)));
#define LOOK LOOK_N
#define ROUNDS ROUNDS_N
// The phases of the library's scatter kernel on a tile of 1024 x 16 keys; where that kernel takes the tile's range of
// every digit with a returning atomic, this one publishes and reads status words as a chained scan would.
extern "C" __global__ __launch_bounds__(1024) void scatter_chain_probe(int* __restrict__ out, int n_out, const int* __restrict__ keys,
                                                                      int n_keys, int* __restrict__ counters, int n_counters,
                                                                      unsigned* __restrict__ status, int n_status, int shift, int mask) {
  extern __shared__ int stage[];
  __shared__ int count[256], start[256], base[256], wave_total[4];
  __shared__ unsigned look[1024];
  const int t = threadIdx.x, lane = t & 63;
  const long tile = (long)blockIdx.x * 16384;
  if (t < 256) count[t] = 0;
  __syncthreads();
  int key[16], rank[16];
  const i32x4* k4 = (const i32x4*)(keys + tile);
  _Pragma("unroll") for (int u = 0; u < 4; ++u) {
    const i32x4 v = __builtin_nontemporal_load(k4 + u * 1024 + t);
    key[4 * u] = v.x; key[4 * u + 1] = v.y; key[4 * u + 2] = v.z; key[4 * u + 3] = v.w;
  }
  _Pragma("unroll") for (int j = 0; j < 16; ++j) rank[j] = atomicAdd(&count[(key[j] >> shift) & mask], 1);
  __syncthreads();
  unsigned seen = 0;
  if (LOOK > 0) {
    const int d = t & 255, q = t >> 8;
    if (t < 256) __hip_atomic_store(status + (long)blockIdx.x * 256 + t, 0x40000000u | (unsigned)count[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    long first = (long)blockIdx.x - 1;
    _Pragma("unroll 1") for (int r = 0; r < ROUNDS; ++r) {
      unsigned part = seen & 1;                       // the next round's addresses wait for this round's words
      _Pragma("unroll") for (int j = 0; j < (LOOK / ROUNDS + 3) / 4; ++j) {
        long p = first - part - (j * 4 + q);
        if (p < 0) p = 0;
        part += __hip_atomic_load(status + p * 256 + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0x3fffffffu;
      }
      seen += part;
      first -= LOOK / ROUNDS;
    }
    look[t] = seen;
    __syncthreads();
    if (t < 256) {
      seen = look[t] + look[256 + t] + look[512 + t] + look[768 + t];
      __hip_atomic_store(status + (long)blockIdx.x * 256 + t, 0x80000000u | (seen & 0x3fffffffu), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (t < 256) {
    const int c = count[t];
    int incl = c;
    _Pragma("unroll") for (int o = 1; o < 64; o <<= 1) { const int up = __shfl_up(incl, o); if (lane >= o) incl += up; }
    if (lane == 63) wave_total[t >> 6] = incl;
    start[t] = incl - c;
    base[t] = counters[t] + (int)(blockIdx.x % 7) * c + (seen == 0xffffffffu ? 1 : 0);   // somewhere inside the output
  }
  __syncthreads();
  if (t < 256) {
    int before = 0;
    for (int w = 0; w < (t >> 6); ++w) before += wave_total[w];
    start[t] += before;
    base[t] -= start[t];
  }
  __syncthreads();
  _Pragma("unroll") for (int j = 0; j < 16; ++j) stage[start[(key[j] >> shift) & mask] + rank[j]] = key[j];
  __syncthreads();
  for (int s = t; s < 16384; s += 1024) {
    const int k = stage[s];
    const long pos = (long)base[(k >> shift) & mask] + s;
    if (pos >= 0 && pos < n_out) out[pos] = k;
  }
}
"""


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


def mfma_stream_rates(torch, hip, launches=15):
    """TFLOP/s of the bare MFMA streams of MFMA_STREAM_SRC (mfma_stream16 = v_mfma_f32_16x16x32_bf16, the GEMM
    kernel's instruction; mfma_stream = v_mfma_f32_32x32x16_bf16), JIT-compiled through the plugin path: each is
    warmed up like a workload (WARMUP_MS of launches, each waited for, after the launch that compiles it), then the
    median of `launches` waited launches is reported (16x16x32, 32x32x16)."""
    out = torch.zeros(256 * 512, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev = Events(hip, stream)
    flop = 256.0 * 8 * 1024 * 16 * 32768
    rates = []
    for entry in ("mfma_stream16", "mfma_stream"):
        def launch():
            ev.start()
            hip.run_source(MFMA_STREAM_SRC, entry, (512, 1, 1), (256, 1, 1), [out, ("i32", 1024), ("i32", 0)])
            return ev.stop_ms()
        launch()
        t_warm = time.perf_counter()
        while (time.perf_counter() - t_warm) * 1e3 < WARMUP_MS:
            launch()
        times = sorted(launch() for _ in range(launches))
        rates.append(round(flop / (times[len(times) // 2] * 1e-3) / 1e12, 1))
    return tuple(rates)


def vendor_gemm_rate(torch, hip, launches=20):
    """TFLOP/s of torch.matmul (hipBLASLt) on the headline's 8192^3 bf16 inputs: WARMUP_MS of launches each waited
    for, then the average of `launches` waited launches by HIP events on the launch stream, as for the kernel."""
    s = 8192
    g = torch.Generator(device="cuda")
    g.manual_seed(0xA4)
    a = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
    g.manual_seed(0xB4)
    b = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
    c = torch.empty(s, s, device="cuda", dtype=torch.bfloat16)
    ev = Events(hip, C.c_void_p(torch.cuda.current_stream().cuda_stream))

    def launch():
        ev.start()
        torch.matmul(a, b, out=c)
        return ev.stop_ms()
    launch()
    t_warm = time.perf_counter()
    while (time.perf_counter() - t_warm) * 1e3 < WARMUP_MS:
        launch()
    ms = sum(launch() for _ in range(launches)) / launches
    return round(2.0 * s ** 3 / (ms * 1e-3) / 1e12, 1)


def event_overhead_ms(torch, hip, launches=20):
    """Median of what the two events round a launch measure when the kernel does nothing: the part of every
    `kernel_ms` that is event and dispatch handling, not kernel."""
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev = Events(hip, stream)
    src = 'extern "C" __global__ void nothing(int n) {}'
    times = []
    for i in range(launches + 3):
        ev.start()
        hip.run_source(src, "nothing", (64, 1, 1), (1, 1, 1), [("i32", 0)])
        ms = ev.stop_ms()
        if i >= 3:
            times.append(ms)
    times.sort()
    return round(times[len(times) // 2], 5)


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
    # threads: the cores this process may run on, at most 16 (the share of a one-GPU box)
    cores = min(len(os.sched_getaffinity(0)) or 1, 16)
    rng = np.random.default_rng(0)
    if name == "triad_sum_2p28":
        n = 1 << 28
        b = rng.random(n, dtype=np.float32)
        c = rng.random(n, dtype=np.float32)
        oracle.triad_sum(b[:1 << 20], c[:1 << 20], 3.0, threads=cores)
        passes = 400
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
        rows, n, k = 8192, 8192, 8192
    a = rng.normal(0, 0.02, (rows, k)).astype(np.float32)
    b = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    if name == "gemm_bf16_8192":
        a, b = oracle.round_bf16(a), oracle.round_bf16(b)
    elif name == "gemm_f16_epilogue":
        a, b = oracle.round_f16(a), oracle.round_f16(b)
    idx = np.arange(rows, dtype=np.int32)
    oracle.gemm_rows(a[:8], b, idx[:8], threads=cores)
    reps = 2 if rows * n * k >= 1 << 38 else 20
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.gemm_rows(a, b, idx, threads=cores)
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(2.0 * rows * n * k / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores,
            "kind": "port",
            "sample": f"all {rows} output rows (n={n}, k={k}) on the workload's rounded operands, double accumulation "
                      f"in k order, mean of {reps} passes, {dt * reps:.1f} s in total"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    if args.measure_build:
        os.environ["SAREK_HIP_MEASURE_BUILD"] = "1"
    import torch
    from spoc_amd import hip
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    global ZERO_OPERANDS, GEMM_SHAPE, WARMUP_MS, TRACE_LAUNCHES, L2_STREAM_SHAPE, CHAIN, TRIAD_SHAPE, FOLD
    FOLD = tuple(int(x) for x in args.fold.split(","))
    if len(FOLD) != 2 or not 1 <= FOLD[0] <= 1 << 28 or FOLD[1] not in (0, 1):
        sys.exit("--fold PARTIALS,TAKE_STAGES: 1 .. 2^28 partials, 0 or 1")
    TRIAD_SHAPE = tuple(int(x) for x in args.triad_shape.split(","))
    if len(TRIAD_SHAPE) != 3 or TRIAD_SHAPE[0] not in (64, 128, 256, 512, 1024) or TRIAD_SHAPE[1] not in (1, 2, 4, 6, 8) or \
            TRIAD_SHAPE[0] * TRIAD_SHAPE[1] > 6144:
        sys.exit("--triad-shape THREADS,FLOAT4_PER_THREAD,PHASES: 64..1024 threads, 1, 2, 4, 6 or 8 pieces, at most 6144 per workgroup")
    CHAIN = tuple(int(x) for x in args.chain.split(","))
    if len(CHAIN) != 2 or CHAIN[0] < 0 or CHAIN[0] > 1024 or CHAIN[1] < 1 or CHAIN[1] > 16:
        sys.exit("--chain PREDECESSORS,ROUNDS with 0..1024 predecessors in 1..16 rounds")
    if args.l2_stream:
        L2_STREAM_SHAPE = tuple(int(x) for x in args.l2_stream.split(","))
        if len(L2_STREAM_SHAPE) != 2 or L2_STREAM_SHAPE[1] not in (1, 2, 4, 8, 16) or L2_STREAM_SHAPE[0] < 1:
            sys.exit("--l2-stream WORKGROUPS,WINDOW_MIB with a window of 1, 2, 4, 8 or 16 MiB")
    WARMUP_MS, TRACE_LAUNCHES = args.warmup_ms, args.trace_launches
    ZERO_OPERANDS = args.zero_operands
    GEMM_SHAPE = tuple(int(x) for x in args.shape.split(","))
    for item in args.tunable:
        name, _, value = item.partition("=")
        hip.check(hip.lib.sarek_hip_set_tunable(name.encode(), int(value)))

    head = measure(args.workload, torch, hip, args.steps, args.warmup)
    out = {
        "metric": head["metric"], "value": head["value"], "unit": head["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic", "config": head["config"], "roofline": head["roofline"],
        "route": head["route"], "served_by": head["served_by"], "ms_per_step_stats": head["ms_per_step_stats"],
        "value_at_median": head["value_at_median"],
        "gpu_ms_per_step_back_to_back": head["gpu_ms_per_step_back_to_back"],
        "warmup_ms": args.warmup_ms, "warmup_steps_done": head["warmup_steps_done"],
    }
    if args.trace_launches:
        out["kernel_us_by_launch"] = head["kernel_us_by_launch"]
    if not args.no_cpu_baseline and args.workload not in ("copy_1gib", "vendor_gemm_bf16_8192", "vendor_gemm_bf16_shape", "gemm_bf16_shape", "gemm_f16_shape", "gemm_f32_shape", "vendor_gemm_f32_shape", "mfma_bf16_stream", "mfma_bf16_stream_32x32x16", "l2_to_lds_stream",
                                                        "stencil_2d_shape", "conv2d_shape", "map_sum_2p28", "radix_scatter_chain_probe", "triad_shape_probe"):
        out["cpu_baseline"] = cpu_baseline(args.workload)
    if not args.no_also:
        also = []
        for name in ["triad_sum_2p28", "map_sum_2p28", "gemm_f32_8192", "gemm_f16_epilogue", "gemm_f32_1024",
                     "gemm_bf16_8192", "histogram_2p28", "radix_scatter_5e7"]:
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            r = measure(name, torch, hip, args.steps, args.warmup)
            if not args.no_cpu_baseline and name == "triad_sum_2p28":
                r["cpu_baseline"] = cpu_baseline(name)
            also.append(r)
        out["also"] = also
    out["event_overhead_ms"] = event_overhead_ms(torch, hip)
    info = hip.device_info(0)
    if args.tunable:
        out["tunables"] = args.tunable
    if args.measure_build:
        out["library"] = "libsarek_hip_measure.so (measurement build)"
    if args.zero_operands:
        out["config"] = dict(out["config"], workload=out["config"]["workload"].replace("N(0,0.02)", "all-zero operands"))
    out["device"] = {"name": info.name.decode(), "arch": info.gcn_arch.decode(),
                     "cus": info.multiprocessor_count, "clock_mhz": info.clock_rate_khz // 1000}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
