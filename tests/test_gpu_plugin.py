"""GPU tests of the plugin-level path: JIT (hiprtc) external kernels through
run_source with the reference's argument convention, the kernel cache, the runtime
wrappers, and the hand-kernel dispatch behind specialise tags.

External-kernel convention follows sarek/tests/e2e/test_external_kernel.ml:46-62:
each vector is passed as (pointer, int length) unless lengths are not injected."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

VECTOR_ADD = r'''
extern "C" __global__ void vector_add(const float* a, int a_len, const float* b, int b_len,
                                      float* c, int c_len, int n) {
  int i = threadIdx.x + blockIdx.x * blockDim.x;
  if (i < n) c[i] = a[i] + b[i];
}
'''

# The generated text for the stream-triad kernel (golden:
# benchmarks/descriptions/generated/stream_triad_generated.md, CUDA section) is valid
# HIP as it stands.
TRIAD_GENERATED = '''
extern "C" {
__global__ void sarek_kern(float* __restrict__ a, int sarek_a_length, float* __restrict__ b, int sarek_b_length, float* __restrict__ c, int sarek_c_length, float scalar, int n) {
  int tid = (threadIdx.x + blockIdx.x * blockDim.x);
  if ((tid < n)) {
    a[tid] = (b[tid] + (c[tid] * scalar));
  }
}
}
'''


def test_runtime_device_info(hip, torch_cuda):
    hip.check(hip.lib.sarek_hip_init())
    n = C.c_int(0)
    hip.check(hip.lib.sarek_hip_device_count(C.byref(n)))
    assert n.value >= 1
    info = hip.device_info(0)
    assert info.warp_size == 64
    assert info.gcn_arch.decode().startswith("gfx950")
    assert info.multiprocessor_count >= 200
    assert info.shared_mem_per_block >= 64 * 1024


def test_device_report_is_the_reference_tools_text(hip, torch_cuda):
    """tools/device_info.ml:16-43,66-90: one block per device, laid out as print_device_info does."""
    import subprocess
    import sys
    text, count = hip.device_report()
    info = hip.device_info(0)
    gb = info.total_global_mem / 1024 ** 3
    block = (f"[0] {info.name.decode()}\n    Backend: HIP\n    Memory: {gb:.2f} GB\n"
             f"    Compute Capability: {info.compute_major}.{info.compute_minor}\n"
             f"    Max Threads/Block: {info.max_threads_per_block}\n    Compute Units: {info.multiprocessor_count}\n"
             f"    Warp/Wavefront Size: 64\n    Features: Atomics, FP64\n\n")
    assert count >= 1 and f"\nFound {count} device{'s' if count > 1 else ''}:\n\n" in text
    assert block in text and f"Device.get N returns device N (0-{count - 1})" in text
    root = __import__("os").path.dirname(__import__("os").path.dirname(__import__("os").path.abspath(__file__)))
    run = subprocess.run([sys.executable, "-m", "spoc_amd.device_info"], cwd=root, capture_output=True, text=True)
    assert run.returncode == 0 and run.stdout == text


def test_runtime_memory_roundtrip_and_double_free(hip, torch_cuda):
    p = C.c_void_p()
    hip.check(hip.lib.sarek_hip_mem_alloc(C.byref(p), 4096))
    src = np.arange(1024, dtype=np.float32)
    dst = np.zeros_like(src)
    hip.check(hip.lib.sarek_hip_memcpy_htod(p, src.ctypes.data, 4096))
    hip.check(hip.lib.sarek_hip_memcpy_dtoh(dst.ctypes.data, p, 4096))
    assert np.array_equal(src, dst)
    hip.check(hip.lib.sarek_hip_memset_d8(p, 0, 4096))
    hip.check(hip.lib.sarek_hip_memcpy_dtoh(dst.ctypes.data, p, 4096))
    assert not dst.any()
    hip.check(hip.lib.sarek_hip_mem_free(p))
    hip.check(hip.lib.sarek_hip_mem_free(p))   # explicit free then finaliser: tolerated


def test_runtime_events_and_streams(hip, torch_cuda):
    s = C.c_void_p()
    e0, e1 = C.c_void_p(), C.c_void_p()
    hip.check(hip.lib.sarek_hip_stream_create(C.byref(s)))
    hip.check(hip.lib.sarek_hip_event_create(C.byref(e0)))
    hip.check(hip.lib.sarek_hip_event_create(C.byref(e1)))
    hip.check(hip.lib.sarek_hip_event_record(e0, s))
    hip.check(hip.lib.sarek_hip_event_record(e1, s))
    hip.check(hip.lib.sarek_hip_event_synchronize(e1))
    ms = C.c_float(-1)
    hip.check(hip.lib.sarek_hip_event_elapsed_ms(e0, e1, C.byref(ms)))
    assert ms.value >= 0
    hip.check(hip.lib.sarek_hip_stream_synchronize(s))
    hip.check(hip.lib.sarek_hip_event_destroy(e0))
    hip.check(hip.lib.sarek_hip_event_destroy(e1))
    hip.check(hip.lib.sarek_hip_stream_destroy(s))
    # enable_profiling / disable_profiling: never an error, with or without a profiler attached
    assert hip.lib.sarek_hip_profiler_start() == 0 and hip.lib.sarek_hip_profiler_stop() == 0
    a = torch_cuda.ones(1024, device="cuda")
    assert float(hip.triad(a, a, 2.0).sum().item()) == 3072.0     # the runtime is left in working order


def test_run_source_external_kernel(hip, torch_cuda):
    torch = torch_cuda
    n = 1000
    a = torch.arange(n, device="cuda", dtype=torch.float32)
    b = torch.full((n,), 2.0, device="cuda")
    c = torch.zeros(n, device="cuda")
    path = hip.run_source(VECTOR_ADD, "vector_add", (256, 1, 1), ((n + 255) // 256, 1, 1),
                          [a, b, c, ("i32", n)])
    torch.cuda.synchronize()
    assert path == "jit"
    assert torch.equal(c, a + 2.0)
    # CUDA_Source text is accepted as HIP text (same dialect for these kernels)
    c.zero_()
    hip.run_source(VECTOR_ADD, "vector_add", (256, 1, 1), ((n + 255) // 256, 1, 1),
                   [a, b, c, ("i32", n)], lang=hip.LANG_CUDA)
    torch.cuda.synchronize()
    assert torch.equal(c, a + 2.0)


def test_run_source_compile_error_has_log(hip, torch_cuda):
    with pytest.raises(hip.SarekHipError) as e:
        hip.run_source("extern \"C\" __global__ void k() { this is not C; }", "k",
                       (1, 1, 1), (1, 1, 1), [])
    assert e.value.status == hip.E_COMPILE
    assert "error" in e.value.message


def test_generated_triad_text_jit_matches_oracle(hip, oracle, torch_cuda):
    torch = torch_cuda
    n = 5000
    b = oracle.fill_uniform(n, seed=0xB)
    c = oracle.fill_uniform(n, seed=0xC)
    db, dc = torch.from_numpy(b).cuda(), torch.from_numpy(c).cuda()
    a = torch.zeros(n, device="cuda")
    path = hip.run_source(TRIAD_GENERATED, "sarek_kern", (256, 1, 1), ((n + 255) // 256, 1, 1),
                          [a, db, dc, ("f32", 3.0), ("i32", n)])
    torch.cuda.synchronize()
    assert path == "jit"
    ref = oracle.triad(b, c, 3.0)
    assert np.abs(a.cpu().numpy() - ref).max() <= 1e-5     # reference tolerance; JIT uses f32 fma


def test_specialise_tag_routes_to_hand_kernel(hip, oracle, torch_cuda):
    torch = torch_cuda
    n = 5000
    b = oracle.fill_uniform(n, seed=0xB)
    c = oracle.fill_uniform(n, seed=0xC)
    db, dc = torch.from_numpy(b).cuda(), torch.from_numpy(c).cuda()
    a = torch.zeros(n, device="cuda")
    # a tag counts on a text generate_source handed out, not on the same line pasted in front of a program
    # (a byte-identical copy of a generated text IS that text, so this one differs by a comment)
    pasted = "// sarek-hip-specialise: stream_triad_f32\n// pasted\n" + TRIAD_GENERATED
    items = [a, db, dc, ("f32", 3.0), ("i32", n)]
    assert hip.run_source(pasted, "sarek_kern", (256, 1, 1), ((n + 255) // 256, 1, 1), items) == "jit"
    a.zero_()
    tagged = hip.generate_source(load_ir("stream_triad"), block=(256, 1, 1))
    assert tagged.startswith("// sarek-hip-specialise: stream_triad_f32\n")
    path = hip.run_source(tagged, "sarek_kern", (256, 1, 1), ((n + 255) // 256, 1, 1), items)
    torch.cuda.synchronize()
    assert path == "stream_triad_f32"
    assert np.array_equal(a.cpu().numpy(), oracle.triad(b, c, 3.0))
    # a grid that does not cover n keeps the generated kernel's partial-coverage semantics
    a.zero_()
    path = hip.run_source(tagged, "sarek_kern", (256, 1, 1), (2, 1, 1), items)
    torch.cuda.synchronize()
    assert path == "jit"
    got = a.cpu().numpy()
    assert (got[512:] == 0).all() and (got[:512] != 0).any()
    # switch off: always JIT
    hip.check(hip.lib.sarek_hip_set_specialisation(0))
    try:
        path = hip.run_source(tagged, "sarek_kern", (256, 1, 1), ((n + 255) // 256, 1, 1), items)
        assert path == "jit"
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))


# ---- the whole plugin path: IR -> generate_source -> run_source ------------------------
# Launch geometry and argument lists are the reference benches' own
# (bench_matrix_mul_tiled.ml:136-141, bench_stream_triad.ml:71-74, bench_reduction.ml:130-150).
import os

IR_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ir")


def load_ir(name):
    return open(os.path.join(IR_DIR, name + ".ir")).read()


@pytest.mark.parametrize("specialise", [1, 0])
@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (100, 72, 52), (256, 256, 256)])
def test_tiled_matmul_ir_end_to_end(hip, oracle, torch_cuda, specialise, m, n, k):
    torch = torch_cuda
    a = oracle.fill_uniform(m * k, seed=0xA11CE, lo=-1, hi=1).reshape(m, k)
    b = oracle.fill_uniform(k * n, seed=0xB0B, lo=-1, hi=1).reshape(k, n)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    dc = torch.full((m, n), float("nan"), device="cuda")   # Vector.create leaves C uninitialised
    src = hip.generate_source(load_ir("matrix_mul_tiled"), block=(16, 16, 1))
    hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
    try:
        path = hip.run_source(src, "sarek_kern", (16, 16, 1), ((n + 15) // 16, (m + 15) // 16, 1),
                              [da.view(-1), db.view(-1), dc.view(-1), ("i32", m), ("i32", n), ("i32", k)],
                              shared_mem=2048)
        hip.check(hip.lib.sarek_hip_device_synchronize())
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    assert path == ("matmul_tiled_f32" if specialise else "jit")
    ref = oracle.gemm(a, b)
    assert np.abs(dc.cpu().numpy() - ref).max() <= 1e-4 * np.sqrt(k)


@pytest.mark.parametrize("specialise", [1, 0])
def test_reduction_and_dot_ir_end_to_end(hip, oracle, torch_cuda, specialise):
    torch = torch_cuda
    n = 100000
    nblocks = (n + 255) // 256
    x = oracle.fill_uniform(n, seed=0x5)
    y = oracle.fill_uniform(n, seed=0x6)
    dx, dy = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    out = torch.zeros(nblocks, device="cuda")
    hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
    try:
        p1 = hip.run_source(hip.generate_source(load_ir("reduction")), "sarek_kern", (256, 1, 1),
                            (nblocks, 1, 1), [dx, out, ("i32", n)])
        hip.check(hip.lib.sarek_hip_device_synchronize())
        part = out.cpu().numpy().copy()
        p2 = hip.run_source(hip.generate_source(load_ir("dot_product")), "sarek_kern", (256, 1, 1),
                            (nblocks, 1, 1), [dx, dy, out, ("i32", n)], shared_mem=1024)
        hip.check(hip.lib.sarek_hip_device_synchronize())
        dot = out.cpu().numpy().copy()
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    assert (p1, p2) == (("reduce_sum_block256_f32", "dot_block256_f32") if specialise else ("jit", "jit"))
    assert np.allclose(part, oracle.reduce_sum_block256(x), rtol=1e-5, atol=1e-6)
    assert np.allclose(dot, oracle.dot_block256(x, y), rtol=1e-5, atol=1e-6)
    # host fold as the bench does it (bench_reduction.ml:154-163), 1e-3 relative
    exp = oracle.fold_partials(oracle.reduce_sum_block256(x))
    assert abs(float(part.astype(np.float64).sum()) - exp) / exp < 1e-3


def test_every_fixture_kernel_compiles_with_hiprtc(hip, torch_cuda):
    """The plain lowering of each golden kernel is accepted by hiprtc for this device."""
    import glob
    for path in sorted(glob.glob(os.path.join(IR_DIR, "*.ir"))):
        if path.endswith("reduction_max.ir"):
            continue   # its golden text holds the OCaml spelling Float.neg_infinity: not C
        src = hip.generate_source(open(path).read())
        k = C.c_void_p()
        log = C.create_string_buffer(8192)
        rc = hip.lib.sarek_hip_kernel_compile_cached(src.encode(), b"sarek_kern", C.byref(k), log, len(log))
        assert rc == 0, (path, log.value.decode())
    # second request for the same text is served from the cache (same handle)
    k2 = C.c_void_p()
    hip.check(hip.lib.sarek_hip_kernel_compile_cached(src.encode(), b"sarek_kern", C.byref(k2), None, 0))
    assert k2.value == k.value


def test_transpose_tiled_ir_end_to_end(hip, torch_cuda):
    """benchmarks/bench_transpose_tiled.ml: 16x16 blocks, padded 17-wide shared tile."""
    torch = torch_cuda
    w, h = 100, 52
    x = torch.arange(w * h, dtype=torch.float32, device="cuda")
    out = torch.full((w * h,), -1.0, device="cuda")
    path = hip.run_source(hip.generate_source(load_ir("transpose_tiled"), block=(16, 16, 1)), "sarek_kern",
                          (16, 16, 1), ((w + 15) // 16, (h + 15) // 16, 1),
                          [x, out, ("i32", w), ("i32", h)], shared_mem=272 * 4)
    hip.check(hip.lib.sarek_hip_device_synchronize())
    assert path == "transpose_tiled_f32"
    assert torch.equal(out.view(w, h), x.view(h, w).t())


def test_scatter_and_radix_ir_end_to_end(hip, torch_cuda):
    """benchmarks/bench_scatter.ml and bench_radix_sort.ml (one 8-bit pass): integer kernels,
    shared and global atomics, bit-exact against numpy."""
    torch = torch_cuda
    n = 10000
    rng = np.random.default_rng(7)
    vals = rng.integers(0, 1 << 20, n, dtype=np.int32)
    perm = rng.permutation(n).astype(np.int32)
    dv, dp = torch.from_numpy(vals).cuda(), torch.from_numpy(perm).cuda()
    out = torch.zeros(n, dtype=torch.int32, device="cuda")
    grid = ((n + 255) // 256, 1, 1)
    hip.run_source(hip.generate_source(load_ir("scatter")), "sarek_kern", (256, 1, 1), grid,
                   [dv, dp, out, ("i32", n)])
    hip.check(hip.lib.sarek_hip_device_synchronize())
    exp = np.zeros(n, np.int32)
    exp[perm] = vals
    assert np.array_equal(out.cpu().numpy(), exp)

    shift, mask = 4, 255
    hist = torch.zeros(256, dtype=torch.int32, device="cuda")
    hip.run_source(hip.generate_source(load_ir("radix_sort_histogram")), "sarek_kern", (256, 1, 1), grid,
                   [dv, hist, ("i32", n), ("i32", shift), ("i32", mask)], shared_mem=1024)
    hip.check(hip.lib.sarek_hip_device_synchronize())
    digits = (vals >> shift) & mask
    counts = np.bincount(digits, minlength=256).astype(np.int32)
    assert np.array_equal(hist.cpu().numpy(), counts)

    # scatter pass: counters start at the exclusive prefix sums (bench_radix_sort.ml:158-200);
    # the order inside a bin is not fixed (global atomics), so compare bins as multisets
    starts = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int32)
    counters = torch.from_numpy(starts.copy()).cuda()
    sorted_out = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    hip.run_source(hip.generate_source(load_ir("radix_sort_scatter")), "sarek_kern", (256, 1, 1), grid,
                   [dv, sorted_out, counters, ("i32", n), ("i32", shift), ("i32", mask)])
    hip.check(hip.lib.sarek_hip_device_synchronize())
    got = sorted_out.cpu().numpy()
    gd = (got >> shift) & mask
    assert np.all(np.diff(gd) >= 0)
    assert np.array_equal(np.sort(got), np.sort(vals))
    assert np.array_equal(counters.cpu().numpy(), starts + counts)


@pytest.mark.parametrize("specialise", [1, 0])
def test_reduction_max_ir_end_to_end(hip, oracle, torch_cuda, specialise):
    """bench_reduction_max.ml as written today (fill -1000000.0): hand kernel and JIT-compiled
    lowering give the tree's result bit for bit."""
    from test_ir_lowering import reduction_max_ir
    torch = torch_cuda
    n = 70001
    nblocks = (n + 255) // 256
    x = (oracle.fill_uniform(n, seed=0x9) * 2000 - 1000).astype(np.float32)
    dx = torch.from_numpy(x).cuda()
    out = torch.zeros(nblocks, device="cuda")
    hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
    try:
        path = hip.run_source(hip.generate_source(reduction_max_ir()), "sarek_kern", (256, 1, 1),
                              (nblocks, 1, 1), [dx, out, ("i32", n)], shared_mem=1024)
        hip.check(hip.lib.sarek_hip_device_synchronize())
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    assert path.startswith("reduce_max_block256_f32:") if specialise else path == "jit"
    assert np.array_equal(out.cpu().numpy(), oracle.reduce_max_block256(x))
    assert out.max().item() == x.max()     # the bench's own check: max of partials = max of input


@pytest.mark.parametrize("name,size,path", [
    ("matrix_mul_tiled", 200, "matmul_tiled_f32"), ("stream_triad", 100003, "stream_triad_f32"),
    ("reduction", 100003, "reduce_sum_block256_f32"), ("dot_product", 100003, "dot_block256_f32"),
    ("reduction_max", 100003, "reduce_max_block256_f32:c9742400")])
def test_reference_benchmarks_run_and_verify(hip, torch_cuda, name, size, path):
    """The mirrors of benchmarks/bench_*.ml: the reference's inputs, geometry and checks, served
    by the hand kernels; and the same with the plain JIT lowering."""
    from spoc_amd import benchmarks
    fn = benchmarks.BENCHMARKS[name][0]
    rec = fn(size, warmup=1, iterations=3)
    assert rec["verified"] and rec["path"] == path and len(rec["iterations"]) == 3
    assert rec["median_ms"] > 0 and rec["throughput_gflops"] > 0 and rec["framework"] == "HIP"
    hip.check(hip.lib.sarek_hip_set_specialisation(0))
    try:
        rec = fn(size, warmup=1, iterations=2)
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    assert rec["verified"] and rec["path"] == "jit"


def test_a_text_with_a_float_of_its_own_is_left_as_written(hip, torch_cuda):
    """Texts that name OCaml's Float.* / Int32.* / Int64.* constants are compiled with their values in front; a text
    that declares an object called Float itself gets nothing added (the two definitions would clash)."""
    torch = torch_cuda
    own = ("struct mine { float neg_infinity; };\n__device__ mine Float = {42.0f};\n"
           "extern \"C\" __global__ void k(float* out, int out_len) { out[0] = Float.neg_infinity; }\n")
    out = torch.zeros(4, device="cuda")
    assert hip.run_source(own, "k", (1, 1, 1), (1, 1, 1), [out]) == "jit"
    torch.cuda.synchronize()
    assert out[0].item() == 42.0
    named = "extern \"C\" __global__ void k2(float* out, int out_len) { out[1] = Float.neg_infinity; out[2] = (float)Int32.max_int; }\n"
    hip.run_source(named, "k2", (1, 1, 1), (1, 1, 1), [out])
    torch.cuda.synchronize()
    assert out[1].item() == float("-inf") and out[2].item() == 2147483648.0
