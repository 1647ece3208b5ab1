"""Vector add, vector copy, transposes and the one-thread-per-element matmul of the reference's
benches (benchmarks/bench_vector_add.ml, bench_vector_copy.ml, bench_transpose.ml,
bench_transpose_tiled.ml, bench_matrix_mul.ml): the hand kernels through the C ABI and the
kernels' IR through generate_source / run_source, both against the CPU oracle, bit for bit
(the matmul to the f32 GEMM bound)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

IR_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ir")


def load_ir(name):
    return open(os.path.join(IR_DIR, name + ".ir")).read()


def run_ir(hip, name, block, grid, args, specialise, shared_mem=0):
    src = hip.generate_source(load_ir(name), block=block)
    hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
    try:
        path = hip.run_source(src, "sarek_kern", block, grid, args, shared_mem=shared_mem)
        hip.check(hip.lib.sarek_hip_device_synchronize())
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    return path


# ---- the kernels through the C ABI -------------------------------------------------------------

@pytest.mark.parametrize("n", [0, 1, 3, 4, 255, 8191, 8192, 8193, 100003, (1 << 24) + 5])
def test_copy_sizes(hip, torch_cuda, n):
    torch = torch_cuda
    src = torch.rand(n + 8, device="cuda")
    dst = torch.full((n + 8,), -1.0, device="cuda")
    hip.check(hip.lib.sarek_hip_copy_f32(dst.data_ptr(), src.data_ptr(), n, None))
    torch.cuda.synchronize()
    assert torch.equal(dst[:n], src[:n]) and bool((dst[n:] == -1).all())


def test_copy_unaligned_and_policies(hip, torch_cuda):
    torch = torch_cuda
    n = 70001
    base_s, base_d = torch.rand(n + 16, device="cuda"), torch.zeros(n + 16, device="cuda")
    for scalar in (0, 1):                                      # the 128-bit kernel and the element-per-thread one
        hip.set_tunable("copy.force_scalar", scalar)
        try:
            for so, do in ((1, 0), (0, 3), (2, 2)):            # 4-byte aligned only
                s, d = base_s[so:so + n], base_d[do:do + n]
                base_d.fill_(-1)
                hip.check(hip.lib.sarek_hip_copy_f32(d.data_ptr(), s.data_ptr(), n, None))
                torch.cuda.synchronize()
                assert torch.equal(d, s)
                assert bool((base_d[:do] == -1).all()) and bool((base_d[do + n:] == -1).all())
        finally:
            hip.set_tunable("copy.force_scalar", 0)
    try:
        for nt in (0, 1):                                      # both load policies
            hip.set_tunable("copy.nt", nt)
            d = hip.copy(base_s)
            torch.cuda.synchronize()
            assert torch.equal(d, base_s)
    finally:
        hip.set_tunable("copy.nt", -1)
    assert hip.lib.sarek_hip_copy_f32(None, base_s.data_ptr(), 4, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_copy_f32(base_d.data_ptr(), base_s.data_ptr(), -1, None) == hip.E_INVALID_ARG


@pytest.mark.parametrize("h,w", [(1, 1), (1, 5), (4, 4), (64, 64), (128, 64), (100, 52), (52, 100), (256, 1024),
                                 (1000, 4096), (4100, 8196), (1023, 777), (4097, 4095), (3, 70000)])
def test_transpose_shapes(hip, oracle, torch_cuda, h, w):
    torch = torch_cuda
    x = torch.rand(h, w, device="cuda")
    out = hip.transpose(x)
    torch.cuda.synchronize()
    assert out.shape == (w, h) and torch.equal(out, x.t())
    if h * w <= 1 << 16:
        ref = oracle.transpose(x.cpu().numpy().reshape(-1), w, h)
        assert np.array_equal(out.cpu().numpy().reshape(-1), ref)


def test_transpose_every_variant(hip, torch_cuda):
    torch = torch_cuda
    x = torch.rand(520, 1032, device="cuda")        # ragged against 64 and 128
    try:
        for variant, rows, order, nt in [(0, r, o, t) for r in (64, 128) for o in (0, 1, 2, 3) for t in (0, 1, 2, 3)] + \
                                        [(1, 64, o, 3) for o in (0, 1, 2, 3)]:
            for name, v in (("variant", variant), ("rows", rows), ("order", order), ("nt", nt)):
                hip.set_tunable("transpose." + name, v)
            out = hip.transpose(x)
            torch.cuda.synchronize()
            assert torch.equal(out, x.t()), (variant, rows, order, nt)
    finally:
        hip.set_tunable("transpose.variant", 0)
        hip.set_tunable("transpose.rows", 128)
        hip.set_tunable("transpose.order", -1)
        hip.set_tunable("transpose.nt", -1)
    # matrices that are only 4-byte aligned: the tiled kernel, and the scalar one behind its knob
    for scalar in (0, 1):
        hip.set_tunable("transpose.force_scalar", scalar)
        try:
            flat = torch.rand(64 * 128 + 1, device="cuda")
            out = torch.full((64 * 128 + 3,), -1.0, device="cuda")
            hip.check(hip.lib.sarek_hip_transpose_f32(flat[1:].data_ptr(), out[1:-2].data_ptr(), 64, 128, None))
            torch.cuda.synchronize()
            assert torch.equal(out[1:-2].view(64, 128), flat[1:].view(128, 64).t())
            assert out[0].item() == -1 and bool((out[-2:] == -1).all())
        finally:
            hip.set_tunable("transpose.force_scalar", 0)
    assert hip.lib.sarek_hip_transpose_f32(flat.data_ptr(), flat.data_ptr(), 8, 8, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_transpose_f32(flat.data_ptr(), out.data_ptr(), -1, 8, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_transpose_f32(flat.data_ptr(), out.data_ptr(), 0, 8, None) == 0


@pytest.mark.parametrize("h,w", [(519, 1031), (130, 66), (5, 3), (1, 7), (257, 1), (1030, 516), (2, 1029)])
def test_ragged_transposes_every_policy_and_guards(hip, torch_cuda, h, w):
    """Widths and heights that are not multiples of 4 run the tiled kernel too (rows then start at any 4-byte offset,
    the pieces across a row's end go element by element): every tile height, order and cache policy, with guard
    elements round the output, and the element-per-access kernel behind its knob."""
    torch = torch_cuda
    flat = torch.rand(h * w + 3, device="cuda")
    x = flat[3:].view(h, w)
    try:
        for rows, order, nt, scalar in [(r, o, t, 0) for r in (64, 128) for o in (0, 1, 2, 3) for t in (0, 1, 2, 3)] + \
                                       [(128, -1, -1, 0), (128, -1, -1, 1)]:
            for name, v in (("rows", rows), ("order", order), ("nt", nt), ("force_scalar", scalar)):
                hip.set_tunable("transpose." + name, v)
            out = torch.full((h * w + 9,), -1.0, device="cuda")
            hip.check(hip.lib.sarek_hip_transpose_f32(x.data_ptr(), out[5:].data_ptr(), w, h, None))
            torch.cuda.synchronize()
            assert torch.equal(out[5:5 + h * w].view(w, h), x.t()), (rows, order, nt, scalar)
            assert bool((out[:5] == -1).all()) and bool((out[5 + h * w:] == -1).all()), (rows, order, nt, scalar)
    finally:
        hip.set_tunable("transpose.rows", 128)
        hip.set_tunable("transpose.order", -1)
        hip.set_tunable("transpose.nt", -1)
        hip.set_tunable("transpose.force_scalar", 0)


# ---- the reference kernels' IR, hand kernel and JIT lowering side by side ------------------------

@pytest.mark.parametrize("specialise", [1, 0])
@pytest.mark.parametrize("n,extra_threads", [(100003, 0), (4096, 0), (1000, 1024), (1, 0)])
def test_vector_add_and_copy_ir(hip, oracle, torch_cuda, specialise, n, extra_threads):
    torch = torch_cuda
    a = oracle.fill_uniform(n + 7, seed=1, lo=-100, hi=100)
    b = oracle.fill_uniform(n + 7, seed=2, lo=-1e-3, hi=1e-3)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    dc = torch.full((n + 7,), -5.0, device="cuda")
    grid = ((n + extra_threads + 255) // 256, 1, 1)
    path = run_ir(hip, "vector_add", (256, 1, 1), grid, [da, db, dc, ("i32", n)], specialise)
    assert path == ("vector_add_f32" if specialise else "jit")
    ref = oracle.vector_add(a, b, np.full(n + 7, -5.0, dtype=np.float32), n, threads=grid[0] * 256)
    assert np.array_equal(dc.cpu().numpy(), ref)
    dd = torch.full((n + 7,), -6.0, device="cuda")
    path = run_ir(hip, "vector_copy", (256, 1, 1), grid, [da, dd, ("i32", n)], specialise)
    assert path == ("vector_copy_f32" if specialise else "jit")
    assert np.array_equal(dd.cpu().numpy(), oracle.vector_copy(a, np.full(n + 7, -6.0, dtype=np.float32), n))
    # in place: c is a
    path = run_ir(hip, "vector_add", (256, 1, 1), grid, [da, db, da, ("i32", n)], specialise)
    assert path == ("vector_add_f32" if specialise else "jit")
    assert np.array_equal(da.cpu().numpy()[:n], (a + b)[:n])


def test_launches_the_hand_kernels_must_not_take(hip, torch_cuda):
    torch = torch_cuda
    n = 5000
    a, b, c = (torch.rand(n, device="cuda") for _ in range(3))
    # too few threads for n: the generated kernel leaves the rest alone, so it has to run
    assert run_ir(hip, "vector_add", (256, 1, 1), (4, 1, 1), [a, b, c, ("i32", n)], 1) == "jit"
    assert torch.equal(c[:1024], (a + b)[:1024])
    # output shifted over an input: a race in the generated kernel, left to it
    assert run_ir(hip, "vector_copy", (256, 1, 1), (20, 1, 1), [a[:-1], a[1:], ("i32", n - 1)], 1) == "jit"
    # vectors that just hold n elements are taken
    assert run_ir(hip, "vector_copy", (256, 1, 1), (20, 1, 1), [a[:100], b, ("i32", 100)], 1) == "vector_copy_f32"
    x, y = torch.rand(64 * 48, device="cuda"), torch.zeros(64 * 48, device="cuda")
    assert run_ir(hip, "transpose_naive", (256, 1, 1), (3, 1, 1), [x, y, ("i32", 64), ("i32", 48)], 1) == "jit"
    assert run_ir(hip, "transpose_tiled", (16, 16, 1), (4, 2, 1), [x, y, ("i32", 64), ("i32", 48)], 1,
                  shared_mem=272 * 4) == "jit"          # grid y covers 32 of 48 rows
    assert run_ir(hip, "transpose_naive", (256, 1, 1), (12, 1, 1), [x, x, ("i32", 64), ("i32", 48)], 1) == "jit"
    m = 40
    A, B, Cm = (torch.rand(m * m, device="cuda") for _ in range(3))
    args = [A, B, Cm, ("i32", m), ("i32", m), ("i32", m)]
    assert run_ir(hip, "matrix_mul", (256, 1, 1), (2, 1, 1), args, 1) == "jit"      # 512 threads < 1600


@pytest.mark.parametrize("specialise", [1, 0])
@pytest.mark.parametrize("w,h", [(100, 52), (64, 64), (256, 128), (17, 3)])
def test_transpose_ir_both_forms(hip, oracle, torch_cuda, specialise, w, h):
    torch = torch_cuda
    x = oracle.fill_uniform(w * h, seed=9, lo=-1, hi=1)
    dx = torch.from_numpy(x).cuda()
    ref = oracle.transpose(x, w, h)
    out = torch.full((w * h,), -1.0, device="cuda")
    path = run_ir(hip, "transpose_naive", (256, 1, 1), ((w * h + 255) // 256, 1, 1),
                  [dx, out, ("i32", w), ("i32", h)], specialise)
    assert path == ("transpose_naive_f32" if specialise else "jit")
    assert np.array_equal(out.cpu().numpy(), ref)
    out.fill_(-1.0)
    path = run_ir(hip, "transpose_tiled", (16, 16, 1), ((w + 15) // 16, (h + 15) // 16, 1),
                  [dx, out, ("i32", w), ("i32", h)], specialise, shared_mem=272 * 4)
    assert path == ("transpose_tiled_f32" if specialise else "jit")
    assert np.array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("specialise", [1, 0])
@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (100, 72, 52), (33, 257, 129)])
def test_naive_matmul_ir(hip, oracle, torch_cuda, specialise, m, n, k):
    torch = torch_cuda
    a = oracle.fill_uniform(m * k, seed=0xA11CE, lo=-1, hi=1)
    b = oracle.fill_uniform(k * n, seed=0xB0B, lo=-1, hi=1)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    dc = torch.full((m * n,), float("nan"), device="cuda")
    path = run_ir(hip, "matrix_mul", (256, 1, 1), ((m * n + 255) // 256, 1, 1),
                  [da, db, dc, ("i32", m), ("i32", n), ("i32", k)], specialise)
    assert path == ("matmul_naive_f32" if specialise else "jit")
    ref = oracle.matmul_naive(a, b, m, n, k)
    # the f32 GEMM bound: 1e-4 * |A|inf |B|inf sqrt(K), operands in [-1, 1)
    assert np.abs(dc.cpu().numpy() - ref).max() <= 1e-4 * np.sqrt(k)


@pytest.mark.parametrize("name,size,path", [
    ("vector_add", 100003, "vector_add_f32"), ("vector_copy", 100003, "vector_copy_f32"),
    ("matrix_mul", 200, "matmul_naive_f32"), ("transpose", 200, "transpose_naive_f32"),
    ("transpose_tiled", 200, "transpose_tiled_f32"), ("scan", 256, "jit"), ("scan", 100, "jit")])
def test_reference_benchmarks_run_and_verify(hip, torch_cuda, name, size, path):
    """The mirrors of the five bench programs: the reference's inputs, geometry and checks, served
    by the hand kernels; and the same with the plain JIT lowering."""
    from spoc_amd import benchmarks
    fn = benchmarks.BENCHMARKS[name][0]
    rec = fn(size, warmup=1, iterations=3)
    assert rec["verified"] and rec["path"] == path and len(rec["iterations"]) == 3
    hip.check(hip.lib.sarek_hip_set_specialisation(0))
    try:
        rec = fn(size, warmup=1, iterations=2)
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    assert rec["verified"] and rec["path"] == "jit"


def test_result_file_has_the_reference_shape(hip, torch_cuda, tmp_path):
    """benchmarks/output.ml:66-90 and benchmarks/system_info.ml:202-236: what the result tools read."""
    from spoc_amd import benchmarks
    (rec,) = benchmarks.run("scan", sizes=[64], iterations=3)
    assert set(rec) == {"benchmark", "system", "results"}
    assert set(rec["benchmark"]) == {"name", "timestamp", "git_commit", "parameters"}
    assert rec["benchmark"]["name"] == "scan" and rec["benchmark"]["timestamp"].endswith("Z")
    assert rec["benchmark"]["parameters"] == {"size": 64, "block_size": 256, "iterations": 3, "warmup": 5}
    assert {"hostname", "os", "kernel", "cpu", "memory_gb", "devices"} <= set(rec["system"])
    assert set(rec["system"]["cpu"]) == {"model", "cores", "threads"}
    dev = rec["system"]["devices"][0]
    assert dev["framework"] == "HIP" and dev["memory_gb"] > 100 and dev["id"] == 0
    (r,) = rec["results"]
    assert {"device_id", "device_name", "framework", "iterations", "mean_ms", "stddev_ms", "median_ms", "min_ms",
            "max_ms", "throughput_gflops", "verified"} <= set(r)
    assert len(r["iterations"]) == 3 and r["verified"] is True
    (tiled,) = benchmarks.run("matrix_mul_tiled", sizes=[64], iterations=2, warmup=1)
    assert tiled["benchmark"]["parameters"]["block_size"] == 256          # tile_size squared
