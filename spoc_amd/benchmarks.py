"""The reference's benchmark programs for the hot path, run through the sarek-hip plugin.

Host-side mirror of benchmarks/bench_matrix_mul_tiled.ml, bench_stream_triad.ml,
bench_reduction.ml, bench_dot_product.ml, bench_reduction_max.ml, bench_vector_add.ml,
bench_vector_copy.ml, bench_matrix_mul.ml, bench_transpose.ml, bench_transpose_tiled.ml, bench_scan.ml,
bench_gather_scatter.ml, bench_histogram.ml, bench_stencil_2d.ml, bench_conv2d.ml, bench_mandelbrot.ml,
bench_nbody.ml, bench_bitonic_sort.ml and bench_radix_sort.ml (the whole suite): same inputs, same
launch geometry, same warmup / timed-iteration protocol (wall clock around the launch plus
the device flush, one sample per iteration), same verification and tolerance, same
throughput formula and statistic, and the same per-device result record
(benchmarks/output.ml:16-28).  The programs are written against Vector / Execute / Transfer
(spoc_amd/sarek.py) as the originals are: Vector.create + Vector.set for the inputs,
Execute.run_vectors ~ir ~args ~block ~grid per launch, Transfer.flush, Vector.to_array for the
check; the plugin decides whether a hand-written kernel or the JIT-compiled lowering serves a
launch (reported as `path`).

    python -m spoc_amd.benchmarks matrix_mul_tiled --sizes 1024,4096
    python -m spoc_amd.benchmarks all --json out.json
"""
import argparse
import ctypes as C
import json
import statistics
import time

import numpy as np

from . import hip, reference_kernels
from .sarek import Execute, Transfer, Vector


def _stats(times_ms):
    t = np.asarray(times_ms, dtype=np.float64)
    return dict(iterations=[float(x) for x in t], mean_ms=float(t.mean()),
                stddev_ms=float(t.std(ddof=1)) if len(t) > 1 else 0.0,
                median_ms=float(statistics.median(t)), min_ms=float(t.min()), max_ms=float(t.max()))


def _time_launches(launch, warmup, iterations):
    """benchmarks/bench_stream_triad.ml:76-116: warmup launches, then one wall-clock sample
    per Execute.run_vectors + Transfer.flush."""
    path = None
    for _ in range(warmup):
        path = launch()
        Transfer.flush()
    times = []
    for _ in range(iterations):
        t0 = time.perf_counter()
        path = launch()
        Transfer.flush()
        times.append((time.perf_counter() - t0) * 1e3)
    return times, path


def _device_record(times, throughput, verified, path, unit):
    info = hip.device_info(0)
    rec = dict(device_id=0, device_name=info.name.decode(), framework="HIP", **_stats(times))
    rec["throughput_gflops"] = throughput       # the reference's field name, whatever the unit
    rec["throughput_unit"] = unit
    rec["verified"] = bool(verified)
    rec["path"] = path
    return rec


def _vector(array, kind=None):
    """Vector.create + a loop of Vector.set, as the benches fill their inputs (in one call)."""
    kind = kind or Vector.float32
    v = Vector.create(kind, len(array))
    v.fill_from(array)
    return v


def bench_matrix_mul_tiled(size, warmup=5, iterations=20, tile_size=16):
    """benchmarks/bench_matrix_mul_tiled.ml:98-251: A[i] = (i mod 10)/10, B[i] = ((i+1) mod 10)/10,
    16x16 blocks over C, every element within 1e-3 of the double-precision product,
    GFLOPS = 2 m n k / median.

    The absolute 1e-3 check is the reference's, and from size 2048 on no f32 accumulation
    passes it: the inputs repeat with period 10 along k, so the rounding errors of a running
    f32 sum add up with one sign (sequential f32 as in the generated kernel, the vendor
    library and this backend all end 4.7e-3 off at 2048 and 1.1e-2 off at 4096, where the
    sums reach 1000)."""
    m = n = k = size
    a = (np.arange(m * k) % 10) / 10.0
    b = ((np.arange(k * n) + 1) % 10) / 10.0
    expected = a.reshape(m, k) @ b.reshape(k, n)              # float64, as ocaml_matmul
    va, vb = _vector(a), _vector(b)
    vc = Vector.create(Vector.float32, m * n)                 # never zeroed, as in the reference
    ir = reference_kernels.matrix_mul_tiled()
    block = Execute.dims2d(tile_size, tile_size)
    grid = Execute.dims2d((n + tile_size - 1) // tile_size, (m + tile_size - 1) // tile_size)
    args = [Execute.Vec(va), Execute.Vec(vb), Execute.Vec(vc), Execute.Int(m), Execute.Int(n), Execute.Int(k)]
    times, path = _time_launches(
        lambda: Execute.run_vectors(ir=ir, args=args, block=block, grid=grid, shared_mem=2 * tile_size * tile_size * 4),
        warmup, iterations)
    verified = bool(np.all(np.abs(vc.to_array().astype(np.float64).reshape(m, n) - expected) <= 1e-3))
    gflops = 2.0 * m * n * k / (statistics.median(times) * 1e6)
    return _device_record(times, gflops, verified, path, "GFLOPS")


def bench_stream_triad(size, warmup=5, iterations=20, block_size=256):
    """benchmarks/bench_stream_triad.ml:35-181: b[i] = (i mod 100)/100, c[i] = ((i+1) mod 100)/100,
    scalar 3, every element within 1e-5, GB/s = 12 n / median."""
    n = size
    b = (np.arange(n) % 100) / 100.0
    c = ((np.arange(n) + 1) % 100) / 100.0
    expected = b + c * 3.0
    va, vb, vc = Vector.create(Vector.float32, n), _vector(b), _vector(c)
    ir = reference_kernels.stream_triad()
    block, grid = Execute.dims1d(block_size), Execute.dims1d((n + block_size - 1) // block_size)
    args = [Execute.Vec(va), Execute.Vec(vb), Execute.Vec(vc), Execute.Float32(3.0), Execute.Int(n)]
    times, path = _time_launches(lambda: Execute.run_vectors(ir=ir, args=args, block=block, grid=grid),
                                 warmup, iterations)
    verified = bool(np.all(np.abs(va.to_array().astype(np.float64) - expected) <= 1e-5))
    gbs = 3.0 * n * 4.0 / (statistics.median(times) / 1e3 * 1e9)
    return _device_record(times, gbs, verified, path, "GB/s")


def _tree_bench(ir, inputs, n, expected, check, bytes_moved, stat, warmup, iterations, fold=np.sum):
    nblocks = (n + 255) // 256
    vins = [_vector(x) for x in inputs]
    vout = Vector.create(Vector.float32, nblocks)
    args = [Execute.Vec(v) for v in vins] + [Execute.Vec(vout), Execute.Int(n)]
    times, path = _time_launches(
        lambda: Execute.run_vectors(ir=ir, args=args, block=Execute.dims1d(256), grid=Execute.dims1d(nblocks),
                                    shared_mem=1024),
        warmup, iterations)
    result = float(fold(vout.to_array().astype(np.float64)))   # host fold over the partials
    verified = check(result, expected)
    t = statistics.mean(times) if stat == "mean" else statistics.median(times)
    return _device_record(times, bytes_moved / (t / 1e3) / 1e9, verified, path, "GB/s")


def bench_reduction(size, warmup=10, iterations=20):
    """benchmarks/bench_reduction.ml:98-215: all ones, sum of the per-block partials within
    1e-3 relative of n, GB/s = 4 n * 1.004 / mean."""
    n = size
    return _tree_bench(reference_kernels.tree(False), [np.ones(n)], n, float(n),
                       lambda r, e: abs(r - e) / e < 1e-3, 4.0 * n * 1.004, "mean", warmup, iterations)


def bench_dot_product(size, warmup=5, iterations=20):
    """benchmarks/bench_dot_product.ml:56-160: a[i] = (i mod 100)/100, b[i] = ((i+1) mod 100)/100,
    |result - expected| < 1e-3 * expected, GB/s = 8 n / median."""
    n = size
    a = (np.arange(n) % 100) / 100.0
    b = ((np.arange(n) + 1) % 100) / 100.0
    return _tree_bench(reference_kernels.tree(True), [a, b], n, float(np.dot(a, b)),
                       lambda r, e: abs(r - e) < 1e-3 * e, 8.0 * n, "median", warmup, iterations)


def bench_reduction_max(size, warmup=5, iterations=20):
    """benchmarks/bench_reduction_max.ml:88-190: input[i] = i mod 10000, maximum of the
    per-block results within 1e-5 of the maximum of the input, GB/s = 4 n / median."""
    n = size
    x = (np.arange(n) % 10000).astype(np.float64)
    return _tree_bench(reference_kernels.reduction_max(-1000000.0), [x], n, float(x.max()),
                       lambda r, e: abs(r - e) < 1e-5, 4.0 * n, "median", warmup, iterations, fold=np.max)


def _benchmark_gpu(init, compute, warmup, iterations):
    """benchmarks/common.ml:200-237 (Common.benchmark_gpu): vectors from init (), one launch to
    compile, `warmup` launches, FRESH vectors from init () again, then `iterations` samples of
    device-idle -> launch -> device-idle.  The fresh vectors are uploaded inside the first timed
    sample, in the reference as here (its statistics are the mean or the minimum of the samples)."""
    kernel_args = init()
    path = compute(kernel_args)
    Transfer.flush()
    for _ in range(warmup):
        compute(kernel_args)
        Transfer.flush()
    kernel_args = init()
    times = []
    for _ in range(iterations):
        Transfer.flush()
        t0 = time.perf_counter()
        path = compute(kernel_args)
        Transfer.flush()
        times.append((time.perf_counter() - t0) * 1e3)
    return times, path, kernel_args


def bench_vector_add(size, warmup=10, iterations=20):
    """benchmarks/bench_vector_add.ml:53-150: a[i] = 0.001 i, b[i] = 0.002 i, every element within
    1e-3 of the double sum, GB/s = 12 n / MINIMUM time."""
    n = size
    a, b = np.arange(n) * 0.001, np.arange(n) * 0.002
    ir = reference_kernels.vector_add()
    block, grid = Execute.dims1d(256), Execute.dims1d((n + 255) // 256)

    def compute(v):
        return Execute.run_vectors(ir=ir, args=[Execute.Vec(v[0]), Execute.Vec(v[1]), Execute.Vec(v[2]), Execute.Int(n)],
                                   block=block, grid=grid)
    times, path, (_, _, vc) = _benchmark_gpu(lambda: (_vector(a), _vector(b), Vector.create(Vector.float32, n)),
                                             compute, warmup, iterations)
    verified = bool(np.all(np.abs(vc.to_array().astype(np.float64) - (a + b)) <= 1e-3))
    return _device_record(times, 12.0 * n / (min(times) / 1e3) / 1e9, verified, path, "GB/s")


def bench_vector_copy(size, warmup=5, iterations=20, block_size=256):
    """benchmarks/bench_vector_copy.ml:21-170: a[i] = (i mod 100)/100, every element within 1e-6,
    GB/s = 8 n / median (launch + flush per sample)."""
    n = size
    a = (np.arange(n) % 100) / 100.0
    va, vb = _vector(a), Vector.create(Vector.float32, n)
    ir = reference_kernels.vector_copy()
    block, grid = Execute.dims1d(block_size), Execute.dims1d((n + block_size - 1) // block_size)
    args = [Execute.Vec(va), Execute.Vec(vb), Execute.Int(n)]
    times, path = _time_launches(lambda: Execute.run_vectors(ir=ir, args=args, block=block, grid=grid),
                                 warmup, iterations)
    verified = bool(np.all(np.abs(vb.to_array().astype(np.float64) - a) <= 1e-6))
    return _device_record(times, 8.0 * n / (statistics.median(times) / 1e3) / 1e9, verified, path, "GB/s")


def bench_matrix_mul(size, warmup=10, iterations=20, block_size=256):
    """benchmarks/bench_matrix_mul.ml:43-165: one thread per element of C, inputs as the tiled
    bench, every element within 1e-3 of the double product, GFLOPS = 2 m n k / MEAN."""
    m = n = k = size
    a = (np.arange(m * k) % 10) / 10.0
    b = ((np.arange(k * n) + 1) % 10) / 10.0
    expected = a.reshape(m, k) @ b.reshape(k, n)
    ir = reference_kernels.matrix_mul()
    block, grid = Execute.dims1d(block_size), Execute.dims1d((m * n + block_size - 1) // block_size)

    def compute(v):
        return Execute.run_vectors(ir=ir, args=[Execute.Vec(v[0]), Execute.Vec(v[1]), Execute.Vec(v[2]),
                                                Execute.Int(m), Execute.Int(n), Execute.Int(k)], block=block, grid=grid)
    times, path, (_, _, vc) = _benchmark_gpu(lambda: (_vector(a), _vector(b), Vector.create(Vector.float32, m * n)),
                                             compute, warmup, iterations)
    verified = bool(np.all(np.abs(vc.to_array().astype(np.float64).reshape(m, n) - expected) <= 1e-3))
    return _device_record(times, 2.0 * m * n * k / (statistics.mean(times) * 1e6), verified, path, "GFLOPS")


def _bench_transpose(ir, block, grid_of, size, warmup, iterations):
    """benchmarks/bench_transpose.ml:100-210 / bench_transpose_tiled.ml:120-240: input[i] = i, output
    zeroed, square size x size, tolerance 1e-3 (10 beyond 2^24 elements), GB/s = 8 n / MEAN."""
    m = size
    n = m * m
    data = np.arange(n, dtype=np.float64)
    grid = grid_of(m)

    def compute(v):
        return Execute.run_vectors(ir=ir, args=[Execute.Vec(v[0]), Execute.Vec(v[1]), Execute.Int(m), Execute.Int(m)],
                                   block=block, grid=grid)
    times, path, (_, vout) = _benchmark_gpu(lambda: (_vector(data), _vector(np.zeros(n))), compute, warmup, iterations)
    tolerance = 10.0 if n > 16_777_216 else 0.001
    expected = data.reshape(m, m).T.reshape(-1)
    verified = bool(np.all(np.abs(vout.to_array().astype(np.float64) - expected) <= tolerance))
    return _device_record(times, 8.0 * n / (statistics.mean(times) / 1e3) / 1e9, verified, path, "GB/s")


def bench_transpose(size, warmup=10, iterations=20):
    return _bench_transpose(reference_kernels.transpose_naive(), Execute.dims1d(256),
                            lambda m: Execute.dims1d((m * m + 255) // 256), size, warmup, iterations)


def bench_transpose_tiled(size, warmup=10, iterations=20, tile_size=16):
    return _bench_transpose(reference_kernels.transpose_tiled(), Execute.dims2d(tile_size, tile_size),
                            lambda m: Execute.dims2d((m + tile_size - 1) // tile_size, (m + tile_size - 1) // tile_size),
                            size, warmup, iterations)


def bench_scan(size, warmup=5, iterations=20):
    """benchmarks/bench_scan.ml:112-221: inclusive prefix sum of [1..n] in one 256-thread block
    (n = min(size, 256)), every element equal to the serial prefix sum, M elements/s = n / median."""
    n = min(size, 256)
    data = np.arange(1, n + 1, dtype=np.int32)
    vin, vout = _vector(data, Vector.int32), Vector.create(Vector.int32, n)
    ir = reference_kernels.inclusive_scan()
    args = [Execute.Vec(vin), Execute.Vec(vout), Execute.Int32(n)]
    times, path = _time_launches(
        lambda: Execute.run_vectors(ir=ir, args=args, block=Execute.dims1d(256), grid=Execute.dims1d(1)),
        warmup, iterations)
    verified = bool(np.array_equal(vout.to_array(), np.cumsum(data, dtype=np.int32)))
    return _device_record(times, n / (statistics.median(times) / 1e3 * 1e6), verified, path, "Melem/s")


def _ocaml_random_ints(n, bound, seed=42):
    """Stand-in for `Random.init 42; Random.int bound`: OCaml's generator is not available here, so
    the values differ from the reference's while the distribution (uniform on [0, bound)) is the same."""
    return np.random.default_rng(seed).integers(0, bound, n).astype(np.int32)


def bench_gather(size, warmup=5, iterations=20):
    """benchmarks/bench_gather_scatter.ml:76-199: input[i] = 2 i, random indices, output[i] =
    input[indices[i]] exactly, M elements/s = n / median."""
    n = size
    data, idx = np.arange(n, dtype=np.int64) * 2, _ocaml_random_ints(n, n)
    vin, vidx, vout = _vector(data, Vector.int32), _vector(idx, Vector.int32), Vector.create(Vector.int32, n)
    ir = reference_kernels.gather()
    args = [Execute.Vec(vin), Execute.Vec(vidx), Execute.Vec(vout), Execute.Int32(n)]
    times, path = _time_launches(
        lambda: Execute.run_vectors(ir=ir, args=args, block=Execute.dims1d(256), grid=Execute.dims1d((n + 255) // 256)),
        warmup, iterations)
    verified = bool(np.array_equal(vout.to_array(), data.astype(np.int32)[idx]))
    return _device_record(times, n / (statistics.median(times) / 1e3 * 1e6), verified, path, "Melem/s")


def bench_scatter(size, warmup=5, iterations=20):
    """benchmarks/bench_gather_scatter.ml:202-340: input[i] = 3 i + 1, random (colliding) indices,
    output zeroed with Vector.set before every launch; every output element is 0 or one of the
    inputs.  After the first launch the output vector is Stale_CPU, and a host write into a
    Stale_CPU vector is not tracked (sarek/core/Vector.ml:104-109): the zeros of the later
    iterations stay on the host and the device keeps scattering over its earlier results, in the
    reference as here, so no upload falls into the timed samples."""
    n = size
    data, idx = (np.arange(n, dtype=np.int64) * 3 + 1).astype(np.int32), _ocaml_random_ints(n, n)
    vin, vidx, vout = _vector(data, Vector.int32), _vector(idx, Vector.int32), _vector(np.zeros(n), Vector.int32)
    ir = reference_kernels.scatter()
    args = [Execute.Vec(vin), Execute.Vec(vidx), Execute.Vec(vout), Execute.Int32(n)]
    zeros = np.zeros(n, dtype=np.int32)

    def one():
        return Execute.run_vectors(ir=ir, args=args, block=Execute.dims1d(256), grid=Execute.dims1d((n + 255) // 256))
    path = None
    for _ in range(warmup):
        vout.fill_from(zeros)
        path = one()
        Transfer.flush()
    times = []
    for _ in range(iterations):
        vout.fill_from(zeros)
        t0 = time.perf_counter()
        path = one()
        Transfer.flush()
        times.append((time.perf_counter() - t0) * 1e3)
    got = vout.to_array()
    verified = bool(np.all((got == 0) | ((got % 3 == 1) & (got >= 1) & (got <= 3 * (n - 1) + 1))))
    # stronger than the reference's membership check: a written slot holds an input that was sent there
    written = got != 0
    verified = verified and bool(np.array_equal(idx[(got[written] - 1) // 3], np.nonzero(written)[0]))
    return _device_record(times, n / (statistics.median(times) / 1e3 * 1e6), verified, path, "Melem/s")


def bench_histogram(size, warmup=5, iterations=20):
    """benchmarks/bench_histogram.ml:86-210: random values in [0, 256), 256 bins, a fresh zeroed
    histogram vector per timed launch, exact counts, M elements/s = n / median."""
    n, bins = size, 256
    data = _ocaml_random_ints(n, bins)
    vin = _vector(data, Vector.int32)
    ir = reference_kernels.histogram()
    block, grid = Execute.dims1d(256), Execute.dims1d((n + 255) // 256)

    def launch(hist):
        return Execute.run_vectors(ir=ir, args=[Execute.Vec(vin), Execute.Vec(hist), Execute.Int32(n), Execute.Int32(bins)],
                                   block=block, grid=grid, shared_mem=bins * 4)
    hist = Vector.create(Vector.int32, bins)
    for _ in range(warmup):
        hist.fill_from(np.zeros(bins))
        path = launch(hist)
        Transfer.flush()
    times = []
    for _ in range(iterations):
        hist = _vector(np.zeros(bins), Vector.int32)
        t0 = time.perf_counter()
        path = launch(hist)
        Transfer.flush()
        times.append((time.perf_counter() - t0) * 1e3)
    verified = bool(np.array_equal(hist.to_array(), np.bincount(data, minlength=bins)))
    return _device_record(times, n / (statistics.median(times) / 1e3 * 1e6), verified, path, "Melem/s")


def _grid_bench(ir, block, grid, size, data, expected, tolerance, warmup, iterations):
    """The loop of bench_stencil_2d.ml:110-150 / bench_conv2d.ml:133-172: warmup launches without a
    flush between them, one flush, then launch + flush per sample; interior cells within `tolerance`."""
    n = size * size
    vin, vout = _vector(data), _vector(np.zeros(n))
    args = [Execute.Vec(vin), Execute.Vec(vout), Execute.Int32(size), Execute.Int32(size)]
    path = None
    for _ in range(warmup):
        path = Execute.run_vectors(ir=ir, args=args, block=block, grid=grid)
    Transfer.flush()
    times = []
    for _ in range(iterations):
        t0 = time.perf_counter()
        path = Execute.run_vectors(ir=ir, args=args, block=block, grid=grid)
        Transfer.flush()
        times.append((time.perf_counter() - t0) * 1e3)
    got = vout.to_array().astype(np.float64).reshape(size, size)
    verified = bool(np.all(np.abs(got[1:-1, 1:-1] - expected[1:-1, 1:-1]) <= tolerance))
    return _device_record(times, n / (statistics.median(times) / 1e3) / 1e6, verified, path, "Mcell/s")


def bench_stencil_2d(size, warmup=5, iterations=20):
    """benchmarks/bench_stencil_2d.ml:60-180: input sin(0.1 x) cos(0.1 y), 16x16 blocks, interior
    within 1e-4 of the double five-point mean, M cells/s = n / median."""
    g = np.arange(size, dtype=np.float64)
    data = (np.sin(g * 0.1)[None, :] * np.cos(g * 0.1)[:, None])
    f = data.astype(np.float32).astype(np.float64)
    expected = np.zeros_like(f)
    expected[1:-1, 1:-1] = (f[:-2, 1:-1] + f[2:, 1:-1] + f[1:-1, :-2] + f[1:-1, 2:] + f[1:-1, 1:-1]) / 5.0
    tiles = (size + 15) // 16
    return _grid_bench(reference_kernels.stencil_2d(), Execute.dims2d(16, 16), Execute.dims2d(tiles, tiles), size,
                       data.reshape(-1), expected, 1e-4, warmup, iterations)


def bench_conv2d(size, warmup=5, iterations=20):
    """benchmarks/bench_conv2d.ml:79-212: input ((x + y) mod 256)/255, 3x3 box filter, one thread per
    pixel, interior within 1e-3, M pixels/s = n / median."""
    g = np.arange(size)
    data = ((g[None, :] + g[:, None]) % 256) / 255.0
    f = data.astype(np.float32).astype(np.float64)
    expected = np.zeros_like(f)
    for dy in (0, 1, 2):
        for dx in (0, 1, 2):
            expected[1:-1, 1:-1] += f[dy:size - 2 + dy, dx:size - 2 + dx] / 9.0
    n = size * size
    return _grid_bench(reference_kernels.conv2d(), Execute.dims1d(256), Execute.dims1d((n + 255) // 256), size,
                       data.reshape(-1), expected, 1e-3, warmup, iterations)


def bench_mandelbrot(size, warmup=10, iterations=20, max_iterations=256):
    """benchmarks/bench_mandelbrot.ml:112-225: size x size image, 16x16 blocks, the first 1001 pixels
    within 10 iterations of the float recurrence, M pixels/s = pixels / MEAN."""
    width = height = size
    n = width * height
    ir = reference_kernels.mandelbrot()
    tiles = (size + 15) // 16
    block, grid = Execute.dims2d(16, 16), Execute.dims2d(tiles, tiles)

    def compute(v):
        return Execute.run_vectors(ir=ir, args=[Execute.Vec(v), Execute.Int(width), Execute.Int(height),
                                                Execute.Int(max_iterations)], block=block, grid=grid)
    times, path, vout = _benchmark_gpu(lambda: _vector(np.zeros(n), Vector.int32), compute, warmup, iterations)
    head = min(1001, n)
    px = (np.arange(head) % width).astype(np.float64)
    py = (np.arange(head) // width).astype(np.float64)
    x0, y0 = 4.0 * (px / width) - 2.5, 3.0 * (py / height) - 1.5
    x, y, it = np.zeros(head), np.zeros(head), np.zeros(head, dtype=np.int64)
    for _ in range(max_iterations):
        live = (x * x + y * y <= 4.0) & (it < max_iterations)
        x, y = np.where(live, x * x - y * y + x0, x), np.where(live, 2.0 * x * y + y0, y)
        it += live
    verified = bool(np.all(np.abs(vout.to_array()[:head].astype(np.int64) - it) <= 10))
    return _device_record(times, n / (statistics.mean(times) / 1e3) / 1e6, verified, path, "Mpixel/s")


def bench_nbody(size, warmup=5, iterations=20):
    """benchmarks/bench_nbody.ml:107-235: positions (i mod 7, i mod 5, i mod 3)/10, blocks of 64,
    accelerations against the double all-pairs sum (off by more than 1e-3 both absolutely and
    relatively counts as an error), G interactions/s = n^2 / median.

    From 4096 bodies on that check fails for any kernel that accumulates in f32 in j order, as the
    generated code does: the lattice repeats every 105 bodies, single terms reach 1e3 and the net
    force on some bodies is below 1 after cancellation; a numpy emulation of the f32 loop counts
    273 such bodies at 4096 (largest difference 0.23 on sums of magnitude 3e4) and none at 2048."""
    n = size
    i = np.arange(n)
    pos = [(i % 7) / 10.0, (i % 5) / 10.0, (i % 3) / 10.0]
    vpos = [_vector(p) for p in pos]
    vacc = [_vector(np.zeros(n)) for _ in range(3)]
    ir = reference_kernels.nbody_accel()
    args = [Execute.Vec(v) for v in vpos + vacc] + [Execute.Int32(n)]
    block, grid = Execute.dims1d(64), Execute.dims1d((n + 63) // 64)
    path = None
    for _ in range(warmup):
        path = Execute.run_vectors(ir=ir, args=args, block=block, grid=grid)
    Transfer.flush()
    times = []
    for _ in range(iterations):
        t0 = time.perf_counter()
        path = Execute.run_vectors(ir=ir, args=args, block=block, grid=grid)
        Transfer.flush()
        times.append((time.perf_counter() - t0) * 1e3)
    p = np.stack(pos)                                # doubles, as cpu_nbody takes them
    verified = True
    for lo in range(0, n, 512):                      # rows of the pair matrix in slabs
        rows = np.arange(lo, min(lo + 512, n))
        d = p[:, None, :] - p[:, rows, None]
        dist2 = (d ** 2).sum(0) + 1e-9
        w = 1.0 / (np.sqrt(dist2) * dist2)
        w[rows - lo, rows] = 0.0                     # j <> i
        exp = (d * w[None]).sum(2)
        for c in range(3):
            diff = np.abs(vacc[c].to_array()[rows].astype(np.float64) - exp[c])
            verified = verified and not bool(np.any((diff > 1e-3) & (diff / (np.abs(exp[c]) + 1e-9) > 1e-3)))
    return _device_record(times, float(n) * n / (statistics.median(times) / 1e3) / 1e9, verified, path,
                          "Ginteraction/s")


def bench_bitonic_sort(size, warmup=5, iterations=20):
    """benchmarks/bench_bitonic_sort.ml:58-215: n = the power of two at or below size, random values
    below 10000 written again with Vector.set before every sort, log^2 n launches per sort, result
    equal to the sorted input, M elements/s = n / median.  Only the first sort sees the random
    values: after it the vector is Stale_CPU and host writes into it are not tracked
    (sarek/core/Vector.ml:104-109), so the later sorts run over the sorted device copy, in the
    reference as here (the network does the same work whatever the data)."""
    n = 1 << int(np.log2(size))
    data = _ocaml_random_ints(n, 10000)
    v = _vector(data, Vector.int32)
    ir = reference_kernels.bitonic_sort_step()
    block, grid = Execute.dims1d(256), Execute.dims1d((n + 255) // 256)

    def sort():
        path, k = None, 2
        while k <= n:
            j = k // 2
            while j >= 1:
                path = Execute.run_vectors(ir=ir, args=[Execute.Vec(v), Execute.Int32(j), Execute.Int32(k),
                                                        Execute.Int32(n)], block=block, grid=grid)
                j //= 2
            k *= 2
        return path
    path = None
    for _ in range(warmup):
        v.fill_from(data)
        path = sort()
        Transfer.flush()
    times = []
    for _ in range(iterations):
        v.fill_from(data)
        t0 = time.perf_counter()
        path = sort()
        Transfer.flush()
        times.append((time.perf_counter() - t0) * 1e3)
    verified = bool(np.array_equal(v.to_array(), np.sort(data)))
    return _device_record(times, n / (statistics.median(times) / 1e3 * 1e6), verified, path, "Melem/s")


def bench_radix_sort(size, warmup=5, iterations=20):
    """benchmarks/bench_radix_sort.ml:118-350: ONE 8-bit pass (the reference's `_num_passes = 1`):
    per-block histogram kernel, histogram back to the host, exclusive prefix sum there, counters up,
    scatter kernel with atomic slot allocation; the output must be ordered by its low 8 bits;
    M elements/s = n / median of the whole pass, uploads included."""
    n, bins, mask, shift = size, 256, 255, 0
    data = _ocaml_random_ints(n, 100000)
    hist_ir, scatter_ir = reference_kernels.radix_sort_histogram(), reference_kernels.radix_sort_scatter()
    block, grid = Execute.dims1d(256), Execute.dims1d((n + 255) // 256)

    def init():
        return (_vector(data, Vector.int32), Vector.create(Vector.int32, n), Vector.create(Vector.int32, bins),
                Vector.create(Vector.int32, bins))

    def compute(vs):
        vin, vout, hist, counters = vs
        vin.fill_from(data)
        Transfer.to_device(vin)
        hist.fill_from(np.zeros(bins))
        Transfer.to_device(hist)
        Execute.run_vectors(ir=hist_ir, args=[Execute.Vec(vin), Execute.Vec(hist), Execute.Int32(n), Execute.Int32(shift),
                                              Execute.Int32(mask)], block=block, grid=grid)
        Transfer.flush()
        Transfer.to_cpu(hist, force=True)
        h = hist.to_array().astype(np.int64)
        counters.fill_from(np.concatenate(([0], np.cumsum(h)[:-1])))
        Transfer.to_device(counters)
        path = Execute.run_vectors(ir=scatter_ir, args=[Execute.Vec(vin), Execute.Vec(vout), Execute.Vec(counters),
                                                        Execute.Int32(n), Execute.Int32(shift), Execute.Int32(mask)],
                                   block=block, grid=grid)
        Transfer.flush()
        Transfer.to_cpu(counters, force=True)
        return path
    times, path, (_, vout, _, _) = _benchmark_gpu(init, compute, warmup, iterations)
    Transfer.to_cpu(vout, force=True)
    out = vout.to_array()
    verified = bool(np.all(np.diff(out & 255) >= 0)) and bool(np.array_equal(np.sort(out), np.sort(data)))
    return _device_record(times, n / (statistics.median(times) / 1e3 * 1e6), verified, path, "Melem/s")


def bench_transfer(size, warmup=2, iterations=7):
    """Not one of the reference's programs: the Transfer.to_device / Transfer.to_cpu legs
    (sarek/core/Transfer.ml:228-333) that its benches run once before and after their timed
    loops, timed alone for a float32 vector of `size` elements in ordinary (pageable) host
    memory.  Throughput is the upload rate; the record also carries the download rate and
    both rates of the driver's own copy."""
    host = (np.arange(size) % 100 / 100.0).astype(np.float32)
    v = _vector(host)
    Transfer.to_device(v)                 # allocates the device block; later uploads reuse it

    def upload():
        v[0] = host[0]                    # Vector.set: Both -> Stale_GPU, so to_device copies again
        Transfer.to_device(v)

    def timed(fn):
        for _ in range(warmup):
            fn()
        ts = []
        for _ in range(iterations):
            t0 = time.perf_counter()
            fn()
            Transfer.flush()
            ts.append((time.perf_counter() - t0) * 1e3)
        return ts
    rates = {}
    for label, threads in (("driver", 0), ("staged", None)):
        if threads is not None:
            hip.set_tunable("transfer.threads", threads)
        up = timed(upload)
        v.host[:] = -1.0                  # behind the vector's back: the download has to restore it
        down = timed(lambda: Transfer.to_cpu(v, force=True))
        hip.set_tunable("transfer.threads", 4)
        rates[label] = (up, down)
    back = v.host
    gbs = lambda ts: host.nbytes / (statistics.median(ts) / 1e3) / 1e9
    rec = _device_record(rates["staged"][0], gbs(rates["staged"][0]), np.array_equal(back, host),
                         "Transfer.to_device", "GB/s")
    rec["download_gbs"] = gbs(rates["staged"][1])
    rec["driver_copy_upload_gbs"] = gbs(rates["driver"][0])
    rec["driver_copy_download_gbs"] = gbs(rates["driver"][1])
    return rec


BENCHMARKS = {
    # name: (function, the reference's default sizes)
    "matrix_mul_tiled": (bench_matrix_mul_tiled, [128, 256, 512, 1024, 2048, 4096]),
    "stream_triad": (bench_stream_triad, [1_000_000, 10_000_000, 50_000_000, 100_000_000, 500_000_000]),
    "reduction": (bench_reduction, [1_000_000, 10_000_000, 50_000_000, 100_000_000]),   # warmup 10 there
    "dot_product": (bench_dot_product, [1_000_000, 10_000_000, 50_000_000, 100_000_000]),
    "reduction_max": (bench_reduction_max, [1_000_000, 10_000_000, 50_000_000, 100_000_000]),
    "vector_add": (bench_vector_add, [1_000_000, 10_000_000, 50_000_000, 100_000_000]),      # warmup 10
    "vector_copy": (bench_vector_copy, [1_000_000, 10_000_000, 50_000_000, 100_000_000, 500_000_000]),
    "matrix_mul": (bench_matrix_mul, [256, 512, 1024, 2048]),                               # warmup 10
    "transpose": (bench_transpose, [256, 512, 1024, 2048, 4096, 8192]),                     # warmup 10
    "transpose_tiled": (bench_transpose_tiled, [256, 512, 1024, 2048, 4096, 8192]),         # warmup 10
    "scan": (bench_scan, [64, 128, 256]),
    "gather": (bench_gather, [1_000_000, 10_000_000, 50_000_000]),          # bench_gather_scatter.ml, first half
    "scatter": (bench_scatter, [1_000_000, 10_000_000, 50_000_000]),        # second half
    "histogram": (bench_histogram, [1_000_000, 10_000_000, 50_000_000]),
    "stencil_2d": (bench_stencil_2d, [256, 512, 1024, 2048]),
    "conv2d": (bench_conv2d, [256, 512, 1024, 2048]),
    "mandelbrot": (bench_mandelbrot, [512, 1024, 2048, 4096]),              # warmup 10
    "nbody": (bench_nbody, [512, 1024, 2048, 4096]),
    "bitonic_sort": (bench_bitonic_sort, [1024, 4096, 16384]),
    "radix_sort": (bench_radix_sort, [1_000_000, 10_000_000, 50_000_000]),
    "transfer": (bench_transfer, [1_000_000, 10_000_000, 100_000_000, 268_435_456]),   # no such program there
}


def _first_line(cmd, default="unknown"):
    import subprocess
    try:
        out = subprocess.run(cmd, shell=True, capture_output=True, text=True, timeout=10).stdout.splitlines()
        return out[0].strip() if out and out[0].strip() else default
    except Exception:
        return default


def system_info():
    """benchmarks/system_info.ml:22-236: host name, OS, kernel, CPU model / cores / threads, memory
    and the devices, in the shape its to_json writes."""
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    threads = int(_first_line("nproc", "1"))
    cores = max(1, threads // 2)
    try:
        import subprocess
        cps = sockets = None
        for line in subprocess.run("lscpu 2>/dev/null", shell=True, capture_output=True, text=True).stdout.splitlines():
            if line.startswith("Core(s) per socket"):
                cps = int(line.split(":")[1])
            elif line.startswith("Socket(s)"):
                sockets = int(line.split(":")[1])
        if cps and sockets:
            cores = cps * sockets
    except Exception:
        pass
    try:
        memory_gb = float(_first_line("free -b | grep Mem | awk '{print $2}'", "0")) / 2 ** 30
    except ValueError:
        memory_gb = 0.0
    info = hip.device_info(0)
    version = C.c_int(0)
    hip.check(hip.lib.sarek_hip_driver_version(C.byref(version)))
    device = {"driver_version": str(version.value), "compute_capability": f"{info.compute_major}.{info.compute_minor}",
              "id": 0, "name": info.name.decode(), "framework": "HIP", "memory_gb": info.total_global_mem / 2 ** 30}
    return {"hostname": _first_line("hostname"), "os": _first_line("uname -s"), "kernel": _first_line("uname -r"),
            "cpu": {"model": model, "cores": cores, "threads": threads}, "memory_gb": memory_gb, "devices": [device]}


def result_record(name, size, block_size, iterations, warmup, device_results, system=None):
    """benchmarks/output.ml:66-90 (Output.to_json): the file the reference's result tools read."""
    import subprocess
    commit = _first_line("git rev-parse HEAD 2>/dev/null", "")
    return {"benchmark": {"name": name, "timestamp": time.strftime("%Y-%m-%dT%H:%M:%SZ", time.gmtime()),
                          "git_commit": commit or None,
                          "parameters": {"size": size, "block_size": block_size, "iterations": iterations,
                                         "warmup": warmup}},
            "system": system if system is not None else system_info(),
            "results": [r for r in device_results                                  # Output.filter_valid_results
                        if r["iterations"] and not (r["median_ms"] == 0.0 and r["verified"] is False)]}


def run(name, sizes=None, warmup=None, iterations=20):
    fn, default_sizes = BENCHMARKS[name]
    out = []
    system = system_info()
    for size in sizes or default_sizes:
        kw = {} if warmup is None else {"warmup": warmup}
        rec = fn(size, iterations=iterations, **kw)
        print(f"  Device: {rec['device_name']} (HIP), Size: {size}")
        print(f"  Mean: {rec['mean_ms']:.3f} ms, Median: {rec['median_ms']:.3f} ms, "
              f"StdDev: {rec['stddev_ms']:.3f} ms")
        print(f"  Throughput: {rec['throughput_gflops']:.3f} {rec['throughput_unit']}  [{rec['path']}]")
        if "download_gbs" in rec:
            print(f"  Download: {rec['download_gbs']:.3f} GB/s; driver's own copy: "
                  f"{rec['driver_copy_upload_gbs']:.3f} up, {rec['driver_copy_download_gbs']:.3f} down")
        print(f"  Verified: {'✓' if rec['verified'] else '✗'}", flush=True)
        import inspect
        defaults = {k: p.default for k, p in inspect.signature(fn).parameters.items()}
        block = defaults.get("block_size", defaults.get("tile_size", 256))
        out.append(result_record(name, size, block * block if "tile_size" in defaults else block, iterations,
                                 warmup if warmup is not None else defaults.get("warmup"), [rec], system))
    return out


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("benchmark", choices=list(BENCHMARKS) + ["all"])
    ap.add_argument("--sizes", default=None, help="comma separated; default: the reference's own list")
    ap.add_argument("--iterations", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=None, help="default: 5 (reduction: 10), as the reference")
    ap.add_argument("--json", default=None, help="write the result records to this file")
    args = ap.parse_args()
    sizes = [int(s) for s in args.sizes.split(",")] if args.sizes else None
    names = list(BENCHMARKS) if args.benchmark == "all" else [args.benchmark]
    results = []
    for name in names:
        print(f"{name} benchmark")
        results += run(name, sizes, args.warmup, args.iterations)
    if args.json:
        with open(args.json, "w") as f:
            json.dump(results, f, indent=1)


if __name__ == "__main__":
    main()
