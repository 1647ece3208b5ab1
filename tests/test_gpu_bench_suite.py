"""The rest of the reference's benchmark suite through the plugin
(benchmarks/bench_gather_scatter.ml, bench_histogram.ml, bench_stencil_2d.ml, bench_conv2d.ml,
bench_mandelbrot.ml, bench_nbody.ml, bench_bitonic_sort.ml, bench_radix_sort.ml): each mirror
builds the reference's inputs, launches with its geometry and applies its own check, so a
passing run says the lowering computes what the bench expects at sizes with ragged last blocks,
colliding scatters, atomics in shared and global memory, records and helper functions; the stencil
and the box filter run both ways, hand kernel and generated code."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,size", [
    ("gather", 100003), ("scatter", 100003),
    ("stencil_2d", 200), ("conv2d", 200), ("conv2d", 37), ("mandelbrot", 100), ("nbody", 300),
    ("bitonic_sort", 1024), ("bitonic_sort", 3000)])
def test_suite_runs_and_verifies(hip, torch_cuda, name, size):
    from spoc_amd import benchmarks
    rec = benchmarks.BENCHMARKS[name][0](size, warmup=1, iterations=3)
    assert rec["verified"], rec
    hand = {"stencil_2d": "stencil_2d_f32", "conv2d": "conv2d_f32"}
    assert rec["path"] == hand.get(name, "jit") and len(rec["iterations"]) == 3 and rec["throughput_gflops"] > 0
    if name in hand:
        hip.check(hip.lib.sarek_hip_set_specialisation(0))
        try:
            rec = benchmarks.BENCHMARKS[name][0](size, warmup=1, iterations=2)
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
        assert rec["verified"] and rec["path"] == "jit"


def test_suite_is_the_reference_suite():
    """benchmarks/ holds 19 bench_*.ml programs; gather and scatter
    share one of them, transfer is this build's addition."""
    from spoc_amd import benchmarks
    assert set(benchmarks.BENCHMARKS) == {
        "matrix_mul_tiled", "stream_triad", "reduction", "dot_product", "reduction_max", "vector_add",
        "vector_copy", "matrix_mul", "transpose", "transpose_tiled", "scan", "gather", "scatter",
        "histogram", "stencil_2d", "conv2d", "mandelbrot", "nbody", "bitonic_sort", "radix_sort", "transfer"}


def test_bitonic_network_sorts_against_numpy(hip, torch_cuda):
    """All k / j steps of the network on 2^12 random keys, driven from here rather than through the
    bench mirror: the final array is the sorted input, and after the k-th stage every run of k keys
    is monotone in the direction the bit of its index gives."""
    from spoc_amd import reference_kernels
    from spoc_amd.sarek import Execute, Vector
    n = 4096
    data = np.random.default_rng(7).integers(-2**31, 2**31 - 1, n).astype(np.int32)
    v = Vector.create(Vector.int32, n)
    v.fill_from(data)
    ir = reference_kernels.bitonic_sort_step()
    k = 2
    while k <= n:
        j = k // 2
        while j >= 1:
            Execute.run_vectors(ir=ir, args=[Execute.Vec(v), Execute.Int32(j), Execute.Int32(k), Execute.Int32(n)],
                                block=Execute.dims1d(256), grid=Execute.dims1d(n // 256))
            j //= 2
        runs = v.to_array().reshape(-1, k).astype(np.int64)
        up = (np.arange(0, n, k) & k) == 0
        d = np.diff(runs, axis=1)
        assert np.all(d[up] >= 0) and np.all(d[~up] <= 0), k
        k *= 2
    assert np.array_equal(v.to_array(), np.sort(data))
