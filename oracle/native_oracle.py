"""ctypes front end of oracle/sarek_native_oracle.c (TEST INFRASTRUCTURE ONLY).

Each wrapper takes and returns numpy arrays; the arithmetic lives in the C
file, which cites the reference lines it restates.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

__all__ = [
    "build", "fill_uniform", "round_bf16", "round_f16", "bf16_bits", "f16_bits",
    "triad", "reduce_sum_block256", "reduce_max_block256", "dot_block256", "fold_partials", "triad_sum",
    "gemm", "gemm_rows", "gemm_bias_relu_rowsum", "matmul_tiled_bsp",
    "vector_add", "vector_copy", "transpose", "histogram", "radix_histogram", "radix_scatter", "matmul_naive",
    "stencil_2d", "conv2d",
]


def build(force=False):
    """Compile liboracle.so with gcc (seconds)."""
    src = os.path.join(_HERE, "sarek_native_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def _L():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        lib = C.CDLL(_SO)
        f32p, u16p, i32p = (C.POINTER(C.c_float), C.POINTER(C.c_uint16),
                            C.POINTER(C.c_int32))
        i64, i32 = C.c_int64, C.c_int
        lib.oracle_fill_uniform_f32.argtypes = [f32p, i64, C.c_uint64, C.c_float, C.c_float, i32]
        lib.oracle_round_bf16_array.argtypes = [f32p, f32p, u16p, i64]
        lib.oracle_round_f16_array.argtypes = [f32p, f32p, u16p, i64]
        lib.oracle_triad_f32.argtypes = [f32p, f32p, f32p, C.c_float, i64, i32]
        lib.oracle_reduce_sum_block256_f32.argtypes = [f32p, i64, f32p, i32]
        lib.oracle_dot_block256_f32.argtypes = [f32p, f32p, i64, f32p, i32]
        lib.oracle_reduce_max_block256_f32.argtypes = [f32p, i64, C.c_double, f32p]
        lib.oracle_fold_partials_f64.argtypes = [f32p, i64]
        lib.oracle_fold_partials_f64.restype = C.c_double
        lib.oracle_triad_sum_f32.argtypes = [f32p, f32p, f32p, C.c_float, i64, f32p, i32]
        lib.oracle_triad_sum_f32.restype = C.c_double
        lib.oracle_gemm_f32.argtypes = [f32p, f32p, f32p, i64, i64, i64, i32]
        lib.oracle_gemm_f32_rows.argtypes = [f32p, f32p, f32p, i32p, i64, i64, i64, i32]
        lib.oracle_gemm_bias_relu_rowsum.argtypes = [f32p, f32p, f32p, f32p, f32p, i32p,
                                                     i64, i64, i64, i32]
        lib.oracle_matmul_tiled_bsp.argtypes = [f32p, f32p, f32p, i32, i32, i32]
        lib.oracle_vector_add_f32.argtypes = [f32p, f32p, f32p, i64, i64]
        lib.oracle_vector_copy_f32.argtypes = [f32p, f32p, i64, i64]
        lib.oracle_transpose_f32.argtypes = [f32p, f32p, i32, i32, i64]
        lib.oracle_stencil_2d_f32.argtypes = [f32p, f32p, i32, i32, i64, i64]
        lib.oracle_conv2d_f32.argtypes = [f32p, f32p, i32, i32, i64]
        lib.oracle_matmul_naive_f32.argtypes = [f32p, f32p, f32p, i32, i32, i32, i64]
        _lib = lib
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(C.POINTER(C.c_float))


def default_threads():
    return max(1, os.cpu_count() or 1)


def fill_uniform(n, seed, lo=0.0, hi=1.0, threads=None):
    out = np.empty(int(n), dtype=np.float32)
    _L().oracle_fill_uniform_f32(out.ctypes.data_as(C.POINTER(C.c_float)), int(n), int(seed),
                                 lo, hi, threads or default_threads())
    return out


def _round16(x, fn):
    x, xp = _f32(x)
    out = np.empty_like(x)
    bits = np.empty(x.shape, dtype=np.uint16)
    fn(xp, out.ctypes.data_as(C.POINTER(C.c_float)),
       bits.ctypes.data_as(C.POINTER(C.c_uint16)), x.size)
    return out, bits


def round_bf16(x):
    return _round16(x, _L().oracle_round_bf16_array)[0]


def bf16_bits(x):
    return _round16(x, _L().oracle_round_bf16_array)[1]


def round_f16(x):
    return _round16(x, _L().oracle_round_f16_array)[0]


def f16_bits(x):
    return _round16(x, _L().oracle_round_f16_array)[1]


def triad(b, c, s, threads=None):
    b, bp = _f32(b)
    c, cp = _f32(c)
    a = np.empty_like(b)
    _L().oracle_triad_f32(a.ctypes.data_as(C.POINTER(C.c_float)), bp, cp, s, b.size,
                          threads or default_threads())
    return a


def reduce_sum_block256(x, threads=None):
    x, xp = _f32(x)
    p = np.empty((x.size + 255) // 256, dtype=np.float32)
    _L().oracle_reduce_sum_block256_f32(xp, x.size, p.ctypes.data_as(C.POINTER(C.c_float)),
                                        threads or default_threads())
    return p


def reduce_max_block256(x, pad=-1000000.0):
    x, xp = _f32(x)
    p = np.empty((x.size + 255) // 256, dtype=np.float32)
    _L().oracle_reduce_max_block256_f32(xp, x.size, float(pad), p.ctypes.data_as(C.POINTER(C.c_float)))
    return p


def dot_block256(a, b, threads=None):
    a, ap = _f32(a)
    b, bp = _f32(b)
    p = np.empty((a.size + 255) // 256, dtype=np.float32)
    _L().oracle_dot_block256_f32(ap, bp, a.size, p.ctypes.data_as(C.POINTER(C.c_float)),
                                 threads or default_threads())
    return p


def fold_partials(p):
    p, pp = _f32(p)
    return float(_L().oracle_fold_partials_f64(pp, p.size))


def triad_sum(b, c, s, threads=None):
    """Returns (a, partials, sum) of the unfused Native pair."""
    b, bp = _f32(b)
    c, cp = _f32(c)
    a = np.empty_like(b)
    p = np.empty((b.size + 255) // 256, dtype=np.float32)
    tot = _L().oracle_triad_sum_f32(a.ctypes.data_as(C.POINTER(C.c_float)), bp, cp, s, b.size,
                                    p.ctypes.data_as(C.POINTER(C.c_float)),
                                    threads or default_threads())
    return a, p, float(tot)


def gemm(a, b, threads=None):
    a, ap = _f32(a)
    b, bp = _f32(b)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    c = np.empty((m, n), dtype=np.float32)
    _L().oracle_gemm_f32(ap, bp, c.ctypes.data_as(C.POINTER(C.c_float)), m, n, k,
                         threads or default_threads())
    return c


def gemm_rows(a, b, rows, threads=None):
    a, ap = _f32(a)
    b, bp = _f32(b)
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    k, n = b.shape
    c = np.empty((rows.size, n), dtype=np.float32)
    _L().oracle_gemm_f32_rows(ap, bp, c.ctypes.data_as(C.POINTER(C.c_float)),
                              rows.ctypes.data_as(C.POINTER(C.c_int32)), rows.size, n, k,
                              threads or default_threads())
    return c


def gemm_bias_relu_rowsum(a, b, bias, rows=None, threads=None):
    a, ap = _f32(a)
    b, bp = _f32(b)
    bias, biasp = _f32(bias)
    k, n = b.shape
    if rows is None:
        rows = np.arange(a.shape[0], dtype=np.int32)
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    y = np.empty((rows.size, n), dtype=np.float32)
    rs = np.empty(rows.size, dtype=np.float32)
    _L().oracle_gemm_bias_relu_rowsum(ap, bp, biasp, y.ctypes.data_as(C.POINTER(C.c_float)),
                                      rs.ctypes.data_as(C.POINTER(C.c_float)),
                                      rows.ctypes.data_as(C.POINTER(C.c_int32)), rows.size, n, k,
                                      threads or default_threads())
    return y, rs


def matmul_tiled_bsp(a, b):
    a, ap = _f32(a)
    b, bp = _f32(b)
    m, k = a.shape
    _, n = b.shape
    c = np.zeros((m, n), dtype=np.float32)
    _L().oracle_matmul_tiled_bsp(ap, bp, c.ctypes.data_as(C.POINTER(C.c_float)), m, n, k)
    return c


def _launch_size(n, threads):
    return int(threads) if threads is not None else int(n)


def vector_add(a, b, out, n, threads=None):
    """In place on `out` (float32 array): what the vector-add kernel leaves there."""
    a, ap = _f32(a)
    b, bp = _f32(b)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    _L().oracle_vector_add_f32(ap, bp, out.ctypes.data_as(C.POINTER(C.c_float)), n, _launch_size(n, threads))
    return out


def vector_copy(a, out, n, threads=None):
    a, ap = _f32(a)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    _L().oracle_vector_copy_f32(ap, out.ctypes.data_as(C.POINTER(C.c_float)), n, _launch_size(n, threads))
    return out


def _i32(x):
    x = np.ascontiguousarray(x, dtype=np.int32)
    return x, x.ctypes.data_as(C.POINTER(C.c_int32))


def histogram(keys, hist, n, num_bins, block=256, grid=None, stale=-7):
    """Adds the launch's counts to `hist` (int32, in place); returns the number of keys without a slot."""
    keys, kp = _i32(keys)
    assert hist.dtype == np.int32 and hist.flags.c_contiguous
    grid = (n + block - 1) // block if grid is None else grid
    f = _L().oracle_histogram_i32
    f.restype = C.c_int64
    return f(kp, hist.ctypes.data_as(C.POINTER(C.c_int32)), C.c_int32(n), C.c_int32(num_bins), C.c_int32(block),
             C.c_int32(grid), C.c_int32(stale))


def radix_histogram(keys, hist, n, shift, mask, block=256, grid=None, stale=-7):
    keys, kp = _i32(keys)
    assert hist.dtype == np.int32 and hist.flags.c_contiguous
    grid = (n + block - 1) // block if grid is None else grid
    f = _L().oracle_radix_histogram_i32
    f.restype = C.c_int64
    return f(kp, hist.ctypes.data_as(C.POINTER(C.c_int32)), C.c_int32(n), C.c_int32(shift), C.c_int32(mask),
             C.c_int32(block), C.c_int32(grid), C.c_int32(stale))


def radix_scatter(keys, out, counters, n, shift, mask, threads=None):
    """In place on `out` and `counters` (int32); returns the number of positions outside `out`."""
    keys, kp = _i32(keys)
    assert out.dtype == np.int32 and out.flags.c_contiguous and counters.dtype == np.int32
    f = _L().oracle_radix_scatter_i32
    f.restype = C.c_int64
    p32 = C.POINTER(C.c_int32)
    return f(kp, out.ctypes.data_as(p32), C.c_int64(len(out)), counters.ctypes.data_as(p32), C.c_int32(n),
             C.c_int32(shift), C.c_int32(mask), C.c_int64(_launch_size(n, threads)))


def transpose(x, width, height, out=None, threads=None):
    x, xp = _f32(x)
    if out is None:
        out = np.zeros(width * height, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    _L().oracle_transpose_f32(xp, out.ctypes.data_as(C.POINTER(C.c_float)), width, height,
                              _launch_size(width * height, threads))
    return out


def stencil_2d(x, width, height, out=None, threads_xy=None):
    """In place on `out` (the border and any cell the launch does not reach keep their values; zeros if not given);
    threads_xy = (threads in x, threads in y) of the 2-D launch, the whole grid by default."""
    x, xp = _f32(x)
    if out is None:
        out = np.zeros(width * height, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    tx, ty = (width, height) if threads_xy is None else threads_xy
    _L().oracle_stencil_2d_f32(xp, out.ctypes.data_as(C.POINTER(C.c_float)), width, height, tx, ty)
    return out


def conv2d(x, width, height, out=None, threads=None):
    x, xp = _f32(x)
    if out is None:
        out = np.zeros(width * height, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    _L().oracle_conv2d_f32(xp, out.ctypes.data_as(C.POINTER(C.c_float)), width, height,
                           _launch_size(width * height, threads))
    return out


def matmul_naive(a, b, m, n, k, out=None, threads=None):
    a, ap = _f32(a)
    b, bp = _f32(b)
    if out is None:
        out = np.zeros(m * n, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    _L().oracle_matmul_naive_f32(ap, bp, out.ctypes.data_as(C.POINTER(C.c_float)), m, n, k,
                                 _launch_size(m * n, threads))
    return out
