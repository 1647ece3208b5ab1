"""Pins the CPU oracle (oracle/sarek_native_oracle.c) without running the reference.

Each check is chosen so that a plausible mistake in the restatement (a transposed
operand, k order reversed, a missing rounding step, f32 instead of double
accumulation, wrong tree order) fails at least one of them.  Known answers come from
the reference's own deterministic inputs and tolerances:
  benchmarks/bench_matrix_mul_tiled.ml:43-52,109-112,194  (inputs, double loop, 1e-3)
  benchmarks/bench_stream_triad.ml:44-49,122              (inputs, 1e-5)
  benchmarks/descriptions/stream_triad.md:143-148         (2 + 1*3 = 5)
  benchmarks/bench_reduction.ml:110-111,154-163           (all ones -> n, 1e-3 rel)
  sarek/tests/e2e/test_reduce.ml:54-58,386-389            (tol max(1, 1e-4*expected))
  benchmarks/bench_dot_product.ml                         (inputs, 1e-3 rel)
"""
import numpy as np
import pytest


def ref_inputs_matmul(m, n, k):
    a = (np.arange(m * k) % 10) / 10.0
    b = ((np.arange(k * n) + 1) % 10) / 10.0
    return a.reshape(m, k), b.reshape(k, n)


def python_double_loop(a, b):
    """ocaml_matmul of the reference bench: sequential double accumulation."""
    m, k = a.shape
    n = b.shape[1]
    c = np.zeros((m, n))
    for r in range(m):
        for cc in range(n):
            s = 0.0
            for i in range(k):
                s = s + a[r, i] * b[i, cc]
            c[r, cc] = s
    return c


def test_gemm_reference_inputs_match_double_loop(oracle):
    m, n, k = 24, 20, 37
    a64, b64 = ref_inputs_matmul(m, n, k)
    a32, b32 = a64.astype(np.float32), b64.astype(np.float32)
    got = oracle.gemm(a32, b32)
    # the bench's expected values use the unrounded double inputs; its tolerance is 1e-3
    assert np.abs(got - python_double_loop(a64, b64)).max() <= 1e-3
    # exact statement: double loop over the f32-rounded inputs, one rounding at the store
    want = python_double_loop(a32.astype(np.float64), b32.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got, want)


def test_gemm_sequential_k_order_is_what_is_restated(oracle):
    # values whose double sum depends on the order: increasing k must be used
    rng = np.random.default_rng(1)
    k = 4096
    a = (rng.standard_normal((1, k)) * 10.0 ** rng.integers(-6, 6, (1, k))).astype(np.float32)
    b = (rng.standard_normal((k, 1)) * 10.0 ** rng.integers(-6, 6, (k, 1))).astype(np.float32)
    fwd = 0.0
    for i in range(k):
        fwd = fwd + float(a[0, i]) * float(b[i, 0])
    rev = 0.0
    for i in reversed(range(k)):
        rev = rev + float(a[0, i]) * float(b[i, 0])
    got = oracle.gemm(a, b)[0, 0]
    assert got == np.float32(fwd)
    # sanity of the test itself: the order matters at double precision for these inputs
    assert fwd != rev


def test_gemm_not_transposed_and_nonsquare(oracle):
    rng = np.random.default_rng(2)
    a = rng.uniform(-1, 1, (7, 13)).astype(np.float32)
    b = rng.uniform(-1, 1, (13, 5)).astype(np.float32)
    want = (a.astype(np.float64) @ b.astype(np.float64))
    got = oracle.gemm(a, b)
    assert got.shape == (7, 5)
    assert np.abs(got - want).max() <= 1e-6
    e = np.zeros((13, 5), np.float32)
    e[3, 2] = 1.0  # picks column 3 of A into column 2 of C
    assert np.array_equal(oracle.gemm(a, e)[:, 2], a[:, 3])


def test_gemm_double_accumulation_not_f32(oracle):
    # 1 + 2^-30 * 4096 terms: lost entirely in f32 accumulation, kept in double
    k = 4097
    a = np.full((1, k), 2.0 ** -15, np.float32)
    b = np.full((k, 1), 2.0 ** -15, np.float32)
    a[0, 0] = 1.0
    b[0, 0] = 1.0
    want = np.float32(1.0 + 4096 * 2.0 ** -30)
    assert want != np.float32(1.0)
    assert oracle.gemm(a, b)[0, 0] == want


@pytest.mark.parametrize("m,n,k", [(16, 16, 16), (17, 33, 19), (1, 1, 1), (5, 40, 48), (32, 15, 1)])
def test_tiled_bsp_restatement_equals_closed_form(oracle, m, n, k):
    """Zero-padded 16x16 tiles + supersteps give exactly the plain product."""
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    assert np.array_equal(oracle.matmul_tiled_bsp(a, b), oracle.gemm(a, b))


def test_gemm_rows_subset(oracle):
    rng = np.random.default_rng(3)
    a = rng.uniform(-1, 1, (50, 64)).astype(np.float32)
    b = rng.uniform(-1, 1, (64, 30)).astype(np.float32)
    rows = np.array([49, 0, 17], np.int32)
    assert np.array_equal(oracle.gemm_rows(a, b, rows), oracle.gemm(a, b)[rows])


def test_gemm_thread_count_does_not_change_result(oracle):
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (33, 100)).astype(np.float32)
    b = rng.uniform(-1, 1, (100, 21)).astype(np.float32)
    assert np.array_equal(oracle.gemm(a, b, threads=1), oracle.gemm(a, b, threads=7))


def test_triad_reference_inputs(oracle):
    n = 1000
    b = ((np.arange(n) % 100) / 100.0).astype(np.float32)
    c = (((np.arange(n) + 1) % 100) / 100.0).astype(np.float32)
    got = oracle.triad(b, c, 3.0)
    expected = (np.arange(n) % 100) / 100.0 + ((np.arange(n) + 1) % 100) / 100.0 * 3.0
    assert np.abs(got - expected).max() <= 1e-5
    # exact: double arithmetic on the f32 inputs, one rounding
    assert np.array_equal(got, (b.astype(np.float64) + c.astype(np.float64) * 3.0).astype(np.float32))
    assert oracle.triad(np.float32([2.0]), np.float32([1.0]), 3.0)[0] == np.float32(5.0)


def test_triad_is_single_rounding_not_two(oracle):
    # c*s rounded to f32 first would lose the low bits: 1 + 2^-24 * 3
    b = np.float32([1.0])
    c = np.float32([1.0 + 2.0 ** -23])
    s = 3.0
    two_roundings = np.float32(np.float32(c[0] * np.float32(s)) + b[0])
    one_rounding = np.float32(float(b[0]) + float(c[0]) * s)
    got = oracle.triad(b, c, s)[0]
    assert got == one_rounding
    # operands are not swapped: b + c*s, not c + b*s
    assert oracle.triad(np.float32([10.0]), np.float32([1.0]), 3.0)[0] == np.float32(13.0)
    del two_roundings


@pytest.mark.parametrize("n", [1, 255, 256, 257, 1000, 4096, 100000])
def test_reduce_all_ones_is_exactly_n(oracle, n):
    p = oracle.reduce_sum_block256(np.ones(n, np.float32))
    assert p.size == (n + 255) // 256
    assert oracle.fold_partials(p) == float(n)
    # full blocks hold 256, the ragged last block holds the remainder
    assert all(p[:-1] == 256.0)
    assert p[-1] == (n - 256 * (p.size - 1))


def test_reduce_tree_order_and_rounding(oracle):
    """Brute-force halving tree in Python doubles, partial rounded to f32."""
    rng = np.random.default_rng(5)
    n = 700
    x = (rng.standard_normal(n) * 10.0 ** rng.integers(-4, 8, n)).astype(np.float32)
    want = []
    for blk in range((n + 255) // 256):
        s = [float(x[blk * 256 + t]) if blk * 256 + t < n else 0.0 for t in range(256)]
        half = 128
        while half >= 1:
            for t in range(half):
                s[t] = s[t] + s[t + half]
            half //= 2
        want.append(np.float32(s[0]))
    got = oracle.reduce_sum_block256(x)
    assert np.array_equal(got, np.array(want, np.float32))
    fold = 0.0
    for v in got:
        fold = fold + float(v)
    assert oracle.fold_partials(got) == fold


def test_reduce_index_sum_reference_vectors(oracle):
    # test_reduce.ml inputs: a[i] = i, b[i] = 1 (dot) and the sum tolerance rule
    n = 4096
    a = np.arange(n, dtype=np.float32)
    ones = np.ones(n, np.float32)
    expected = float(n * (n - 1) // 2)
    got = oracle.fold_partials(oracle.dot_block256(a, ones))
    assert abs(got - expected) <= max(1.0, 1e-4 * expected)
    assert got == expected  # all partials are exact integers below 2^24


def test_dot_reference_inputs(oracle):
    n = 100000
    a = ((np.arange(n) % 100) / 100.0).astype(np.float32)
    b = (((np.arange(n) + 1) % 100) / 100.0).astype(np.float32)
    expected = float(np.sum(((np.arange(n) % 100) / 100.0) * (((np.arange(n) + 1) % 100) / 100.0)))
    got = oracle.fold_partials(oracle.dot_block256(a, b))
    assert abs(got - expected) < 1e-3 * expected
    # product is formed in double (exact), not rounded to f32 before the tree
    x = np.float32([1.0 + 2.0 ** -12]); y = np.float32([1.0 + 2.0 ** -12])
    exact = float(x[0]) * float(y[0])
    assert oracle.dot_block256(x, y)[0] == np.float32(exact)


def test_triad_sum_is_the_unfused_pair(oracle):
    rng = np.random.default_rng(6)
    n = 3000
    b = rng.random(n, dtype=np.float32)
    c = rng.random(n, dtype=np.float32)
    a, partials, total = oracle.triad_sum(b, c, 3.0)
    assert np.array_equal(a, oracle.triad(b, c, 3.0))
    assert np.array_equal(partials, oracle.reduce_sum_block256(a))
    assert total == oracle.fold_partials(partials)
    assert abs(total - float(np.sum(a.astype(np.float64)))) <= 1e-6 * total


def test_rounding_to_bf16_and_f16_match_library_casts(oracle):
    import torch
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(200000) * np.exp(rng.uniform(-30, 12, 200000))).astype(np.float32)
    x[:8] = [0.0, -0.0, 65504.0, 65519.0, 65520.0, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25]
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.f16_bits(x), x.astype(np.float16).view(np.uint16))
    t = torch.from_numpy(x)
    assert torch.equal(torch.from_numpy(oracle.round_bf16(x)), t.bfloat16().float())
    assert np.array_equal(oracle.bf16_bits(x), t.bfloat16().view(torch.int16).numpy().view(np.uint16))
    assert torch.equal(torch.from_numpy(oracle.round_f16(x[np.abs(x) < 6e4])),
                       t[t.abs() < 6e4].half().float())


def test_epilogue_definition(oracle):
    """relu(A.B + bias) and its row sums, against numpy float64 (no reference counterpart)."""
    rng = np.random.default_rng(8)
    a = oracle.round_f16(rng.normal(0, 0.02, (9, 64)).astype(np.float32))
    b = oracle.round_f16(rng.normal(0, 0.02, (64, 24)).astype(np.float32))
    bias = rng.uniform(-0.1, 0.1, 24).astype(np.float32)
    y, rs = oracle.gemm_bias_relu_rowsum(a, b, bias)
    want = np.maximum(a.astype(np.float64) @ b.astype(np.float64) + bias.astype(np.float64), 0.0)
    assert np.abs(y - want).max() <= 1e-7
    assert (y >= 0).all() and (y == 0).any() and (y > 0).any()
    assert np.abs(rs - want.sum(axis=1)).max() <= 1e-6
    rows = np.array([8, 2], np.int32)
    y2, rs2 = oracle.gemm_bias_relu_rowsum(a, b, bias, rows=rows)
    assert np.array_equal(y2, y[rows]) and np.array_equal(rs2, rs[rows])


def test_fill_uniform_is_counter_based_and_in_range(oracle):
    x = oracle.fill_uniform(100000, seed=0xB, lo=0.0, hi=1.0)
    assert x.min() >= 0.0 and x.max() < 1.0
    assert abs(float(x.mean()) - 0.5) < 0.01
    assert np.array_equal(x, oracle.fill_uniform(100000, seed=0xB, threads=3))
    assert not np.array_equal(x, oracle.fill_uniform(100000, seed=0xC))
    y = oracle.fill_uniform(1000, seed=0xA11CE, lo=-1.0, hi=1.0)
    assert y.min() >= -1.0 and y.max() < 1.0


def test_max_tree_equals_plain_max_and_keeps_tree_nan_rules(oracle):
    """bench_reduction_max.ml:18-100: on NaN-free data the tree is the plain maximum of the
    block with the fill value for missing slots; with a NaN the strict '>' keeps whatever
    sits in the left slot, which a literal thread-by-thread replay of the supersteps fixes."""
    rng = np.random.default_rng(11)
    n = 256 * 5 + 77
    x = (rng.standard_normal(n) * 100).astype(np.float32)
    got = oracle.reduce_max_block256(x)
    exp = np.array([max(x[i:i + 256].max(), np.float32(-1000000.0)) for i in range(0, n, 256)], np.float32)
    assert np.array_equal(got, exp)
    # all values below the fill: the partial block reports the fill, full blocks do not
    y = np.full(300, -2000000.0, np.float32)
    assert oracle.reduce_max_block256(y).tolist() == [-2000000.0, -1000000.0]
    # the reference's own input and check (bench_reduction_max.ml:95-101,159-166):
    # input[i] = i mod 10000, max over the partials = max over the input, within 1e-5
    z = (np.arange(25000) % 10000).astype(np.float32)
    assert abs(float(oracle.reduce_max_block256(z).max()) - 9999.0) < 1e-5

    def replay(block):
        s = [float(v) for v in block] + [-1000000.0] * (256 - len(block))
        half = 128
        while half >= 1:
            for t in range(half):       # one superstep: reads and writes touch disjoint slots
                a, b = s[t], s[t + half]
                if b > a:
                    s[t] = b
            half //= 2
        return np.float32(s[0])
    w = x[:256].copy()
    w[3] = np.nan      # left slot of a pair: survives every comparison it takes part in
    w[200] = np.nan    # right slot: never greater, dropped
    got = oracle.reduce_max_block256(w)
    exp = replay(w)
    assert (np.isnan(got[0]) and np.isnan(exp)) or got[0] == exp


# ---- the other memory-bound kernels and the one-thread-per-element matmul ----------------------
#   benchmarks/bench_vector_add.ml:68-71,108     (a = 0.001 i, b = 0.002 i, 1e-3)
#   benchmarks/bench_vector_copy.ml:41-43,109    ((i mod 100)/100, 1e-6)
#   benchmarks/bench_transpose.ml:50-57,103,143-148 (input[i] = i, cpu_transpose, 1e-3)
#   benchmarks/bench_matrix_mul.ml:43-52,86-90   (inputs and double loop of the tiled bench)

def test_vector_add_reference_inputs_and_single_rounding(oracle):
    n = 10007
    a, b = np.arange(n) * 0.001, np.arange(n) * 0.002
    out = np.full(n, -7.0, dtype=np.float32)
    oracle.vector_add(a, b, out, n)
    assert np.all(np.abs(out.astype(np.float64) - (a + b)) <= 1e-3)        # the bench's check
    # two binary32 values add exactly in double, so one rounding gives the binary32 sum
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(4096) * 10.0 ** rng.integers(-20, 20, 4096)).astype(np.float32)
    y = (rng.standard_normal(4096) * 10.0 ** rng.integers(-20, 20, 4096)).astype(np.float32)
    out = np.zeros(4096, dtype=np.float32)
    assert np.array_equal(oracle.vector_add(x, y, out, 4096), x + y)
    # `if tid < n`: a longer vector keeps its tail, a shorter launch leaves its own tail alone
    out = np.full(100, -7.0, dtype=np.float32)
    oracle.vector_add(x[:100], y[:100], out, 60, threads=256)
    assert np.array_equal(out[:60], (x + y)[:60]) and np.all(out[60:] == -7.0)
    out = np.full(100, -7.0, dtype=np.float32)
    oracle.vector_add(x[:100], y[:100], out, 100, threads=64)
    assert np.array_equal(out[:64], (x + y)[:64]) and np.all(out[64:] == -7.0)


def test_vector_copy_reference_inputs(oracle):
    n = 1000
    a = (np.arange(n) % 100) / 100.0
    out = np.full(n + 5, 9.0, dtype=np.float32)
    oracle.vector_copy(a, out, n)
    assert np.all(np.abs(out[:n].astype(np.float64) - a) <= 1e-6) and np.all(out[n:] == 9.0)
    assert np.array_equal(out[:n], a.astype(np.float32))


def test_transpose_reference_inputs_and_shapes(oracle):
    m = 48
    data = np.arange(m * m, dtype=np.float64)
    out = oracle.transpose(data, m, m)
    expected = np.zeros(m * m)
    for row in range(m):                       # cpu_transpose of the bench
        for col in range(m):
            expected[col * m + row] = data[row * m + col]
    assert np.all(np.abs(out - expected) <= 1e-3)
    # rectangular: `width` columns in, `height` columns out; a wrong pitch fails this
    w, h = 7, 5
    x = np.arange(w * h, dtype=np.float32)
    assert np.array_equal(oracle.transpose(x, w, h).reshape(w, h), x.reshape(h, w).T)
    part = oracle.transpose(x, w, h, out=np.full(w * h, -1, dtype=np.float32), threads=w * 2)   # two input rows
    assert np.array_equal(part.reshape(w, h)[:, :2], x.reshape(h, w).T[:, :2]) and np.all(part.reshape(w, h)[:, 2:] == -1)
    twice = oracle.transpose(oracle.transpose(x, w, h), h, w)
    assert np.array_equal(twice, x)


def test_naive_matmul_is_the_same_sum_as_the_tiled_kernel(oracle):
    m, n, k = 19, 23, 41
    a = oracle.fill_uniform(m * k, seed=3, lo=-1, hi=1)
    b = oracle.fill_uniform(k * n, seed=4, lo=-1, hi=1)
    c = oracle.matmul_naive(a, b, m, n, k)
    # zero padding of the tiles adds exact zeros: both kernels compute the same double sums
    assert np.array_equal(c.reshape(m, n), oracle.gemm(a.reshape(m, k), b.reshape(k, n)))
    assert np.array_equal(c.reshape(m, n), oracle.matmul_tiled_bsp(a.reshape(m, k), b.reshape(k, n)))
    a64, b64 = ref_inputs_matmul(16, 16, 16)
    c = oracle.matmul_naive(a64.reshape(-1), b64.reshape(-1), 16, 16, 16)
    assert np.all(np.abs(c.reshape(16, 16) - python_double_loop(a64, b64)) <= 1e-3)
    # row = tid / n, col = tid mod n: a launch of n + 3 threads fills row 0 and three of row 1
    part = oracle.matmul_naive(a, b, m, n, k, out=np.full(m * n, -1, dtype=np.float32), threads=n + 3)
    assert np.array_equal(part[:n + 3], c_full := oracle.matmul_naive(a, b, m, n, k)[:n + 3]) and np.all(part[n + 3:] == -1)


# ---- the 2-D neighbourhood kernels -------------------------------------------------------------------
#   benchmarks/bench_stencil_2d.ml:39-51,88-93,158-164 (sin(0.1 x) cos(0.1 y), cpu_stencil_2d, 1e-4)
#   benchmarks/bench_conv2d.ml:40-60,103-111,179-185 (((x + y) mod 256) / 255, cpu_conv2d with nine 1/9 taps, 1e-3)

def _grid(w, h, f):
    y, x = np.mgrid[0:h, 0:w]
    return f(x.astype(np.float64), y.astype(np.float64))


def test_stencil_2d_reference_inputs_closed_forms_and_order(oracle):
    w, h = 37, 29                                                    # a wrong pitch fails on a rectangle
    data = _grid(w, h, lambda x, y: np.sin(x * 0.1) * np.cos(y * 0.1))
    out = oracle.stencil_2d(data.reshape(-1), w, h, out=np.full(w * h, -7.0, dtype=np.float32)).reshape(h, w)
    expected = np.zeros((h, w))
    for y in range(1, h - 1):                                        # cpu_stencil_2d of the bench
        for x in range(1, w - 1):
            expected[y, x] = (data[y - 1, x] + data[y + 1, x] + data[y, x - 1] + data[y, x + 1] + data[y, x]) / 5.0
    assert np.all(np.abs(out[1:-1, 1:-1] - expected[1:-1, 1:-1]) <= 1e-4)
    border = np.ones((h, w), dtype=bool)
    border[1:-1, 1:-1] = False
    assert np.all(out[border] == -7.0)                               # boundaries unchanged
    # closed forms on small integers (every step exact): a constant and a plane are fixed points; x^2 gains 2/5 (a
    # dropped or doubled horizontal neighbour shows), y^2 likewise, x y is a fixed point only with the right pitch
    for f, g in [(lambda x, y: 0 * x + 3, lambda x, y: 0 * x + 3), (lambda x, y: 3 * x + 7 * y, lambda x, y: 3 * x + 7 * y),
                 (lambda x, y: x * x, lambda x, y: x * x + 0.4), (lambda x, y: y * y, lambda x, y: y * y + 0.4),
                 (lambda x, y: x * y, lambda x, y: x * y), (lambda x, y: x * x * y, lambda x, y: x * x * y + 0.4 * y)]:
        got = oracle.stencil_2d(_grid(w, h, f).reshape(-1), w, h).reshape(h, w)
        assert np.array_equal(got[1:-1, 1:-1], _grid(w, h, g).astype(np.float32)[1:-1, 1:-1])
    # the sum runs up, down, left, right, center in double: 2^60 + 1 + 1 + 1 - 2^60 loses the ones, 2^60 - 2^60 first keeps them
    cell = np.zeros((3, 3), dtype=np.float32)
    cell[0, 1], cell[2, 1], cell[1, 0], cell[1, 2], cell[1, 1] = 2.0 ** 60, 1, 1, 1, -2.0 ** 60
    assert oracle.stencil_2d(cell.reshape(-1), 3, 3)[4] == 0.0
    cell[0, 1], cell[2, 1], cell[1, 0], cell[1, 2], cell[1, 1] = 2.0 ** 60, -2.0 ** 60, 1, 1, 1
    assert oracle.stencil_2d(cell.reshape(-1), 3, 3)[4] == np.float32(0.6)
    # one rounding: the double quotient, not a quotient of float32 partial sums
    rng = np.random.default_rng(11)
    x = rng.standard_normal((h, w)).astype(np.float32)
    x64 = x.astype(np.float64)
    exact = ((((x64[:-2, 1:-1] + x64[2:, 1:-1]) + x64[1:-1, :-2]) + x64[1:-1, 2:]) + x64[1:-1, 1:-1]) / 5.0
    assert np.array_equal(oracle.stencil_2d(x.reshape(-1), w, h).reshape(h, w)[1:-1, 1:-1], exact.astype(np.float32))
    # a launch that reaches 10 x 6 threads computes the interior cells among them and nothing else
    part = oracle.stencil_2d(x.reshape(-1), w, h, out=np.full(w * h, -7.0, dtype=np.float32), threads_xy=(10, 6)).reshape(h, w)
    assert np.array_equal(part[1:6, 1:10], exact.astype(np.float32)[:5, :9])
    part[1:6, 1:10] = -7.0
    assert np.all(part == -7.0)
    # grids without an interior write nothing
    for ww, hh in [(1, 1), (2, 5), (5, 2), (1, 9)]:
        assert np.all(oracle.stencil_2d(np.ones(ww * hh), ww, hh, out=np.full(ww * hh, -7.0, dtype=np.float32)) == -7.0)


def test_conv2d_reference_inputs_closed_forms_and_order(oracle):
    w, h = 41, 23
    data = _grid(w, h, lambda x, y: ((x + y) % 256) / 255.0)
    out = oracle.conv2d(data.reshape(-1), w, h, out=np.full(w * h, -7.0, dtype=np.float32)).reshape(h, w)
    taps = [1.0 / 9.0] * 9
    expected = np.zeros((h, w))
    for y in range(1, h - 1):                                        # cpu_conv2d of the bench
        for x in range(1, w - 1):
            acc = 0.0
            for ky in range(3):
                for kx in range(3):
                    acc = acc + data[y + ky - 1, x + kx - 1] * taps[ky * 3 + kx]
            expected[y, x] = acc
    assert np.all(np.abs(out - expected) <= 1e-3)                    # boundaries are 0 in both
    assert np.all(out[0] == 0) and np.all(out[-1] == 0) and np.all(out[:, 0] == 0) and np.all(out[:, -1] == 0)
    for f, g in [(lambda x, y: 0 * x + 3, lambda x, y: 0 * x + 3), (lambda x, y: 3 * x + 7 * y, lambda x, y: 3 * x + 7 * y),
                 (lambda x, y: x * y, lambda x, y: x * y)]:
        got = oracle.conv2d(_grid(w, h, f).reshape(-1), w, h).reshape(h, w)
        assert np.array_equal(got[1:-1, 1:-1], _grid(w, h, g).astype(np.float32)[1:-1, 1:-1])
    for f, extra in [(lambda x, y: x * x, 6.0), (lambda x, y: y * y, 6.0)]:     # (9 v + 6) / 9, rounded once
        got = oracle.conv2d(_grid(w, h, f).reshape(-1), w, h).reshape(h, w)
        assert np.array_equal(got[1:-1, 1:-1], ((9.0 * _grid(w, h, f) + extra) / 9.0).astype(np.float32)[1:-1, 1:-1])
    # p00 first, p22 last: 2^60 + seven ones - 2^60 is 0 in that order and 7/9 when the two large cells meet first
    cell = np.ones((3, 3), dtype=np.float32)
    cell[0, 0], cell[2, 2] = 2.0 ** 60, -2.0 ** 60
    big = np.zeros((5, 5), dtype=np.float32)
    big[1:4, 1:4] = cell
    assert oracle.conv2d(big.reshape(-1), 5, 5)[12] == 0.0
    big[1, 1], big[1, 2] = 2.0 ** 60, -2.0 ** 60
    big[3, 3] = 1.0
    assert oracle.conv2d(big.reshape(-1), 5, 5)[12] == np.float32(7.0 / 9.0)
    # row-major taps: a single 1 at (y, x) reaches the nine cells round it and no others
    one = np.zeros((7, 9), dtype=np.float32)
    one[2, 5] = 9.0
    got = oracle.conv2d(one.reshape(-1), 9, 7).reshape(7, 9)
    want = np.zeros((7, 9), dtype=np.float32)
    want[1:4, 4:7] = 1.0
    assert np.array_equal(got, want)
    # tid < n, x = tid mod width, y = tid / width: a short launch fills the first cells in row-major order
    rng = np.random.default_rng(12)
    x = rng.standard_normal((h, w)).astype(np.float32)
    full = oracle.conv2d(x.reshape(-1), w, h)
    part = oracle.conv2d(x.reshape(-1), w, h, out=np.full(w * h, -7.0, dtype=np.float32), threads=3 * w + 5)
    assert np.array_equal(part[:3 * w + 5], full[:3 * w + 5]) and np.all(part[3 * w + 5:] == -7.0)
    # grids that are all border
    for ww, hh in [(1, 1), (2, 5), (5, 2), (1, 9)]:
        assert np.all(oracle.conv2d(np.ones(ww * hh), ww, hh, out=np.full(ww * hh, -7.0, dtype=np.float32)) == 0.0)


# ---- histograms (benchmarks/bench_histogram.ml, bench_radix_sort.ml) -------------------------------

@pytest.mark.parametrize("n,bins,block", [(0, 256, 256), (1, 256, 256), (1000, 256, 256), (100003, 256, 256),
                                           (5000, 10, 64), (5000, 200, 256), (777, 1, 32), (4096, 256, 1024)])
def test_histogram_is_numpy_bincount(oracle, n, bins, block):
    keys = np.random.default_rng(n + bins).integers(0, 1 << 30, n).astype(np.int32)
    hist = np.full(256, 3, dtype=np.int32)                       # accumulated into, not cleared
    assert oracle.histogram(keys, hist, n, bins, block=block) == 0
    expected = np.full(256, 3, dtype=np.int64)
    expected[:bins] += np.bincount(keys.astype(np.int64) % bins, minlength=bins)
    assert np.array_equal(hist, expected)


def test_histogram_of_a_short_launch_and_of_narrow_blocks(oracle):
    keys = (np.arange(4000) % 100).astype(np.int32)
    hist = np.zeros(256, dtype=np.int32)
    assert oracle.histogram(keys, hist, 4000, 100, block=256, grid=4) == 0      # 1024 threads: the first 1024 keys
    assert np.array_equal(hist[:100], np.bincount(keys[:1024], minlength=100)) and not hist[100:].any()
    # a block of 32 threads clears and merges bins 0..31 only; the others hold what the shared
    # array held before (here -7) and never reach the result
    hist = np.zeros(256, dtype=np.int32)
    assert oracle.histogram(keys, hist, 4000, 100, block=32) == 0
    assert np.array_equal(hist[:32], np.bincount(keys, minlength=100)[:32]) and not hist[32:].any()


def test_histogram_remainder_has_the_sign_of_the_key(oracle):
    keys = np.array([-512, -256, -255, -1, 0, 1, 255, 256, -2**31], dtype=np.int32)
    hist = np.zeros(256, dtype=np.int32)
    assert oracle.histogram(keys, hist, len(keys), 256) == 2                     # -255 and -1 have no slot
    expected = np.zeros(256, dtype=np.int32)
    expected[0], expected[1], expected[255] = 5, 1, 1
    assert np.array_equal(hist, expected)


@pytest.mark.parametrize("shift,mask", [(0, 255), (8, 255), (16, 255), (24, 255), (3, 15), (0, 0), (31, 1)])
def test_radix_histogram_counts_digits(oracle, shift, mask):
    n = 50021
    keys = np.random.default_rng(shift * 256 + mask).integers(-2**31, 2**31 - 1, n).astype(np.int32)
    hist = np.zeros(256, dtype=np.int32)
    assert oracle.radix_histogram(keys, hist, n, shift, mask) == 0
    digits = (keys.view(np.uint32) >> np.uint32(shift)) & np.uint32(mask)
    assert np.array_equal(hist, np.bincount(digits, minlength=256))
    if shift <= 24:   # the eight digit bits are key bits under an arithmetic shift too
        assert np.array_equal(digits, (keys >> shift) & mask)


@pytest.mark.parametrize("shift", [0, 8, 24])
def test_radix_scatter_in_thread_order_is_a_stable_sort_by_digit(oracle, shift):
    n = 30011
    keys = np.random.default_rng(shift).integers(-2**31, 2**31 - 1, n).astype(np.int32)
    digits = ((keys.view(np.uint32) >> np.uint32(shift)) & np.uint32(255)).astype(np.int64)
    counts = np.bincount(digits, minlength=256)
    starts = np.concatenate(([0], np.cumsum(counts)[:-1])).astype(np.int32)
    counters, out = starts.copy(), np.full(n, -1, dtype=np.int32)
    assert oracle.radix_scatter(keys, out, counters, n, shift, 255) == 0
    assert np.array_equal(out, keys[np.argsort(digits, kind="stable")])
    assert np.array_equal(counters, starts + counts)
    # a launch that reaches only the first 1000 keys; positions past the output are reported, not written
    counters, out = starts.copy(), np.full(n, -1, dtype=np.int32)
    assert oracle.radix_scatter(keys, out, counters, n, shift, 255, threads=1000) == 0
    assert np.array_equal(np.sort(out[out != -1]), np.sort(keys[:1000])) or -1 in keys[:1000]
    counters, small = starts.copy(), np.full(100, -1, dtype=np.int32)
    assert oracle.radix_scatter(keys, small, counters, n, shift, 255) == n - 100
