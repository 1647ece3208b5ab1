"""Element-wise kernels rebuilt in the stream kernels' shape (tag map_f32) and fused with the block-256 sum
(benchmarks/bench_reduction.ml:62-96) in Execute.run_pipeline: the vector they write is the generated kernel's bit
for bit, the sums are the hand block-256 kernel's on that vector."""
import os

import numpy as np
import pytest

from map_kernels import MAPS, MAX_TREES, TREES

pytestmark = pytest.mark.gpu

IR_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ir")


@pytest.fixture()
def sarek(hip, torch_cuda):
    from spoc_amd import sarek as s
    s.Device.init()
    yield s
    hip.check(hip.lib.sarek_hip_set_specialisation(1))
SIZES = [1, 3, 255, 256, 257, 4095, 4096, 4097, 8191, 100003, (1 << 20) + 5]


def arguments(sarek, name, n, rng):
    """(launch arguments in parameter order, output vector) of MAPS[name] over n elements."""
    E, V = sarek.Execute, sarek.Vector

    def vec():
        return V.of_array((rng.standard_normal(n) * 10.0 ** rng.integers(-3, 3, n)).astype(np.float32))

    out = V.create(V.float32, n)
    out.host[:] = np.nan
    if name == "scale":
        return [E.Vec(vec()), E.Vec(out), E.Float32(1.7), E.Int32(n)], out
    if name == "saxpy_with_let":
        return [E.Vec(vec()), E.Vec(vec()), E.Vec(out), E.Float32(-0.3), E.Int32(n)], out
    if name == "norm3":
        return [E.Vec(out), E.Vec(vec()), E.Vec(vec()), E.Vec(vec()), E.Int32(n)], out
    if name == "ramp_select":
        return [E.Vec(vec()), E.Vec(vec()), E.Vec(out), E.Int32(5), E.Int32(n)], out
    if name == "six_inputs":
        return [E.Vec(vec()) for _ in range(6)] + [E.Vec(out), E.Int32(n)], out
    if name == "fill_const":
        return [E.Vec(out), E.Float32(2.5), E.Int32(n)], out
    if name == "short_names":
        return [E.Vec(vec()), E.Vec(vec()), E.Vec(out), E.Float32(0.75), E.Float32(-1.25), E.Int32(9), E.Int32(n)], out
    raise KeyError(name)


def both_ways(hip, run):
    res = []
    for on in (1, 0):
        hip.check(hip.lib.sarek_hip_set_specialisation(on))
        try:
            res.append(run())
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
    return res


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("name", sorted(MAPS))
def test_a_map_alone_writes_what_the_generated_kernel_writes(hip, sarek, name, n):
    E = sarek.Execute
    ir = MAPS[name]()

    def run():
        args, out = arguments(sarek, name, n, np.random.default_rng(n))
        path = E.run_vectors(ir, args, (256, 1, 1), ((n + 255) // 256, 1, 1))
        return path, out.to_array().copy()

    (p_map, got), (p_jit, want) = both_ways(hip, run)
    assert (p_map, p_jit) == ("map_f32", "jit")
    assert not np.isnan(want).any() or name == "norm3"
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("name", sorted(MAPS))
def test_map_then_block_sum_is_one_launch(hip, sarek, name, n):
    E, V = sarek.Execute, sarek.Vector
    ir = MAPS[name]()
    reduction = open(os.path.join(IR_DIR, "reduction.ir")).read()
    nblocks = (n + 255) // 256

    def run():
        args, out = arguments(sarek, name, n, np.random.default_rng(n))
        sums = V.create(V.float32, nblocks)
        sums.host[:] = np.nan
        stages = [(ir, args, (256, 1, 1), (nblocks, 1, 1)),
                  (reduction, [E.Vec(out), E.Vec(sums), E.Int32(n)], (256, 1, 1), (nblocks, 1, 1))]
        return E.run_pipeline(stages), out.to_array().copy(), sums.to_array().copy(), (stages, sums)

    (fused, a_fused, s_fused, (stages, sums)), (jit, a_jit, s_jit, _) = both_ways(hip, run)
    assert fused == ("map_f32+reduce_sum_block256_f32", 1) and jit == ("jit;jit", 2)
    assert np.array_equal(a_fused.view(np.uint32), a_jit.view(np.uint32))
    # the hand block-256 kernel on the same vector gives the same bits; the generated tree kernel is within the
    # sum's tolerance (it adds the same values in another association)
    assert E.run_vectors(*stages[1]) == "reduce_sum_block256_f32"
    assert np.array_equal(sums.to_array().view(np.uint32), s_fused.view(np.uint32))
    scale = np.abs(a_jit.astype(np.float64)).reshape(-1)
    bound = np.add.reduceat(scale, np.arange(0, n, 256)) * 1e-5 + 1e-30
    assert np.all(np.abs(s_fused.astype(np.float64) - s_jit.astype(np.float64)) <= bound)


@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_MAP_SEEDS", "32"))))
def test_seeded_random_maps_alone_and_in_front_of_the_sum(hip, sarek, seed):
    """Kernels nobody wrote by hand: seeded expression trees (arithmetic, divisions, math intrinsics, `if`
    expressions on values and on the index, casts of index arithmetic, lets) over one to four inputs.  The rebuilt
    kernel writes the generated kernel's bits, alone and fused with the block sums, whose bits are the hand
    block-256 kernel's on that vector."""
    from map_kernels import random_map
    _rebuilt_map_against_generated(hip, sarek, *random_map(seed), seed)


@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_MAP_SEEDS", "32")) // 2))
def test_seeded_random_maps_whose_lets_hide_each_other(hip, sarek, seed):
    """The same check for maps whose lets reuse names -- an earlier let's, the scalar parameter a's --, which the
    lowering prints under names of their own in both texts."""
    from map_kernels import random_map_rebinding
    _rebuilt_map_against_generated(hip, sarek, *random_map_rebinding(seed), seed)


def _rebuilt_map_against_generated(hip, sarek, ir, n_in, seed):
    E, V = sarek.Execute, sarek.Vector
    reduction = open(os.path.join(IR_DIR, "reduction.ir")).read()
    for n in (4097, 100003):
        nblocks = (n + 255) // 256
        rng = np.random.default_rng(seed * 7 + n)
        inputs = [(rng.standard_normal(n) * 10.0 ** rng.integers(-2, 2, n)).astype(np.float32) for _ in range(n_in)]

        def run(pipeline):
            out = V.create(V.float32, n)
            out.host[:] = np.nan
            args = [E.Vec(V.of_array(x)) for x in inputs] + [E.Vec(out), E.Float32(0.75), E.Float32(-1.25), E.Int32(3),
                                                            E.Int32(n)]
            shape = ((256, 1, 1), (nblocks, 1, 1))
            if not pipeline:
                return E.run_vectors(ir, args, *shape), out.to_array().copy(), None
            sums = V.create(V.float32, nblocks)
            path = E.run_pipeline([(ir, args) + shape, (reduction, [E.Vec(out), E.Vec(sums), E.Int32(n)]) + shape])
            fused_sums = sums.to_array().copy()
            assert E.run_vectors(reduction, [E.Vec(out), E.Vec(sums), E.Int32(n)], *shape) == \
                ("reduce_sum_block256_f32" if pipeline == "on" else "jit")
            return path, out.to_array().copy(), (fused_sums, sums.to_array().copy())

        (p_map, got, _), (p_jit, want, _) = both_ways(hip, lambda: run(None))
        assert (p_map, p_jit) == ("map_f32", "jit"), (seed, n)
        same = got.view(np.uint32) == want.view(np.uint32)
        assert bool((same | (np.isnan(got) & np.isnan(want))).all()), (seed, n, int((~same).sum()))
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
        path, fused, (fused_sums, hand_sums) = run("on")
        assert path == ("map_f32+reduce_sum_block256_f32", 1), (seed, n)
        same = fused.view(np.uint32) == want.view(np.uint32)
        assert bool((same | (np.isnan(fused) & np.isnan(want))).all()), (seed, n)
        same = fused_sums.view(np.uint32) == hand_sums.view(np.uint32)
        assert bool((same | (np.isnan(fused_sums) & np.isnan(hand_sums))).all()), (seed, n)


def test_a_map_that_binds_a_name_again(hip, sarek):
    """out[i] = let t = x[i] * a in let t = t + x[i] in let a = t * t in a - b: lets that reuse a name and then a
    parameter's, which the lowering prints as t_2 and a_2.  Rebuilt or generated, alone or compiled into the block
    sums' kernel, the map writes the bits of the expression evaluated in OCaml's scoping."""
    E, V = sarek.Execute, sarek.Vector
    n = 4096 + 37
    nblocks = (n + 255) // 256
    tid = "(var tid 9 i32)"
    xi = f"(read x {tid})"
    body = (f"(let (var t 10 f32) (mul {xi} (var a 3 f32)) (let (var t 11 f32) (add (var t 10 f32) {xi}) "
            f"(let (var a 12 f32) (mul (var t 11 f32) (var t 11 f32)) "
            f"(assign (lelem out {tid}) (sub (var a 12 f32) (var b 4 f32))))))")
    ir = ("(kernel sarek_kern (params (param (var x 1 (vec f32))) (param (var out 2 (vec f32))) (param (var a 3 f32)) "
          f"(param (var b 4 f32)) (param (var n 5 i32))) (locals) (body (let {tid} (intr (Std) global_thread_id) "
          f"(if (lt {tid} (var n 5 i32)) {body}))) (native_fn true))")
    text = hip.generate_source(ir)
    assert "float t_2 = (t + x[tid]);" in text and "float a_2 = (t_2 * t_2);" in text
    reduction = open(os.path.join(IR_DIR, "reduction.ir")).read()
    x = np.random.default_rng(5).standard_normal(n).astype(np.float32)
    a, b = np.float32(1.25), np.float32(-0.375)
    t2 = x * a + x
    want = t2 * t2 - b
    shape = ((256, 1, 1), (nblocks, 1, 1))

    def run(pipeline):
        out = V.create(V.float32, n)
        out.host[:] = np.nan
        args = [E.Vec(V.of_array(x)), E.Vec(out), E.Float32(a), E.Float32(b), E.Int32(n)]
        if not pipeline:
            return E.run_vectors(ir, args, *shape), out.to_array().copy()
        sums = V.create(V.float32, nblocks)
        path = E.run_pipeline([(ir, args) + shape, (reduction, [E.Vec(out), E.Vec(sums), E.Int32(n)]) + shape])
        fused_sums = sums.to_array().copy()
        E.run_vectors(reduction, [E.Vec(out), E.Vec(sums), E.Int32(n)], *shape)
        return path, out.to_array().copy(), fused_sums, sums.to_array().copy()

    (p_map, got), (p_jit, generated) = both_ways(hip, lambda: run(False))
    assert (p_map, p_jit) == ("map_f32", "jit")
    assert np.array_equal(got, want) and np.array_equal(generated, want)
    hip.check(hip.lib.sarek_hip_set_specialisation(1))
    path, fused, fused_sums, hand_sums = run(True)
    assert path == ("map_f32+reduce_sum_block256_f32", 1)
    assert np.array_equal(fused, want) and np.array_equal(fused_sums, hand_sums)


@pytest.mark.parametrize("maximum", [False, True])
@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_MAP_SEEDS", "32")) // 2))
def test_seeded_random_trees(hip, sarek, torch_cuda, seed, maximum):
    """The block-256 sum and maximum trees with seeded expressions where they read their input.  Sum: the hand
    block-256 kernel's sums of the expression's values (the values the map kernel of the same expression stores), bit
    for bit, and the generated tree's within the sum's tolerance.  Maximum: the generated tree's maxima, bit for bit."""
    from map_kernels import random_tree
    torch = torch_cuda
    E, V = sarek.Execute, sarek.Vector
    tree_ir, map_ir, n_in = random_tree(seed, maximum)
    for n in (4097, 100003):
        nblocks = (n + 255) // 256
        rng = np.random.default_rng(seed * 11 + n)
        inputs = [(rng.standard_normal(n) * 10.0 ** rng.integers(-2, 2, n)).astype(np.float32) for _ in range(n_in)]
        scalars = [E.Float32(0.75), E.Float32(-1.25), E.Int32(3), E.Int32(n)]

        def run_tree():
            out = V.create(V.float32, nblocks)
            out.host[:] = -7.0
            args = [E.Vec(V.of_array(x)) for x in inputs] + [E.Vec(out)] + scalars
            return E.run_vectors(tree_ir, args, (256, 1, 1), (nblocks, 1, 1)), out.to_array().copy()

        (p_hand, got), (p_jit, want) = both_ways(hip, run_tree)
        assert (p_hand, p_jit) == ("tree_max_map_f32" if maximum else "tree_sum_map_f32", "jit"), (seed, n)
        same = got.view(np.uint32) == want.view(np.uint32)
        if maximum:
            assert bool((same | (np.isnan(got) & np.isnan(want))).all()), (seed, n, int((~same).sum()))
            continue
        values = V.create(V.float32, n)
        hip.check(hip.lib.sarek_hip_set_specialisation(0))
        try:
            args = [E.Vec(V.of_array(x)) for x in inputs] + [E.Vec(values)] + scalars
            assert E.run_vectors(map_ir, args, (256, 1, 1), (nblocks, 1, 1)) == "jit"
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
        vals = values.to_array().copy()
        ref = hip.reduce_sum_block256(torch.from_numpy(vals).cuda()).cpu().numpy()
        same = got.view(np.uint32) == ref.view(np.uint32)
        assert bool((same | (np.isnan(got) & np.isnan(ref))).all()), (seed, n, int((~same).sum()))
        finite = np.isfinite(vals)
        bound = np.add.reduceat(np.where(finite, np.abs(vals.astype(np.float64)), 0.0), np.arange(0, n, 256)) * 1e-5 + 1e-30
        ok = np.abs(got.astype(np.float64) - want.astype(np.float64)) <= bound
        blocks_finite = np.logical_and.reduceat(finite, np.arange(0, n, 256))
        assert bool((ok | ~blocks_finite).all()), (seed, n)


def test_pairs_the_fused_kernel_does_not_serve(hip, sarek):
    E, V = sarek.Execute, sarek.Vector
    n = 70000
    nblocks = (n + 255) // 256
    reduction = open(os.path.join(IR_DIR, "reduction.ir")).read()
    rng = np.random.default_rng(1)
    ir = MAPS["scale"]()
    args, out = arguments(sarek, "scale", n, rng)
    sums = V.create(V.float32, nblocks)
    other = V.of_array(rng.standard_normal(n).astype(np.float32))
    shape = ((256, 1, 1), (nblocks, 1, 1))
    # the sum reads another vector, or fewer elements
    assert E.run_pipeline([(ir, args) + shape, (reduction, [E.Vec(other), E.Vec(sums), E.Int32(n)]) + shape]) == \
        ("map_f32;reduce_sum_block256_f32", 2)
    assert E.run_pipeline([(ir, args) + shape, (reduction, [E.Vec(out), E.Vec(sums), E.Int32(n - 256)], (256, 1, 1),
                                                (nblocks - 1, 1, 1))]) == ("map_f32;reduce_sum_block256_f32", 2)
    # a launch that does not reach every element runs as generated
    assert E.run_vectors(ir, args, (256, 1, 1), (nblocks - 1, 1, 1)) == "jit"


@pytest.mark.parametrize("n", [1, 255, 256, 257, 2047, 2048, 8191, 8192, 8193, 100003, (1 << 20) + 5])
@pytest.mark.parametrize("name", sorted(TREES))
def test_tree_sum_with_an_expression_in_front(hip, sarek, torch_cuda, name, n):
    """Served in the hand block-256 kernel's shape: the sums are that kernel's on the vector of the expression's
    values, bit for bit, and the generated tree's within the sum's tolerance."""
    torch = torch_cuda
    E, V = sarek.Execute, sarek.Vector
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 10.0 ** rng.integers(-2, 2, n)).astype(np.float32)
    y = (rng.standard_normal(n) * 10.0 ** rng.integers(-2, 2, n)).astype(np.float32)
    nblocks = (n + 255) // 256
    alpha = np.float32(0.37)
    if name == "sum_of_squares":
        values, tail = x * x, lambda out: [E.Vec(V.of_array(x)), E.Vec(out), E.Int32(n)]
    elif name == "short_named_tree":
        values = (alpha * x) * y
        tail = lambda out: [E.Vec(V.of_array(x)), E.Vec(V.of_array(y)), E.Vec(out), E.Float32(float(alpha)), E.Int32(n)]  # noqa: E731
    elif name == "weighted_abs_sum":
        values = (alpha * np.abs(x)) * y
        tail = lambda out: [E.Vec(V.of_array(x)), E.Vec(V.of_array(y)), E.Vec(out), E.Float32(float(alpha)), E.Int32(n)]  # noqa: E731
    else:
        values, tail = (x - y) * (x - y), lambda out: [E.Vec(V.of_array(x)), E.Vec(V.of_array(y)), E.Vec(out), E.Int32(n)]
    ir = TREES[name]()

    def run():
        out = V.create(V.float32, nblocks + 3)
        out.host[:] = -7.0
        path = E.run_vectors(ir, tail(out), (256, 1, 1), (nblocks, 1, 1))
        return path, out.to_array().copy()

    (p_hand, got), (p_jit, want) = both_ways(hip, run)
    assert (p_hand, p_jit) == ("tree_sum_map_f32", "jit")
    assert np.all(got[nblocks:] == -7.0) and np.all(want[nblocks:] == -7.0)
    ref = hip.reduce_sum_block256(torch.from_numpy(values).cuda()).cpu().numpy()
    assert np.array_equal(got[:nblocks].view(np.uint32), ref.view(np.uint32))
    bound = np.add.reduceat(np.abs(values.astype(np.float64)), np.arange(0, n, 256)) * 1e-5 + 1e-30
    assert np.all(np.abs(got[:nblocks].astype(np.float64) - want[:nblocks].astype(np.float64)) <= bound)
    # a grid that is not exactly ceil(n / 256) blocks is left to the generated kernel
    out = V.create(V.float32, nblocks + 3)
    assert E.run_vectors(ir, tail(out), (256, 1, 1), (nblocks + 1, 1, 1)) == "jit"


@pytest.mark.parametrize("n", [1, 255, 256, 257, 2047, 2048, 8193, 100003, (1 << 20) + 5])
@pytest.mark.parametrize("name", sorted(MAX_TREES))
def test_tree_maximum_with_an_expression_in_front(hip, sarek, torch_cuda, name, n):
    """The tree's comparisons in the tree's order: the maxima are the generated kernel's bit for bit (NaNs and a
    last block filled with the kernel's own fill value included), and the hand maximum's on the expression's values."""
    torch = torch_cuda
    E, V = sarek.Execute, sarek.Vector
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 10.0 ** rng.integers(-2, 2, n)).astype(np.float32)
    y = (rng.standard_normal(n) * 10.0 ** rng.integers(-2, 2, n)).astype(np.float32)
    if n > 300:
        x[17], x[n // 2], y[n - 3] = np.nan, np.inf, -np.inf
    nblocks = (n + 255) // 256
    if name == "max_abs":
        values, pad, tail = np.abs(x), 0.0, lambda out: [E.Vec(V.of_array(x)), E.Vec(out), E.Int32(n)]
    else:
        values, pad = np.abs(x - y), -1000000.0
        tail = lambda out: [E.Vec(V.of_array(x)), E.Vec(V.of_array(y)), E.Vec(out), E.Int32(n)]  # noqa: E731
    ir = MAX_TREES[name]()

    def run():
        out = V.create(V.float32, nblocks + 3)
        out.host[:] = -7.0
        path = E.run_vectors(ir, tail(out), (256, 1, 1), (nblocks, 1, 1))
        return path, out.to_array().copy()

    (p_hand, got), (p_jit, want) = both_ways(hip, run)
    assert (p_hand, p_jit) == ("tree_max_map_f32", "jit")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ref = hip.reduce_max_block256(torch.from_numpy(values).cuda(), pad=pad).cpu().numpy()
    assert np.array_equal(got[:nblocks].view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("n", [1, 255, 257, 4095, 4097, 100003, (1 << 20) + 5])
@pytest.mark.parametrize("name", ["saxpy_with_let", "norm3", "scale"])
def test_map_then_block_maximum_is_one_launch(hip, sarek, name, n):
    """The maximum tree of bench_reduction_max.ml behind a map: the tree's comparisons in the tree's order, so the
    maxima are the generated pair's bit for bit (NaNs from norm3's 0/0-free but inf-prone division included)."""
    from test_ir_lowering import reduction_max_ir
    E, V = sarek.Execute, sarek.Vector
    ir, reduction_max = MAPS[name](), reduction_max_ir("(f32 -3.5)")
    nblocks = (n + 255) // 256

    def run():
        args, out = arguments(sarek, name, n, np.random.default_rng(n))
        maxima = V.create(V.float32, nblocks + 2)
        maxima.host[:] = -7.0
        stages = [(ir, args, (256, 1, 1), (nblocks, 1, 1)),
                  (reduction_max, [E.Vec(out), E.Vec(maxima), E.Int32(n)], (256, 1, 1), (nblocks, 1, 1))]
        return E.run_pipeline(stages), out.to_array().copy(), maxima.to_array().copy()

    (fused, a_fused, m_fused), (jit, a_jit, m_jit) = both_ways(hip, run)
    assert fused[1] == 1 and fused[0].startswith("map_f32+reduce_max_block256_f32:") and jit == ("jit;jit", 2)
    assert np.array_equal(a_fused.view(np.uint32), a_jit.view(np.uint32))
    assert np.array_equal(m_fused.view(np.uint32), m_jit.view(np.uint32))
    assert np.all(m_fused[nblocks:] == -7.0)
