"""Seeded integer programs through the generic route -- IR, lowered text, the run-time compiler, a launch -- against a
walker of the IR written from the reference's own (tests/ir_programs.py; sarek/sarek/Sarek_ir_interp.ml:76-91,
171-266, 844-941).  The programs are lets, mutable variables, assignments, branches, `for` loops in both directions,
counted `while` loops and blocks over a handful of names that hide each other all the time, so what is under test
is the statement layer of the lowering: scopes, names bound again, loop bounds, evaluation order.  Integer work:
every element of the output must be the walker's."""
import os

import numpy as np
import pytest

import ir_programs

pytestmark = pytest.mark.gpu

THREADS = 24


def run(sarek, ir, vectors, scalars, block=32):
    E, T, V = sarek.Execute, sarek.Transfer, sarek.Vector
    held = [V.of_array(v) for v in vectors]
    path = E.run_vectors(ir, [E.Vec(v) for v in held] + [E.Int32(s) for s in scalars], (block, 1, 1), (1, 1, 1))
    T.flush()
    assert path == "jit"
    return [v.to_array().copy() for v in held]


@pytest.fixture()
def sarek(hip, torch_cuda):
    from spoc_amd import sarek as s
    s.Device.init()
    return s


@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_PROGRAM_SEEDS", "48"))))
def test_seeded_programs_compute_what_the_walker_computes(hip, sarek, seed):
    ir, x, k = ir_programs.random_program(seed, THREADS)
    want = ir_programs.expected(ir, x, k, THREADS)
    out = np.full(ir_programs.SLOTS * THREADS, -1, np.int32)
    _, got = run(sarek, ir, [x, out], [k, THREADS])
    assert np.array_equal(got, want), (seed, np.flatnonzero(got != want)[:8].tolist())


def test_loop_bounds_the_body_changes(hip, sarek):
    """The three loops whose text tests/test_ir_lowering.py pins, run by one thread: the results OCaml's
    evaluate-the-bounds-once gives."""
    from test_ir_lowering import LOOP_BOUNDS, REBOUND_PARAMS, kernel_with_body
    for name, (body, _, want) in LOOP_BOUNDS.items():
        (got,) = run(sarek, kernel_with_body(body, REBOUND_PARAMS), [np.full(8, -1, np.int32)], [3], block=1)
        assert got.tolist() == want, name


@pytest.mark.parametrize("seed", range(12))
def test_seeded_parameter_lists_arrive_as_given(hip, sarek, seed):
    """Kernels with four to twelve parameters in a seeded order -- int32, int64, float32 and float64 scalars between
    the four output vectors, each vector followed by its injected length -- store every scalar and every length
    into the output of its type: what arrives is what was passed, whatever the mix does to the alignment of the
    parameter block."""
    import random
    rng = random.Random(9000 + seed)
    E, T, V = sarek.Execute, sarek.Transfer, sarek.Vector
    kinds = {"i32": (V.int32, np.int32, E.Int32), "i64": (V.int64, np.int64, E.Int64),
             "f32": (V.float32, np.float32, E.Float32), "f64": (V.float64, np.float64, E.Float64)}
    outs = {t: (f"o_{t}", rng.randint(5, 40)) for t in kinds}                      # output vector of each type, its length
    params = [("vec", t) for t in kinds] + [("scalar", rng.choice(list(kinds))) for _ in range(rng.randint(0, 8))]
    rng.shuffle(params)
    decls, args, stores, want, slot, vid = [], [], [], {t: {} for t in kinds}, {t: 0 for t in kinds}, 1
    vectors = {}
    for what, t in params:
        if what == "vec":
            name, length = outs[t]
            decls.append(f"(param (var {name} {vid} (vec {t})))")
            vectors[t] = V.of_array(np.full(length, 77, kinds[t][1]))
            args.append(E.Vec(vectors[t]))
        else:
            name = f"s{vid}"
            value = {"i32": rng.randint(-2**31, 2**31 - 1), "i64": rng.randint(-2**63, 2**63 - 1),
                     "f32": float(np.float32(rng.uniform(-1e6, 1e6))), "f64": rng.uniform(-1e300, 1e300)}[t]
            decls.append(f"(param (var {name} {vid} {t}))")
            args.append(kinds[t][2](value))
            stores.append(f"(assign (lelem {outs[t][0]} (i32 {slot[t]})) (var {name} {vid} {t}))")
            want[t][slot[t]] = value
            slot[t] += 1
        vid += 1
    for t in kinds:                                         # every vector's injected length, into the int32 output
        stores.append(f"(assign (lelem o_i32 (i32 {slot['i32']})) (len {outs[t][0]}))")
        want["i32"][slot["i32"]] = outs[t][1]
        slot["i32"] += 1
    assert max(slot.values()) <= 5 + 8
    outs_len_ok = all(slot[t] <= outs[t][1] for t in kinds)
    if not outs_len_ok:
        pytest.skip("more scalars of a type than its output holds")
    ir = (f"(kernel sarek_kern (params {' '.join(decls)}) (locals) (body (if (eq (intr (Std) global_thread_id) (i32 0)) "
          f"(seq {' '.join(stores)}))) (native_fn true))")
    assert E.run_vectors(ir, args, (64, 1, 1), (1, 1, 1)) == "jit"
    T.flush()
    for t in kinds:
        got = vectors[t].to_array()
        for k, value in want[t].items():
            assert got[k] == kinds[t][1](value), (seed, t, k, got[k], value)
        assert (got[slot[t]:] == 77).all(), (seed, t)


@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_PROGRAM_SEEDS", "48")) // 2))
def test_seeded_float_programs_compute_what_the_walker_computes(hip, sarek, seed):
    """Float programs whose every value both float types hold exactly (multiples of 1/8 and of powers of two, small):
    sums, products with powers of two, conditionals, floor / ceil / abs, conversions between int32,
    float32 and float64, lets of both types that hide each other.  Nothing is rounded anywhere, so the device's
    float32 and float64 arithmetic, fused or not, gives the walker's values bit for bit."""
    E, T, V = sarek.Execute, sarek.Transfer, sarek.Vector
    ir, x, s = ir_programs.random_float_program(seed, THREADS)
    want, want_wide = ir_programs.expected_floats(ir, x, s, THREADS)
    out = V.of_array(np.full(ir_programs.SLOTS * THREADS, -1, np.float32))
    wide = V.of_array(np.full(ir_programs.SLOTS * THREADS, -1, np.float64))
    path = E.run_vectors(ir, [E.Vec(V.of_array(x)), E.Vec(out), E.Float32(s), E.Vec(wide), E.Int32(THREADS)], (32, 1, 1), (1, 1, 1))
    T.flush()
    assert path in ("jit", "map_f32")
    got, got_wide = out.to_array(), wide.to_array()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (seed, np.flatnonzero(got != want)[:8].tolist())
    assert np.array_equal(got_wide.view(np.uint64), want_wide.view(np.uint64)), (seed, np.flatnonzero(got_wide != want_wide)[:8].tolist())


@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_PROGRAM_SEEDS", "48")) // 2))
def test_seeded_supersteps_over_shared_arrays(hip, sarek, seed):
    """Block-level programs: two shared arrays (one sized by the block dimension), two to six supersteps separated by
    barriers, each writing the thread's own slot from slots other threads wrote in earlier supersteps (seeded strides
    and offsets round the block), three blocks of 64 threads.  The walker runs a block superstep by superstep; every
    element of the output is its."""
    E, T, V = sarek.Execute, sarek.Transfer, sarek.Vector
    block, grid = 64, 3
    ir, x, k = ir_programs.random_block_program(seed, block, grid)
    want = np.full(x.size, -1, np.int32)
    ir_programs.evaluate_blocks(ir, {"x": x.copy(), "out": want, "k": k}, block, grid)
    out = V.of_array(np.full(x.size, -1, np.int32))
    assert E.run_vectors(ir, [E.Vec(V.of_array(x)), E.Vec(out), E.Int32(k)], (block, 1, 1), (grid, 1, 1)) == "jit"
    T.flush()
    got = out.to_array()
    assert np.array_equal(got, want), (seed, np.flatnonzero(got != want)[:8].tolist())


@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_PROGRAM_SEEDS", "48")) // 2))
def test_seeded_record_programs_compute_what_the_walker_computes(hip, sarek, seed):
    """Programs over point {x; y} and seg {a : point; b : point; w}: literals, elements of record vectors, fields of
    fields, conditionals between records, a helper from seg to point, mutable records whose fields are assigned,
    stores of whole records and of single fields.  The two record vectors and the int32 output end as the walker
    leaves them."""
    E, T, V = sarek.Execute, sarek.Transfer, sarek.Vector
    ir, ps, ss = ir_programs.random_record_program(seed, THREADS)
    want_ps, want_ss, want_out = ir_programs.expected_records(ir, ps, ss, THREADS)
    vps, vss = V.create_custom(8, THREADS), V.create_custom(20, THREADS)
    vps.host.view(np.int32).reshape(THREADS, 2)[:] = ps
    vss.host.view(np.int32).reshape(THREADS, 5)[:] = ss
    out = V.of_array(np.full(ir_programs.SLOTS * THREADS, -1, np.int32))
    assert E.run_vectors(ir, [E.Vec(vps), E.Vec(vss), E.Vec(out), E.Int32(THREADS)], (32, 1, 1), (1, 1, 1)) == "jit"
    T.flush()
    assert np.array_equal(out.to_array(), want_out), (seed, "out")
    assert np.array_equal(vps.to_array().view(np.int32).reshape(THREADS, 2), want_ps), (seed, "ps")
    assert np.array_equal(vss.to_array().view(np.int32).reshape(THREADS, 5), want_ss), (seed, "ss")


@pytest.mark.parametrize("seed", range(6))
def test_every_geometry_intrinsic_under_seeded_three_dimensional_launches(hip, sarek, seed):
    """thread_idx / block_idx / block_dim / grid_dim in x, y and z (both spellings of the indices), the global indices
    and global_size, stored by every thread of a seeded three-dimensional launch at its linear position: what the
    reference's walker computes for them (sarek/sarek/Sarek_ir_interp.ml:296-375: global_idx_a = block_idx_a *
    block_dim_a + thread_idx_a)."""
    import random
    rng = random.Random(4242 + seed)
    E, T, V = sarek.Execute, sarek.Transfer, sarek.Vector
    block = (rng.choice([1, 3, 8, 16]), rng.choice([1, 2, 4]), rng.choice([1, 2, 3]))
    grid = (rng.randint(1, 5), rng.randint(1, 4), rng.randint(1, 3))
    names = ["thread_idx_x", "thread_idx_y", "thread_idx_z", "block_idx_x", "block_idx_y", "block_idx_z",
             "block_dim_x", "block_dim_y", "block_dim_z", "grid_dim_x", "grid_dim_y", "grid_dim_z",
             "global_idx_x", "global_idx_y", "global_idx_z", "global_thread_id", "global_size",
             "thread_id_x", "block_id_y"]
    g = lambda n: f"(intr (Gpu) {n})"
    gx, gy, gz = g("global_idx_x"), g("global_idx_y"), g("global_idx_z")
    wx = f"(mul {g('block_dim_x')} {g('grid_dim_x')})"
    wy = f"(mul {g('block_dim_y')} {g('grid_dim_y')})"
    linear = f"(add {gx} (mul {wx} (add {gy} (mul {wy} {gz}))))"
    stores = " ".join(f"(assign (lelem out (add (mul (var at 9 i32) (i32 {len(names)})) (i32 {k}))) {g(n)})"
                      for k, n in enumerate(names))
    ir = (f"(kernel sarek_kern (params (param (var out 1 (vec i32)))) (locals) (body (let (var at 9 i32) {linear} "
          f"(seq {stores}))) (native_fn true))")
    total = block[0] * block[1] * block[2] * grid[0] * grid[1] * grid[2]
    out = V.of_array(np.full(total * len(names), -1, np.int32))
    assert E.run_vectors(ir, [E.Vec(out)], block, grid) == "jit"
    T.flush()
    got = out.to_array().reshape(total, len(names))
    width = (block[0] * grid[0], block[1] * grid[1])
    for bz in range(grid[2]):
        for by in range(grid[1]):
            for bx in range(grid[0]):
                for tz in range(block[2]):
                    for ty in range(block[1]):
                        for tx in range(block[0]):
                            ix, iy, iz = bx * block[0] + tx, by * block[1] + ty, bz * block[2] + tz
                            want = [tx, ty, tz, bx, by, bz, *block, *grid, ix, iy, iz, ix, block[0] * grid[0], tx, by]
                            at = ix + width[0] * (iy + width[1] * iz)
                            assert got[at].tolist() == want, (seed, block, grid, at)
