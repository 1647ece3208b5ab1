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
