"""Seeded random launch geometries for the kernels the plugin recognises.  A hand kernel takes over a launch only when
the caller's block and grid cover the problem the way the generated kernel assumes; under any other geometry (too few
threads, blocks of another width, a grid that overshoots) the generated code runs, and what it leaves -- partial
results included -- is the result.  So for every drawn geometry the launch is made twice, with the hand kernels on and
off, into vectors pre-filled with a guard value, and the two results are compared:

  vector add, copy, naive transpose, histogram, block maximum     bit for bit
  stream triad                                                    one ulp (the generated code is an fma in binary32,
                                                                  the hand kernel the Native backend's double arithmetic)
  naive and tiled matmul                                          1e-4 of max|C|
  block sums, block dot products                                  1e-5 x 256 x the inputs' scale

The kernels are the reference benches' own IR (spoc_amd.reference_kernels); which route served each launch is counted,
and both routes must have been taken for most kernels over the run."""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture()
def sarek(hip, torch_cuda):
    from spoc_amd import sarek as s
    s.Device.init()
    yield s
    hip.check(hip.lib.sarek_hip_set_specialisation(1))


def draw(rng, nrng, E, V, rk):
    """One case: (kind, description, run() -> (path, result array), comparison)."""
    def fvec(x):
        return V.of_array(np.ascontiguousarray(x, dtype=np.float32))

    kind = rng.choice(["triad", "add", "copy", "transpose", "matmul", "matmul_tiled", "sum", "dot", "max", "histogram"])
    if kind in ("triad", "add", "copy"):
        n = rng.choice([1, 100, 255, 256, 257, 1000, 4096, 4097, 70001])
        block = rng.choice([32, 64, 128, 256, 512, 1024])
        need = (n + block - 1) // block
        grid = max(1, need + rng.choice([0, 0, 0, 1, -1, 3, -need // 2]))
        b, c = nrng.standard_normal(n), nrng.standard_normal(n)

        def run():
            out = fvec(np.full(n, 7.0))
            if kind == "triad":
                ir, args = rk.stream_triad(), [E.Vec(out), E.Vec(fvec(b)), E.Vec(fvec(c)), E.Float32(3.0), E.Int32(n)]
            elif kind == "add":
                ir, args = rk.vector_add(), [E.Vec(fvec(b)), E.Vec(fvec(c)), E.Vec(out), E.Int32(n)]
            else:
                ir, args = rk.vector_copy(), [E.Vec(fvec(b)), E.Vec(out), E.Int32(n)]
            return E.run_vectors(ir, args, (block, 1, 1), (grid, 1, 1)), out.to_array().copy()
        return kind, (n, block, grid), run, "ulp" if kind == "triad" else "bits"
    if kind == "transpose":
        w, h = rng.choice([1, 7, 16, 64, 100, 257]), rng.choice([1, 5, 32, 64, 99, 300])
        block = rng.choice([64, 256, 512])
        need = (w * h + block - 1) // block
        grid = max(1, need + rng.choice([0, 0, 1, -1, 2]))
        x = nrng.standard_normal(w * h)

        def run():
            out = fvec(np.full(w * h, 7.0))
            path = E.run_vectors(rk.transpose_naive(), [E.Vec(fvec(x)), E.Vec(out), E.Int32(w), E.Int32(h)],
                                 (block, 1, 1), (grid, 1, 1))
            return path, out.to_array().copy()
        return kind, (w, h, block, grid), run, "bits"
    if kind in ("matmul", "matmul_tiled"):
        m, n, k = rng.choice([1, 16, 17, 48, 100]), rng.choice([1, 16, 33, 64, 72]), rng.choice([1, 8, 16, 52, 64, 100])
        a, b = nrng.standard_normal((m, k)), nrng.standard_normal((k, n))
        if kind == "matmul":
            width = rng.choice([64, 256])
            need = (m * n + width - 1) // width
            ir, block, grid, lds = rk.matrix_mul(), (width, 1, 1), (max(1, need + rng.choice([0, 0, 1, -1])), 1, 1), 0
        else:
            gx, gy = (n + 15) // 16 + rng.choice([0, 0, 1, -1]), (m + 15) // 16 + rng.choice([0, 0, 1, -1])
            ir, block, grid, lds = rk.matrix_mul_tiled(), (16, 16, 1), (max(1, gx), max(1, gy), 1), 2048

        def run():
            out = fvec(np.full(m * n, 7.0))
            args = [E.Vec(fvec(a)), E.Vec(fvec(b)), E.Vec(out), E.Int32(m), E.Int32(n), E.Int32(k)]
            return E.run_vectors(ir, args, block, grid, shared_mem=lds), out.to_array().copy()
        return kind, (m, n, k, block, grid), run, "gemm"
    if kind in ("sum", "dot", "max"):
        n = rng.choice([1, 255, 256, 257, 1000, 4096, 70001])
        need = (n + 255) // 256
        grid = max(1, need + rng.choice([0, 0, 0, 1, -1, 2]))
        x, y = nrng.standard_normal(n), nrng.standard_normal(n)

        def run():
            out = fvec(np.full(max(grid, need) + 2, 7.0))
            if kind == "sum":
                ir, args = rk.tree(False), [E.Vec(fvec(x)), E.Vec(out), E.Int32(n)]
            elif kind == "dot":
                ir, args = rk.tree(True), [E.Vec(fvec(x)), E.Vec(fvec(y)), E.Vec(out), E.Int32(n)]
            else:
                ir, args = rk.reduction_max(-1000000.0), [E.Vec(fvec(x)), E.Vec(out), E.Int32(n)]
            return E.run_vectors(ir, args, (256, 1, 1), (grid, 1, 1)), out.to_array().copy()
        return kind, (n, grid), run, "bits" if kind == "max" else "sums"
    n, bins = rng.choice([1, 100, 256, 1000, 4097, 70001]), rng.choice([1, 16, 100, 256])
    block = rng.choice([64, 128, 256, 512])
    need = (n + block - 1) // block
    grid = max(1, need + rng.choice([0, 0, 1, -1, 2]))
    keys = nrng.integers(0, 1 << 20, n).astype(np.int32)

    def run():
        hist = V.of_array(np.arange(256, dtype=np.int32))
        args = [E.Vec(V.of_array(keys)), E.Vec(hist), E.Int32(n), E.Int32(bins)]
        return E.run_vectors(rk.histogram(), args, (block, 1, 1), (grid, 1, 1), shared_mem=1024), hist.to_array().copy()
    return kind, (n, bins, block, grid), run, "bits"


def agree(how, hand, generated):
    if how == "bits":
        return np.array_equal(hand.view(np.uint32), generated.view(np.uint32))
    if how == "ulp":
        return bool(np.all(np.abs(hand.view(np.int32).astype(np.int64) - generated.view(np.int32).astype(np.int64)) <= 1))
    if how == "gemm":
        return bool(np.all(np.abs(hand - generated) <= 1e-4 * max(1.0, np.abs(generated).max())))
    return bool(np.all(np.abs(hand - generated) <= 1e-5 * 256 * 4))


@pytest.mark.parametrize("seed", [1, 2])
def test_hand_and_generated_routes_agree_under_any_geometry(hip, sarek, seed):
    from spoc_amd import reference_kernels as rk
    E, V = sarek.Execute, sarek.Vector
    rng = random.Random(seed)
    routes, failures = {}, []
    for it in range(200):
        kind, what, run, how = draw(rng, np.random.default_rng(seed * 1000 + it), E, V, rk)
        results = []
        for on in (1, 0):
            hip.check(hip.lib.sarek_hip_set_specialisation(on))
            try:
                results.append(run())
            finally:
                hip.check(hip.lib.sarek_hip_set_specialisation(1))
        (p_hand, r_hand), (p_jit, r_jit) = results
        assert p_jit == "jit"
        routes.setdefault(kind, set()).add("jit" if p_hand == "jit" else "hand")
        if not agree(how, r_hand, r_jit):
            failures.append((seed, it, kind, what, p_hand))
    assert failures == []
    assert all("hand" in r for r in routes.values()), routes
    assert sum("jit" in r for r in routes.values()) >= 6, routes


@pytest.mark.parametrize("seed", [1, 2])
def test_pipelines_agree_with_their_stages_run_as_generated(hip, sarek, seed):
    """Execute.run_pipeline on [producer; block reduction] pairs drawn at random: the stream triad, the vector add or a
    seeded random map in front of the block-256 sum or maximum; geometries that fit or are off by a block, the
    reduction over the producer's vector or another one, over all of it or fewer elements.  One launch serves a pair
    only when the pair is the fused operation; whatever route is taken, the vector and the block results are what the
    two generated kernels leave (triad: one ulp, the hand kernel rounds the double result; sums: 1e-5 x 256 x scale,
    another association; everything else bit for bit)."""
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from map_kernels import random_map
    from spoc_amd import reference_kernels as rk
    E, V = sarek.Execute, sarek.Vector
    rng = random.Random(seed)
    routes, failures = {}, []

    def fvec(x):
        return V.of_array(np.ascontiguousarray(x, dtype=np.float32))

    for it in range(150):
        n = rng.choice([1, 255, 256, 257, 1000, 4096, 4097, 70001, 300000])
        first, second = rng.choice(["triad", "add", "map"]), rng.choice(["sum", "max"])
        blocks = (n + 255) // 256
        n_red = n if rng.random() < 0.8 else max(1, n - rng.choice([1, 256, 300]))
        blocks_red = (n_red + 255) // 256
        g1 = max(1, blocks + rng.choice([0, 0, 0, 1, -1]))
        g2 = max(1, blocks_red + rng.choice([0, 0, 0, 1, -1]))
        another_vector = rng.random() < 0.1
        map_seed = rng.randrange(100)

        def run():
            nrng = np.random.default_rng(seed * 1000 + it)
            out, res = fvec(np.full(n, 7.0)), fvec(np.full(max(g2, blocks_red) + 2, 7.0))
            b, c = fvec(nrng.standard_normal(n)), fvec(nrng.standard_normal(n))
            if first == "triad":
                ir, args = rk.stream_triad(), [E.Vec(out), E.Vec(b), E.Vec(c), E.Float32(3.0), E.Int32(n)]
            elif first == "add":
                ir, args = rk.vector_add(), [E.Vec(b), E.Vec(c), E.Vec(out), E.Int32(n)]
            else:
                ir, n_in = random_map(map_seed)
                args = [E.Vec(fvec(nrng.standard_normal(n))) for _ in range(n_in)] + \
                    [E.Vec(out), E.Float32(0.75), E.Float32(-1.25), E.Int32(3), E.Int32(n)]
            source = fvec(np.arange(n) % 7) if another_vector else out
            reduction = rk.tree(False) if second == "sum" else rk.reduction_max(-1000000.0)
            path = E.run_pipeline([(ir, args, (256, 1, 1), (g1, 1, 1)),
                                   (reduction, [E.Vec(source), E.Vec(res), E.Int32(n_red)], (256, 1, 1), (g2, 1, 1))])
            return path, out.to_array().copy(), res.to_array().copy()

        results = []
        for on in (1, 0):
            hip.check(hip.lib.sarek_hip_set_specialisation(on))
            try:
                results.append(run())
            finally:
                hip.check(hip.lib.sarek_hip_set_specialisation(1))
        (path, vec, red), (p_jit, vec_jit, red_jit) = results
        assert p_jit == ("jit;jit", 2)
        routes[path[0]] = routes.get(path[0], 0) + 1
        ulps = np.abs(vec.view(np.int32).astype(np.int64) - vec_jit.view(np.int32).astype(np.int64))
        vec_ok = (ulps <= (1 if first == "triad" else 0)) | (np.isnan(vec) & np.isnan(vec_jit))
        if second == "max":
            red_ok = (red == red_jit) | (np.isnan(red) & np.isnan(red_jit))
        else:
            scale = max(1.0, float(np.abs(np.nan_to_num(vec_jit, nan=0.0, posinf=0.0, neginf=0.0)).max()))
            with np.errstate(invalid="ignore"):              # inf - inf where a random map overflowed
                red_ok = (np.abs(red - red_jit) <= 1e-5 * 256 * scale) | ~np.isfinite(red_jit)
        if not (vec_ok.all() and red_ok.all()):
            failures.append((seed, it, first, second, n, n_red, g1, g2, another_vector, path))
    assert failures == []
    fused = [r for r in routes if "+" in r]
    assert len(fused) >= 5 and "jit;jit" in routes and any(";" in r and r != "jit;jit" for r in routes), routes
