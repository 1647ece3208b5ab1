"""More kernels of the reference's end-to-end suite (sarek/tests/e2e/) through the plugin path:
the let%shared / let%superstep family (sizes left to the block dimension included), shared and
global atomics, an if / else-if chain, an unroll pragma, barriers inside loops, a 2-D launch.
IR transcribed from the cited kernel sources with the rules of sarek/ppx/Sarek_lower_ir.ml
(let%shared with no size -> block_dim_x elements :496-507; let%superstep -> block; barrier
:508-515)."""
import numpy as np
import pytest

from spoc_amd.reference_kernels import (BARRIER, KERNELS, add, assign_elem, assign_var, block, f32, for_, fresh, i32,
                                        if_, intr, kernel, land, let, letmut, lets, lt, mod, mul, op, read, seq, sub,
                                        var, while_)

pytestmark = pytest.mark.gpu

TIDX = intr("thread_idx_x")
GTID = intr("global_thread_id", "Std")


def run(hip, ir, block, grid, items, shared_mem=0, expect="jit"):
    path = hip.run_source(hip.generate_source(ir, block=block), "sarek_kern", block, grid, items, shared_mem=shared_mem)
    hip.check(hip.lib.sarek_hip_device_synchronize())
    assert path == expect


def shared_n(name, ty, size_expr, body):
    return let(var(name, f"(array {ty} shared)"), f"(newarray {ty} {size_expr} shared)", body)


BLOCK_DIM = "(intr (Sarek_stdlib Gpu) block_dim_x)"          # what an unsized let%shared lowers to


@pytest.mark.parametrize("block_size", [64, 256])
def test_superstep_family(hip, torch_cuda, block_size):
    """test_superstep.ml:18-86, all seven kernels; the reference only compiles them."""
    torch = torch_cuda
    n = block_size * 5
    x = torch.arange(n, dtype=torch.float32, device="cuda") * 0.5
    params = [("input", "(vec f32)"), ("output", "(vec f32)")]

    def go(body, expect):
        fresh()
        for p, t in params:
            var(p, t)
        out = torch.full((n,), -1.0, device="cuda")
        run(hip, kernel(params, body), (block_size, 1, 1), (n // block_size, 1, 1), [x, out])
        assert torch.equal(out, expect), body

    load = assign_elem("tile", TIDX, read("input", GTID))
    store = assign_elem("output", GTID, read("tile", TIDX))
    barrier_call = f"(expr {intr('block_barrier')})"
    # 1, 2: explicit barrier; shared array sized by the block, then by a constant
    go(shared_n("tile", "f32", BLOCK_DIM, seq(load, barrier_call, store)), x)
    if block_size <= 64:
        go(shared_n("tile", "f32", i32(64), seq(load, barrier_call, store)), x)
    # 3, 4: supersteps
    go(shared_n("tile", "f32", BLOCK_DIM, seq(block(load), BARRIER, store)), x)
    bump = let(var("v", "f32"), add(read("tile", TIDX), f32("1.0")), assign_elem("tile", TIDX, var("v", "f32")))
    go(shared_n("tile", "f32", BLOCK_DIM, seq(block(load), BARRIER, seq(block(bump), BARRIER, store))), x + 1.0)
    # 5: divergent superstep: thread 0 of every block writes output[0] (same value race: block 0's
    # tile[0] is input[0] only for block 0, so restrict the check to a single block launch)
    fresh()
    for p, t in params:
        var(p, t)
    out = torch.full((n,), -1.0, device="cuda")
    fin = if_(op("eq", TIDX, i32(0)), assign_elem("output", i32(0), read("tile", i32(0))))
    body = shared_n("tile", "f32", BLOCK_DIM, seq(block(load), BARRIER, seq(block(fin), BARRIER, "(expr (unit))")))
    run(hip, kernel(params, body), (block_size, 1, 1), (1, 1, 1), [x, out])
    assert out[0].item() == 0.0 and bool((out[1:] == -1.0).all())
    # 6: block-uniform condition inside a superstep
    cond_load = if_(op("gt", intr("block_idx_x"), i32(0)), load, assign_elem("tile", TIDX, f32("0.0")))
    exp = x.clone()
    exp[:block_size] = 0.0
    go(shared_n("tile", "f32", BLOCK_DIM, seq(block(cond_load), BARRIER, store)), exp)
    # 7: two shared arrays, one sized by the block and one by a constant
    two = seq(assign_elem("tile1", TIDX, read("input", GTID)),
              assign_elem("tile2", TIDX, add(read("input", GTID), f32("1.0"))))
    both = assign_elem("output", GTID, add(read("tile1", TIDX), read("tile2", TIDX)))
    go(shared_n("tile1", "f32", BLOCK_DIM, shared_n("tile2", "f32", i32(max(32, block_size)),
                                                    seq(block(two), BARRIER, both))), x + (x + 1.0))


def test_unsized_shared_needs_the_block(hip, torch_cuda):
    """Without the launch block the declaration keeps blockDim.x, as the reference's generator
    writes it, and the device compiler refuses it."""
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)")]
    for p, t in params:
        var(p, t)
    ir = kernel(params, shared_n("tile", "f32", BLOCK_DIM, assign_elem("output", GTID, read("input", GTID))))
    assert "__shared__ float tile[blockDim.x];" in hip.generate_source(ir)
    assert "__shared__ float tile[128];" in hip.generate_source(ir, block=(128, 1, 1))
    x = torch_cuda.zeros(128, device="cuda")
    with pytest.raises(hip.SarekHipError) as e:
        hip.run_source(hip.generate_source(ir), "sarek_kern", (128, 1, 1), (1, 1, 1), [x, x])
    assert e.value.status == hip.E_COMPILE


@pytest.mark.parametrize("strided", [False, True])
def test_histogram_shared_and_global_atomics(hip, torch_cuda, strided):
    """test_histogram.ml:43-96: per-block histogram in shared memory by atomic adds, merged into
    the global one by atomic adds; the strided form walks the input in a while loop."""
    torch = torch_cuda
    n, bins = 100003, 256
    data = np.random.default_rng(42).integers(0, bins, n).astype(np.int32)
    fresh()
    params = [("input", "(vec i32)"), ("histogram", "(vec i32)"), ("n", "i32"), ("num_bins", "i32")]
    for p, t in params:
        var(p, t)
    nn, nb = var("n"), var("num_bins")
    tid, gid, stride, i = var("tid"), var("gid"), var("stride"), var("i", mut=True)
    lh = var("local_hist", "(array i32 shared)")
    count_one = lambda idx: let(var("bin"), mod(read("input", idx), nb),                     # noqa: E731
                                let(var("_old"), intr("atomic_add_int32", "Gpu", lh, var("bin"), i32(1)), "(expr (unit))"))
    merge = if_(lt(tid, nb), let(var("_old2").replace("_old2", "_old", 1),
                                 intr("atomic_add_global_int32", "Gpu", var("histogram", "(vec i32)"), tid,
                                      read("local_hist", tid)), "(expr (unit))"))
    init = block(if_(lt(tid, nb), assign_elem("local_hist", tid, i32(0))))
    if strided:
        body = lets([(tid, TIDX), (gid, GTID), (stride, mul(intr("block_dim_x"), intr("grid_dim_x")))],
                    seq(init, BARRIER,
                        letmut(i, gid, seq(while_(lt(i, nn), seq(count_one(i), assign_var(i, add(i, stride)))),
                                           f"(expr {intr('block_barrier')})", merge))))
        grid = 64
    else:
        body = lets([(tid, TIDX), (gid, GTID)],
                    seq(init, BARRIER, seq(block(if_(lt(gid, nn), count_one(gid))), BARRIER,
                                           seq(block(merge), BARRIER, "(expr (unit))"))))
        grid = (n + 255) // 256
    ir = kernel(params, let(lh, "(newarray i32 (i32 256) shared)", body))
    # the one-key-per-thread form is the bench kernel: the plugin takes it over; with that switched
    # off it runs as generated, like the strided form
    for specialise in (1, 0):
        hist = torch.zeros(bins, dtype=torch.int32, device="cuda")
        hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
        try:
            run(hip, ir, (256, 1, 1), (grid, 1, 1), [torch.from_numpy(data).cuda(), hist, ("i32", n), ("i32", bins)],
                shared_mem=bins * 4, expect="histogram_i32" if specialise and not strided else "jit")
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
        assert np.array_equal(hist.cpu().numpy(), np.bincount(data, minlength=bins))


def test_convolution_if_else_if_chain(hip, torch_cuda):
    """test_convolution.ml: a 1-2-1 filter inside, the input copied at the two ends."""
    torch = torch_cuda
    n = 50001
    x = np.random.default_rng(3).random(n).astype(np.float32)
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid, nn = var("tid"), var("n")
    l, c, r = var("left", "f32"), var("center", "f32"), var("right", "f32")
    inner = lets([(l, read("input", sub(tid, i32(1)))), (c, read("input", tid)), (r, read("input", add(tid, i32(1))))],
                 assign_elem("output", tid, add(add(mul(f32("0.25"), l), mul(f32("0.5"), c)), mul(f32("0.25"), r))))
    ends = if_(op("or", op("eq", tid, i32(0)), op("eq", tid, sub(nn, i32(1)))), assign_elem("output", tid, read("input", tid)))
    ir = kernel(params, let(tid, GTID, if_(land(op("gt", tid, i32(0)), lt(tid, sub(nn, i32(1)))), inner, ends)))
    out = torch.full((n + 200,), -1.0, device="cuda")
    run(hip, ir, (256, 1, 1), ((n + 255) // 256, 1, 1), [torch.from_numpy(x).cuda(), out, ("i32", n)])
    exp = x.copy()
    exp[1:-1] = (np.float32(0.25) * x[:-2] + np.float32(0.5) * x[1:-1]) + np.float32(0.25) * x[2:]
    got = out.cpu().numpy()
    assert np.allclose(got[:n], exp, rtol=1e-6) and np.all(got[n:] == -1.0)


def test_unroll_pragma_and_barrier_in_loop(hip, torch_cuda):
    """test_pragma.ml (pragma ["unroll"] over a 4-step loop) and test_barrier_converged.ml
    (a barrier in a uniform loop; an if as an expression before a barrier)."""
    torch = torch_cuda
    fresh()
    params = [("a", "(vec i32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid, s, i = var("tid"), var("sum", mut=True), var("i", mut=True)
    loop = f"(pragma (unroll) {for_(i, i32(0), i32(3), assign_var(s, add(s, read('a', add(tid, i)))))})"
    ir = kernel(params, let(tid, TIDX, letmut(s, i32(0), seq(loop, assign_elem("a", tid, s)))))
    src = hip.generate_source(ir)
    assert "#pragma unroll" in src
    # one wave, so every lane reads its neighbours before any lane stores (the kernel has no barrier)
    a = torch.arange(64 + 3, dtype=torch.int32, device="cuda")
    run(hip, ir, (64, 1, 1), (1, 1, 1), [a, ("i32", 64)])
    base = np.arange(67)
    assert np.array_equal(a.cpu().numpy()[:64], base[:64] * 4 + 6)

    fresh()
    params = [("v", "(vec f32)")]
    for p, t in params:
        var(p, t)
    x = var("x", "f32")
    pick = f"(if {op('gt', TIDX, i32(16))} {f32('1.0')} {f32('2.0')})"
    spin = for_(var("_i", mut=True), i32(0), i32(10), f"(expr {intr('block_barrier')})")
    ir = kernel(params, let(x, pick, seq(spin, f"(expr {intr('block_barrier')})", assign_elem("v", TIDX, x))))
    v = torch.zeros(64, device="cuda")
    run(hip, ir, (64, 1, 1), (1, 1, 1), [v])
    assert np.array_equal(v.cpu().numpy(), np.where(np.arange(64) > 16, 1.0, 2.0).astype(np.float32))


def test_mandelbrot_two_dimensional_launch(hip, torch_cuda):
    """test_mandelbrot.ml / benchmarks/bench_mandelbrot.ml through a 16x16 launch; iteration counts
    against the same recurrence in float32 (the device compiler may contract a multiply-add, which
    moves a pixel on the set's edge by an iteration: nearly all pixels must agree exactly)."""
    torch = torch_cuda
    w, h, max_iter = 192, 128, 100
    out = torch.full((w * h,), -1, dtype=torch.int32, device="cuda")
    run(hip, KERNELS["mandelbrot"](), (16, 16, 1), (w // 16, h // 16, 1),
        [out, ("i32", w), ("i32", h), ("i32", max_iter)])
    px, py = np.meshgrid(np.arange(w, dtype=np.float32), np.arange(h, dtype=np.float32))
    x0 = np.float32(4.0) * (px / np.float32(w)) - np.float32(2.5)
    y0 = np.float32(3.0) * (py / np.float32(h)) - np.float32(1.5)
    x, y = np.zeros_like(x0), np.zeros_like(x0)
    it = np.zeros(x0.shape, dtype=np.int32)
    for _ in range(max_iter):
        live = (x * x + y * y <= np.float32(4.0)) & (it < max_iter)
        xt = x * x - y * y + x0
        y = np.where(live, np.float32(2.0) * x * y + y0, y)
        x = np.where(live, xt, x)
        it += live
    got = out.cpu().numpy().reshape(h, w)
    assert got.min() >= 0 and got.max() == max_iter
    assert (got == it).mean() > 0.995 and np.abs(got - it).max() <= max_iter


@pytest.mark.parametrize("elt", ["i32", "f32", "f64", "point3d"])
def test_transpose_through_a_shared_helper_at_four_types(hip, torch_cuda, elt):
    """test_transpose.ml:87-138: one module-level helper over 'a vectors, monomorphised at int32,
    float32, float64 and a three-float record; run with Vector / Execute.run_vectors, the record
    vector as a custom vector of 12-byte elements."""
    from spoc_amd.sarek import Execute, Stale_CPU, Vector
    w, h = 37, 53
    n = w * h
    ty = "(record point3d (x f32) (y f32) (z f32))" if elt == "point3d" else elt
    types = "(types (point3d (x f32) (y f32) (z f32)))" if elt == "point3d" else ""
    helper = f"""(func do_transpose (params (var input 20 (vec {ty})) (var output 21 (vec {ty})) (var width 22 i32)
                                          (var height 23 i32) (var tid 24 i32)) unit
      (let (var n 25 i32) (mul (var width 22 i32) (var height 23 i32))
       (if (lt (var tid 24 i32) (var n 25 i32))
        (let (var col 26 i32) (mod (var tid 24 i32) (var width 22 i32))
        (let (var row 27 i32) (div (var tid 24 i32) (var width 22 i32))
        (let (var in_idx 28 i32) (add (mul (var row 27 i32) (var width 22 i32)) (var col 26 i32))
        (let (var out_idx 29 i32) (add (mul (var col 26 i32) (var height 23 i32)) (var row 27 i32))
         (assign (lelem output (var out_idx 29 i32)) (read input (var in_idx 28 i32))))))))))"""
    ir = f"""(kernel sarek_kern (params (param (var input 1 (vec {ty}))) (param (var output 2 (vec {ty})))
                                       (param (var width 3 i32)) (param (var height 4 i32)))
      (locals) (body (expr (app (var do_transpose 30 unit) (var input 1 (vec {ty})) (var output 2 (vec {ty}))
                                (var width 3 i32) (var height 4 i32) (intr (Std) global_thread_id))))
      {types} (funcs {helper}) (native_fn true))"""
    if elt == "point3d":
        vin, vout = Vector.create_custom(12, n), Vector.create_custom(12, n)
        data = np.arange(3 * n, dtype=np.float32).reshape(n, 3)
        vin.host.view(np.float32).reshape(n, 3)[:] = data
        vout.host.view(np.uint8)[:] = 0
    else:
        kind = {"i32": Vector.int32, "f32": Vector.float32, "f64": Vector.float64}[elt]
        vin, vout = Vector.create(kind, n), Vector.create(kind, n)
        data = (np.arange(n) * (1.0 if elt == "i32" else 1.0 + 2.0 ** -30)).astype(kind.dtype)
        vin.fill_from(data)
        vout.fill_from(np.zeros(n))
    path = Execute.run_vectors(ir=ir, args=[Execute.Vec(vin), Execute.Vec(vout), Execute.Int32(w), Execute.Int32(h)],
                               block=Execute.dims1d(256), grid=Execute.dims1d((n + 255) // 256))
    assert path == "jit" and vout.location == Stale_CPU
    if elt == "point3d":
        got = vout.to_array().view(np.float32).reshape(w, h, 3)
        assert np.array_equal(got, data.reshape(h, w, 3).transpose(1, 0, 2))
    else:
        assert np.array_equal(vout.to_array().reshape(w, h), data.reshape(h, w).T)
