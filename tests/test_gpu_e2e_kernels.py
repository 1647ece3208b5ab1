"""Kernels of the reference's end-to-end suite (sarek/tests/e2e/) through the plugin path on
the GPU: IR -> generate_source -> hiprtc -> launch, results against numpy.  They exercise
what the benchmark kernels do not: bit operations, while loops over mutable locals, math
intrinsics, records in vectors, helper functions, variants with match, expression-level
if, double-buffered shared memory.  The IR is transcribed from the kernel sources cited at
each test with the lowering rules of sarek/ppx/Sarek_lower_ir.ml."""
import numpy as np
import pytest

from spoc_amd.reference_kernels import (BARRIER, add, assign_elem, assign_var, block, div, f32, fresh, i32,
                                        if_, intr, kernel, land, let, letmut, lets, lt, mul, op, read, seq,
                                        shared, sub, var, while_)

pytestmark = pytest.mark.gpu

GID = add(intr("thread_idx_x"), mul(intr("block_dim_x"), intr("block_idx_x")))


def launch(hip, ir, n, items, block=256, shared_mem=0, path="jit"):
    took = hip.run_source(hip.generate_source(ir, block=(block, 1, 1)), "sarek_kern", (block, 1, 1),
                          ((n + block - 1) // block, 1, 1), items, shared_mem=shared_mem)
    hip.check(hip.lib.sarek_hip_device_synchronize())
    assert took == path


def ints(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).cuda()


def test_bitwise_and_shifts(hip, torch_cuda):
    """test_bitwise_ops.ml: land / lor / lxor, lsl / lsr."""
    torch = torch_cuda
    n = 1000
    rng = np.random.default_rng(1)
    a, b = rng.integers(0, 1 << 30, n), rng.integers(0, 1 << 30, n)
    fresh()
    params = [(p, "(vec i32)") for p in ("a", "b", "and_out", "or_out", "xor_out")] + [("n", "i32")]
    for p, t in params:
        var(p, t)
    tid, x, y = var("tid"), var("x"), var("y")
    ir = kernel(params, let(tid, intr("global_thread_id", "Std"), if_(lt(tid, var("n")), lets(
        [(x, read("a", tid)), (y, read("b", tid))],
        seq(assign_elem("and_out", tid, op("bitand", x, y)), assign_elem("or_out", tid, op("bitor", x, y)),
            assign_elem("xor_out", tid, op("bitxor", x, y)))))))
    outs = [torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(3)]
    launch(hip, ir, n, [ints(torch, a), ints(torch, b), *outs, ("i32", n)])
    assert np.array_equal(outs[0].cpu().numpy(), a & b)
    assert np.array_equal(outs[1].cpu().numpy(), a | b)
    assert np.array_equal(outs[2].cpu().numpy(), a ^ b)

    s = rng.integers(0, 8, n)
    fresh()
    params = [(p, "(vec i32)") for p in ("input", "shift_amt", "left_out", "right_out")] + [("n", "i32")]
    for p, t in params:
        var(p, t)
    tid, x, sh = var("tid"), var("x"), var("s")
    ir = kernel(params, let(tid, GID, if_(lt(tid, var("n")), lets(
        [(x, read("input", tid)), (sh, read("shift_amt", tid))],
        seq(assign_elem("left_out", tid, op("shl", x, sh)), assign_elem("right_out", tid, op("shr", x, sh)))))))
    small = rng.integers(0, 1 << 20, n)
    lo, ro = (torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(2))
    launch(hip, ir, n, [ints(torch, small), ints(torch, s), lo, ro, ("i32", n)])
    assert np.array_equal(lo.cpu().numpy(), small << s) and np.array_equal(ro.cpu().numpy(), small >> s)


def test_popcount_while_loop_over_mutables(hip, torch_cuda):
    """test_bitwise_ops.ml (popcount): while x <> 0 do count := count + (x land 1); x := x lsr 1."""
    torch = torch_cuda
    n = 777
    v = np.random.default_rng(2).integers(0, 1 << 31, n)
    fresh()
    params = [("input", "(vec i32)"), ("output", "(vec i32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid, x, count = var("tid"), var("x", "i32", True), var("count", "i32", True)
    ir = kernel(params, let(tid, GID, if_(lt(tid, var("n")), letmut(x, read("input", tid), letmut(count, i32(0), seq(
        while_(op("ne", x, i32(0)), seq(assign_var(count, add(count, op("bitand", x, i32(1)))),
                                       assign_var(x, op("shr", x, i32(1))))),
        assign_elem("output", tid, count)))))))
    out = torch.zeros(n, dtype=torch.int32, device="cuda")
    launch(hip, ir, n, [ints(torch, v), out, ("i32", n)])
    assert np.array_equal(out.cpu().numpy(), [bin(int(q)).count("1") for q in v])


def test_math_intrinsics(hip, torch_cuda):
    """test_math_intrinsics.ml: Float32 math functions lower to the device library's."""
    torch = torch_cuda
    n = 4096
    x = np.random.default_rng(3).uniform(0.1, 4.0, n).astype(np.float32)
    fresh()
    params = [("x", "(vec f32)"), ("out", "(vec f32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid, v = var("tid"), var("v", "f32")

    def m(name, *a):
        return intr(name, "Float32", *a)
    expr = add(add(mul(m("sin", v), m("cos", v)), m("exp", op("sub", f32("0.0"), v))),
               add(m("sqrt", v), add(m("log", add(v, f32("1.0"))), m("pow", v, f32("1.5")))))
    ir = kernel(params, let(tid, intr("global_thread_id", "Std"),
                            if_(lt(tid, var("n")), let(v, read("x", tid), assign_elem("out", tid, expr)))))
    x64 = x.astype(np.float64)
    exp = np.sin(x64) * np.cos(x64) + np.exp(-x64) + np.sqrt(x64) + np.log(x64 + 1) + x64 ** 1.5
    # an element-wise kernel: rebuilt in the stream kernels' shape from the same lowered expression, and as generated
    results = []
    for on, path in ((1, "map_f32"), (0, "jit")):
        out = torch.zeros(n, device="cuda")
        hip.check(hip.lib.sarek_hip_set_specialisation(on))
        try:
            launch(hip, ir, n, [torch.from_numpy(x).cuda(), out, ("i32", n)], path=path)
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
        results.append(out.cpu().numpy())
        assert np.allclose(results[-1], exp, rtol=2e-6, atol=2e-6)
    assert np.array_equal(results[0], results[1])


def test_records_helper_function_and_variant_match(hip, torch_cuda):
    """test_ktype_record.ml / test_klet_fun.ml / test_klet_variant.ml: a vector of {x; y}
    records, a helper function, a variant built and matched inside the kernel."""
    torch = torch_cuda
    n = 500
    pts = np.random.default_rng(4).normal(size=(n, 2)).astype(np.float32)
    point = "(record point (x f32) (y f32))"
    shape = "(variant shape (Circle f32) (Rect f32 f32))"
    ir = f"""
    (kernel sarek_kern
      (params (param (var ps 1 (vec {point}))) (param (var dist 2 (vec f32))) (param (var area 3 (vec f32)))
              (param (var n 4 i32)))
      (locals)
      (body (let (var tid 5 i32) (intr (Std) global_thread_id)
        (if (lt (var tid 5 i32) (var n 4 i32))
          (let (var p 6 {point}) (read ps (var tid 5 i32))
           (seq
            (assign (lelem dist (var tid 5 i32))
                    (intr (Float32) sqrt (add (app (var sq 0 f32) (field (var p 6 {point}) x))
                                              (app (var sq 0 f32) (field (var p 6 {point}) y)))))
            (let (var s 7 {shape})
                 (if (gt (field (var p 6 {point}) x) (f32 0.0))
                     (variant shape Circle (field (var p 6 {point}) x))
                     (variant shape Rect (field (var p 6 {point}) x) (field (var p 6 {point}) y)))
              (match (var s 7 {shape})
                (case (Circle r) (assign (lelem area (var tid 5 i32))
                                         (mul (f32 3.0) (mul (var r 8 f32) (var r 8 f32)))))
                (case (Rect w h) (assign (lelem area (var tid 5 i32)) (mul (var w 9 f32) (var h 10 f32)))))))))))
      (types (point (x f32) (y f32)))
      (variants (shape (Circle f32) (Rect f32 f32)))
      (funcs (func sq (params (var a 11 f32)) f32 (return (mul (var a 11 f32) (var a 11 f32)))))
      (native_fn false))"""
    dist, area = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    launch(hip, ir, n, [("buf", torch.from_numpy(pts).cuda()), ("i32", n), dist, area, ("i32", n)])
    assert np.allclose(dist.cpu().numpy(), np.hypot(pts[:, 0], pts[:, 1]), rtol=1e-6)
    exp = np.where(pts[:, 0] > 0, np.float32(3.0) * pts[:, 0] * pts[:, 0], pts[:, 0] * pts[:, 1])
    assert np.allclose(area.cpu().numpy(), exp, rtol=1e-6)


def test_stencil_1d(hip, torch_cuda):
    """test_stencil.ml:35-46: interior points take the mean of their three neighbours."""
    torch = torch_cuda
    n = 10001
    x = np.random.default_rng(5).random(n).astype(np.float32)
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid = var("tid")
    left, center, right = var("left", "f32"), var("center", "f32"), var("right", "f32")
    ir = kernel(params, let(tid, intr("global_thread_id", "Std"), if_(
        land(op("gt", tid, i32(0)), lt(tid, sub(var("n"), i32(1)))),
        lets([(left, read("input", sub(tid, i32(1)))), (center, read("input", tid)),
              (right, read("input", add(tid, i32(1))))],
             assign_elem("output", tid, div(add(add(left, center), right), f32("3.0")))))))
    out = torch.full((n,), -1.0, device="cuda")
    launch(hip, ir, n, [torch.from_numpy(x).cuda(), out, ("i32", n)])
    exp = np.full(n, -1.0, np.float32)
    exp[1:-1] = ((x[:-2] + x[1:-1]) + x[2:]) / np.float32(3.0)
    assert np.allclose(out.cpu().numpy(), exp, rtol=1e-6)


def test_block_scan_with_two_shared_buffers(hip, torch_cuda):
    """test_scan.ml: inclusive scan of each 256-block, eight supersteps ping-ponging between
    two shared arrays, `let add = if tid >= d then temp.(tid - d) else 0l` as an expression."""
    torch = torch_cuda
    n = 256 * 9 + 100
    v = np.random.default_rng(6).integers(-50, 50, n)
    fresh()
    params = [("input", "(vec i32)"), ("output", "(vec i32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    nn = var("n")
    t1, t2 = var("temp", "(array i32 shared)"), var("temp2", "(array i32 shared)")
    tid, gid = var("tid"), var("gid")
    steps = [block(if_(lt(gid, nn), assign_elem("temp", tid, read("input", gid)), assign_elem("temp", tid, i32(0)))),
             BARRIER]
    src, dst, d = "temp", "temp2", 1
    while d < 256:
        val, inc = var(f"v{d}").replace(f"v{d}", "v", 1), var(f"add{d}").replace(f"add{d}", "add", 1)
        pick = f"(if {op('ge', tid, i32(d))} {read(src, sub(tid, i32(d)))} {i32(0)})"
        steps += [block(let(val, read(src, tid), let(inc, pick, assign_elem(dst, tid, add(val, inc))))), BARRIER]
        src, dst, d = dst, src, 2 * d
    steps.append(if_(lt(gid, nn), assign_elem("output", gid, read(src, tid))))
    ir = kernel(params, shared(t1, "i32", 512, shared(t2, "i32", 512, lets(
        [(tid, intr("thread_idx_x")), (gid, GID)], seq(*steps)))))
    out = torch.zeros(n, dtype=torch.int32, device="cuda")
    launch(hip, ir, n, [ints(torch, v), out, ("i32", n)], shared_mem=4096)
    exp = np.concatenate([np.cumsum(v[i:i + 256]) for i in range(0, n, 256)])
    assert np.array_equal(out.cpu().numpy(), exp)


def test_bitonic_sort_many_launches_of_one_cached_kernel(hip, torch_cuda):
    """test_sort.ml (bitonic step): data.(i) / data.(i lxor j) compare-exchange, launched
    log^2(n) times with different scalars; boolean logic with `not`, `&&`, `||`."""
    torch = torch_cuda
    n = 1 << 12
    v = np.random.default_rng(7).integers(-10000, 10000, n)
    fresh()
    params = [("data", "(vec i32)"), ("j", "i32"), ("k", "i32"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    i, ij, di, dij, asc = var("i"), var("ij"), var("di"), var("dij"), var("ascending", "bool")
    j, k = var("j"), var("k")
    cond = op("or", land(asc, op("gt", di, dij)), land(f"(not {asc})", lt(di, dij)))
    ir = kernel(params, let(i, intr("global_thread_id", "Std"), if_(lt(i, var("n")), let(
        ij, op("bitxor", i, j), if_(op("gt", ij, i), lets(
            [(di, read("data", i)), (dij, read("data", ij)), (asc, op("eq", op("bitand", i, k), i32(0)))],
            if_(cond, seq(assign_elem("data", i, dij), assign_elem("data", ij, di)))))))))
    src = hip.generate_source(ir, block=(256, 1, 1))
    d = ints(torch, v)
    kk = 2
    while kk <= n:
        jj = kk // 2
        while jj >= 1:
            hip.run_source(src, "sarek_kern", (256, 1, 1), (n // 256, 1, 1),
                           [d, ("i32", jj), ("i32", kk), ("i32", n)])
            jj //= 2
        kk *= 2
    hip.check(hip.lib.sarek_hip_device_synchronize())
    assert np.array_equal(d.cpu().numpy(), np.sort(v))


def test_nbody_record_constructor_and_inner_loop(hip, torch_cuda):
    """test_nbody_ppx.ml: a record built by a helper function, an inner for loop over all
    bodies with mutable accumulators, sqrt and division."""
    torch = torch_cuda
    n = 300
    rng = np.random.default_rng(8)
    pos = rng.normal(size=(3, n)).astype(np.float32)
    part = "(record particle (x f32) (y f32) (z f32))"
    P, Q = f"(var p 20 {part})", f"(var q 21 {part})"

    def mk(idx):
        return f"(app (var make_p 0 {part}) (read xs {idx}) (read ys {idx}) (read zs {idx}))"
    tid, jv = "(var tid 8 i32)", "(var j 9 i32 mut)"
    fx, fy, fz = ("(var f%s %d f32 mut)" % (c, 10 + i) for i, c in enumerate("xyz"))
    dx, dy, dz = ("(var d%s %d f32)" % (c, 13 + i) for i, c in enumerate("xyz"))
    dist2, inv = "(var dist2 16 f32)", "(var inv 17 f32)"
    ir = f"""
    (kernel sarek_kern
      (params (param (var xs 1 (vec f32))) (param (var ys 2 (vec f32))) (param (var zs 3 (vec f32)))
              (param (var ax 4 (vec f32))) (param (var ay 5 (vec f32))) (param (var az 6 (vec f32)))
              (param (var n 7 i32)))
      (locals)
      (body (let {tid} (add (intr (Gpu) thread_idx_x) (mul (intr (Gpu) block_idx_x) (intr (Gpu) block_dim_x)))
        (if (lt {tid} (var n 7 i32))
          (let {P} {mk(tid)}
          (letmut {fx} (f32 0.0) (letmut {fy} (f32 0.0) (letmut {fz} (f32 0.0)
           (seq
            (for {jv} (i32 0) (sub (var n 7 i32) (i32 1)) upto
              (if (ne {jv} {tid})
                (let {Q} {mk(jv)}
                (let {dx} (sub (field {Q} x) (field {P} x))
                (let {dy} (sub (field {Q} y) (field {P} y))
                (let {dz} (sub (field {Q} z) (field {P} z))
                (let {dist2} (add (add (add (mul {dx} {dx}) (mul {dy} {dy})) (mul {dz} {dz})) (f32 1e-9))
                (let {inv} (div (f32 1.0) (mul (intr (Float32) sqrt {dist2}) {dist2}))
                  (seq (assign (lvar {fx}) (add {fx} (mul {dx} {inv})))
                       (assign (lvar {fy}) (add {fy} (mul {dy} {inv})))
                       (assign (lvar {fz}) (add {fz} (mul {dz} {inv}))))))))))))
            (assign (lelem ax {tid}) {fx}) (assign (lelem ay {tid}) {fy}) (assign (lelem az {tid}) {fz})))))))))
      (types (particle (x f32) (y f32) (z f32)))
      (funcs (func make_p (params (var x 30 f32) (var y 31 f32) (var z 32 f32)) {part}
               (return (record particle (x (var x 30 f32)) (y (var y 31 f32)) (z (var z 32 f32))))))
      (native_fn false))"""
    xs, ys, zs = (torch.from_numpy(pos[c].copy()).cuda() for c in range(3))
    acc = [torch.zeros(n, device="cuda") for _ in range(3)]
    launch(hip, ir, n, [xs, ys, zs, *acc, ("i32", n)])
    p64 = pos.astype(np.float64)
    d = p64[:, None, :] - p64[:, :, None]                 # d[c, i, j] = pos[c, j] - pos[c, i]
    dist2 = (d ** 2).sum(0) + 1e-9
    w = 1.0 / (np.sqrt(dist2) * dist2)
    np.fill_diagonal(w, 0.0)
    exp = (d * w[None]).sum(2)
    for c in range(3):
        assert np.allclose(acc[c].cpu().numpy(), exp[c], rtol=2e-3, atol=2e-3)
