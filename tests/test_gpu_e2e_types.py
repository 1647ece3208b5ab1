"""Record-typed kernels of the reference's end-to-end suite through Vector / Execute.run_vectors on
the GPU: sarek/tests/e2e/test_complex_types.ml (vectors of 2-, 3-, 4- and 5-field records, read as
values and stored as record literals) and test_ray_ppx.ml (helper functions that take and return
records and call one another).  The IR is transcribed from the kernel sources with the lowering
rules of sarek/ppx/Sarek_lower_ir.ml; inputs, launch geometry (64-thread blocks) and tolerances are
the tests' own."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TID = "(var tid 90 i32)"
GID = "(add (intr (Gpu) thread_idx_x) (mul (intr (Gpu) block_dim_x) (intr (Gpu) block_idx_x)))"


def record(name, fields):
    return f"(record {name} " + " ".join(f"({f} f32)" for f in fields) + ")"


def types(name, fields):
    return f"(types ({name} " + " ".join(f"({f} f32)" for f in fields) + "))"


def kernel(params, body, aux):
    ps = " ".join(f"(param {p})" for p in params)
    return (f"(kernel sarek_kern (params {ps}) (locals) (body (let {TID} {GID} (if (lt {TID} (var n 91 i32)) {body})))"
            f" {aux} (native_fn true))")


def record_vector(data):
    from spoc_amd.sarek import Vector
    n, nf = data.shape
    v = Vector.create_custom(4 * nf, n)
    v.host.view(np.float32).reshape(n, nf)[:] = data
    return v


def run(ir, args, n):
    from spoc_amd.sarek import Execute, Transfer
    path = Execute.run_vectors(ir=ir, args=args, block=Execute.dims1d(64), grid=Execute.dims1d((n + 63) // 64))
    Transfer.flush()
    assert path == "jit"


def fields_of(v, nf):
    return v.to_array().view(np.float32).reshape(-1, nf)


def test_point2d_distance(hip, torch_cuda):
    """test_complex_types.ml:47-56,120-150: distances.(tid) <- sqrt (p.px * p.px + p.py * p.py)."""
    from spoc_amd.sarek import Execute, Vector
    n = 1000
    ty = record("point2d", ["px", "py"])
    p = f"(var p 1 {ty})"
    body = (f"(let {p} (read points {TID}) (assign (lelem distances {TID}) (intr (Float32) sqrt "
            f"(add (mul (field {p} px) (field {p} px)) (mul (field {p} py) (field {p} py))))))")
    ir = kernel([f"(var points 2 (vec {ty}))", "(var distances 3 (vec f32))", "(var n 91 i32)"], body,
                types("point2d", ["px", "py"]))
    i = np.arange(n, dtype=np.float32)
    pts = record_vector(np.stack([i, n - i], axis=1))
    dist = Vector.create(Vector.float32, n)
    dist.fill_from(np.zeros(n))
    run(ir, [Execute.Vec(pts), Execute.Vec(dist), Execute.Int32(n)], n)
    expected = np.sqrt(i.astype(np.float64) ** 2 + (n - i.astype(np.float64)) ** 2)
    assert np.all(np.abs(dist.to_array() - expected) <= np.maximum(1e-4, expected * 1e-6))


def test_point3d_normalize_in_place(hip, torch_cuda):
    """test_complex_types.ml:62-74: points.(tid) <- {x = p.x * inv; ...} under `if len > 0.0`; the
    zero vector stays as it is."""
    from spoc_amd.sarek import Execute
    n = 777
    f = ["x", "y", "z"]
    ty = record("point3d", f)
    p, ln, inv = f"(var p 1 {ty})", "(var len 2 f32)", "(var inv 3 f32)"
    norm2 = f"(add (add (mul (field {p} x) (field {p} x)) (mul (field {p} y) (field {p} y))) (mul (field {p} z) (field {p} z)))"
    lit = "(record point3d " + " ".join(f"({c} (mul (field {p} {c}) {inv}))" for c in f) + ")"
    body = (f"(let {p} (read points {TID}) (let {ln} (intr (Float32) sqrt {norm2}) (if (gt {ln} (f32 0.0)) "
            f"(let {inv} (div (f32 1.0) {ln}) (assign (lelem points {TID}) {lit})))))")
    ir = kernel([f"(var points 4 (vec {ty}))", "(var n 91 i32)"], body, types("point3d", f))
    i = np.arange(n, dtype=np.float32)
    pts = record_vector(np.stack([i, 2 * i, 3 * i], axis=1))
    run(ir, [Execute.Vec(pts), Execute.Int32(n)], n)
    got = fields_of(pts, 3).astype(np.float64)
    assert np.array_equal(got[0], [0, 0, 0])
    assert np.all(np.abs(np.sqrt((got[1:] ** 2).sum(1)) - 1.0) <= 1e-3)            # the test's own check
    assert np.allclose(got[1:], np.array([1, 2, 3]) / np.sqrt(14.0), atol=1e-6)


def test_particle_update_and_color_blend(hip, torch_cuda):
    """test_complex_types.ml:80-118: a five-field record rebuilt with two fields advanced by dt, and
    a four-field blend of two record vectors into a third."""
    from spoc_amd.sarek import Execute
    n = 500
    f = ["pos_x", "pos_y", "vel_x", "vel_y", "mass"]
    ty = record("particle", f)
    p, dt = f"(var p 1 {ty})", "(var dt 2 f32)"
    lit = (f"(record particle (pos_x (add (field {p} pos_x) (mul (field {p} vel_x) {dt}))) "
           f"(pos_y (add (field {p} pos_y) (mul (field {p} vel_y) {dt}))) (vel_x (field {p} vel_x)) "
           f"(vel_y (field {p} vel_y)) (mass (field {p} mass)))")
    ir = kernel([f"(var particles 3 (vec {ty}))", dt, "(var n 91 i32)"],
                f"(let {p} (read particles {TID}) (assign (lelem particles {TID}) {lit}))", types("particle", f))
    i = np.arange(n, dtype=np.float32)
    start = np.stack([i, 2 * i, np.ones(n), 2 * np.ones(n), np.ones(n)], axis=1).astype(np.float32)
    parts = record_vector(start)
    run(ir, [Execute.Vec(parts), Execute.Float32(0.1), Execute.Int32(n)], n)
    got = fields_of(parts, 5)
    assert np.all(np.abs(got[:, 0] - (i + 0.1)) <= 1e-3) and np.all(np.abs(got[:, 1] - (2 * i + 0.2)) <= 1e-3)
    assert np.array_equal(got[:, 2:], start[:, 2:])

    f = ["r", "g", "b", "a"]
    ty = record("color", f)
    p1, p2, t, it = f"(var p1 1 {ty})", f"(var p2 2 {ty})", "(var t 3 f32)", "(var inv_t 4 f32)"
    lit = "(record color " + " ".join(f"({c} (add (mul (field {p1} {c}) {it}) (mul (field {p2} {c}) {t})))" for c in f) + ")"
    body = (f"(let {p1} (read c1 {TID}) (let {p2} (read c2 {TID}) (let {it} (sub (f32 1.0) {t}) "
            f"(assign (lelem out {TID}) {lit}))))")
    ir = kernel([f"(var c1 5 (vec {ty}))", f"(var c2 6 (vec {ty}))", f"(var out 7 (vec {ty}))", t, "(var n 91 i32)"],
                body, types("color", f))
    c1 = record_vector(np.tile(np.float32([1, 0, 0, 1]), (n, 1)))
    c2 = record_vector(np.tile(np.float32([0, 1, 0, 1]), (n, 1)))
    out = record_vector(np.zeros((n, 4), dtype=np.float32))
    run(ir, [Execute.Vec(c1), Execute.Vec(c2), Execute.Vec(out), Execute.Float32(0.5), Execute.Int32(n)], n)
    assert np.array_equal(fields_of(out, 4), np.tile(np.float32([0.5, 0.5, 0, 1]), (n, 1)))


def test_ray_helpers_that_call_helpers(hip, torch_cuda):
    """test_ray_ppx.ml:20-75: make_vec3, dot and normalize (which calls both) over a record type
    declared inside the kernel; one sphere at z = -2 of radius 0.5 against a sky gradient; every
    channel within 1e-3 of the double-precision loop of the test."""
    from spoc_amd.sarek import Execute, Vector
    v3 = record("vec3", ["x", "y", "z"])

    def v(name, vid, ty="f32"):
        return f"(var {name} {vid} {ty})"
    a, b, vv, inv = v("a", 40, v3), v("b", 41, v3), v("v", 42, v3), v("inv", 43)
    funcs = f"""(funcs
      (func make_vec3 (params {v('x', 30)} {v('y', 31)} {v('z', 32)}) {v3}
        (return (record vec3 (x {v('x', 30)}) (y {v('y', 31)}) (z {v('z', 32)}))))
      (func dot (params {a} {b}) f32
        (return (add (add (mul (field {a} x) (field {b} x)) (mul (field {a} y) (field {b} y))) (mul (field {a} z) (field {b} z)))))
      (func normalize (params {vv}) {v3}
        (let {inv} (div (f32 1.0) (intr (Float32) sqrt (app (var dot 0 f32) {vv} {vv})))
          (return (app (var make_vec3 0 {v3}) (mul (field {vv} x) {inv}) (mul (field {vv} y) {inv}) (mul (field {vv} z) {inv}))))))"""
    names = ["dx", "dy", "dz", "dxn", "dyn", "dzn", "a", "half_b", "c", "disc", "t", "hx", "hy", "hz", "nx", "ny", "nz",
             "r", "g", "b", "t2"]
    s = {nm: v(nm, 50 + k) for k, nm in enumerate(names)}
    dirv, nrm, idx = v("dir", 80, v3), v("nrm", 81, v3), v("idx", 82, "i32")

    def lets(binds, body):
        for var_, e in reversed(binds):
            body = f"(let {var_} {e} {body})"
        return body

    def store(off, e):
        at = idx if off == 0 else f"(add {idx} (i32 {off}))"
        return f"(assign (lelem out {at}) {e})"
    hit = lets([(s["t"], f"(div (sub (neg {s['half_b']}) (intr (Float32) sqrt {s['disc']})) {s['a']})"),
                (s["hx"], f"(mul {s['t']} {s['dxn']})"), (s["hy"], f"(mul {s['t']} {s['dyn']})"),
                (s["hz"], f"(mul {s['t']} {s['dzn']})"),
                (s["nx"], f"(sub {s['hx']} (f32 0.0))"), (s["ny"], f"(sub {s['hy']} (f32 0.0))"),
                (s["nz"], f"(add {s['hz']} (f32 2.0))"),
                (nrm, f"(app (var normalize 0 {v3}) (app (var make_vec3 0 {v3}) {s['nx']} {s['ny']} {s['nz']}))")],
               "(seq " + " ".join(store(k, f"(mul (f32 0.5) (add (field {nrm} {c}) (f32 1.0)))") for k, c in enumerate("xyz")) + ")")
    sky = lets([(s["t2"], f"(mul (f32 0.5) (add {s['dyn']} (f32 1.0)))"),
                (s["r"], f"(add (sub (f32 1.0) {s['t2']}) (mul {s['t2']} (f32 0.5)))"),
                (s["g"], f"(add (sub (f32 1.0) {s['t2']}) (mul {s['t2']} (f32 0.7)))"), (s["b"], "(f32 1.0)")],
               f"(seq {store(0, s['r'])} {store(1, s['g'])} {store(2, s['b'])})")
    body = lets([(s["dx"], f"(read dirx {TID})"), (s["dy"], f"(read diry {TID})"), (s["dz"], f"(read dirz {TID})"),
                 (dirv, f"(app (var normalize 0 {v3}) (app (var make_vec3 0 {v3}) {s['dx']} {s['dy']} {s['dz']}))"),
                 (s["dxn"], f"(field {dirv} x)"), (s["dyn"], f"(field {dirv} y)"), (s["dzn"], f"(field {dirv} z)"),
                 (s["a"], f"(app (var dot 0 f32) {dirv} {dirv})"), (s["half_b"], f"(mul (f32 2.0) {s['dzn']})"),
                 (s["c"], "(f32 3.75)"),
                 (s["disc"], f"(sub (mul {s['half_b']} {s['half_b']}) (mul {s['a']} {s['c']}))"),
                 (idx, f"(mul {TID} (i32 3))")],
                f"(if (gt {s['disc']} (f32 0.0)) {hit} {sky})")
    ir = kernel(["(var dirx 1 (vec f32))", "(var diry 2 (vec f32))", "(var dirz 3 (vec f32))", "(var out 4 (vec f32))",
                 "(var n 91 i32)"], body, types("vec3", ["x", "y", "z"]) + " " + funcs)

    w = h = 96
    n = w * h
    i = np.arange(n)
    bax, bay, baz = 2.0 * (i % w) / (w - 1) - 1.0, 2.0 * (i // w) / (h - 1) - 1.0, np.full(n, -1.5)
    vecs = [Vector.create(Vector.float32, n) for _ in range(3)]
    for vec, data in zip(vecs, (bax, bay, baz)):
        vec.fill_from(data)
    out = Vector.create(Vector.float32, 3 * n)
    out.fill_from(np.zeros(3 * n))
    run(ir, [Execute.Vec(x) for x in vecs] + [Execute.Vec(out), Execute.Int32(n)], n)

    ln = np.sqrt(bax ** 2 + bay ** 2 + baz ** 2)
    dxn, dyn, dzn = bax / ln, bay / ln, baz / ln
    aa = dxn ** 2 + dyn ** 2 + dzn ** 2
    hb = 2.0 * dzn
    disc = hb * hb - aa * 3.75
    t = (-hb - np.sqrt(np.maximum(disc, 0))) / aa
    nx, ny, nz = t * dxn, t * dyn, t * dzn + 2.0
    inv = 1.0 / np.sqrt(nx ** 2 + ny ** 2 + nz ** 2)
    tt = 0.5 * (dyn + 1.0)
    expected = np.where((disc > 0)[:, None],
                        np.stack([0.5 * (nx * inv + 1), 0.5 * (ny * inv + 1), 0.5 * (nz * inv + 1)], axis=1),
                        np.stack([1 - tt + tt * 0.5, 1 - tt + tt * 0.7, np.ones(n)], axis=1))
    assert 0 < int((disc > 0).sum()) < n                        # both branches are taken
    assert np.all(np.abs(out.to_array().reshape(n, 3) - expected) <= 1e-3)


def test_literals_at_the_edges_of_their_types(hip, torch_cuda):
    """Constants a kernel may hold and the text must carry to the bit: infinities, a NaN, the signed zero, the
    largest float and the smallest denormals of both float types, the ends of int32 and int64, and the negation of
    each negative one (`(- -5LL)`, not a decrement).  One thread stores them; the host compares bit patterns."""
    from spoc_amd.sarek import Execute, Transfer, Vector
    f32s = ["inf", "-inf", "nan", "-0.0", "3.4028234663852886e+38", "1.401298464324817e-45", "-1.1754942106924411e-38",
            "0.1", "16777217.0"]
    f64s = ["inf", "-inf", "nan", "-0.0", "1.7976931348623157e+308", "5e-324", "0.1", "1e-320"]
    i32s = [-2147483648, 2147483647, -1, 0]
    i64s = [-9223372036854775808, 9223372036854775807, -5, 4294967301]
    stores = []
    for k, v in enumerate(f32s):
        stores.append(f"(assign (lelem a (i32 {k})) (f32 {v}))")
    stores.append(f"(assign (lelem a (i32 {len(f32s)})) (neg (f32 -2.5)))")
    for k, v in enumerate(f64s):
        stores.append(f"(assign (lelem b (i32 {k})) (f64 {v}))")
    stores.append(f"(assign (lelem b (i32 {len(f64s)})) (neg (f64 -2.5)))")
    stores.append(f"(assign (lelem b (i32 {len(f64s) + 1})) (div (f64 1.0) (f64 2.0)))")     # not the integer 1 / 2
    stores.append(f"(assign (lelem c (i32 6)) (if (lt (sub (i32 -2147483648) (i32 1)) (i32 0)) (i32 1) (i32 2)))")
    for k, v in enumerate(i32s):
        stores.append(f"(assign (lelem c (i32 {k})) (i32 {v}))")
    stores.append(f"(assign (lelem c (i32 {len(i32s)})) (neg (i32 -7)))")
    for k, v in enumerate(i64s):
        stores.append(f"(assign (lelem d (i32 {k})) (i64 {v}))")
    stores.append(f"(assign (lelem d (i32 {len(i64s)})) (neg (i64 -5)))")
    stores.append(f"(assign (lelem d (i32 {len(i64s) + 1})) (cast i64 (i32 -3)))")
    stores.append(f"(assign (lelem c (i32 {len(i32s) + 1})) (cast i32 (i64 4294967301)))")
    ir = ("(kernel sarek_kern (params (param (var a 1 (vec f32))) (param (var b 2 (vec f64))) (param (var c 3 (vec i32))) "
          "(param (var d 4 (vec i64)))) (locals) (body (if (eq (intr (Std) global_thread_id) (i32 0)) "
          f"(seq {' '.join(stores)}))) (native_fn true))")
    a, b = Vector.create(Vector.float32, 16), Vector.create(Vector.float64, 16)
    c, d = Vector.create(Vector.int32, 8), Vector.create(Vector.int64, 8)
    path = Execute.run_vectors(ir=ir, args=[Execute.Vec(a), Execute.Vec(b), Execute.Vec(c), Execute.Vec(d)],
                               block=Execute.dims1d(64), grid=Execute.dims1d(1))
    Transfer.flush()
    assert path == "jit"
    want_a = np.array([float(v) for v in f32s] + [2.5], np.float32)
    got_a = a.to_array()[:len(want_a)]
    assert np.isnan(got_a[2]) and np.isnan(want_a[2])
    keep = np.arange(len(want_a)) != 2
    assert np.array_equal(got_a.view(np.uint32)[keep], want_a.view(np.uint32)[keep]), got_a
    want_b = np.array([float(v) for v in f64s] + [2.5, 0.5], np.float64)
    got_b = b.to_array()[:len(want_b)]
    assert np.isnan(got_b[2])
    assert np.array_equal(got_b.view(np.uint64)[keep[:len(want_b)]], want_b.view(np.uint64)[keep[:len(want_b)]]), got_b
    # min_int - 1 wraps to max_int in int32 arithmetic (a `-2147483648` in the text would be a 64-bit operand)
    assert c.to_array()[:len(i32s) + 3].tolist() == i32s + [7, 5, 2]
    assert d.to_array()[:len(i64s) + 2].tolist() == i64s + [5, -3]


def test_a_match_used_as_a_value(hip, torch_cuda):
    """A variant built by nested `if`s and taken apart by a match in expression position, payload variables and all
    (the kernel whose text tests/test_ir_lowering.py pins)."""
    from test_ir_lowering import MATCH_AS_A_VALUE
    from spoc_amd.sarek import Execute, Transfer, Vector
    n = 1000
    x = np.random.default_rng(2).uniform(-3, 3, n).astype(np.float32)
    dst = Vector.create(Vector.float32, n)
    path = Execute.run_vectors(ir=MATCH_AS_A_VALUE, args=[Execute.Vec(Vector.of_array(x)), Execute.Vec(dst), Execute.Int32(n)],
                               block=Execute.dims1d(128), grid=Execute.dims1d((n + 127) // 128))
    Transfer.flush()
    assert path == "jit"
    want = np.where(x > 1, x * x, np.where(x < -1, x * np.float32(2), x))
    assert np.array_equal(dst.to_array(), want)


def test_a_pattern_that_names_the_value(hip, torch_cuda):
    """`match s with Circle r -> r | other -> (match other with Rect (w, h) -> w *. h | rest -> -1.)`."""
    from test_ir_lowering import MATCH_WITH_A_VARIABLE_PATTERN
    from spoc_amd.sarek import Execute, Transfer, Vector
    n = 500
    x = np.random.default_rng(4).uniform(-3, 3, n).astype(np.float32)
    dst = Vector.create(Vector.float32, n)
    path = Execute.run_vectors(ir=MATCH_WITH_A_VARIABLE_PATTERN, args=[Execute.Vec(Vector.of_array(x)), Execute.Vec(dst), Execute.Int32(n)],
                               block=Execute.dims1d(64), grid=Execute.dims1d((n + 63) // 64))
    Transfer.flush()
    assert path == "jit"
    assert np.array_equal(dst.to_array(), np.where(x > 1, x, x * np.float32(3)))


def test_ocaml_constants_a_kernel_names(hip, torch_cuda):
    """A reference to a value outside the kernel lowers to a variable of that name (Sarek_lower_ir.ml:378-380): the
    reference's own generated maximum reduction says `sdata[tid] = Float.neg_infinity;`
    (benchmarks/generate_backend_code.ml:164, the golden text of reduction_max).  The run-time compiler is given
    OCaml's values for Float.*, Int32.* and Int64.* when a text names them: the golden kernel runs as generated,
    block maxima bit for bit, and a kernel that stores a few of the others holds OCaml's values."""
    from spoc_amd import reference_kernels as rk
    from spoc_amd.sarek import Execute, Transfer, Vector
    n = 1000
    x = np.random.default_rng(8).standard_normal(n).astype(np.float32) - 5
    out = Vector.create(Vector.float32, 4)
    ir = rk.reduction_max()
    assert "Float.neg_infinity" in hip.generate_source(ir, block=(256, 1, 1))
    for specialise, served_by in ((0, "jit"), (1, "reduce_max_block256_f32:ff800000")):   # as generated, then by the hand kernel
        hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
        try:
            out.fill(np.float32(7))
            path = Execute.run_vectors(ir=ir, args=[Execute.Vec(Vector.of_array(x)), Execute.Vec(out), Execute.Int32(n)],
                                       block=Execute.dims1d(256), grid=Execute.dims1d(4))
            Transfer.flush()
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
        assert path == served_by
        assert np.array_equal(out.to_array(), [x[b * 256:(b + 1) * 256].max() for b in range(4)])

    stores = [("(var Float.pi 10 f64)", "d", np.pi), ("(var Float.epsilon 11 f64)", "d", np.finfo(np.float64).eps),
              ("(var Float.infinity 12 f64)", "d", np.inf), ("(var Float.max_float 13 f64)", "d", np.finfo(np.float64).max),
              ("(var Int32.max_int 14 i32)", "i", 2**31 - 1), ("(var Int32.min_int 15 i32)", "i", -2**31),
              ("(var Int64.max_int 16 i64)", "l", 2**63 - 1), ("(var Int64.min_int 17 i64)", "l", -2**63),
              ("(add (var Int32.max_int 14 i32) (var Int32.one 18 i32))", "i", -2**31),
              # Gpu.spoc_powint's device text is a call of that name (Gpu.ml:235-247), which the compile step defines
              ("(intr (Gpu) spoc_powint (i32 3) (i32 4))", "i", 81), ("(intr (Gpu) spoc_powint (i32 -2) (i32 31))", "i", -2**31),
              ("(intr (Gpu) spoc_powint (i32 7) (i32 0))", "i", 1)]
    body = " ".join(f"(assign (lelem {v} (i32 {k})) {e})" for k, (e, v, _) in enumerate(stores))
    ir = ("(kernel sarek_kern (params (param (var d 1 (vec f64))) (param (var i 2 (vec i32))) (param (var l 3 (vec i64)))) "
          f"(locals) (body (if (eq (intr (Std) global_thread_id) (i32 0)) (seq {body}))) (native_fn true))")
    d, i, l = Vector.create(Vector.float64, 16), Vector.create(Vector.int32, 16), Vector.create(Vector.int64, 16)
    Execute.run_vectors(ir=ir, args=[Execute.Vec(d), Execute.Vec(i), Execute.Vec(l)], block=Execute.dims1d(64),
                        grid=Execute.dims1d(1))
    Transfer.flush()
    got = {"d": d.to_array(), "i": i.to_array(), "l": l.to_array()}
    for k, (e, v, want) in enumerate(stores):
        assert got[v][k] == want, (e, got[v][k], want)


def test_the_references_known_answers_for_ir_semantics(hip, torch_cuda):
    """The cases of sarek/tests/unit/test_ir_interp.ml (array read, length and creation, a record's field, a
    variant's payload, conditionals, casts, operators, assignment, let, while, for, the conversions to int32 and to
    bool), lowered, compiled and run by one thread: every result is the one the reference's test asserts."""
    import interp_cases
    from spoc_amd.sarek import Execute, Transfer, Vector
    data, seven = Vector.of_array(np.array([10, 20, 30], np.int32)), Vector.of_array(np.zeros(7, np.int32))
    out, fout = Vector.of_array(np.full(32, -7, np.int32)), Vector.of_array(np.full(4, -7, np.float32))
    path = Execute.run_vectors(ir=interp_cases.kernel(), args=[Execute.Vec(data), Execute.Vec(seven), Execute.Vec(out), Execute.Vec(fout)],
                               block=Execute.dims1d(64), grid=Execute.dims1d(1))
    Transfer.flush()
    assert path == "jit"
    got = out.to_array()
    for k, want in interp_cases.EXPECTED.items():
        assert got[k] == want, (k, got[k], want)
    assert fout.to_array()[0] == 42.0
