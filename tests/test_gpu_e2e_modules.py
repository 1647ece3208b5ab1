"""Kernels of the reference's end-to-end suite that reach module items: helper functions bound in the kernel payload
or taken from another module's registry, recursion rewritten by the front end, polymorphic helpers in one copy per
type, module constants, registered record and variant types.  Each runs through Vector / Execute.run_vectors with the
test's own inputs, launch geometry and check:

  test_bounded_recursion.ml   tail-recursive factorial, power and gcd as while loops (Sarek_tailrec_elim.ml:28-370:
                              loop variables __p, _continue, _result, arguments evaluated into _tmp_i before assigning)
  test_inline_pragma.ml       pow2 and fib with pragma ["sarek.inline 6"]: the body substituted into its own calls six
                              times (Sarek_tailrec_pragma.ml:258-377), the calls that remain left as calls
  test_polymorphism.ml, test_module_poly.ml   add_one, times_two; identity at int32 and float32 as identity__i32 and
                              identity__f32 (Sarek_mono.ml:97-128)
  test_module_const.ml        `let (scale : float32) = 2.0` in front of the kernel function: a let with an empty body in
                              sequence with the kernel body (Sarek_lower_ir.ml:634-671)
  test_ktype_helper.ml, test_registered_type.ml, test_cross_module_type.ml, test_registered_const.ml,
  test_visibility_private.ml  record literals, a helper that returns a record, helpers of another module that take a
                              record or a scalar (a call by name into kern_funcs, Sarek_lower_ir.ml:309-346)
  test_registered_variant.ml  a variant built by an if expression and matched
  test_convention_kernel.ml   a vector of records whose type name carries its module (Geometry_lib.point)

The IR is transcribed from the kernel sources with the lowering rules of sarek/ppx/Sarek_lower_ir.ml (helper
parameters numbered by position, `make_returning` on the helper bodies)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GID = "(add (intr (Gpu) thread_idx_x) (mul (intr (Gpu) block_idx_x) (intr (Gpu) block_dim_x)))"
STD_GID = "(intr (Std) global_idx_x)"


def run(ir, args, block, grid):
    from spoc_amd.sarek import Execute, Transfer
    path = Execute.run_vectors(ir=ir, args=args, block=Execute.dims1d(block), grid=Execute.dims1d(grid))
    Transfer.flush()
    assert path == "jit"


def i32v(name, i):
    return f"(var {name} {i} i32)"


def one_thread_kernel(params, call, funcs):
    """fun (output : int32 vector) ... -> let idx = global_idx_x in if idx = 0l then output.(idx) <- CALL"""
    ps = " ".join(f"(param {p})" for p in ["(var output 1 (vec i32))"] + params)
    idx = i32v("idx", 50)
    return (f"(kernel sarek_kern (params {ps}) (locals) (body (let {idx} {STD_GID} (if (eq {idx} (i32 0)) "
            f"(assign (lelem output {idx}) {call})))) (funcs {funcs}) (native_fn true))")


def tail_recursive(name, params, cond, base, next_args):
    """`let rec NAME params = if COND then BASE else NAME next_args` as eliminate_tail_recursion leaves it:
    letmut spoc_prof_cond, _result, _continue, __p ...; while _continue do if COND then (_result := BASE; _continue :=
    false) else let _tmp_i = ARG_i in (__p_i := _tmp_i ...) done; _result.  cond / base / next_args are written over the
    loop variables (the parameters' references are substituted)."""
    loop = {p: f"(var __{p} {100 + i} i32 mut)" for i, p in enumerate(params)}
    cont, res, prof = "(var _continue 120 bool mut)", "(var _result 121 i32 mut)", "(var spoc_prof_cond 122 bool mut)"
    c, b, args = cond(loop), base(loop), next_args(loop)
    tmps = [f"(var _tmp_{i} {130 + i} i32)" for i in range(len(args))]
    assigns = " ".join(f"(assign (lvar {loop[p]}) {t})" for p, t in zip(params, tmps))
    step = f"(seq {assigns})"
    for t, a in reversed(list(zip(tmps, args))):
        step = f"(let {t} {a} {step})"
    body = (f"(seq (while {cont} (if {c} (seq (assign (lvar {res}) {b}) (assign (lvar {cont}) (bool false))) {step})) "
            f"(return {res}))")
    for p in reversed(params):
        body = f"(letmut {loop[p]} {i32v(p, params.index(p))} {body})"
    body = f"(letmut {prof} (bool true) (letmut {res} (i32 0) (letmut {cont} (bool true) {body})))"
    formals = " ".join(i32v(p, i) for i, p in enumerate(params))
    return f"(func {name} (params {formals}) i32 {body})"


def test_tail_recursion_as_loops(hip, torch_cuda):
    """test_bounded_recursion.ml:24-61: fact(10) = 3628800, power(2, 10) = 1024, gcd(48, 18) = 6, one thread each."""
    from spoc_amd.sarek import Execute, Vector
    fact = tail_recursive("fact_aux", ["acc", "n"], lambda v: f"(le {v['n']} (i32 1))", lambda v: v["acc"],
                          lambda v: [f"(mul {v['acc']} {v['n']})", f"(sub {v['n']} (i32 1))"])
    power = tail_recursive("power_aux", ["acc", "base", "exp"], lambda v: f"(le {v['exp']} (i32 0))", lambda v: v["acc"],
                           lambda v: [f"(mul {v['acc']} {v['base']})", v["base"], f"(sub {v['exp']} (i32 1))"])
    gcd = tail_recursive("gcd", ["a", "b"], lambda v: f"(eq {v['b']} (i32 0))", lambda v: v["a"],
                         lambda v: [v["b"], f"(mod {v['a']} {v['b']})"])
    cases = [
        (one_thread_kernel([i32v("n", 2)], f"(app (var fact_aux 0 i32) (i32 1) {i32v('n', 2)})", fact), [10], 3628800),
        (one_thread_kernel([i32v("base", 2), i32v("exp", 3)],
                           f"(app (var power_aux 0 i32) (i32 1) {i32v('base', 2)} {i32v('exp', 3)})", power), [2, 10], 1024),
        (one_thread_kernel([i32v("a", 2), i32v("b", 3)], f"(app (var gcd 0 i32) {i32v('a', 2)} {i32v('b', 3)})", gcd),
         [48, 18], 6),
        (one_thread_kernel([i32v("a", 2), i32v("b", 3)], f"(app (var gcd 0 i32) {i32v('a', 2)} {i32v('b', 3)})", gcd),
         [1071, 462], 21),
    ]
    for ir, scalars, expected in cases:
        out = Vector.create(Vector.int32, 1)
        out.host[:] = 0
        run(ir, [Execute.Vec(out)] + [Execute.Int32(s) for s in scalars], 1, 1)
        assert out.to_array()[0] == expected, (scalars, expected)


def inlined(body_of, params, depth):
    """The body of a recursive function after `depth` rounds of substituting the body for its own calls: body_of(args,
    call) writes the body over argument expressions, `call(args)` is what a recursive call becomes."""
    def at(level):
        if level == depth:
            return lambda args: body_of(args, lambda a: "(app (var %s 0 i32) %s)" % (params[0], " ".join(a)))
        deeper = at(level + 1)
        return lambda args: body_of(args, deeper)
    return at(0)


def test_bounded_inlining_of_non_tail_recursion(hip, torch_cuda):
    """test_inline_pragma.ml:28-53: pow2(5) = 32; fib(0, 1, 5, 7) = 0, 1, 5, 13 (fib 7 goes one level past the six
    inlined ones: the call that remains there is an ordinary recursive call of the helper)."""
    from spoc_amd.sarek import Execute, Vector
    n0 = i32v("n", 0)

    def pow2_body(args, call):
        (n,) = args
        return f"(if (le {n} (i32 0)) (i32 1) (mul (i32 2) {call([f'(sub {n} (i32 1))'])}))"

    def fib_body(args, call):
        (n,) = args
        rec = f"(add {call([f'(sub {n} (i32 1))'])} {call([f'(sub {n} (i32 2))'])})"
        return f"(if (le {n} (i32 0)) (i32 0) (if (eq {n} (i32 1)) (i32 1) {rec}))"

    def helper(name, body_of):
        # the outermost `if` is the helper's statement (a return in each branch), the inlined copies are expressions
        deeper = inlined(body_of, [name], 5)
        if name == "pow2":
            stmt = (f"(if (le {n0} (i32 0)) (return (i32 1)) (return (mul (i32 2) {deeper([f'(sub {n0} (i32 1))'])})))")
        else:
            rec = f"(add {deeper([f'(sub {n0} (i32 1))'])} {deeper([f'(sub {n0} (i32 2))'])})"
            stmt = f"(if (le {n0} (i32 0)) (return (i32 0)) (if (eq {n0} (i32 1)) (return (i32 1)) (return {rec})))"
        return f"(func {name} (params {n0}) i32 {stmt})"

    for name, body_of, cases in (("pow2", pow2_body, [(5, 32), (0, 1), (6, 64)]),
                                 ("fib", fib_body, [(0, 0), (1, 1), (5, 5), (7, 13)])):
        ir = one_thread_kernel([i32v("n", 2)], f"(app (var {name} 0 i32) {i32v('n', 2)})", helper(name, body_of))
        for n, expected in cases:
            out = Vector.create(Vector.int32, 1)
            out.host[:] = 0
            run(ir, [Execute.Vec(out), Execute.Int32(n)], 1, 1)
            assert out.to_array()[0] == expected, (name, n)


def test_module_functions_and_one_copy_per_type(hip, torch_cuda):
    """test_polymorphism.ml:30-62, test_module_poly.ml:29-42: add_one, times_two (n = 1024, blocks of 256, no bound
    check in the kernels), and identity used at int32 and at float32 in one kernel."""
    from spoc_amd.sarek import Execute, Vector
    n = 1024
    idx = i32v("idx", 50)
    for helper, name, expected in (
            ("(func add_one (params (var x 0 i32)) i32 (return (add (var x 0 i32) (i32 1))))", "add_one", lambda i: i + 1),
            ("(func times_two (params (var x 0 i32)) i32 (return (add (var x 0 i32) (var x 0 i32))))", "times_two",
             lambda i: 2 * i)):
        ir = (f"(kernel sarek_kern (params (param (var src 1 (vec i32))) (param (var dst 2 (vec i32)))) (locals) "
              f"(body (let {idx} {STD_GID} (assign (lelem dst {idx}) (app (var {name} 0 i32) (read src {idx}))))) "
              f"(funcs {helper}) (native_fn true))")
        src, dst = Vector.of_array(np.arange(n, dtype=np.int32)), Vector.create(Vector.int32, n)
        run(ir, [Execute.Vec(src), Execute.Vec(dst)], 256, n // 256)
        assert np.array_equal(dst.to_array(), expected(np.arange(n, dtype=np.int32)))
    funcs = ("(func identity__i32 (params (var x 0 i32)) i32 (return (var x 0 i32))) "
             "(func identity__f32 (params (var x 0 f32)) f32 (return (var x 0 f32)))")
    ir = (f"(kernel sarek_kern (params (param (var src_i 1 (vec i32))) (param (var src_f 2 (vec f32))) "
          f"(param (var dst_i 3 (vec i32))) (param (var dst_f 4 (vec f32)))) (locals) "
          f"(body (let {idx} {STD_GID} (seq (assign (lelem dst_i {idx}) (app (var identity__i32 0 i32) (read src_i {idx}))) "
          f"(assign (lelem dst_f {idx}) (app (var identity__f32 0 f32) (read src_f {idx})))))) "
          f"(funcs {funcs}) (native_fn true))")
    src_i, src_f = Vector.of_array(np.arange(n, dtype=np.int32)), Vector.of_array(np.arange(n, dtype=np.float32))
    dst_i, dst_f = Vector.create(Vector.int32, n), Vector.create(Vector.float32, n)
    run(ir, [Execute.Vec(src_i), Execute.Vec(src_f), Execute.Vec(dst_i), Execute.Vec(dst_f)], 256, n // 256)
    assert np.array_equal(dst_i.to_array(), np.arange(n, dtype=np.int32))
    assert np.array_equal(dst_f.to_array(), np.arange(n, dtype=np.float32))


def guarded(params, body, extra=""):
    """fun params -> let tid = thread_idx_x + block_idx_x * block_dim_x in if tid < n then BODY"""
    tid = i32v("tid", 50)
    ps = " ".join(f"(param {p})" for p in params)
    return (f"(kernel sarek_kern (params {ps}) (locals) (body {{front}}(let {tid} {GID} (if (lt {tid} (var n 9 i32)) "
            f"{body})){{back}}) {extra} (native_fn true))")


XS_YS_DST = ["(var xs 1 (vec f32))", "(var ys 2 (vec f32))", "(var dst 3 (vec f32))", "(var n 9 i32)"]
TID = i32v("tid", 50)


def xy_vectors(n, y_of):
    from spoc_amd.sarek import Vector
    i = np.arange(n, dtype=np.float32)
    xs, ys, dst = Vector.of_array(i), Vector.of_array(y_of(i).astype(np.float32)), Vector.create(Vector.float32, n)
    dst.host[:] = 0
    return i, y_of(i).astype(np.float32), xs, ys, dst


def test_module_constant_in_front_of_the_kernel(hip, torch_cuda):
    """test_module_const.ml:20-27 (the reference only generates it; run here): dst = scale * src with scale a module
    constant, lowered as `SSeq [SSeq [SLet (scale, 2.0, SEmpty); SEmpty]; body]`."""
    from spoc_amd.sarek import Execute, Vector
    n = 1000
    scale = "(var scale 7 f32)"
    ir = guarded(["(var src 1 (vec f32))", "(var dst 2 (vec f32))", "(var n 9 i32)"],
                 f"(assign (lelem dst {TID}) (mul {scale} (read src {TID})))")
    ir = ir.format(front=f"(seq (seq (let {scale} (f32 2.0) (empty)) (empty)) ", back=")")
    src = Vector.of_array(np.linspace(-3, 3, n).astype(np.float32))
    dst = Vector.create(Vector.float32, n)
    run(ir, [Execute.Vec(src), Execute.Vec(dst), Execute.Int32(n)], 128, (n + 127) // 128)
    assert np.array_equal(dst.to_array(), np.float32(2.0) * src.to_array())


def test_record_literal_and_helpers_over_records(hip, torch_cuda):
    """test_registered_type.ml:21-30 (a record literal, its fields read back), test_ktype_helper.ml:26-40 (a helper
    that returns the record), test_cross_module_type.ml:26-37 (a record of another module handed to that module's
    helper): sqrt(x^2 + y^2) to 1e-3 and x + y to 1e-4, the tests' own tolerances."""
    from spoc_amd.sarek import Execute
    point = "(record point (x f32) (y f32))"
    p = f"(var p 60 {point})"
    length = f"(intr (Float32) sqrt (add (mul (field {p} x) (field {p} x)) (mul (field {p} y) (field {p} y))))"
    literal = f"(record point (x (read xs {TID})) (y (read ys {TID})))"
    for n, block, make, funcs in (
            (1024, 64, literal, ""),
            (256, 128, f"(app (var make_point 0 {point}) (read xs {TID}) (read ys {TID}))",
             f"(funcs (func make_point (params (var x 0 f32) (var y 1 f32)) {point} "
             f"(return (record point (x (var x 0 f32)) (y (var y 1 f32))))))")):
        ir = guarded(XS_YS_DST, f"(let {p} {make} (assign (lelem dst {TID}) {length}))",
                     "(types (point (x f32) (y f32))) " + funcs).format(front="", back="")
        i, y, xs, ys, dst = xy_vectors(n, lambda i: n - i)
        run(ir, [Execute.Vec(xs), Execute.Vec(ys), Execute.Vec(dst), Execute.Int(n)], block, (n + block - 1) // block)
        expected = np.sqrt(i.astype(np.float64) ** 2 + y.astype(np.float64) ** 2)
        assert np.abs(dst.to_array() - expected).max() <= 1e-3
    vec2 = "(record Registered_defs.vec2 (x f32) (y f32))"
    q = f"(var p 60 {vec2})"
    ir = guarded(XS_YS_DST,
                 f"(let {q} (record Registered_defs.vec2 (x (read xs {TID})) (y (read ys {TID}))) "
                 f"(assign (lelem dst {TID}) (app (var add_vec 0 f32) {q})))",
                 f"(types (Registered_defs.vec2 (x f32) (y f32))) (funcs (func add_vec (params (var p 0 {vec2})) f32 "
                 f"(return (add (field (var p 0 {vec2}) x) (field (var p 0 {vec2}) y)))))").format(front="", back="")
    n = 64
    i, y, xs, ys, dst = xy_vectors(n, lambda i: 2 * i)
    run(ir, [Execute.Vec(xs), Execute.Vec(ys), Execute.Vec(dst), Execute.Int(n)], 64, 1)
    assert np.abs(dst.to_array() - (i + y)).max() <= 1e-4


def test_functions_of_another_module(hip, torch_cuda):
    """test_registered_const.ml:26-36: dst = scale_fun (xs + ys) with scale_fun x = x * 2.0 taken from Registered_defs'
    registry, a call by name into kern_funcs.  test_visibility_private.ml:9-18 calls Visibility_lib.public_add by its
    qualified name, which the typer lets through as an external function (Sarek_typer.ml:688-696) and no generator
    resolves: the reference stops at the IR there, and so does this test -- the lowering prints the call as it stands,
    as sarek-cuda/Sarek_ir_cuda.ml:136-144 does."""
    from spoc_amd.sarek import Execute
    n = 64
    call = f"(app (var scale_fun 0 f32) (add (read xs {TID}) (read ys {TID})))"
    funcs = "(func scale_fun (params (var x 0 f32)) f32 (return (mul (var x 0 f32) (f32 2.0))))"
    ir = guarded(XS_YS_DST, f"(assign (lelem dst {TID}) {call})", f"(funcs {funcs})").format(front="", back="")
    i, y, xs, ys, dst = xy_vectors(n, lambda i: n - i)
    run(ir, [Execute.Vec(xs), Execute.Vec(ys), Execute.Vec(dst), Execute.Int(n)], 64, 1)
    assert np.abs(dst.to_array() - (i + y) * 2.0).max() <= 1e-4
    call = f"(app (var Visibility_lib.public_add 70 f32) (read xs {TID}) (read ys {TID}))"
    text = hip.generate_source(guarded(XS_YS_DST, f"(assign (lelem dst {TID}) {call})").format(front="", back=""))
    assert "dst[tid] = Visibility_lib.public_add(xs[tid], ys[tid]);" in text


def test_registered_variant_built_by_an_if_and_matched(hip, torch_cuda):
    """test_registered_variant.ml:21-33: c = if xs > 0 then Value xs else Red; Red -> 0, Value v -> v + 1; inputs -1 at
    even indices and i at odd ones, n = 1000, blocks of 64, 1e-3."""
    from spoc_amd.sarek import Execute, Vector
    n = 1000
    color = "(variant color (Red) (Value f32))"
    c = f"(var c 60 {color})"
    body = (f"(let {c} (if (gt (read xs {TID}) (f32 0.0)) (variant color Value (read xs {TID})) (variant color Red)) "
            f"(match {c} (case (Red) (assign (lelem dst {TID}) (f32 0.0))) "
            f"(case (Value v) (assign (lelem dst {TID}) (add (var v 61 f32) (f32 1.0))))))")
    ir = guarded(["(var xs 1 (vec f32))", "(var dst 3 (vec f32))", "(var n 9 i32)"], body,
                 "(variants (color (Red) (Value f32)))").format(front="", back="")
    i = np.arange(n)
    xs = Vector.of_array(np.where(i % 2 == 0, -1.0, i).astype(np.float32))
    dst = Vector.create(Vector.float32, n)
    dst.host[:] = 0
    run(ir, [Execute.Vec(xs), Execute.Vec(dst), Execute.Int32(n)], 64, (n + 63) // 64)
    assert np.abs(dst.to_array() - np.where(i % 2 == 0, 0.0, i + 1.0)).max() <= 1e-3


def test_vector_of_records_of_a_library_module(hip, torch_cuda):
    """test_convention_kernel.ml:9-25 (the reference only generates it; run here): points : Geometry_lib.point vector,
    p.x and p.y bound to lets, distances.(tid) <- sqrt (x * x + y * y)."""
    from spoc_amd.sarek import Execute, Vector
    n = 500
    ty = "(record Geometry_lib.point (x f32) (y f32))"
    p, x, y = f"(var p 60 {ty})", "(var x 61 f32)", "(var y 62 f32)"
    body = (f"(let {p} (read points {TID}) (let {x} (field {p} x) (let {y} (field {p} y) "
            f"(assign (lelem distances {TID}) (intr (Float32) sqrt (add (mul {x} {x}) (mul {y} {y})))))))")
    ir = guarded([f"(var points 1 (vec {ty}))", "(var distances 2 (vec f32))", "(var n 9 i32)"], body,
                 "(types (Geometry_lib.point (x f32) (y f32)))").format(front="", back="")
    pts = np.random.default_rng(5).normal(size=(n, 2)).astype(np.float32)
    points = Vector.create_custom(8, n)
    points.host.view(np.float32).reshape(n, 2)[:] = pts
    dist = Vector.create(Vector.float32, n)
    run(ir, [Execute.Vec(points), Execute.Vec(dist), Execute.Int32(n)], 64, (n + 63) // 64)
    assert np.allclose(dist.to_array(), np.hypot(pts[:, 0], pts[:, 1]), rtol=1e-6)


def test_nested_types_inside_kernels(hip, torch_cuda):
    """The types of test_nested_types.ml (a record inside a record, an enum variant as a field, int32 and float32 fields
    side by side, a variant whose payloads are records) read from vectors, built and matched in kernels.  That file
    itself checks the PPX-made host accessors of those types, OCaml code with no counterpart below the C ABI; what a
    backend owes those types is a device struct that lays them out the same way (fields in order, 4 bytes each, an
    int32 tag in front of a variant's payload) whatever order the kernel lists its types in: here the outer types
    come first, as out of the front end's hash table."""
    from spoc_amd.sarek import Execute, Vector
    n = 1000
    point = "(record point (x f32) (y f32))"
    color = "(variant color (Red) (Green) (Blue))"
    cp = f"(record colored_point (color {color}) (pt {point}))"
    c = f"(var c 60 {cp})"
    pt = lambda f: f"(field (field {c} pt) {f})"  # noqa: E731
    body = (f"(let {c} (read pts {TID}) (match (field {c} color) (case (Red) (assign (lelem dst {TID}) {pt('x')})) "
            f"(case (Green) (assign (lelem dst {TID}) {pt('y')})) "
            f"(case (Blue) (assign (lelem dst {TID}) (add {pt('x')} {pt('y')})))))")
    ir = guarded([f"(var pts 1 (vec {cp}))", "(var dst 2 (vec f32))", "(var n 9 i32)"], body,
                 f"(types (colored_point (color {color}) (pt {point})) (point (x f32) (y f32))) "
                 f"(variants (color (Red) (Green) (Blue)))").format(front="", back="")
    rng = np.random.default_rng(11)
    tags = rng.integers(0, 3, n).astype(np.int32)
    xy = rng.normal(size=(n, 2)).astype(np.float32)
    pts = Vector.create_custom(12, n)
    raw = pts.host.view(np.int32).reshape(n, 3)
    raw[:, 0] = tags
    raw[:, 1:] = xy.view(np.int32)
    dst = Vector.create(Vector.float32, n)
    run(ir, [Execute.Vec(pts), Execute.Vec(dst), Execute.Int32(n)], 64, (n + 63) // 64)
    want = np.where(tags == 0, xy[:, 0], np.where(tags == 1, xy[:, 1], xy[:, 0] + xy[:, 1]))
    assert np.array_equal(dst.to_array(), want.astype(np.float32))

    # int32 and float32 fields side by side: read, recombined, and a record literal stored back
    mixed = "(record mixed_record (count i32) (value f32) (flags i32))"
    r = f"(var r 60 {mixed})"
    lit = (f"(record mixed_record (count (add (field {r} count) (i32 1))) (value (mul (field {r} value) (f32 2.0))) "
           f"(flags (field {r} flags)))")
    body = (f"(let {r} (read recs {TID}) (seq (assign (lelem dst {TID}) (add (mul (cast f32 (field {r} count)) (field {r} value)) "
            f"(cast f32 (field {r} flags)))) (assign (lelem recs {TID}) {lit})))")
    ir = guarded([f"(var recs 1 (vec {mixed}))", "(var dst 2 (vec f32))", "(var n 9 i32)"], body,
                 "(types (mixed_record (count i32) (value f32) (flags i32)))").format(front="", back="")
    recs = Vector.create_custom(12, n)
    raw = recs.host.view(np.int32).reshape(n, 3)
    i = np.arange(n, dtype=np.int32)
    value = (i * np.float32(1.5)).astype(np.float32)
    raw[:, 0], raw[:, 1], raw[:, 2] = i, value.view(np.int32), i * 10
    run(ir, [Execute.Vec(recs), Execute.Vec(dst), Execute.Int32(n)], 64, (n + 63) // 64)
    assert np.array_equal(dst.to_array(), i.astype(np.float32) * value + (i * 10).astype(np.float32))
    back = recs.to_array().view(np.int32).reshape(n, 3)
    assert np.array_equal(back[:, 0], i + 1) and np.array_equal(back[:, 2], i * 10)
    assert np.array_equal(back[:, 1].view(np.float32), value * np.float32(2.0))

    # a variant with record payloads, one of them the nested record: built from the index, matched, payload fields read
    mcp = f"(variant maybe_colored_point (Red_pt {point}) (Blue_pt {point}) (Any_pt {cp}) (No_point))"
    here = f"(record point (x (read xs {TID})) (y (read ys {TID})))"
    k = f"(mod {TID} (i32 4))"
    m = f"(var m 61 {mcp})"
    build = (f"(if (eq {k} (i32 0)) (variant maybe_colored_point Red_pt {here}) "
             f"(if (eq {k} (i32 1)) (variant maybe_colored_point Blue_pt {here}) "
             f"(if (eq {k} (i32 2)) (variant maybe_colored_point Any_pt (record colored_point (color (variant color Green)) (pt {here}))) "
             f"(variant maybe_colored_point No_point))))")
    p, q = f"(var p 62 {point})", f"(var q 63 {cp})"
    body = (f"(let {m} {build} (match {m} (case (Red_pt p) (assign (lelem dst {TID}) (field {p} x))) "
            f"(case (Blue_pt p) (assign (lelem dst {TID}) (field {p} y))) "
            f"(case (Any_pt q) (assign (lelem dst {TID}) (mul (field (field {q} pt) x) (field (field {q} pt) y)))) "
            f"(case (No_point) (assign (lelem dst {TID}) (f32 -1.0)))))")
    ir = guarded(XS_YS_DST, body,
                 f"(types (colored_point (color {color}) (pt {point})) (point (x f32) (y f32))) "
                 f"(variants (maybe_colored_point (Red_pt {point}) (Blue_pt {point}) (Any_pt {cp}) (No_point)) "
                 f"(color (Red) (Green) (Blue)))").format(front="", back="")
    i, y, xs, ys, dst = xy_vectors(n, lambda i: 2 * i + 1)
    run(ir, [Execute.Vec(xs), Execute.Vec(ys), Execute.Vec(dst), Execute.Int32(n)], 64, (n + 63) // 64)
    kk = np.arange(n) % 4
    want = np.where(kk == 0, i, np.where(kk == 1, y, np.where(kk == 2, i * y, -1.0))).astype(np.float32)
    assert np.array_equal(dst.to_array(), want)


def test_the_two_smallest_kernels(hip, torch_cuda):
    """test_debug_native.ml:19-32 (there run on the Native device to debug its runtime): a constant fill and the
    thread id as a float, 1024 elements in blocks of 256 -- both element-wise maps without an input vector."""
    from spoc_amd.sarek import Execute, Transfer, Vector
    n = 1024
    tid = "(var tid 3 i32)"

    def kernel(value):
        return (f"(kernel sarek_kern (params (param (var output 1 (vec f32))) (param (var n 2 i32))) (locals) (body "
                f"(let {tid} (intr (Std) global_thread_id) (if (lt {tid} (var n 2 i32)) "
                f"(assign (lelem output {tid}) {value})))) (native_fn true))")

    for value, want in (("(f32 42.0)", np.full(n, 42.0, np.float32)),
                        (f"(cast f32 {tid})", np.arange(n, dtype=np.float32))):
        out = Vector.create(Vector.float32, n)
        path = Execute.run_vectors(ir=kernel(value), args=[Execute.Vec(out), Execute.Int32(n)],
                                   block=Execute.dims1d(256), grid=Execute.dims1d(n // 256))
        Transfer.flush()
        assert path == "map_f32"
        assert np.array_equal(out.to_array(), want)


def test_names_bound_again_mean_what_ocaml_says(hip, torch_cuda):
    """`let x = 1 in let x = x + 1 in ...`, two sibling lets of one name, a let named like a parameter, a loop counter
    named like a visible let: each run by one thread, the vector then holds what OCaml's scoping gives.  The bodies
    and expected values are those the lowering tests pin the text of."""
    from test_ir_lowering import REBOUND, REBOUND_PARAMS, kernel_with_body
    from spoc_amd.sarek import Execute, Transfer, Vector
    for name, (body, _, want) in REBOUND.items():
        v = Vector.of_array(np.full(8, -1, np.int32))
        path = Execute.run_vectors(ir=kernel_with_body(body, REBOUND_PARAMS), args=[Execute.Vec(v), Execute.Int32(3)],
                                   block=Execute.dims1d(1), grid=Execute.dims1d(1))
        Transfer.flush()
        assert path == "jit", name
        expected = np.full(8, -1, np.int32)
        for at, value in want.items():
            expected[at] = value
        assert np.array_equal(v.to_array(), expected), name



def test_arguments_that_do_not_fit_the_kernel_are_refused_before_the_launch(hip, torch_cuda):
    """A launch with too few arguments, a scalar where a vector goes, an int for a float or a vector of another
    element size would give the kernel a parameter block of another layout (a length read as a pointer).  The
    reference passes on what it is given (Execute.ml:197-216); here each is an error that names the argument, and
    nothing runs: the output vector keeps what it held."""
    from spoc_amd.sarek import Execute, Transfer, Vector
    ir = ("(kernel scale_kernel (params (param (var x 1 (vec f32))) (param (var out 2 (vec f32))) (param (var a 3 f32)) "
          "(param (var n 4 i32))) (locals) (body (let (var tid 5 i32) (intr (Std) global_thread_id) "
          "(if (lt (var tid 5 i32) (var n 4 i32)) (assign (lelem out (var tid 5 i32)) "
          "(add (mul (read x (var tid 5 i32)) (var a 3 f32)) (f32 1.0)))))) (native_fn true))")
    n = 256
    x = Vector.of_array(np.arange(n, dtype=np.float32))
    out = Vector.of_array(np.full(n, -7, np.float32))
    wide = Vector.of_array(np.zeros(n, np.float64))
    good = [Execute.Vec(x), Execute.Vec(out), Execute.Float32(2.0), Execute.Int32(n)]
    cases = [
        (good[:3], "takes 4 arguments, 3 given"),
        (good + [Execute.Int32(1)], "takes 4 arguments, 5 given"),
        ([Execute.Vec(x), Execute.Float32(2.0), Execute.Vec(out), Execute.Int32(n)], "argument 1 (out) of kernel scale_kernel is a vector, a float32 given"),
        ([Execute.Vec(x), Execute.Vec(out), Execute.Int32(2), Execute.Int32(n)], "argument 2 (a) of kernel scale_kernel is a float32, an int32 given"),
        ([Execute.Vec(x), Execute.Vec(out), Execute.Float64(2.0), Execute.Int32(n)], "is a float32, a float64 given"),
        ([Execute.Vec(x), Execute.Vec(out), Execute.Float32(2.0), Execute.Int64(n)], "argument 3 (n) of kernel scale_kernel is an int32, an int64 given"),
        ([Execute.Vec(wide), Execute.Vec(out), Execute.Float32(2.0), Execute.Int32(n)], "is a vector of 4-byte elements, the vector given has 8-byte elements"),
    ]
    for args, message in cases:
        with pytest.raises(hip.SarekHipError) as err:
            Execute.run_vectors(ir=ir, args=args, block=Execute.dims1d(64), grid=Execute.dims1d(4))
        assert err.value.status == hip.E_INVALID_ARG and message in str(err.value), (message, str(err.value))
        with pytest.raises(hip.SarekHipError) as err:
            Execute.run_pipeline([(ir, args, (64, 1, 1), (4, 1, 1))])
        assert err.value.status == hip.E_INVALID_ARG and message in str(err.value), (message, str(err.value))
    Transfer.flush()
    assert np.array_equal(out.to_array(), np.full(n, -7, np.float32))
    assert Execute.run_vectors(ir=ir, args=good, block=Execute.dims1d(64), grid=Execute.dims1d(4)) in ("map_f32", "jit")
    Transfer.flush()
    assert np.array_equal(out.to_array(), np.arange(n, dtype=np.float32) * 2 + 1)
