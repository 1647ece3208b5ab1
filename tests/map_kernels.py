"""IR of element-wise kernels for the map tests: the shape `if tid < n then out[tid] <- f(in[tid] ..., scalars, tid)`
that a user's [%kernel] lowers to (sarek/ppx/Sarek_lower_ir.ml), written with the builders of the bench kernels."""
from spoc_amd.reference_kernels import (add, assign_elem, div, f32, fresh, i32, if_, intr, kernel, let, lets, lt, mod,
                                        mul, op, read, sub, var)

GID_SUM = None


def _params(params):
    fresh()
    for p, t in params:
        var(p, t)


def scale():
    """out = alpha * x"""
    params = [("x", "(vec f32)"), ("out", "(vec f32)"), ("alpha", "f32"), ("n", "i32")]
    _params(params)
    tid = var("tid")
    return kernel(params, let(tid, intr("global_thread_id", "Std"),
                              if_(lt(tid, var("n")), assign_elem("out", tid, mul(var("alpha", "f32"), read("x", tid))))))


def saxpy_with_let():
    """t = alpha * x; out = t + y, thread id written out as threadIdx + blockIdx * blockDim"""
    params = [("x", "(vec f32)"), ("y", "(vec f32)"), ("out", "(vec f32)"), ("alpha", "f32"), ("n", "i32")]
    _params(params)
    tid, t = var("tid"), var("t", "f32")
    gid = add(intr("thread_idx_x"), mul(intr("block_idx_x"), intr("block_dim_x")))
    return kernel(params, let(tid, gid, if_(lt(tid, var("n")),
                                           let(t, mul(var("alpha", "f32"), read("x", tid)),
                                               assign_elem("out", tid, add(t, read("y", tid)))))))


def norm3():
    """out = sqrt(x*x + y*y + z*z) / (1 + fabs(z)): three inputs, math intrinsics, a division"""
    params = [("out", "(vec f32)"), ("x", "(vec f32)"), ("y", "(vec f32)"), ("z", "(vec f32)"), ("n", "i32")]
    _params(params)
    tid, s = var("tid"), var("s", "f32")
    x, y, z = read("x", tid), read("y", tid), read("z", tid)
    e = div(intr("sqrt", "Float32", s), add(f32("1.0"), intr("fabs", "Float32", z)))
    return kernel(params, let(tid, intr("global_thread_id", "Std"),
                              if_(lt(tid, var("n")),
                                  let(s, add(add(mul(x, x), mul(y, y)), mul(z, z)), assign_elem("out", tid, e)))))


def ramp_select():
    """out = if tid mod k < 3 then x else y * float(tid mod 7): the element's index, an int scalar, an if expression"""
    params = [("x", "(vec f32)"), ("y", "(vec f32)"), ("out", "(vec f32)"), ("k", "i32"), ("n", "i32")]
    _params(params)
    tid = var("tid")
    e = f"(if {lt(mod(tid, var('k')), i32(3))} {read('x', tid)} {mul(read('y', tid), '(cast f32 ' + mod(tid, i32(7)) + ')')})"
    return kernel(params, let(tid, intr("global_thread_id", "Std"), if_(lt(tid, var("n")), assign_elem("out", tid, e))))


def fill_const():
    """out = c: no input vector at all"""
    params = [("out", "(vec f32)"), ("c", "f32"), ("n", "i32")]
    _params(params)
    tid = var("tid")
    return kernel(params, let(tid, intr("global_thread_id", "Std"),
                              if_(lt(tid, var("n")), assign_elem("out", tid, var("c", "f32")))))


def six_inputs():
    """out = ((v0 + v1) + v2 * v3) + (v4 - v5): the most inputs the class takes"""
    params = [(f"v{i}", "(vec f32)") for i in range(6)] + [("out", "(vec f32)"), ("n", "i32")]
    _params(params)
    tid = var("tid")
    r = [read(f"v{i}", tid) for i in range(6)]
    e = add(add(add(r[0], r[1]), mul(r[2], r[3])), sub(r[4], r[5]))
    return kernel(params, let(tid, intr("global_thread_id", "Std"), if_(lt(tid, var("n")), assign_elem("out", tid, e))))


def short_names():
    """e = u * i + v * t + float(tid mod j), over q elements: every parameter carries one of the short names a kernel
    text likes for its own loop variables (the rebuilt texts keep theirs under a prefix, so these are the kernel's)"""
    params = [("i", "(vec f32)"), ("t", "(vec f32)"), ("e", "(vec f32)"), ("u", "f32"), ("v", "f32"), ("j", "i32"),
              ("q", "i32")]
    _params(params)
    tid = var("tid")
    ex = add(add(mul(var("u", "f32"), read("i", tid)), mul(var("v", "f32"), read("t", tid))),
             "(cast f32 " + mod(tid, var("j")) + ")")
    return kernel(params, let(tid, intr("global_thread_id", "Std"), if_(lt(tid, var("q")), assign_elem("e", tid, ex))))


MAPS = {"short_names": short_names, "six_inputs": six_inputs, "scale": scale, "saxpy_with_let": saxpy_with_let, "norm3": norm3, "ramp_select": ramp_select,
        "fill_const": fill_const}


def near_misses():
    """(name, IR) of kernels one step outside the class: each must be left to the plain lowering."""
    out = []
    base = [("x", "(vec f32)"), ("out", "(vec f32)"), ("n", "i32")]

    def k(params, body_of):
        _params(params)
        tid = var("tid")
        return kernel(params, let(tid, intr("global_thread_id", "Std"), body_of(tid)))

    out.append(("neighbour read", k(base, lambda t: if_(lt(t, var("n")), assign_elem("out", t, read("x", add(t, i32(1))))))))
    out.append(("reads its output", k(base, lambda t: if_(lt(t, var("n")),
                                                          assign_elem("out", t, add(read("out", t), read("x", t)))))))
    out.append(("shifted store", k(base, lambda t: if_(lt(t, var("n")), assign_elem("out", sub(t, i32(1)), read("x", t))))))
    out.append(("else branch", k(base, lambda t: if_(lt(t, var("n")), assign_elem("out", t, read("x", t)),
                                                     assign_elem("out", t, f32("0.0"))))))
    out.append(("launch geometry in the expression",
                k(base, lambda t: if_(lt(t, var("n")),
                                      assign_elem("out", t, mul(read("x", t), "(cast f32 " + intr("block_idx_x") + ")"))))))
    out.append(("guard on another bound", k(base, lambda t: if_(lt(t, i32(1000)), assign_elem("out", t, read("x", t))))))
    out.append(("no guard", k(base, lambda t: assign_elem("out", t, read("x", t)))))
    own = [("x", "(vec f32)"), ("out", "(vec f32)"), ("sarek_f_n", "f32"), ("n", "i32")]
    out.append(("a scalar that carries the rebuilt texts' own prefix",
                k(own, lambda t: if_(lt(t, var("n")), assign_elem("out", t, mul(read("x", t), var("sarek_f_n", "f32")))))))
    ints = [("x", "(vec i32)"), ("out", "(vec i32)"), ("n", "i32")]
    out.append(("int32 vectors", k(ints, lambda t: if_(lt(t, var("n")), assign_elem("out", t, read("x", t))))))
    two = [("x", "(vec f32)"), ("out", "(vec f32)"), ("out2", "(vec f32)"), ("n", "i32")]
    out.append(("two stores", k(two, lambda t: if_(lt(t, var("n")),
                                                   "(seq " + assign_elem("out", t, read("x", t)) + " " +
                                                   assign_elem("out2", t, read("x", t)) + ")"))))
    m = var("acc", "f32", mut=True)
    out.append(("mutable local", k(base, lambda t: if_(lt(t, var("n")),
                                                       f"(letmut {var('acc', 'f32', mut=True)} {read('x', t)} " +
                                                       assign_elem("out", t, var("acc", "f32", mut=True)) + ")"))))
    return out


# ---- block-256 tree sums with an expression in front (benchmarks/bench_reduction.ml:62-96 with a map where it reads) ----

def _tree_with(leaf_of, params):
    """The reference's tree kernel text with `leaf_of(gid)` where it reads input[gid]."""
    from spoc_amd import reference_kernels as rk
    base = rk.tree(False)
    gid = "(var gid 6 i32)"
    old = f"(read input {gid})"
    assert base.count(old) == 1
    text = base.replace(old, leaf_of(gid))
    head = "(params (param (var input 1 (vec f32))) (param (var output 2 (vec f32))) (param (var n 3 i32)))"
    assert head in text
    return text.replace(head, "(params " + " ".join(f"(param (var {n} {i} {t}))" for n, i, t in params) + ")")


def sum_of_squares():
    """sum of x^2"""
    return _tree_with(lambda g: f"(mul (read input {g}) (read input {g}))",
                      [("input", 1, "(vec f32)"), ("output", 2, "(vec f32)"), ("n", 3, "i32")])


def weighted_abs_sum():
    """sum of alpha * |x| * w: two inputs, a scalar, a math intrinsic"""
    return _tree_with(lambda g: f"(mul (mul (var alpha 31 f32) (intr (Float32) fabs (read input {g}))) (read w {g}))",
                      [("input", 1, "(vec f32)"), ("w", 30, "(vec f32)"), ("output", 2, "(vec f32)"), ("alpha", 31, "f32"),
                       ("n", 3, "i32")])


def squared_distance():
    """sum of (x - y)^2"""
    return _tree_with(lambda g: f"(mul (sub (read input {g}) (read y {g})) (sub (read input {g}) (read y {g})))",
                      [("input", 1, "(vec f32)"), ("y", 30, "(vec f32)"), ("output", 2, "(vec f32)"), ("n", 3, "i32")])


def short_named_tree():
    """sum of u * i * t with the vectors named i and t, the output e, the scalar u, the length q"""
    text = _tree_with(lambda g: f"(mul (mul (var u 31 f32) (read input {g})) (read t {g}))",
                      [("input", 1, "(vec f32)"), ("t", 30, "(vec f32)"), ("output", 2, "(vec f32)"), ("u", 31, "f32"),
                       ("n", 3, "i32")])
    return text.replace("input", "i").replace("(var n 3 i32)", "(var q 3 i32)").replace("output", "e")


TREES = {"short_named_tree": short_named_tree, "sum_of_squares": sum_of_squares, "weighted_abs_sum": weighted_abs_sum, "squared_distance": squared_distance}


def tree_near_misses():
    sq = sum_of_squares()
    out = [("a neighbour in the expression", sq.replace("(mul (read input (var gid 6 i32))", "(mul (read input (add (var gid 6 i32) (i32 1)))", 1)),
           ("a tree of 128", sq.replace("(i32 128)", "(i32 64)", 1)),
           ("padding with one", sq.replace("(f32 0.0)", "(f32 1.0)", 1)),
           ("a product tree", sq.replace("(add (read sdata", "(mul (read sdata", 1)),
           ("the sum stored elsewhere", sq.replace("(lelem output (intr (Gpu) block_idx_x))", "(lelem output (intr (Gpu) thread_idx_x))"))]
    for _, text in out:
        assert text != sq
    return out


def _max_tree_with(leaf_of, params, pad="(f32 -1000000.0)"):
    """benchmarks/bench_reduction_max.ml:18-100 with `leaf_of(gid)` where it reads input[gid]."""
    import os
    ir = open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ir", "reduction_max.ir")).read()
    free = "(var Float.neg_infinity"
    i = ir.index(free)
    j = ir.index(")", i) + 1
    ir = ir[:i] + pad + ir[j:]
    gid = "(var gid 6 i32)"
    old = f"(read input {gid})"
    assert ir.count(old) == 1, ir
    ir = ir.replace(old, leaf_of(gid))
    head = ir[ir.index("(params"):ir.index("(locals)")]
    return ir.replace(head, "(params " + " ".join(f"(param (var {n} {k} {t}))" for n, k, t in params) + ")\n ")


def max_abs():
    """max |x|: the infinity norm"""
    return _max_tree_with(lambda g: f"(intr (Float32) fabs (read input {g}))",
                          [("input", 1, "(vec f32)"), ("output", 2, "(vec f32)"), ("n", 3, "i32")], pad="(f32 0.0)")


def max_abs_difference():
    """max |x - y|"""
    return _max_tree_with(lambda g: f"(intr (Float32) fabs (sub (read input {g}) (read y {g})))",
                          [("input", 1, "(vec f32)"), ("y", 30, "(vec f32)"), ("output", 2, "(vec f32)"), ("n", 3, "i32")])


MAX_TREES = {"max_abs": max_abs, "max_abs_difference": max_abs_difference}
