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


def _random_expression(rng, reads, index, scalars=("a", "b"), lets_made=(), depth=None):
    """A seeded f32 expression tree over the element's inputs (`reads`: the read forms), the f32 scalars, the int
    scalar k and the element's index: arithmetic, a guarded division, one-argument math intrinsics, `if` expressions
    on values and on the index, casts of index arithmetic, negation."""
    def int_expr(d):
        pick = rng.randint(0, 3 if d > 0 else 1)
        if pick == 0:
            return index
        if pick == 1:
            return i32(rng.randint(1, 9))
        if pick == 2:
            return mod(int_expr(d - 1), add(var("k"), i32(rng.randint(1, 5))))     # k >= 0 at the call sites
        return add(int_expr(d - 1), mul(int_expr(d - 1), i32(rng.randint(1, 3))))

    def leaf():
        pick = rng.randint(0, 5)
        if pick <= 2:
            return rng.choice(reads)
        if pick == 3:
            return var(rng.choice(scalars), "f32")
        if pick == 4 and lets_made:
            return rng.choice(lets_made)
        return f32(repr(round(rng.uniform(-4, 4), 3)))

    def expr(d):
        if d == 0:
            return leaf()
        pick = rng.randint(0, 9)
        if pick <= 3:
            return op(rng.choice(["add", "sub", "mul"]), expr(d - 1), expr(d - 1))
        if pick == 4:
            return div(expr(d - 1), add(intr("fabs", "Float32", expr(d - 1)), f32("1.5")))
        if pick == 5:
            return intr(rng.choice(["sqrt", "exp", "log", "sin", "cos", "tanh", "floor", "fabs"]), "Float32", expr(d - 1))
        if pick == 6:
            cond = op(rng.choice(["lt", "le", "gt"]), expr(d - 1), expr(d - 1))
            return f"(if {cond} {expr(d - 1)} {expr(d - 1)})"
        if pick == 7:
            cond = op(rng.choice(["lt", "eq"]), mod(index, i32(rng.randint(2, 7))), i32(rng.randint(0, 3)))
            return f"(if {cond} {expr(d - 1)} {expr(d - 1)})"
        if pick == 8:
            return f"(cast f32 {int_expr(2)})"
        return f"(neg {expr(d - 1)})"

    return expr(rng.randint(2, 4) if depth is None else depth)


def random_map(seed):
    """A seeded element-wise kernel of the shape the map class takes: one to four input vectors, two f32 scalars, an
    int scalar, immutable lets in front of the store.  Returns (ir, number of input vectors)."""
    import random
    rng = random.Random(seed)
    n_in = rng.randint(1, 4)
    params = [(f"x{i}", "(vec f32)") for i in range(n_in)] + [("out", "(vec f32)"), ("a", "f32"), ("b", "f32"),
                                                               ("k", "i32"), ("n", "i32")]
    _params(params)
    tid = var("tid")
    reads = [read(f"x{i}", tid) for i in range(n_in)]
    lets_made, bindings = [], []
    for j in range(rng.randint(0, 3)):
        e = _random_expression(rng, reads, tid, lets_made=tuple(lets_made), depth=rng.randint(1, 3))
        v = var(f"t{j}", "f32")
        bindings.append((v, e))
        lets_made.append(v)
    body = assign_elem("out", tid, _random_expression(rng, reads, tid, lets_made=tuple(lets_made)))
    for v, e in reversed(bindings):
        body = let(v, e, body)
    return kernel(params, let(tid, intr("global_thread_id", "Std"), if_(lt(tid, var("n")), body))), n_in


def random_map_rebinding(seed):
    """Like random_map, with two to five lets whose names come from (t, u, a): lets hide earlier lets of the same
    name and the scalar parameter a, every binding under an id of its own, every use with the id of the binding
    OCaml's scoping gives it.  Returns (ir, number of input vectors)."""
    import random
    rng = random.Random(77000 + seed)
    n_in = rng.randint(1, 3)
    params = [(f"x{i}", "(vec f32)") for i in range(n_in)] + [("out", "(vec f32)"), ("a", "f32"), ("b", "f32"),
                                                               ("k", "i32"), ("n", "i32")]
    _params(params)
    tid = var("tid")
    reads = [read(f"x{i}", tid) for i in range(n_in)]
    in_force, bindings, scalars = {}, [], ("a", "b")
    for j in range(rng.randint(2, 5)):
        e = _random_expression(rng, reads, tid, scalars=scalars, lets_made=tuple(in_force.values()), depth=rng.randint(1, 2))
        name = rng.choice(["t", "u", "a"])
        v = f"(var {name} {100 + j} f32)"
        bindings.append((v, e))
        in_force[name] = v
        if name == "a":
            scalars = ("b",)
    body = assign_elem("out", tid, _random_expression(rng, reads, tid, scalars=scalars, lets_made=tuple(in_force.values())))
    for v, e in reversed(bindings):
        body = let(v, e, body)
    return kernel(params, let(tid, intr("global_thread_id", "Std"), if_(lt(tid, var("n")), body))), n_in


def random_tree(seed, maximum=False):
    """The reference's block-256 sum (or maximum) tree with a seeded expression of one to three inputs, two f32
    scalars and an int scalar where it reads input[gid].  Returns (tree ir, map ir, number of inputs): the map
    kernel stores the same expression element by element, for the values the tree adds up or compares."""
    import random
    rng = random.Random(seed * 2 + int(maximum))
    n_in = rng.randint(1, 3)
    names = ["input", "y", "z"][:n_in]
    fresh()
    for name in ("a", "b"):
        var(name, "f32")
    var("k")
    tree_params = [("input", 1, "(vec f32)")] + [(nm, 30 + 2 * i, "(vec f32)") for i, nm in enumerate(names[1:])] + \
        [("output", 2, "(vec f32)"), ("a", 41, "f32"), ("b", 42, "f32"), ("k", 43, "i32"), ("n", 3, "i32")]
    # the tree classes want every input vector read: draw until the expression reads them all
    while True:
        state = rng.getstate()
        probe = _random_expression(rng, [read(nm, "@") for nm in names], "@", depth=rng.randint(1, 3))
        if all(f"(read {nm} @)" in probe for nm in names):
            break

    def leaf_of(index):
        rng.setstate(state)                       # the same tree for the tree kernel and for the map kernel
        return _random_expression(rng, [read(nm, index) for nm in names], index, depth=rng.randint(1, 3))

    def with_ids(text):                            # the builders number a, b, k as they like: the parameters' ids
        for name, ident, ty in (("a", 41, "f32"), ("b", 42, "f32"), ("k", 43, "i32")):
            import re
            text = re.sub(r"\(var " + name + r" \d+ " + ty + r"\)", f"(var {name} {ident} {ty})", text)
        return text

    build = _max_tree_with if maximum else _tree_with
    tree_ir = with_ids(build(leaf_of, tree_params))
    tid = "(var tid 50 i32)"
    map_params = " ".join(f"(param (var {nm} {i} {t}))" for nm, i, t in tree_params)
    map_ir = (f"(kernel sarek_kern (params {map_params}) (locals) (body (let {tid} (intr (Std) global_thread_id) "
              f"(if (lt {tid} (var n 3 i32)) (assign (lelem output {tid}) {with_ids(leaf_of(tid))})))) (native_fn true))")
    return tree_ir, map_ir, n_in
