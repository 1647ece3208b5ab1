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


MAPS = {"scale": scale, "saxpy_with_let": saxpy_with_let, "norm3": norm3, "ramp_select": ramp_select,
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
