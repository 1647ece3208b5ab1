"""Sarek IR of the reference's benchmark kernels, in the s-expression form that
sarek_hip_generate_source reads.

In the reference this IR comes out of the PPX at compile time (`[%kernel ...]` in
benchmarks/bench_*.ml -> Kirc_types.body_ir); without an OCaml toolchain the same trees are
written down here, transcribed from the kernel sources with the reference's lowering rules
(sarek/ppx/Sarek_lower_ir.ml: let%shared -> let of an array creation :496-507,
let%superstep -> block; barrier :508-515, for -> inclusive loop :476-484, vector store ->
assignment to an array element :422-431) and pinned by the golden generated text of each
kernel (benchmarks/descriptions/generated/*_generated.md): the HIP lowering of these trees
has to reproduce that text.  KERNELS maps a kernel name to a function returning its IR.
"""
_ids = {}


def var(name, ty="i32", mut=False):
    vid = _ids.setdefault(name, len(_ids) + 1)
    return f"(var {name} {vid} {ty}{' mut' if mut else ''})"


def i32(n):
    return f"(i32 {n})"


def f32(x):
    return f"(f32 {x})"


def op(name, a, b):
    return f"({name} {a} {b})"


def add(a, b): return op("add", a, b)
def sub(a, b): return op("sub", a, b)
def mul(a, b): return op("mul", a, b)
def div(a, b): return op("div", a, b)
def mod(a, b): return op("mod", a, b)
def lt(a, b): return op("lt", a, b)
def le(a, b): return op("le", a, b)
def gt(a, b): return op("gt", a, b)
def eq(a, b): return op("eq", a, b)
def land(a, b): return op("and", a, b)
def read(arr, idx): return f"(read {arr} {idx})"
def intr(name, mod="Gpu", *args): return f"(intr ({mod}) {name}{''.join(' ' + a for a in args)})"
def assign_elem(arr, idx, e): return f"(assign (lelem {arr} {idx}) {e})"
def assign_var(v, e): return f"(assign (lvar {v}) {e})"
def let(v, e, body): return f"(let {v} {e}\n {body})"
def letmut(v, e, body): return f"(letmut {v} {e}\n {body})"
def seq(*s): return "(seq\n " + "\n ".join(s) + ")"
def block(s): return f"(block {s})"
def if_(c, t, e=None): return f"(if {c} {t}{' ' + e if e else ''})"
def for_(v, lo, hi, body): return f"(for {v} {lo} {hi} upto {body})"
def while_(c, body): return f"(while {c} {body})"
def shared(v, ty, n, body): return let(v, f"(newarray {ty} {i32(n)} shared)", body)
BARRIER = "(barrier)"


def lets(bindings, body):
    for v, e in reversed(bindings):
        body = let(v, e, body)
    return body


def kernel(params, body):
    ps = []
    for name, ty in params:
        ps.append(f"(param {var(name, ty)})")
    return ("(kernel sarek_kern\n (params " + " ".join(ps) + ")\n (locals)\n (body\n " + body +
            ")\n (native_fn true))\n")


def fresh():
    _ids.clear()


def stream_triad():
    fresh()
    params = [("a", "(vec f32)"), ("b", "(vec f32)"), ("c", "(vec f32)"), ("scalar", "f32"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid = var("tid")
    body = let(tid, intr("global_thread_id", "Std"),
               if_(lt(tid, var("n")),
                   assign_elem("a", tid, add(read("b", tid), mul(read("c", tid), var("scalar", "f32"))))))
    return kernel(params, body)


def vector_add():
    fresh()
    params = [("a", "(vec f32)"), ("b", "(vec f32)"), ("c", "(vec f32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid = var("tid")
    body = let(tid, intr("global_thread_id", "Std"),
               if_(lt(tid, var("n")), assign_elem("c", tid, add(read("a", tid), read("b", tid)))))
    return kernel(params, body)


def vector_copy():
    fresh()
    params = [("a", "(vec f32)"), ("b", "(vec f32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    tid = var("tid")
    body = let(tid, intr("global_thread_id", "Std"),
               if_(lt(tid, var("n")), assign_elem("b", tid, read("a", tid))))
    return kernel(params, body)


def matrix_mul():
    fresh()
    params = [("a", "(vec f32)"), ("b", "(vec f32)"), ("c", "(vec f32)"), ("m", "i32"), ("n", "i32"), ("k", "i32")]
    for p, t in params:
        var(p, t)
    tid, row, col, i = var("tid"), var("row"), var("col"), var("i", mut=True)
    s = var("sum", "f32", mut=True)
    n, m, k = var("n"), var("m"), var("k")
    inner = letmut(s, f32("0.0"), seq(
        for_(i, i32(0), sub(k, i32(1)),
             assign_var(s, add(s, mul(read("a", add(mul(row, k), i)), read("b", add(mul(i, n), col)))))),
        assign_elem("c", add(mul(row, n), col), s)))
    body = lets([(tid, intr("global_thread_id", "Std")), (row, div(tid, n)), (col, mod(tid, n))],
                if_(land(lt(row, m), lt(col, n)), inner))
    return kernel(params, body)


def matrix_mul_tiled():
    fresh()
    params = [("a", "(vec f32)"), ("b", "(vec f32)"), ("c", "(vec f32)"), ("m", "i32"), ("n", "i32"), ("k", "i32")]
    for p, t in params:
        var(p, t)
    m, n, k = var("m"), var("n"), var("k")
    ta, tb = var("tile_a", "(array f32 shared)"), var("tile_b", "(array f32 shared)")
    tx, ty, row, col = var("tx"), var("ty"), var("row"), var("col")
    ts, nt = var("tile_size"), var("num_tiles")
    s = var("sum", "f32", mut=True)
    t, i = var("t", mut=True), var("i", mut=True)
    a_col, b_row = var("a_col"), var("b_row")
    slot = add(mul(ty, ts), tx)
    load_a = block(let(a_col, add(mul(t, ts), tx),
                       if_(land(lt(row, m), lt(a_col, k)),
                           assign_elem("tile_a", slot, read("a", add(mul(row, k), a_col))),
                           assign_elem("tile_a", slot, f32("0.0")))))
    load_b = block(let(b_row, add(mul(t, ts), ty),
                       if_(land(lt(b_row, k), lt(col, n)),
                           assign_elem("tile_b", slot, read("b", add(mul(b_row, n), col))),
                           assign_elem("tile_b", slot, f32("0.0")))))
    compute = block(for_(i, i32(0), sub(ts, i32(1)),
                         assign_var(s, add(s, mul(read("tile_a", add(mul(ty, ts), i)),
                                                  read("tile_b", add(mul(i, ts), tx)))))))
    loop = for_(t, i32(0), sub(nt, i32(1)), seq(load_a, BARRIER, load_b, BARRIER, compute, BARRIER))
    store = if_(land(lt(row, m), lt(col, n)), assign_elem("c", add(mul(row, n), col), s))
    body = shared(ta, "f32", 256, shared(tb, "f32", 256, lets(
        [(tx, intr("thread_idx_x")), (ty, intr("thread_idx_y")),
         (row, add(ty, mul(intr("block_dim_y"), intr("block_idx_y")))),
         (col, add(tx, mul(intr("block_dim_x"), intr("block_idx_x")))),
         (ts, i32(16)), (nt, div(sub(add(k, ts), i32(1)), ts))],
        letmut(s, f32("0.0"), seq(loop, store)))))
    return kernel(params, body)


def tree(dot):
    fresh()
    if dot:
        params = [("a", "(vec f32)"), ("b", "(vec f32)"), ("output", "(vec f32)"), ("n", "i32")]
    else:
        params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    n = var("n")
    sdata = var("sdata", "(array f32 shared)")
    tid, gid = var("tid"), var("gid")
    value = mul(read("a", gid), read("b", gid)) if dot else read("input", gid)
    steps = [block(if_(lt(gid, n), assign_elem("sdata", tid, value), assign_elem("sdata", tid, f32("0.0")))),
             BARRIER]
    half = 128
    while half >= 1:
        steps += [block(if_(lt(tid, i32(half)),
                            assign_elem("sdata", tid, add(read("sdata", tid), read("sdata", add(tid, i32(half))))))),
                  BARRIER]
        half //= 2
    final = if_(eq(tid, i32(0)), assign_elem("output", intr("block_idx_x"), read("sdata", i32(0))))
    # the golden text of the reduction kernel wraps the final store in a scope followed by a
    # barrier; the dot-product kernel's does not
    steps += [final] if dot else [block(final), BARRIER]
    body = shared(sdata, "f32", 256, lets(
        [(tid, intr("thread_idx_x")),
         (gid, add(intr("thread_idx_x"), mul(intr("block_dim_x"), intr("block_idx_x"))))],
        seq(*steps)))
    return kernel(params, body)


def transpose_naive():
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("width", "i32"), ("height", "i32")]
    for p, t in params:
        var(p, t)
    w, h = var("width"), var("height")
    tid, n, col, row, ii, oi = var("tid"), var("n"), var("col"), var("row"), var("in_idx"), var("out_idx")
    inner = lets([(col, mod(tid, w)), (row, div(tid, w)), (ii, add(mul(row, w), col)),
                  (oi, add(mul(col, h), row))], assign_elem("output", oi, read("input", ii)))
    body = lets([(tid, intr("global_thread_id", "Std")), (n, mul(w, h))], if_(lt(tid, n), inner))
    return kernel(params, body)


def gather():
    fresh()
    params = [("input", "(vec i32)"), ("indices", "(vec i32)"), ("output", "(vec i32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    i, idx = var("i"), var("idx")
    body = let(i, intr("global_thread_id", "Std"),
               if_(lt(i, var("n")), let(idx, read("indices", i), assign_elem("output", i, read("input", idx)))))
    return kernel(params, body)


def mandelbrot():
    fresh()
    params = [("output", "(vec i32)"), ("width", "i32"), ("height", "i32"), ("max_iter", "i32")]
    for p, t in params:
        var(p, t)
    w, h, mi = var("width"), var("height"), var("max_iter")
    px, py = var("px"), var("py")
    x0, y0 = var("x0", "f32"), var("y0", "f32")
    x, y = var("x", "f32", True), var("y", "f32", True)
    it = var("iter", "i32", True)
    xt = var("xtemp", "f32")

    def tofloat(e):
        return f"(intr (Float32) of_int (template \"(float)(%s)\") {e})"
    loop = while_(land(le(add(mul(x, x), mul(y, y)), f32("4.0")), lt(it, mi)),
                  let(xt, add(sub(mul(x, x), mul(y, y)), x0),
                      seq(assign_var(y, add(mul(mul(f32("2.0"), x), y), y0)), assign_var(x, xt),
                          assign_var(it, add(it, i32(1))))))
    inner = lets([(x0, sub(mul(f32("4.0"), div(tofloat(px), tofloat(w))), f32("2.5"))),
                  (y0, sub(mul(f32("3.0"), div(tofloat(py), tofloat(h))), f32("1.5")))],
                 letmut(x, f32("0.0"), letmut(y, f32("0.0"), letmut(it, i32(0), seq(
                     loop, assign_elem("output", add(mul(py, w), px), it))))))
    body = lets([(px, intr("global_idx_x", "Std")), (py, intr("global_idx_y", "Std"))],
                if_(land(lt(px, w), lt(py, h)), inner))
    return kernel(params, body)


def reduction_max(fill=None):
    """fill=None gives the tree as the golden generated text has it (out-of-range slots take
    the free variable Float.neg_infinity); a number gives the kernel as
    benchmarks/bench_reduction_max.ml:18-100 writes it today (fill = -1000000.0)."""
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    n = var("n")
    sdata = var("sdata", "(array f32 shared)")
    tid, gid = var("tid"), var("gid")
    # the golden text was generated from a source that wrote Float.neg_infinity: a global
    # reference, which lowers to a plain variable of that name (Sarek_lower_ir.ml:378-380)
    ninf = var("Float.neg_infinity", "f32") if fill is None else f32(repr(float(fill)))
    steps = [block(if_(lt(gid, n), assign_elem("sdata", tid, read("input", gid)),
                       assign_elem("sdata", tid, ninf))), BARRIER]
    half = 128
    while half >= 1:
        a, b = var("a%d" % half, "f32"), var("b%d" % half, "f32")
        a, b = a.replace("a%d" % half, "a", 1), b.replace("b%d" % half, "b", 1)
        steps += [block(if_(lt(tid, i32(half)),
                            let(a, read("sdata", tid),
                                let(b, read("sdata", add(tid, i32(half))),
                                    if_(gt(b, a), assign_elem("sdata", tid, b)))))), BARRIER]
        half //= 2
    steps += [block(if_(eq(tid, i32(0)), assign_elem("output", intr("block_idx_x"), read("sdata", i32(0))))),
              BARRIER]
    body = shared(sdata, "f32", 256, lets(
        [(tid, intr("thread_idx_x")),
         (gid, add(intr("thread_idx_x"), mul(intr("block_dim_x"), intr("block_idx_x"))))],
        seq(*steps)))
    return kernel(params, body)


def transpose_tiled():
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("width", "i32"), ("height", "i32")]
    for p, t in params:
        var(p, t)
    w, h = var("width"), var("height")
    tile = var("tile", "(array f32 shared)")
    ts, tx, ty = var("tile_size"), var("tx"), var("ty")
    bc, br, rc, rr = var("block_col"), var("block_row"), var("read_col"), var("read_row")
    ri, ti = var("read_idx"), var("tile_idx")
    wc, wr = var("write_col"), var("write_row")
    ti2, wi = var("tile_idx2"), var("write_idx")
    ti2 = ti2.replace("tile_idx2", "tile_idx", 1)
    load = block(if_(land(lt(rc, w), lt(rr, h)),
                     let(ri, add(mul(rr, w), rc),
                         let(ti, add(mul(ty, i32(17)), tx),
                             assign_elem("tile", ti, read("input", ri))))))
    store = block(if_(land(lt(wc, h), lt(wr, w)),
                      let(ti2, add(mul(tx, i32(17)), ty),
                          let(wi, add(mul(wr, h), wc),
                              assign_elem("output", wi, read("tile", ti2))))))
    body = shared(tile, "f32", 272, lets(
        [(ts, i32(16)), (tx, intr("thread_idx_x")), (ty, intr("thread_idx_y")),
         (bc, mul(intr("block_idx_x"), ts)), (br, mul(intr("block_idx_y"), ts)),
         (rc, add(bc, tx)), (rr, add(br, ty))],
        seq(load, BARRIER, lets([(wc, add(br, tx)), (wr, add(bc, ty))], seq(store, BARRIER)))))
    return kernel(params, body)


def scatter():
    fresh()
    params = [("input", "(vec i32)"), ("indices", "(vec i32)"), ("output", "(vec i32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    i, idx = var("i"), var("idx")
    body = let(i, intr("global_thread_id", "Std"),
               if_(lt(i, var("n")), let(idx, read("indices", i), assign_elem("output", idx, read("input", i)))))
    return kernel(params, body)


def radix_sort_histogram():
    fresh()
    params = [("input", "(vec i32)"), ("histogram", "(vec i32)"), ("n", "i32"), ("shift", "i32"), ("mask", "i32")]
    for p, t in params:
        var(p, t)
    n, shift, mask = var("n"), var("shift"), var("mask")
    lh = var("local_hist", "(array i32 shared)")
    hist = var("histogram", "(vec i32)")
    tid, gid, nb = var("tid"), var("gid"), var("num_bins")
    value, digit = var("value"), var("digit")
    old1, old2 = var("_old"), var("_old2").replace("_old2", "_old", 1)
    clear = block(if_(lt(tid, nb), assign_elem("local_hist", tid, i32(0))))
    count = block(if_(lt(gid, n),
                      let(value, read("input", gid),
                          let(digit, op("bitand", op("shr", value, shift), mask),
                              let(old1, intr("atomic_add_int32", "Gpu", lh, digit, i32(1)), "(empty)")))))
    flush = block(if_(lt(tid, nb),
                      let(old2, intr("atomic_add_global_int32", "Gpu", hist, tid, read("local_hist", tid)),
                          "(empty)")))
    body = shared(lh, "i32", 256, lets(
        [(tid, intr("thread_idx_x")), (gid, intr("global_thread_id", "Std")), (nb, i32(256))],
        seq(clear, BARRIER, count, BARRIER, flush, BARRIER)))
    return kernel(params, body)


def radix_sort_scatter():
    fresh()
    params = [("input", "(vec i32)"), ("output", "(vec i32)"), ("counters", "(vec i32)"), ("n", "i32"),
              ("shift", "i32"), ("mask", "i32")]
    for p, t in params:
        var(p, t)
    n, shift, mask = var("n"), var("shift"), var("mask")
    counters = var("counters", "(vec i32)")
    gid, value, digit, pos = var("gid"), var("value"), var("digit"), var("pos")
    body = let(gid, intr("global_thread_id", "Std"),
               if_(lt(gid, n),
                   let(value, read("input", gid),
                       let(digit, op("bitand", op("shr", value, shift), mask),
                           let(pos, intr("atomic_add_global_int32", "Gpu", counters, digit, i32(1)),
                               assign_elem("output", pos, value))))))
    return kernel(params, body)


def inclusive_scan():
    """benchmarks/bench_scan.ml:48-109: Hillis-Steele inclusive scan of one 256-element block in
    two shared int32 arrays that swap roles every superstep.  No golden generated text exists
    for this kernel; the transcription is pinned by its result (a prefix sum, exact in int32)."""
    fresh()
    params = [("input", "(vec i32)"), ("output", "(vec i32)"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    n = var("n")
    temp, temp2 = var("temp", "(array i32 shared)"), var("temp2", "(array i32 shared)")
    tid, gid = var("tid"), var("gid")
    steps = [block(if_(lt(gid, n), assign_elem("temp", tid, read("input", gid)), assign_elem("temp", tid, i32(0)))),
             BARRIER]
    src, dst = "temp", "temp2"
    d = 1
    while d <= 128:
        v, a = var(f"v{d}"), var(f"add{d}")
        steps += [block(let(v, read(src, tid),
                            let(a, f"(if {op('ge', tid, i32(d))} {read(src, sub(tid, i32(d)))} {i32(0)})",
                                assign_elem(dst, tid, add(v, a))))),
                  BARRIER]
        src, dst = dst, src
        d *= 2
    steps.append(if_(lt(gid, n), assign_elem("output", gid, read(src, tid))))
    body = shared(temp, "i32", 512, shared(temp2, "i32", 512, lets(
        [(tid, intr("thread_idx_x")),
         (gid, add(intr("thread_idx_x"), mul(intr("block_dim_x"), intr("block_idx_x"))))],
        seq(*steps))))
    return kernel(params, body)


KERNELS = {
    "stream_triad": stream_triad, "vector_add": vector_add, "vector_copy": vector_copy,
    "matrix_mul": matrix_mul, "matrix_mul_tiled": matrix_mul_tiled,
    "reduction": lambda: tree(False), "dot_product": lambda: tree(True),
    "transpose_naive": transpose_naive, "gather": gather, "mandelbrot": mandelbrot,
    "reduction_max": reduction_max, "transpose_tiled": transpose_tiled, "scatter": scatter,
    "radix_sort_histogram": radix_sort_histogram, "radix_sort_scatter": radix_sort_scatter,
}


