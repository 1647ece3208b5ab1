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


def histogram():
    """benchmarks/bench_histogram.ml:54-84 (= sarek/tests/e2e/test_histogram.ml:43-69): per-block
    histogram in shared memory by atomic adds, merged into the global one by atomic adds."""
    fresh()
    params = [("input", "(vec i32)"), ("histogram", "(vec i32)"), ("n", "i32"), ("num_bins", "i32")]
    for p, t in params:
        var(p, t)
    nn, nb = var("n"), var("num_bins")
    lh = var("local_hist", "(array i32 shared)")
    tid, gid, b = var("tid"), var("gid"), var("bin")
    old1, old2 = var("_old"), var("_old#2").replace("_old#2", "_old", 1)
    count = if_(lt(gid, nn), let(b, mod(read("input", gid), nb),
                                 let(old1, intr("atomic_add_int32", "Gpu", lh, b, i32(1)), "(expr (unit))")))
    merge = if_(lt(tid, nb), let(old2, intr("atomic_add_global_int32", "Gpu", var("histogram", "(vec i32)"), tid,
                                            read("local_hist", tid)), "(expr (unit))"))
    body = shared(lh, "i32", 256, lets(
        [(tid, intr("thread_idx_x")), (gid, intr("global_thread_id", "Std"))],
        seq(block(if_(lt(tid, nb), assign_elem("local_hist", tid, i32(0)))), BARRIER,
            seq(block(count), BARRIER, seq(block(merge), BARRIER, "(expr (unit))")))))
    return kernel(params, body)


def stencil_2d():
    """benchmarks/bench_stencil_2d.ml:43-58: five-point mean over the interior of a 2-D grid."""
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("width", "i32"), ("height", "i32")]
    for p, t in params:
        var(p, t)
    w, h = var("width"), var("height")
    x, y, idx = var("x"), var("y"), var("idx")
    names = ["up", "down", "left", "right", "center"]
    up, down, left, right, center = (var(n, "f32") for n in names)
    inside = land(land(land(gt(x, i32(0)), lt(x, sub(w, i32(1)))), gt(y, i32(0))), lt(y, sub(h, i32(1))))
    mean = div(add(add(add(add(up, down), left), right), center), f32("5.0"))
    inner = lets([(idx, add(mul(y, w), x)),
                  (up, read("input", add(mul(sub(y, i32(1)), w), x))),
                  (down, read("input", add(mul(add(y, i32(1)), w), x))),
                  (left, read("input", sub(add(mul(y, w), x), i32(1)))),
                  (right, read("input", add(add(mul(y, w), x), i32(1)))),
                  (center, read("input", idx))], assign_elem("output", idx, mean))
    body = lets([(x, add(intr("thread_idx_x"), mul(intr("block_idx_x"), intr("block_dim_x")))),
                 (y, add(intr("thread_idx_y"), mul(intr("block_idx_y"), intr("block_dim_y"))))], if_(inside, inner))
    return kernel(params, body)


def conv2d():
    """benchmarks/bench_conv2d.ml:49-77: 3x3 box filter, one thread per pixel of a 1-D launch,
    zero on the border."""
    fresh()
    params = [("input", "(vec f32)"), ("output", "(vec f32)"), ("width", "i32"), ("height", "i32")]
    for p, t in params:
        var(p, t)
    w, h = var("width"), var("height")
    tid, n, x, y = var("tid"), var("n"), var("x"), var("y")
    border = op("or", op("or", op("or", eq(x, i32(0)), eq(x, sub(w, i32(1)))), eq(y, i32(0))), eq(y, sub(h, i32(1))))
    taps, binds = [], []
    for r, dy in enumerate((-1, 0, 1)):
        row = y if dy == 0 else (sub(y, i32(1)) if dy < 0 else add(y, i32(1)))
        for c, dx in enumerate((-1, 0, 1)):
            at = add(mul(row, w), x)
            at = at if dx == 0 else (sub(at, i32(1)) if dx < 0 else add(at, i32(1)))
            v = var(f"p{r}{c}", "f32")
            taps.append(v)
            binds.append((v, read("input", at)))
    total = taps[0]
    for t in taps[1:]:
        total = add(total, t)
    s = var("sum", "f32")
    inner = lets(binds, let(s, total, assign_elem("output", tid, div(s, f32("9.0")))))
    body = lets([(tid, intr("global_thread_id", "Std")), (n, mul(w, h))],
                if_(lt(tid, n), lets([(x, mod(tid, w)), (y, div(tid, w))],
                                     if_(border, assign_elem("output", tid, f32("0.0")), inner))))
    return kernel(params, body)


def bitonic_sort_step():
    """benchmarks/bench_bitonic_sort.ml:39-56: one compare-exchange step of a bitonic network."""
    fresh()
    params = [("data", "(vec i32)"), ("j", "i32"), ("k", "i32"), ("n", "i32")]
    for p, t in params:
        var(p, t)
    i, ij, di, dij, asc = var("i"), var("ij"), var("di"), var("dij"), var("ascending", "bool")
    cond = op("or", land(asc, gt(di, dij)), land(f"(not {asc})", lt(di, dij)))
    body = let(i, intr("global_thread_id", "Std"), if_(lt(i, var("n")), let(
        ij, op("bitxor", i, var("j")), if_(gt(ij, i), lets(
            [(di, read("data", i)), (dij, read("data", ij)), (asc, eq(op("bitand", i, var("k")), i32(0)))],
            if_(cond, seq(assign_elem("data", i, dij), assign_elem("data", ij, di))))))))
    return kernel(params, body)


def nbody_accel():
    """benchmarks/bench_nbody.ml:63-105: accelerations of n bodies, all pairs; positions go through
    a record built by a helper function."""
    part = "(record particle (x f32) (y f32) (z f32))"
    P, Q = f"(var p 20 {part})", f"(var q 21 {part})"

    def mk(idx):
        return f"(app (var make_p 0 {part}) (read xs {idx}) (read ys {idx}) (read zs {idx}))"
    tid, iv, jv = "(var tid 8 i32)", "(var i 18 i32)", "(var j 9 i32 mut)"
    fx, fy, fz = ("(var f%s %d f32 mut)" % (c, 10 + k) for k, c in enumerate("xyz"))
    dx, dy, dz = ("(var d%s %d f32)" % (c, 13 + k) for k, c in enumerate("xyz"))
    dist2, inv = "(var dist2 16 f32)", "(var inv 17 f32)"
    return f"""(kernel sarek_kern
      (params (param (var xs 1 (vec f32))) (param (var ys 2 (vec f32))) (param (var zs 3 (vec f32)))
              (param (var ax 4 (vec f32))) (param (var ay 5 (vec f32))) (param (var az 6 (vec f32)))
              (param (var n 7 i32)))
      (locals)
      (body (let {tid} (add (intr (Gpu) thread_idx_x) (mul (intr (Gpu) block_idx_x) (intr (Gpu) block_dim_x)))
        (if (lt {tid} (var n 7 i32))
          (let {P} {mk(tid)}
          (letmut {fx} (f32 0.0) (letmut {fy} (f32 0.0) (letmut {fz} (f32 0.0)
          (let {iv} {tid}
           (seq
            (for {jv} (i32 0) (sub (var n 7 i32) (i32 1)) upto
              (if (ne {jv} {iv})
                (let {Q} {mk(jv)}
                (let {dx} (sub (field {Q} x) (field {P} x))
                (let {dy} (sub (field {Q} y) (field {P} y))
                (let {dz} (sub (field {Q} z) (field {P} z))
                (let {dist2} (add (add (add (mul {dx} {dx}) (mul {dy} {dy})) (mul {dz} {dz})) (f32 1e-9))
                (let {inv} (div (f32 1.0) (mul (intr (Float32) sqrt {dist2}) {dist2}))
                  (seq (assign (lvar {fx}) (add {fx} (mul {dx} {inv})))
                       (assign (lvar {fy}) (add {fy} (mul {dy} {inv})))
                       (assign (lvar {fz}) (add {fz} (mul {dz} {inv}))))))))))))
            (assign (lelem ax {tid}) {fx}) (assign (lelem ay {tid}) {fy}) (assign (lelem az {tid}) {fz}))))))))))
      (types (particle (x f32) (y f32) (z f32)))
      (funcs (func make_p (params (var x 30 f32) (var y 31 f32) (var z 32 f32)) {part}
               (return (record particle (x (var x 30 f32)) (y (var y 31 f32)) (z (var z 32 f32))))))
      (native_fn true))
"""


KERNELS = {
    "stream_triad": stream_triad, "vector_add": vector_add, "vector_copy": vector_copy,
    "matrix_mul": matrix_mul, "matrix_mul_tiled": matrix_mul_tiled,
    "reduction": lambda: tree(False), "dot_product": lambda: tree(True),
    "transpose_naive": transpose_naive, "gather": gather, "mandelbrot": mandelbrot,
    "reduction_max": reduction_max, "transpose_tiled": transpose_tiled, "scatter": scatter,
    "radix_sort_histogram": radix_sort_histogram, "radix_sort_scatter": radix_sort_scatter,
}


