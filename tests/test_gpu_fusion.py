"""Fused kernels on the device: what the fusion pass writes goes through generate_source and
run_source like any other IR, and computes what the unfused launches compute (bit-exact for
the integer pipelines of sarek/tests/e2e/test_fusion_api.ml; to rounding for floats)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TID = "(intr (Gpu) thread_idx_x)"
GID = "(intr (Std) global_thread_id)"


def i32(n): return f"(i32 {n})"
def op(o, a, b): return f"({o} {a} {b})"
def read(arr, idx): return f"(read {arr} {idx})"
def store(arr, idx, e): return f"(assign (lelem {arr} {idx}) {e})"


def kernel(name, params, body, locals_=""):
    ps = " ".join(f"(param (var {n} {i + 1} {t}))" for i, (n, t) in enumerate(params))
    return f"(kernel {name} (params {ps}) (locals{locals_}) (body {body}) (native_fn false))"


def launch(hip, ir, name, n_threads, args, block=256):
    src = hip.generate_source(ir, block=(block, 1, 1))
    hip.run_source(src, name, (block, 1, 1), (n_threads // block, 1, 1), args)


@pytest.fixture
def env():
    import torch
    from spoc_amd import fusion, hip
    return torch, hip, fusion


def test_three_stage_pipeline_matches_three_launches(env):
    torch, hip, F = env
    n = 1 << 16
    vec = "(vec i32)"
    s1 = kernel("stage1", [("a", vec), ("input", vec)], store("a", GID, op("mul", read("input", GID), i32(2))))
    s2 = kernel("stage2", [("b", vec), ("a", vec)], store("b", GID, op("add", read("a", GID), i32(1))))
    s3 = kernel("stage3", [("output", vec), ("b", vec)], store("output", GID, op("mul", read("b", GID), i32(3))))
    fused, eliminated = F.fuse_pipeline([s1, s2, s3])
    assert eliminated == ["b", "a"]
    inp = torch.randint(-2**20, 2**20, (n,), dtype=torch.int32, device="cuda")
    a, b, out, out_fused = (torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(4))
    launch(hip, s1, "stage1", n, [a, inp])
    launch(hip, s2, "stage2", n, [b, a])
    launch(hip, s3, "stage3", n, [out, b])
    launch(hip, fused, "stage3_fused", n, [out_fused, inp])      # parameters: output, then input
    torch.cuda.synchronize()
    assert torch.equal(out, out_fused)
    assert torch.equal(out, (inp * 2 + 1) * 3)
    auto, eliminated, skipped = F.auto_fuse_pipeline([s1, s2, s3])
    assert sorted(eliminated) == ["a", "b"] and skipped == []
    out_auto = torch.zeros_like(out)
    launch(hip, auto, "stage3_fused", n, [out_auto, inp])
    torch.cuda.synchronize()
    assert torch.equal(out, out_auto)


def test_float_map_into_map(env):
    torch, hip, F = env
    n = 1 << 18
    vec = "(vec f32)"
    triad = kernel("triad", [("a", vec), ("b", vec), ("c", vec), ("s", "f32")],
                   store("a", GID, op("add", read("b", GID), op("mul", read("c", GID), "(var s 4 f32)"))))
    scale = kernel("scale", [("out", vec), ("a", vec)],
                   store("out", GID, op("add", op("mul", read("a", GID), "(f32 0.5)"), "(f32 1.0)")))
    assert F.should_fuse(triad, scale, "a").decision == F.Fuse
    fused = F.try_fuse(triad, scale, "a")
    b = torch.rand(n, device="cuda")
    c = torch.rand(n, device="cuda")
    a, out, out_fused = (torch.zeros(n, device="cuda") for _ in range(3))
    launch(hip, triad, "triad", n, [a, b, c, ("f32", 3.0)])
    launch(hip, scale, "scale", n, [out, a])
    launch(hip, fused, "scale_fused", n, [out_fused, b, c, ("f32", 3.0)])   # out, then b, c, s
    torch.cuda.synchronize()
    # same operations on the same f32 values; the compiler may contract differently across
    # the former kernel boundary, hence one ulp of slack
    assert torch.allclose(out, out_fused, rtol=2e-7, atol=0)
    assert torch.allclose(out_fused.double(), (b.double() + 3.0 * c.double()) * 0.5 + 1.0, rtol=1e-6)
    # a consumer that reads the element twice is a stencil of offset 0 to the analysis
    # (Sarek_fusion.ml:301-320): the element-wise rewrite refuses it, the stencil rewrite takes it
    square = kernel("square", [("out", vec), ("a", vec)], store("out", GID, op("mul", read("a", GID), read("a", GID))))
    assert not F.can_fuse(triad, square, "a") and F.try_fuse(triad, square, "a") is None
    fused2 = F.try_fuse_all(triad, square, "a")
    launch(hip, square, "square", n, [out, a])
    launch(hip, fused2, "square_stencil_fused", n, [out_fused, b, c, ("f32", 3.0)])
    torch.cuda.synchronize()
    assert torch.allclose(out, out_fused, rtol=2e-7, atol=0)


def test_stencil_consumer(env):
    torch, hip, F = env
    n = 1 << 14
    vec = "(vec i32)"
    prod = kernel("producer", [("temp", vec), ("input", vec)],
                  store("temp", GID, op("mul", read("input", GID), i32(2))))
    inside = op("and", op("ge", GID, i32(1)), op("lt", GID, i32(n - 1)))
    cons = kernel("consumer", [("output", vec), ("temp", vec)],
                  f"(if {inside} " + store("output", GID, op("add", read("temp", op("sub", GID, i32(1))),
                                                             read("temp", op("add", GID, i32(1))))) + ")")
    assert F.should_fuse(prod, cons, "temp").decision == F.MaybeFuse
    fused = F.fuse_stencil(prod, cons, "temp")
    inp = torch.randint(-1000, 1000, (n,), dtype=torch.int32, device="cuda")
    temp, out, out_fused = (torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(3))
    launch(hip, prod, "producer", n, [temp, inp])
    launch(hip, cons, "consumer", n, [out, temp])
    launch(hip, fused, "consumer_stencil_fused", n, [out_fused, inp])
    torch.cuda.synchronize()
    assert torch.equal(out, out_fused)
    expect = torch.zeros_like(out)
    expect[1:-1] = 2 * inp[:-2] + 2 * inp[2:]
    assert torch.equal(out, expect)


def test_map_into_serial_reduction_runs_as_written(env):
    """The reduction rewrite keeps the producer's own index (Sarek_fusion.ml:693-699), so each
    thread of the fused kernel folds ITS element `count` times; that is what must come out."""
    torch, hip, F = env
    count, threads = 100, 256
    vec = "(vec i32)"
    m = kernel("map", [("temp", vec), ("input", vec)], store("temp", TID, op("mul", read("input", TID), i32(2))))
    acc, i = "(var sum 7 i32 mut)", "(var i 8 i32 mut)"
    loop = f"(for {i} {i32(0)} {i32(count - 1)} upto (assign (lvar {acc}) (add {acc} {read('temp', i)})))"
    body = f"(seq (assign (lvar {acc}) {i32(0)}) {loop} {store('out', TID, acc)})"
    r = kernel("reduce", [("out", vec), ("temp", vec)], body, locals_=f" (local {acc})")
    assert F.can_fuse_reduction(m, r, "temp")
    fused = F.try_fuse_all(m, r, "temp")
    inp = torch.randint(-1000, 1000, (threads,), dtype=torch.int32, device="cuda")
    out = torch.zeros(threads, dtype=torch.int32, device="cuda")
    launch(hip, fused, "reduce_fused", threads, [out, inp])
    torch.cuda.synchronize()
    assert torch.equal(out, inp * 2 * count)
    # the unfused pair, for contrast: every thread sums temp[0..count-1]
    temp = torch.zeros(threads, dtype=torch.int32, device="cuda")
    out2 = torch.zeros_like(out)
    launch(hip, m, "map", threads, [temp, inp])
    launch(hip, r, "reduce", threads, [out2, temp])
    torch.cuda.synchronize()
    assert torch.equal(out2, torch.full_like(out2, int((inp[:count] * 2).sum())))


@pytest.mark.parametrize("seed", range(24))
def test_seeded_integer_pipelines_fused_and_unfused(env, seed):
    """Pipelines of two to four element-wise int32 stages with seeded expressions (the intermediate read once or
    several times, a second input vector or a scalar here and there, some of them shared by name between stages), fused by fuse_pipeline and by
    auto_fuse_pipeline: the fused kernel's output is the last stage's after the launches one by one, element for
    element (Int32 arithmetic wraps on both sides).  The fused kernel's arguments are given in the order of its own
    parameter list."""
    import random
    import re
    torch, hip, F = env
    rng = random.Random(31000 + seed)
    n, vec = 4096, "(vec i32)"
    tensors = {"input": torch.randint(-2**20, 2**20, (n,), dtype=torch.int32, device="cuda")}
    scalars = {}

    def expr(depth, leaves):
        if depth == 0:
            return rng.choice(leaves)
        a, b = expr(depth - 1, leaves), expr(depth - 1, leaves)
        pick = rng.randint(0, 5)
        if pick == 0:
            return op(rng.choice(["add", "sub", "mul"]), a, b)
        if pick == 1:
            return op(rng.choice(["bitand", "bitor", "bitxor"]), a, b)
        if pick == 2:
            return op("shl", op("bitand", a, i32(1023)), i32(rng.randint(0, 5)))
        if pick == 3:
            return f"(neg {a})"
        if pick == 4:
            return f"(if (lt {a} {b}) {b} {a})"
        return op("add", op("mul", a, i32(1103515245)), i32(12345))

    stages, prev = [], "input"
    for k in range(rng.randint(2, 4)):
        out = f"v{k}"
        tensors[out] = torch.zeros(n, dtype=torch.int32, device="cuda")
        params, leaves = [(out, vec), (prev, vec)], [read(prev, GID), read(prev, GID), i32(rng.randint(-9, 9)), GID]
        if rng.random() < 0.5:
            extra = rng.choice([f"e{k}", "e"])                  # `e` may belong to several stages: one argument by name
            if extra not in tensors:
                tensors[extra] = torch.randint(-1000, 1000, (n,), dtype=torch.int32, device="cuda")
            params.append((extra, vec))
            leaves.append(read(extra, GID))
        if rng.random() < 0.5:
            s = rng.choice([f"s{k}", "k"])                      # likewise (Sarek_fusion.ml:502-527 merges parameters by name)
            scalars.setdefault(s, rng.randint(-50, 50))
            params.append((s, "i32"))
            leaves.append(f"(var {s} {len(params)} i32)")
        stages.append((f"stage{k}", params, kernel(f"stage{k}", params, store(out, GID, expr(rng.randint(1, 3), leaves)))))
        prev = out

    def arguments(ir):
        head = ir[ir.index("(params"):ir.index("(locals")]
        names = re.findall(r"\(param \(var ([A-Za-z0-9_]+) ", head)
        return [tensors[m] if m in tensors else ("i32", scalars[m]) for m in names]

    for name, params, ir in stages:
        launch(hip, ir, name, n, arguments(ir))
    torch.cuda.synchronize()
    want = tensors[prev].clone()
    last = stages[-1][0]
    for fused_ir in (F.fuse_pipeline([ir for _, _, ir in stages])[0], F.auto_fuse_pipeline([ir for _, _, ir in stages])[0]):
        tensors[prev].zero_()
        fused_name = re.search(r"\(kernel ([A-Za-z0-9_]+)", fused_ir).group(1)
        assert fused_name == last + "_fused" or fused_name == last
        launch(hip, fused_ir, fused_name, n, arguments(fused_ir))
        torch.cuda.synchronize()
        assert torch.equal(tensors[prev], want), (seed, fused_name)
