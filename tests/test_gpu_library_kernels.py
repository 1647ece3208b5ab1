"""The headline kernels through the plugin path.

16-bit GEMMs, the fused GEMM epilogue and triad + sum have no kernel in the reference's suite; a caller
reaches them the way sarek/tests/e2e/test_external_kernel.ml:46-62 runs its own text, Execute.run_source
with the source the backend hands out (`library_kernel`).  Each test runs the text twice: with
specialisation on (the hand-written kernel must be the one that ran: last_run_path names its tag) and off
(the text itself, JIT-compiled), and checks both against the oracle and against each other.

The pair `stream triad, block-256 sum` of the reference's benches (bench_stream_triad.ml:22-32,
bench_reduction.ml:62-96) goes through Execute.run_pipeline from the two kernels' IR.

Bars: triad `a` bit-exact; sums and block sums 1e-5 relative; 16-bit GEMM 2e-2 relative to max|C|
(observed < 1e-4); f32 GEMM 1e-4 * sqrt(K)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

IR_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ir")


def load_ir(name):
    return open(os.path.join(IR_DIR, name + ".ir")).read()


@pytest.fixture()
def sarek(hip, torch_cuda):
    from spoc_amd import sarek as s
    s.Device.init()
    yield s
    hip.check(hip.lib.sarek_hip_set_specialisation(1))


def bits16(oracle, x, bf16):
    """f32 values that are exactly representable in the 16-bit format -> their bit patterns."""
    if bf16:
        return (oracle.round_bf16(x).view(np.uint32) >> 16).astype(np.uint16)
    return oracle.round_f16(x).astype(np.float16).view(np.uint16)


def custom16(sarek, bits):
    v = sarek.Vector.create_custom(2, bits.size)
    v.host.view(np.uint16)[:] = bits.reshape(-1)
    return v


def both_ways(hip, run):
    """run() with the hand kernels on, then off; returns [(path, result), (path, result)]."""
    out = []
    for on in (1, 0):
        hip.check(hip.lib.sarek_hip_set_specialisation(on))
        try:
            out.append(run())
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
    return out


def test_library_kernel_listing(hip):
    assert hip.library_kernel_names() == ["gemm_bf16", "gemm_f16", "gemm_f16_bias_relu_rowsum", "triad_sum_f32"]
    for name in hip.library_kernel_names():
        src, entry = hip.library_kernel(name)
        assert src.startswith("// sarek-hip-specialise: " + name + "\n") and f"void {entry}(" in src


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (300, 136, 200), (257, 129, 65), (512, 768, 256)])
def test_gemm16_through_run_source(hip, oracle, sarek, bf16, m, n, k):
    E, V = sarek.Execute, sarek.Vector
    rng = np.random.default_rng(m * 131 + n * 7 + k)
    rnd = oracle.round_bf16 if bf16 else oracle.round_f16
    a = rnd(rng.normal(0, 0.02, (m, k)).astype(np.float32))
    b = rnd(rng.normal(0, 0.02, (k, n)).astype(np.float32))
    ref = oracle.gemm(a, b)
    name = "gemm_bf16" if bf16 else "gemm_f16"
    src, entry = E.library_kernel(name)

    def run():
        va, vb = custom16(sarek, bits16(oracle, a, bf16)), custom16(sarek, bits16(oracle, b, bf16))
        vc = V.create(V.float32, m * n)
        vc.host[:] = np.nan
        path = E.run_source(src, entry, (16, 16, 1), ((n + 15) // 16, (m + 15) // 16, 1),
                            [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(m), E.Int32(n), E.Int32(k)])
        return path, vc.to_array().reshape(m, n).copy()

    (p_hand, c_hand), (p_jit, c_jit) = both_ways(hip, run)
    assert p_hand == name and p_jit == "jit"
    scale = np.abs(ref).max()
    assert np.array_equal(c_jit, ref)                      # the text restates the oracle's arithmetic
    assert np.abs(c_hand - ref).max() <= 2e-2 * scale
    assert np.abs(c_hand - ref).max() <= 1e-4 * scale      # observed: f32 accumulation error only


def test_gemm16_run_source_geometry_that_does_not_cover_c_is_left_to_the_text(hip, oracle, sarek):
    E, V = sarek.Execute, sarek.Vector
    m = n = k = 64
    a = oracle.round_bf16(np.full((m, k), 0.5, np.float32))
    b = oracle.round_bf16(np.full((k, n), 0.25, np.float32))
    src, entry = E.library_kernel("gemm_bf16")
    va, vb = custom16(sarek, bits16(oracle, a, True)), custom16(sarek, bits16(oracle, b, True))
    vc = V.create(V.float32, m * n)
    vc.host[:] = -1.0
    # 32 x 32 threads: only the top-left quarter of C is computed, by the text itself
    assert E.run_source(src, entry, (16, 16, 1), (2, 2, 1),
                        [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(m), E.Int32(n), E.Int32(k)]) == "jit"
    c = vc.to_array().reshape(m, n)
    assert np.all(c[:32, :32] == 8.0) and np.all(c[32:, :] == -1.0) and np.all(c[:, 32:] == -1.0)
    # the same arguments under a launch that covers C go to the MFMA kernel
    assert E.run_source(src, entry, (16, 16, 1), (4, 4, 1),
                        [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(m), E.Int32(n), E.Int32(k)]) == "gemm_bf16"
    assert np.all(vc.to_array() == 8.0)
    # C laid over A (raw device ranges, as the plugin-level run_source sees them): a race in the text,
    # never handed to the MFMA kernel
    torch = __import__("torch")
    raw = torch.zeros(4 * m * n, dtype=torch.uint8, device="cuda")
    a16, c32 = raw[:2 * m * k].view(torch.int16), raw[:4 * m * n].view(torch.float32)
    b16 = torch.zeros(k * n, dtype=torch.int16, device="cuda")
    assert hip.run_source(src, entry, (16, 16, 1), (4, 4, 1),
                          [a16, b16, c32, ("i32", m), ("i32", n), ("i32", k)]) == "jit"


def test_a_library_tag_on_somebody_elses_text_is_not_honoured(hip, oracle, sarek):
    """The hand kernel stands in for the library's own text only: a text that merely starts with the same tag
    line is compiled and run as it is written."""
    E, V = sarek.Execute, sarek.Vector
    m = n = k = 32
    mine = ("// sarek-hip-specialise: gemm_bf16\n"
            'extern "C" __global__ void sarek_gemm_bf16(const unsigned short* a, int a_len, const unsigned short* b, '
            "int b_len, float* c, int c_len, int m, int n, int k) {\n"
            "  int col = threadIdx.x + blockIdx.x * blockDim.x, row = threadIdx.y + blockIdx.y * blockDim.y;\n"
            "  if (row < m && col < n) c[row * n + col] = 42.0f;\n}\n")
    va, vb = custom16(sarek, np.zeros(m * k, np.uint16)), custom16(sarek, np.zeros(k * n, np.uint16))
    vc = V.create(V.float32, m * n)
    path = E.run_source(mine, "sarek_gemm_bf16", (16, 16, 1), (2, 2, 1),
                        [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(m), E.Int32(n), E.Int32(k)])
    assert path == "jit" and np.all(vc.to_array() == 42.0)
    # the library's text with trailing whitespace added is no longer the library's text either
    src, entry = E.library_kernel("gemm_bf16")
    assert E.run_source(src + "\n", entry, (16, 16, 1), (2, 2, 1),
                        [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(m), E.Int32(n), E.Int32(k)]) == "jit"
    assert np.all(vc.to_array() == 0.0)


@pytest.mark.parametrize("m,n,k", [(127, 264, 128), (300, 136, 200), (4095 // 8, 1376, 512)])
def test_epilogue_through_run_source(hip, oracle, sarek, m, n, k):
    E, V = sarek.Execute, sarek.Vector
    rng = np.random.default_rng(m + n + k)
    a = oracle.round_f16(rng.normal(0, 0.02, (m, k)).astype(np.float32))
    b = oracle.round_f16(rng.normal(0, 0.02, (k, n)).astype(np.float32))
    bias = oracle.fill_uniform(n, seed=5, lo=-0.1, hi=0.1)
    y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias)
    src, entry = E.library_kernel("gemm_f16_bias_relu_rowsum")

    def run():
        va, vb = custom16(sarek, bits16(oracle, a, False)), custom16(sarek, bits16(oracle, b, False))
        vbias = V.of_array(bias)
        vy, vrs = V.create(V.float32, m * n), V.create(V.float32, m)
        vy.host[:] = np.nan
        vrs.host[:] = np.nan
        path = E.run_source(src, entry, (256, 1, 1), (min(m, 1024), 1, 1),
                            [E.Vec(va), E.Vec(vb), E.Vec(vbias), E.Vec(vy), E.Vec(vrs),
                             E.Int32(m), E.Int32(n), E.Int32(k)])
        return path, (vy.to_array().reshape(m, n).copy(), vrs.to_array().copy())

    (p_hand, (y_hand, rs_hand)), (p_jit, (y_jit, rs_jit)) = both_ways(hip, run)
    assert p_hand == "gemm_f16_bias_relu_rowsum" and p_jit == "jit"
    assert np.array_equal(y_jit, y_ref) and np.array_equal(rs_jit, rs_ref)
    assert np.abs(y_hand - y_ref).max() <= 1e-4 * np.abs(y_ref).max()
    assert (np.abs(rs_hand.astype(np.float64) - rs_ref) <= 1e-5 * np.abs(rs_ref)).all()   # row by row
    assert (y_hand >= 0).all()


@pytest.mark.parametrize("n", [1, 3, 255, 4099, 100003, (1 << 20) + 5])
def test_triad_sum_through_run_source(hip, oracle, sarek, n):
    E, V = sarek.Execute, sarek.Vector
    b = oracle.fill_uniform(n, seed=0xB)
    c = oracle.fill_uniform(n, seed=0xC)
    a_ref, _, sum_ref = oracle.triad_sum(b, c, 3.0)
    src, entry = E.library_kernel("triad_sum_f32")

    def run():
        va, vb, vc = V.create(V.float32, n), V.of_array(b), V.of_array(c)
        vs = V.create(V.float64, 1)
        va.host[:] = np.nan
        vs.host[:] = np.nan
        path = E.run_source(src, entry, (256, 1, 1), (1, 1, 1),
                            [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Vec(vs), E.Float32(3.0), E.Int32(n)])
        return path, (va.to_array().copy(), float(vs.to_array()[0]))

    (p_hand, (a_hand, s_hand)), (p_jit, (a_jit, s_jit)) = both_ways(hip, run)
    assert p_hand == "triad_sum_f32" and p_jit == "jit"
    assert np.array_equal(a_hand, a_ref) and np.array_equal(a_jit, a_ref)
    assert abs(s_hand - sum_ref) <= 1e-5 * abs(sum_ref)
    assert abs(s_jit - sum_ref) <= 1e-5 * abs(sum_ref)


def test_triad_sum_text_with_more_than_one_workgroup_is_not_taken_over(hip, oracle, sarek):
    """The text is written for one workgroup; with two, both write sum[0]: whatever that gives is the
    text's own business, the hand kernel does not step in."""
    E, V = sarek.Execute, sarek.Vector
    n = 1000
    src, entry = E.library_kernel("triad_sum_f32")
    va, vb, vc, vs = V.create(V.float32, n), V.of_array(np.ones(n, np.float32)), V.of_array(np.ones(n, np.float32)), \
        V.create(V.float64, 1)
    args = [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Vec(vs), E.Float32(3.0), E.Int32(n)]
    assert E.run_source(src, entry, (256, 1, 1), (2, 1, 1), args) == "jit"
    assert E.run_source(src, entry, (96, 1, 1), (1, 1, 1), args) == "jit"        # not a power of two
    assert E.run_source(src, entry, (64, 1, 1), (1, 1, 1), args) == "triad_sum_f32"
    assert float(vs.to_array()[0]) == 4.0 * n


# ---- the pair of reference kernels through the pipeline entry ---------------------------------------

def triad_then_sum(sarek, b, c, n, n_sum=None, sum_input=None):
    """(stages, vectors) of: stream triad over n, then the block-256 sum of its output."""
    E, V = sarek.Execute, sarek.Vector
    n_sum = n if n_sum is None else n_sum
    va, vb, vc = V.create(V.float32, n), V.of_array(b), V.of_array(c)
    vout = V.create(V.float32, (n_sum + 255) // 256)
    va.host[:] = np.nan
    vout.host[:] = np.nan
    stages = [
        (load_ir("stream_triad"), [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Float32(3.0), E.Int32(n)],
         (256, 1, 1), ((n + 255) // 256, 1, 1)),
        (load_ir("reduction"), [E.Vec(sum_input or va), E.Vec(vout), E.Int32(n_sum)],
         (256, 1, 1), ((n_sum + 255) // 256, 1, 1)),
    ]
    return stages, (va, vb, vc, vout)


@pytest.mark.parametrize("n", [1, 5, 255, 256, 257, 4096, 4099, 65537, 1000003, (1 << 22) + 1])
def test_triad_then_block_sum_pipeline_is_one_launch(hip, oracle, sarek, n):
    E = sarek.Execute
    b = oracle.fill_uniform(n, seed=0xB)
    c = oracle.fill_uniform(n, seed=0xC)
    a_ref, partials_ref, sum_ref = oracle.triad_sum(b, c, 3.0)

    def run():
        stages, (va, _, _, vout) = triad_then_sum(sarek, b, c, n)
        path, launches = E.run_pipeline(stages)
        return (path, launches), (va.to_array().copy(), vout.to_array().copy())

    ((p_hand, l_hand), (a_hand, o_hand)), ((p_jit, l_jit), (a_jit, o_jit)) = both_ways(hip, run)
    assert (p_hand, l_hand) == ("stream_triad_f32+reduce_sum_block256_f32", 1)
    assert (p_jit, l_jit) == ("jit;jit", 2)
    assert np.array_equal(a_hand, a_ref)
    assert len(partials_ref) == len(o_hand) == (n + 255) // 256
    tol = 1e-5 * np.abs(partials_ref).max()
    assert np.abs(o_hand - partials_ref).max() <= tol and np.abs(o_jit - partials_ref).max() <= tol
    # the fold the bench does on the host (bench_reduction.ml:154-160)
    assert abs(o_hand.astype(np.float64).sum() - sum_ref) <= 1e-5 * abs(sum_ref)
    # the same two kernels launched one by one by the hand kernels give the same bits
    stages, (va, _, _, vout) = triad_then_sum(sarek, b, c, n)
    assert E.run_vectors(*stages[0]) == "stream_triad_f32" and E.run_vectors(*stages[1]) == "reduce_sum_block256_f32"
    assert np.array_equal(va.to_array(), a_hand) and np.array_equal(vout.to_array(), o_hand)


@pytest.mark.parametrize("n", [1, 255, 257, 4099, 1000003])
def test_vector_add_then_block_sum_pipeline_is_one_launch(hip, oracle, sarek, n):
    """The other element-wise producer of the reference's benches in front of the block-256 sum
    (bench_vector_add.ml, bench_reduction.ml): c = a + b and the sums of c in one pass, the same bits as the two hand
    kernels one after the other, the generated pair within the sum's tolerance."""
    E, V = sarek.Execute, sarek.Vector
    a = oracle.fill_uniform(n, seed=0xA)
    b = oracle.fill_uniform(n, seed=0xB)
    c_ref, partials_ref, _ = oracle.triad_sum(a, b, 1.0)      # a + 1.0 * b rounded once is the f32 sum
    assert np.array_equal(c_ref, a + b)

    def stages_and_vectors():
        va, vb, vc = V.of_array(a), V.of_array(b), V.create(V.float32, n)
        vout = V.create(V.float32, (n + 255) // 256)
        vc.host[:] = np.nan
        vout.host[:] = np.nan
        grid = ((n + 255) // 256, 1, 1)
        return [(load_ir("vector_add"), [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(n)], (256, 1, 1), grid),
                (load_ir("reduction"), [E.Vec(vc), E.Vec(vout), E.Int32(n)], (256, 1, 1), grid)], (vc, vout)

    def run():
        stages, (vc, vout) = stages_and_vectors()
        return E.run_pipeline(stages), (vc.to_array().copy(), vout.to_array().copy())

    (hand, (c_hand, o_hand)), (jit, (c_jit, o_jit)) = both_ways(hip, run)
    assert hand == ("vector_add_f32+reduce_sum_block256_f32", 1) and jit == ("jit;jit", 2)
    assert np.array_equal(c_hand, c_ref) and np.array_equal(c_jit, c_ref)
    tol = 1e-5 * np.abs(partials_ref).max()
    assert np.abs(o_hand - partials_ref).max() <= tol and np.abs(o_jit - partials_ref).max() <= tol
    stages, (vc, vout) = stages_and_vectors()
    assert E.run_vectors(*stages[0]) == "vector_add_f32" and E.run_vectors(*stages[1]) == "reduce_sum_block256_f32"
    assert np.array_equal(vc.to_array(), c_hand) and np.array_equal(vout.to_array(), o_hand)


def test_pipeline_pairs_that_are_not_the_fused_operation_run_one_by_one(hip, oracle, sarek):
    E, V = sarek.Execute, sarek.Vector
    n = 70000
    b = oracle.fill_uniform(n, seed=1)
    c = oracle.fill_uniform(n, seed=2)
    # the sum reads another vector than the triad wrote
    other = V.of_array(oracle.fill_uniform(n, seed=3))
    stages, (va, _, _, vout) = triad_then_sum(sarek, b, c, n, sum_input=other)
    assert E.run_pipeline(stages) == ("stream_triad_f32;reduce_sum_block256_f32", 2)
    assert np.array_equal(va.to_array(), oracle.triad(b, c, 3.0))
    want = oracle.triad_sum(other.to_array() / 1.0, np.zeros(n, np.float32), 0.0)[1]
    assert np.abs(vout.to_array() - want).max() <= 1e-5 * np.abs(want).max()
    # the sum covers fewer elements than the triad
    stages, (va, _, _, vout) = triad_then_sum(sarek, b, c, n, n_sum=n - 300)
    assert E.run_pipeline(stages) == ("stream_triad_f32;reduce_sum_block256_f32", 2)
    # three stages: the pair is found wherever it sits; a stage alone runs alone
    stages, (va, vb, vc, vout) = triad_then_sum(sarek, b, c, n)
    vd = V.create(V.float32, n)
    copy = (load_ir("vector_copy"), [E.Vec(vb), E.Vec(vd), E.Int32(n)], (256, 1, 1), ((n + 255) // 256, 1, 1))
    assert E.run_pipeline([copy] + stages) == ("vector_copy_f32;stream_triad_f32+reduce_sum_block256_f32", 2)
    assert np.array_equal(vd.to_array(), b)
    assert E.run_pipeline([]) == ("none", 0)


def test_run_sources_at_the_plugin_boundary(hip, oracle, torch_cuda):
    """The sequence entry a plugin calls with raw buffers (what Hip_plugin would marshal from run_source_arg lists):
    generated triad and block-sum sources one after the other are one launch, anything else one launch each."""
    torch = torch_cuda
    n = 300007
    nb = (n + 255) // 256
    b = torch.from_numpy(oracle.fill_uniform(n, seed=0xB)).cuda()
    c = torch.from_numpy(oracle.fill_uniform(n, seed=0xC)).cuda()
    a = torch.full((n,), float("nan"), device="cuda")
    sums = torch.full((nb,), float("nan"), device="cuda")
    tri, red = hip.generate_source(load_ir("stream_triad")), hip.generate_source(load_ir("reduction"), block=(256, 1, 1))
    l0 = (tri, "sarek_kern", (256, 1, 1), (nb, 1, 1), [a, b, c, ("f32", 3.0), ("i32", n)])
    l1 = (red, "sarek_kern", (256, 1, 1), (nb, 1, 1), [a, sums, ("i32", n)])
    assert hip.run_sources([l0, l1]) == ("stream_triad_f32+reduce_sum_block256_f32", 1)
    torch.cuda.synchronize()
    a_ref, p_ref, _ = oracle.triad_sum(b.cpu().numpy(), c.cpu().numpy(), 3.0)
    assert np.array_equal(a.cpu().numpy(), a_ref)
    assert np.abs(sums.cpu().numpy() - p_ref).max() <= 1e-5 * np.abs(p_ref).max()
    fused = sums.clone()
    # the other order, and a single entry, run as they are
    sums.fill_(0)
    assert hip.run_sources([l1, l0]) == ("reduce_sum_block256_f32;stream_triad_f32", 2)
    assert hip.run_sources([l0]) == ("stream_triad_f32", 1)
    assert hip.run_sources([l1]) == ("reduce_sum_block256_f32", 1)
    torch.cuda.synchronize()
    assert torch.equal(sums, fused)
    assert hip.run_sources([]) == ("none", 0)
    # a failing entry reports how far the sequence got
    import ctypes as C
    arr = (hip.Launch * 2)()
    args, na = hip.make_args(l0[4])
    arr[0].source, arr[0].lang, arr[0].kernel_name = tri.encode(), hip.LANG_HIP, b"sarek_kern"
    arr[0].block, arr[0].grid, arr[0].args, arr[0].n_args = (C.c_int * 3)(256, 1, 1), (C.c_int * 3)(nb, 1, 1), args, na
    arr[1].source, arr[1].lang, arr[1].kernel_name = b"this is not HIP", hip.LANG_HIP, b"nope"
    arr[1].block, arr[1].grid, arr[1].args, arr[1].n_args = (C.c_int * 3)(1, 1, 1), (C.c_int * 3)(1, 1, 1), args, 0
    made, done = C.c_int(-1), C.c_int(-1)
    assert hip.lib.sarek_hip_run_sources(arr, 2, C.byref(made), C.byref(done)) != 0
    assert (made.value, done.value) == (1, 1)


def test_fused_pair_kernel_at_full_size_properties(hip, torch_cuda):
    """n = 2^28, the size of the bandwidth config: constants make every value exact, so the vector, every
    block sum and the folded total have closed forms."""
    torch = torch_cuda
    n = 1 << 28
    b = torch.full((n,), 0.25, device="cuda")
    c = torch.full((n,), 0.5, device="cuda")
    a, sums = hip.triad_block256_sum(b, c, 3.0)
    total = torch.zeros(1, dtype=torch.float64, device="cuda")
    hip.check(hip.lib.sarek_hip_fold_partials_f64(sums.data_ptr(), sums.numel(), total.data_ptr(), None))
    torch.cuda.synchronize()
    assert sums.numel() == n // 256
    assert bool((a == 1.75).all()) and bool((sums == 448.0).all())
    assert total.item() == 1.75 * n


@pytest.mark.parametrize("n", [256, 4097, 100003])
def test_fused_pair_keeps_the_sign_of_a_zero_sum(hip, torch_cuda, n):
    """Blocks whose 256 elements are all -0 sum to -0 in the block-256 kernel (-0 + -0 = -0); the fused kernel adds
    the scalar tail's share to every block and must not turn that into +0.  Bits, not values."""
    torch = torch_cuda
    b = torch.full((n,), -0.0, device="cuda")
    c = torch.full((n,), -0.0, device="cuda")
    for runs in (1, 0):
        hip.check(hip.lib.sarek_hip_set_tunable(b"triad.block_sum_runs", runs))
        try:
            a, sums = hip.triad_block256_sum(b, c, 3.0)
        finally:
            hip.check(hip.lib.sarek_hip_set_tunable(b"triad.block_sum_runs", 1))
        a2 = hip.triad(b, c, 3.0)
        s2 = torch.empty((n + 255) // 256, device="cuda")
        hip.check(hip.lib.sarek_hip_reduce_sum_block256_f32(a2.data_ptr(), s2.data_ptr(), n, None))
        torch.cuda.synchronize()
        assert bool(torch.signbit(a).all()) and torch.equal(a.view(torch.int32), a2.view(torch.int32))
        assert torch.equal(sums.view(torch.int32), s2.view(torch.int32)), runs
        assert bool(torch.signbit(s2[: n // 256]).all())          # the full blocks: -0; a padded last block: +0


@pytest.mark.parametrize("n", [1, 255, 1000, 4097, 65536 + 777, (1 << 20) + 3, 5_000_001])
def test_fused_pair_block_sum_layouts_agree(hip, oracle, torch_cuda, n):
    """The fused kernel's two layouts (a wave's four blocks neighbours, one 16-byte store; or a workgroup's width
    apart, four 4-byte stores) and the two hand kernels launched one after the other leave the same bits; block
    sums that do not start on 16 bytes take the second layout."""
    torch = torch_cuda
    b = torch.from_numpy(oracle.fill_uniform(n, seed=n)).cuda()
    c = torch.from_numpy(oracle.fill_uniform(n, seed=n + 1)).cuda()
    nb = (n + 255) // 256
    try:
        got = []
        for runs in (1, 0):
            hip.check(hip.lib.sarek_hip_set_tunable(b"triad.block_sum_runs", runs))
            a, sums = hip.triad_block256_sum(b, c, 3.0)
            torch.cuda.synchronize()
            got.append((a.clone(), sums.clone()))
    finally:
        hip.check(hip.lib.sarek_hip_set_tunable(b"triad.block_sum_runs", 1))
    assert torch.equal(got[0][0], got[1][0]) and torch.equal(got[0][1], got[1][1])
    a_ref, p_ref, _ = oracle.triad_sum(b.cpu().numpy(), c.cpu().numpy(), 3.0)
    assert np.array_equal(got[0][0].cpu().numpy(), a_ref)
    assert np.abs(got[0][1].cpu().numpy() - p_ref).max() <= 1e-5 * np.abs(p_ref).max()
    # the triad kernel, then the block-256 sum kernel on its output
    a2 = hip.triad(b, c, 3.0)
    s2 = torch.empty(nb, device="cuda")
    hip.check(hip.lib.sarek_hip_reduce_sum_block256_f32(a2.data_ptr(), s2.data_ptr(), n, None))
    # block sums that start 4 bytes into an allocation
    pool = torch.full((nb + 1,), float("nan"), device="cuda")
    a3 = torch.empty_like(b)
    hip.check(hip.lib.sarek_hip_triad_block256_sum_f32(a3.data_ptr(), b.data_ptr(), c.data_ptr(), 3.0, n,
                                                       pool.data_ptr() + 4, None))
    torch.cuda.synchronize()
    assert torch.equal(a2, got[0][0]) and torch.equal(s2, got[0][1])
    assert torch.equal(a3, got[0][0]) and torch.equal(pool[1:], got[0][1]) and bool(torch.isnan(pool[0]))


@pytest.mark.parametrize("count", [0, 1, 1000, (1 << 17) - 1, 1 << 17, (1 << 17) + 3, (1 << 20) + 77, 3_000_001])
def test_fold_of_long_partial_vectors(hip, torch_cuda, count):
    """The device fold by one workgroup (short) and by 256 whose last one adds their sums up (from 2^17 partials
    on) against a float64 sum."""
    torch = torch_cuda
    rng = np.random.default_rng(count)
    x = rng.uniform(0, 500, count).astype(np.float32)
    d = torch.from_numpy(x).cuda()
    out = torch.full((1,), -1.0, dtype=torch.float64, device="cuda")
    hip.check(hip.lib.sarek_hip_fold_partials_f64(d.data_ptr() if count else None, count, out.data_ptr(), None))
    torch.cuda.synchronize()
    want = float(x.astype(np.float64).sum())
    assert abs(out.item() - want) <= 1e-12 * max(want, 1.0)
    if count > 8:   # unaligned start: the scalar path of every piece
        hip.check(hip.lib.sarek_hip_fold_partials_f64(d.data_ptr() + 4, count - 1, out.data_ptr(), None))
        torch.cuda.synchronize()
        want = float(x[1:].astype(np.float64).sum())
        assert abs(out.item() - want) <= 1e-12 * max(want, 1.0)


def test_long_folds_on_many_streams_do_not_meet(hip, torch_cuda):
    """Long folds queued on twenty streams at once (sixteen stages per device: the streams past the sixteenth fold
    with one workgroup), three rounds on the same streams so that every stage's ticket counter is used again:
    every sum is its own vector's, and a stream's repeated folds give the same bits."""
    torch = torch_cuda
    streams = [torch.cuda.Stream() for _ in range(20)]
    rng = np.random.default_rng(7)
    xs = [rng.uniform(0, 500, (1 << 17) + 1000 * i + 5).astype(np.float32) for i in range(len(streams))]
    ds = [torch.from_numpy(x).cuda() for x in xs]
    outs = torch.full((3, len(streams)), -1.0, dtype=torch.float64, device="cuda")
    torch.cuda.synchronize()
    for rnd in range(3):
        for i, st in enumerate(streams):
            hip.check(hip.lib.sarek_hip_fold_partials_f64(ds[i].data_ptr(), ds[i].numel(),
                                                          outs[rnd, i:].data_ptr(), st.cuda_stream))
    torch.cuda.synchronize()
    got = outs.cpu().numpy()
    for i, x in enumerate(xs):
        want = float(x.astype(np.float64).sum())
        assert abs(got[0, i] - want) <= 1e-12 * want, i
        assert got[0, i] == got[1, i] == got[2, i], i


def test_a_long_fold_recorded_into_a_graph_keeps_no_shared_state(hip, torch_cuda):
    """A fold of 2^20 partials recorded under stream capture takes a one-workgroup kernel (a graph may be replayed
    on any stream, next to anything, so it gets no stage of the library's): four replays with eager long folds on the
    same stream and new data between them, each checked against numpy's double sum of what the vector held then, and
    against the eager fold bit for bit -- the one workgroup adds piece by piece what the 256 add."""
    torch = torch_cuda
    n = 1 << 20
    rng = np.random.default_rng(11)
    x = torch.from_numpy(rng.uniform(0, 4, n).astype(np.float32)).cuda()
    out = torch.zeros(1, dtype=torch.float64, device="cuda")
    eager = torch.zeros(1, dtype=torch.float64, device="cuda")
    stream = torch.cuda.Stream()
    hip.check(hip.lib.sarek_hip_fold_partials_f64(x.data_ptr(), n, eager.data_ptr(), stream.cuda_stream))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        hip.check(hip.lib.sarek_hip_fold_partials_f64(x.data_ptr(), n, out.data_ptr(), torch.cuda.current_stream().cuda_stream))
    for replay in range(4):
        x.mul_(0.5 + 0.25 * replay)
        torch.cuda.synchronize()
        want = float(x.cpu().numpy().astype(np.float64).sum())
        hip.check(hip.lib.sarek_hip_fold_partials_f64(x.data_ptr(), n, eager.data_ptr(), stream.cuda_stream))
        graph.replay()
        torch.cuda.synchronize()
        assert abs(out.item() - want) <= 1e-12 * want, replay
        assert abs(eager.item() - want) <= 1e-12 * want, replay
        assert out.item() == eager.item(), replay


def test_tiled_matmul_through_run_vectors_at_1024(hip, oracle, sarek):
    """bench_matrix_mul_tiled's kernel from IR through Execute.run_vectors at the size of the first config."""
    E, V = sarek.Execute, sarek.Vector
    m = n = k = 1024
    a = oracle.fill_uniform(m * k, seed=0xA11CE, lo=-1, hi=1).reshape(m, k)
    b = oracle.fill_uniform(k * n, seed=0xB0B, lo=-1, hi=1).reshape(k, n)
    ref = oracle.gemm(a, b)

    def run():
        va, vb, vc = V.of_array(a), V.of_array(b), V.create(V.float32, m * n)
        vc.host[:] = np.nan
        path = E.run_vectors(load_ir("matrix_mul_tiled"),
                             [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(m), E.Int32(n), E.Int32(k)],
                             (16, 16, 1), (n // 16, m // 16, 1))
        return path, vc.to_array().reshape(m, n).copy()

    (p_hand, c_hand), (p_jit, c_jit) = both_ways(hip, run)
    assert p_hand == "matmul_tiled_f32" and p_jit == "jit"
    bound = 1e-4 * np.sqrt(k)           # ||A||inf ||B||inf <= 1
    assert np.abs(c_hand - ref).max() <= bound and np.abs(c_jit - ref).max() <= bound


def test_overlapping_outputs_are_left_to_the_generated_code(hip, oracle, sarek):
    """C over A in the tiled matmul and a shifted `a` over `b` in the triad are races in the generated kernels;
    the hand kernels assume distinct ranges, so such launches are not taken over."""
    torch = __import__("torch")
    m = n = k = 64
    buf = torch.zeros(2 * m * n, device="cuda")
    src = hip.generate_source(load_ir("matrix_mul_tiled"), block=(16, 16, 1))
    args = [buf[:m * k], buf[m * k:], buf[32:32 + m * n], ("i32", m), ("i32", n), ("i32", k)]
    assert hip.run_source(src, "sarek_kern", (16, 16, 1), (4, 4, 1), args, shared_mem=2048) == "jit"
    tri = hip.generate_source(load_ir("stream_triad"))
    v = torch.ones(4096 + 8, device="cuda")
    w = torch.ones(4096, device="cuda")
    shifted = [v[8:], v[:4096], w, ("f32", 3.0), ("i32", 4096)]
    assert hip.run_source(tri, "sarek_kern", (256, 1, 1), (16, 1, 1), shifted) == "jit"
    in_place = [v[:4096], v[:4096], w, ("f32", 3.0), ("i32", 4096)]
    v.fill_(1.0)
    assert hip.run_source(tri, "sarek_kern", (256, 1, 1), (16, 1, 1), in_place) == "stream_triad_f32"
    torch.cuda.synchronize()
    assert bool((v[:4096] == 4.0).all())


def test_hand_and_generated_triad_agree(hip, oracle, torch_cuda):
    """The hand triad rounds b + c*s once from double (the Native backend's rule), the generated kernel once from
    the fused multiply-add: the same f32 unless the double sum itself lands on a rounding boundary."""
    torch = torch_cuda
    n = 1 << 22
    b = torch.from_numpy(oracle.fill_uniform(n, seed=0xB)).cuda()
    c = torch.from_numpy(oracle.fill_uniform(n, seed=0xC)).cuda()
    src = hip.generate_source(load_ir("stream_triad"))
    outs = []
    for on in (1, 0):
        a = torch.empty(n, device="cuda")
        hip.check(hip.lib.sarek_hip_set_specialisation(on))
        try:
            path = hip.run_source(src, "sarek_kern", (256, 1, 1), (n // 256, 1, 1), [a, b, c, ("f32", 3.0), ("i32", n)])
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
        assert path == ("stream_triad_f32" if on else "jit")
        outs.append(a)
    torch.cuda.synchronize()
    hand, jit = outs
    differ = (hand != jit)
    assert int(differ.sum()) <= 2
    assert bool(((hand - jit).abs() <= torch.finfo(torch.float32).eps * hand.abs()).all())


@pytest.mark.parametrize("producer", ["stream_triad", "vector_add"])
@pytest.mark.parametrize("n", [1, 3, 255, 256, 257, 4099, 65537, 1000003])
def test_elementwise_then_block_max_is_one_launch(hip, oracle, torch_cuda, producer, n):
    """{stream triad, vector add} followed by the block-256 maximum of its output (bench_reduction_max.ml's tree, fill
    -1000000.0): one launch at the plugin boundary, the element-wise result and the maxima bit for bit those of the
    oracle's tree (elements past the end count as the fill), and of the generated pair."""
    from test_ir_lowering import reduction_max_ir
    torch = torch_cuda
    nb = (n + 255) // 256
    x = (oracle.fill_uniform(n, seed=0x9) * 2000 - 1000).astype(np.float32)
    y = (oracle.fill_uniform(n, seed=0xA) * 20 - 10).astype(np.float32)
    s = 3.0 if producer == "stream_triad" else 1.0
    a_ref = oracle.triad(x, y, s)
    dx, dy = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    red = hip.generate_source(reduction_max_ir(), block=(256, 1, 1))
    src = hip.generate_source(load_ir(producer))
    got = {}
    for specialise in (1, 0):
        a = torch.full((n,), float("nan"), device="cuda")
        mx = torch.full((nb,), float("nan"), device="cuda")
        if producer == "stream_triad":
            l0 = (src, "sarek_kern", (256, 1, 1), (nb, 1, 1), [a, dx, dy, ("f32", s), ("i32", n)])
        else:
            l0 = (src, "sarek_kern", (256, 1, 1), (nb, 1, 1), [dx, dy, a, ("i32", n)])
        l1 = (red, "sarek_kern", (256, 1, 1), (nb, 1, 1), [a, mx, ("i32", n)], 1024)
        hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
        try:
            got[specialise] = hip.run_sources([l0, l1]), a.cpu().numpy(), mx.cpu().numpy()
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
    tag = {"stream_triad": "stream_triad_f32", "vector_add": "vector_add_f32"}[producer]
    assert got[1][0] == (tag + "+reduce_max_block256_f32:c9742400", 1)
    assert got[0][0] == ("jit;jit", 2)
    for _, a, mx in got.values():
        assert np.array_equal(a, a_ref)
        assert np.array_equal(mx, oracle.reduce_max_block256(a_ref))


def test_fused_block_max_keeps_the_trees_order_for_nans_and_signed_zeros(hip, oracle, torch_cuda):
    """The tree compares with a strict ">", so which of two equal zeros or which side of a NaN survives depends on
    the order of the comparisons: the fused kernel's maxima are the bits of the stand-alone tree kernel's and of the
    oracle's, on inputs full of both."""
    torch = torch_cuda
    n = 256 * 37 + 129
    rng = np.random.default_rng(5)
    b = rng.choice(np.array([0.0, -0.0, 1.0, -1.0, np.nan, -7.5], np.float32), size=n)
    c = rng.choice(np.array([0.0, -0.0, 2.0, np.nan], np.float32), size=n)
    # whole blocks of zeros of both signs, and a block that is all NaN
    b[:256], c[:256] = rng.choice(np.array([0.0, -0.0], np.float32), size=256), 0.0
    b[256:512], c[256:512] = np.nan, 0.0
    db, dc = torch.from_numpy(b).cuda(), torch.from_numpy(c).cuda()
    for pad in (-1000000.0, 0.0, -0.0):
        a, mx = hip.triad_block256_max(db, dc, 1.0, pad)
        a_ref = oracle.triad(b, c, 1.0)
        assert np.array_equal(a.cpu().numpy().view(np.uint32), a_ref.view(np.uint32))
        want = oracle.reduce_max_block256(a_ref, pad=pad)
        alone = hip.reduce_max_block256(a, pad)
        assert np.array_equal(mx.cpu().numpy().view(np.uint32), want.view(np.uint32))
        assert np.array_equal(alone.cpu().numpy().view(np.uint32), want.view(np.uint32))
