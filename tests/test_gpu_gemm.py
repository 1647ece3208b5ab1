"""GPU parity: f32 / bf16 / fp16 GEMMs and the fused bias+ReLU+row-sum epilogue through
the C ABI against the CPU oracle (Native-backend semantics: double accumulation in
increasing k, one rounding at the store).

Tolerances (stated by the task for this path):
  f32 GEMM      max|err| <= 1e-4 * |A|_inf-elem * |B|_inf-elem * sqrt(K)
  bf16/fp16-in  <= 2e-2 relative, measured as max|err| / max|C_ref|
The 16-bit inputs are rounded once (RNE) and both sides consume the same rounded values,
so the observed error is f32-accumulation error only and is asserted much tighter."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def rowsums_ok(rs, rs_ref):
    """Row sums of non-negative values: every row within 1e-5 of its own reference (the bar for f32 reductions)."""
    rs, rs_ref = np.asarray(rs, np.float64), np.asarray(rs_ref, np.float64)
    return bool((np.abs(rs - rs_ref) <= 1e-5 * np.abs(rs_ref) + 1e-30).all())


def dev(torch, x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def f32_tol(a, b, k):
    return 1e-4 * float(np.abs(a).max()) * float(np.abs(b).max()) * np.sqrt(k)


F32_SHAPES = [(1, 1, 1), (16, 16, 16), (17, 33, 19), (128, 128, 128), (256, 256, 64),
              (257, 255, 100), (300, 520, 36), (512, 512, 512), (1024, 1024, 1024)]


@pytest.mark.parametrize("m,n,k", F32_SHAPES)
def test_gemm_f32_vs_oracle(hip, oracle, torch_cuda, m, n, k):
    torch = torch_cuda
    a = oracle.fill_uniform(m * k, seed=0xA11CE, lo=-1.0, hi=1.0).reshape(m, k)
    b = oracle.fill_uniform(k * n, seed=0xB0B, lo=-1.0, hi=1.0).reshape(k, n)
    c = hip.gemm_f32(dev(torch, a), dev(torch, b)).cpu().numpy()
    ref = oracle.gemm(a, b)
    err = float(np.abs(c - ref).max())
    assert err <= f32_tol(a, b, k), (err, f32_tol(a, b, k))
    assert err <= 4e-6 * np.sqrt(k) + 1e-6  # what f32 accumulation actually gives


def test_gemm_f32_reference_bench_inputs(hip, oracle, torch_cuda):
    """bench_matrix_mul_tiled.ml:109-112 inputs, its 1e-3 absolute check (:194)."""
    torch = torch_cuda
    m = n = k = 256
    a = ((np.arange(m * k) % 10) / 10.0).astype(np.float32).reshape(m, k)
    b = (((np.arange(k * n) + 1) % 10) / 10.0).astype(np.float32).reshape(k, n)
    c = hip.gemm_f32(dev(torch, a), dev(torch, b)).cpu().numpy()
    expected = ((np.arange(m * k) % 10) / 10.0).reshape(m, k) @ (((np.arange(k * n) + 1) % 10) / 10.0).reshape(k, n)
    assert np.abs(c - expected).max() <= 1e-3
    assert np.abs(c - oracle.gemm(a, b)).max() <= 1e-4


def test_gemm_f32_identity_and_selector(hip, torch_cuda):
    torch = torch_cuda
    torch.manual_seed(0)
    a = torch.rand(300, 260, device="cuda") * 2 - 1
    eye = torch.eye(260, device="cuda")
    assert torch.equal(hip.gemm_f32(a, eye), a)       # exact: one nonzero product per sum
    e = torch.zeros(260, 40, device="cuda")
    e[7, 3] = 1.0
    c = hip.gemm_f32(a, e)
    assert torch.equal(c[:, 3], a[:, 7]) and float(c.abs().sum()) == float(a[:, 7].abs().sum())


def test_gemm_f32_full_size_rows(hip, oracle, torch_cuda):
    """8192^3: sampled rows against the oracle + linearity."""
    torch = torch_cuda
    m = n = k = 8192
    a = oracle.fill_uniform(m * k, seed=0xA11CE, lo=-1.0, hi=1.0).reshape(m, k)
    b = oracle.fill_uniform(k * n, seed=0xB0B, lo=-1.0, hi=1.0).reshape(k, n)
    da, db = dev(torch, a), dev(torch, b)
    c = hip.gemm_f32(da, db)
    rows = np.array([0, 1, 255, 256, 4095, 4096, 8191], np.int32)
    ref = oracle.gemm_rows(a, b, rows)
    got = c[torch.from_numpy(rows).long().cuda()].cpu().numpy()
    err = float(np.abs(got - ref).max())
    assert err <= f32_tol(a, b, k), err
    c2 = hip.gemm_f32(da * 2.0, db)           # scaling by 2 is exact in binary
    assert torch.equal(c2, c * 2.0)


BF_SHAPES = [(8, 8, 8), (32, 32, 16), (256, 256, 64), (256, 256, 128), (264, 520, 72),
             (1, 8, 8), (100, 64, 200), (512, 768, 256), (1024, 1024, 1024)]


def normal16(oracle, shape, seed, kind):
    rng = np.random.default_rng(seed)
    x = rng.normal(0.0, 0.02, shape).astype(np.float32)
    return oracle.round_bf16(x) if kind == "bf16" else oracle.round_f16(x)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k", BF_SHAPES)
def test_gemm16_vs_oracle(hip, oracle, torch_cuda, kind, m, n, k):
    torch = torch_cuda
    a = normal16(oracle, (m, k), 0xA4, kind)
    b = normal16(oracle, (k, n), 0xB4, kind)
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    da, db = dev(torch, a).to(tdt), dev(torch, b).to(tdt)   # exact: values already representable
    assert torch.equal(da.float().cpu(), torch.from_numpy(a))
    fn = hip.gemm_bf16 if kind == "bf16" else hip.gemm_f16
    c = fn(da, db).cpu().numpy()
    ref = oracle.gemm(a, b)
    scale = float(np.abs(ref).max())
    rel = float(np.abs(c - ref).max()) / scale
    assert rel <= 2e-2, rel
    assert rel <= 1e-4, rel


@pytest.mark.parametrize("kind", ["bf16", "f16"])
def test_gemm16_unaligned_shapes_use_fallback(hip, oracle, torch_cuda, kind):
    torch = torch_cuda
    m, n, k = 37, 51, 29   # k below one LDS stage and not a multiple of 8
    assert hip.gemm16_tile(m, n, k) == 0
    a = normal16(oracle, (m, k), 1, kind)
    b = normal16(oracle, (k, n), 2, kind)
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    fn = hip.gemm_bf16 if kind == "bf16" else hip.gemm_f16
    c = fn(dev(torch, a).to(tdt), dev(torch, b).to(tdt)).cpu().numpy()
    ref = oracle.gemm(a, b)
    assert np.abs(c - ref).max() <= 1e-4 * np.abs(ref).max()


def test_gemm16_integer_inputs_exact(hip, torch_cuda):
    """Small integers: every product and partial sum is exact in f32, so any indexing or
    k-permutation mistake shows up as a wrong integer."""
    torch = torch_cuda
    torch.manual_seed(3)
    m, n, k = 320, 384, 192
    a = torch.randint(-3, 4, (m, k), device="cuda").float()
    b = torch.randint(-3, 4, (k, n), device="cuda").float()
    want = (a.double() @ b.double()).float()
    assert torch.equal(hip.gemm_bf16(a.bfloat16(), b.bfloat16()), want)
    assert torch.equal(hip.gemm_f16(a.half(), b.half()), want)
    assert torch.equal(hip.gemm_f32(a, b), want)


@pytest.mark.parametrize("m,n,k", [(64, 256, 64), (255, 512, 128), (300, 264, 72), (33, 40, 24)])
def test_epilogue_vs_oracle(hip, oracle, torch_cuda, m, n, k):
    torch = torch_cuda
    a = normal16(oracle, (m, k), 0xA5, "f16")
    b = normal16(oracle, (k, n), 0xB5, "f16")
    bias = oracle.fill_uniform(n, seed=0xB1A5, lo=-0.1, hi=0.1)
    y, rs = hip.gemm_f16_bias_relu_rowsum(dev(torch, a).half(), dev(torch, b).half(), dev(torch, bias))
    y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias)
    y = y.cpu().numpy()
    rs = rs.cpu().numpy()
    assert np.abs(y - y_ref).max() <= 2e-2 * np.abs(y_ref).max()
    assert np.abs(y - y_ref).max() <= 1e-5 * max(1.0, np.abs(y_ref).max())
    assert (y >= 0).all()
    assert rowsums_ok(rs, rs_ref)


def test_epilogue_full_size_config(hip, oracle, torch_cuda):
    """M=4095 (non tile multiple), N=11008, K=4096: sampled rows vs oracle, row sums vs Y."""
    torch = torch_cuda
    m, n, k = 4095, 11008, 4096
    rng = np.random.default_rng(0xC5)
    a = oracle.round_f16(rng.normal(0, 0.02, (m, k)).astype(np.float32))
    b = oracle.round_f16(rng.normal(0, 0.02, (k, n)).astype(np.float32))
    bias = oracle.fill_uniform(n, seed=0xB1A5, lo=-0.1, hi=0.1)
    y, rs = hip.gemm_f16_bias_relu_rowsum(dev(torch, a).half(), dev(torch, b).half(), dev(torch, bias))
    rows = np.array([0, 127, 128, 2047, 3968, 4094], np.int32)
    y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias, rows=rows)
    idx = torch.from_numpy(rows).long().cuda()
    got = y[idx].cpu().numpy()
    assert np.abs(got - y_ref).max() <= 2e-2 * np.abs(y_ref).max()
    assert rowsums_ok(rs[idx].cpu().numpy(), rs_ref)
    # size-independent: the fused row sums equal the row sums of the stored Y, row by row, and a second run's bits
    assert rowsums_ok(rs.cpu().numpy(), y.double().sum(dim=1).cpu().numpy())
    assert torch.equal(hip.gemm_f16_bias_relu_rowsum(dev(torch, a).half(), dev(torch, b).half(), dev(torch, bias))[1], rs)


def test_epilogue_row_sums_are_the_same_bits_on_every_run(hip, oracle, torch_cuda):
    """The tiles' shares of a row are added in tile order, in double, with one rounding -- not in the order the
    tiles finish: five runs of a shape with 43 tile columns give the same bits, on the main stream and on another;
    both tile sizes, an odd N (whose last column comes from a kernel of its own) and the one-thread-per-element kernel
    each agree with themselves run to run and with the oracle row by row.  Under stream capture no plane block is
    handed out and the shares are added by atomicAdd: that path is checked against the oracle too."""
    torch = torch_cuda
    rng = np.random.default_rng(0xD7)
    for (m, n, k), tile in [((300, 11008, 128), 256), ((300, 11008, 128), 128), ((259, 1001, 192), 0), ((70, 200, 24), 0),
                            ((33, 130, 20), 0)]:
        a = oracle.round_f16(rng.normal(0, 0.02, (m, k)).astype(np.float32))
        b = oracle.round_f16(rng.normal(0, 0.02, (k, n)).astype(np.float32))
        bias = oracle.fill_uniform(n, seed=n, lo=-0.1, hi=0.1)
        da, db, dbias = dev(torch, a).half(), dev(torch, b).half(), dev(torch, bias)
        _, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias)
        hip.set_tunable("gemm16.tile", tile)
        try:
            runs = [hip.gemm_f16_bias_relu_rowsum(da, db, dbias)[1].clone() for _ in range(5)]
            side = side_stream(torch)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                runs.append(hip.gemm_f16_bias_relu_rowsum(da, db, dbias)[1].clone())
            side.synchronize()
        finally:
            hip.set_tunable("gemm16.tile", 0)
        torch.cuda.synchronize()
        for r in runs[1:]:
            assert torch.equal(r, runs[0]), (m, n, k, tile)
        assert rowsums_ok(runs[0].cpu().numpy(), rs_ref), (m, n, k, tile)
    # captured: atomics
    m, n, k = 300, 1024, 128
    a = oracle.round_f16(rng.normal(0, 0.02, (m, k)).astype(np.float32))
    b = oracle.round_f16(rng.normal(0, 0.02, (k, n)).astype(np.float32))
    bias = oracle.fill_uniform(n, seed=n, lo=-0.1, hi=0.1)
    da, db, dbias = dev(torch, a).half(), dev(torch, b).half(), dev(torch, bias)
    y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias)
    y, rs = torch.empty(m, n, device="cuda"), torch.empty(m, device="cuda")
    hip.gemm_f16_bias_relu_rowsum(da, db, dbias, out=y, rowsum=rs)    # warm: kernels loaded before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hip.gemm_f16_bias_relu_rowsum(da, db, dbias, out=y, rowsum=rs)
    for _ in range(3):
        rs.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert rowsums_ok(rs.cpu().numpy(), rs_ref)
        assert np.abs(y.cpu().numpy() - y_ref).max() <= 1e-4 * np.abs(y_ref).max()


def test_epilogue_row_sums_beyond_the_plane_block_are_added_by_atomics(hip, torch_cuda):
    """More row-sum shares than the per-stream block holds (rows x planes x 4 bytes > 64 MiB; here the
    one-thread-per-element kernel's plane per 64 columns on an 8192 x 131136 product with K = 20): the shares go to the
    zeroed vector by atomicAdd, in no fixed order -- every row within 1e-4 of the double sum of the stored row."""
    torch = torch_cuda
    m, n, k = 8192, 131136, 20
    assert m * ((n + 63) // 64) * 4 > 64 << 20
    g = torch.Generator(device="cuda")
    g.manual_seed(0xE9)
    a = (torch.randn(m, k, device="cuda", generator=g) * 0.2).half()
    b = (torch.randn(k, n, device="cuda", generator=g) * 0.2).half()
    bias = torch.rand(n, device="cuda", generator=g) * 0.2 - 0.1
    y, rs = hip.gemm_f16_bias_relu_rowsum(a, b, bias)
    sums = torch.sum(y, dim=1, dtype=torch.float64)
    assert bool((sums > 0).all()) and bool(((rs.double() - sums).abs() <= 1e-4 * sums).all())
    # sampled elements against the definition
    rows = torch.tensor([0, 4097, 8191], device="cuda")
    want = torch.relu(a[rows].double() @ b.double() + bias.double())
    assert bool(((y[rows].double() - want).abs() <= 1e-5 * want.abs().max()).all())


def test_gemm_bf16_full_size_rows(hip, oracle, torch_cuda):
    torch = torch_cuda
    m = n = k = 8192
    torch.manual_seed(0xA4)
    a = (torch.randn(m, k, device="cuda") * 0.02).bfloat16()
    b = (torch.randn(k, n, device="cuda") * 0.02).bfloat16()
    c = hip.gemm_bf16(a, b)
    rows = np.array([0, 255, 256, 5000, 8191], np.int32)
    ref = oracle.gemm_rows(a.float().cpu().numpy(), b.float().cpu().numpy(), rows)
    got = c[torch.from_numpy(rows).long().cuda()].cpu().numpy()
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
    # exact power-of-two scaling commutes with the kernel
    assert torch.equal(hip.gemm_bf16(a * 2, b), c * 2)


def test_the_product_library_refuses_the_measurement_knobs(hip, torch_cuda):
    """The knobs of the ablation studies (kernel variants that leave parts of the K loop out and compute wrong
    results on purpose, retired kernel shapes, the in-kernel clock probe) exist in the measurement build only:
    the product library answers each with "unsupported", also when it is asked through the environment, and a
    product computed afterwards is the one from before."""
    torch = torch_cuda
    assert hip.lib.sarek_hip_is_measurement_build() == 0
    m, n, k = 512, 768, 512
    torch.manual_seed(7)
    a = (torch.randn(m, k, device="cuda") * 0.1).bfloat16()
    b = (torch.randn(k, n, device="cuda") * 0.1).bfloat16()
    good = hip.gemm_bf16(a, b)
    for knob, value in (("gemm16.ablate", 1), ("gemm16.ablate", 8), ("gemm16.mfma", 32), ("gemm16.ring", 4),
                        ("gemm16.tj", 4), ("gemm16.waves", 4), ("gemm16.barriers", 1)):
        with pytest.raises(hip.SarekHipError) as e:
            hip.set_tunable(knob, value)
        assert e.value.status == hip.E_UNSUPPORTED and "measurement build" in e.value.message
    buf = torch.zeros(128, dtype=torch.int64, device="cuda")
    rate = C.c_int64(0)
    assert hip.lib.sarek_hip_set_clock_probe(C.c_void_p(buf.data_ptr()), 64, C.byref(rate)) == hip.E_UNSUPPORTED
    assert torch.equal(hip.gemm_bf16(a, b), good)
    torch.cuda.synchronize()
    assert int(buf.abs().sum().item()) == 0


def test_the_measurement_build_in_a_process_of_its_own():
    """libsarek_hip_measure.so, loaded by a fresh interpreter (a process holds one of the two libraries): it says what it
    is, takes the knobs, every variant runs within the operands' bounds, the 32 x 32 x 16 kernel's ring and wave
    shapes agree with the product's kernel, the clock probe records, and with the knobs back the default kernel
    gives the product's bits."""
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    env = dict(os.environ, SAREK_HIP_MEASURE_BUILD="1")
    r = subprocess.run([sys.executable, os.path.join(here, "measure_build_checks.py")], env=env, capture_output=True,
                       text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "measurement build ok" in r.stdout


def test_gemm_rejects_bad_arguments(hip, torch_cuda):
    torch = torch_cuda
    a = torch.zeros(4, 4, device="cuda")
    with pytest.raises(hip.SarekHipError) as e:
        hip.check(hip.lib.sarek_hip_gemm_f32(a.data_ptr(), a.data_ptr(), a.data_ptr(), 4, -1, 4, None))
    assert e.value.status == hip.E_INVALID_ARG


def test_shader_clock_sampler_reads_a_plausible_clock(hip, torch_cuda):
    """The sampling waves next to a GEMM: a clock between the idle and the peak engine clock, with nothing added to
    the GEMM's own kernels (the product library has no probe inside them)."""
    torch = torch_cuda
    m = n = k = 4096
    a = (torch.randn(m, k, device="cuda") * 0.02).to(torch.bfloat16)
    b = (torch.randn(k, n, device="cuda") * 0.02).to(torch.bfloat16)
    c = torch.empty(m, n, device="cuda")
    for _ in range(20):
        hip.gemm_bf16(a, b, out=c)
    torch.cuda.synchronize()
    sampler = hip.shader_clock_sampler()
    try:
        sampler.start(0.08)
        hip.gemm_bf16(a, b, out=c)
        mhz = sampler.mhz()
    finally:
        sampler.close()
    assert mhz is not None and 400 < mhz < 2600, mhz


@pytest.mark.parametrize("tile", [64, 128, 256])
@pytest.mark.parametrize("m,n,k", [(300, 520, 32), (257, 132, 96), (512, 768, 160), (70, 1028, 288)])
def test_gemm_f32_every_tile_shape(hip, oracle, torch_cuda, tile, m, n, k):
    """The three direct-to-LDS tile shapes on ragged M, N and on K values that end the ring
    at every position (K/32 = 1, 3, 5, 9 slabs against a ring of 4)."""
    a = oracle.fill_uniform(m * k, seed=m + tile, lo=-1, hi=1).reshape(m, k)
    b = oracle.fill_uniform(k * n, seed=n + tile, lo=-1, hi=1).reshape(k, n)
    hip.set_tunable("gemm_f32.tile", tile)
    try:
        c = hip.gemm_f32(dev(torch_cuda, a), dev(torch_cuda, b)).cpu().numpy()
    finally:
        hip.set_tunable("gemm_f32.tile", 0)
    assert np.abs(c - oracle.gemm(a, b)).max() <= f32_tol(a, b, k)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k", [(128, 128, 64), (1, 8, 64), (130, 136, 128), (300, 520, 192), (257, 264, 320),
                                   (512, 768, 448), (70, 1032, 1216), (640, 384, 768)])
def test_gemm16_both_tile_sizes(hip, oracle, torch_cuda, kind, m, n, k):
    """The 256 x 256 and the 128 x 128 workgroup tile of the 16 x 16 x 32 kernel, plain and with the fused epilogue,
    on ragged M and N and on K values that end the stage patterns (periods of 4 and 12 slabs) at different
    positions: each against the oracle, and the two against each other (same products, same k order per element:
    the plain results are the same bits)."""
    torch = torch_cuda
    a = normal16(oracle, (m, k), m + 11, kind)
    b = normal16(oracle, (k, n), n + 12, kind)
    bias = oracle.fill_uniform(n, seed=n + 1, lo=-0.1, hi=0.1)
    dt = torch.bfloat16 if kind == "bf16" else torch.float16
    da, db = dev(torch, a).to(dt), dev(torch, b).to(dt)
    ref = oracle.gemm(a, b)
    got = {}
    try:
        for tile in (128, 256):
            hip.set_tunable("gemm16.tile", tile)
            c = (hip.gemm_bf16 if kind == "bf16" else hip.gemm_f16)(da, db)
            assert hip.gemm16_tile(m, n, k) == tile
            c = c.cpu().numpy()
            assert np.abs(c - ref).max() / np.abs(ref).max() < 1e-4
            got[tile] = c
            if kind == "f16":
                y, rs = hip.gemm_f16_bias_relu_rowsum(da, db, dev(torch, bias))
                y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias)
                assert np.abs(y.cpu().numpy() - y_ref).max() <= 1e-4 * np.abs(y_ref).max()
                assert rowsums_ok(rs.cpu().numpy(), rs_ref)
    finally:
        hip.set_tunable("gemm16.tile", 0)
    assert np.array_equal(got[128], got[256])


def test_gemm16_tile_choice_by_shape(hip, torch_cuda):
    """Left to itself the launcher takes the small tile where the large one would leave CUs idle and the large one
    for products of several rounds; shapes the direct-to-LDS kernels do not take report 0."""
    for (m, n, k), want in [((1024, 1024, 64), 128), ((2048, 2048, 2048), 128), ((1024, 4096, 4096), 128),
                            ((4096, 2048, 8192), 128), ((3072, 3072, 3072), 256), ((4096, 4096, 4096), 256),
                            ((8192, 8192, 8192), 256), ((4095, 11008, 4096), 256), ((512, 512, 72), 128), ((4096, 4100, 4096), 256),
                            ((1000, 1001, 1000), 128), ((1000, 1001, 1001), 128), ((512, 512, 29), 0),
                            ((37, 51, 29), 0)]:
        assert hip.gemm16_tile(m, n, k) == want, (m, n, k)


_SIDE_STREAM = []


def side_stream(torch):
    """One second stream for the whole module: the library keeps a block of device memory per stream it has split a
    product on (16 streams at most), so the cases share theirs."""
    if not _SIDE_STREAM:
        _SIDE_STREAM.append(torch.cuda.Stream())
    return _SIDE_STREAM[0]


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k,splits", [(128, 128, 8192, 0), (256, 256, 4096, 0), (130, 136, 1024, 2),
                                          (300, 520, 448, 3), (1, 8, 4096, 16), (512, 384, 2048, 5),
                                          (777, 1000, 320, 2)])
def test_gemm16_split_k(hip, oracle, torch_cuda, kind, m, n, k, splits):
    """Products with few tiles and a long K are cut along K over several workgroups per tile and the partial tiles
    added in a fixed order: against the oracle, the same bits on every run and on another stream, and the count the
    library reports.  splits = 0 leaves the choice to the launcher (these two shapes split), n forces n pieces
    (piece sizes that are not equal included: 448 = 192 + 192 + 64)."""
    torch = torch_cuda
    a = normal16(oracle, (m, k), m + 21, kind)
    b = normal16(oracle, (k, n), n + 22, kind)
    dt = torch.bfloat16 if kind == "bf16" else torch.float16
    da, db = dev(torch, a).to(dt), dev(torch, b).to(dt)
    fn = hip.gemm_bf16 if kind == "bf16" else hip.gemm_f16
    ref = oracle.gemm(a, b)
    hip.set_tunable("gemm16.split_k", splits)
    try:
        reported = hip.gemm16_k_splits(m, n, k)
        assert reported >= 2 and (splits == 0 or reported <= splits)
        c1 = fn(da, db)
        c2 = fn(da, db)
        side = side_stream(torch)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            c3 = fn(da, db)
        side.synchronize()
        # an output that is not 16-byte aligned is computed unsplit
        odd = torch.empty(m * n + 1, device="cuda")[1:].view(m, n)
        fn(da, db, out=odd)
        hip.set_tunable("gemm16.split_k", 1)
        assert hip.gemm16_k_splits(m, n, k) == 1
        whole = fn(da, db)
    finally:
        hip.set_tunable("gemm16.split_k", 0)
    assert torch.equal(c1, c2) and torch.equal(c1, c3)
    assert torch.equal(odd, whole)
    for c in (c1, whole):
        assert np.abs(c.cpu().numpy() - ref).max() / np.abs(ref).max() < 1e-4
    assert (c1 - whole).abs().max().item() <= 1e-5 * float(np.abs(ref).max())


def test_gemm16_split_k_rule_and_epilogue(hip, oracle, torch_cuda):
    """The launcher splits only where it pays (few tiles, long K), never the fused epilogue, and never the large tile."""
    torch = torch_cuda
    for (m, n, k), want_split in [((256, 256, 8192), True), ((512, 512, 8192), True), ((128, 4096, 4096), True),
                                  ((1024, 1024, 1024), False), ((2048, 2048, 2048), False), ((512, 512, 512), False),
                                  ((8192, 8192, 8192), False), ((4096, 4096, 4096), False)]:
        assert (hip.gemm16_k_splits(m, n, k) > 1) == want_split, (m, n, k)
    m, n, k = 128, 256, 4096
    assert hip.gemm16_k_splits(m, n, k) > 1
    a = normal16(oracle, (m, k), 31, "f16")
    b = normal16(oracle, (k, n), 32, "f16")
    bias = oracle.fill_uniform(n, seed=33, lo=-0.1, hi=0.1)
    y, rs = hip.gemm_f16_bias_relu_rowsum(dev(torch, a).half(), dev(torch, b).half(), dev(torch, bias))
    y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias)
    assert np.abs(y.cpu().numpy() - y_ref).max() <= 1e-4 * np.abs(y_ref).max()
    assert rowsums_ok(rs.cpu().numpy(), rs_ref)


def test_gemm16_split_k_under_graph_capture(hip, torch_cuda):
    """A split-eligible product captured into a HIP graph on a stream that has no partial-plane block yet runs unsplit
    (nothing may be allocated under capture); every replay gives the eager result for the inputs of that moment."""
    torch = torch_cuda
    m, n, k = 256, 256, 4096
    assert hip.gemm16_k_splits(m, n, k) > 1
    a = (torch.randn(m, k, device="cuda") * 0.02).bfloat16()
    b = (torch.randn(k, n, device="cuda") * 0.02).bfloat16()
    out = torch.empty(m, n, device="cuda")
    hip.gemm_bf16(a, b, out=out)          # warm: kernels loaded before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hip.gemm_bf16(a, b, out=out)
    for seed in (1, 2, 3):
        torch.manual_seed(seed)
        a.copy_((torch.randn(m, k, device="cuda") * 0.02).bfloat16())
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        hip.set_tunable("gemm16.split_k", 1)
        try:
            want = hip.gemm_bf16(a, b)
        finally:
            hip.set_tunable("gemm16.split_k", 0)
        assert torch.equal(got, want), seed


RAGGED_SHAPES = [(1, 1, 8), (3, 5, 8), (37, 51, 24), (130, 137, 40), (256, 255, 64), (257, 1001, 1000),
                 (300, 262, 136), (512, 514, 4104), (777, 1003, 328), (64, 4100, 96), (1000, 3, 2056),
                 (130, 137, 65), (257, 1001, 1001), (300, 263, 75), (64, 65, 67), (512, 514, 4107), (33, 40, 127),
                 (33, 40, 129), (100, 64, 100)]


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k", RAGGED_SHAPES)
def test_gemm16_ragged_shapes_stay_on_the_mfma_kernels(hip, oracle, torch_cuda, kind, m, n, k):
    """Any N (odd ones included: rows of B and C then have no alignment at all), any K from one LDS stage (64) on
    and the multiples of 8 below it, operands that are only 2-byte aligned (where K reaches a stage): all run on the
    direct-to-LDS kernels, both tiles, K split or not: against the oracle; nothing is stored outside C; NaNs lying
    next to A and B in memory (what the transfers fetch past a row's or the matrix's end) do not reach the result."""
    torch = torch_cuda
    a = normal16(oracle, (m, k), m + 41, kind)
    b = normal16(oracle, (k, n), n + 42, kind)
    dt = torch.bfloat16 if kind == "bf16" else torch.float16
    fn = hip.gemm_bf16 if kind == "bf16" else hip.gemm_f16
    ref = oracle.gemm(a, b)
    # operands as views into NaN-filled buffers: 16-byte aligned below one stage of K, 2-byte aligned from there on
    off = 129 if k >= 64 else 128
    buf_a = torch.full((m * k + 256,), float("nan"), device="cuda").to(dt)
    buf_b = torch.full((k * n + 256,), float("nan"), device="cuda").to(dt)
    da, db = buf_a[off:off + m * k].view(m, k), buf_b[off:off + k * n].view(k, n)
    da.copy_(dev(torch, a).to(dt))
    db.copy_(dev(torch, b).to(dt))
    try:
        for tile, split in ((128, 1), (128, 0), (128, 3), (256, 1)):
            hip.set_tunable("gemm16.tile", tile)
            hip.set_tunable("gemm16.split_k", split)
            assert hip.gemm16_tile(m, n, k) == tile
            guard = torch.full((m * n + 64,), 7.0, device="cuda")
            c = guard[32:32 + m * n].view(m, n)
            fn(da, db, out=c)
            assert bool((guard[:32] == 7).all()) and bool((guard[32 + m * n:] == 7).all())
            got = c.cpu().numpy()
            assert np.isfinite(got).all()
            assert np.abs(got - ref).max() / np.abs(ref).max() < 1e-4, (tile, split)
    finally:
        hip.set_tunable("gemm16.tile", 0)
        hip.set_tunable("gemm16.split_k", 0)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_seeded_random_shapes_through_every_gemm_entry_point(hip, torch_cuda, seed):
    """150 seeded shapes per seed (dimensions at and next to 1, 8, 16, 32, 64, 128, 256, 512 and at random up to
    700 x 1100 x 900), an entry point (bf16, fp16, f32, fused epilogue), a tile choice and a K split drawn for each;
    A, B and C at element offsets 0 to 129 inside buffers that are NaN (operands) or a guard value (results) everywhere
    else.  Against the float64 product of the same rounded operands, computed on the device (it differs from the
    oracle's k-ordered double sum by 1e-16 relative, far inside the bars): 1e-4 of max|C| for 16-bit operands, 1e-5 for
    f32, row sums 1e-5 per row; nothing stored outside C or the row sums, nothing non-finite."""
    import random
    torch = torch_cuda
    rng = random.Random(seed)

    def dim(hi):
        base = rng.choice([1, 2, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 512,
                           513, hi])
        return max(1, min(hi, base + rng.choice([0, 0, 0, 1, -1, 3, rng.randint(0, 40)])))

    knobs = ("gemm16.tile", "gemm16.split_k", "gemm_f32.tile", "gemm_f32.split_k")
    for it in range(150):
        m, n, k = dim(700), dim(1100), dim(900)
        kind = rng.choice(["bf16", "f16", "f32", "epi"])
        tile = rng.choice([0, 0, 128, 256]) if kind != "f32" else rng.choice([0, 0, 64, 128, 256])
        split = rng.choice([0, 0, 1, 2, 3])
        case = (seed, it, kind, m, n, k, tile, split)
        g = torch.Generator(device="cuda")
        g.manual_seed(seed * 1000 + it)
        dt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32, "epi": torch.float16}[kind]
        offa, offb, offc = rng.choice([0, 1, 3, 8, 129]), rng.choice([0, 1, 5, 8, 129]), rng.choice([32, 33, 35])
        buf_a = torch.full((m * k + 300,), float("nan"), device="cuda").to(dt)
        buf_b = torch.full((k * n + 300,), float("nan"), device="cuda").to(dt)
        da, db = buf_a[offa:offa + m * k].view(m, k), buf_b[offb:offb + k * n].view(k, n)
        da.copy_((torch.randn(m, k, device="cuda", generator=g) * 0.1).to(dt))
        db.copy_((torch.randn(k, n, device="cuda", generator=g) * 0.1).to(dt))
        ref = da.double() @ db.double()
        guard = torch.full((m * n + 64,), 7.0, device="cuda")
        c = guard[offc:offc + m * n].view(m, n)
        try:
            hip.set_tunable("gemm_f32.tile" if kind == "f32" else "gemm16.tile", tile)
            hip.set_tunable("gemm_f32.split_k" if kind == "f32" else "gemm16.split_k", split)
            if kind == "epi":
                bias = torch.rand(n, device="cuda", generator=g) * 0.2 - 0.1
                rs = torch.full((m + 16,), 7.0, device="cuda")
                hip.gemm_f16_bias_relu_rowsum(da, db, bias, out=c, rowsum=rs[8:8 + m])
                ref = torch.relu(ref + bias.double())
                sums = ref.sum(dim=1)
                assert bool((rs[:8] == 7).all()) and bool((rs[8 + m:] == 7).all()), case
                assert bool(((rs[8:8 + m].double() - sums).abs() <= 1e-5 * sums.abs() + 1e-6 * sums.abs().max()).all()), case
            else:
                {"bf16": hip.gemm_bf16, "f16": hip.gemm_f16, "f32": hip.gemm_f32}[kind](da, db, out=c)
        finally:
            for t in knobs:
                hip.set_tunable(t, 0)
        torch.cuda.synchronize()
        assert bool((guard[:offc] == 7).all()) and bool((guard[offc + m * n:] == 7).all()), case
        assert bool(torch.isfinite(c).all()), case
        err = (c.double() - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)
        assert err <= (1e-5 if kind == "f32" else 1e-4), (case, err)


@pytest.mark.parametrize("m,n,k", [(130, 137, 40), (257, 1001, 1000), (64, 4100, 96), (4, 1, 64), (300, 263, 136)])
def test_epilogue_ragged_shapes(hip, oracle, torch_cuda, m, n, k):
    """The fused epilogue on the same kinds of shape (the last column of an odd N comes from the matrix-vector kernel,
    which applies bias and ReLU and adds into the row sums like the tiled kernels)."""
    torch = torch_cuda
    a = normal16(oracle, (m, k), m + 51, "f16")
    b = normal16(oracle, (k, n), n + 52, "f16")
    bias = oracle.fill_uniform(n, seed=n + 53, lo=-0.1, hi=0.1)
    y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a, b, bias)
    try:
        for tile in (128, 256):
            hip.set_tunable("gemm16.tile", tile)
            y, rs = hip.gemm_f16_bias_relu_rowsum(dev(torch, a).half(), dev(torch, b).half(), dev(torch, bias))
            assert np.abs(y.cpu().numpy() - y_ref).max() <= 1e-4 * max(np.abs(y_ref).max(), 1e-30)
            assert rowsums_ok(rs.cpu().numpy(), rs_ref)
    finally:
        hip.set_tunable("gemm16.tile", 0)


@pytest.mark.parametrize("tile", [0, 64, 128, 256])
@pytest.mark.parametrize("m,n,k", [(130, 137, 41), (257, 1001, 1001), (300, 263, 35), (64, 65, 33), (512, 514, 1030),
                                   (1000, 3, 2051), (1, 1, 4), (37, 51, 24), (256, 255, 64), (70, 1028, 288)])
def test_gemm_f32_ragged_shapes_stay_on_the_mfma_kernel(hip, oracle, torch_cuda, tile, m, n, k):
    """Any N, any K of at least a slab (or a multiple of 4 below it) and any alignment of A, B and C run on the
    direct-to-LDS kernel, every tile shape: against the oracle; nothing is stored outside C; NaNs lying next to A and B
    in memory (what the transfers fetch past a row's or the matrix's end) do not reach the result."""
    torch = torch_cuda
    a = oracle.fill_uniform(m * k, seed=m + 61, lo=-1, hi=1).reshape(m, k)
    b = oracle.fill_uniform(k * n, seed=n + 62, lo=-1, hi=1).reshape(k, n)
    ref = oracle.gemm(a, b)
    off = 129 if k >= 32 else 128          # a base that is only 4-byte aligned where the kernel allows it
    buf_a = torch.full((m * k + 256,), float("nan"), device="cuda")
    buf_b = torch.full((k * n + 256,), float("nan"), device="cuda")
    da, db = buf_a[off:off + m * k].view(m, k), buf_b[off:off + k * n].view(k, n)
    da.copy_(dev(torch, a))
    db.copy_(dev(torch, b))
    hip.set_tunable("gemm_f32.tile", tile)
    try:
        for c_off in (32, 33):
            guard = torch.full((m * n + 80,), 7.0, device="cuda")
            c = guard[c_off:c_off + m * n].view(m, n)
            hip.gemm_f32(da, db, out=c)
            assert bool((guard[:c_off] == 7).all()) and bool((guard[c_off + m * n:] == 7).all())
            got = c.cpu().numpy()
            assert np.isfinite(got).all()
            assert np.abs(got - ref).max() <= f32_tol(a, b, k)
    finally:
        hip.set_tunable("gemm_f32.tile", 0)


@pytest.mark.parametrize("knob", ["force_staged", "force_simple"])
@pytest.mark.parametrize("m,n,k", [(264, 520, 72), (100, 64, 200), (8, 8, 8), (300, 264, 192)])
def test_fallback_kernels_stay_correct(hip, oracle, torch_cuda, knob, m, n, k):
    """The one-thread-per-element kernels (16-bit and f32) and the f32 register-staged kernel are what is left when a
    transfer offset would not fit 32 bits or K is too short for a slab; the direct-to-LDS kernels take the shapes
    that used to reach them, so they are switched on by their knobs here (the 16-bit library has no staged kernel:
    with that knob it runs its usual kernels)."""
    torch = torch_cuda
    a16 = normal16(oracle, (m, k), m + 71, "bf16")
    b16 = normal16(oracle, (k, n), n + 72, "bf16")
    a32 = oracle.fill_uniform(m * k, seed=m + 73, lo=-1, hi=1).reshape(m, k)
    b32 = oracle.fill_uniform(k * n, seed=n + 74, lo=-1, hi=1).reshape(k, n)
    hip.set_tunable("gemm16." + knob, 1)
    hip.set_tunable("gemm_f32." + knob, 1)
    try:
        assert (hip.gemm16_tile(m, n, k) == 0) == (knob == "force_simple")
        c16 = hip.gemm_bf16(dev(torch, a16).bfloat16(), dev(torch, b16).bfloat16()).cpu().numpy()
        c32 = hip.gemm_f32(dev(torch, a32), dev(torch, b32)).cpu().numpy()
    finally:
        hip.set_tunable("gemm16." + knob, 0)
        hip.set_tunable("gemm_f32." + knob, 0)
    ref16 = oracle.gemm(a16, b16)
    assert np.abs(c16 - ref16).max() / np.abs(ref16).max() < 1e-4
    assert np.abs(c32 - oracle.gemm(a32, b32)).max() <= f32_tol(a32, b32, k)


@pytest.mark.parametrize("m,n,k,splits", [(256, 256, 8192, 0), (128, 128, 4096, 0), (130, 136, 1024, 2), (300, 520, 448, 3),
                                          (1, 8, 4096, 16), (512, 384, 2048, 5), (64, 1001, 2048, 4)])
def test_gemm_f32_split_k(hip, oracle, torch_cuda, m, n, k, splits):
    """The f32 product cut along K on the 64 x 64 tile (few tiles, long K): against the oracle, the same bits on every
    run and on another stream, and the count the library reports.  splits = 0 leaves the choice to the launcher
    (these two shapes split), n forces n pieces."""
    torch = torch_cuda
    a = oracle.fill_uniform(m * k, seed=m + 81, lo=-1, hi=1).reshape(m, k)
    b = oracle.fill_uniform(k * n, seed=n + 82, lo=-1, hi=1).reshape(k, n)
    da, db = dev(torch, a), dev(torch, b)
    ref = oracle.gemm(a, b)
    hip.set_tunable("gemm_f32.split_k", splits)
    if splits:
        hip.set_tunable("gemm_f32.tile", 64)
    try:
        reported = hip.gemm_f32_k_splits(m, n, k)
        assert reported >= 2 and (splits == 0 or reported <= splits)
        c1 = hip.gemm_f32(da, db)
        c2 = hip.gemm_f32(da, db)
        side = side_stream(torch)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            c3 = hip.gemm_f32(da, db)
        side.synchronize()
        hip.set_tunable("gemm_f32.split_k", 1)
        assert hip.gemm_f32_k_splits(m, n, k) == 1
        whole = hip.gemm_f32(da, db)
    finally:
        hip.set_tunable("gemm_f32.split_k", 0)
        hip.set_tunable("gemm_f32.tile", 0)
    assert torch.equal(c1, c2) and torch.equal(c1, c3)
    for c in (c1, whole):
        assert np.abs(c.cpu().numpy() - ref).max() <= f32_tol(a, b, k)


def test_gemm_f32_split_k_rule(hip, torch_cuda):
    for (m, n, k), want_split in [((256, 256, 8192), True), ((512, 512, 8192), True), ((128, 4096, 4096), True),
                                  ((1024, 1024, 1024), False), ((2048, 2048, 2048), False), ((8192, 8192, 8192), False),
                                  ((1024, 1024, 8192), False), ((512, 512, 100), False)]:
        assert (hip.gemm_f32_k_splits(m, n, k) > 1) == want_split, (m, n, k)
