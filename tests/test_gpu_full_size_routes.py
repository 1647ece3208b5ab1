"""The BASELINE configurations at their full sizes through the plugin routes that bench.py times -- the very calls of
bench.make_workload, with the same geometry -- checked against the oracle on sampled rows and through size-independent
properties, with the code path that served each launch asserted:

  f32 GEMM 8192^3            Execute.run_vectors, matrix_mul_tiled IR (bench_matrix_mul_tiled.ml:55-95), 16 x 16 blocks
  bf16 GEMM 8192^3           Execute.run_source, library kernel text gemm_bf16, one thread per element of C
  fp16 epilogue 4095x11008x4096   Execute.run_source, library kernel text gemm_f16_bias_relu_rowsum
  triad + sum, n = 2^28      Execute.run_pipeline [stream_triad IR; block-256 reduction IR], then the device fold

Inputs are made on the device and copied into the vectors' buffers as bench.py does (a vector of Location Both, as
after an upload); results are read from the vectors' device buffers.

Bars: f32 GEMM 1e-4 * |A|max * |B|max * sqrt(K); 16-bit GEMMs 2e-2 relative to max|C| (asserted at 1e-4); row sums and
the folded sum 1e-5 relative; the triad's vector and block sums bit for bit."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture()
def sarek(hip, torch_cuda):
    from spoc_amd import sarek as s
    s.Device.init()
    return s


def device_vector(sarek, hip, tensor, kind=None, elem_size=None):
    V = sarek.Vector
    v = V.create_custom(elem_size, tensor.numel()) if elem_size else V.create(kind, tensor.numel())
    sarek.Transfer.to_device(v)
    hip.check(hip.lib.sarek_hip_memcpy_dtod(v.device_ptr, tensor.data_ptr(), tensor.numel() * tensor.element_size()))
    return v


def device_contents(hip, torch, v, count, dtype):
    """The first `count` elements of a vector's device buffer as a torch tensor (a device-to-device copy)."""
    out = torch.empty(count, dtype=dtype, device="cuda")
    torch.cuda.synchronize()
    hip.check(hip.lib.sarek_hip_memcpy_dtod(out.data_ptr(), v.device_ptr, count * out.element_size()))
    torch.cuda.synchronize()
    return out


def test_f32_gemm_8192_through_run_vectors(hip, oracle, torch_cuda, sarek):
    torch = torch_cuda
    from spoc_amd import reference_kernels as rk
    E, V = sarek.Execute, sarek.Vector
    s = 8192
    g = torch.Generator(device="cuda")
    g.manual_seed(0xA11CE)
    a = torch.rand(s, s, device="cuda", generator=g) * 2 - 1
    g.manual_seed(0xB0B)
    b = torch.rand(s, s, device="cuda", generator=g) * 2 - 1
    va, vb = device_vector(sarek, hip, a, V.float32), device_vector(sarek, hip, b, V.float32)
    vc = V.create(V.float32, s * s)
    sarek.Transfer.to_device(vc)
    path = E.run_vectors(rk.matrix_mul_tiled(), [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(s), E.Int32(s), E.Int32(s)],
                         (16, 16, 1), (s // 16, s // 16, 1), shared_mem=2048)
    assert path == "matmul_tiled_f32"
    c = device_contents(hip, torch, vc, s * s, torch.float32).view(s, s)
    rows = np.array([0, 63, 64, 4097, 8191], np.int32)
    a_h, b_h = a[torch.from_numpy(rows).long().cuda()].cpu().numpy(), b.cpu().numpy()
    ref = oracle.gemm_rows(a_h, b_h, np.arange(len(rows), dtype=np.int32))
    got = c[torch.from_numpy(rows).long().cuda()].cpu().numpy()
    assert np.abs(got - ref).max() <= 1e-4 * float(a.abs().max()) * float(b.abs().max()) * np.sqrt(s)
    # B = identity gives A back bit for bit (every product is exact, every sum has one non-zero term)
    hip.check(hip.lib.sarek_hip_memcpy_dtod(vb.device_ptr, torch.eye(s, device="cuda").data_ptr(), s * s * 4))
    assert E.run_vectors(rk.matrix_mul_tiled(), [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(s), E.Int32(s), E.Int32(s)],
                         (16, 16, 1), (s // 16, s // 16, 1), shared_mem=2048) == "matmul_tiled_f32"
    assert torch.equal(device_contents(hip, torch, vc, s * s, torch.float32).view(s, s), a)


def test_bf16_gemm_8192_through_run_source(hip, oracle, torch_cuda, sarek):
    torch = torch_cuda
    E, V = sarek.Execute, sarek.Vector
    s = 8192
    g = torch.Generator(device="cuda")
    g.manual_seed(0xA4)
    a = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
    g.manual_seed(0xB4)
    b = (torch.randn(s, s, device="cuda", generator=g) * 0.02).bfloat16()
    va, vb = device_vector(sarek, hip, a, elem_size=2), device_vector(sarek, hip, b, elem_size=2)
    vc = V.create(V.float32, s * s)
    sarek.Transfer.to_device(vc)
    src, entry = E.library_kernel("gemm_bf16")
    args = [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Int32(s), E.Int32(s), E.Int32(s)]
    assert E.run_source(src, entry, (16, 16, 1), (s // 16, s // 16, 1), args) == "gemm_bf16"
    c = device_contents(hip, torch, vc, s * s, torch.float32).view(s, s)
    rows = np.array([0, 255, 256, 5000, 8191], np.int32)
    idx = torch.from_numpy(rows).long().cuda()
    ref = oracle.gemm_rows(a[idx].float().cpu().numpy(), b.float().cpu().numpy(), np.arange(len(rows), dtype=np.int32))
    got = c[idx].cpu().numpy()
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
    # an exact power-of-two scaling of A commutes with the kernel
    hip.check(hip.lib.sarek_hip_memcpy_dtod(va.device_ptr, (a * 2).data_ptr(), s * s * 2))
    assert E.run_source(src, entry, (16, 16, 1), (s // 16, s // 16, 1), args) == "gemm_bf16"
    assert torch.equal(device_contents(hip, torch, vc, s * s, torch.float32).view(s, s), c * 2)


def test_f16_epilogue_full_size_through_run_source(hip, oracle, torch_cuda, sarek):
    torch = torch_cuda
    E, V = sarek.Execute, sarek.Vector
    m, n, k = 4095, 11008, 4096
    g = torch.Generator(device="cuda")
    g.manual_seed(0xA5)
    a = (torch.randn(m, k, device="cuda", generator=g) * 0.02).half()
    g.manual_seed(0xB5)
    b = (torch.randn(k, n, device="cuda", generator=g) * 0.02).half()
    bias = torch.rand(n, device="cuda", generator=g) * 0.2 - 0.1
    va, vb = device_vector(sarek, hip, a, elem_size=2), device_vector(sarek, hip, b, elem_size=2)
    vbias = device_vector(sarek, hip, bias, V.float32)
    vy, vrs = V.create(V.float32, m * n), V.create(V.float32, m)
    sarek.Transfer.to_device(vy)
    sarek.Transfer.to_device(vrs)
    src, entry = E.library_kernel("gemm_f16_bias_relu_rowsum")
    args = [E.Vec(va), E.Vec(vb), E.Vec(vbias), E.Vec(vy), E.Vec(vrs), E.Int32(m), E.Int32(n), E.Int32(k)]
    assert E.run_source(src, entry, (256, 1, 1), (1024, 1, 1), args) == "gemm_f16_bias_relu_rowsum"
    y = device_contents(hip, torch, vy, m * n, torch.float32).view(m, n)
    rs = device_contents(hip, torch, vrs, m, torch.float32)
    rows = np.array([0, 127, 128, 2047, 3968, 4094], np.int32)
    idx = torch.from_numpy(rows).long().cuda()
    y_ref, rs_ref = oracle.gemm_bias_relu_rowsum(a[idx].float().cpu().numpy(), b.float().cpu().numpy(),
                                                 bias.cpu().numpy())
    got = y[idx].cpu().numpy()
    assert np.abs(got - y_ref).max() <= 2e-2 * np.abs(y_ref).max()
    assert np.abs(got - y_ref).max() <= 1e-4 * np.abs(y_ref).max()
    assert (np.abs(rs[idx].cpu().numpy().astype(np.float64) - rs_ref) <= 1e-5 * np.abs(rs_ref)).all()
    # every row: the fused row sum is the sum of the stored row, and nothing is negative
    sums = y.double().sum(dim=1)
    assert bool(((rs.double() - sums).abs() <= 1e-5 * sums).all()) and bool((y >= 0).all())
    # a second run leaves the same bits (the tiles' shares are added in tile order)
    assert E.run_source(src, entry, (256, 1, 1), (1024, 1, 1), args) == "gemm_f16_bias_relu_rowsum"
    assert torch.equal(device_contents(hip, torch, vrs, m, torch.float32), rs)


def test_triad_sum_2p28_through_run_pipeline(hip, oracle, torch_cuda, sarek):
    torch = torch_cuda
    from spoc_amd import reference_kernels as rk
    E, V = sarek.Execute, sarek.Vector
    n = 1 << 28
    g = torch.Generator(device="cuda")
    g.manual_seed(0xB)
    b = torch.rand(n, device="cuda", generator=g)
    g.manual_seed(0xC)
    c = torch.rand(n, device="cuda", generator=g)
    vb, vc = device_vector(sarek, hip, b, V.float32), device_vector(sarek, hip, c, V.float32)
    va, vout = V.create(V.float32, n), V.create(V.float32, n // 256)
    sarek.Transfer.to_device(va)
    sarek.Transfer.to_device(vout)
    stages = [(rk.stream_triad(), [E.Vec(va), E.Vec(vb), E.Vec(vc), E.Float32(3.0), E.Int32(n)], (256, 1, 1), (n // 256, 1, 1)),
              (rk.tree(False), [E.Vec(va), E.Vec(vout), E.Int32(n)], (256, 1, 1), (n // 256, 1, 1))]
    path, launches = E.run_pipeline(stages)
    assert (path, launches) == ("stream_triad_f32+reduce_sum_block256_f32", 1)
    total = torch.zeros(1, dtype=torch.float64, device="cuda")
    hip.check(hip.lib.sarek_hip_fold_partials_f64(vout.device_ptr, n // 256, total.data_ptr(), None))
    a = device_contents(hip, torch, va, n, torch.float32)
    sums = device_contents(hip, torch, vout, n // 256, torch.float32)
    # the oracle on the whole workload: the vector and every block sum bit for bit, the folded sum to 1e-5
    a_ref, sums_ref, sum_ref = oracle.triad_sum(b.cpu().numpy(), c.cpu().numpy(), 3.0, threads=16)
    assert torch.equal(a.cpu(), torch.from_numpy(a_ref))
    assert np.abs(sums.cpu().numpy() - sums_ref).max() <= 1e-5 * np.abs(sums_ref).max()
    assert abs(total.item() - sum_ref) <= 1e-5 * abs(sum_ref)
    # and bit for bit what the two hand kernels launched one after the other leave
    a2 = hip.triad(b, c, 3.0)
    s2 = torch.empty(n // 256, device="cuda")
    hip.check(hip.lib.sarek_hip_reduce_sum_block256_f32(a2.data_ptr(), s2.data_ptr(), n, None))
    torch.cuda.synchronize()
    assert torch.equal(a2, a) and torch.equal(s2, sums)
