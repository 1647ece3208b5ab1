"""GPU parity: stream triad, fused triad+sum, block-256 reductions, casts — HIP kernels
through the C ABI against the CPU oracle on the same seeded inputs.

Bars: `a` bit-exact (the kernel evaluates b + c*s in double and rounds once, as the
Native backend does); sums within 1e-5 relative (f32 reductions); block partials within
the reference's own tolerance (1e-3 relative, bench_reduction.ml:161-163) and in practice
~1e-6."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 3, 4, 5, 255, 256, 257, 1023, 4096, 65537, 1 << 20, (1 << 22) + 3]


def dev(torch, x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


@pytest.mark.parametrize("n", SIZES)
def test_triad_bit_exact(hip, oracle, torch_cuda, n):
    torch = torch_cuda
    b = oracle.fill_uniform(n, seed=0xB)
    c = oracle.fill_uniform(n, seed=0xC)
    a = hip.triad(dev(torch, b), dev(torch, c), 3.0)
    torch.cuda.synchronize()
    assert np.array_equal(a.cpu().numpy(), oracle.triad(b, c, 3.0))


def test_triad_reference_inputs(hip, oracle, torch_cuda):
    torch = torch_cuda
    n = 100000
    b = ((np.arange(n) % 100) / 100.0).astype(np.float32)
    c = (((np.arange(n) + 1) % 100) / 100.0).astype(np.float32)
    a = hip.triad(dev(torch, b), dev(torch, c), 3.0).cpu().numpy()
    expected = (np.arange(n) % 100) / 100.0 + ((np.arange(n) + 1) % 100) / 100.0 * 3.0
    assert np.abs(a - expected).max() <= 1e-5  # bench_stream_triad.ml:122
    assert np.array_equal(a, oracle.triad(b, c, 3.0))


@pytest.mark.parametrize("n", SIZES)
def test_triad_sum(hip, oracle, torch_cuda, n):
    torch = torch_cuda
    b = oracle.fill_uniform(n, seed=0xB)
    c = oracle.fill_uniform(n, seed=0xC)
    a, total = hip.triad_sum(dev(torch, b), dev(torch, c), 3.0)
    torch.cuda.synchronize()
    a_ref, _, sum_ref = oracle.triad_sum(b, c, 3.0)
    assert np.array_equal(a.cpu().numpy(), a_ref)
    got = float(total.item())
    assert abs(got - sum_ref) <= 1e-5 * abs(sum_ref) + 0.0 if n else got == 0.0


def test_triad_sum_unaligned_pointers(hip, oracle, torch_cuda):
    torch = torch_cuda
    n = 10001
    b = oracle.fill_uniform(n + 1, seed=1)
    c = oracle.fill_uniform(n + 1, seed=2)
    db, dc = dev(torch, b)[1:], dev(torch, c)[1:]   # 4-byte aligned only
    out = torch.empty(n + 1, dtype=torch.float32, device="cuda")[1:]
    a, total = hip.triad_sum(db, dc, 3.0, out=out)
    a_ref, _, sum_ref = oracle.triad_sum(b[1:], c[1:], 3.0)
    assert np.array_equal(a.cpu().numpy(), a_ref)
    assert abs(float(total.item()) - sum_ref) <= 1e-5 * sum_ref


def test_triad_sum_workspace_too_small_is_an_error(hip, torch_cuda):
    torch = torch_cuda
    n = 1 << 20
    b = torch.zeros(n, device="cuda")
    ws = (torch.empty(1, device="cuda"), torch.empty(1, dtype=torch.float64, device="cuda"))
    with pytest.raises(hip.SarekHipError) as e:
        hip.triad_sum(b, b, 3.0, workspace=ws)
    assert e.value.status == hip.E_WORKSPACE


def test_triad_sum_full_size_properties(hip, torch_cuda):
    """n = 2^28 (the benchmark size): properties that need no CPU pass.
    b = c = 1 -> every a is exactly 4 and the sum is exactly 4n; linearity in s."""
    torch = torch_cuda
    n = 1 << 28
    b = torch.ones(n, device="cuda")
    c = torch.ones(n, device="cuda")
    a, total = hip.triad_sum(b, c, 3.0)
    assert float(total.item()) == 4.0 * n
    assert bool((a == 4.0).all())
    a2, total2 = hip.triad_sum(b, c, 0.0, out=a)
    assert float(total2.item()) == float(n)
    # pseudo-random input: compare the fused sum with a float64 device sum of a
    torch.manual_seed(7)
    b.uniform_(0, 1)
    c.uniform_(0, 1)
    a, total = hip.triad_sum(b, c, 3.0, out=a)
    ref = float(a.double().sum().item())
    assert abs(float(total.item()) - ref) <= 1e-5 * ref
    want = (b.double() + c.double() * 3.0).float()
    assert torch.equal(a, want)


@pytest.mark.parametrize("n", [1, 255, 256, 257, 1000, 65536, 1000003])
def test_reduce_sum_block256(hip, oracle, torch_cuda, n):
    torch = torch_cuda
    ones = torch.ones(n, device="cuda")
    p = hip.reduce_sum_block256(ones)
    assert p.numel() == (n + 255) // 256
    assert float(hip.fold_partials(p).item()) == float(n)  # bench_reduction.ml:110-111
    x = oracle.fill_uniform(n, seed=0x5)
    p = hip.reduce_sum_block256(dev(torch, x)).cpu().numpy()
    p_ref = oracle.reduce_sum_block256(x)
    assert np.allclose(p, p_ref, rtol=1e-5, atol=1e-6)
    got = float(hip.fold_partials(dev(torch, p)).item())
    assert abs(got - oracle.fold_partials(p_ref)) <= 1e-5 * oracle.fold_partials(p_ref)


@pytest.mark.parametrize("n", [1, 256, 1000, 100000])
def test_dot_block256(hip, oracle, torch_cuda, n):
    torch = torch_cuda
    a = ((np.arange(n) % 100) / 100.0).astype(np.float32)
    b = (((np.arange(n) + 1) % 100) / 100.0).astype(np.float32)
    p = hip.dot_block256(dev(torch, a), dev(torch, b)).cpu().numpy()
    p_ref = oracle.dot_block256(a, b)
    assert np.allclose(p, p_ref, rtol=1e-5, atol=1e-6)
    expected = oracle.fold_partials(p_ref)
    assert abs(float(p.astype(np.float64).sum()) - expected) <= 1e-3 * max(expected, 1e-30)


def test_casts_bit_exact(hip, oracle, torch_cuda):
    torch = torch_cuda
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(100003) * np.exp(rng.uniform(-30, 12, 100003))).astype(np.float32)
    x[:6] = [0.0, -0.0, 65504.0, 65520.0, 2.0 ** -24, 2.0 ** -25]
    d = dev(torch, x)
    assert np.array_equal(hip.cast_bf16(d).view(torch.int16).cpu().numpy().view(np.uint16),
                          oracle.bf16_bits(x))
    assert np.array_equal(hip.cast_f16(d).view(torch.int16).cpu().numpy().view(np.uint16),
                          oracle.f16_bits(x))


@pytest.mark.parametrize("n", [1, 255, 256, 257, 100000, 1 << 20])
def test_block256_max_matches_tree_bit_for_bit(hip, oracle, torch_cuda, n):
    torch = torch_cuda
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 1000).astype(np.float32)
    if n > 300:
        x[5] = np.nan
        x[300] = -0.0
        x[301] = 0.0
    got = hip.reduce_max_block256(torch.from_numpy(x).cuda()).cpu().numpy()
    exp = oracle.reduce_max_block256(x)
    assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))
    # another fill value
    got = hip.reduce_max_block256(torch.from_numpy(x).cuda(), pad=float("-inf")).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.reduce_max_block256(x, pad=float("-inf")).view(np.uint32))


@pytest.mark.parametrize("offsets", [(1, 1, 1), (1, 2, 3), (0, 1, 0), (3, 0, 2)])
@pytest.mark.parametrize("n", [1, 5, 1023, 4099, 300007])
def test_stream_kernels_take_vectors_at_any_alignment(hip, oracle, torch_cuda, offsets, n):
    """Sub-vectors start anywhere (Vector.sub_vector): the triad, the fused triad + block sum / maximum and the block
    reductions run their 128-bit kernels on vectors that are only 4-byte aligned and give the aligned results; the
    element-per-thread kernel stays reachable behind stream.force_scalar."""
    torch = torch_cuda
    oa, ob, oc = offsets
    b = oracle.fill_uniform(n, seed=11)
    c = (oracle.fill_uniform(n, seed=12) * 2000 - 1000).astype(np.float32)
    db = torch.full((n + 8,), float("nan"), device="cuda")[ob:ob + n]
    dc = torch.full((n + 8,), float("nan"), device="cuda")[oc:oc + n]
    db.copy_(dev(torch, b))
    dc.copy_(dev(torch, c))
    guard = torch.full((n + 8,), 7.0, device="cuda")
    out = guard[oa:oa + n]
    a_ref, partials_ref, sum_ref = oracle.triad_sum(b, c, 3.0)
    for scalar in (0, 1):
        hip.set_tunable("stream.force_scalar", scalar)
        try:
            guard.fill_(7.0)
            a, total = hip.triad_sum(db, dc, 3.0, out=out)
            assert np.array_equal(a.cpu().numpy(), a_ref)
            assert bool((guard[:oa] == 7).all()) and bool((guard[oa + n:] == 7).all())
            assert abs(float(total.item()) - sum_ref) <= 1e-5 * abs(sum_ref)
        finally:
            hip.set_tunable("stream.force_scalar", 0)
    guard.fill_(7.0)
    a, sums = hip.triad_block256_sum(db, dc, 3.0, out=out)
    assert np.array_equal(a.cpu().numpy(), a_ref) and bool((guard[:oa] == 7).all()) and bool((guard[oa + n:] == 7).all())
    assert np.abs(sums.cpu().numpy() - partials_ref).max() <= 1e-5 * np.abs(partials_ref).max()
    a, mx = hip.triad_block256_max(db, dc, 3.0, -1000000.0, out=out)
    assert np.array_equal(a.cpu().numpy(), a_ref)
    assert np.array_equal(mx.cpu().numpy(), oracle.reduce_max_block256(a_ref))
    # the block reductions on an unaligned input
    assert np.array_equal(hip.reduce_max_block256(dc).cpu().numpy(), oracle.reduce_max_block256(c))
    got = hip.reduce_sum_block256(db).cpu().numpy()
    want = oracle.reduce_sum_block256(b)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    got = hip.dot_block256(db, dc).cpu().numpy()
    want = oracle.dot_block256(b, c)
    assert np.abs(got - want).max() <= 1e-5 * max(np.abs(want).max(), 1e-30)
