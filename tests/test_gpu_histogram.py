"""Histogram kernels (benchmarks/bench_histogram.ml:54-84 and the counting kernel of
benchmarks/bench_radix_sort.ml:82-116): the hand kernels through the C ABI and the kernels' IR
through Execute.run_vectors, against the CPU oracle bit for bit; the generated code and the hand
kernel must be interchangeable."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def keys_of(n, seed, lo=0, hi=1 << 30):
    return np.random.default_rng(seed).integers(lo, hi, n).astype(np.int32)


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 1023, 4096, 65537, 1_000_003, (1 << 24) + 7])
@pytest.mark.parametrize("bins", [256, 100])
def test_histogram_sizes(hip, torch_cuda, oracle, n, bins):
    torch = torch_cuda
    keys = keys_of(n, n + bins)
    hist = torch.full((256,), 5, dtype=torch.int32, device="cuda")
    hip.histogram(torch.from_numpy(keys).cuda(), hist, bins)
    expected = np.full(256, 5, dtype=np.int32)
    assert oracle.histogram(keys, expected, n, bins) == 0
    assert np.array_equal(hist.cpu().numpy(), expected)


@pytest.mark.parametrize("bins", [1, 2, 7, 64, 255, 256])
def test_histogram_bin_counts_and_negative_keys(hip, torch_cuda, oracle, bins):
    """Keys of both signs: a negative key counts only where its remainder is 0, as in the oracle
    (which reports the others as without a slot); skewed keys (one value) go through the same adds."""
    torch = torch_cuda
    n = 200_001
    keys = keys_of(n, bins, -2**31, 2**31 - 1)
    keys[:1000] = -bins * 3                                        # remainder 0
    keys[1000:5000] = 42                                           # one hot bin
    hist = torch.zeros(256, dtype=torch.int32, device="cuda")
    hip.histogram(torch.from_numpy(keys).cuda(), hist, bins)
    expected = np.zeros(256, dtype=np.int32)
    skipped = oracle.histogram(keys, expected, n, bins)
    assert np.array_equal(hist.cpu().numpy(), expected)
    assert int(expected.sum()) + skipped == n


@pytest.mark.parametrize("shift,mask", [(0, 255), (8, 255), (16, 255), (24, 255), (5, 31), (0, 0)])
def test_radix_histogram(hip, torch_cuda, oracle, shift, mask):
    torch = torch_cuda
    n = 300_007
    keys = keys_of(n, shift + mask, -2**31, 2**31 - 1)
    hist = torch.zeros(256, dtype=torch.int32, device="cuda")
    hip.radix_histogram(torch.from_numpy(keys).cuda(), hist, shift, mask)
    expected = np.zeros(256, dtype=np.int32)
    assert oracle.radix_histogram(keys, expected, n, shift, mask) == 0
    assert np.array_equal(hist.cpu().numpy(), expected)


def test_argument_checks(hip, torch_cuda):
    torch = torch_cuda
    keys = torch.zeros(64, dtype=torch.int32, device="cuda")
    hist = torch.zeros(256, dtype=torch.int32, device="cuda")
    for bins in (0, -1, 257):
        assert hip.lib.sarek_hip_histogram_i32(hist.data_ptr(), keys.data_ptr(), 64, bins, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_histogram_i32(hist.data_ptr(), keys.data_ptr(), -1, 256, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_histogram_i32(hist.data_ptr(), keys.data_ptr() + 4, 8, 256, None) == hip.E_INVALID_ARG
    assert "16-byte" in hip.lib.sarek_hip_last_error().decode()
    assert hip.lib.sarek_hip_radix_histogram_i32(hist.data_ptr(), keys.data_ptr(), 64, 32, 255, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_radix_histogram_i32(hist.data_ptr(), keys.data_ptr(), 64, 0, 256, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_histogram_i32(None, None, 0, 256, None) == hip.OK
    assert not bool(hist.any())


def run_histogram_ir(n, bins, block, grid, keys, specialise, hip, radix=None):
    from spoc_amd import reference_kernels
    from spoc_amd.sarek import Execute, Vector
    vk = Vector.create(Vector.int32, len(keys))
    vk.fill_from(keys)
    vh = Vector.create(Vector.int32, 256)
    vh.fill_from(np.full(256, 2))
    if radix is None:
        ir, tail = reference_kernels.histogram(), [Execute.Int32(n), Execute.Int32(bins)]
    else:
        ir, tail = reference_kernels.radix_sort_histogram(), [Execute.Int32(n), Execute.Int32(radix[0]), Execute.Int32(radix[1])]
    hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
    try:
        path = Execute.run_vectors(ir=ir, args=[Execute.Vec(vk), Execute.Vec(vh)] + tail, block=Execute.dims1d(block),
                                   grid=Execute.dims1d(grid), shared_mem=1024)
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    return path, vh.to_array()


@pytest.mark.parametrize("n,bins,block,grid,tag", [
    (100_003, 256, 256, 391, "histogram_i32"),
    (100_003, 100, 256, 391, "histogram_i32"),
    (100_003, 100, 128, 782, "histogram_i32"),          # a block wider than the bin range is enough
    (100_003, 256, 256, 100, "histogram_i32"),          # a launch that reaches only 25600 keys
    (100_003, 256, 128, 782, "jit"),                    # narrower than the bins: the generated code keeps its own ways
    (1000, 300, 256, 4, "jit"),                         # more bins than slots
])
def test_histogram_ir_dispatch_matches_generated_code(hip, torch_cuda, oracle, n, bins, block, grid, tag):
    keys = keys_of(n, 17)
    if bins > 256:
        keys %= 256                                     # keep the generated code inside its shared array
    path, got = run_histogram_ir(n, bins, block, grid, keys, 1, hip)
    assert path == tag
    jit_path, jit = run_histogram_ir(n, bins, block, grid, keys, 0, hip)
    assert jit_path == "jit" and np.array_equal(got, jit)
    if block >= min(bins, 256) and bins <= 256:
        expected = np.full(256, 2, dtype=np.int32)
        assert oracle.histogram(keys, expected, n, bins, block=block, grid=grid) == 0
        assert np.array_equal(got, expected)


@pytest.mark.parametrize("shift", [0, 8, 24])
def test_radix_histogram_ir_dispatch(hip, torch_cuda, oracle, shift):
    n = 77_777
    keys = keys_of(n, shift, -2**31, 2**31 - 1)
    path, got = run_histogram_ir(n, 256, 256, (n + 255) // 256, keys, 1, hip, radix=(shift, 255))
    assert path == "radix_histogram_i32"
    jit_path, jit = run_histogram_ir(n, 256, 256, (n + 255) // 256, keys, 0, hip, radix=(shift, 255))
    expected = np.full(256, 2, dtype=np.int32)
    assert oracle.radix_histogram(keys, expected, n, shift, 255) == 0
    assert jit_path == "jit" and np.array_equal(got, jit) and np.array_equal(got, expected)
    # a shift above 24 would let the sign fill reach the digit: left to the generated code
    assert run_histogram_ir(n, 256, 256, (n + 255) // 256, keys, 1, hip, radix=(25, 255))[0] == "jit"


def test_bench_mirrors_take_the_hand_kernels(hip, torch_cuda):
    from spoc_amd import benchmarks
    rec = benchmarks.bench_histogram(1_000_003, warmup=1, iterations=3)
    assert rec["verified"] and rec["path"] == "histogram_i32"
    hip.check(hip.lib.sarek_hip_set_specialisation(0))
    try:
        rec = benchmarks.bench_histogram(100_003, warmup=1, iterations=2)
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    assert rec["verified"] and rec["path"] == "jit"
    rec = benchmarks.bench_radix_sort(300_001, warmup=1, iterations=2)
    assert rec["verified"] and rec["path"] == "jit"          # the last launch of a pass is the scatter kernel
