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


def check_scatter(got, counters_after, keys, n, starts, shift, mask, oracle, out_len=None):
    """Digit by digit the same keys as the thread-order scatter, whatever their order in the range."""
    out_len = len(got) if out_len is None else out_len
    exp, exp_counters = np.full(out_len, -1, dtype=np.int32), starts.copy()
    outside = oracle.radix_scatter(keys, exp, exp_counters, n, shift, mask)
    assert np.array_equal(counters_after, exp_counters)
    if outside == 0:
        digit = lambda a: (a.view(np.uint32) >> np.uint32(shift)) & np.uint32(mask)     # noqa: E731
        written = exp != -1
        assert np.array_equal(got[~written], exp[~written])                    # nothing else touched
        assert np.array_equal(digit(got[written]), digit(exp[written]))        # every range holds its digit
        order_g, order_e = np.lexsort((got[written], digit(got[written]))), np.lexsort((exp[written], digit(exp[written])))
        assert np.array_equal(got[written][order_g], exp[written][order_e])
    return outside


@pytest.mark.parametrize("n", [0, 1, 5, 8191, 8192, 8193, 100_003, 1_000_003])
@pytest.mark.parametrize("shift,mask", [(0, 255), (8, 255), (4, 15)])
def test_radix_scatter_sizes(hip, torch_cuda, oracle, n, shift, mask):
    torch = torch_cuda
    keys = keys_of(n, n + shift, 1, 2**31 - 1)                    # -1 marks untouched slots below
    digits = (keys >> shift) & mask
    counts = np.bincount(digits, minlength=256)
    starts = np.concatenate(([0], np.cumsum(counts)[:-1])).astype(np.int32)
    out = torch.full((n + 64,), -1, dtype=torch.int32, device="cuda")
    counters = torch.from_numpy(starts.copy()).cuda()
    hip.radix_scatter(torch.from_numpy(keys).cuda(), out, counters, shift, mask)
    assert check_scatter(out.cpu().numpy(), counters.cpu().numpy(), keys, n, starts, shift, mask, oracle) == 0


@pytest.mark.parametrize("n,shape", [(100_003, 2), (100_003, 3), (100_003, 4), (40_000, 4), ((1 << 22) + 4099, 0)])
def test_radix_scatter_tile_shapes(hip, torch_cuda, oracle, n, shape):
    """Every tile shape of the kernel (8192 to 32768 keys; 0 = the library's choice, which from 2^22 keys on
    is the 16384-key tile), ragged last tiles included."""
    torch = torch_cuda
    shift, mask = 8, 255
    keys = keys_of(n, shape, 1, 2**31 - 1)
    counts = np.bincount((keys >> shift) & mask, minlength=256)
    starts = np.concatenate(([0], np.cumsum(counts)[:-1])).astype(np.int32)
    out = torch.full((n + 64,), -1, dtype=torch.int32, device="cuda")
    counters = torch.from_numpy(starts.copy()).cuda()
    hip.set_tunable("radix_scatter.tile", shape)
    try:
        hip.radix_scatter(torch.from_numpy(keys).cuda(), out, counters, shift, mask)
        torch.cuda.synchronize()
    finally:
        hip.set_tunable("radix_scatter.tile", 0)
    assert check_scatter(out.cpu().numpy(), counters.cpu().numpy(), keys, n, starts, shift, mask, oracle) == 0


def test_radix_scatter_skips_positions_outside_the_output(hip, torch_cuda, oracle):
    """Counters that start 40 too high push the last keys of the last digit past the output: those
    stores are dropped (the slots behind the output keep their contents), the counters still advance."""
    torch = torch_cuda
    n, shift, mask = 50_000, 0, 255
    keys = keys_of(n, 3, 1, 2**31 - 1)
    counts = np.bincount(keys & mask, minlength=256)
    starts = (np.concatenate(([0], np.cumsum(counts)[:-1])) + 40).astype(np.int32)
    whole = torch.full((n + 4096,), -1, dtype=torch.int32, device="cuda")
    counters = torch.from_numpy(starts.copy()).cuda()
    hip.radix_scatter(torch.from_numpy(keys).cuda(), whole[:n], counters, shift, mask)
    got = whole.cpu().numpy()
    assert np.all(got[n:] == -1) and np.all(got[:40] == -1) and np.all(got[40:n] != -1)
    assert np.array_equal(counters.cpu().numpy(), starts + counts)
    exp, c = np.full(n, -1, dtype=np.int32), starts.copy()
    assert oracle.radix_scatter(keys, exp, c, n, shift, mask) == 40


def test_radix_scatter_ir_dispatch(hip, torch_cuda, oracle):
    from spoc_amd import reference_kernels
    from spoc_amd.sarek import Execute, Vector
    n, shift, mask = 77_777, 8, 255
    keys = keys_of(n, 9, 1, 2**31 - 1)
    counts = np.bincount((keys >> shift) & mask, minlength=256)
    starts = np.concatenate(([0], np.cumsum(counts)[:-1])).astype(np.int32)
    for specialise, tag, reach in ((1, "radix_scatter_i32", n), (0, "jit", n), (1, "radix_scatter_i32", 25_600)):
        vk, vo, vc = Vector.create(Vector.int32, n), Vector.create(Vector.int32, n), Vector.create(Vector.int32, 256)
        vk.fill_from(keys)
        vo.fill_from(np.full(n, -1))
        vc.fill_from(starts)
        hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
        try:
            path = Execute.run_vectors(ir=reference_kernels.radix_sort_scatter(),
                                       args=[Execute.Vec(vk), Execute.Vec(vo), Execute.Vec(vc), Execute.Int32(n),
                                             Execute.Int32(shift), Execute.Int32(mask)],
                                       block=Execute.dims1d(256), grid=Execute.dims1d((reach + 255) // 256))
        finally:
            hip.check(hip.lib.sarek_hip_set_specialisation(1))
        assert path == tag
        assert check_scatter(vo.to_array(), vc.to_array(), keys, min(n, reach), starts, shift, mask, oracle) == 0


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
    hip.check(hip.lib.sarek_hip_set_specialisation(0))
    try:
        rec = benchmarks.bench_radix_sort(100_003, warmup=1, iterations=2)
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    assert rec["verified"] and rec["path"] == "jit"
    rec = benchmarks.bench_radix_sort(300_001, warmup=1, iterations=2)
    assert rec["verified"] and rec["path"] == "radix_scatter_i32"      # the last launch of a pass


@pytest.mark.parametrize("off", [1, 2, 3])
@pytest.mark.parametrize("n", [1, 5, 4099, 100_003, 1_000_003])
def test_keys_at_any_alignment(hip, torch_cuda, oracle, off, n):
    """Keys that start on any 4-byte boundary (a sub-vector): the histograms and the scatter pass run the same
    kernels and give the aligned results."""
    torch = torch_cuda
    keys = keys_of(n, n + off, 1, 2**31 - 1)
    dk = torch.zeros(n + 8, dtype=torch.int32, device="cuda")[off:off + n]
    dk.copy_(torch.from_numpy(keys))
    hist = torch.zeros(256, dtype=torch.int32, device="cuda")
    hip.histogram(dk, hist, 256)
    expected = np.zeros(256, dtype=np.int32)
    assert oracle.histogram(keys, expected, n, 256) == 0
    assert np.array_equal(hist.cpu().numpy(), expected)
    hist.zero_()
    hip.radix_histogram(dk, hist, 8, 255)
    expected = np.zeros(256, dtype=np.int32)
    assert oracle.radix_histogram(keys, expected, n, 8, 255) == 0
    assert np.array_equal(hist.cpu().numpy(), expected)
    digits = (keys >> 8) & 255
    counts = np.bincount(digits, minlength=256)
    starts = np.concatenate(([0], np.cumsum(counts)[:-1])).astype(np.int32)
    out = torch.full((n + 64,), -1, dtype=torch.int32, device="cuda")
    counters = torch.from_numpy(starts.copy()).cuda()
    hip.radix_scatter(dk, out, counters, 8, 255)
    assert check_scatter(out.cpu().numpy(), counters.cpu().numpy(), keys, n, starts, 8, 255, oracle) == 0
