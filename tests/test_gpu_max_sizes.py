"""The largest vectors the dispatcher can express: a vector's length travels as an int32
(sarek/sarek/Execute.ml:197-216), so n = 2^31 - 1 elements (8 GiB of f32 or int32) is the ceiling.
The kernels index with 64-bit offsets; these tests run them there and check closed forms, since no
CPU oracle finishes such sizes in test time."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

N_MAX = 2 ** 31 - 1


def run_ir(hip, ir, block, grid, items, specialise):
    hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
    try:
        path = hip.run_source(hip.generate_source(ir, block=block), "sarek_kern", block, grid, items)
        hip.check(hip.lib.sarek_hip_device_synchronize())
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    return path


@pytest.mark.parametrize("specialise,tag", [(1, "stream_triad_f32"), (0, "jit")])
def test_triad_at_the_largest_vector(hip, torch_cuda, specialise, tag):
    """a = b + 3 c over 2^31 - 1 elements through the plugin path (hand kernel and generated code):
    the grid is 2^23 blocks of 256, the last three elements take the scalar tail of the hand kernel."""
    torch = torch_cuda
    from spoc_amd import reference_kernels
    n = N_MAX
    b = torch.full((n,), 1.0, device="cuda")
    c = torch.full((n,), 2.0, device="cuda")
    b[-1], c[-1], b[12345], c[n // 2] = 5.0, 0.5, -1.0, 4.0
    a = torch.full((n,), float("nan"), device="cuda")
    assert run_ir(hip, reference_kernels.stream_triad(), (256, 1, 1), ((n + 255) // 256, 1, 1),
                  [a, b, c, ("f32", 3.0), ("i32", n)], specialise) == tag
    assert float(a[-1]) == 6.5 and float(a[12345]) == 5.0 and float(a[n // 2]) == 13.0
    ordinary = (a == 7.0)
    assert int(ordinary.sum()) == n - 3
    del a, b, c, ordinary
    torch.cuda.empty_cache()


def test_histogram_at_the_largest_vector(hip, torch_cuda):
    torch = torch_cuda
    n = N_MAX
    keys = torch.arange(n, dtype=torch.int32, device="cuda")
    keys &= 255
    hist = torch.zeros(256, dtype=torch.int32, device="cuda")
    hip.histogram(keys, hist, 256)
    expected = np.full(256, n // 256, dtype=np.int64) + (np.arange(256) < n % 256)
    assert np.array_equal(hist.cpu().numpy().astype(np.int64), expected)
    del keys
    torch.cuda.empty_cache()


def test_radix_scatter_at_the_largest_vector(hip, torch_cuda):
    """One 8-bit pass over 2^31 - 1 keys: positions run up to 2^31 - 2, the counters end at the next
    digit's start, every range holds its digit, and the keys' sum, minimum and maximum are kept."""
    torch = torch_cuda
    n = N_MAX
    keys = torch.arange(n, dtype=torch.int32, device="cuda")
    keys *= -1640531535                                    # an odd multiplier: a bijection on 32 bits, mixes the low byte
    keys &= 0x7FFFFFFF
    hist = torch.zeros(256, dtype=torch.int32, device="cuda")
    hip.radix_histogram(keys, hist, 0, 255)
    counts = hist.cpu().numpy().astype(np.int64)
    assert counts.sum() == n
    starts = np.concatenate(([0], np.cumsum(counts)[:-1]))
    counters = torch.from_numpy(starts.astype(np.int32)).cuda()
    out = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    hip.radix_scatter(keys, out, counters, 0, 255)
    assert np.array_equal(counters.cpu().numpy().astype(np.int64), starts + counts)
    digits = out & 255
    assert bool((digits[1:] >= digits[:-1]).all())
    del digits
    assert int(out.sum(dtype=torch.int64)) == int(keys.sum(dtype=torch.int64))
    assert int(out.min()) >= 0 and int(out.max()) == int(keys.max())
    del keys, out
    torch.cuda.empty_cache()
