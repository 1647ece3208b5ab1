"""The five-point stencil and the 3 x 3 box filter of the reference's benches
(benchmarks/bench_stencil_2d.ml:43-58, bench_conv2d.ml:49-77): the hand kernels through the C ABI and the
kernels' IR through generate_source / run_source, against the CPU oracle bit for bit (the generated code, which
adds in binary32, to a few ulp)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (2, 9), (9, 2), (3, 3), (4, 3), (5, 7), (255, 9), (256, 8), (257, 33), (259, 5), (1000, 37),
          (1024, 64), (2048, 130), (4100, 17), (513, 1030), (1025, 40), (3, 300001), (260, 262150)]


def wide_range(rng, n):
    """Normal values over 16 decades: sums in binary32 would round differently from the double ones."""
    return (rng.standard_normal(n) * 10.0 ** rng.integers(-8, 8, n)).astype(np.float32)


def run_abi(hip, torch, which, x, w, h, offset=0, fill=-7.0):
    """The entry point on grids that start `offset` elements into their allocations, with 8 guard
    elements behind the output; returns (output, guards untouched)."""
    n = w * h
    din = torch.zeros(n + offset + 8, device="cuda")
    din[offset:offset + n] = torch.from_numpy(x).cuda()
    dout = torch.full((n + offset + 8,), fill, device="cuda")
    fn = hip.lib.sarek_hip_stencil_2d_f32 if which == "stencil" else hip.lib.sarek_hip_conv2d_f32
    hip.check(fn(din.data_ptr() + 4 * offset, dout.data_ptr() + 4 * offset, w, h, None))
    torch.cuda.synchronize()
    got = dout.cpu().numpy()
    return got[offset:offset + n], bool(np.all(got[:offset] == fill) and np.all(got[offset + n:] == fill))


@pytest.mark.parametrize("w,h", SHAPES)
@pytest.mark.parametrize("which", ["stencil", "conv"])
def test_kernels_match_the_oracle_bit_for_bit(hip, oracle, torch_cuda, which, w, h):
    x = wide_range(np.random.default_rng(w * 131 + h), w * h)
    for offset in (0, 1, 3):                       # 128-bit accesses at 4-byte alignment
        got, guards = run_abi(hip, torch_cuda, which, x, w, h, offset)
        if which == "stencil":
            ref = oracle.stencil_2d(x, w, h, out=np.full(w * h, -7.0, dtype=np.float32))
        else:
            ref = oracle.conv2d(x, w, h, out=np.full(w * h, -7.0, dtype=np.float32))
        assert guards
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (which, w, h, offset)


@pytest.mark.parametrize("rows", [1, 2, 5, 8, 32, 200])
@pytest.mark.parametrize("which", ["stencil", "conv"])
def test_any_band_height_gives_the_same_grid(hip, oracle, torch_cuda, which, rows):
    w, h = 777, 101
    x = wide_range(np.random.default_rng(rows), w * h)
    hip.set_tunable("stencil.rows", rows)
    try:
        got, guards = run_abi(hip, torch_cuda, which, x, w, h)
    finally:
        hip.set_tunable("stencil.rows", 0)
    ref = (oracle.stencil_2d if which == "stencil" else oracle.conv2d)(x, w, h, out=np.full(w * h, -7.0, dtype=np.float32))
    assert guards and np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_special_values_and_refusals(hip, oracle, torch_cuda):
    torch = torch_cuda
    w, h = 300, 40
    x = wide_range(np.random.default_rng(3), w * h)
    x[5 * w + 7], x[9 * w + 100], x[20 * w + 299], x[11 * w + 11] = np.nan, np.inf, -np.inf, -0.0
    x[30 * w + 50], x[30 * w + 51] = 3.0e38, 3.0e38          # their sum overflows binary32, not double
    for which, f in (("stencil", oracle.stencil_2d), ("conv", oracle.conv2d)):
        got, _ = run_abi(hip, torch, which, x, w, h)
        ref = f(x, w, h, out=np.full(w * h, -7.0, dtype=np.float32))
        assert np.array_equal(np.isnan(got), np.isnan(ref))
        ok = ~np.isnan(ref)
        assert np.array_equal(got[ok].view(np.uint32), ref[ok].view(np.uint32))
    d = torch.zeros(64, device="cuda")
    for fn in (hip.lib.sarek_hip_stencil_2d_f32, hip.lib.sarek_hip_conv2d_f32):
        assert fn(d.data_ptr(), d.data_ptr(), 8, 8, None) != 0            # in place
        assert fn(d.data_ptr(), d.data_ptr() + 4 * 8, 8, 4, None) != 0    # shifted overlap
        assert fn(None, d.data_ptr(), 8, 8, None) != 0
        assert fn(d.data_ptr(), d.data_ptr(), -1, 8, None) != 0
        assert fn(d.data_ptr(), d.data_ptr(), 0, 8, None) == 0            # an empty grid: nothing to do
        assert fn(d.data_ptr(), d.data_ptr() + 4 * 32, 1 << 16, 1 << 15, None) != 0   # 2^31 cells


def run_kernel_ir(hip, ir, block, grid, args, specialise):
    src = hip.generate_source(ir, block=block)
    hip.check(hip.lib.sarek_hip_set_specialisation(specialise))
    try:
        path = hip.run_source(src, "sarek_kern", block, grid, args)
        hip.check(hip.lib.sarek_hip_device_synchronize())
    finally:
        hip.check(hip.lib.sarek_hip_set_specialisation(1))
    return path


@pytest.mark.parametrize("specialise", [1, 0])
@pytest.mark.parametrize("w,h", [(100, 52), (256, 128), (17, 3), (333, 77)])
def test_ir_both_ways(hip, oracle, torch_cuda, specialise, w, h):
    from spoc_amd import reference_kernels
    torch = torch_cuda
    x = oracle.fill_uniform(w * h, seed=21, lo=-1, hi=1)
    dx = torch.from_numpy(x).cuda()
    cases = [("stencil_2d_f32", reference_kernels.stencil_2d(), (16, 16, 1), ((w + 15) // 16, (h + 15) // 16, 1),
              oracle.stencil_2d),
             ("conv2d_f32", reference_kernels.conv2d(), (256, 1, 1), ((w * h + 255) // 256, 1, 1), oracle.conv2d)]
    for tag, ir, block, grid, f in cases:
        out = torch.full((w * h,), -7.0, device="cuda")
        path = run_kernel_ir(hip, ir, block, grid, [dx, out, ("i32", w), ("i32", h)], specialise)
        assert path == (tag if specialise else "jit")
        ref = f(x, w, h, out=np.full(w * h, -7.0, dtype=np.float32))
        got = out.cpu().numpy()
        if specialise:
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
        else:                                      # binary32 sums of values in [-1, 1): a few ulp of 1
            assert np.abs(got - ref).max() <= 1e-6


def test_launches_the_hand_kernels_do_not_serve(hip, oracle, torch_cuda):
    """A launch that does not reach every cell, grids that overlap, vectors shorter than the grid: the generated
    code runs, and computes what the oracle computes for that launch."""
    from spoc_amd import reference_kernels
    torch = torch_cuda
    w, h = 64, 48
    x = oracle.fill_uniform(w * h, seed=22, lo=-1, hi=1)
    dx = torch.from_numpy(x).cuda()
    st, cv = reference_kernels.stencil_2d(), reference_kernels.conv2d()
    out = torch.full((w * h,), -7.0, device="cuda")
    assert run_kernel_ir(hip, st, (16, 16, 1), (4, 2, 1), [dx, out, ("i32", w), ("i32", h)], 1) == "jit"   # 32 of 48 rows
    ref = oracle.stencil_2d(x, w, h, out=np.full(w * h, -7.0, dtype=np.float32), threads_xy=(64, 32))
    assert np.abs(out.cpu().numpy() - ref).max() <= 1e-6
    out.fill_(-7.0)
    assert run_kernel_ir(hip, cv, (256, 1, 1), (5, 1, 1), [dx, out, ("i32", w), ("i32", h)], 1) == "jit"    # 1280 of 3072 cells
    ref = oracle.conv2d(x, w, h, out=np.full(w * h, -7.0, dtype=np.float32), threads=1280)
    assert np.abs(out.cpu().numpy() - ref).max() <= 1e-6
    # a 1-D launch of the 2-D kernel reaches row 0 only: nothing is interior
    out.fill_(-7.0)
    assert run_kernel_ir(hip, st, (256, 1, 1), (12, 1, 1), [dx, out, ("i32", w), ("i32", h)], 1) == "jit"
    assert bool((out == -7.0).all())
    both = torch.zeros(w * h + w, device="cuda")
    assert run_kernel_ir(hip, cv, (256, 1, 1), (12, 1, 1), [both[:w * h], both[w:], ("i32", w), ("i32", h)], 1) == "jit"
    assert run_kernel_ir(hip, st, (16, 16, 1), (4, 3, 1), [dx[:w * h - 1], out, ("i32", w), ("i32", h)], 1) == "jit"
    # and a launch larger than the grid is served
    assert run_kernel_ir(hip, st, (16, 16, 1), (5, 4, 1), [dx, out, ("i32", w), ("i32", h)], 1) == "stencil_2d_f32"
    assert run_kernel_ir(hip, cv, (256, 1, 1), (13, 1, 1), [dx, out, ("i32", w), ("i32", h)], 1) == "conv2d_f32"
