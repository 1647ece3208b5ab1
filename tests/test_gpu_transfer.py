"""Host <-> device copies through the C ABI (Memory.host_ptr_to_device / device_to_host_ptr,
sarek/core/Transfer.ml:228-333): byte-exact round trips, with the pinned-staging pipeline
and the plain driver copy checked against each other, and the ordering the reference relies
on (a copy issued right after a launch sees that launch's result)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MIB = 1 << 20


@pytest.fixture
def hip():
    from spoc_amd import hip as h
    h.set_tunable("transfer.min_up_kib", 0)       # every copy of 2 MiB and more takes the staged path
    h.set_tunable("transfer.min_down_kib", 0)
    yield h
    for name, value in (("transfer.threads", 4), ("transfer.chunk_kib", 8192),
                        ("transfer.min_up_kib", 12288), ("transfer.min_down_kib", 2048)):
        h.set_tunable(name, value)


def _pattern(nbytes, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 256, size=nbytes, dtype=np.uint8)


def _round_trip(hip, host, up_threads, down_threads):
    """Upload `host`, download into a fresh block, with the given thread counts
    (0 = the driver's own copy); returns the downloaded bytes."""
    dptr = hip.mem_alloc(host.nbytes)
    try:
        hip.set_tunable("transfer.threads", up_threads)
        hip.memcpy_htod(dptr, host)
        back = np.full(host.shape, 0xA5, dtype=np.uint8)
        hip.set_tunable("transfer.threads", down_threads)
        hip.memcpy_dtoh(back, dptr)
    finally:
        hip.mem_free(dptr)
    return back


@pytest.mark.parametrize("nbytes", [0, 1, 4097, 2 * MIB - 1, 2 * MIB, 2 * MIB + 1, 5 * MIB + 3,
                                    16 * MIB - 3, 16 * MIB, 24 * MIB + 5, 100 * MIB + 7, 300 * MIB + 1])
def test_round_trip_sizes(hip, nbytes):
    host = _pattern(nbytes, nbytes % 1000)
    # staged up / plain down, plain up / staged down, staged both ways
    for up, down in ((4, 0), (0, 4), (4, 4)):
        back = _round_trip(hip, host, up, down)
        assert np.array_equal(back, host), (nbytes, up, down)


def test_unaligned_host_block(hip):
    base = _pattern(40 * MIB + 64, 7)
    for shift in (1, 3, 13):
        host = base[shift:shift + 40 * MIB + 11]
        assert host.ctypes.data % 4 != 0 or shift % 4 == 0
        assert np.array_equal(_round_trip(hip, host, 4, 4), host)


@pytest.mark.parametrize("threads,chunk_kib", [(1, 8192), (3, 1024), (8, 2048), (16, 4096)])
def test_pool_shapes(hip, threads, chunk_kib):
    hip.set_tunable("transfer.chunk_kib", chunk_kib)
    host = _pattern(19 * MIB + 123, threads)
    assert np.array_equal(_round_trip(hip, host, threads, threads), host)
    # fewer chunks than threads
    small = _pattern(2 * chunk_kib * 1024 + 5, 99)
    assert np.array_equal(_round_trip(hip, small, threads, threads), small)


def test_copy_is_ordered_after_launches(hip):
    """Transfer.to_cpu right after Execute.run (no flush between them in
    sarek/core/Vector.ml:80-96 -> ensure_cpu_sync): the download must see the kernel's result,
    and an upload into a vector the kernel still reads must not overtake it."""
    import torch
    n = 64 * MIB // 4                     # 64 MiB per vector: staged path
    b = torch.arange(n, dtype=torch.float32, device="cuda") % 1024
    c = torch.ones(n, dtype=torch.float32, device="cuda")
    a = torch.zeros(n, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    fresh = np.full(n, 7.0, dtype=np.float32)
    got = np.empty(n, dtype=np.float32)
    for _ in range(3):
        a.zero_()
        hip.triad(b, c, 2.0, out=a)                       # a = b + 2 c, asynchronous
        hip.memcpy_dtoh(got.view(np.uint8), a.data_ptr())
        assert np.array_equal(got, (np.arange(n) % 1024 + 2.0).astype(np.float32))
        hip.triad(b, c, 3.0, out=a)                       # reads c ...
        hip.memcpy_htod(c.data_ptr(), fresh.view(np.uint8))   # ... which is replaced right behind it
        torch.cuda.synchronize()
        assert torch.equal(a, b + 3.0)
        assert torch.equal(c, torch.full_like(c, 7.0))
        c.fill_(1.0)
        torch.cuda.synchronize()


def test_pinned_host_block(hip):
    n = 6 * MIB
    with hip.pinned_array(n, np.float32) as host:
        host[:] = np.arange(n, dtype=np.float32)
        dptr = hip.mem_alloc(host.nbytes)
        try:
            hip.memcpy_htod(dptr, host.view(np.uint8))
            with hip.pinned_array(n, np.float32) as back:
                back[:] = -1
                hip.memcpy_dtoh(back.view(np.uint8), dptr)
                assert np.array_equal(back, host)
            # pinned up, pageable down
            page = np.empty(n, dtype=np.float32)
            hip.memcpy_dtoh(page.view(np.uint8), dptr)
            assert np.array_equal(page, host)
        finally:
            hip.mem_free(dptr)
    hip.check(hip.lib.sarek_hip_host_free(None))
    empty = hip.pinned_array(0, np.uint8)
    assert empty.array.size == 0
    empty.close()


def test_null_pointers_are_rejected(hip):
    import ctypes as C
    host = np.zeros(16, dtype=np.uint8)
    assert hip.lib.sarek_hip_memcpy_htod(None, C.c_void_p(host.ctypes.data), 16) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_memcpy_dtoh(C.c_void_p(host.ctypes.data), None, 16) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_memcpy_htod(None, None, 0) == 0
    assert hip.lib.sarek_hip_host_alloc(None, 16) == hip.E_INVALID_ARG
