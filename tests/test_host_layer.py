"""Vector / Transfer / Execute above the plugin boundary (sarek/core/Vector.ml,
sarek/core/Transfer.ml, sarek/sarek/Execute.ml): host-only behaviour on the CPU, the location
state machine and the dispatcher on the GPU, each step checked against what the reference's
code does in that state."""
import numpy as np
import pytest

from spoc_amd import reference_kernels
from spoc_amd.sarek import CPU, Both, Device, Execute, Stale_CPU, Stale_GPU, Transfer, Vector

gpu = pytest.mark.gpu


# ---- host only --------------------------------------------------------------------------------

def test_create_get_set_and_bounds():
    v = Vector.create(Vector.float32, 10)
    assert v.length == 10 and len(v) == 10 and v.kind is Vector.float32 and v.location == CPU
    for i in range(10):
        v[i] = i * 0.5                                    # Vector.set
    assert v.location == CPU                              # a host-only vector stays CPU (Vector.ml:104-109)
    assert v[3] == np.float32(1.5) and v.get(9) == np.float32(4.5)
    assert np.array_equal(v.to_array(), np.arange(10, dtype=np.float32) * 0.5)
    with pytest.raises(IndexError, match=r"Vector.get: index 10 out of bounds \[0, 10\)"):      # Vector.ml:82-88
        v.get(10)
    with pytest.raises(IndexError, match=r"Vector.set: index -1 out of bounds \[0, 10\)"):      # Vector.ml:97-103
        v.set(-1, 0.0)
    with pytest.raises(IndexError):
        v.fill_from(np.zeros(4), first=8)
    v.destroy()
    v.destroy()                                           # idempotent, like the GC finaliser after an explicit free


@pytest.mark.parametrize("kind,size,value", [
    (Vector.float32, 4, 1.25), (Vector.float64, 8, 1e-300), (Vector.int32, 4, -7), (Vector.int64, 8, 1 << 40),
    (Vector.char, 1, 200), (Vector.complex32, 8, 1 + 2j)])
def test_kinds_and_element_sizes(kind, size, value):
    from spoc_amd import hip
    v = Vector.create(kind, 3)
    assert hip.lib.sarek_hip_vector_elem_size(v._h) == size      # Vector_types.scalar_elem_size
    v[1] = value
    assert v[1] == kind.dtype.type(value)
    assert v.host.dtype == kind.dtype and v.host.size == 3


def test_custom_and_empty_vectors_and_bad_arguments():
    from spoc_amd import hip
    c = Vector.create_custom(12, 5)
    assert hip.lib.sarek_hip_vector_elem_size(c._h) == 12 and c.host.nbytes == 60
    e = Vector.create(Vector.int32, 0)
    assert e.length == 0 and e.to_array().size == 0
    with pytest.raises(hip.SarekHipError):
        Vector.create(Vector.float32, -1)
    with pytest.raises(hip.SarekHipError):
        Vector.create_custom(0, 4)


def test_of_array_writes_the_host_block_directly():
    x = np.arange(6, dtype=np.int32)
    v = Vector.of_array(x)
    assert v.kind is Vector.int32 and v.location == CPU and np.array_equal(v.to_array(), x)


# ---- the location state machine on the device ---------------------------------------------------

@gpu
def test_location_walk(torch_cuda):
    n = 1000
    v = Vector.create(Vector.float32, n)
    v.fill_from(np.arange(n))
    assert v.location == CPU and v.device_ptr is None
    Transfer.to_device(v)                                  # CPU -> Both (Transfer.ml:245-268)
    assert v.location == Both and v.device_ptr is not None
    ptr = v.device_ptr
    v.host[0] = -1.0                                       # behind the vector's back: nothing is tracked
    Transfer.to_device(v)                                  # Both: skipped (Transfer.ml:241-243)
    assert v.location == Both and v.device_ptr == ptr
    Transfer.to_cpu(v)                                     # Both without force: nothing moves (:289)
    assert v.host[0] == -1.0
    Transfer.to_cpu(v, force=True)                         # forced: the device copy comes back
    assert v.host[0] == 0.0 and v.location == Both
    v[5] = 55.0                                            # Vector.set on Both -> Stale_GPU (Vector.ml:106-107)
    assert v.location == Stale_GPU
    Transfer.to_cpu(v)                                     # Stale_GPU: the host copy is the good one (:290)
    assert v[5] == 55.0 and v.location == Stale_GPU
    Transfer.to_device(v)                                  # Stale_GPU -> upload again -> Both
    assert v.location == Both
    Transfer.to_cpu(v, force=True)
    assert v[5] == 55.0
    Transfer.free_all_buffers(v)                           # Transfer.ml:371-381
    assert v.location == CPU and v.device_ptr is None and v[5] == 55.0


@gpu
def test_device_buffers_are_tracked_as_the_reference_tracks_them(torch_cuda):
    """Transfer.ensure_buffer -> Gpu_memory.track_alloc (Transfer.ml:218); free_all_buffers -> track_free (:375); a
    vector that goes away with a buffer -> the finaliser's gc_free_count / gc_freed_bytes (Gpu_memory.ml:163-178)."""
    import gc
    from spoc_amd.sarek import GpuMemory
    gc.collect()                                           # vectors of earlier tests go now, not in the middle of this one
    GpuMemory.reset_stats()
    v = Vector.create(Vector.float32, 1000)
    w = Vector.create(Vector.int64, 500)
    Transfer.to_device(v)
    Transfer.to_device(v)                                  # the buffer is there: nothing new
    Transfer.to_device(w)
    s = GpuMemory.stats()
    assert (s.current_bytes, s.peak_bytes, s.alloc_count, s.free_count) == (8000, 8000, 2, 0)
    Transfer.free_all_buffers(v)
    s = GpuMemory.stats()
    assert (s.current_bytes, s.peak_bytes, s.alloc_count, s.free_count, s.gc_free_count) == (4000, 8000, 2, 1, 0)
    w.destroy()                                            # what a finaliser does
    s = GpuMemory.stats()
    assert (s.current_bytes, s.free_count, s.gc_free_count, s.gc_freed_bytes) == (0, 1, 1, 4000)
    v.destroy()                                            # no buffer left: nothing to count
    assert GpuMemory.stats().gc_free_count == 1 and GpuMemory.usage() == 0
    # a sub-vector's buffer is its own share
    parent = Vector.create(Vector.float32, 100)
    sub = parent.sub_vector(10, 20)
    Transfer.to_device(sub)
    assert GpuMemory.usage() == 80
    Transfer.free_all_buffers(sub)
    assert GpuMemory.usage() == 0


@gpu
def test_launch_marks_stale_and_reads_download(torch_cuda):
    n = 100003
    b, c = Vector.create(Vector.float32, n), Vector.create(Vector.float32, n)
    a = Vector.create(Vector.float32, n)
    b.fill_from(np.arange(n) % 100 / 100.0)
    c.fill_from((np.arange(n) + 1) % 100 / 100.0)
    ir = reference_kernels.stream_triad()
    args = [Execute.Vec(a), Execute.Vec(b), Execute.Vec(c), Execute.Float32(3.0), Execute.Int(n)]
    block, grid = Execute.dims1d(256), Execute.dims1d((n + 255) // 256)
    path = Execute.run_vectors(ir=ir, args=args, block=block, grid=grid)
    assert path == "stream_triad_f32"
    # every vector argument was uploaded (Both) and is now Stale_CPU, inputs included (Execute.ml:321-335)
    assert a.location == b.location == c.location == Stale_CPU
    Transfer.flush()
    expected = (b.host.astype(np.float64) + 3.0 * c.host.astype(np.float64)).astype(np.float32)
    assert a[7] == expected[7]                             # Vector.get downloads (ensure_cpu_sync) ...
    assert a.location == Both                              # ... and leaves Both (Transfer.ml:322)
    assert np.array_equal(a.to_array(), expected)
    # second launch: nothing to upload, same buffers
    pa, pb = a.device_ptr, b.device_ptr
    Execute.run_vectors(ir=ir, args=args, block=block, grid=grid)
    assert (a.device_ptr, b.device_ptr) == (pa, pb) and a.location == Stale_CPU
    assert b.location == Stale_CPU                         # b was never read back, so it was not Both: unchanged
    # a host write into a Stale_CPU vector is not tracked and is lost at the next download
    b[0] = 123.0
    assert b.location == Stale_CPU                         # Vector.ml:108-109
    Transfer.to_cpu(b)
    assert b[0] == np.float32(0.0) and b.location == Both
    # after a tracked write the next launch uploads again
    c[0] = 0.5
    assert c.location == Stale_CPU                         # still never synced: Stale_CPU stays
    Transfer.to_cpu(c)
    c[0] = 0.5
    assert c.location == Stale_GPU
    Execute.run_vectors(ir=ir, args=args, block=block, grid=grid)
    assert c.location == Stale_CPU and a[0] == np.float32(b[0] + 3.0 * 0.5)


@gpu
def test_auto_sync_switches(torch_cuda):
    n = 4096
    x, y = Vector.create(Vector.float32, n), Vector.create(Vector.float32, n)
    x.fill_from(np.ones(n))
    y.fill_from(np.zeros(n))
    args = [Execute.Vec(x), Execute.Vec(y), Execute.Int(n)]
    Execute.run_vectors(ir=reference_kernels.vector_copy(), args=args, block=(256, 1, 1), grid=(16, 1, 1))
    Transfer.flush()
    try:
        Transfer.set_auto(False)                           # Transfer.auto_mode off: reads see the stale block
        assert y[0] == 0.0 and y.location == Stale_CPU
        Transfer.set_auto(True)
        y.set_auto_sync(False)                             # per-vector switch (Vector_types.auto_sync)
        assert y[0] == 0.0 and y.location == Stale_CPU
        y.set_auto_sync(True)
        assert y[0] == 1.0 and y.location == Both
    finally:
        Transfer.set_auto(True)
    Execute.run_vectors(ir=reference_kernels.vector_copy(), args=args, block=(256, 1, 1), grid=(16, 1, 1))
    Execute.sync_vectors_to_cpu(args)                      # Execute.ml:546-547
    assert x.location == Both and y.location == Both
    Transfer.sync(y)
    assert y.location == Both


@gpu
def test_run_source_external_kernel_with_and_without_lengths(torch_cuda):
    """sarek/tests/e2e/test_external_kernel.ml:46-62: a hand-written kernel through Execute.run_source."""
    n = 1000
    a, b, c = (Vector.create(Vector.float32, n) for _ in range(3))
    a.fill_from(np.arange(n))
    b.fill_from(np.arange(n) * 2)
    with_len = ('extern "C" __global__ void vadd(const float* a, int al, const float* b, int bl, float* c, int cl, int n) '
                '{ int i = threadIdx.x + blockIdx.x * blockDim.x; if (i < n && i < cl) c[i] = a[i] + b[i]; }')
    bare = ('extern "C" __global__ void vadd(const float* a, const float* b, float* c, int n) '
            '{ int i = threadIdx.x + blockIdx.x * blockDim.x; if (i < n) c[i] = a[i] + b[i] + 1.0f; }')
    args = [Execute.Vec(a), Execute.Vec(b), Execute.Vec(c), Execute.Int32(n)]
    assert Execute.run_source(with_len, "vadd", (256, 1, 1), (4, 1, 1), args) == "jit"
    assert c.location == Stale_CPU and np.array_equal(c.to_array(), np.arange(n, dtype=np.float32) * 3)
    Execute.run_source(bare, "vadd", (256, 1, 1), (4, 1, 1), args, inject_lengths=False)
    assert np.array_equal(c.to_array(), np.arange(n, dtype=np.float32) * 3 + 1)
    from spoc_amd import hip
    # Execute.run_source refuses the language itself (Execute.ml:622-633); below it, the plugin's
    # run_source has its own refusal (Cuda_plugin.ml:211-220)
    with pytest.raises(hip.SarekHipError, match="Unsupported argument type PTX in HIP backend"):
        Execute.run_source(bare, "vadd", (256, 1, 1), (4, 1, 1), args, lang=hip.LANG_PTX)
    with pytest.raises(hip.SarekHipError, match="does not support PTX"):
        hip.run_source(bare, "vadd", (256, 1, 1), (4, 1, 1), [], lang=hip.LANG_PTX)


@gpu
def test_lowering_failure_and_pinned_vectors(torch_cuda):
    from spoc_amd import hip
    v = Vector.create(Vector.float32, 8, pinned=True)
    v.fill_from(np.arange(8))
    with pytest.raises(hip.SarekHipError, match="Backend failed to generate source"):      # Execute.ml:257-263
        Execute.run_vectors(ir="(kernel k (params) (locals) (body (frob)))", args=[Execute.Vec(v)],
                            block=(1, 1, 1), grid=(1, 1, 1))
    assert v.location == Both                              # the upload had happened before the lowering failed
    big = Vector.create(Vector.float32, 1 << 22, pinned=True)
    big.fill_from(np.arange(1 << 22) % 977)
    out = Vector.create(Vector.float32, 1 << 22, pinned=True)
    Execute.run_vectors(ir=reference_kernels.vector_copy(), args=[Execute.Vec(big), Execute.Vec(out), Execute.Int(1 << 22)],
                        block=(256, 1, 1), grid=((1 << 22) // 256, 1, 1))
    assert np.array_equal(out.to_array(), big.host)


@gpu
def test_zero_copy_vectors(torch_cuda):
    """Memory.alloc_zero_copy returning Some (sarek/core/Transfer.ml:85-126, 185-203): the device
    buffer is the host block; transfers move nothing; the location states change as usual."""
    from spoc_amd import hip
    n = 1 << 20
    b = Vector.create(Vector.float32, n, zero_copy=True)
    c = Vector.create(Vector.float32, n, zero_copy=True)
    a = Vector.create(Vector.float32, n, zero_copy=True)
    b.fill_from(np.arange(n) % 100 / 100.0)
    c.fill_from((np.arange(n) + 1) % 100 / 100.0)
    a.host[:] = -1.0
    args = [Execute.Vec(a), Execute.Vec(b), Execute.Vec(c), Execute.Float32(3.0), Execute.Int(n)]
    path = Execute.run_vectors(ir=reference_kernels.stream_triad(), args=args, block=(256, 1, 1),
                               grid=((n + 255) // 256, 1, 1))
    assert path == "stream_triad_f32" and a.location == Stale_CPU
    host_addr = a.host.ctypes.data
    assert a.device_ptr is not None
    expected = (b.host.astype(np.float64) + 3.0 * c.host.astype(np.float64)).astype(np.float32)
    assert np.array_equal(a.to_array(), expected)           # to_array waits for the kernel; nothing is copied
    assert a.location == Both and a.host.ctypes.data == host_addr and np.array_equal(a.host, expected)
    # a host write is seen by the next launch without an upload
    b[0] = 10.0
    assert b.location == Stale_CPU or b.location == Stale_GPU
    Transfer.to_cpu(b)
    b[0] = 10.0
    Execute.run_vectors(ir=reference_kernels.stream_triad(), args=args, block=(256, 1, 1), grid=((n + 255) // 256, 1, 1))
    assert a[0] == np.float32(10.0 + 3.0 * c.host[0])
    # alloc_zero_copy itself: None for ordinary memory, a device view for pinned blocks
    ordinary = np.zeros(16, dtype=np.float32)
    import ctypes as C
    dptr, ok = C.c_void_p(), C.c_int(-1)
    hip.check(hip.lib.sarek_hip_mem_alloc_zero_copy(C.c_void_p(ordinary.ctypes.data), 64, C.byref(dptr), C.byref(ok)))
    assert ok.value == 0 and dptr.value is None
    with hip.pinned_array(16, np.float32) as pinned:
        hip.check(hip.lib.sarek_hip_mem_alloc_zero_copy(C.c_void_p(pinned.ctypes.data), 64, C.byref(dptr), C.byref(ok)))
        assert ok.value == 1 and dptr.value is not None
        hip.check(hip.lib.sarek_hip_mem_free(dptr))          # a view needs no free; freeing it is harmless


# ---- the rest of the Vector module: ids, printing, fill / copy / blit, sub-vectors ----------------

def test_ids_printing_fill_copy_init():
    a, b = Vector.create(Vector.float32, 8), Vector.create(Vector.int64, 3)
    assert b.id == a.id + 1 and a.id >= 1                  # Vector_storage.next_id
    assert str(a) == f"Vector#{a.id}<Float32>[8] @ CPU" and str(b) == f"Vector#{b.id}<Int64>[3] @ CPU"
    assert str(Vector.create_custom(12, 5)).endswith("<Custom(12)>[5] @ CPU")
    a.fill(2.5)
    assert a.location == CPU and np.array_equal(a.to_array(), np.full(8, 2.5, dtype=np.float32))
    c = a.copy()
    c[0] = 7.0
    assert a[0] == 2.5 and c.id > b.id and c.location == CPU and len(c) == 8
    sq = Vector.init(Vector.int32, 6, lambda i: i * i)
    assert sq.to_array().tolist() == [0, 1, 4, 9, 16, 25]
    assert a.is_on_cpu and not a.is_on_gpu and not a.is_synced and not a.needs_gpu_update and not a.needs_cpu_update


def test_sub_vectors_share_the_host_block():
    v = Vector.init(Vector.float32, 10, float)
    s = v.sub_vector(3, 4)
    assert (len(s), s.is_sub, s.depth, s.parent_id, s.sub_start, s.sub_ok_range, s.sub_ko_range) == (4, True, 1, v.id, 3, 4, 0)
    assert (v.is_sub, v.depth, v.parent_id, v.sub_start) == (False, 0, None, None)
    assert s.to_array().tolist() == [3, 4, 5, 6] and s.location == CPU
    s[1] = -4.0                                            # one block: the parent sees it
    v[6] = -6.0
    assert v[4] == -4.0 and s[3] == -6.0
    g = s.sub_vector(1, 2, ok_range=1, ko_range=1)          # grandchild: start is relative to its parent
    assert (g.depth, g.parent_id, g.sub_start, g.sub_ok_range, g.sub_ko_range) == (2, s.id, 1, 1, 1)
    assert g.to_array().tolist() == [-4.0, 5.0]
    for start, length in ((-1, 2), (8, 3), (0, 11)):
        with pytest.raises(IndexError, match=r"sub_vector: range \[-?\d+, \d+\) out of bounds \[0, 10\)"):
            v.sub_vector(start, length)
    assert len(v.sub_vector(10, 0)) == 0
    # the block outlives the parent while a view exists
    v.destroy()
    s.destroy()
    assert g.to_array().tolist() == [-4.0, 5.0]


def test_partition_and_blit():
    v = Vector.init(Vector.int32, 10, int)
    parts = v.partition([0, 0, 0])                          # Vector_storage.partition_host: 4, 3, 3
    assert [len(p) for p in parts] == [4, 3, 3] and [p.sub_start for p in parts] == [0, 4, 7]
    assert all(p.location == Stale_GPU and p.needs_gpu_update and p.depth == 1 for p in parts)
    assert np.concatenate([p.to_array() for p in parts]).tolist() == list(range(10))
    assert v.partition([]) == []
    even = Vector.init(Vector.int32, 7, int).partition([0] * 7)
    assert [len(p) for p in even] == [1] * 7
    w = Vector.create(Vector.int32, 6)
    w.fill(0)
    Vector.blit(v, 2, w, 1, 4)
    assert w.to_array().tolist() == [0, 2, 3, 4, 5, 0]
    Vector.blit(v, 0, v, 1, 5)                               # ascending element order smears the first element
    assert v.to_array().tolist() == [0, 0, 0, 0, 0, 0, 6, 7, 8, 9]
    with pytest.raises(IndexError, match="Vector.blit: source range out of bounds"):
        Vector.blit(v, 8, w, 0, 3)
    with pytest.raises(IndexError, match="Vector.blit: destination range out of bounds"):
        Vector.blit(v, 0, w, 4, 3)


@gpu
def test_fill_copy_blit_follow_the_location(torch_cuda):
    n = 5000
    v = Vector.init(Vector.float32, n, float)
    Transfer.to_device(v)
    assert str(v).startswith(f"Vector#{v.id}<Float32>[{n}] @ Both(") and v.is_synced and v.is_on_gpu and v.is_on_cpu
    v.fill(1.0)                                            # Both -> Stale_GPU (Vector.ml:230-233)
    assert v.location == Stale_GPU
    ir = reference_kernels.vector_add()
    out = Vector.create(Vector.float32, n)
    Execute.run_vectors(ir=ir, args=[Execute.Vec(v), Execute.Vec(v), Execute.Vec(out), Execute.Int(n)],
                        block=Execute.dims1d(256), grid=Execute.dims1d((n + 255) // 256))
    assert out.location == Stale_CPU and out.needs_cpu_update and not out.is_on_cpu
    c = out.copy()                                         # downloads first (ensure_cpu_sync), host data only
    assert out.location == Both and c.location == CPU and c.device_ptr is None
    assert np.array_equal(c.to_array(), np.full(n, 2.0, dtype=np.float32))
    # a fill of a Stale_CPU vector is not tracked: the download that follows wins
    Execute.run_vectors(ir=ir, args=[Execute.Vec(v), Execute.Vec(v), Execute.Vec(out), Execute.Int(n)],
                        block=Execute.dims1d(256), grid=Execute.dims1d((n + 255) // 256))
    out.fill(9.0)
    assert out.location == Stale_CPU and out[0] == 2.0
    # blit: the source is downloaded first, the destination becomes Stale_GPU
    Execute.run_vectors(ir=ir, args=[Execute.Vec(v), Execute.Vec(out), Execute.Vec(out), Execute.Int(n)],
                        block=Execute.dims1d(256), grid=Execute.dims1d((n + 255) // 256))
    assert out.location == Stale_CPU
    Transfer.to_device(c)
    Vector.blit(out, 0, c, 10, 5)
    assert out.location == Both and c.location == Stale_GPU and c.to_array()[8:16].tolist() == [2, 2, 3, 3, 3, 3, 3, 2]


@gpu
@pytest.mark.parametrize("zero_copy", [False, True])
def test_kernels_on_sub_vectors_and_partitions(torch_cuda, zero_copy):
    """A launch on a sub-vector uploads, computes and downloads that range only; the parts of a
    partition together rebuild the parent on the host (the reference's multi-device pattern, here
    with every part on the one device)."""
    n = 100_000
    v = Vector.create(Vector.float32, n, zero_copy=zero_copy)
    v.fill_from(np.arange(n))
    mid = v.sub_vector(1000, 50_000)
    out = Vector.create(Vector.float32, 50_000)
    ir = reference_kernels.vector_add()
    Execute.run_vectors(ir=ir, args=[Execute.Vec(mid), Execute.Vec(mid), Execute.Vec(out), Execute.Int(50_000)],
                        block=Execute.dims1d(256), grid=Execute.dims1d(196))
    assert v.location == CPU and mid.location == Stale_CPU and v.device_ptr is None
    assert np.array_equal(out.to_array(), 2 * np.arange(1000, 51_000, dtype=np.float32))
    parts = v.partition([0, 0, 0])
    for p in parts:                                        # p <- p + p, in place, part by part
        Execute.run_vectors(ir=ir, args=[Execute.Vec(p), Execute.Vec(p), Execute.Vec(p), Execute.Int(len(p))],
                            block=Execute.dims1d(256), grid=Execute.dims1d((len(p) + 255) // 256))
    assert all(p.location == Stale_CPU for p in parts)
    Transfer.to_cpu_all(parts)                             # downloads land in the parent's block
    assert all(p.location == Both for p in parts)
    assert np.array_equal(v.host, 2 * np.arange(n, dtype=np.float32))
    Transfer.sync_all(parts)
    Transfer.to_device_all(parts)


@gpu
def test_streams(torch_cuda):
    s = Transfer.create_stream()
    assert s.value
    Transfer.synchronize_stream(s)
    Transfer.destroy_stream(s)
    d = Transfer.default_stream()
    Transfer.synchronize_stream(d)
    Transfer.destroy_stream(d)                             # a no-op, as in the reference


# ---- external kernels from files (Execute.ml:589-593, 654-726) ------------------------------------

def test_detect_lang_and_grid_helpers():
    from spoc_amd import hip
    assert Execute.detect_lang("k/optimized.cu") == hip.LANG_CUDA and Execute.detect_lang("a.hip") == hip.LANG_HIP
    assert [Execute.detect_lang("x" + e) for e in (".cl", ".ptx", ".spv", ".comp", ".glsl")] == \
        [hip.LANG_OPENCL, hip.LANG_PTX, hip.LANG_SPIRV, hip.LANG_GLSL, hip.LANG_GLSL]
    with pytest.raises(ValueError, match=r"Invalid file k.txt: Unknown source file extension \(expected .cu, .cl"):
        Execute.detect_lang("k.txt")
    assert Execute.supports_lang(hip.LANG_HIP) and Execute.supports_lang(hip.LANG_CUDA)
    assert not any(Execute.supports_lang(x) for x in (hip.LANG_OPENCL, hip.LANG_PTX, hip.LANG_SPIRV, hip.LANG_GLSL))
    assert Execute.grid_for_size(1000, 256) == 4 and Execute.grid_for(1024, 256) == (4, 1, 1)


@gpu
def test_run_source_file(torch_cuda, tmp_path):
    from spoc_amd import hip
    n = 3000
    src = 'extern "C" __global__ void scale(float* x, int len, float f) {\n' \
          '  int i = blockIdx.x * blockDim.x + threadIdx.x;\n  if (i < len) x[i] *= f;\n}\n'
    for name in ("scale.cu", "scale.hip"):
        path = tmp_path / name
        path.write_text(src)
        v = Vector.init(Vector.float32, n, float)
        assert Execute.run_source_file(path, "scale", Execute.dims1d(256), Execute.grid_for(n, 256),
                                       [Execute.Vec(v), Execute.Float32(0.5)]) == "jit"
        assert v.location == Stale_CPU and np.array_equal(v.to_array(), np.arange(n, dtype=np.float32) * 0.5)
    cl = tmp_path / "scale.cl"
    cl.write_text(src)
    v = Vector.init(Vector.float32, n, float)
    with pytest.raises(hip.SarekHipError, match="Unsupported argument type OpenCL source in HIP backend"):
        Execute.run_source_file(cl, "scale", Execute.dims1d(256), Execute.grid_for(n, 256), [Execute.Vec(v)])
    assert v.location == Both                              # uploaded before the language is checked (Execute.ml:618-633)
    with pytest.raises(hip.SarekHipError, match="No such file"):
        Execute.run_source_file(tmp_path / "none.cu", "scale", Execute.dims1d(1), Execute.dims1d(1), [])


# ---- Device (sarek/core/Device.ml) ------------------------------------------------------------------

def test_device_enumeration_without_a_gpu_gives_no_devices():
    Device.reset()
    devs = Device.init()                                   # never raises (Framework_registry.ml:77-87)
    assert Device.count() == len(devs) and Device.get(len(devs)) is None and Device.get(-1) is None
    assert Device.by_framework("CUDA") == [] and Device.by_framework("HIP") == devs
    assert (Device.first() is None) == (len(devs) == 0)


@gpu
def test_device_capabilities(torch_cuda):
    Device.reset()
    d = Device.best()
    assert d is not None and d.id == 0 and d.framework == "HIP" and d.is_gpu and not d.is_cpu
    assert d.warp_size == 64 and d.multiprocessor_count == 256 and d.max_threads_per_block == 1024
    assert d.allows_fp64 and d.supports_atomics and d.shared_mem_per_block >= 64 * 1024
    assert d.max_registers_per_block >= 65536 and d.total_memory > 200 * 2 ** 30 and d.arch.startswith("gfx950")
    assert 0 < d.free_memory() <= d.total_memory
    text = d.to_string()
    assert text.startswith(f"[0] {d.name} (HIP) - SM ") and text.endswith("GB, 256 MPs")
    d.synchronize()
