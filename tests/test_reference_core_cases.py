"""The reference's own device-free unit tests of the layers either side of a launch, case by case, on the native
Vector / Transfer / Execute / Gpu_memory layer (spoc_amd.sarek over the C ABI):

  sarek/core/test/test_vector.ml:15-375          46 cases: kinds, creation, location, element access, fill / init,
                                                 copy, conversions, iterators, folds, predicates, aggregates,
                                                 sub-vectors, blit, printing, the auto-sync flag, ids
  sarek/core/test/test_vector_storage.ml:13-65   copy of host data, sub-vector metadata, partition over three devices
  sarek/core/test/test_vector_transfer.ml:29-38  the host pointer of a vector's block (the sync-callback case wires an
                                                 OCaml closure into Vector.ensure_cpu_sync: here the download is the
                                                 library's own, tests/test_host_layer.py::test_launch_marks_stale_...)
  sarek/tests/unit/test_execute.ml:13-96         argument constructors, dims1d/2d/3d, grid_for_size, vectors as arguments
  sarek/core/test/test_gpu_memory.ml:10-108      the auto_gc flag, usage tracking, with_retry (first try, one retry,
                                                 three failures, retry switched off), trigger_gc, stats, reset_stats

None of them needs a device, there or here.  A numpy array stands in for a Bigarray and Python's collector for
OCaml's."""
import numpy as np
import pytest

from spoc_amd import hip
from spoc_amd.sarek import CPU, Execute, GpuMemory, Vector


def f32(values):
    return Vector.of_list(Vector.float32, values)


# ---- test_vector.ml: kinds --------------------------------------------------------------------------------------

def test_scalar_kinds_and_kind_constructors():
    kinds = (Vector.float32, Vector.float64, Vector.int32, Vector.int64, Vector.char, Vector.complex32)
    assert len({k.code for k in kinds}) == 6


def test_elem_size_and_kind_name():
    assert [Vector.elem_size(k) for k in (Vector.float32, Vector.float64, Vector.int32, Vector.int64)] == [4, 8, 4, 8]
    assert [Vector.kind_name(k) for k in (Vector.float32, Vector.float64, Vector.int32, Vector.int64)] == \
        ["Float32", "Float64", "Int32", "Int64"]


# ---- creation ---------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("create, length, name", [(Vector.create_float32, 100, "Float32"),
                                                  (Vector.create_float64, 50, "Float64"),
                                                  (Vector.create_int32, 200, "Int32"),
                                                  (Vector.create_int64, 75, "Int64")])
def test_create_by_kind(create, length, name):
    v = create(length)
    assert v.length == length and Vector.kind_name(v.kind) == name
    assert hip.lib.sarek_hip_vector_elem_size(v._h) == Vector.elem_size(v.kind)


def test_create_generic():
    assert Vector.create(Vector.float32, 100).length == 100


# ---- location ---------------------------------------------------------------------------------------------------

def test_initial_location_and_predicates():
    v = Vector.create_float32(10)
    assert v.location == CPU and str(v.location) == "CPU"
    assert v.is_on_cpu and not v.is_on_gpu and not v.is_synced


# ---- element access ---------------------------------------------------------------------------------------------

def test_get_set_float32():
    v = Vector.create_float32(10)
    v.set(0, 1.5), v.set(5, 2.5), v.set(9, 3.5)
    assert (v.get(0), v.get(5), v.get(9)) == (1.5, 2.5, 3.5)


def test_get_set_int32_and_int64():
    v = Vector.create_int32(10)
    v.set(0, 100), v.set(5, 200)
    assert (v.get(0), v.get(5)) == (100, 200)
    w = Vector.create_int64(10)
    w.set(0, 1000), w.set(5, 2000)
    assert (w.get(0), w.get(5)) == (1000, 2000)


def test_bounds_check():
    v = Vector.create_float32(10)
    for bad in (-1, 10):
        with pytest.raises(IndexError):          # Invalid_argument there
            v.set(bad, 1.0)
        with pytest.raises(IndexError):
            v.get(bad)


def test_unsafe_get_set():
    v = Vector.create_float32(10)
    v.unsafe_set(0, 42.0)
    assert v.unsafe_get(0) == 42.0


# ---- fill, init, copy -------------------------------------------------------------------------------------------

def test_fill_and_init():
    v = Vector.create_float32(5)
    v.fill(7.0)
    assert all(v.get(i) == 7.0 for i in range(5))
    w = Vector.init(Vector.float32, 5, float)
    assert (w.get(0), w.get(1), w.get(4)) == (0.0, 1.0, 4.0)


def test_copy_is_independent():
    v1 = Vector.create_float32(5)
    v1.fill(3.0)
    v2 = v1.copy()
    assert v2.length == v1.length and v2.get(0) == 3.0
    v1.set(0, 99.0)
    assert v2.get(0) == 3.0
    # test_vector_storage.ml:13-22, the same on explicit values
    v = Vector.create_float32(4)
    v.set(0, 1.0), v.set(1, 2.0)
    c = v.copy()
    assert c.length == 4 and c.get(1) == 2.0
    v.set(1, 9.0)
    assert c.get(1) == 2.0


# ---- conversions ------------------------------------------------------------------------------------------------

def test_of_bigarray_and_to_bigarray():
    ba = np.full(5, 2.0, np.float32)
    v = Vector.of_bigarray(Vector.float32, ba)
    assert v.length == 5 and v.get(0) == 2.0
    w = Vector.create_float32(5)
    w.fill(4.0)
    out = w.to_bigarray()
    assert out.shape == (5,) and out[0] == 4.0
    with pytest.raises(ValueError):              # invalid_arg "to_bigarray: vector uses custom storage"
        Vector.create_custom(12, 3).to_bigarray()


def test_lists_and_arrays():
    v = Vector.of_list(Vector.float32, [1.0, 2.0, 3.0, 4.0, 5.0])
    assert v.length == 5 and v.get(0) == 1.0 and v.get(4) == 5.0
    w = Vector.create_float32(3)
    w.set(0, 1.0), w.set(1, 2.0), w.set(2, 3.0)
    assert w.to_list() == [1.0, 2.0, 3.0]
    a = Vector.of_array(np.array([10.0, 20.0, 30.0], np.float32), Vector.float32)
    assert a.length == 3 and a.get(1) == 20.0
    b = Vector.create_float32(3)
    b.set(0, 100.0), b.set(1, 200.0), b.set(2, 300.0)
    arr = b.to_array()
    assert arr[0] == 100.0 and arr[2] == 300.0


# ---- iterators, folds, predicates, aggregates -------------------------------------------------------------------

def test_iter_and_iteri():
    seen = []
    f32([1.0, 2.0, 3.0]).iter(seen.append)
    assert sum(seen) == 6.0
    indices = []
    f32([10.0, 20.0, 30.0]).iteri(lambda i, _: indices.append(i))
    assert sum(indices) == 3


def test_map_mapi_map_inplace():
    v2 = f32([1.0, 2.0, 3.0]).map(lambda x: x * 2.0, Vector.float32)
    assert [v2.get(i) for i in range(3)] == [2.0, 4.0, 6.0]
    v3 = f32([10.0, 20.0, 30.0]).mapi(lambda i, x: x + float(i), Vector.float32)
    assert [v3.get(i) for i in range(3)] == [10.0, 21.0, 32.0]
    v = f32([1.0, 2.0, 3.0])
    v.map_inplace(lambda x: x * 10.0)
    assert [v.get(i) for i in range(3)] == [10.0, 20.0, 30.0]


def test_folds():
    assert f32([1.0, 2.0, 3.0, 4.0]).fold_left(lambda acc, x: acc + x, 0.0) == 10.0
    assert f32([1.0, 2.0, 3.0]).fold_right(lambda x, acc: [x] + acc, []) == [1.0, 2.0, 3.0]


def test_predicates():
    v = f32([2.0, 4.0, 6.0, 8.0])
    assert v.for_all(lambda x: x > 0.0) and not v.for_all(lambda x: x > 5.0)
    w = f32([1.0, 2.0, 3.0, 4.0])
    assert w.exists(lambda x: x == 3.0) and not w.exists(lambda x: x == 99.0)
    assert w.find(lambda x: x > 2.5) == 3.0 and w.find(lambda x: x > 100.0) is None
    u = f32([10.0, 20.0, 30.0, 40.0])
    assert u.find_index(lambda x: x == 30.0) == 2 and u.find_index(lambda x: x == 99.0) is None


def test_aggregates():
    assert f32([1.0, 2.0, 3.0, 4.0, 5.0]).sum(0.0, lambda a, b: a + b) == 15.0
    v = f32([3.0, 1.0, 4.0, 1.5, 9.0])
    compare = lambda a, b: int(a > b) - int(a < b)      # noqa: E731 -- Float.compare
    assert v.min_elt(compare) == 1.0 and v.max_elt(compare) == 9.0
    assert Vector.create_float32(0).min_elt(compare) is None


# ---- sub-vectors, blit, printing, flags, ids --------------------------------------------------------------------

def test_sub_vector_and_is_sub():
    v = f32([float(i) for i in range(10)])
    sub = v.sub_vector(2, 5)
    assert sub.length == 5 and sub.get(0) == 2.0 and sub.get(4) == 6.0
    w = f32([0.0, 1.0, 2.0, 3.0, 4.0])
    assert not w.is_sub and w.sub_vector(1, 3).is_sub


def test_sub_vector_metadata():                      # test_vector_storage.ml:24-32
    v = Vector.create_int32(10)
    sub = v.sub_vector(2, 5)
    assert sub.is_sub and sub.parent_id == v.id and sub.sub_start == 2 and sub.depth == 1


def test_partition_host():                           # test_vector_storage.ml:34-65: nine int64 over three devices
    parts = Vector.create_int64(9).partition([0, 1, 2])
    assert len(parts) == 3 and parts[0].length == 3 and parts[1].sub_start == 3 and parts[2].depth == 1


def test_blit():
    src = f32([1.0, 2.0, 3.0, 4.0, 5.0])
    dst = Vector.create_float32(10)
    dst.fill(0.0)
    Vector.blit(src, 1, dst, 3, 3)
    assert (dst.get(3), dst.get(4), dst.get(5)) == (2.0, 3.0, 4.0)


def test_to_string_auto_sync_flag_unique_ids():
    v = Vector.create_float32(10)
    assert len(str(v)) > 0
    assert v.auto_sync
    v.set_auto_sync(False)
    assert not v.auto_sync
    v.set_auto_sync(True)
    assert v.auto_sync
    ids = [Vector.create_float32(10).id for _ in range(3)]
    assert len(set(ids)) == 3


# ---- test_vector_transfer.ml: host pointer ----------------------------------------------------------------------

def test_host_ptr_helpers():
    v = Vector.create_float32(1)
    v.to_bigarray()[0] = 3.14
    ptr = hip.lib.sarek_hip_vector_host_ptr(v._h)
    assert ptr not in (None, 0)
    assert np.isclose(v.get(0), 3.14)


# ---- test_execute.ml --------------------------------------------------------------------------------------------

def test_argument_constructors_and_dims():
    assert Execute.Int(42) == ("i32", 42) and Execute.Int32(42) == ("i32", 42)
    assert Execute.Float32(3.14)[0] == "f32" and Execute.Float64(2.71828)[0] == "f64"
    assert Execute.dims1d(1024) == (1024, 1, 1)
    assert Execute.dims2d(32, 64) == (32, 64, 1)
    assert Execute.dims3d(16, 32, 8) == (16, 32, 8)


def test_grid_for_size():
    assert Execute.grid_for_size(1024, 256) == 4
    assert Execute.grid_for_size(1000, 256) == 4
    assert Execute.grid_for_size(100, 256) == 1
    assert Execute.grid_for_size(0, 256) == 0


def test_vectors_as_arguments():
    v = Vector.create(Vector.int32, 10)
    v.set(5, 42)
    assert v.length == 10 and v.get(5) == 42
    w = Vector.create(Vector.float32, 8)
    w.set(3, 3.14)
    assert w.length == 8 and abs(w.get(3) - 3.14) < 0.001
    args = [Execute.Vec(v), Execute.Int(42), Execute.Vec(Vector.create(Vector.float32, 20)), Execute.Float32(3.14)]
    packed, n = Execute._args(args)
    assert n == 4 and [packed[i].kind for i in range(4)] == [0, 1, 0, 3]


# ---- test_gpu_memory.ml -----------------------------------------------------------------------------------------

@pytest.fixture()
def gpu_memory():
    GpuMemory.set_auto_gc(True)
    yield GpuMemory
    GpuMemory.set_auto_gc(True)


def test_auto_gc_flag(gpu_memory):
    assert gpu_memory.get_auto_gc()
    gpu_memory.set_auto_gc(False)
    assert not gpu_memory.get_auto_gc()
    gpu_memory.set_auto_gc(True)
    assert gpu_memory.get_auto_gc()


def test_memory_tracking(gpu_memory):
    initial = gpu_memory.usage()
    gpu_memory.track_alloc(1024)
    assert gpu_memory.usage() == initial + 1024
    gpu_memory.track_free(512)
    assert gpu_memory.usage() == initial + 512
    gpu_memory.track_free(512)
    assert gpu_memory.usage() == initial


def test_with_retry(gpu_memory):
    calls = []

    def succeeds():
        calls.append(1)
        return 42
    assert gpu_memory.with_retry(succeeds) == 42 and len(calls) == 1

    calls.clear()
    collections = []
    reclaim = GpuMemory._RECLAIM(lambda ctx, attempt: collections.append(attempt))
    hip.lib.sarek_hip_gpu_memory_set_reclaim(hip.C.cast(reclaim, hip.C.c_void_p), None)
    try:
        before = gpu_memory.stats().retry_count

        def fails_once():
            calls.append(1)
            if len(calls) < 2:
                raise RuntimeError("OOM")
            return 99
        assert gpu_memory.with_retry(fails_once) == 99 and len(calls) == 2
        assert collections == [1] and gpu_memory.stats().retry_count == before + 1

        calls.clear()
        collections.clear()

        def always_fails():
            calls.append(1)
            raise RuntimeError(f"persistent OOM {len(calls)}")
        with pytest.raises(RuntimeError, match="persistent OOM 1"):      # the first failure is the one raised
            gpu_memory.with_retry(always_fails)
        assert len(calls) == 3 and collections == [1, 2]

        calls.clear()
        gpu_memory.set_auto_gc(False)
        with pytest.raises(RuntimeError):
            gpu_memory.with_retry(always_fails)
        assert len(calls) == 1                                           # no retry when switched off
        gpu_memory.set_auto_gc(True)

        collections.clear()
        gpu_memory.trigger_gc()
        assert collections == [1]
    finally:
        hip.lib.sarek_hip_gpu_memory_set_reclaim(None, None)
    gpu_memory.trigger_gc()                                              # no callback: nothing to run, no error


def test_with_retry_keeps_the_first_failures_status_and_message():
    """Through the C ABI itself: three failing attempts with different messages give the first one back."""
    n = [0]
    v = Vector.create_float32(1)
    out = np.empty(1, np.float32)

    def attempt(ctx):
        n[0] += 1
        # a failing library call leaves its message (with the index) in the thread's last-error slot
        return hip.lib.sarek_hip_vector_get(v._h, 1000 + n[0], hip.C.c_void_p(out.ctypes.data))
    cb = GpuMemory._ATTEMPT(attempt)
    st = hip.lib.sarek_hip_gpu_memory_with_retry(hip.C.cast(cb, hip.C.c_void_p), None)
    assert st == hip.E_INVALID_ARG and n[0] == 3
    assert "1001" in hip.lib.sarek_hip_last_error().decode()
    assert hip.lib.sarek_hip_gpu_memory_with_retry(None, None) == hip.E_INVALID_ARG


def test_stats_and_reset(gpu_memory):
    gpu_memory.reset_stats()
    gpu_memory.track_alloc(4096)
    gpu_memory.track_alloc(8192)
    gpu_memory.track_free(4096)
    s = gpu_memory.stats()
    assert (s.current_bytes, s.peak_bytes, s.alloc_count, s.free_count) == (8192, 12288, 2, 1)
    assert gpu_memory.peak_usage() == 12288
    gpu_memory.reset_stats()
    s = gpu_memory.stats()
    assert (s.current_bytes, s.peak_bytes, s.alloc_count) == (0, 0, 0)
    assert hip.lib.sarek_hip_gpu_memory_stats(None) == hip.E_INVALID_ARG
