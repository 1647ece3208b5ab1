"""ctypes binding of libsarek_hip.so plus tensor-level helpers.

Mirrors the surface a plugin's ``Hip_bindings``/``Hip_api`` pair would expose
(sarek-cuda/Cuda_bindings.ml, sarek-cuda/Cuda_api.ml in the reference): raw symbols
in :data:`lib`, checked wrappers below.  torch is used for device memory and the
current stream only.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# SAREK_HIP_MEASURE_BUILD=1 (bench.py --measure-build) loads the measurement build instead: the product's code plus the
# kernel variants of the ablation studies (`make -C spoc_amd/csrc measure`).  Tests and the default bench use the product.
MEASURE_BUILD = os.environ.get("SAREK_HIP_MEASURE_BUILD", "0") == "1"
LIB_PATH = os.path.join(_HERE, "libsarek_hip_measure.so" if MEASURE_BUILD else "libsarek_hip.so")


class SarekHipError(RuntimeError):
    """Non-zero status from libsarek_hip (cf. Backend_error in the reference)."""

    def __init__(self, status, name, message):
        super().__init__(f"{name} ({status}): {message}")
        self.status = status
        self.name = name
        self.message = message


# Status codes of include/sarek_hip.h
OK = 0
E_INVALID_ARG = -1
E_UNSUPPORTED = -2
E_COMPILE = -3
E_NO_DEVICE = -4
E_WORKSPACE = -5
E_PARSE = -6
E_CODEGEN = -7
E_BUFFER_TOO_SMALL = -8

LANG_CUDA, LANG_OPENCL, LANG_PTX, LANG_SPIRV, LANG_GLSL, LANG_HIP = range(6)
ARG_BUFFER, ARG_INT32, ARG_INT64, ARG_FLOAT32, ARG_FLOAT64 = range(5)


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 256), ("gcn_arch", C.c_char * 64),
        ("total_global_mem", C.c_uint64), ("max_threads_per_block", C.c_int),
        ("max_block_dim", C.c_int * 3), ("max_grid_dim", C.c_int * 3),
        ("shared_mem_per_block", C.c_int), ("warp_size", C.c_int),
        ("multiprocessor_count", C.c_int), ("clock_rate_khz", C.c_int),
        ("memory_clock_rate_khz", C.c_int), ("memory_bus_width_bits", C.c_int),
        ("l2_cache_size", C.c_int), ("compute_major", C.c_int), ("compute_minor", C.c_int),
        ("max_registers_per_block", C.c_int),
    ]


class Arg(C.Structure):
    _fields_ = [("kind", C.c_int), ("buffer", C.c_void_p), ("length", C.c_int64),
                ("i32", C.c_int32), ("i64", C.c_int64), ("f32", C.c_float), ("f64", C.c_double)]


_vp, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float
_int3 = C.POINTER(C.c_int)
_uint3 = C.POINTER(C.c_uint)

class VArg(C.Structure):
    """sarek_hip_varg: one Execute.vector_arg."""
    _fields_ = [("kind", C.c_int), ("vec", C.c_void_p), ("i32", C.c_int32), ("i64", C.c_int64),
                ("f32", C.c_float), ("f64", C.c_double)]


class Launch(C.Structure):
    """sarek_hip_launch: one run_source call of a sequence."""
    _fields_ = [("source", C.c_char_p), ("lang", C.c_int), ("kernel_name", C.c_char_p), ("block", C.c_int * 3),
                ("grid", C.c_int * 3), ("shared_mem_bytes", C.c_int), ("args", C.POINTER(Arg)), ("n_args", C.c_int)]


class PipelineStage(C.Structure):
    """sarek_hip_pipeline_stage: one Execute.run_vectors call of a kernel sequence."""
    _fields_ = [("ir_text", C.c_char_p), ("block", C.c_int * 3), ("grid", C.c_int * 3),
                ("shared_mem_bytes", C.c_int), ("args", C.POINTER(VArg)), ("n_args", C.c_int)]


# Every symbol include/sarek_hip.h declares: (restype, argtypes).
SYMBOLS = {
    "sarek_hip_abi_version": (_i, []),
    "sarek_hip_device_info_size": (_i, []),
    "sarek_hip_device_report": (_i, [C.c_char_p, _sz, C.POINTER(_sz), C.POINTER(_i)]),
    "sarek_hip_last_error": (C.c_char_p, []),
    "sarek_hip_status_name": (C.c_char_p, [_i]),
    "sarek_hip_init": (_i, []),
    "sarek_hip_is_available": (_i, []),
    "sarek_hip_device_count": (_i, [C.POINTER(_i)]),
    "sarek_hip_device_get_info": (_i, [_i, C.POINTER(DeviceInfo)]),
    "sarek_hip_device_set_current": (_i, [_i]),
    "sarek_hip_device_get_current": (_i, [C.POINTER(_i)]),
    "sarek_hip_device_synchronize": (_i, []),
    "sarek_hip_mem_get_info": (_i, [C.POINTER(_sz), C.POINTER(_sz)]),
    "sarek_hip_driver_version": (_i, [C.POINTER(_i)]),
    "sarek_hip_mem_alloc": (_i, [C.POINTER(_vp), _sz]),
    "sarek_hip_mem_free": (_i, [_vp]),
    "sarek_hip_memcpy_htod": (_i, [_vp, _vp, _sz]),
    "sarek_hip_memcpy_dtoh": (_i, [_vp, _vp, _sz]),
    "sarek_hip_memcpy_dtod": (_i, [_vp, _vp, _sz]),
    "sarek_hip_host_alloc": (_i, [C.POINTER(_vp), _sz]),
    "sarek_hip_host_free": (_i, [_vp]),
    "sarek_hip_mem_alloc_zero_copy": (_i, [_vp, _sz, C.POINTER(_vp), C.POINTER(_i)]),
    "sarek_hip_memset_d8": (_i, [_vp, C.c_ubyte, _sz]),
    "sarek_hip_stream_create": (_i, [C.POINTER(_vp)]),
    "sarek_hip_stream_destroy": (_i, [_vp]),
    "sarek_hip_stream_synchronize": (_i, [_vp]),
    "sarek_hip_event_create": (_i, [C.POINTER(_vp)]),
    "sarek_hip_event_destroy": (_i, [_vp]),
    "sarek_hip_event_record": (_i, [_vp, _vp]),
    "sarek_hip_event_synchronize": (_i, [_vp]),
    "sarek_hip_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(_f)]),
    "sarek_hip_profiler_start": (_i, []),
    "sarek_hip_profiler_stop": (_i, []),
    "sarek_hip_kernel_compile": (_i, [C.c_char_p, C.c_char_p, C.POINTER(_vp), C.c_char_p, _sz]),
    "sarek_hip_kernel_compile_cached": (_i, [C.c_char_p, C.c_char_p, C.POINTER(_vp), C.c_char_p, _sz]),
    "sarek_hip_kernel_clear_cache": (_i, []),
    "sarek_hip_kernel_destroy": (_i, [_vp]),
    "sarek_hip_kernel_launch": (_i, [_vp, _uint3, _uint3, C.c_uint, _vp, C.POINTER(_vp), _i]),
    "sarek_hip_generate_source": (_i, [C.c_char_p, _int3, C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_rebuilt_source": (_i, [C.c_char_p, _i, C.c_uint32, C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_run_source": (_i, [C.c_char_p, _i, C.c_char_p, _int3, _int3, _i, C.POINTER(Arg), _i]),
    "sarek_hip_set_specialisation": (_i, [_i]),
    "sarek_hip_last_run_path": (C.c_char_p, []),
    "sarek_hip_triad_f32": (_i, [_vp, _vp, _vp, _f, _i64, _vp]),
    "sarek_hip_triad_sum_workspace_floats": (_i64, [_i64]),
    "sarek_hip_triad_sum_f32": (_i, [_vp, _vp, _vp, _f, _i64, _vp, _i64, _vp, _vp]),
    "sarek_hip_triad_sum_static_max_n": (_i64, []),
    "sarek_hip_triad_sum_f32_static": (_i, [_vp, _vp, _vp, _f, _i64, _vp, _vp]),
    "sarek_hip_reduce_sum_block256_f32": (_i, [_vp, _vp, _i64, _vp]),
    "sarek_hip_dot_block256_f32": (_i, [_vp, _vp, _vp, _i64, _vp]),
    "sarek_hip_reduce_max_block256_f32": (_i, [_vp, _vp, _i64, _f, _vp]),
    "sarek_hip_fold_partials_f64": (_i, [_vp, _i64, _vp, _vp]),
    "sarek_hip_copy_f32": (_i, [_vp, _vp, _i64, _vp]),
    "sarek_hip_transpose_f32": (_i, [_vp, _vp, _i, _i, _vp]),
    "sarek_hip_stencil_2d_f32": (_i, [_vp, _vp, _i, _i, _vp]),
    "sarek_hip_conv2d_f32": (_i, [_vp, _vp, _i, _i, _vp]),
    "sarek_hip_histogram_i32": (_i, [_vp, _vp, _i64, _i, _vp]),
    "sarek_hip_radix_histogram_i32": (_i, [_vp, _vp, _i64, _i, _i, _vp]),
    "sarek_hip_radix_scatter_i32": (_i, [_vp, _i64, _vp, _vp, _i64, _i, _i, _vp]),
    "sarek_hip_gemm_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "sarek_hip_gemm_bf16": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "sarek_hip_gemm_f16": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "sarek_hip_gemm_f32_k_splits": (_i, [_i, _i, _i]),
    "sarek_hip_gemm16_tile": (_i, [_i, _i, _i]),
    "sarek_hip_gemm16_k_splits": (_i, [_i, _i, _i]),
    "sarek_hip_gemm_f16_bias_relu_rowsum": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "sarek_hip_cast_f32_to_bf16": (_i, [_vp, _vp, _i64, _vp]),
    "sarek_hip_cast_f32_to_f16": (_i, [_vp, _vp, _i64, _vp]),
    "sarek_hip_cache_dir": (_i, [C.c_char_p, _sz]),
    "sarek_hip_cache_compute_key": (_i, [C.c_char_p, C.c_char_p, C.c_char_p, C.c_char_p]),
    "sarek_hip_cache_get": (_i, [C.c_char_p, _vp, _sz, C.POINTER(_sz), C.POINTER(_i)]),
    "sarek_hip_cache_put": (_i, [C.c_char_p, _vp, _sz]),
    "sarek_hip_cache_get_stats": (_i, [C.POINTER(_i64)]),
    "sarek_hip_cache_reset_stats": (_i, []),
    "sarek_hip_fusion_analyze": (_i, [C.c_char_p, C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_fusion_can_fuse": (_i, [C.c_char_p, C.c_char_p, C.c_char_p, _i, C.POINTER(_i)]),
    "sarek_hip_fusion_fuse": (_i, [C.c_char_p, C.c_char_p, C.c_char_p, _i, C.POINTER(_i), C.c_char_p, _sz,
                                   C.POINTER(_sz)]),
    "sarek_hip_fusion_should_fuse": (_i, [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(_i), C.c_char_p, _sz]),
    "sarek_hip_fusion_pipeline": (_i, [C.POINTER(C.c_char_p), _i, _i, C.c_char_p, _sz, C.POINTER(_sz),
                                       C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_fusion_analyze_pipeline": (_i, [C.POINTER(C.c_char_p), _i, C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_fusion_stencil_info": (_i, [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(_i), C.POINTER(_i),
                                           C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_fusion_expr_equal": (_i, [C.c_char_p, C.c_char_p, C.POINTER(_i)]),
    "sarek_hip_fusion_subst_array_read": (_i, [C.c_char_p, C.c_char_p, C.c_char_p, C.c_char_p, C.c_char_p, _sz,
                                               C.POINTER(_sz)]),
    "sarek_hip_fusion_detect_reduction": (_i, [C.c_char_p, C.POINTER(_i), C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_fusion_is_reduction_kernel": (_i, [C.c_char_p, C.c_char_p, C.POINTER(_i), C.c_char_p]),
    "sarek_hip_vector_create": (_i, [_i, _i64, _i64, _i, C.POINTER(_vp)]),
    "sarek_hip_vector_destroy": (_i, [_vp]),
    "sarek_hip_vector_id": (_i64, [_vp]),
    "sarek_hip_vector_to_string": (_i, [_vp, C.c_char_p, C.c_size_t]),
    "sarek_hip_vector_fill": (_i, [_vp, _vp]),
    "sarek_hip_vector_copy": (_i, [_vp, C.POINTER(_vp)]),
    "sarek_hip_vector_sub": (_i, [_vp, _i64, _i64, _i64, _i64, C.POINTER(_vp)]),
    "sarek_hip_vector_sub_meta": (_i, [_vp, C.POINTER(_i), C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64),
                                       C.POINTER(_i64), C.POINTER(_i)]),
    "sarek_hip_vector_partition": (_i, [_vp, _i, C.POINTER(_i), C.POINTER(_vp)]),
    "sarek_hip_vector_blit": (_i, [_vp, _i64, _vp, _i64, _i64]),
    "sarek_hip_vector_length": (_i64, [_vp]),
    "sarek_hip_vector_elem_size": (_i64, [_vp]),
    "sarek_hip_vector_kind": (_i, [_vp]),
    "sarek_hip_vector_location": (_i, [_vp, C.POINTER(_i), C.POINTER(_i)]),
    "sarek_hip_vector_host_ptr": (_vp, [_vp]),
    "sarek_hip_vector_device_ptr": (_i, [_vp, C.POINTER(_vp)]),
    "sarek_hip_vector_set_auto_sync": (_i, [_vp, _i]),
    "sarek_hip_vector_auto_sync": (_i, [_vp]),
    "sarek_hip_gpu_memory_set_auto_gc": (None, [_i]),
    "sarek_hip_gpu_memory_get_auto_gc": (_i, []),
    "sarek_hip_gpu_memory_track_alloc": (None, [_i64]),
    "sarek_hip_gpu_memory_track_free": (None, [_i64]),
    "sarek_hip_gpu_memory_usage": (_i64, []),
    "sarek_hip_gpu_memory_peak_usage": (_i64, []),
    "sarek_hip_gpu_memory_stats": (_i, [_vp]),
    "sarek_hip_gpu_memory_reset_stats": (None, []),
    "sarek_hip_gpu_memory_set_reclaim": (None, [_vp, _vp]),
    "sarek_hip_gpu_memory_trigger_gc": (None, []),
    "sarek_hip_gpu_memory_with_retry": (_i, [_vp, _vp]),
    "sarek_hip_vector_get": (_i, [_vp, _i64, _vp]),
    "sarek_hip_vector_set": (_i, [_vp, _i64, _vp]),
    "sarek_hip_vector_read": (_i, [_vp, _vp, _i64, _i64]),
    "sarek_hip_vector_write": (_i, [_vp, _vp, _i64, _i64]),
    "sarek_hip_transfer_set_auto": (_i, [_i]),
    "sarek_hip_transfer_to_device": (_i, [_vp]),
    "sarek_hip_transfer_to_cpu": (_i, [_vp, _i]),
    "sarek_hip_transfer_sync": (_i, [_vp]),
    "sarek_hip_transfer_free_buffers": (_i, [_vp]),
    "sarek_hip_transfer_flush": (_i, []),
    "sarek_hip_execute_run_vectors": (_i, [C.c_char_p, _int3, _int3, _i, C.POINTER(VArg), _i]),
    "sarek_hip_execute_run_source": (_i, [C.c_char_p, _i, C.c_char_p, _int3, _int3, _i, _i, C.POINTER(VArg), _i]),
    "sarek_hip_execute_sync_vectors_to_cpu": (_i, [C.POINTER(VArg), _i]),
    "sarek_hip_execute_run_pipeline": (_i, [C.POINTER(PipelineStage), _i, C.POINTER(_i)]),
    "sarek_hip_run_sources": (_i, [C.POINTER(Launch), _i, C.POINTER(_i), C.POINTER(_i)]),
    "sarek_hip_library_kernel_source": (_i, [C.c_char_p, C.c_char_p, _sz, C.POINTER(_sz), C.c_char_p, _sz]),
    "sarek_hip_library_kernel_list": (_i, [C.c_char_p, _sz, C.POINTER(_sz)]),
    "sarek_hip_triad_block256_sum_f32": (_i, [_vp, _vp, _vp, _f, _i64, _vp, _vp]),
    "sarek_hip_triad_block256_max_f32": (_i, [_vp, _vp, _vp, _f, _i64, _f, _vp, _vp]),
    "sarek_hip_backend_name": (C.c_char_p, []),
    "sarek_hip_backend_version": (_i, [C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)]),
    "sarek_hip_execution_model": (_i, []),
    "sarek_hip_intrinsic_register": (_i, [C.c_char_p, C.c_char_p, _i]),
    "sarek_hip_intrinsic_find": (_i, [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(_i), C.POINTER(_i)]),
    "sarek_hip_intrinsic_list": (_i, [C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]),
    "sarek_hip_supports_lang": (_i, [_i]),
    "sarek_hip_execute_detect_lang": (_i, [C.c_char_p, C.POINTER(_i)]),
    "sarek_hip_execute_run_source_file": (_i, [C.c_char_p, C.c_char_p, _int3, _int3, _i, _i, C.POINTER(VArg), _i]),
    "sarek_hip_set_tunable": (_i, [C.c_char_p, _i64]),
    "sarek_hip_set_clock_probe": (_i, [_vp, _i64, C.POINTER(_i64)]),
    "sarek_hip_is_measurement_build": (_i, []),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C spoc_amd/csrc`).  There is no CPU fallback.")
    # One HIP runtime per process: the torch wheel ships its own libamdhip64 /
    # libhsa-runtime64 and loads them by path, so if this library pulled in the system
    # copies first the process would hold two runtimes and the second sees no device.
    # Loading torch first makes both sides share torch's copy (same sonames).
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(status):
    if status != OK:
        raise SarekHipError(status, lib.sarek_hip_status_name(status).decode(),
                            lib.sarek_hip_last_error().decode(errors="replace"))


def set_tunable(name, value):
    check(lib.sarek_hip_set_tunable(name.encode(), int(value)))


# ---------------------------------------------------------------------------
# Persistent kernel cache (the reference's Framework_cache)

def cache_dir():
    buf = C.create_string_buffer(4096)
    check(lib.sarek_hip_cache_dir(buf, len(buf)))
    return buf.value.decode()


def cache_compute_key(dev_name, driver_version, source):
    out = C.create_string_buffer(33)
    check(lib.sarek_hip_cache_compute_key(dev_name.encode(), driver_version.encode(), source.encode(), out))
    return out.value.decode()


def cache_put(key, data):
    check(lib.sarek_hip_cache_put(key.encode(), data, len(data)))


def cache_get(key):
    """bytes of the entry, or None."""
    size, found = _sz(0), _i(0)
    buf = C.create_string_buffer(1 << 16)
    st = lib.sarek_hip_cache_get(key.encode(), buf, len(buf), C.byref(size), C.byref(found))
    if st == E_BUFFER_TOO_SMALL:
        buf = C.create_string_buffer(size.value)
        st = lib.sarek_hip_cache_get(key.encode(), buf, len(buf), C.byref(size), C.byref(found))
    check(st)
    return buf.raw[:size.value] if found.value else None


def cache_stats():
    out = (_i64 * 4)()
    check(lib.sarek_hip_cache_get_stats(out))
    return dict(hits=out[0], misses=out[1], puts=out[2], errors=out[3])


def cache_reset_stats():
    check(lib.sarek_hip_cache_reset_stats())


SHADER_CLOCK_SRC = r"""
// One wave per workgroup sleeps for `ticks` of the constant-rate clock and reports how many shader cycles passed.
extern "C" __global__ void shader_clock_sample(unsigned long long* out, int ticks) {
  const long long t0 = wall_clock64(), c0 = clock64();
  long long t1 = t0;
  while (t1 - t0 < ticks) {           // bounded by the constant-rate clock: the wave always leaves
    __builtin_amdgcn_s_sleep(64);
    t1 = wall_clock64();
  }
  if (threadIdx.x == 0) {
    out[2 * blockIdx.x] = (unsigned long long)(clock64() - c0);
    out[2 * blockIdx.x + 1] = (unsigned long long)(t1 - t0);
  }
}
"""


class shader_clock_sampler:
    """The shader clock while other kernels run, without anything inside those kernels: eight sleeping waves on a stream
    of their own count shader cycles against the constant-rate clock for `window_ms`, next to whatever the caller
    launches right after `start()`.  They hold no LDS and eight registers, so they sit beside any resident workgroup."""

    def __init__(self, waves=8):
        torch = _torch()
        self.waves = waves
        self.buf = torch.zeros(2 * waves, dtype=torch.int64, device="cuda")
        self.stream = C.c_void_p()
        check(lib.sarek_hip_stream_create(C.byref(self.stream)))
        self.kernel = C.c_void_p()
        log = C.create_string_buffer(4096)
        check(lib.sarek_hip_kernel_compile_cached(SHADER_CLOCK_SRC.encode(), b"shader_clock_sample", C.byref(self.kernel),
                                                  log, len(log)))
        self.ticks_per_ms = None

    def _rate(self):
        """Ticks of the constant-rate clock per millisecond, from one 2 ms sample against HIP events."""
        if self.ticks_per_ms is None:
            torch = _torch()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            st = torch.cuda.ExternalStream(self.stream.value)
            self.buf.zero_()
            torch.cuda.synchronize()
            e0.record(st)
            self._launch(200_000)     # 2 ms at the usual 100 MHz; only the ratio below is used
            e1.record(st)
            torch.cuda.synchronize()
            ticks = int(self.buf.view(-1, 2)[0, 1].item())
            self.ticks_per_ms = ticks / e0.elapsed_time(e1)
        return self.ticks_per_ms

    def _launch(self, ticks):
        out, t = C.c_void_p(self.buf.data_ptr()), C.c_int(int(ticks))
        params = (C.c_void_p * 2)(C.cast(C.pointer(out), C.c_void_p), C.cast(C.pointer(t), C.c_void_p))
        grid, block = (C.c_uint * 3)(self.waves, 1, 1), (C.c_uint * 3)(64, 1, 1)
        check(lib.sarek_hip_kernel_launch(self.kernel, grid, block, 0, self.stream, params, 2))
        self._keep = (out, t, params)

    def start(self, window_ms):
        """Queue the sampling waves; the caller launches its own work next and waits for the device."""
        rate = self._rate()
        self.buf.zero_()
        _torch().cuda.synchronize()
        self._launch(min(window_ms, 20.0) * rate)

    def mhz(self):
        _torch().cuda.synchronize()
        p = self.buf.view(-1, 2).cpu().numpy()
        p = p[p[:, 1] > 0]
        if len(p) == 0:
            return None
        return float(p[:, 0].sum()) / float(p[:, 1].sum()) * self._rate() / 1e3

    def close(self):
        if self.stream:
            _torch().cuda.synchronize()
            check(lib.sarek_hip_stream_destroy(self.stream))
            self.stream = C.c_void_p()


class clock_probe:
    """Measurement build only.  Context manager: MFMA GEMM launches inside it record, per workgroup, the shader-clock
    cycles and wall-clock ticks it was resident.  `mhz()` is the shader clock those
    workgroups ran at, averaged over the last launch that fitted the buffer."""

    def __init__(self, workgroups=4096):
        torch = _torch()
        self.buf = torch.zeros(2 * workgroups, dtype=torch.int64, device="cuda")
        self.rate = C.c_int64(0)

    def __enter__(self):
        check(lib.sarek_hip_set_clock_probe(C.c_void_p(self.buf.data_ptr()), self.buf.numel() // 2,
                                            C.byref(self.rate)))
        return self

    def __exit__(self, *exc):
        check(lib.sarek_hip_set_clock_probe(None, 0, None))
        return False

    def pairs(self):
        _torch().cuda.synchronize()
        p = self.buf.view(-1, 2).cpu().numpy()
        return p[p[:, 1] > 0]

    def mhz(self):
        p = self.pairs()
        if len(p) == 0:
            return None
        return float(p[:, 0].sum()) / float(p[:, 1].sum()) * self.rate.value / 1e6


# ---------------------------------------------------------------------------
# Tensor-level helpers (torch = device memory + stream plumbing only)

def _torch():
    import torch
    return torch


def _stream():
    return C.c_void_p(_torch().cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def _need(t, dtype, name):
    torch = _torch()
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous()):
        raise TypeError(f"{name}: expected a contiguous device tensor of {dtype}")


def mem_alloc(nbytes):
    """Memory.alloc: device block, as an integer address."""
    p = _vp()
    check(lib.sarek_hip_mem_alloc(C.byref(p), nbytes))
    return p.value


def mem_free(dptr):
    check(lib.sarek_hip_mem_free(_vp(dptr)))


def memcpy_htod(dptr, host):
    """Memory.host_ptr_to_device from a contiguous numpy array."""
    check(lib.sarek_hip_memcpy_htod(_vp(dptr), _vp(host.ctypes.data), host.nbytes))


def memcpy_dtoh(host, dptr):
    """Memory.device_to_host_ptr into a contiguous numpy array."""
    check(lib.sarek_hip_memcpy_dtoh(_vp(host.ctypes.data), _vp(dptr), host.nbytes))


class pinned_array:
    """numpy array over a block from sarek_hip_host_alloc; freed by close() or on exit of
    a with-block (the array must not be used afterwards)."""

    def __init__(self, count, dtype):
        import numpy as np
        dtype = np.dtype(dtype)
        self._ptr = _vp()
        nbytes = int(count) * dtype.itemsize
        check(lib.sarek_hip_host_alloc(C.byref(self._ptr), nbytes))
        buf = (C.c_char * nbytes).from_address(self._ptr.value)
        self.array = np.frombuffer(buf, dtype=dtype, count=int(count))

    def close(self):
        if self._ptr is not None:
            self.array = None
            check(lib.sarek_hip_host_free(self._ptr))
            self._ptr = None

    def __enter__(self):
        return self.array

    def __exit__(self, *exc):
        self.close()


def device_report():
    """(text, device count) of the device-information tool (tools/device_info.ml)."""
    need, count = C.c_size_t(0), C.c_int(0)
    lib.sarek_hip_device_report(None, 0, C.byref(need), C.byref(count))
    buf = C.create_string_buffer(need.value)
    check(lib.sarek_hip_device_report(buf, need.value, None, C.byref(count)))
    return buf.value.decode(), count.value


def device_info(device=0):
    info = DeviceInfo()
    check(lib.sarek_hip_device_get_info(device, C.byref(info)))
    return info


def triad(b, c, s, out=None):
    """a = b + c*s (f32 vectors).  Returns a."""
    torch = _torch()
    _need(b, torch.float32, "b")
    _need(c, torch.float32, "c")
    a = torch.empty_like(b) if out is None else out
    check(lib.sarek_hip_triad_f32(_ptr(a), _ptr(b), _ptr(c), float(s), b.numel(), _stream()))
    return a


def triad_sum_workspace(n, device="cuda"):
    torch = _torch()
    cnt = int(lib.sarek_hip_triad_sum_workspace_floats(int(n)))
    return (torch.empty(cnt, dtype=torch.float32, device=device),
            torch.empty(1, dtype=torch.float64, device=device))


def triad_sum(b, c, s, out=None, workspace=None):
    """Fused a = b + c*s and sum(a).  Returns (a, sum_tensor[1] f64 on device)."""
    torch = _torch()
    _need(b, torch.float32, "b")
    _need(c, torch.float32, "c")
    a = torch.empty_like(b) if out is None else out
    partials, total = workspace if workspace is not None else triad_sum_workspace(b.numel(), b.device)
    check(lib.sarek_hip_triad_sum_f32(_ptr(a), _ptr(b), _ptr(c), float(s), b.numel(),
                                      _ptr(partials), partials.numel(), _ptr(total), _stream()))
    return a, total


def triad_block256_sum(b, c, s, out=None):
    """a = b + c*s and the block-256 sums of a in one pass.  Returns (a, block_sums)."""
    torch = _torch()
    _need(b, torch.float32, "b")
    _need(c, torch.float32, "c")
    a = torch.empty_like(b) if out is None else out
    sums = torch.empty((b.numel() + 255) // 256, dtype=torch.float32, device=b.device)
    check(lib.sarek_hip_triad_block256_sum_f32(_ptr(a), _ptr(b), _ptr(c), float(s), b.numel(), _ptr(sums), _stream()))
    return a, sums


def triad_block256_max(b, c, s, pad, out=None):
    """a = b + c*s and the block-256 maxima of a (elements past the end count as pad) in one pass.
    Returns (a, block_max)."""
    torch = _torch()
    _need(b, torch.float32, "b")
    _need(c, torch.float32, "c")
    a = torch.empty_like(b) if out is None else out
    mx = torch.empty((b.numel() + 255) // 256, dtype=torch.float32, device=b.device)
    check(lib.sarek_hip_triad_block256_max_f32(_ptr(a), _ptr(b), _ptr(c), float(s), b.numel(), float(pad), _ptr(mx),
                                               _stream()))
    return a, mx


def library_kernel(name):
    """(source text, kernel_name) of a library kernel, for Execute.run_source."""
    need = C.c_size_t(0)
    entry = C.create_string_buffer(128)
    rc = lib.sarek_hip_library_kernel_source(name.encode(), None, 0, C.byref(need), None, 0)
    if rc != E_BUFFER_TOO_SMALL:
        check(rc)
    buf = C.create_string_buffer(need.value)
    check(lib.sarek_hip_library_kernel_source(name.encode(), buf, need.value, None, entry, 128))
    return buf.value.decode(), entry.value.decode()


def library_kernel_names():
    need = C.c_size_t(0)
    lib.sarek_hip_library_kernel_list(None, 0, C.byref(need))
    buf = C.create_string_buffer(need.value)
    check(lib.sarek_hip_library_kernel_list(buf, need.value, None))
    return buf.value.decode().split()


def reduce_sum_block256(x):
    torch = _torch()
    _need(x, torch.float32, "x")
    out = torch.empty((x.numel() + 255) // 256, dtype=torch.float32, device=x.device)
    check(lib.sarek_hip_reduce_sum_block256_f32(_ptr(x), _ptr(out), x.numel(), _stream()))
    return out


def reduce_max_block256(x, pad=-1000000.0):
    torch = _torch()
    _need(x, torch.float32, "x")
    out = torch.empty((x.numel() + 255) // 256, dtype=torch.float32, device=x.device)
    check(lib.sarek_hip_reduce_max_block256_f32(_ptr(x), _ptr(out), x.numel(), float(pad), _stream()))
    return out


def dot_block256(a, b):
    torch = _torch()
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    out = torch.empty((a.numel() + 255) // 256, dtype=torch.float32, device=a.device)
    check(lib.sarek_hip_dot_block256_f32(_ptr(a), _ptr(b), _ptr(out), a.numel(), _stream()))
    return out


def fold_partials(p):
    torch = _torch()
    _need(p, torch.float32, "partials")
    out = torch.empty(1, dtype=torch.float64, device=p.device)
    check(lib.sarek_hip_fold_partials_f64(_ptr(p), p.numel(), _ptr(out), _stream()))
    return out


def copy(src, out=None):
    """out[i] = src[i] (bench_vector_copy's kernel)."""
    torch = _torch()
    _need(src, torch.float32, "src")
    out = torch.empty_like(src) if out is None else out
    _need(out, torch.float32, "out")
    if out.numel() < src.numel():
        raise ValueError("copy: out is shorter than src")
    check(lib.sarek_hip_copy_f32(_ptr(out), _ptr(src), src.numel(), _stream()))
    return out


def transpose(x, out=None):
    """x: [height, width] row-major -> out: [width, height] (bench_transpose's kernels)."""
    torch = _torch()
    _need(x, torch.float32, "x")
    h, w = x.shape
    out = torch.empty((w, h), dtype=torch.float32, device=x.device) if out is None else out
    _need(out, torch.float32, "out")
    if out.numel() != x.numel():
        raise ValueError("transpose: out has the wrong size")
    check(lib.sarek_hip_transpose_f32(_ptr(x), _ptr(out), w, h, _stream()))
    return out


def stencil_2d(x, out):
    """x, out: [height, width] row-major; the interior of out becomes the five-point mean of x
    (bench_stencil_2d's kernel over the whole grid), its border keeps what it holds."""
    torch = _torch()
    _need(x, torch.float32, "x")
    _need(out, torch.float32, "out")
    h, w = x.shape
    if out.numel() != x.numel():
        raise ValueError("stencil_2d: out has the wrong size")
    check(lib.sarek_hip_stencil_2d_f32(_ptr(x), _ptr(out), w, h, _stream()))
    return out


def conv2d(x, out=None):
    """x: [height, width] row-major -> its 3 x 3 box filter, 0 on the border (bench_conv2d's kernel)."""
    torch = _torch()
    _need(x, torch.float32, "x")
    h, w = x.shape
    out = torch.empty_like(x) if out is None else out
    _need(out, torch.float32, "out")
    if out.numel() != x.numel():
        raise ValueError("conv2d: out has the wrong size")
    check(lib.sarek_hip_conv2d_f32(_ptr(x), _ptr(out), w, h, _stream()))
    return out


def histogram(keys, hist, num_bins):
    """hist[b] += #{keys mod num_bins == b} (bench_histogram's kernel over all the keys)."""
    torch = _torch()
    _need(keys, torch.int32, "keys")
    _need(hist, torch.int32, "hist")
    if hist.numel() < num_bins:
        raise ValueError("histogram: hist is shorter than num_bins")
    check(lib.sarek_hip_histogram_i32(_ptr(hist), _ptr(keys), keys.numel(), num_bins, _stream()))
    return hist


def radix_histogram(keys, hist, shift, mask=255):
    """hist[d] += #{(keys >> shift) & mask == d}, 256 bins (bench_radix_sort's counting kernel)."""
    torch = _torch()
    _need(keys, torch.int32, "keys")
    _need(hist, torch.int32, "hist")
    if hist.numel() < 256:
        raise ValueError("radix_histogram: hist has fewer than 256 bins")
    check(lib.sarek_hip_radix_histogram_i32(_ptr(hist), _ptr(keys), keys.numel(), shift, mask, _stream()))
    return hist


def radix_scatter(keys, out, counters, shift, mask=255):
    """out[counters[d]++] = key for every key, d = (key >> shift) & mask (bench_radix_sort's scatter kernel)."""
    torch = _torch()
    for x, name in ((keys, "keys"), (out, "out"), (counters, "counters")):
        _need(x, torch.int32, name)
    if counters.numel() < mask + 1:
        raise ValueError("radix_scatter: counters shorter than mask + 1")
    check(lib.sarek_hip_radix_scatter_i32(_ptr(out), out.numel(), _ptr(counters), _ptr(keys), keys.numel(), shift, mask,
                                          _stream()))
    return out


def gemm_f32(a, b, out=None):
    torch = _torch()
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    m, k = a.shape
    k2, n = b.shape
    if k != k2:
        raise ValueError("gemm_f32: inner dimensions differ")
    c = torch.empty((m, n), dtype=torch.float32, device=a.device) if out is None else out
    check(lib.sarek_hip_gemm_f32(_ptr(a), _ptr(b), _ptr(c), m, n, k, _stream()))
    return c


def gemm_f32_k_splits(m, n, k):
    """Into how many pieces the f32 GEMM cuts K for this shape now (1 = none)."""
    return int(lib.sarek_hip_gemm_f32_k_splits(m, n, k))


def _gemm16(fn, dtype, a, b, out):
    torch = _torch()
    _need(a, dtype, "a")
    _need(b, dtype, "b")
    m, k = a.shape
    k2, n = b.shape
    if k != k2:
        raise ValueError("gemm16: inner dimensions differ")
    c = torch.empty((m, n), dtype=torch.float32, device=a.device) if out is None else out
    check(fn(_ptr(a), _ptr(b), _ptr(c), m, n, k, _stream()))
    return c


def gemm_bf16(a, b, out=None):
    return _gemm16(lib.sarek_hip_gemm_bf16, _torch().bfloat16, a, b, out)


def gemm16_tile(m, n, k):
    """256 / 128: the workgroup tile the 16-bit GEMMs take for this shape now; 0: the staged or simple kernel."""
    return int(lib.sarek_hip_gemm16_tile(m, n, k))


def gemm16_k_splits(m, n, k):
    """Into how many pieces the plain 16-bit GEMMs cut K for this shape now (1 = none)."""
    return int(lib.sarek_hip_gemm16_k_splits(m, n, k))


def gemm_f16(a, b, out=None):
    return _gemm16(lib.sarek_hip_gemm_f16, _torch().float16, a, b, out)


def gemm_f16_bias_relu_rowsum(a, b, bias, out=None, rowsum=None):
    torch = _torch()
    _need(a, torch.float16, "a")
    _need(b, torch.float16, "b")
    _need(bias, torch.float32, "bias")
    m, k = a.shape
    k2, n = b.shape
    if k != k2 or bias.numel() != n:
        raise ValueError("gemm_f16_bias_relu_rowsum: shape mismatch")
    y = torch.empty((m, n), dtype=torch.float32, device=a.device) if out is None else out
    rs = torch.empty(m, dtype=torch.float32, device=a.device) if rowsum is None else rowsum
    check(lib.sarek_hip_gemm_f16_bias_relu_rowsum(_ptr(a), _ptr(b), _ptr(bias), _ptr(y), _ptr(rs),
                                                  m, n, k, _stream()))
    return y, rs


def cast_bf16(x):
    torch = _torch()
    _need(x, torch.float32, "x")
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    check(lib.sarek_hip_cast_f32_to_bf16(_ptr(x), _ptr(out), x.numel(), _stream()))
    return out


def cast_f16(x):
    torch = _torch()
    _need(x, torch.float32, "x")
    out = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    check(lib.sarek_hip_cast_f32_to_f16(_ptr(x), _ptr(out), x.numel(), _stream()))
    return out


def make_args(items):
    """Build a run_source argument array.

    items: device tensors (expanded to buffer + int32 length, as the reference's
    dispatcher does for vectors), ("i32", v), ("i64", v), ("f32", v), ("f64", v),
    or ("buf", tensor) for a bare buffer without the injected length.
    """
    torch = _torch()
    out = []
    for it in items:
        if isinstance(it, torch.Tensor):
            out.append(Arg(kind=ARG_BUFFER, buffer=it.data_ptr(), length=it.numel()))
            out.append(Arg(kind=ARG_INT32, i32=it.numel()))
        else:
            kind, v = it
            if kind == "buf":
                out.append(Arg(kind=ARG_BUFFER, buffer=v.data_ptr(), length=v.numel()))
            elif kind == "i32":
                out.append(Arg(kind=ARG_INT32, i32=int(v)))
            elif kind == "i64":
                out.append(Arg(kind=ARG_INT64, i64=int(v)))
            elif kind == "f32":
                out.append(Arg(kind=ARG_FLOAT32, f32=float(v)))
            elif kind == "f64":
                out.append(Arg(kind=ARG_FLOAT64, f64=float(v)))
            else:
                raise ValueError(f"unknown argument kind {kind!r}")
    return (Arg * len(out))(*out), len(out)


def run_source(source, kernel_name, block, grid, items, shared_mem=0, lang=LANG_HIP):
    """Plugin-level run_source on the default stream."""
    args, n = make_args(items)
    blk = (C.c_int * 3)(*block)
    grd = (C.c_int * 3)(*grid)
    check(lib.sarek_hip_run_source(source.encode(), lang, kernel_name.encode(), blk, grd,
                                   int(shared_mem), args, n))
    return lib.sarek_hip_last_run_path().decode()


def run_sources(launches):
    """launches: [(source, kernel_name, block, grid, items)] or [(..., shared_mem)]; one call for the
    sequence.  Returns (code paths, device launches made)."""
    arr = (Launch * max(len(launches), 1))()
    keep = []
    for l, item in zip(arr, launches):
        source, name, block, grid, items = item[:5]
        args, n = make_args(items)
        src, nm = source.encode(), name.encode()
        keep.append((args, src, nm))
        l.source, l.lang, l.kernel_name = src, LANG_HIP, nm
        l.block, l.grid = (C.c_int * 3)(*block), (C.c_int * 3)(*grid)
        l.shared_mem_bytes = item[5] if len(item) > 5 else 0
        l.args, l.n_args = args, n
    made, done = C.c_int(0), C.c_int(0)
    check(lib.sarek_hip_run_sources(arr, len(launches), C.byref(made), C.byref(done)))
    assert done.value == len(launches)
    return lib.sarek_hip_last_run_path().decode(), made.value


def rebuilt_source(ir_text, reduce=0, pad_bits=0):
    """The text run_source compiles for an IR of one of the rebuilt classes (an element-wise kernel, a tree sum or
    maximum with an expression in front); raises SarekHipError (unsupported) for any other IR."""
    needed = C.c_size_t(0)
    buf = C.create_string_buffer(1 << 16)
    rc = lib.sarek_hip_rebuilt_source(ir_text.encode(), reduce, pad_bits, buf, len(buf), C.byref(needed))
    if rc == E_BUFFER_TOO_SMALL:
        buf = C.create_string_buffer(needed.value + 1)
        rc = lib.sarek_hip_rebuilt_source(ir_text.encode(), reduce, pad_bits, buf, len(buf), C.byref(needed))
    check(rc)
    return buf.value.decode()


def generate_source(ir_text, block=None):
    blk = (C.c_int * 3)(*block) if block is not None else None
    needed = C.c_size_t(0)
    buf = C.create_string_buffer(1 << 16)
    rc = lib.sarek_hip_generate_source(ir_text.encode(), blk, buf, len(buf), C.byref(needed))
    if rc == E_BUFFER_TOO_SMALL:
        buf = C.create_string_buffer(needed.value + 1)
        rc = lib.sarek_hip_generate_source(ir_text.encode(), blk, buf, len(buf), C.byref(needed))
    check(rc)
    return buf.value.decode()
