(* ctypes-foreign stubs over libsarek_hip.so (include/sarek_hip.h).  One stub per C entry point
   the plugin uses; the comment above each group names what it stands in for in the CUDA plugin
   (sarek-cuda/Cuda_bindings.ml:39-525 binds the CUDA driver API and NVRTC function by function;
   here the driver, hiprtc, the IR lowering and the kernels sit behind one C ABI).

   Conventions of every symbol: int status (0 = success, > 0 = hipError_t, >= 1000 = hiprtc,
   < 0 = a SAREK_HIP_E_ code), the text of the last failure from sarek_hip_last_error, results through
   out-pointers, device pointers as void*. *)
open Ctypes
open Foreign

let library_names = ["libsarek_hip.so"]

let lib : Dl.library option Lazy.t =
  lazy
    (List.find_map
       (fun filename ->
         try Some (Dl.dlopen ~filename ~flags:[Dl.RTLD_LAZY; Dl.RTLD_GLOBAL])
         with _ -> None)
       library_names)

let is_available () = Lazy.force lib <> None

let get_lib () =
  match Lazy.force lib with
  | Some l -> l
  | None ->
      Hip_error.raise_error
        (Hip_error.library_not_found "libsarek_hip" library_names)

(* Symbols are looked up at first use, so that loading this module never fails on a machine
   without the library (Cuda_bindings.ml does the same with its lazy foreign values). *)
let bind name typ = lazy (foreign ~from:(get_lib ()) name typ)

(* status and error text *)
let abi_version = bind "sarek_hip_abi_version" (void @-> returning int)
let last_error = bind "sarek_hip_last_error" (void @-> returning string)
let status_name = bind "sarek_hip_status_name" (int @-> returning string)

(* BACKEND.name / version / execution_model / Intrinsics (Framework_sig.ml:107-143,285,314) *)
let backend_name = bind "sarek_hip_backend_name" (void @-> returning string)
let backend_version =
  bind "sarek_hip_backend_version" (ptr int @-> ptr int @-> ptr int @-> returning int)
let execution_model = bind "sarek_hip_execution_model" (void @-> returning int)
let intrinsic_register =
  bind "sarek_hip_intrinsic_register" (string @-> string @-> int @-> returning int)
let intrinsic_find =
  bind "sarek_hip_intrinsic_find"
    (string @-> ptr char @-> size_t @-> ptr int @-> ptr int @-> returning int)
let intrinsic_list =
  bind "sarek_hip_intrinsic_list" (ptr char @-> size_t @-> ptr size_t @-> returning int)

(* Device: cuInit / cuDeviceGet* / cuCtx* (Cuda_bindings.ml:85-180) *)
type device_info
let device_info : device_info structure typ = structure "sarek_hip_device_info"
let di_name = field device_info "name" (array 256 char)
let di_arch = field device_info "gcn_arch" (array 64 char)
let di_mem = field device_info "total_global_mem" uint64_t
let di_threads = field device_info "max_threads_per_block" int
let di_bdim = field device_info "max_block_dim" (array 3 int)
let di_gdim = field device_info "max_grid_dim" (array 3 int)
let di_lds = field device_info "shared_mem_per_block" int
let di_warp = field device_info "warp_size" int
let di_cus = field device_info "multiprocessor_count" int
let di_clock = field device_info "clock_rate_khz" int
let di_mclock = field device_info "memory_clock_rate_khz" int
let di_bus = field device_info "memory_bus_width_bits" int
let di_l2 = field device_info "l2_cache_size" int
let di_major = field device_info "compute_major" int
let di_minor = field device_info "compute_minor" int
let di_regs = field device_info "max_registers_per_block" int
let () = seal device_info

let init = bind "sarek_hip_init" (void @-> returning int)
let available = bind "sarek_hip_is_available" (void @-> returning int)
let device_count = bind "sarek_hip_device_count" (ptr int @-> returning int)
let device_info_size = bind "sarek_hip_device_info_size" (void @-> returning int)
let device_get_info =
  bind "sarek_hip_device_get_info" (int @-> ptr device_info @-> returning int)
let device_report =
  bind "sarek_hip_device_report" (ptr char @-> size_t @-> ptr size_t @-> ptr int @-> returning int)
let device_set_current = bind "sarek_hip_device_set_current" (int @-> returning int)
let device_get_current = bind "sarek_hip_device_get_current" (ptr int @-> returning int)
let device_synchronize = bind "sarek_hip_device_synchronize" (void @-> returning int)
let mem_get_info = bind "sarek_hip_mem_get_info" (ptr size_t @-> ptr size_t @-> returning int)
let driver_version = bind "sarek_hip_driver_version" (ptr int @-> returning int)

(* Memory: cuMemAlloc / cuMemFree / cuMemcpy* (Cuda_bindings.ml:184-300) *)
let mem_alloc = bind "sarek_hip_mem_alloc" (ptr (ptr void) @-> size_t @-> returning int)
let mem_free = bind "sarek_hip_mem_free" (ptr void @-> returning int)
let memcpy_htod =
  bind "sarek_hip_memcpy_htod" (ptr void @-> ptr void @-> size_t @-> returning int)
let memcpy_dtoh =
  bind "sarek_hip_memcpy_dtoh" (ptr void @-> ptr void @-> size_t @-> returning int)
let memcpy_dtod =
  bind "sarek_hip_memcpy_dtod" (ptr void @-> ptr void @-> size_t @-> returning int)
let memset_d8 = bind "sarek_hip_memset_d8" (ptr void @-> uchar @-> size_t @-> returning int)
(* pinned host blocks and device views of them (no counterpart in the CUDA plugin, whose
   alloc_zero_copy returns None, Cuda_plugin_base.ml:213-216) *)
let host_alloc = bind "sarek_hip_host_alloc" (ptr (ptr void) @-> size_t @-> returning int)
let host_free = bind "sarek_hip_host_free" (ptr void @-> returning int)
let mem_alloc_zero_copy =
  bind "sarek_hip_mem_alloc_zero_copy"
    (ptr void @-> size_t @-> ptr (ptr void) @-> ptr int @-> returning int)

(* Stream / Event: cuStream* / cuEvent* (Cuda_bindings.ml:300-420) *)
let stream_create = bind "sarek_hip_stream_create" (ptr (ptr void) @-> returning int)
let stream_destroy = bind "sarek_hip_stream_destroy" (ptr void @-> returning int)
let stream_synchronize = bind "sarek_hip_stream_synchronize" (ptr void @-> returning int)
let event_create = bind "sarek_hip_event_create" (ptr (ptr void) @-> returning int)
let event_destroy = bind "sarek_hip_event_destroy" (ptr void @-> returning int)
let event_record = bind "sarek_hip_event_record" (ptr void @-> ptr void @-> returning int)
let event_synchronize = bind "sarek_hip_event_synchronize" (ptr void @-> returning int)
let event_elapsed_ms =
  bind "sarek_hip_event_elapsed_ms" (ptr void @-> ptr void @-> ptr float @-> returning int)
let profiler_start = bind "sarek_hip_profiler_start" (void @-> returning int)
let profiler_stop = bind "sarek_hip_profiler_stop" (void @-> returning int)

(* Kernel: nvrtc* / cuModule* / cuLaunchKernel (Cuda_nvrtc.ml:141-229, Cuda_bindings.ml:420-470) *)
let kernel_compile =
  bind "sarek_hip_kernel_compile"
    (string @-> string @-> ptr (ptr void) @-> ptr char @-> size_t @-> returning int)
let kernel_compile_cached =
  bind "sarek_hip_kernel_compile_cached"
    (string @-> string @-> ptr (ptr void) @-> ptr char @-> size_t @-> returning int)
let kernel_clear_cache = bind "sarek_hip_kernel_clear_cache" (void @-> returning int)
let kernel_destroy = bind "sarek_hip_kernel_destroy" (ptr void @-> returning int)
let kernel_launch =
  bind "sarek_hip_kernel_launch"
    (ptr void @-> ptr uint @-> ptr uint @-> uint @-> ptr void @-> ptr (ptr void) @-> int
   @-> returning int)

(* Plugin level: generate_source / run_source (Cuda_plugin.ml:155-157,170-221) *)
type arg
let arg : arg structure typ = structure "sarek_hip_arg"
let a_kind = field arg "kind" int
let a_buffer = field arg "buffer" (ptr void)
let a_length = field arg "length" int64_t
let a_i32 = field arg "i32" int32_t
let a_i64 = field arg "i64" int64_t
let a_f32 = field arg "f32" float
let a_f64 = field arg "f64" double
let () = seal arg

let generate_source =
  bind "sarek_hip_generate_source"
    (string @-> ptr int @-> ptr char @-> size_t @-> ptr size_t @-> returning int)
let rebuilt_source =
  bind "sarek_hip_rebuilt_source"
    (string @-> int @-> uint32_t @-> ptr char @-> size_t @-> ptr size_t @-> returning int)
let run_source =
  bind "sarek_hip_run_source"
    (string @-> int @-> string @-> ptr int @-> ptr int @-> int @-> ptr arg @-> int
   @-> returning int)
let supports_lang = bind "sarek_hip_supports_lang" (int @-> returning int)
let set_specialisation = bind "sarek_hip_set_specialisation" (int @-> returning int)
let last_run_path = bind "sarek_hip_last_run_path" (void @-> returning string)
let set_tunable = bind "sarek_hip_set_tunable" (string @-> int64_t @-> returning int)

(* several run_source calls handed over at once, so that neighbouring kernels can share a pass *)
type launch
let launch : launch structure typ = structure "sarek_hip_launch"
let l_source = field launch "source" (ptr char)
let l_lang = field launch "lang" int
let l_name = field launch "kernel_name" (ptr char)
let l_block = field launch "block" (array 3 int)
let l_grid = field launch "grid" (array 3 int)
let l_shmem = field launch "shared_mem_bytes" int
let l_args = field launch "args" (ptr arg)
let l_nargs = field launch "n_args" int
let () = seal launch

let run_sources =
  bind "sarek_hip_run_sources" (ptr launch @-> int @-> ptr int @-> ptr int @-> returning int)

(* library kernel texts for Execute.run_source *)
let library_kernel_source =
  bind "sarek_hip_library_kernel_source"
    (string @-> ptr char @-> size_t @-> ptr size_t @-> ptr char @-> size_t @-> returning int)
let library_kernel_list =
  bind "sarek_hip_library_kernel_list" (ptr char @-> size_t @-> ptr size_t @-> returning int)

(* Hand-written kernels, for direct use on device pointers (Execute.run_source is the usual
   route: the plugin picks them by the tag of the source) *)
let gemm_f32 =
  bind "sarek_hip_gemm_f32"
    (ptr float @-> ptr float @-> ptr float @-> int @-> int @-> int @-> ptr void @-> returning int)
let gemm_bf16 =
  bind "sarek_hip_gemm_bf16"
    (ptr uint16_t @-> ptr uint16_t @-> ptr float @-> int @-> int @-> int @-> ptr void
   @-> returning int)
let gemm_f16 =
  bind "sarek_hip_gemm_f16"
    (ptr uint16_t @-> ptr uint16_t @-> ptr float @-> int @-> int @-> int @-> ptr void
   @-> returning int)
let gemm_f32_k_splits = bind "sarek_hip_gemm_f32_k_splits" (int @-> int @-> int @-> returning int)
let gemm16_tile = bind "sarek_hip_gemm16_tile" (int @-> int @-> int @-> returning int)
let gemm16_k_splits = bind "sarek_hip_gemm16_k_splits" (int @-> int @-> int @-> returning int)
let gemm_f16_bias_relu_rowsum =
  bind "sarek_hip_gemm_f16_bias_relu_rowsum"
    (ptr uint16_t @-> ptr uint16_t @-> ptr float @-> ptr float @-> ptr float @-> int @-> int
   @-> int @-> ptr void @-> returning int)
let cast_f32_to_bf16 =
  bind "sarek_hip_cast_f32_to_bf16"
    (ptr float @-> ptr uint16_t @-> int64_t @-> ptr void @-> returning int)
let cast_f32_to_f16 =
  bind "sarek_hip_cast_f32_to_f16"
    (ptr float @-> ptr uint16_t @-> int64_t @-> ptr void @-> returning int)
let triad =
  bind "sarek_hip_triad_f32"
    (ptr float @-> ptr float @-> ptr float @-> float @-> int64_t @-> ptr void @-> returning int)
let triad_sum_workspace_floats =
  bind "sarek_hip_triad_sum_workspace_floats" (int64_t @-> returning int64_t)
let triad_sum =
  bind "sarek_hip_triad_sum_f32"
    (ptr float @-> ptr float @-> ptr float @-> float @-> int64_t @-> ptr float @-> int64_t
   @-> ptr double @-> ptr void @-> returning int)
let triad_block256_sum =
  bind "sarek_hip_triad_block256_sum_f32"
    (ptr float @-> ptr float @-> ptr float @-> float @-> int64_t @-> ptr float @-> ptr void
   @-> returning int)
let triad_block256_max =
  bind "sarek_hip_triad_block256_max_f32"
    (ptr float @-> ptr float @-> ptr float @-> float @-> int64_t @-> float @-> ptr float @-> ptr void
   @-> returning int)
(* the same sum for callers that may not allocate: n <= triad_sum_static_max_n, the partial
   sums live inside the library's device image *)
let triad_sum_static_max_n =
  bind "sarek_hip_triad_sum_static_max_n" (void @-> returning int64_t)
let triad_sum_static =
  bind "sarek_hip_triad_sum_f32_static"
    (ptr float @-> ptr float @-> ptr float @-> float @-> int64_t @-> ptr double @-> ptr void
   @-> returning int)
let reduce_sum_block256 =
  bind "sarek_hip_reduce_sum_block256_f32"
    (ptr float @-> ptr float @-> int64_t @-> ptr void @-> returning int)
let dot_block256 =
  bind "sarek_hip_dot_block256_f32"
    (ptr float @-> ptr float @-> ptr float @-> int64_t @-> ptr void @-> returning int)
let reduce_max_block256 =
  bind "sarek_hip_reduce_max_block256_f32"
    (ptr float @-> ptr float @-> int64_t @-> float @-> ptr void @-> returning int)
let fold_partials =
  bind "sarek_hip_fold_partials_f64"
    (ptr float @-> int64_t @-> ptr double @-> ptr void @-> returning int)
let copy_f32 =
  bind "sarek_hip_copy_f32" (ptr float @-> ptr float @-> int64_t @-> ptr void @-> returning int)
let transpose_f32 =
  bind "sarek_hip_transpose_f32"
    (ptr float @-> ptr float @-> int @-> int @-> ptr void @-> returning int)
let stencil_2d_f32 =
  bind "sarek_hip_stencil_2d_f32"
    (ptr float @-> ptr float @-> int @-> int @-> ptr void @-> returning int)
let conv2d_f32 =
  bind "sarek_hip_conv2d_f32"
    (ptr float @-> ptr float @-> int @-> int @-> ptr void @-> returning int)
let histogram_i32 =
  bind "sarek_hip_histogram_i32"
    (ptr int32_t @-> ptr int32_t @-> int64_t @-> int @-> ptr void @-> returning int)
let radix_histogram_i32 =
  bind "sarek_hip_radix_histogram_i32"
    (ptr int32_t @-> ptr int32_t @-> int64_t @-> int @-> int @-> ptr void @-> returning int)
let radix_scatter_i32 =
  bind "sarek_hip_radix_scatter_i32"
    (ptr int32_t @-> int64_t @-> ptr int32_t @-> ptr int32_t @-> int64_t @-> int @-> int
   @-> ptr void @-> returning int)

(* Persistent code-object cache = Framework_cache (same directory rule, same MD5 key,
   sarek/framework/Framework_cache.ml:90-141).  The compile path uses it by itself; these are
   for Framework_cache-style callers and for the statistics. *)
let cache_dir = bind "sarek_hip_cache_dir" (ptr char @-> size_t @-> returning int)
let cache_compute_key =
  bind "sarek_hip_cache_compute_key" (string @-> string @-> string @-> ptr char @-> returning int)
let cache_get =
  bind "sarek_hip_cache_get"
    (string @-> ptr void @-> size_t @-> ptr size_t @-> ptr int @-> returning int)
let cache_put = bind "sarek_hip_cache_put" (string @-> ptr void @-> size_t @-> returning int)
let cache_get_stats = bind "sarek_hip_cache_get_stats" (ptr int64_t @-> returning int)
let cache_reset_stats = bind "sarek_hip_cache_reset_stats" (void @-> returning int)

(* diagnostic: (shader cycles, wall-clock ticks) per workgroup of the MFMA GEMMs *)
let set_clock_probe =
  bind "sarek_hip_set_clock_probe" (ptr uint64_t @-> int64_t @-> ptr int64_t @-> returning int)
