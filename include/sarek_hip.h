/*
 * sarek_hip.h - C ABI of libsarek_hip.so, the native half of the `sarek-hip`
 * backend plugin for Sarek/SPOC on AMD Instinct MI355X (gfx950).
 *
 * The OCaml side of the plugin (Hip_bindings / Hip_api / Hip_plugin) binds
 * these symbols with ctypes-foreign, exactly as sarek-cuda binds libcuda and
 * libnvrtc (sarek-cuda/Cuda_bindings.ml:39-81, sarek-cuda/Cuda_nvrtc.ml:99-137).
 *
 * Conventions (same as the CUDA driver symbols the reference binds,
 * sarek-cuda/Cuda_types.ml:249): every function returns an `int` status,
 * 0 = success; results come back through caller-allocated out-pointers;
 * strings are NUL terminated; handles are opaque pointers; device pointers
 * are plain `void*`; no callbacks into the caller.  Positive status values
 * are hipError_t / hiprtcResult+1000 codes, negative values are
 * SAREK_HIP_E_* below.  `sarek_hip_last_error()` returns a thread-local
 * human-readable message for the last non-zero status.
 *
 * All launches are asynchronous on the given stream (NULL = the default
 * stream); copies are synchronous, as in the reference
 * (sarek-cuda/Cuda_api.ml:224-243).
 */
#ifndef SAREK_HIP_H
#define SAREK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 3: entry points added since 2 (sarek_hip_run_sources, sarek_hip_execute_run_pipeline, sarek_hip_rebuilt_source,
 * the library kernels, the stencil, layout and histogram kernels, sarek_hip_is_measurement_build); the measurement
 * knobs and the in-kernel clock probe left the product library; nothing that version 2 declared changed its meaning. */
#define SAREK_HIP_ABI_VERSION 3

/* Library-level status codes (negative; HIP codes are positive). */
#define SAREK_HIP_OK 0
#define SAREK_HIP_E_INVALID_ARG (-1)    /* NULL pointer, negative size, ... */
#define SAREK_HIP_E_UNSUPPORTED (-2)    /* source language / shape not supported */
#define SAREK_HIP_E_COMPILE (-3)        /* hiprtc compilation failed; see log */
#define SAREK_HIP_E_NO_DEVICE (-4)      /* no gfx950-class device selected */
#define SAREK_HIP_E_WORKSPACE (-5)      /* caller workspace too small */
#define SAREK_HIP_E_PARSE (-6)          /* malformed IR text */
#define SAREK_HIP_E_CODEGEN (-7)        /* IR construct the lowering rejects */
#define SAREK_HIP_E_BUFFER_TOO_SMALL (-8)

typedef void *sarek_hip_stream;  /* hipStream_t */
typedef void *sarek_hip_event;   /* hipEvent_t */
typedef struct sarek_hip_kernel_s *sarek_hip_kernel; /* compiled module+function */

int sarek_hip_abi_version(void);
const char *sarek_hip_last_error(void);
const char *sarek_hip_status_name(int status);

/* BACKEND.name / version / execution_model (spoc/framework/Framework_sig.ml:137-143,285): "HIP",
 * (1, 0, 0), JIT.  execute_direct does not exist here: a JIT backend refuses it
 * (sarek-cuda/Cuda_plugin.ml:158-161).                                                         */
enum { SAREK_HIP_EXECUTION_JIT = 0, SAREK_HIP_EXECUTION_DIRECT = 1, SAREK_HIP_EXECUTION_CUSTOM = 2 };
const char *sarek_hip_backend_name(void);
int sarek_hip_backend_version(int *major, int *minor, int *patch);
int sarek_hip_execution_model(void);
/* BACKEND.Intrinsics, an INTRINSIC_REGISTRY (Framework_sig.ml:107-119): name -> device code and
 * convergence.  Preloaded with the thirteen entries of sarek-cuda/Cuda_plugin.ml:47-143 in HIP
 * spelling (warp_barrier is a wave barrier); register replaces an entry of the same name; list
 * writes the names sorted, one per line (*needed = bytes incl. NUL, may be asked with out = NULL,
 * which returns SAREK_HIP_E_BUFFER_TOO_SMALL).                                                  */
enum { SAREK_HIP_CONVERGENCE_UNIFORM = 0, SAREK_HIP_CONVERGENCE_DIVERGENT = 1, SAREK_HIP_CONVERGENCE_SYNC = 2 };
int sarek_hip_intrinsic_register(const char *name, const char *codegen, int convergence);
int sarek_hip_intrinsic_find(const char *name, char *codegen /* may be NULL */, size_t cap,
                             int *convergence /* may be NULL */, int *found);
int sarek_hip_intrinsic_list(char *out, size_t cap, size_t *needed);

/* ---------------------------------------------------------------------- */
/* Device  (replaces the cuInit, cuDeviceGet.. and cuCtx.. groups,
 * sarek-cuda/Cuda_api.ml:35-179)                                            */

typedef struct {
  char name[256];
  char gcn_arch[64];            /* e.g. "gfx950:sramecc+:xnack-" */
  uint64_t total_global_mem;    /* bytes */
  int max_threads_per_block;
  int max_block_dim[3];
  int max_grid_dim[3];
  int shared_mem_per_block;     /* LDS bytes usable by one workgroup */
  int warp_size;                /* 64 on CDNA */
  int multiprocessor_count;     /* compute units */
  int clock_rate_khz;
  int memory_clock_rate_khz;
  int memory_bus_width_bits;
  int l2_cache_size;
  int compute_major, compute_minor;
  int max_registers_per_block;  /* Framework_sig.capabilities.max_registers_per_block (the CUDA plugin
                                   puts a constant 65536 there, sarek-cuda/Cuda_plugin_base.ml:190)      */
} sarek_hip_device_info;

int sarek_hip_init(void);                       /* hipInit(0); idempotent */
int sarek_hip_is_available(void);               /* 1/0, never fails (Framework_registry.ml:77-87) */
int sarek_hip_device_count(int *count);
int sarek_hip_device_get_info(int device, sarek_hip_device_info *out);
/* sizeof(sarek_hip_device_info) as this library was built: sarek_hip_device_get_info writes that many
 * bytes, so a binding checks its own struct against it once (no counterpart in the reference, whose
 * ctypes layer reads one attribute per call, sarek-cuda/Cuda_api.ml:77-129).                         */
int sarek_hip_device_info_size(void);
/* The text tools/device_info.ml:45-93 prints (banner, "Found N device(s)", one block per device as its
 * print_device_info :16-43 lays it out, usage lines; or its "No devices found" text) for the devices of this
 * backend.  *device_count (may be NULL) gets the number of devices: the tool exits 1 when it is 0.
 * SAREK_HIP_E_BUFFER_TOO_SMALL with *needed set when the text does not fit.  Never fails for lack of a GPU. */
int sarek_hip_device_report(char *out, size_t cap, size_t *needed, int *device_count);
int sarek_hip_device_set_current(int device);
int sarek_hip_device_get_current(int *device);
int sarek_hip_device_synchronize(void);         /* Transfer.flush -> Device.synchronize */
int sarek_hip_mem_get_info(size_t *free_bytes, size_t *total_bytes);
int sarek_hip_driver_version(int *version);

/* ---------------------------------------------------------------------- */
/* Memory  (replaces cuMemAlloc/Free/Memcpy.., sarek-cuda/Cuda_api.ml:183-244).
 * `sarek_hip_mem_free(NULL)` and a double free of the same pointer are
 * accepted: the reference frees buffers both explicitly and from a GC
 * finaliser that may run late (sarek/core/Gpu_memory.ml:163-178).  The library
 * recognises a freed buffer by its ADDRESS: a second free that arrives after
 * sarek_hip_mem_alloc has handed the same address out again frees the new
 * buffer.  A binding therefore keeps its own `freed` flag per buffer record and
 * calls this once (the reference's finaliser does: Gpu_memory.ml:166-172); the
 * tolerance here only covers a late free of an address not yet reused.        */
int sarek_hip_mem_alloc(void **dptr, size_t bytes);
int sarek_hip_mem_free(void *dptr);
/* Memory.host_ptr_to_device / device_to_host_ptr (sarek-cuda/Cuda_api.ml:207-230, called
 * with a vector's whole host block by sarek/core/Transfer.ml:228-333).  Synchronous:
 * the copy is complete on return, and it starts only after the device has finished
 * the work it was given before.  Larger copies from or to ordinary (pageable)
 * host memory (uploads from 12 MiB, downloads from 2 MiB) are pipelined through
 * pinned staging slots by 4 host threads, three of them helpers that sleep
 * between copies (64 MiB of pinned memory per device, kept until the process
 * ends); tunables "transfer.threads" (0 = always the driver's own copy),
 * "transfer.chunk_kib" (slot size), "transfer.min_up_kib", "transfer.min_down_kib". */
int sarek_hip_memcpy_htod(void *dst_device, const void *src_host, size_t bytes);
int sarek_hip_memcpy_dtoh(void *dst_host, const void *src_device, size_t bytes);
/* Pinned host memory for a vector's host block (the reference allocates it as an
 * ordinary Bigarray, sarek/core/Vector_storage.ml:22; wrapping a block from here with
 * Ctypes.bigarray_of_ptr lets the two copies above run at the full PCIe rate with no
 * staging).  `sarek_hip_host_free(NULL)` is accepted.                           */
int sarek_hip_host_alloc(void **host_ptr, size_t bytes);
int sarek_hip_host_free(void *host_ptr);
/* Memory.alloc_zero_copy (spoc/framework/Framework_sig.ml; used by
 * sarek/core/Transfer.ml:85-126, 185-203): *supported = 1 and *dptr = the device's view
 * of the host block when `host_ptr` lies in a block from sarek_hip_host_alloc (then
 * kernels read and write the host block over the link, and the vector's transfers are
 * no-ops); *supported = 0 (the reference's None) for any other memory, and the caller
 * allocates and copies.  The view needs no free (sarek_hip_mem_free ignores it).     */
int sarek_hip_mem_alloc_zero_copy(void *host_ptr, size_t bytes, void **dptr, int *supported);
int sarek_hip_memcpy_dtod(void *dst_device, const void *src_device, size_t bytes);
int sarek_hip_memset_d8(void *dst_device, unsigned char value, size_t bytes);

/* ---------------------------------------------------------------------- */
/* Stream / Event  (sarek-cuda/Cuda_api.ml:248-293).  Default priority only. */
int sarek_hip_stream_create(sarek_hip_stream *out);
int sarek_hip_stream_destroy(sarek_hip_stream s);
int sarek_hip_stream_synchronize(sarek_hip_stream s);
int sarek_hip_event_create(sarek_hip_event *out);
int sarek_hip_event_destroy(sarek_hip_event e);
int sarek_hip_event_record(sarek_hip_event e, sarek_hip_stream s);
int sarek_hip_event_synchronize(sarek_hip_event e);
int sarek_hip_event_elapsed_ms(sarek_hip_event start, sarek_hip_event stop, float *ms);

/* BACKEND.enable_profiling / disable_profiling (cuProfilerStart / cuProfilerStop,
 * sarek-cuda/Cuda_plugin_base.ml:294-300; optional symbols there,
 * sarek-cuda/Cuda_bindings.ml:497-525): the range markers an attached profiler
 * honours.  Like the reference, the result of the underlying call is ignored; both
 * always return SAREK_HIP_OK.                                                  */
int sarek_hip_profiler_start(void);
int sarek_hip_profiler_stop(void);

/* ---------------------------------------------------------------------- */
/* Kernel JIT + launch  (replaces the nvrtc.., cuModule.. groups and cuLaunchKernel,
 * sarek-cuda/Cuda_nvrtc.ml:263-389, sarek-cuda/Cuda_api.ml:315-486).
 * `source` is HIP C++ text; it is compiled by hiprtc for the current
 * device's architecture (--offload-arch=<gcnArchName>), -O3, with wrapping
 * signed arithmetic (-fwrapv: OCaml's Int32 / Int64 wrap) and without packed
 * FP32 instructions.  A text that names Float.x, Int32.x or Int64.x without
 * declaring an object of that name is given OCaml's constants of those modules
 * in front (a value outside the kernel lowers to a variable of its name,
 * sarek/ppx/Sarek_lower_ir.ml:378-380; line numbers in the log then count
 * those lines).  On failure the compiler log is copied into `log` (truncated
 * to log_len-1 bytes).                                                      */
int sarek_hip_kernel_compile(const char *source, const char *kernel_name,
                             sarek_hip_kernel *out, char *log, size_t log_len);
/* Same, memoised on (device, hash(source), kernel_name)
 * (Kernel.compile_cached, sarek-cuda/Cuda_api.ml:399-412).                 */
int sarek_hip_kernel_compile_cached(const char *source, const char *kernel_name,
                                    sarek_hip_kernel *out, char *log, size_t log_len);
int sarek_hip_kernel_clear_cache(void);
int sarek_hip_kernel_destroy(sarek_hip_kernel k);
/* params: array of n_params pointers to the argument values, the
 * cuLaunchKernel convention (sarek-cuda/Cuda_api.ml:473-486).              */
int sarek_hip_kernel_launch(sarek_hip_kernel k, const unsigned grid[3], const unsigned block[3],
                            unsigned shared_mem_bytes, sarek_hip_stream stream, void **params,
                            int n_params);

/* ---------------------------------------------------------------------- */
/* Plugin level: what Hip_plugin.generate_source / Hip_plugin.run_source call
 * (sarek-cuda/Cuda_plugin.ml:155-157,174-220).                             */

/* Source language tags, numbered like Framework_sig.source_lang
 * (spoc/framework/Framework_sig.ml:72-77) with HIP_Source appended.        */
enum {
  SAREK_HIP_LANG_CUDA_SOURCE = 0,
  SAREK_HIP_LANG_OPENCL_SOURCE = 1,
  SAREK_HIP_LANG_PTX = 2,
  SAREK_HIP_LANG_SPIR_V = 3,
  SAREK_HIP_LANG_GLSL_SOURCE = 4,
  SAREK_HIP_LANG_HIP_SOURCE = 5
};

/* One element of Framework_sig.run_source_arg list
 * (spoc/framework/Framework_sig.ml:88-96).                                 */
enum {
  SAREK_HIP_ARG_BUFFER = 0,
  SAREK_HIP_ARG_INT32 = 1,
  SAREK_HIP_ARG_INT64 = 2,
  SAREK_HIP_ARG_FLOAT32 = 3,
  SAREK_HIP_ARG_FLOAT64 = 4
};
typedef struct {
  int kind;
  void *buffer;     /* SAREK_HIP_ARG_BUFFER: device pointer */
  int64_t length;   /* SAREK_HIP_ARG_BUFFER: vector length in elements */
  int32_t i32;
  int64_t i64;
  float f32;
  double f64;
} sarek_hip_arg;

/* IR text (the s-expression form written by the plugin's IR serialiser) ->
 * HIP source for gfx950.  When the IR is one of the recognised hot kernels
 * (tiled matmul, stream triad, block-256 tree sum / dot product) and
 * specialisation is enabled, the source carries a leading
 * `// sarek-hip-specialise: <tag>` line that run_source honours; the plain
 * lowering always follows, so the text is valid HIP either way.
 * block: launch block dims or NULL (BACKEND.generate_source ?block).  When given,
 * the size of a shared array written in terms of the block dimensions (an unsized
 * let%shared lowers to block_dim_x elements, sarek/ppx/Sarek_lower_ir.ml:496-507) is
 * emitted as the constant a __shared__ declaration needs; the reference's generators
 * leave blockDim.x there, which no device compiler accepts.
 * The text is what sarek-cuda/Sarek_ir_cuda.ml:751-786 prints for the same IR -- byte for
 * byte on the reference's golden kernels -- except where that text does not compile or
 * computes something else than the CPU backends do: a name bound again gets a variable of
 * its own (x_2, ...), a `for` bound the body may change is evaluated once, a match used as
 * a value binds its cases' variables, variable patterns and lets of type unit are taken,
 * infinities / NaN / the least integers / whole-valued doubles are spelled so that they
 * keep their value and type, a thread's own arrays start at zero, the standard library's
 * logical shifts give a signed value.
 * Writes at most out_len bytes incl. NUL; *needed gets the full size.          */
int sarek_hip_generate_source(const char *ir_text, const int block[3], char *out, size_t out_len,
                              size_t *needed);
/* The text run_source compiles in place of the generated kernel when the IR is of one of the classes
 * it rebuilds from the kernel's own expression: an element-wise kernel (reduce = 0: alone, 1: with the
 * block-256 sums of its output, 2: with their maxima, slots past n counting as the f32 with the bits
 * pad_bits), or a block-256 tree sum / maximum with an expression where the reference's kernels
 * (benchmarks/bench_reduction.ml:62-96, bench_reduction_max.ml:18-100) read their input (reduce and
 * pad_bits ignored).  For diagnostics and for compiling the texts ahead of time; no counterpart in the
 * reference.  SAREK_HIP_E_UNSUPPORTED when the IR is of no such class.  Buffer convention as above.     */
int sarek_hip_rebuilt_source(const char *ir_text, int reduce, uint32_t pad_bits, char *out, size_t out_len,
                             size_t *needed);

/* Compile (cached) + bind + launch on the default stream.  Only
 * SAREK_HIP_LANG_HIP_SOURCE and SAREK_HIP_LANG_CUDA_SOURCE (treated as HIP
 * text) are accepted; others return SAREK_HIP_E_UNSUPPORTED.  A specialise
 * tag reroutes the call to the matching hand-written kernel when (1) the text
 * is one this library wrote -- byte for byte a text sarek_hip_generate_source
 * returned in this process, or a library kernel's text -- and (2) block, grid
 * and the arguments fit what that kernel assumes (the launch covers the
 * problem, output buffers do not lie over inputs).  Anything else, a caller's
 * own program that starts with the same line included, is compiled and
 * launched as written.                                                      */
int sarek_hip_run_source(const char *source, int lang, const char *kernel_name,
                         const int block[3], const int grid[3], int shared_mem_bytes,
                         const sarek_hip_arg *args, int n_args);

/* Library kernels: complete HIP sources, each with a specialise tag on its first line, for the
 * operations that have no kernel in the reference's suite.  A caller passes the text to
 * sarek_hip_run_source / sarek_hip_execute_run_source (Execute.run_source ~lang:HIP_Source,
 * sarek/sarek/Execute.ml:613-651, as sarek/tests/e2e/test_external_kernel.ml:46-62 does with its
 * own text) with lengths injected; with specialisation on and arguments that fit, the hand-written
 * kernel runs, otherwise the text itself is compiled and gives the same result under the launch
 * geometry stated in its comment.  The hand-written kernel stands in for the library's own text only (compared
 * byte for byte): a caller's text that merely starts with the same tag line is compiled as written.
 * Names, arguments (v = device pointer + int32 length) and geometry:
 *   gemm_bf16, gemm_f16          (a v, b v, c v, m, n, k)   a, b: 2-byte custom elements (bit patterns),
 *                                c f32; 2-D launch, one thread per element of C
 *   gemm_f16_bias_relu_rowsum    (a v, b v, bias v, y v, rowsum v, m, n, k)   1-D launch, any size
 *   triad_sum_f32                (a v, b v, c v, sum v (float64, >= 1 element), scalar f32, n)
 *                                one 1-D workgroup of a power-of-two size up to 1024
 * source / entry: buffers for the text and for the kernel_name to launch it under; *source_needed
 * gets the text's size incl. NUL (SAREK_HIP_E_BUFFER_TOO_SMALL when it does not fit).            */
int sarek_hip_library_kernel_source(const char *name, char *source, size_t source_cap, size_t *source_needed,
                                    char *entry /* may be NULL */, size_t entry_cap);
int sarek_hip_library_kernel_list(char *out, size_t cap, size_t *needed);   /* names, space separated */

/* A sequence of run_source calls made in one: what a plugin does for a list of kernels launched one after the
 * other on the default stream (no counterpart in BACKEND, whose run_source takes one kernel:
 * spoc/framework/Framework_sig.ml:324-336).  The results are those of the separate calls; two neighbouring
 * entries that one hand-written kernel computes in a single pass over the data (a source tagged
 * stream_triad_f32 followed by one tagged reduce_sum_block256_f32 that reads the vector the first writes,
 * over the same n) are launched as that kernel.  *device_launches (may be NULL): launches made; *completed
 * (may be NULL): entries fully served, also when the call fails part of the way.  sarek_hip_last_run_path()
 * joins the paths with ';', a shared launch reads "<tag>+<tag>".                                              */
typedef struct sarek_hip_launch {
  const char *source;
  int lang;
  const char *kernel_name;
  int block[3], grid[3];
  int shared_mem_bytes;
  const sarek_hip_arg *args;
  int n_args;
} sarek_hip_launch;
int sarek_hip_run_sources(const sarek_hip_launch *launches, int n_launches, int *device_launches, int *completed);

/* 1 (default) / 0: honour specialise tags.  Also read once from the
 * environment variable SAREK_HIP_SPECIALISE (0 disables).                  */
int sarek_hip_set_specialisation(int enabled);
/* Name of the code path the last sarek_hip_run_source call took on this
 * thread: "jit" or the specialise tag.                                     */
const char *sarek_hip_last_run_path(void);

/* ---------------------------------------------------------------------- */
/* The host side of a launch, for callers without the reference's OCaml core:
 * vectors with a host block, per-device buffers and a location state
 * (sarek/core/Vector.ml, Vector_types.ml:198-203), the transfers between them
 * (sarek/core/Transfer.ml:173-388) and the dispatcher (sarek/sarek/Execute.ml:188-216,
 * 321-335, 520-543, 613-651).  Semantics follow the reference state by state.     */
typedef struct sarek_hip_vector_s *sarek_hip_vector;
enum {                                  /* Vector_types.scalar_kind + Custom            */
  SAREK_HIP_KIND_FLOAT32 = 0, SAREK_HIP_KIND_FLOAT64 = 1, SAREK_HIP_KIND_INT32 = 2,
  SAREK_HIP_KIND_INT64 = 3, SAREK_HIP_KIND_CHAR = 4, SAREK_HIP_KIND_COMPLEX32 = 5,
  SAREK_HIP_KIND_CUSTOM = 6
};
enum {                                  /* Vector_types.location                         */
  SAREK_HIP_LOC_CPU = 0, SAREK_HIP_LOC_GPU = 1, SAREK_HIP_LOC_BOTH = 2,
  SAREK_HIP_LOC_STALE_CPU = 3,          /* the device copy is the good one               */
  SAREK_HIP_LOC_STALE_GPU = 4           /* the host copy is the good one                 */
};
/* Vector.create / create_custom: host block of `length` elements, contents unspecified,
 * location CPU.  pinned = 1 takes the block from sarek_hip_host_alloc; pinned = 2 does
 * too and makes the vector zero-copy: its device buffer is the host block itself
 * (sarek_hip_mem_alloc_zero_copy), uploads and downloads move nothing (a download
 * waits for the device), the location states change as for any vector.             */
int sarek_hip_vector_create(int kind, int64_t length, int64_t custom_elem_size, int pinned,
                            sarek_hip_vector *out);
int sarek_hip_vector_destroy(sarek_hip_vector v);          /* device buffers; the host block with its last vector */
/* Vector.id (sarek/core/Vector_storage.ml: next_id; the first vector of a process is #1) and
 * Vector.to_string (sarek/core/Vector.ml:181-195), "Vector#3<Float32>[1024] @ Both(<device name>)";
 * a custom vector's kind prints as Custom(<element size>).                                          */
int64_t sarek_hip_vector_id(sarek_hip_vector v);
int sarek_hip_vector_to_string(sarek_hip_vector v, char *buf, size_t cap);
/* Vector.fill (Vector.ml:222-233): every element set to *elem, then as a host write (Both / GPU ->
 * Stale_GPU; a Stale_CPU vector stays Stale_CPU, its next download overwrites the fill).            */
int sarek_hip_vector_fill(sarek_hip_vector v, const void *elem);
/* Vector.copy (Vector.ml:245-249): a new vector on the CPU with the host data, downloaded first
 * when the host copy is stale and auto-sync is on; no device buffers.                               */
int sarek_hip_vector_copy(sarek_hip_vector v, sarek_hip_vector *out);
/* Vector.sub_vector (Vector.ml:259-267, Vector_storage.ml:215-259): `len` elements of v's HOST block
 * from `start`, shared with v (and kept alive by either); device buffers and location (CPU) are the
 * sub-vector's own.  ok_range: elements safe to read (negative = len), ko_range: elements not to
 * write; both are only recorded.  Out of range: SAREK_HIP_E_INVALID_ARG with the reference's text. */
int sarek_hip_vector_sub(sarek_hip_vector v, int64_t start, int64_t len, int64_t ok_range, int64_t ko_range,
                         sarek_hip_vector *out);
/* Vector.is_sub / get_sub_meta / depth / parent_id / sub_start / sub_ok_range / sub_ko_range
 * (Vector.ml:252-257,300-317); any out pointer but is_sub may be NULL.                              */
int sarek_hip_vector_sub_meta(sarek_hip_vector v, int *is_sub, int64_t *parent_id, int64_t *start,
                              int64_t *ok_range, int64_t *ko_range, int *depth);
/* Vector.partition (Vector.ml:273-281): n_devices sub-vectors covering v, the first length mod n one
 * element longer; sub-vector i is Stale_GPU of devices[i].  Nothing is copied.                      */
int sarek_hip_vector_partition(sarek_hip_vector v, int n_devices, const int *devices, sarek_hip_vector *out);
/* Vector.blit (Vector.ml:500-517): len elements from src[src_off..] to dst[dst_off..] on the host,
 * in ascending order; src is downloaded first if stale (auto-sync), dst is marked as written.       */
int sarek_hip_vector_blit(sarek_hip_vector src, int64_t src_off, sarek_hip_vector dst, int64_t dst_off,
                          int64_t len);
int64_t sarek_hip_vector_length(sarek_hip_vector v);
int64_t sarek_hip_vector_elem_size(sarek_hip_vector v);
int sarek_hip_vector_kind(sarek_hip_vector v);
int sarek_hip_vector_location(sarek_hip_vector v, int *location, int *device /* may be NULL */);
void *sarek_hip_vector_host_ptr(sarek_hip_vector v);       /* Vector.host_ptr: raw, no sync  */
int sarek_hip_vector_device_ptr(sarek_hip_vector v, void **dptr);   /* NULL: no buffer yet */
int sarek_hip_vector_set_auto_sync(sarek_hip_vector v, int enabled);
int sarek_hip_vector_auto_sync(sarek_hip_vector v);         /* Vector.auto_sync: 1 / 0; NULL vector: 0 */
/* Vector.get / Vector.set (Vector.ml:80-109): bounds-checked ("Vector.get: index I out
 * of bounds [0, N)" with SAREK_HIP_E_INVALID_ARG); get first downloads a Stale_CPU
 * vector when auto-sync is on; set marks a Both / GPU vector Stale_GPU and does not
 * download first.  read / write are the same for a range of elements (Vector.to_array,
 * a loop of Vector.set).                                                           */
int sarek_hip_vector_get(sarek_hip_vector v, int64_t index, void *out_elem);
int sarek_hip_vector_set(sarek_hip_vector v, int64_t index, const void *elem);
int sarek_hip_vector_read(sarek_hip_vector v, void *dst, int64_t first, int64_t count);
int sarek_hip_vector_write(sarek_hip_vector v, const void *src, int64_t first, int64_t count);
/* Transfer.set_auto, to_device (to the current device), to_cpu ?force, sync,
 * free_all_buffers, flush.                                                         */
int sarek_hip_transfer_set_auto(int enabled);
int sarek_hip_transfer_to_device(sarek_hip_vector v);
int sarek_hip_transfer_to_cpu(sarek_hip_vector v, int force);
int sarek_hip_transfer_sync(sarek_hip_vector v);
int sarek_hip_transfer_free_buffers(sarek_hip_vector v);
int sarek_hip_transfer_flush(void);
/* Gpu_memory (sarek/core/Gpu_memory.ml:20-141): bookkeeping of the device memory that vectors
 * hold, kept by the native Vector layer as the reference keeps it from Transfer.ensure_buffer
 * (track_alloc, Transfer.ml:218), free_buffer / free_all_buffers (track_free, :359,375) and the
 * vector's finaliser (gc_free_count, gc_freed_bytes; here sarek_hip_vector_destroy, which is what a
 * host language's finaliser calls).  with_retry is the reference's retry of a failed allocation
 * after a collection (Gpu_memory.ml:123-141): up to three attempts, the reclaim callback between
 * them (attempt 1 where the reference runs Gc.full_major, 2 where it runs Gc.compact), the first
 * failure's status and message returned when all three fail, one attempt when auto_gc is off.
 * The native Vector layer allocates its device buffers through it.  A host with a garbage collector
 * registers the callback; without one the retries find nothing new and the first error comes back.
 * With the OCaml veneer the reference's own Gpu_memory module does all of this and these entry
 * points stay unused.                                                                          */
typedef struct sarek_hip_gpu_memory_stats_t {
  int64_t current_bytes, peak_bytes, alloc_count, free_count, gc_free_count, gc_freed_bytes, retry_count;
} sarek_hip_gpu_memory_stats_t;
typedef void (*sarek_hip_reclaim_fn)(void *ctx, int attempt);
typedef int (*sarek_hip_attempt_fn)(void *ctx);          /* a status: 0 = success */
void sarek_hip_gpu_memory_set_auto_gc(int enabled);
int sarek_hip_gpu_memory_get_auto_gc(void);
void sarek_hip_gpu_memory_track_alloc(int64_t bytes);
void sarek_hip_gpu_memory_track_free(int64_t bytes);
int64_t sarek_hip_gpu_memory_usage(void);
int64_t sarek_hip_gpu_memory_peak_usage(void);
int sarek_hip_gpu_memory_stats(sarek_hip_gpu_memory_stats_t *out);
void sarek_hip_gpu_memory_reset_stats(void);
void sarek_hip_gpu_memory_set_reclaim(sarek_hip_reclaim_fn fn, void *ctx);
void sarek_hip_gpu_memory_trigger_gc(void);                /* Gpu_memory.trigger_gc: the callback, attempt 1 */
int sarek_hip_gpu_memory_with_retry(sarek_hip_attempt_fn attempt, void *ctx);
/* Execute.vector_arg (Execute.ml:28-35; Int goes as INT32, as expand_to_run_source_args sends it). */
enum { SAREK_HIP_VARG_VEC = 0, SAREK_HIP_VARG_INT32 = 1, SAREK_HIP_VARG_INT64 = 2,
       SAREK_HIP_VARG_FLOAT32 = 3, SAREK_HIP_VARG_FLOAT64 = 4 };
typedef struct sarek_hip_varg {
  int kind;
  sarek_hip_vector vec;
  int32_t i32;
  int64_t i64;
  float f32;
  double f64;
} sarek_hip_varg;
/* Execute.run_vectors (Execute.ml:520-543): uploads what is not on the device yet,
 * lowers the IR (one lowering per distinct text is kept), expands vectors to
 * (buffer, int32 length), launches through sarek_hip_run_source under the kernel's own
 * name, then marks the Both vectors Stale_CPU.  A kernel the lowering refuses is
 * "Backend failed to generate source" (Execute.ml:257-263).  The arguments are held to the
 * kernel's parameter list first -- their number, vector or scalar, int32 / int64 / float32 /
 * float64, a vector's element size -- and a mismatch is SAREK_HIP_E_INVALID_ARG naming the
 * argument, with nothing launched (the reference passes on what it is given, Execute.ml:197-216,
 * and the kernel then reads a parameter block of another layout).                  */
int sarek_hip_execute_run_vectors(const char *ir_text, const int block[3], const int grid[3],
                                  int shared_mem_bytes, const sarek_hip_varg *args, int n_args);
/* A sequence of kernels over shared vectors, each stage what one Execute.run_vectors call takes:
 * the launches a caller makes for the kernel list Sarek_fusion.auto_fuse_pipeline hands back
 * (sarek/sarek/Sarek_fusion.ml:1133-1165; that pass cannot fuse a kernel with barriers, :641-661, so
 * `stream triad, block-256 tree sum` stays two kernels there).  Stages run in order with the
 * results of separate launches: per stage the uploads, the lowering and the argument expansion of
 * Execute.run_vectors, then all launches through sarek_hip_run_sources (two consecutive stages that
 * one hand-written kernel computes in a single pass over the data — stream triad, then the block-256
 * sum of the vector it wrote — are launched as that kernel), then the vectors of the stages that
 * ran are marked stale.  *launches (may be NULL) gets the number of device launches made;
 * sarek_hip_last_run_path() then reads e.g. "stream_triad_f32+reduce_sum_block256_f32", paths of
 * separate launches joined by ';'.                                                              */
typedef struct sarek_hip_pipeline_stage {
  const char *ir_text;
  int block[3], grid[3];
  int shared_mem_bytes;
  const sarek_hip_varg *args;
  int n_args;
} sarek_hip_pipeline_stage;
int sarek_hip_execute_run_pipeline(const sarek_hip_pipeline_stage *stages, int n_stages, int *launches);

/* Execute.run_source (Execute.ml:613-651): an external kernel; inject_lengths = 0 passes
 * bare buffers (sarek/tests/e2e/test_external_kernel.ml:46-62).                      */
int sarek_hip_execute_run_source(const char *source, int lang, const char *kernel_name,
                                 const int block[3], const int grid[3], int shared_mem_bytes,
                                 int inject_lengths, const sarek_hip_varg *args, int n_args);
int sarek_hip_execute_sync_vectors_to_cpu(const sarek_hip_varg *args, int n_args);
/* Execute.supports_lang for this backend (sarek/sarek/Execute.ml:589-593): 1 for HIP and CUDA source
 * (CUDA text is compiled as HIP), 0 otherwise.                                                     */
int sarek_hip_supports_lang(int lang);
/* Execute.detect_lang (Execute.ml:658-675) by file extension: .cu, .cl, .ptx, .spv, .comp / .glsl
 * as there, and .hip for this backend's own language; anything else fails with the reference's
 * "Invalid file <path>: Unknown source file extension ..." text.                                  */
int sarek_hip_execute_detect_lang(const char *path, int *lang);
/* Execute.run_source_file (Execute.ml:711-726): the file's text through run_source in the language
 * its extension names.                                                                             */
int sarek_hip_execute_run_source_file(const char *path, const char *kernel_name, const int block[3],
                                      const int grid[3], int shared_mem_bytes, int inject_lengths,
                                      const sarek_hip_varg *args, int n_args);

/* ---------------------------------------------------------------------- */
/* Hand-written CDNA4 kernels.  All pointers are device pointers.  These have
 * no counterpart symbol in the reference: they replace the JIT-compiled
 * generated kernels named in each comment.                                 */

/* Stream triad  a[i] = b[i] + c[i]*s, i < n   (generated kernel
 * benchmarks/descriptions/generated/stream_triad_generated.md:9-17; source
 * benchmarks/bench_stream_triad.ml:22-32).                                 */
int sarek_hip_triad_f32(float *a, const float *b, const float *c, float s, int64_t n,
                        sarek_hip_stream stream);

/* Fused triad + sum: writes a as above and *sum_out = sum_i a[i] (double,
 * device memory).  Every workgroup leaves an f32 partial in `partials`
 * (caller workspace of at least sarek_hip_triad_sum_workspace_floats(n)
 * floats; contents on entry are irrelevant) and a one-workgroup kernel on
 * the same stream folds them in double, in index order: the result does
 * not depend on scheduling.                                                */
int64_t sarek_hip_triad_sum_workspace_floats(int64_t n);
int sarek_hip_triad_sum_f32(float *a, const float *b, const float *c, float s, int64_t n,
                            float *partials, int64_t partials_len, double *sum_out,
                            sarek_hip_stream stream);

/* The pair `stream triad, then block-256 sum of its output` in one pass over the data: writes a as
 * sarek_hip_triad_f32 does and block_sums[j] = sum of a[256j .. 256j+255] (zero padded),
 * j < ceil(n/256), with the bits sarek_hip_reduce_sum_block256_f32 would produce from that a
 * (benchmarks/bench_stream_triad.ml:22-32 followed by benchmarks/bench_reduction.ml:62-96; what
 * sarek_hip_execute_run_pipeline launches for that pair of kernels).  Vectors at any alignment (16-byte
 * aligned ones are the fast case: the others cost the pass about 7 %).                                */
int sarek_hip_triad_block256_sum_f32(float *a, const float *b, const float *c, float s, int64_t n,
                                     float *block_sums, sarek_hip_stream stream);
/* The same with the block-256 maximum in place of the sum: block_max[j] = what the reference's halving tree
 * leaves for a[256j .. 256j+255], elements past n counting as `pad` (benchmarks/bench_reduction_max.ml:18-100),
 * with the bits sarek_hip_reduce_max_block256_f32 would produce from that a.  With s = 1 the triad is the vector
 * add of benchmarks/bench_vector_add.ml, so the four pairs {triad, add} x {sum, max} of a pipeline are one pass. */
int sarek_hip_triad_block256_max_f32(float *a, const float *b, const float *c, float s, int64_t n, float pad,
                                     float *block_max, sarek_hip_stream stream);

/* The same operation for callers that cannot allocate device memory or carry a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc); it has no
 * counterpart in the reference.  The partials live in an array inside the library's own device
 * image (2 MiB per device, held until the process ends), so the call makes no hipMalloc / hipFree
 * and no allocating library call.  n may be at most sarek_hip_triad_sum_static_max_n() = 2^31
 * elements; a longer vector is refused with SAREK_HIP_E_WORKSPACE before anything is launched.
 * Results are bit for bit those of sarek_hip_triad_sum_f32.  All calls on one device share that
 * device's array: calls that overlap in time on one device (different streams, or different host
 * threads without ordering between their streams) race on it; calls on one stream do not.  The
 * first call on a device looks the array's address up (hipGetSymbolAddress); make that call
 * outside a stream capture (under one it is refused with SAREK_HIP_E_UNSUPPORTED).              */
int64_t sarek_hip_triad_sum_static_max_n(void);
int sarek_hip_triad_sum_f32_static(float *a, const float *b, const float *c, float s, int64_t n,
                                   double *sum_out, sarek_hip_stream stream);

/* Block-256 tree reductions: out[j] = sum of in[256j .. 256j+255] (zero
 * padded), j < ceil(n/256)  (benchmarks/bench_reduction.ml:62-96;
 * generated kernel reduction_generated.md:9-75).  dot: sum of a[i]*b[i]
 * (benchmarks/bench_dot_product.ml:16-54).                                 */
int sarek_hip_reduce_sum_block256_f32(const float *in, float *out, int64_t n,
                                      sarek_hip_stream stream);
int sarek_hip_dot_block256_f32(const float *a, const float *b, float *out, int64_t n,
                               sarek_hip_stream stream);
/* out[j] = what the reference's block-256 "take the greater" tree leaves for block j
 * (benchmarks/bench_reduction_max.ml:18-100), elements past n read as `pad`
 * (-1000000.0 in that file); same comparison pairs and order as the tree.   */
int sarek_hip_reduce_max_block256_f32(const float *in, float *out, int64_t n, float pad,
                                      sarek_hip_stream stream);
/* *sum_out = double fold of partials[0..count) in an order fixed by count and the pointer's
 * alignment (host fold of benchmarks/bench_reduction.ml:154-160, kept on device): one launch.  From
 * 2^17 partials on, 256 workgroups fold a piece each into a stage inside the library's device image
 * and the one that finishes last adds those up in index order.  Every (device, stream) gets a stage of
 * its own (16 per device), so long folds on different streams do not meet; a stream beyond the
 * sixteenth, and any fold recorded under stream capture (a graph may be replayed on any stream, next
 * to anything), fold with one workgroup that takes the 256 pieces in turn and needs no shared stage:
 * slower, and the same bits, since it adds what the 256 add in the same order.                       */
int sarek_hip_fold_partials_f64(const float *partials, int64_t count, double *sum_out,
                                sarek_hip_stream stream);

/* dst[i] = src[i], i < n: the kernel of benchmarks/bench_vector_copy.ml:21-27
 * (`if tid < n then b.(tid) <- a.(tid)`); elements past n are not touched.          */
int sarek_hip_copy_f32(float *dst, const float *src, int64_t n, sarek_hip_stream stream);
/* out[c * height + r] = in[r * width + c] for r < height, c < width: the kernels of
 * benchmarks/bench_transpose.ml and bench_transpose_tiled.ml (`in` has `height` rows
 * of `width` floats).  in and out must not overlap.                                 */
int sarek_hip_transpose_f32(const float *in, float *out, int width, int height, sarek_hip_stream stream);
/* output[y * width + x] = (up + down + left + right + center) / 5 for 0 < x < width - 1 and
 * 0 < y < height - 1, the operands widened to double, added in that order and rounded once at
 * the store; the border keeps what it holds: the kernel of benchmarks/bench_stencil_2d.ml:43-58
 * launched over the whole grid.  Any width and height (below 3 nothing is written), grids at
 * any alignment; input and output must not overlap; width * height < 2^31.            */
int sarek_hip_stencil_2d_f32(const float *input, float *output, int width, int height, sarek_hip_stream stream);
/* The 3 x 3 box filter of benchmarks/bench_conv2d.ml:49-77 launched over all width * height
 * cells: 0 on the border, elsewhere the nine cells round (x, y) added row by row, left to
 * right, in double, divided by 9 and rounded once.  Same conditions as the stencil.    */
int sarek_hip_conv2d_f32(const float *input, float *output, int width, int height, sarek_hip_stream stream);

/* histogram[b] += #{ i < n : keys[i] mod num_bins == b } for b < num_bins, 1 <= num_bins <= 256:
 * what a launch of the kernel of benchmarks/bench_histogram.ml:54-84 over n keys adds to the
 * global histogram (`mod` is the generated code's `%`: a negative key with a non-zero
 * remainder has no bin and is not counted, where that kernel indexes its shared array with
 * it).  The histogram is accumulated into, not cleared.                                 */
int sarek_hip_histogram_i32(int32_t *histogram, const int32_t *keys, int64_t n, int num_bins,
                            sarek_hip_stream stream);
/* histogram[d] += #{ i < n : (keys[i] >> shift) & mask == d }, 256 bins, 0 <= mask <= 255,
 * 0 <= shift <= 31: the counting kernel of one radix-sort pass,
 * benchmarks/bench_radix_sort.ml:82-116 (`>>` as in the generated code: arithmetic).   */
int sarek_hip_radix_histogram_i32(int32_t *histogram, const int32_t *keys, int64_t n, int shift, int mask,
                                  sarek_hip_stream stream);
/* The scatter kernel of the same pass, benchmarks/bench_radix_sort.ml:120-137: every key i < n takes
 * the next free position of its digit d = (keys[i] >> shift) & mask,
 *     pos = counters[d]++;  out[pos] = keys[i].
 * Afterwards counters[d] has grown by the number of keys with digit d and out holds them in
 * [old counters[d], new counters[d]), in an order that kernel can produce (it fixes none: its
 * positions come from global atomics).  A position outside [0, out_len) is skipped, where that
 * kernel writes out of bounds.  The three vectors must not overlap.                              */
int sarek_hip_radix_scatter_i32(int32_t *out, int64_t out_len, int32_t *counters, const int32_t *keys, int64_t n,
                                int shift, int mask, sarek_hip_stream stream);

/* Row-major GEMM  C[m x n] = A[m x k] . B[k x n]  (replaces the generated
 * 16x16 tiled kernel, matrix_mul_tiled_generated.md:9-50; source
 * benchmarks/bench_matrix_mul_tiled.ml:55-95).  Any m,n,k >= 1.            */
int sarek_hip_gemm_f32(const float *a, const float *b, float *c, int m, int n, int k,
                       sarek_hip_stream stream);
/* Into how many pieces sarek_hip_gemm_f32 cuts K for this shape now (1 = none):
 * as for the 16-bit products (sarek_hip_gemm16_k_splits below), same per-stream
 * memory and fixed-order sum; tunable gemm_f32.split_k.                      */
int sarek_hip_gemm_f32_k_splits(int m, int n, int k);

/* 16-bit-input, f32-accumulate GEMMs.  a, b hold bf16 / IEEE fp16 bit
 * patterns, row-major [m x k] and [k x n]; c is f32 row-major.  Any m, n,
 * k >= 1 and any alignment of the three (sarek_hip_gemm16_tile below says
 * which kernel serves a shape).                                             */
int sarek_hip_gemm_bf16(const uint16_t *a, const uint16_t *b, float *c, int m, int n, int k,
                        sarek_hip_stream stream);
int sarek_hip_gemm_f16(const uint16_t *a, const uint16_t *b, float *c, int m, int n, int k,
                       sarek_hip_stream stream);

/* Which kernel the three 16-bit GEMM entry points take for a shape under the
 * present tunables: 256 or 128 = the workgroup tile of the direct-to-LDS MFMA
 * kernels (the small tile where large ones would leave CUs idle; any n, any
 * k >= 64 and the multiples of 8 below, any alignment of a and b from k = 64
 * on), 0 = the one-thread-per-element kernel (k < 64 that is not a multiple
 * of 8; below 64 an a or b that is not 16-byte aligned has the same effect).
 * No counterpart in the reference, whose tiled
 * kernel has one shape (bench_matrix_mul_tiled.ml:55-95); needs no device.  */
int sarek_hip_gemm16_tile(int m, int n, int k);
/* Into how many pieces sarek_hip_gemm_bf16 / _f16 cut K for this shape now (1 =
 * none): products with few 128 x 128 tiles and a long K are spread over the
 * CUs that way, the partial tiles added up in a fixed order by a second
 * kernel.  Device memory for them: one 64 MiB block per stream, allocated at
 * the first such call on the stream and kept until the process ends, for up
 * to 16 streams; calls on further streams, and calls under stream capture on
 * a stream that has no block yet, run unsplit (same result up to the order of
 * the f32 additions).  The fused-epilogue entry point never splits.         */
int sarek_hip_gemm16_k_splits(int m, int n, int k);

/* Fused epilogue chain: y = relu(A.B + bias[col]) (f32, [m x n]) and
 * rowsum[r] = sum_c y[r,c] (f32, [m]).  fp16 inputs.                        */
int sarek_hip_gemm_f16_bias_relu_rowsum(const uint16_t *a, const uint16_t *b, const float *bias,
                                        float *y, float *rowsum, int m, int n, int k,
                                        sarek_hip_stream stream);

/* Round-to-nearest-even narrowing of an f32 vector to bf16 / fp16 bit
 * patterns (the input cast of the 16-bit GEMM path).                       */
int sarek_hip_cast_f32_to_bf16(const float *in, uint16_t *out, int64_t n, sarek_hip_stream stream);
int sarek_hip_cast_f32_to_f16(const float *in, uint16_t *out, int64_t n, sarek_hip_stream stream);

/* Persistent cache of compiled kernels: the reference's Framework_cache
 * (sarek/framework/Framework_cache.ml:63-141; used there by the Vulkan plugin,
 * sarek-vulkan/Vulkan_api.ml:1254-1283).  Directory: $XDG_CACHE_HOME, else
 * $HOME/.cache, else the temp dir, then "/spoc"; key = MD5 hex of
 * dev_name ^ driver_version ^ source; one file per key.  A miss or an I/O error
 * is never an error of the call: `found` says whether an entry was read, the
 * counters say why not.  sarek_hip_kernel_compile(_cached) stores hiprtc code
 * objects here and looks there before compiling; SAREK_HIP_DISK_CACHE=0 in the
 * environment switches that off.
 * stats: out[0] hits, out[1] misses, out[2] puts, out[3] I/O errors.        */
int sarek_hip_cache_dir(char *out, size_t out_len);
int sarek_hip_cache_compute_key(const char *dev_name, const char *driver_version,
                                const char *source, char out_hex[33]);
int sarek_hip_cache_get(const char *key, void *out, size_t out_len, size_t *size, int *found);
int sarek_hip_cache_put(const char *key, const void *data, size_t len);
int sarek_hip_cache_get_stats(int64_t out[4]);
int sarek_hip_cache_reset_stats(void);

/* ---------------------------------------------------------------------- */
/* IR fusion: sarek/sarek/Sarek_fusion.ml over IR text (same grammar as
 * sarek_hip_generate_source reads; results are written in it too), for hosts
 * that hold kernels as text and have no OCaml.  Results follow the reference
 * kernel for kernel, its limits included (see sarek_hip_fusion_fuse).  Text
 * outputs use the generate_source buffer convention (at most out_len bytes
 * incl. NUL, *needed = full size, SAREK_HIP_E_BUFFER_TOO_SMALL when short).  */
enum {                                   /* `mode` below                              */
  SAREK_HIP_FUSION_VERTICAL = 0,         /* can_fuse / fuse                 :401-547   */
  SAREK_HIP_FUSION_REDUCTION = 1,        /* can_fuse_reduction / fuse_reduction :641-757 */
  SAREK_HIP_FUSION_STENCIL = 2,          /* can_fuse_stencil / fuse_stencil :795-1019  */
  SAREK_HIP_FUSION_TRY = 3,              /* try_fuse                        :760-766   */
  SAREK_HIP_FUSION_TRY_ALL = 4           /* try_fuse_all                    :1022-1030 */
};
enum { SAREK_HIP_FUSION_FUSE = 0, SAREK_HIP_FUSION_DONT_FUSE = 1, SAREK_HIP_FUSION_MAYBE_FUSE = 2 };

/* analyze (:340-354).  out: (info (reads (ARRAY pattern)*) (writes (ARRAY pattern)*)
 * (barriers true|false) (atomics false)), arrays sorted by name,
 * pattern ::= (one_to_one expr) | (stencil OFFSET*) | (reduction OP) | gather | unknown */
int sarek_hip_fusion_analyze(const char *kernel_ir, char *out, size_t out_len, size_t *needed);
/* *result = 1 when the producer can be fused into the consumer through array
 * `intermediate` under `mode` (TRY modes: when the corresponding try_* returns Some). */
int sarek_hip_fusion_can_fuse(const char *producer_ir, const char *consumer_ir, const char *intermediate,
                              int mode, int *result);
/* The fused kernel as IR text: "<consumer>_fused" ("<consumer>_stencil_fused" for the
 * stencil rewrite), consumer parameters without the intermediate followed by the
 * producer's new ones, native_fn false.  As in the reference, the fixed modes return
 * the consumer unchanged when the producer's store cannot be inlined (conditional store,
 * no read of the intermediate); the TRY modes set *fused = 0 and write "" when no rewrite
 * applies.  The reduction rewrite inserts the producer's expression as it stands.      */
int sarek_hip_fusion_fuse(const char *producer_ir, const char *consumer_ir, const char *intermediate, int mode,
                          int *fused, char *out, size_t out_len, size_t *needed);
/* should_fuse (:1068-1098): decision + the reference's reason text.                 */
int sarek_hip_fusion_should_fuse(const char *producer_ir, const char *consumer_ir, const char *intermediate,
                                 int *decision, char *reason, size_t reason_len);
/* fuse_pipeline (automatic = 0, :570-598) / auto_fuse_pipeline (1, :1133-1165).
 * out: the resulting kernel; report: one line per entry, "eliminated ARRAY" then
 * "skipped REASON", each list in the reference's order (latest first).  An empty
 * list is SAREK_HIP_E_INVALID_ARG with Fusion_error's text.                         */
int sarek_hip_fusion_pipeline(const char *const *kernel_irs, int n_kernels, int automatic, char *out,
                              size_t out_len, size_t *needed, char *report, size_t report_len,
                              size_t *report_needed);
/* analyze_pipeline (:1180-1214): the text it prints.                                */
int sarek_hip_fusion_analyze_pipeline(const char *const *kernel_irs, int n_kernels, char *out, size_t out_len,
                                      size_t *needed);
/* analyze_stencil_fusion (:829-871): radii = {combined, producer, consumer};
 * inputs = the producer's input arrays, space separated.                            */
int sarek_hip_fusion_stencil_info(const char *producer_ir, const char *consumer_ir, const char *intermediate,
                                  int *found, int radii[3], char *inputs, size_t inputs_len, size_t *needed);
/* The expression-level pieces (:35-48, :77-124, :611-634).
 * detect_reduction out: (reduction ACC ACC_ID OP ARRAY LOOPVAR LOOPVAR_ID).          */
int sarek_hip_fusion_expr_equal(const char *expr_a, const char *expr_b, int *equal);
int sarek_hip_fusion_subst_array_read(const char *array, const char *index_expr, const char *replacement_expr,
                                      const char *expr, char *out, size_t out_len, size_t *needed);
int sarek_hip_fusion_detect_reduction(const char *stmt_ir, int *found, char *out, size_t out_len, size_t *needed);
int sarek_hip_fusion_is_reduction_kernel(const char *kernel_ir, const char *array, int *found, char op[8]);

/* Integer tuning knob (launch shapes, tile variants), for sweeps without a
 * rebuild.  Unknown names are stored and ignored.  Every knob of the product
 * library leaves results as they are; the knobs of the measurement build
 * (gemm16.ablate, gemm16.ring, gemm16.tj, gemm16.mfma, gemm16.waves,
 * gemm16.barriers) are refused by the product library with
 * SAREK_HIP_E_UNSUPPORTED.                                                   */
int sarek_hip_set_tunable(const char *name, int64_t value);

/* 1 in libsarek_hip_measure.so (built with -DSAREK_HIP_MEASURE by `make measure`: the
 * product's code plus retired kernel shapes, variants of the 16-bit GEMMs that leave parts of
 * the K loop out -- their results are wrong on purpose -- and the in-kernel clock probe; what
 * the ablation studies are made with), 0 in libsarek_hip.so.                                 */
int sarek_hip_is_measurement_build(void);

/* Diagnostic of the measurement build (no reference counterpart; the product library
 * answers SAREK_HIP_E_UNSUPPORTED): while a probe buffer is set, every
 * workgroup of the MFMA GEMM kernels (sarek_hip_gemm_bf16/_f16/_f16_bias_relu_rowsum,
 * direct-to-LDS path) writes two 64-bit counts when it retires:
 * pairs[2*w] = shader-clock cycles it was resident, pairs[2*w+1] = ticks of the
 * constant-rate wall clock over the same interval (rate in *ticks_per_second).
 * cycles/ticks gives the shader clock the kernel actually ran at.  A launch
 * with more workgroups than capacity_pairs records nothing.  Pass NULL to
 * switch the probe off (the default).                                        */
int sarek_hip_set_clock_probe(uint64_t *device_pairs, int64_t capacity_pairs,
                              int64_t *ticks_per_second);

#ifdef __cplusplus
}
#endif
#endif /* SAREK_HIP_H */
