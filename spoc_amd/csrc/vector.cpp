// Host side of a launch above the plugin boundary: vectors with a host block, per-device
// buffers and a location state (sarek/core/Vector.ml, Vector_types.ml:198-203), the
// transfers that move them (sarek/core/Transfer.ml:173-388) and the dispatcher that turns
// a kernel's IR plus a list of vectors and scalars into a run_source call
// (sarek/sarek/Execute.ml:188-216, 231-304, 321-335, 520-543, 613-651).  In the reference
// these are backend-agnostic OCaml; a host without OCaml gets them here, state machine
// and corner cases included:
//   - to_device copies only from CPU / Stale_GPU (or another device) and leaves Both;
//   - a launch marks only Both vectors Stale_CPU;
//   - a host write marks Both / GPU vectors Stale_GPU and does NOT first fetch a stale
//     host copy (a write into a Stale_CPU vector is overwritten by the next download);
//   - a host read downloads a Stale_CPU vector when auto-sync is on (vector and global).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "common.hpp"
#include "gpu_memory.hpp"
#include "host/ir.hpp"
#include "plugin.hpp"

// The allocation behind a vector's host block; sub-vectors view their parent's, and it lives as
// long as any of them (a Bigarray.Array1.sub keeps its parent's memory alive the same way).
struct sarek_hip_host_block {
  void *base = nullptr;
  bool pinned = false;
  ~sarek_hip_host_block() {
    if (!base) return;
    if (pinned) sarek_hip_host_free(base);
    else std::free(base);
  }
};

struct sarek_hip_vector_s {
  int kind = SAREK_HIP_KIND_FLOAT32;
  int64_t length = 0, elem_size = 4;
  int64_t id = 0;                        // Vector_types.t.id (Vector_storage.next_id)
  std::shared_ptr<sarek_hip_host_block> block;
  void *host = nullptr;                  // first element: block->base, or inside it for a sub-vector
  // Vector_storage.sub_meta (Vector_storage.ml:147-175)
  bool is_sub = false;
  int64_t parent_id = 0, sub_start = 0, ok_range = 0, ko_range = 0;
  int depth = 0;
  bool pinned = false;
  bool zero_copy = false;                // device buffers alias the pinned host block
  bool auto_sync = true;                 // Vector_types.t.auto_sync
  int location = SAREK_HIP_LOC_CPU;
  int device = -1;                       // the device of a non-CPU location
  std::map<int, void *> buffers;         // device id -> device block (vec.device_buffers)
};

namespace sarek_hip {
namespace {

bool g_auto_mode = true;                 // Transfer.auto_mode (Transfer.ml:20-28)
std::atomic<int64_t> g_next_id{0};       // Vector_storage.next_id: the first vector is #1

int64_t kind_elem_size(int kind, int64_t custom) {
  switch (kind) {                        // Vector_types.scalar_elem_size
    case SAREK_HIP_KIND_FLOAT32: case SAREK_HIP_KIND_INT32: return 4;
    case SAREK_HIP_KIND_FLOAT64: case SAREK_HIP_KIND_INT64: case SAREK_HIP_KIND_COMPLEX32: return 8;
    case SAREK_HIP_KIND_CHAR: return 1;
    case SAREK_HIP_KIND_CUSTOM: return custom;
    default: return 0;
  }
}

size_t bytes_of(const sarek_hip_vector_s *v) { return static_cast<size_t>(v->length * v->elem_size); }

int current_device(int *dev) {
  SAREK_HIP_TRY(hipGetDevice(dev));
  return SAREK_HIP_OK;
}

// Transfer.ensure_buffer: the vector's block on `dev`, allocated on first use.
int ensure_buffer(sarek_hip_vector_s *v, int dev, void **out) {
  auto it = v->buffers.find(dev);
  if (it != v->buffers.end()) {
    *out = it->second;
    return SAREK_HIP_OK;
  }
  // Gpu_memory.with_retry round the allocation, track_alloc after it (Transfer.ml:184-218)
  struct Attempt {
    sarek_hip_vector_s *v;
    void *p;
  } attempt{v, nullptr};
  int st = sarek_hip_gpu_memory_with_retry(
      [](void *ctx) -> int {
        auto *a = static_cast<Attempt *>(ctx);
        if (a->v->zero_copy) {
          // Memory.alloc_zero_copy returning Some (Transfer.ml:85-126): the buffer is the host block
          // as the device sees it; its transfers are no-ops.
          int supported = 0;
          int st = sarek_hip_mem_alloc_zero_copy(a->v->host, bytes_of(a->v), &a->p, &supported);
          if (st != SAREK_HIP_OK) return st;
          if (!supported)
            return fail(SAREK_HIP_E_UNSUPPORTED, "zero-copy vector: the host block is not device-accessible");
          return SAREK_HIP_OK;
        }
        return sarek_hip_mem_alloc(&a->p, bytes_of(a->v));
      },
      &attempt);
  if (st != SAREK_HIP_OK) return st;
  v->buffers[dev] = attempt.p;
  sarek_hip_gpu_memory_track_alloc(static_cast<int64_t>(bytes_of(v)));
  *out = attempt.p;
  return SAREK_HIP_OK;
}

bool on_device(const sarek_hip_vector_s *v, int loc, int dev) { return v->location == loc && v->device == dev; }

// Transfer.to_device (Transfer.ml:228-268)
int to_device(sarek_hip_vector_s *v, int dev) {
  if (on_device(v, SAREK_HIP_LOC_GPU, dev) || on_device(v, SAREK_HIP_LOC_BOTH, dev) ||
      on_device(v, SAREK_HIP_LOC_STALE_CPU, dev))
    return SAREK_HIP_OK;
  void *buf = nullptr;
  int st = ensure_buffer(v, dev, &buf);
  if (st != SAREK_HIP_OK) return st;
  if (!v->zero_copy) {
    st = sarek_hip_memcpy_htod(buf, v->host, bytes_of(v));
    if (st != SAREK_HIP_OK) return st;
  }
  v->location = SAREK_HIP_LOC_BOTH;
  v->device = dev;
  return SAREK_HIP_OK;
}

// Transfer.to_cpu ?force (Transfer.ml:274-333)
int to_cpu(sarek_hip_vector_s *v, bool force) {
  bool needed = false;
  switch (v->location) {
    case SAREK_HIP_LOC_BOTH: needed = force; break;
    case SAREK_HIP_LOC_GPU: case SAREK_HIP_LOC_STALE_CPU: needed = true; break;
    default: break;                      // CPU: no device copy; Stale_GPU: the host copy is the good one
  }
  if (!needed) return SAREK_HIP_OK;
  auto it = v->buffers.find(v->device);
  if (it == v->buffers.end()) return fail(SAREK_HIP_E_INVALID_ARG, "to_cpu: no device buffer to transfer from");
  // A copy waits for the launches before it; a zero-copy vector has nothing to copy, but the
  // kernel that wrote the host block must have finished before the host reads it.
  int st = v->zero_copy ? sarek_hip_device_synchronize() : sarek_hip_memcpy_dtoh(v->host, it->second, bytes_of(v));
  if (st != SAREK_HIP_OK) return st;
  v->location = SAREK_HIP_LOC_BOTH;
  return SAREK_HIP_OK;
}

// Vector_transfer.ensure_cpu_sync + the callback Transfer registers (Transfer.ml:454-464)
int ensure_cpu_sync(sarek_hip_vector_s *v) {
  if (v->auto_sync && v->location == SAREK_HIP_LOC_STALE_CPU && g_auto_mode) return to_cpu(v, false);
  return SAREK_HIP_OK;
}

// Vector.set's bookkeeping (Vector.ml:104-109)
void host_written(sarek_hip_vector_s *v) {
  if (v->location == SAREK_HIP_LOC_BOTH || v->location == SAREK_HIP_LOC_GPU) v->location = SAREK_HIP_LOC_STALE_GPU;
}

// Bulk copies between a caller's array and a host block.  One core moves about 30 GB/s; from
// 16 MiB on the copy is cut into four pieces, three of them on threads of their own (a thread
// costs some tens of microseconds, a 16 MiB copy half a millisecond).
void host_copy(void *dst, const void *src, size_t bytes) {
  constexpr size_t kParallelFrom = size_t{16} << 20;
  constexpr int kPieces = 4;
  if (bytes < kParallelFrom) {
    std::memcpy(dst, src, bytes);
    return;
  }
  const size_t piece = (bytes / kPieces + 4095) & ~size_t{4095};
  std::thread helpers[kPieces - 1];
  int started = 0;
  for (int i = 1; i < kPieces; ++i) {
    const size_t from = piece * i;
    if (from >= bytes) break;
    const size_t len = std::min(piece, bytes - from);
    try {
      helpers[started] = std::thread([=] { std::memcpy(static_cast<char *>(dst) + from, static_cast<const char *>(src) + from, len); });
      ++started;
    } catch (...) {                      // no thread to be had: this one does the piece itself
      std::memcpy(static_cast<char *>(dst) + from, static_cast<const char *>(src) + from, len);
    }
  }
  std::memcpy(dst, src, std::min(piece, bytes));
  for (int i = 0; i < started; ++i) helpers[i].join();
}

// Range check of a bulk access, reported like the element accessors report theirs
// (Vector.ml:80-103).
int bounds(const sarek_hip_vector_s *v, int64_t first, int64_t count, const char *what) {
  if (first >= 0 && count >= 0 && first + count <= v->length) return SAREK_HIP_OK;
  const int64_t bad = first < 0 ? first : (count < 0 ? count : v->length);
  return fail(SAREK_HIP_E_INVALID_ARG, "Vector.%s: index %lld out of bounds [0, %lld)", what,
              static_cast<long long>(bad), static_cast<long long>(v->length));
}

// Execute.transfer_vectors_to_device
int transfer_args(const sarek_hip_varg *args, int n, int dev) {
  for (int i = 0; i < n; ++i)
    if (args[i].kind == SAREK_HIP_VARG_VEC) {
      if (!args[i].vec) return fail(SAREK_HIP_E_INVALID_ARG, "argument %d: NULL vector", i);
      int st = to_device(args[i].vec, dev);
      if (st != SAREK_HIP_OK) return st;
    }
  return SAREK_HIP_OK;
}

// Execute.expand_to_run_source_args
int expand_args(const sarek_hip_varg *args, int n, int dev, bool inject_lengths, std::vector<sarek_hip_arg> &out) {
  for (int i = 0; i < n; ++i) {
    sarek_hip_arg a;
    std::memset(&a, 0, sizeof(a));
    switch (args[i].kind) {
      case SAREK_HIP_VARG_VEC: {
        sarek_hip_vector_s *v = args[i].vec;
        auto it = v->buffers.find(dev);
        if (it == v->buffers.end()) return fail(SAREK_HIP_E_INVALID_ARG, "Vector has no device buffer");
        a.kind = SAREK_HIP_ARG_BUFFER;
        a.buffer = it->second;
        a.length = v->length;
        out.push_back(a);
        // the length parameter of a kernel is an int32 (sarek-cuda/Sarek_ir_cuda.ml:668-672); a longer
        // vector would wrap round where the reference passes Int32.of_int of it
        if (inject_lengths && v->length > 0x7FFFFFFF)
          return fail(SAREK_HIP_E_INVALID_ARG,
                      "argument %d: vector of %lld elements, a kernel's length parameter holds at most 2147483647",
                      i, static_cast<long long>(v->length));
        if (inject_lengths) {
          sarek_hip_arg l;
          std::memset(&l, 0, sizeof(l));
          l.kind = SAREK_HIP_ARG_INT32;
          l.i32 = static_cast<int32_t>(v->length);
          out.push_back(l);
        }
        continue;
      }
      case SAREK_HIP_VARG_INT32: a.kind = SAREK_HIP_ARG_INT32; a.i32 = args[i].i32; break;
      case SAREK_HIP_VARG_INT64: a.kind = SAREK_HIP_ARG_INT64; a.i64 = args[i].i64; break;
      case SAREK_HIP_VARG_FLOAT32: a.kind = SAREK_HIP_ARG_FLOAT32; a.f32 = args[i].f32; break;
      case SAREK_HIP_VARG_FLOAT64: a.kind = SAREK_HIP_ARG_FLOAT64; a.f64 = args[i].f64; break;
      default: return fail(SAREK_HIP_E_INVALID_ARG, "argument %d: unknown kind %d", i, args[i].kind);
    }
    out.push_back(a);
  }
  return SAREK_HIP_OK;
}

// Execute.mark_vectors_stale: only a vector that was in step with the device goes stale.
void mark_stale(const sarek_hip_varg *args, int n, int dev) {
  for (int i = 0; i < n; ++i)
    if (args[i].kind == SAREK_HIP_VARG_VEC && args[i].vec->location == SAREK_HIP_LOC_BOTH) {
      args[i].vec->location = SAREK_HIP_LOC_STALE_CPU;
      args[i].vec->device = dev;
    }
}

// IR text -> (kernel name, source).  The reference regenerates and re-hashes the source at
// every launch (Execute.ml:256); here one lowering per distinct IR text is kept.
struct Lowered {
  std::string name, source;
  // What each parameter takes: 'v' a vector (element size in bytes, 0 when the IR does not fix it: records), 'i' / 'l'
  // / 'f' / 'd' an int32 / int64 / float32 / float64 scalar, '?' anything (a record passed by value).
  struct Param {
    std::string name;
    char kind;
    int elem_size;
  };
  std::vector<Param> params;
};

int scalar_size(const ir::Type &t) {
  switch (t.kind) {
    case ir::Type::Int32: case ir::Type::Float32: case ir::Type::Bool: return 4;
    case ir::Type::Int64: case ir::Type::Float64: return 8;
    default: return 0;
  }
}

// A launch with the wrong number or kinds of arguments would hand the kernel a parameter block of another layout:
// lengths read as pointers, a float's bits as an element count.  The reference passes on what it is given
// (Execute.ml:197-216); here the mismatch is an error before anything is launched.
int check_args(const Lowered &k, const sarek_hip_varg *args, int n, const char *what) {
  if (static_cast<size_t>(n) != k.params.size())
    return fail(SAREK_HIP_E_INVALID_ARG, "%s: kernel %s takes %zu arguments, %d given", what, k.name.c_str(),
                k.params.size(), n);
  static const char *given[] = {"a vector", "an int32", "an int64", "a float32", "a float64"};
  for (int i = 0; i < n; ++i) {
    const Lowered::Param &p = k.params[static_cast<size_t>(i)];
    const int kind = args[i].kind;
    const char *is = kind >= 0 && kind <= 4 ? given[kind] : "of an unknown kind";
    const char *wants = nullptr;
    switch (p.kind) {
      case 'v':
        if (kind != SAREK_HIP_VARG_VEC) wants = "a vector";
        else if (args[i].vec && p.elem_size > 0 && static_cast<int64_t>(p.elem_size) != args[i].vec->elem_size)
          return fail(SAREK_HIP_E_INVALID_ARG,
                      "%s: argument %d (%s) of kernel %s is a vector of %d-byte elements, the vector given has %lld-byte elements",
                      what, i, p.name.c_str(), k.name.c_str(), p.elem_size, static_cast<long long>(args[i].vec->elem_size));
        break;
      case 'i': if (kind != SAREK_HIP_VARG_INT32) wants = "an int32"; break;
      case 'l': if (kind != SAREK_HIP_VARG_INT64) wants = "an int64"; break;
      case 'f': if (kind != SAREK_HIP_VARG_FLOAT32) wants = "a float32"; break;
      case 'd': if (kind != SAREK_HIP_VARG_FLOAT64) wants = "a float64"; break;
      default: break;
    }
    if (wants)
      return fail(SAREK_HIP_E_INVALID_ARG, "%s: argument %d (%s) of kernel %s is %s, %s given", what, i, p.name.c_str(),
                  k.name.c_str(), wants, is);
  }
  return SAREK_HIP_OK;
}
std::mutex g_lowered_mu;
std::unordered_map<std::string, std::shared_ptr<const Lowered>> g_lowered;

// The lowering of (ir_text, block), made once: a launch loop calls this every time, so a hit
// hands out the kept text without copying it.
int lower(const char *ir_text, const int block[3], std::shared_ptr<const Lowered> &out) {
  // the text can depend on the block (sizes of shared arrays): it is part of the key
  thread_local std::string key;
  char head[48];
  const int head_len = std::snprintf(head, sizeof(head), "%d,%d,%d;", block[0], block[1], block[2]);
  key.assign(head, static_cast<size_t>(head_len));
  key.append(ir_text);
  {
    std::lock_guard<std::mutex> lock(g_lowered_mu);
    auto it = g_lowered.find(key);
    if (it != g_lowered.end()) {
      out = it->second;
      return SAREK_HIP_OK;
    }
  }
  size_t needed = 0;
  int st = sarek_hip_generate_source(ir_text, block, nullptr, 0, &needed);
  if (st != SAREK_HIP_E_BUFFER_TOO_SMALL) {
    // generate_source returning None: Execute.run raises Compilation_failed (Execute.ml:257-263)
    const std::string why = sarek_hip_last_error();
    return fail(st == SAREK_HIP_OK ? SAREK_HIP_E_CODEGEN : st, "Backend failed to generate source: %s", why.c_str());
  }
  std::string src(needed, '\0');
  st = sarek_hip_generate_source(ir_text, block, src.data(), src.size(), &needed);
  if (st != SAREK_HIP_OK) return st;
  src.resize(std::strlen(src.c_str()));
  auto made = std::make_shared<Lowered>();
  made->source = src;
  const ir::Kernel parsed = ir::parse_kernel(ir_text);
  made->name = parsed.name;
  for (const ir::Decl &d : parsed.params) {
    Lowered::Param p{d.var.name, '?', 0};
    if (d.var.type) {
      const ir::Type &t = *d.var.type;
      switch (t.kind) {
        case ir::Type::Vec: case ir::Type::Array:
          p.kind = 'v';
          p.elem_size = t.elt ? scalar_size(*t.elt) : 0;
          break;
        case ir::Type::Int32: case ir::Type::Bool: p.kind = 'i'; break;
        case ir::Type::Int64: p.kind = 'l'; break;
        case ir::Type::Float32: p.kind = 'f'; break;
        case ir::Type::Float64: p.kind = 'd'; break;
        default: break;
      }
    }
    made->params.push_back(p);
  }
  out = made;
  std::lock_guard<std::mutex> lock(g_lowered_mu);
  if (g_lowered.size() > 256) g_lowered.clear();
  g_lowered[key] = out;
  return SAREK_HIP_OK;
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_vector_create(int kind, int64_t length, int64_t custom_elem_size, int pinned, sarek_hip_vector *out) {
  if (!out) return fail(SAREK_HIP_E_INVALID_ARG, "vector_create: NULL out pointer");
  *out = nullptr;
  const int64_t es = kind_elem_size(kind, custom_elem_size);
  if (es <= 0) return fail(SAREK_HIP_E_INVALID_ARG, "vector_create: unknown kind %d or element size %lld", kind,
                           static_cast<long long>(custom_elem_size));
  if (length < 0) return fail(SAREK_HIP_E_INVALID_ARG, "vector_create: negative length");
  auto *v = new sarek_hip_vector_s;
  v->kind = kind;
  v->length = length;
  v->elem_size = es;
  v->pinned = pinned != 0;
  v->zero_copy = pinned == 2;
  const size_t bytes = static_cast<size_t>(length * es);
  v->block = std::make_shared<sarek_hip_host_block>();
  v->block->pinned = v->pinned;
  if (v->pinned) {
    int st = sarek_hip_host_alloc(&v->block->base, bytes);
    if (st != SAREK_HIP_OK) {
      delete v;
      return st;
    }
  } else {
    v->block->base = std::malloc(bytes ? bytes : 1);   // like a fresh Bigarray: contents unspecified
    if (!v->block->base) {
      delete v;
      return fail(SAREK_HIP_E_INVALID_ARG, "vector_create: out of host memory (%zu bytes)", bytes);
    }
  }
  v->host = v->block->base;
  v->id = ++g_next_id;
  *out = v;
  return SAREK_HIP_OK;
}

int sarek_hip_vector_destroy(sarek_hip_vector v) {
  if (!v) return SAREK_HIP_OK;
  int first = SAREK_HIP_OK;
  for (auto &b : v->buffers) {      // what the reference's finaliser does (Gpu_memory.ml:163-178)
    int st = sarek_hip_mem_free(b.second);
    if (st == SAREK_HIP_OK) sarek_hip::track_gc_free(static_cast<int64_t>(v->length * v->elem_size));
    if (first == SAREK_HIP_OK) first = st;
  }
  delete v;        // the host block goes with its last vector
  return first;
}

int64_t sarek_hip_vector_id(sarek_hip_vector v) { return v ? v->id : -1; }

// Vector.to_string (Vector.ml:189-195): "Vector#<id><<kind>>[<length>] @ <location>"
int sarek_hip_vector_to_string(sarek_hip_vector v, char *buf, size_t cap) {
  if (!v || !buf || cap == 0) return fail(SAREK_HIP_E_INVALID_ARG, "vector_to_string: NULL argument");
  static const char *kinds[] = {"Float32", "Float64", "Int32", "Int64", "Char", "Complex32"};
  static const char *locs[] = {"CPU", "GPU", "Both", "Stale_CPU", "Stale_GPU"};
  std::string kind = v->kind == SAREK_HIP_KIND_CUSTOM ? "Custom(" + std::to_string(v->elem_size) + ")"
                                                      : std::string(kinds[v->kind]);
  std::string where = locs[v->location];
  if (v->location != SAREK_HIP_LOC_CPU) {
    sarek_hip_device_info info;
    where += sarek_hip_device_get_info(v->device, &info) == SAREK_HIP_OK ? "(" + std::string(info.name) + ")" : "(?)";
  }
  std::snprintf(buf, cap, "Vector#%lld<%s>[%lld] @ %s", static_cast<long long>(v->id), kind.c_str(),
                static_cast<long long>(v->length), where.c_str());
  return SAREK_HIP_OK;
}

// Vector.fill (Vector.ml:222-233): every element of the host block, then the bookkeeping of a host write.
int sarek_hip_vector_fill(sarek_hip_vector v, const void *elem) {
  if (!v || !elem) return fail(SAREK_HIP_E_INVALID_ARG, "vector_fill: NULL argument");
  char *p = static_cast<char *>(v->host);
  for (int64_t i = 0; i < v->length; ++i) std::memcpy(p + i * v->elem_size, elem, static_cast<size_t>(v->elem_size));
  host_written(v);
  return SAREK_HIP_OK;
}

// Vector.copy (Vector.ml:245-249, Vector_storage.copy_host_only): the host data, after a download if
// the host copy is stale and auto-sync is on; the copy starts on the CPU with no device buffers.
int sarek_hip_vector_copy(sarek_hip_vector v, sarek_hip_vector *out) {
  if (!v || !out) return fail(SAREK_HIP_E_INVALID_ARG, "vector_copy: NULL argument");
  int st = ensure_cpu_sync(v);
  if (st != SAREK_HIP_OK) return st;
  st = sarek_hip_vector_create(v->kind, v->length, v->elem_size, 0, out);
  if (st != SAREK_HIP_OK) return st;
  std::memcpy((*out)->host, v->host, bytes_of(v));
  (*out)->auto_sync = v->auto_sync;
  return SAREK_HIP_OK;
}

// Vector.sub_vector (Vector.ml:259-267, Vector_storage.ml:215-259): a view of `len` elements of the
// parent's host block from `start`, with device buffers and a location of its own (CPU).
// ok_range < 0 stands for the default (len).
int sarek_hip_vector_sub(sarek_hip_vector v, int64_t start, int64_t len, int64_t ok_range, int64_t ko_range,
                         sarek_hip_vector *out) {
  if (!v || !out) return fail(SAREK_HIP_E_INVALID_ARG, "sub_vector: NULL argument");
  *out = nullptr;
  if (start < 0 || len < 0 || start + len > v->length)
    return fail(SAREK_HIP_E_INVALID_ARG, "sub_vector: range [%lld, %lld) out of bounds [0, %lld)",
                static_cast<long long>(start), static_cast<long long>(start + len),
                static_cast<long long>(v->length));
  auto *s = new sarek_hip_vector_s;
  s->kind = v->kind;
  s->length = len;
  s->elem_size = v->elem_size;
  s->id = ++g_next_id;
  s->block = v->block;
  s->host = static_cast<char *>(v->host) + start * v->elem_size;
  s->pinned = v->pinned;
  s->zero_copy = v->zero_copy;
  s->auto_sync = v->auto_sync;
  s->is_sub = true;
  s->parent_id = v->id;
  s->sub_start = start;
  s->ok_range = ok_range < 0 ? len : ok_range;
  s->ko_range = ko_range;
  s->depth = v->depth + 1;
  *out = s;
  return SAREK_HIP_OK;
}

int sarek_hip_vector_sub_meta(sarek_hip_vector v, int *is_sub, int64_t *parent_id, int64_t *start,
                              int64_t *ok_range, int64_t *ko_range, int *depth) {
  if (!v || !is_sub) return fail(SAREK_HIP_E_INVALID_ARG, "vector_sub_meta: NULL argument");
  *is_sub = v->is_sub;
  if (parent_id) *parent_id = v->parent_id;
  if (start) *start = v->sub_start;
  if (ok_range) *ok_range = v->ok_range;
  if (ko_range) *ko_range = v->ko_range;
  if (depth) *depth = v->depth;
  return SAREK_HIP_OK;
}

// Vector.partition (Vector.ml:273-281, Vector_storage.partition_host): n sub-vectors that cover the
// vector, the first length mod n one element longer, sub-vector i marked Stale_GPU of devices[i]
// (host data valid, that device's copy to be made).
int sarek_hip_vector_partition(sarek_hip_vector v, int n_devices, const int *devices, sarek_hip_vector *out) {
  if (!v || n_devices < 0 || (n_devices > 0 && (!devices || !out)))
    return fail(SAREK_HIP_E_INVALID_ARG, "vector_partition: bad arguments");
  const int64_t base = n_devices ? v->length / n_devices : 0, rem = n_devices ? v->length % n_devices : 0;
  for (int i = 0; i < n_devices; ++i) out[i] = nullptr;
  for (int i = 0; i < n_devices; ++i) {
    const int64_t len = base + (i < rem ? 1 : 0), start = i * base + (i < rem ? i : rem);
    int st = sarek_hip_vector_sub(v, start, len, len, 0, &out[i]);
    if (st != SAREK_HIP_OK) {
      for (int j = 0; j < i; ++j) {
        sarek_hip_vector_destroy(out[j]);
        out[j] = nullptr;
      }
      return st;
    }
    out[i]->location = SAREK_HIP_LOC_STALE_GPU;
    out[i]->device = devices[i];
  }
  return SAREK_HIP_OK;
}

// Vector.blit (Vector.ml:500-517): source downloaded first if stale (auto-sync), destination written
// element by element with the bookkeeping of a host write.
int sarek_hip_vector_blit(sarek_hip_vector src, int64_t src_off, sarek_hip_vector dst, int64_t dst_off, int64_t len) {
  if (!src || !dst) return fail(SAREK_HIP_E_INVALID_ARG, "vector_blit: NULL argument");
  if (src->elem_size != dst->elem_size || src->kind != dst->kind)
    return fail(SAREK_HIP_E_INVALID_ARG, "Vector.blit: vectors of different kinds");
  if (len < 0 || src_off < 0 || src_off + len > src->length)
    return fail(SAREK_HIP_E_INVALID_ARG, "Vector.blit: source range out of bounds");
  if (dst_off < 0 || dst_off + len > dst->length)
    return fail(SAREK_HIP_E_INVALID_ARG, "Vector.blit: destination range out of bounds");
  int st = ensure_cpu_sync(src);
  if (st != SAREK_HIP_OK) return st;
  // ascending element order, as the reference's loop: overlapping ranges of one block smear forward
  const char *s = static_cast<const char *>(src->host) + src_off * src->elem_size;
  char *d = static_cast<char *>(dst->host) + dst_off * dst->elem_size;
  for (int64_t i = 0; i < len; ++i)
    std::memmove(d + i * dst->elem_size, s + i * src->elem_size, static_cast<size_t>(src->elem_size));
  if (len > 0) host_written(dst);
  return SAREK_HIP_OK;
}

int64_t sarek_hip_vector_length(sarek_hip_vector v) { return v ? v->length : -1; }
int64_t sarek_hip_vector_elem_size(sarek_hip_vector v) { return v ? v->elem_size : -1; }
int sarek_hip_vector_kind(sarek_hip_vector v) { return v ? v->kind : -1; }
void *sarek_hip_vector_host_ptr(sarek_hip_vector v) { return v ? v->host : nullptr; }

int sarek_hip_vector_location(sarek_hip_vector v, int *location, int *device) {
  if (!v || !location) return fail(SAREK_HIP_E_INVALID_ARG, "vector_location: NULL argument");
  *location = v->location;
  if (device) *device = v->location == SAREK_HIP_LOC_CPU ? -1 : v->device;
  return SAREK_HIP_OK;
}

int sarek_hip_vector_device_ptr(sarek_hip_vector v, void **dptr) {
  if (!v || !dptr) return fail(SAREK_HIP_E_INVALID_ARG, "vector_device_ptr: NULL argument");
  int dev = 0;
  int st = current_device(&dev);
  if (st != SAREK_HIP_OK) return st;
  auto it = v->buffers.find(dev);
  *dptr = it == v->buffers.end() ? nullptr : it->second;
  return SAREK_HIP_OK;
}

int sarek_hip_vector_auto_sync(sarek_hip_vector v) { return v && v->auto_sync ? 1 : 0; }

int sarek_hip_vector_set_auto_sync(sarek_hip_vector v, int enabled) {
  if (!v) return fail(SAREK_HIP_E_INVALID_ARG, "vector_set_auto_sync: NULL vector");
  v->auto_sync = enabled != 0;
  return SAREK_HIP_OK;
}

int sarek_hip_vector_get(sarek_hip_vector v, int64_t index, void *out_elem) {
  if (!v || !out_elem) return fail(SAREK_HIP_E_INVALID_ARG, "vector_get: NULL argument");
  if (index < 0 || index >= v->length)
    return fail(SAREK_HIP_E_INVALID_ARG, "Vector.get: index %lld out of bounds [0, %lld)",
                static_cast<long long>(index), static_cast<long long>(v->length));
  int st = ensure_cpu_sync(v);
  if (st != SAREK_HIP_OK) return st;
  std::memcpy(out_elem, static_cast<const char *>(v->host) + index * v->elem_size, v->elem_size);
  return SAREK_HIP_OK;
}

int sarek_hip_vector_set(sarek_hip_vector v, int64_t index, const void *elem) {
  if (!v || !elem) return fail(SAREK_HIP_E_INVALID_ARG, "vector_set: NULL argument");
  if (index < 0 || index >= v->length)
    return fail(SAREK_HIP_E_INVALID_ARG, "Vector.set: index %lld out of bounds [0, %lld)",
                static_cast<long long>(index), static_cast<long long>(v->length));
  std::memcpy(static_cast<char *>(v->host) + index * v->elem_size, elem, v->elem_size);
  host_written(v);
  return SAREK_HIP_OK;
}

int sarek_hip_vector_read(sarek_hip_vector v, void *dst, int64_t first, int64_t count) {
  if (!v || (!dst && count > 0)) return fail(SAREK_HIP_E_INVALID_ARG, "vector_read: NULL argument");
  int st = bounds(v, first, count, "get");
  if (st != SAREK_HIP_OK) return st;
  st = ensure_cpu_sync(v);
  if (st != SAREK_HIP_OK) return st;
  host_copy(dst, static_cast<const char *>(v->host) + first * v->elem_size, static_cast<size_t>(count * v->elem_size));
  return SAREK_HIP_OK;
}

int sarek_hip_vector_write(sarek_hip_vector v, const void *src, int64_t first, int64_t count) {
  if (!v || (!src && count > 0)) return fail(SAREK_HIP_E_INVALID_ARG, "vector_write: NULL argument");
  int st = bounds(v, first, count, "set");
  if (st != SAREK_HIP_OK) return st;
  host_copy(static_cast<char *>(v->host) + first * v->elem_size, src, static_cast<size_t>(count * v->elem_size));
  if (count > 0) host_written(v);
  return SAREK_HIP_OK;
}

int sarek_hip_transfer_set_auto(int enabled) {
  g_auto_mode = enabled != 0;
  return SAREK_HIP_OK;
}

int sarek_hip_transfer_to_device(sarek_hip_vector v) {
  if (!v) return fail(SAREK_HIP_E_INVALID_ARG, "to_device: NULL vector");
  int dev = 0;
  int st = current_device(&dev);
  return st != SAREK_HIP_OK ? st : to_device(v, dev);
}

int sarek_hip_transfer_to_cpu(sarek_hip_vector v, int force) {
  if (!v) return fail(SAREK_HIP_E_INVALID_ARG, "to_cpu: NULL vector");
  return to_cpu(v, force != 0);
}

// Transfer.sync (Transfer.ml:336-350)
int sarek_hip_transfer_sync(sarek_hip_vector v) {
  if (!v) return fail(SAREK_HIP_E_INVALID_ARG, "sync: NULL vector");
  switch (v->location) {
    case SAREK_HIP_LOC_GPU: case SAREK_HIP_LOC_STALE_CPU: return to_cpu(v, false);
    case SAREK_HIP_LOC_STALE_GPU: return to_device(v, v->device);
    default: return SAREK_HIP_OK;
  }
}

// Transfer.free_buffer / free_all_buffers (Transfer.ml:353-381)
int sarek_hip_transfer_free_buffers(sarek_hip_vector v) {
  if (!v) return fail(SAREK_HIP_E_INVALID_ARG, "free_buffers: NULL vector");
  int first = SAREK_HIP_OK;
  for (auto &b : v->buffers) {
    int st = sarek_hip_mem_free(b.second);
    sarek_hip_gpu_memory_track_free(static_cast<int64_t>(v->length * v->elem_size));
    if (first == SAREK_HIP_OK) first = st;
  }
  v->buffers.clear();
  v->location = SAREK_HIP_LOC_CPU;
  v->device = -1;
  return first;
}

int sarek_hip_transfer_flush(void) { return sarek_hip_device_synchronize(); }

int sarek_hip_execute_run_vectors(const char *ir_text, const int block[3], const int grid[3], int shared_mem_bytes,
                                  const sarek_hip_varg *args, int n_args) {
  if (!ir_text || !block || !grid || n_args < 0 || (n_args > 0 && !args))
    return fail(SAREK_HIP_E_INVALID_ARG, "run_vectors: NULL or negative argument");
  int dev = 0;
  int st = current_device(&dev);
  if (st != SAREK_HIP_OK) return st;
  if ((st = transfer_args(args, n_args, dev)) != SAREK_HIP_OK) return st;
  std::shared_ptr<const Lowered> k;
  try {
    if ((st = lower(ir_text, block, k)) != SAREK_HIP_OK) return st;
  } catch (const std::exception &e) {
    return fail(SAREK_HIP_E_PARSE, "run_vectors: %s", e.what());
  }
  if ((st = check_args(*k, args, n_args, "run_vectors")) != SAREK_HIP_OK) return st;
  std::vector<sarek_hip_arg> rs;
  if ((st = expand_args(args, n_args, dev, true, rs)) != SAREK_HIP_OK) return st;
  st = sarek_hip_run_source(k->source.c_str(), SAREK_HIP_LANG_HIP_SOURCE, k->name.c_str(), block, grid,
                            shared_mem_bytes, rs.data(), static_cast<int>(rs.size()));
  if (st != SAREK_HIP_OK) return st;
  mark_stale(args, n_args, dev);
  return SAREK_HIP_OK;
}

int sarek_hip_execute_run_pipeline(const sarek_hip_pipeline_stage *stages, int n_stages, int *launches) {
  if (n_stages < 0 || (n_stages > 0 && !stages)) return fail(SAREK_HIP_E_INVALID_ARG, "run_pipeline: NULL or negative argument");
  if (launches) *launches = 0;
  for (int i = 0; i < n_stages; ++i) {
    const sarek_hip_pipeline_stage &s = stages[i];
    if (!s.ir_text || s.n_args < 0 || (s.n_args > 0 && !s.args))
      return fail(SAREK_HIP_E_INVALID_ARG, "run_pipeline: stage %d: NULL or negative argument", i);
  }
  int dev = 0;
  int st = current_device(&dev);
  if (st != SAREK_HIP_OK) return st;
  // per stage what Execute.run_vectors does before and after B.run_source (upload, lower, expand ...
  // mark stale); the launches themselves go to the plugin as one sequence, which may serve neighbours together
  std::vector<std::shared_ptr<const Lowered>> lowered(n_stages);
  std::vector<std::vector<sarek_hip_arg>> expanded(n_stages);
  std::vector<sarek_hip_launch> seq(n_stages);
  for (int i = 0; i < n_stages; ++i) {
    const sarek_hip_pipeline_stage &s = stages[i];
    if ((st = transfer_args(s.args, s.n_args, dev)) != SAREK_HIP_OK) return st;
    try {
      if ((st = lower(s.ir_text, s.block, lowered[i])) != SAREK_HIP_OK) return st;
    } catch (const std::exception &e) {
      return fail(SAREK_HIP_E_PARSE, "run_pipeline: stage %d: %s", i, e.what());
    }
    if ((st = check_args(*lowered[i], s.args, s.n_args, "run_pipeline")) != SAREK_HIP_OK) return st;
    if ((st = expand_args(s.args, s.n_args, dev, true, expanded[i])) != SAREK_HIP_OK) return st;
    sarek_hip_launch &l = seq[i];
    l.source = lowered[i]->source.c_str();
    l.lang = SAREK_HIP_LANG_HIP_SOURCE;
    l.kernel_name = lowered[i]->name.c_str();
    for (int d = 0; d < 3; ++d) {
      l.block[d] = s.block[d];
      l.grid[d] = s.grid[d];
    }
    l.shared_mem_bytes = s.shared_mem_bytes;
    l.args = expanded[i].data();
    l.n_args = static_cast<int>(expanded[i].size());
  }
  int done = 0;
  st = sarek_hip_run_sources(seq.data(), n_stages, launches, &done);
  for (int i = 0; i < done; ++i) mark_stale(stages[i].args, stages[i].n_args, dev);
  return st;
}

int sarek_hip_execute_run_source(const char *source, int lang, const char *kernel_name, const int block[3],
                                 const int grid[3], int shared_mem_bytes, int inject_lengths,
                                 const sarek_hip_varg *args, int n_args) {
  if (!source || !kernel_name || !block || !grid || n_args < 0 || (n_args > 0 && !args))
    return fail(SAREK_HIP_E_INVALID_ARG, "run_source: NULL or negative argument");
  int dev = 0;
  int st = current_device(&dev);
  if (st != SAREK_HIP_OK) return st;
  if ((st = transfer_args(args, n_args, dev)) != SAREK_HIP_OK) return st;
  // Execute.ml:622-633: checked after the uploads, reported as an unsupported argument
  if (!sarek_hip_supports_lang(lang)) {
    static const char *names[] = {"CUDA source", "OpenCL source", "PTX", "SPIR-V", "GLSL source", "HIP source"};
    return fail(SAREK_HIP_E_UNSUPPORTED, "Unsupported argument type %s in HIP backend",
                lang >= 0 && lang <= 5 ? names[lang] : "of an unknown source language");
  }
  std::vector<sarek_hip_arg> rs;
  if ((st = expand_args(args, n_args, dev, inject_lengths != 0, rs)) != SAREK_HIP_OK) return st;
  st = sarek_hip_run_source(source, lang, kernel_name, block, grid, shared_mem_bytes, rs.data(),
                            static_cast<int>(rs.size()));
  if (st != SAREK_HIP_OK) return st;
  mark_stale(args, n_args, dev);
  return SAREK_HIP_OK;
}

// B.supported_source_langs of this backend, as Execute.supports_lang asks it (Execute.ml:589-593)
int sarek_hip_supports_lang(int lang) {
  return lang == SAREK_HIP_LANG_HIP_SOURCE || lang == SAREK_HIP_LANG_CUDA_SOURCE;
}

// Execute.detect_lang (Execute.ml:658-675), with .hip for this backend's own language
int sarek_hip_execute_detect_lang(const char *path, int *lang) {
  if (!path || !lang) return fail(SAREK_HIP_E_INVALID_ARG, "detect_lang: NULL argument");
  const std::string p(path);
  auto ends = [&](const char *suffix) {
    const size_t n = std::strlen(suffix);
    return p.size() >= n && p.compare(p.size() - n, n, suffix) == 0;
  };
  if (ends(".cu")) *lang = SAREK_HIP_LANG_CUDA_SOURCE;
  else if (ends(".hip")) *lang = SAREK_HIP_LANG_HIP_SOURCE;
  else if (ends(".cl")) *lang = SAREK_HIP_LANG_OPENCL_SOURCE;
  else if (ends(".ptx")) *lang = SAREK_HIP_LANG_PTX;
  else if (ends(".spv")) *lang = SAREK_HIP_LANG_SPIR_V;
  else if (ends(".comp") || ends(".glsl")) *lang = SAREK_HIP_LANG_GLSL_SOURCE;
  else
    return fail(SAREK_HIP_E_INVALID_ARG,
                "Invalid file %s: Unknown source file extension (expected .cu, .cl, .ptx, .spv, .comp, or .glsl)", path);
  return SAREK_HIP_OK;
}

// Execute.run_source_file (Execute.ml:711-726): load_source, detect_lang, run_source
int sarek_hip_execute_run_source_file(const char *path, const char *kernel_name, const int block[3], const int grid[3],
                                      int shared_mem_bytes, int inject_lengths, const sarek_hip_varg *args,
                                      int n_args) {
  if (!path) return fail(SAREK_HIP_E_INVALID_ARG, "run_source_file: NULL path");
  std::FILE *f = std::fopen(path, "rb");
  if (!f) return fail(SAREK_HIP_E_INVALID_ARG, "%s: No such file or directory", path);   // Sys_error in the reference
  std::string source;
  char chunk[65536];
  size_t got;
  while ((got = std::fread(chunk, 1, sizeof(chunk), f)) > 0) source.append(chunk, got);
  std::fclose(f);
  int lang = 0;
  int st = sarek_hip_execute_detect_lang(path, &lang);
  if (st != SAREK_HIP_OK) return st;
  return sarek_hip_execute_run_source(source.c_str(), lang, kernel_name, block, grid, shared_mem_bytes, inject_lengths,
                                      args, n_args);
}

// Execute.sync_vectors_to_cpu
int sarek_hip_execute_sync_vectors_to_cpu(const sarek_hip_varg *args, int n_args) {
  if (n_args < 0 || (n_args > 0 && !args)) return fail(SAREK_HIP_E_INVALID_ARG, "sync_vectors_to_cpu: bad arguments");
  for (int i = 0; i < n_args; ++i)
    if (args[i].kind == SAREK_HIP_VARG_VEC && args[i].vec) {
      int st = to_cpu(args[i].vec, false);
      if (st != SAREK_HIP_OK) return st;
    }
  return SAREK_HIP_OK;
}

}  // extern "C"
