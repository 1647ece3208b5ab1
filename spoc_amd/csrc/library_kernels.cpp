// Library kernels: named HIP sources for the operations that have no kernel in the reference's
// bench suite (16-bit-input GEMMs, the fused GEMM epilogue, triad + sum).  A caller fetches the
// text with sarek_hip_library_kernel_source and runs it like any external kernel,
//   Execute.run_source ~lang:HIP_Source ~source ~kernel_name ~block ~grid args
// (sarek/sarek/Execute.ml:613-651; sarek/tests/e2e/test_external_kernel.ml:46-62).  Every text is a
// complete program: plain HIP that computes the operation with the arithmetic the Native backend
// would use (operands widened to double, one rounding at each store), under the launch geometry
// its comment states.  Its first line is a specialise tag, so run_source serves the launch with
// the hand-written MFMA / streaming kernel instead when specialisation is on and the arguments fit.
//
// Arguments follow Execute.expand_to_run_source_args (Execute.ml:197-216): every vector is a
// device pointer followed by its int32 length.  bf16 / fp16 matrices are vectors of 2-byte
// custom elements (Vector.create_custom, sarek/core/Vector.ml:60-76) holding the bit patterns.
#include <cstring>
#include <string>

#include "common.hpp"
#include "plugin.hpp"

namespace sarek_hip {
namespace {

struct LibraryKernel {
  const char *name;     // also the specialise tag
  const char *entry;    // kernel_name to pass to run_source
  const char *source;
};

#define SAREK_GEMM16_BODY(DECODE)                                                                  \
  "  int col = threadIdx.x + blockIdx.x * blockDim.x;\n"                                          \
  "  int row = threadIdx.y + blockIdx.y * blockDim.y;\n"                                          \
  "  if (row < m && col < n) {\n"                                                                 \
  "    double sum = 0.0;\n"                                                                       \
  "    for (int i = 0; i < k; ++i)\n"                                                             \
  "      sum += (double)" DECODE "(a[(long long)row * k + i]) * (double)" DECODE "(b[(long long)i * n + col]);\n" \
  "    c[(long long)row * n + col] = (float)sum;\n"                                               \
  "  }\n"

const char kBf16Decode[] =
    "__device__ inline float sarek_bf16(unsigned short h) { return __uint_as_float((unsigned)h << 16); }\n";
const char kF16Decode[] =
    "__device__ inline float sarek_f16(unsigned short h) { return (float)__builtin_bit_cast(_Float16, h); }\n";

const std::string kGemmBf16 =
    std::string("// sarek-hip-specialise: gemm_bf16\n"
                "// C[m x n] = A[m x k] . B[k x n], row-major; a, b: bf16 bit patterns, c: f32.\n"
                "// Launch: 2-D, one thread per element of C (block.x * grid.x >= n, block.y * grid.y >= m).\n") +
    kBf16Decode +
    "extern \"C\" __global__ void sarek_gemm_bf16(const unsigned short* a, int a_len, const unsigned short* b, int b_len,\n"
    "                                           float* c, int c_len, int m, int n, int k) {\n" SAREK_GEMM16_BODY("sarek_bf16") "}\n";

const std::string kGemmF16 =
    std::string("// sarek-hip-specialise: gemm_f16\n"
                "// C[m x n] = A[m x k] . B[k x n], row-major; a, b: IEEE fp16 bit patterns, c: f32.\n"
                "// Launch: 2-D, one thread per element of C (block.x * grid.x >= n, block.y * grid.y >= m).\n") +
    kF16Decode +
    "extern \"C\" __global__ void sarek_gemm_f16(const unsigned short* a, int a_len, const unsigned short* b, int b_len,\n"
    "                                          float* c, int c_len, int m, int n, int k) {\n" SAREK_GEMM16_BODY("sarek_f16") "}\n";

const std::string kGemmF16Epilogue =
    std::string("// sarek-hip-specialise: gemm_f16_bias_relu_rowsum\n"
                "// y = relu(A . B + bias[col]) (f32, [m x n]) and rowsum[r] = sum over c of y[r, c]; a, b: fp16 bit patterns.\n"
                "// Launch: 1-D, any block and grid; a workgroup takes whole rows (row = blockIdx.x, + gridDim.x, ...).\n") +
    kF16Decode +
    "extern \"C\" __global__ void sarek_gemm_f16_bias_relu_rowsum(const unsigned short* a, int a_len, const unsigned short* b, int b_len,\n"
    "    const float* bias, int bias_len, float* y, int y_len, float* rowsum, int rowsum_len, int m, int n, int k) {\n"
    "  for (int row = blockIdx.x; row < m; row += gridDim.x) {\n"
    "    for (int col = threadIdx.x; col < n; col += blockDim.x) {\n"
    "      double sum = 0.0;\n"
    "      for (int i = 0; i < k; ++i)\n"
    "        sum += (double)sarek_f16(a[(long long)row * k + i]) * (double)sarek_f16(b[(long long)i * n + col]);\n"
    "      sum += (double)bias[col];\n"
    "      y[(long long)row * n + col] = (float)(sum > 0.0 ? sum : 0.0);\n"
    "    }\n"
    "    __syncthreads();\n"
    "    if (threadIdx.x == 0) {\n"
    "      double s = 0.0;\n"
    "      for (int col = 0; col < n; ++col) s += (double)y[(long long)row * n + col];\n"
    "      rowsum[row] = (float)s;\n"
    "    }\n"
    "    __syncthreads();\n"
    "  }\n"
    "}\n";

const std::string kTriadSum =
    "// sarek-hip-specialise: triad_sum_f32\n"
    "// a[i] = b[i] + c[i] * scalar for i < n, and sum[0] = sum of a (double).\n"
    "// Launch: ONE 1-D workgroup of a power-of-two size up to 1024 (grid 1 x 1 x 1); it walks the vector.\n"
    "extern \"C\" __global__ void sarek_triad_sum_f32(float* a, int a_len, const float* b, int b_len, const float* c, int c_len,\n"
    "                                               double* sum, int sum_len, float scalar, int n) {\n"
    "  __shared__ double part[1024];\n"
    "  double acc = 0.0;\n"
    "  for (int i = threadIdx.x; i < n; i += blockDim.x) {\n"
    "    float v = (float)((double)b[i] + (double)c[i] * (double)scalar);\n"
    "    a[i] = v;\n"
    "    acc += (double)v;\n"
    "  }\n"
    "  part[threadIdx.x] = acc;\n"
    "  __syncthreads();\n"
    "  for (int half = blockDim.x / 2; half >= 1; half /= 2) {\n"
    "    if (threadIdx.x < half) part[threadIdx.x] += part[threadIdx.x + half];\n"
    "    __syncthreads();\n"
    "  }\n"
    "  if (threadIdx.x == 0) sum[0] = part[0];\n"
    "}\n";

const LibraryKernel kKernels[] = {
    {"gemm_bf16", "sarek_gemm_bf16", kGemmBf16.c_str()},
    {"gemm_f16", "sarek_gemm_f16", kGemmF16.c_str()},
    {"gemm_f16_bias_relu_rowsum", "sarek_gemm_f16_bias_relu_rowsum", kGemmF16Epilogue.c_str()},
    {"triad_sum_f32", "sarek_triad_sum_f32", kTriadSum.c_str()},
};

int copy_out(const std::string &text, char *out, size_t cap, size_t *needed, const char *what) {
  if (needed) *needed = text.size() + 1;
  if (!out || cap < text.size() + 1)
    return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "%s: %zu bytes needed", what, text.size() + 1);
  std::memcpy(out, text.c_str(), text.size() + 1);
  return SAREK_HIP_OK;
}

}  // namespace

// Whether `source` is, byte for byte, the library's text of that name: only then does a hand-written
// kernel stand in for it (a caller's own text that merely starts with the same tag line is compiled).
bool is_library_kernel_text(const std::string &name, const char *source) {
  for (const LibraryKernel &k : kKernels)
    if (name == k.name) return std::strcmp(k.source, source) == 0;
  return false;
}
bool is_library_kernel_name(const std::string &name) {
  for (const LibraryKernel &k : kKernels)
    if (name == k.name) return true;
  return false;
}
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_library_kernel_source(const char *name, char *source, size_t source_cap, size_t *source_needed,
                                    char *entry, size_t entry_cap) {
  if (!name) return fail(SAREK_HIP_E_INVALID_ARG, "library_kernel_source: NULL name");
  for (const LibraryKernel &k : kKernels) {
    if (std::strcmp(k.name, name) != 0) continue;
    if (entry) {
      int rc = copy_out(k.entry, entry, entry_cap, nullptr, "library_kernel_source (entry name)");
      if (rc != SAREK_HIP_OK) return rc;
    }
    return copy_out(k.source, source, source_cap, source_needed, "library_kernel_source");
  }
  return fail(SAREK_HIP_E_INVALID_ARG, "library_kernel_source: no library kernel is called '%s'", name);
}

int sarek_hip_library_kernel_list(char *out, size_t cap, size_t *needed) {
  std::string all;
  for (const LibraryKernel &k : kKernels) {
    if (!all.empty()) all += ' ';
    all += k.name;
  }
  return copy_out(all, out, cap, needed, "library_kernel_list");
}
}
