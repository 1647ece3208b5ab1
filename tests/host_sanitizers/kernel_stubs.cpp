// Stand-ins for the entry points defined in the .hip files, so that the host sources link without them.
// Nothing in the sanitizer run launches a kernel.
#include "sarek_hip.h"
extern "C" {
int sarek_hip_copy_f32(float *, const float *, int64_t, sarek_hip_stream) { return -1; }
int sarek_hip_dot_block256_f32(const float *, const float *, float *, int64_t, sarek_hip_stream) { return -1; }
int sarek_hip_gemm_f32(const float *, const float *, float *, int, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_histogram_i32(int32_t *, const int32_t *, int64_t, int, sarek_hip_stream) { return -1; }
int sarek_hip_radix_histogram_i32(int32_t *, const int32_t *, int64_t, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_radix_scatter_i32(int32_t *, int64_t, int32_t *, const int32_t *, int64_t, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_reduce_max_block256_f32(const float *, float *, int64_t, float, sarek_hip_stream) { return -1; }
int sarek_hip_reduce_sum_block256_f32(const float *, float *, int64_t, sarek_hip_stream) { return -1; }
int sarek_hip_transpose_f32(const float *, float *, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_stencil_2d_f32(const float *, float *, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_conv2d_f32(const float *, float *, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_triad_f32(float *, const float *, const float *, float, int64_t, sarek_hip_stream) { return -1; }
int sarek_hip_triad_block256_sum_f32(float *, const float *, const float *, float, int64_t, float *, sarek_hip_stream) { return -1; }
int sarek_hip_triad_block256_max_f32(float *, const float *, const float *, float, int64_t, float, float *, sarek_hip_stream) { return -1; }
int sarek_hip_triad_sum_f32_static(float *, const float *, const float *, float, int64_t, double *, sarek_hip_stream) { return -1; }
int sarek_hip_gemm_bf16(const uint16_t *, const uint16_t *, float *, int, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_gemm_f16(const uint16_t *, const uint16_t *, float *, int, int, int, sarek_hip_stream) { return -1; }
int sarek_hip_gemm_f16_bias_relu_rowsum(const uint16_t *, const uint16_t *, const float *, float *, float *, int, int, int,
                                        sarek_hip_stream) { return -1; }
}

namespace sarek_hip { extern const char *const kSpecialiseMarker; }
