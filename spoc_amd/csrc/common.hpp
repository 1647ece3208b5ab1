// Shared helpers of libsarek_hip: status handling and the thread-local error text.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "sarek_hip.h"

namespace sarek_hip {

// Thread-local message returned by sarek_hip_last_error().
std::string &last_error_slot();
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

inline int check_hip(hipError_t e, const char *what) {
  if (e == hipSuccess) return SAREK_HIP_OK;
  return fail(static_cast<int>(e), "%s: %s (%s)", what, hipGetErrorString(e), hipGetErrorName(e));
}

#define SAREK_HIP_TRY(expr)                                        \
  do {                                                             \
    int _st = ::sarek_hip::check_hip((expr), #expr);               \
    if (_st != SAREK_HIP_OK) return _st;                           \
  } while (0)

// Call after a kernel launch: reports launch-configuration errors.
inline int check_launch(const char *what) { return check_hip(hipGetLastError(), what); }

inline hipStream_t as_stream(sarek_hip_stream s) { return reinterpret_cast<hipStream_t>(s); }

constexpr int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// The measurement build (-DSAREK_HIP_MEASURE, libsarek_hip_measure.so) carries kernel variants and probes that the
// product library does not have: ablated K loops, retired kernel shapes, the in-kernel clock probe.
#ifdef SAREK_HIP_MEASURE
constexpr bool kMeasureBuild = true;
#else
constexpr bool kMeasureBuild = false;
#endif

}  // namespace sarek_hip
