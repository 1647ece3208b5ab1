#include "common.hpp"
extern "C" int sarek_hip_generate_source(const char *, const int *, char *, size_t, size_t *) {
  return sarek_hip::fail(SAREK_HIP_E_UNSUPPORTED, "generate_source: IR lowering not built in");
}
