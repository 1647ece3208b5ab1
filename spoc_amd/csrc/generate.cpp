// sarek_hip_generate_source: IR text -> HIP source, with a specialise tag in front when
// the kernel is one a hand-written CDNA4 kernel computes (Hip_plugin.generate_source;
// the reference's counterpart is sarek-cuda/Cuda_plugin.ml:155-157).
#include <cstring>
#include <string>

#include "common.hpp"
#include "host/ir.hpp"
#include "plugin.hpp"

using namespace sarek_hip;

extern "C" int sarek_hip_generate_source(const char *ir_text, const int block[3], char *out,
                                         size_t out_len, size_t *needed) {
  if (!ir_text) return fail(SAREK_HIP_E_INVALID_ARG, "generate_source: NULL IR text");
  std::string src;
  try {
    ir::Kernel k = ir::parse_kernel(ir_text);
    std::string tag = ir::recognise(k);
    if (!tag.empty()) src = std::string(kSpecialiseMarker) + tag + "\n";
    src += ir::generate(k, block);
  } catch (const ir::ParseError &e) {
    return fail(SAREK_HIP_E_PARSE, "%s", e.what());
  } catch (const ir::CodegenError &e) {
    return fail(SAREK_HIP_E_CODEGEN, "%s", e.what());
  } catch (const std::exception &e) {
    return fail(SAREK_HIP_E_CODEGEN, "generate_source: %s", e.what());
  }
  if (needed) *needed = src.size() + 1;
  if (!out || out_len < src.size() + 1)
    return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "generate_source: output needs %zu bytes", src.size() + 1);
  std::memcpy(out, src.c_str(), src.size() + 1);
  return SAREK_HIP_OK;
}
