// sarek_hip_generate_source: IR text -> HIP source, with a specialise tag in front when
// the kernel is one a hand-written CDNA4 kernel computes (Hip_plugin.generate_source;
// the reference's counterpart is sarek-cuda/Cuda_plugin.ml:155-157).
#include <cstring>
#include <mutex>
#include <string>
#include <string_view>
#include <unordered_map>
#include <unordered_set>

#include "common.hpp"
#include "host/ir.hpp"
#include "host/map_fuse.hpp"
#include "plugin.hpp"

namespace sarek_hip {
namespace {
// Every tagged text this process has handed out.  The recogniser matched the whole IR body before it wrote
// the tag, so exactly these texts may be served by a hand-written kernel; any other text that starts with
// the same line is somebody else's program.
struct ViewHash {
  using is_transparent = void;
  size_t operator()(std::string_view v) const { return std::hash<std::string_view>{}(v); }
};
std::mutex g_tagged_mu;
std::unordered_set<std::string, ViewHash, std::equal_to<>> g_tagged;
constexpr size_t kTaggedMax = 4096;     // beyond this the set starts over: forgotten texts run as compiled
// The element-wise kernels among them (tag map_f32), by their text: what run_source needs to rebuild them
std::unordered_map<std::string, std::shared_ptr<MapEntry>, ViewHash, std::equal_to<>> g_maps;
}  // namespace

std::shared_ptr<MapEntry> find_generated_map(const char *source) {
  std::lock_guard<std::mutex> lock(g_tagged_mu);
  const auto it = g_maps.find(std::string_view(source));
  return it == g_maps.end() ? nullptr : it->second;
}

bool is_generated_tagged_text(const char *source) {
  std::lock_guard<std::mutex> lock(g_tagged_mu);
  return g_tagged.find(std::string_view(source)) != g_tagged.end();
}
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" int sarek_hip_generate_source(const char *ir_text, const int block[3], char *out,
                                         size_t out_len, size_t *needed) {
  if (!ir_text) return fail(SAREK_HIP_E_INVALID_ARG, "generate_source: NULL IR text");
  std::string src, tag;
  std::optional<ir::MapKernel> map;
  try {
    ir::Kernel k = ir::parse_kernel(ir_text);
    tag = ir::recognise(k);
    if (tag.empty() && (map = ir::match_map(k))) tag = "map_f32";
    if (tag.empty() && (map = ir::match_tree_sum(k))) tag = "tree_sum_map_f32";
    if (tag.empty() && (map = ir::match_tree_max(k))) tag = "tree_max_map_f32";
    if (!tag.empty()) src = std::string(kSpecialiseMarker) + tag + "\n";
    // A kernel of one of the three rebuilt classes has two texts, this one and the one rebuilt from its expression
    // (host/map_fuse.cpp), and either may serve a launch.  Both evaluate the expression as it is written, every
    // operation rounded once: where the compiler may contract a product into a sum, which products it contracts
    // depends on the code round the expression (an arm of an `if` turned into a branch or a select, a
    // scalar-only product shared by the sixteen elements of a thread), and the two texts would differ in last bits.
    if (map) src += "#pragma clang fp contract(off)\n";
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
  if (!tag.empty()) {
    std::lock_guard<std::mutex> lock(g_tagged_mu);
    if (g_tagged.size() >= kTaggedMax) {
      g_tagged.clear();
      g_maps.clear();
    }
    if (map && g_maps.find(std::string_view(src)) == g_maps.end()) {
      auto entry = std::make_shared<MapEntry>();
      entry->m = std::move(*map);
      g_maps.emplace(src, std::move(entry));
    }
    g_tagged.insert(std::move(src));
  }
  return SAREK_HIP_OK;
}

extern "C" int sarek_hip_rebuilt_source(const char *ir_text, int reduce, uint32_t pad_bits, char *out, size_t out_len,
                                        size_t *needed) {
  if (!ir_text) return fail(SAREK_HIP_E_INVALID_ARG, "rebuilt_source: NULL IR text");
  if (reduce < 0 || reduce > 2) return fail(SAREK_HIP_E_INVALID_ARG, "rebuilt_source: reduce must be 0, 1 or 2");
  std::string src;
  try {
    ir::Kernel k = ir::parse_kernel(ir_text);
    if (!ir::recognise(k).empty())
      return fail(SAREK_HIP_E_UNSUPPORTED, "rebuilt_source: a hand-written kernel serves this IR");
    if (auto m = ir::match_map(k)) src = ir::map_source(*m, reduce, true, pad_bits);
    else if (auto t = ir::match_tree_sum(k)) src = ir::tree_sum_source(*t, true);
    else if (auto x = ir::match_tree_max(k)) src = ir::tree_max_source(*x);
    else return fail(SAREK_HIP_E_UNSUPPORTED, "rebuilt_source: the IR is of none of the rebuilt classes");
  } catch (const ir::ParseError &e) {
    return fail(SAREK_HIP_E_PARSE, "%s", e.what());
  } catch (const std::exception &e) {
    return fail(SAREK_HIP_E_CODEGEN, "rebuilt_source: %s", e.what());
  }
  if (needed) *needed = src.size() + 1;
  if (!out || out_len < src.size() + 1)
    return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "rebuilt_source: output needs %zu bytes", src.size() + 1);
  std::memcpy(out, src.c_str(), src.size() + 1);
  return SAREK_HIP_OK;
}
