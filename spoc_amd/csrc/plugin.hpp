// Internal declarations shared by the plugin-level sources.
#pragma once
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "host/map_fuse.hpp"
namespace sarek_hip {
// First line of a generated source that a hand-written kernel can serve:
// "// sarek-hip-specialise: <tag>".
extern const char *const kSpecialiseMarker;

// generate.cpp: whether sarek_hip_generate_source handed out exactly this tagged text in this process
bool is_generated_tagged_text(const char *source);
// generate.cpp: the rebuilt-class kernel (tags map_f32, tree_sum_map_f32, tree_max_map_f32) behind such a text, if it
// is one, with the kernels compiled from its rebuilt texts so far: a warm launch finds its handle here and builds no text
struct MapEntry {
  ir::MapKernel m;
  struct Built {
    int reduce;          // 0 the map alone, 1 with block sums, 2 with block maxima
    bool nt;             // non-temporal loads
    uint32_t pad_bits;   // fill value of a maximum
    void *kernel;        // sarek_hip_kernel, or nullptr when the rebuilt text did not compile (the generated text serves)
  };
  std::mutex mu;
  std::vector<Built> built;
  uint64_t cache_generation = 0;   // kernel_cache_generation() the handles in `built` belong to
};
// runtime.cpp: changes whenever sarek_hip_kernel_clear_cache has unloaded the cached kernels
uint64_t kernel_cache_generation();
std::shared_ptr<MapEntry> find_generated_map(const char *source);

// library_kernels.cpp: the texts sarek_hip_library_kernel_source hands out
bool is_library_kernel_name(const std::string &name);
bool is_library_kernel_text(const std::string &name, const char *source);
}  // namespace sarek_hip
