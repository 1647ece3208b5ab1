// Internal declarations shared by the plugin-level sources.
#pragma once
#include <string>
namespace sarek_hip {
// First line of a generated source that a hand-written kernel can serve:
// "// sarek-hip-specialise: <tag>".
extern const char *const kSpecialiseMarker;

// generate.cpp: whether sarek_hip_generate_source handed out exactly this tagged text in this process
bool is_generated_tagged_text(const char *source);
// generate.cpp: the element-wise kernel (tag map_f32) behind such a text, if it is one
namespace ir { struct MapKernel; }
bool find_generated_map(const char *source, ir::MapKernel *out);

// library_kernels.cpp: the texts sarek_hip_library_kernel_source hands out
bool is_library_kernel_name(const std::string &name);
bool is_library_kernel_text(const std::string &name, const char *source);
}  // namespace sarek_hip
