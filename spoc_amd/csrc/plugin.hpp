// Internal declarations shared by the plugin-level sources.
#pragma once
namespace sarek_hip {
// First line of a generated source that a hand-written kernel can serve:
// "// sarek-hip-specialise: <tag>".
extern const char *const kSpecialiseMarker;
}  // namespace sarek_hip
