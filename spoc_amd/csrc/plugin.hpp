// Internal declarations shared by the plugin-level sources.
#pragma once
#include <string>

#include "sarek_hip.h"

namespace sarek_hip {
// First line of a generated source that a hand-written kernel can serve:
// "// sarek-hip-specialise: <tag>".
extern const char *const kSpecialiseMarker;

// What sarek_hip_last_run_path reports for this thread.
void set_last_run_path(const std::string &path);

// Two consecutive launches (generated sources with their specialise tags, launch geometry, expanded
// arguments) that one hand-written kernel can serve: returns 1 and its status in *rc, else 0 and
// nothing was launched.
int run_specialised_pair(const char *source0, const int block0[3], const int grid0[3], const sarek_hip_arg *args0,
                         int n_args0, const char *source1, const int block1[3], const int grid1[3],
                         const sarek_hip_arg *args1, int n_args1, int *rc);
}  // namespace sarek_hip
