// Integer tuning knobs (launch shapes, tile variants) that can be changed at run
// time through sarek_hip_set_tunable() without rebuilding; used for sweeps.
#pragma once
#include <cstdint>

namespace sarek_hip {
// Value of knob `name`, or `fallback` when it was never set.  An environment
// variable SAREK_HIP_TUNE_<name with '.' replaced by '_'> seeds the knob on first use.
int64_t tunable(const char *name, int64_t fallback);
void set_tunable(const char *name, int64_t value);
// Clock-probe buffer for a launch of `workgroups` workgroups, or nullptr.
unsigned long long *clock_probe(int64_t workgroups);
}  // namespace sarek_hip
