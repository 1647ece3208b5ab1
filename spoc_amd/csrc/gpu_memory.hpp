#pragma once
#include <cstdint>

namespace sarek_hip {
// A device buffer released because its vector went away (the reference's finaliser), as opposed to an
// explicit Transfer.free_buffer: counted apart (Gpu_memory.ml:163-178).
void track_gc_free(int64_t bytes);
}  // namespace sarek_hip
