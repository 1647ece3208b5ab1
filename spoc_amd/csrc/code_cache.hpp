// On-disk cache of compiled kernels (see code_cache.cpp).
#pragma once
#include <cstddef>
#include <string>
#include <vector>

namespace sarek_hip {
std::string cache_compute_key(const std::string &dev_name, const std::string &driver_version,
                              const std::string &source);
bool cache_dir(std::string *out);
bool cache_get(const std::string &key, std::vector<char> *data);          // counts a hit or a miss
bool cache_put(const std::string &key, const void *data, size_t len);     // counts a put or an error
void cache_note_error();
bool cache_enabled();   // SAREK_HIP_DISK_CACHE != "0"
}  // namespace sarek_hip
