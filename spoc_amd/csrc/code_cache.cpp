// Persistent on-disk cache of compiled kernels, the counterpart of the reference's
// Framework_cache (sarek/framework/Framework_cache.ml:63-141): same directory rule
// ($XDG_CACHE_HOME, else $HOME/.cache, else the temp dir, then "spoc"), same key
// (MD5 hex of device name ^ driver version ^ source), one file per key, counters for hits,
// misses, puts and I/O errors; cache failures never fail the caller.  Here the stored
// bytes are hiprtc code objects; sarek_hip_kernel_compile(_cached) consults it before
// compiling (SAREK_HIP_DISK_CACHE=0 switches that off).
#include "code_cache.hpp"

#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "common.hpp"
#include "sarek_hip.h"

namespace sarek_hip {
namespace {

std::mutex g_mu;
int64_t g_hits = 0, g_misses = 0, g_puts = 0, g_errors = 0;

// ---- MD5 (RFC 1321) ---------------------------------------------------------------
struct Md5 {
  uint32_t a = 0x67452301u, b = 0xefcdab89u, c = 0x98badcfeu, d = 0x10325476u;
  uint64_t bytes = 0;
  unsigned char buf[64];
  size_t fill = 0;

  static uint32_t rol(uint32_t x, int s) { return (x << s) | (x >> (32 - s)); }

  void block(const unsigned char *p) {
    static const uint32_t K[64] = {
        0xd76aa478, 0xe8c7b756, 0x242070db, 0xc1bdceee, 0xf57c0faf, 0x4787c62a, 0xa8304613, 0xfd469501,
        0x698098d8, 0x8b44f7af, 0xffff5bb1, 0x895cd7be, 0x6b901122, 0xfd987193, 0xa679438e, 0x49b40821,
        0xf61e2562, 0xc040b340, 0x265e5a51, 0xe9b6c7aa, 0xd62f105d, 0x02441453, 0xd8a1e681, 0xe7d3fbc8,
        0x21e1cde6, 0xc33707d6, 0xf4d50d87, 0x455a14ed, 0xa9e3e905, 0xfcefa3f8, 0x676f02d9, 0x8d2a4c8a,
        0xfffa3942, 0x8771f681, 0x6d9d6122, 0xfde5380c, 0xa4beea44, 0x4bdecfa9, 0xf6bb4b60, 0xbebfbc70,
        0x289b7ec6, 0xeaa127fa, 0xd4ef3085, 0x04881d05, 0xd9d4d039, 0xe6db99e5, 0x1fa27cf8, 0xc4ac5665,
        0xf4292244, 0x432aff97, 0xab9423a7, 0xfc93a039, 0x655b59c3, 0x8f0ccc92, 0xffeff47d, 0x85845dd1,
        0x6fa87e4f, 0xfe2ce6e0, 0xa3014314, 0x4e0811a1, 0xf7537e82, 0xbd3af235, 0x2ad7d2bb, 0xeb86d391};
    static const int S[64] = {7, 12, 17, 22, 7, 12, 17, 22, 7, 12, 17, 22, 7, 12, 17, 22,
                              5, 9,  14, 20, 5, 9,  14, 20, 5, 9,  14, 20, 5, 9,  14, 20,
                              4, 11, 16, 23, 4, 11, 16, 23, 4, 11, 16, 23, 4, 11, 16, 23,
                              6, 10, 15, 21, 6, 10, 15, 21, 6, 10, 15, 21, 6, 10, 15, 21};
    uint32_t m[16];
    for (int i = 0; i < 16; ++i)
      m[i] = static_cast<uint32_t>(p[4 * i]) | (static_cast<uint32_t>(p[4 * i + 1]) << 8) |
             (static_cast<uint32_t>(p[4 * i + 2]) << 16) | (static_cast<uint32_t>(p[4 * i + 3]) << 24);
    uint32_t A = a, B = b, C = c, D = d;
    for (int i = 0; i < 64; ++i) {
      uint32_t f;
      int g;
      if (i < 16) {
        f = (B & C) | (~B & D);
        g = i;
      } else if (i < 32) {
        f = (D & B) | (~D & C);
        g = (5 * i + 1) & 15;
      } else if (i < 48) {
        f = B ^ C ^ D;
        g = (3 * i + 5) & 15;
      } else {
        f = C ^ (B | ~D);
        g = (7 * i) & 15;
      }
      const uint32_t t = D;
      D = C;
      C = B;
      B = B + rol(A + f + K[i] + m[g], S[i]);
      A = t;
    }
    a += A;
    b += B;
    c += C;
    d += D;
  }

  void update(const void *data, size_t n) {
    const unsigned char *p = static_cast<const unsigned char *>(data);
    bytes += n;
    while (n > 0) {
      const size_t take = n < 64 - fill ? n : 64 - fill;
      std::memcpy(buf + fill, p, take);
      fill += take;
      p += take;
      n -= take;
      if (fill == 64) {
        block(buf);
        fill = 0;
      }
    }
  }

  std::string hex() {
    const uint64_t bits = bytes * 8;
    const unsigned char one = 0x80, zero = 0;
    update(&one, 1);
    while (fill != 56) update(&zero, 1);
    unsigned char len[8];
    for (int i = 0; i < 8; ++i) len[i] = static_cast<unsigned char>(bits >> (8 * i));
    update(len, 8);
    const uint32_t w[4] = {a, b, c, d};
    char out[33];
    for (int i = 0; i < 16; ++i)
      std::snprintf(out + 2 * i, 3, "%02x", static_cast<unsigned>((w[i / 4] >> (8 * (i % 4))) & 0xff));
    return std::string(out, 32);
  }
};

bool is_dir(const std::string &p) {
  struct stat st;
  return ::stat(p.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

// A key names a file directly under the cache directory: no separators, no "." / "..".
bool key_ok(const char *key) {
  if (!key || !*key || std::strlen(key) > 200) return false;
  if (!std::strcmp(key, ".") || !std::strcmp(key, "..")) return false;
  for (const char *p = key; *p; ++p)
    if (*p == '/' || *p == '\\') return false;
  return true;
}

}  // namespace

std::string cache_compute_key(const std::string &dev_name, const std::string &driver_version,
                              const std::string &source) {
  Md5 h;
  h.update(dev_name.data(), dev_name.size());
  h.update(driver_version.data(), driver_version.size());
  h.update(source.data(), source.size());
  return h.hex();
}

bool cache_dir(std::string *out) {
  std::string base;
  if (const char *x = std::getenv("XDG_CACHE_HOME"); x && *x) {
    base = x;
  } else if (const char *h = std::getenv("HOME"); h && *h) {
    base = std::string(h) + "/.cache";
    if (!is_dir(base)) ::mkdir(base.c_str(), 0755);
  } else {
    const char *t = std::getenv("TMPDIR");
    base = (t && *t) ? t : "/tmp";
  }
  const std::string dir = base + "/spoc";
  if (!is_dir(dir) && ::mkdir(dir.c_str(), 0755) != 0 && !is_dir(dir)) return false;
  *out = dir;
  return true;
}

bool cache_get(const std::string &key, std::vector<char> *data) {
  std::lock_guard<std::mutex> lock(g_mu);
  std::string dir;
  if (!key_ok(key.c_str()) || !cache_dir(&dir)) {
    ++g_errors;
    return false;
  }
  const std::string path = dir + "/" + key;
  std::FILE *f = std::fopen(path.c_str(), "rb");
  if (!f) {
    if (errno == ENOENT) ++g_misses; else ++g_errors;
    return false;
  }
  bool ok = std::fseek(f, 0, SEEK_END) == 0;
  const long len = ok ? std::ftell(f) : -1;
  ok = ok && len >= 0 && std::fseek(f, 0, SEEK_SET) == 0;
  if (ok) {
    data->resize(static_cast<size_t>(len));
    ok = len == 0 || std::fread(data->data(), 1, static_cast<size_t>(len), f) == static_cast<size_t>(len);
  }
  std::fclose(f);
  if (ok) ++g_hits; else ++g_errors;
  return ok;
}

bool cache_put(const std::string &key, const void *data, size_t len) {
  std::lock_guard<std::mutex> lock(g_mu);
  std::string dir;
  if (!key_ok(key.c_str()) || !cache_dir(&dir)) {
    ++g_errors;
    return false;
  }
  // write to a private name, then rename: readers never see a half-written entry
  const std::string path = dir + "/" + key;
  const std::string tmp = path + ".tmp" + std::to_string(static_cast<long>(::getpid()));
  std::FILE *f = std::fopen(tmp.c_str(), "wb");
  bool ok = f != nullptr;
  if (ok) {
    ok = len == 0 || std::fwrite(data, 1, len, f) == len;
    ok = (std::fclose(f) == 0) && ok;
    ok = ok && std::rename(tmp.c_str(), path.c_str()) == 0;
    if (!ok) std::remove(tmp.c_str());
  }
  if (ok) ++g_puts; else ++g_errors;
  return ok;
}

void cache_note_error() {
  std::lock_guard<std::mutex> lock(g_mu);
  ++g_errors;
}

bool cache_enabled() {
  const char *e = std::getenv("SAREK_HIP_DISK_CACHE");
  return !(e && e[0] == '0');
}

}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_cache_dir(char *out, size_t out_len) {
  std::string dir;
  if (!out || out_len == 0) return fail(SAREK_HIP_E_INVALID_ARG, "cache_dir: NULL buffer");
  if (!cache_dir(&dir)) return fail(SAREK_HIP_E_UNSUPPORTED, "cache_dir: cannot create the cache directory");
  if (dir.size() + 1 > out_len) return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "cache_dir: buffer too small");
  std::memcpy(out, dir.c_str(), dir.size() + 1);
  return SAREK_HIP_OK;
}

int sarek_hip_cache_compute_key(const char *dev_name, const char *driver_version, const char *source,
                                char out_hex[33]) {
  if (!dev_name || !driver_version || !source || !out_hex)
    return fail(SAREK_HIP_E_INVALID_ARG, "cache_compute_key: NULL argument");
  const std::string k = cache_compute_key(dev_name, driver_version, source);
  std::memcpy(out_hex, k.c_str(), 33);
  return SAREK_HIP_OK;
}

int sarek_hip_cache_get(const char *key, void *out, size_t out_len, size_t *size, int *found) {
  if (!key || !size || !found) return fail(SAREK_HIP_E_INVALID_ARG, "cache_get: NULL argument");
  std::vector<char> data;
  *size = 0;
  *found = cache_get(key, &data) ? 1 : 0;
  if (!*found) return SAREK_HIP_OK;
  *size = data.size();
  if (data.size() > out_len || (!out && !data.empty()))
    return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "cache_get: entry has %zu bytes, buffer %zu", data.size(), out_len);
  if (!data.empty()) std::memcpy(out, data.data(), data.size());
  return SAREK_HIP_OK;
}

int sarek_hip_cache_put(const char *key, const void *data, size_t len) {
  if (!key || (!data && len)) return fail(SAREK_HIP_E_INVALID_ARG, "cache_put: NULL argument");
  cache_put(key, data, len);   // failures are counted, never reported (as in the reference)
  return SAREK_HIP_OK;
}

int sarek_hip_cache_get_stats(int64_t out[4]) {
  if (!out) return fail(SAREK_HIP_E_INVALID_ARG, "cache_get_stats: NULL argument");
  std::lock_guard<std::mutex> lock(g_mu);
  out[0] = g_hits;
  out[1] = g_misses;
  out[2] = g_puts;
  out[3] = g_errors;
  return SAREK_HIP_OK;
}

int sarek_hip_cache_reset_stats(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  g_hits = g_misses = g_puts = g_errors = 0;
  return SAREK_HIP_OK;
}
}
