// Host code of the library under AddressSanitizer and UndefinedBehaviorSanitizer (and, with "threads" as the second
// argument, under ThreadSanitizer), without a GPU:
//  - every record of the input file (IR texts, most of them damaged) through the reader, the HIP
//    lowering and the fusion entry points;
//  - the Vector module's storage functions (views over a shared host block, partition, blit, copy,
//    the threaded bulk copy), none of which touches the device.
// Built and run by test_host_sanitizers.py; the hand-kernel entry points that plugin.cpp refers to
// are stubbed (kernel_stubs.cpp), the .hip files are not part of the build.
#include <atomic>
#include <cstdio>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "sarek_hip.h"

static int damaged_ir(const char *path) {
  FILE *f = std::fopen(path, "rb");
  if (!f) return 10;
  std::string all;
  char buf[65536];
  size_t n;
  while ((n = std::fread(buf, 1, sizeof(buf), f)) > 0) all.append(buf, n);
  std::fclose(f);
  std::vector<std::string> recs;            // NUL-separated records
  for (size_t at = 0; at < all.size();) {
    size_t e = all.find('\0', at);
    if (e == std::string::npos) e = all.size();
    recs.emplace_back(all.substr(at, e - at));
    at = e + 1;
  }
  std::vector<char> out(1 << 18);
  long ok = 0, bad = 0, fused = 0;
  const int block[3] = {256, 1, 1};
  for (size_t i = 0; i < recs.size(); ++i) {
    size_t need = 0;
    int rc = sarek_hip_generate_source(recs[i].c_str(), (i & 1) ? block : nullptr, out.data(), out.size(), &need);
    rc == 0 ? ++ok : ++bad;
    size_t need2 = 0;
    sarek_hip_fusion_analyze(recs[i].c_str(), out.data(), out.size(), &need2);
    if (i > 0) {
      int can = 0;
      static const char *names[] = {"output", "a"};
      for (const char *nm : names)
        for (int mode = 0; mode < 5; ++mode) {
          int did = 0;
          sarek_hip_fusion_can_fuse(recs[i - 1].c_str(), recs[i].c_str(), nm, mode, &can);
          if (sarek_hip_fusion_fuse(recs[i - 1].c_str(), recs[i].c_str(), nm, mode, &did, out.data(), out.size(), &need2) == 0 && did) ++fused;
          int dec = 0; char reason[256];
          sarek_hip_fusion_should_fuse(recs[i - 1].c_str(), recs[i].c_str(), nm, &dec, reason, sizeof(reason));
        }
    }
  }
  std::printf("records %zu ok %ld bad %ld fused %ld\n", recs.size(), ok, bad, fused);
  return 0;
}


#define CHECK(x) do { int _rc = (x); if (_rc != 0) { std::printf("line %d: rc %d %s\n", __LINE__, _rc, sarek_hip_last_error()); return 1; } } while (0)
static int vector_storage() {
  sarek_hip_vector v, s, g, c, parts[3];
  CHECK(sarek_hip_vector_create(SAREK_HIP_KIND_FLOAT32, 1000, 0, 0, &v));
  float x = 2.5f;
  CHECK(sarek_hip_vector_fill(v, &x));
  CHECK(sarek_hip_vector_sub(v, 100, 500, -1, 0, &s));
  CHECK(sarek_hip_vector_sub(s, 10, 20, 5, 5, &g));
  CHECK(sarek_hip_vector_copy(s, &c));
  std::vector<float> buf(500, 1.0f);
  CHECK(sarek_hip_vector_write(s, buf.data(), 0, 500));
  CHECK(sarek_hip_vector_read(v, buf.data(), 100, 500));
  CHECK(sarek_hip_vector_blit(v, 0, c, 10, 490));
  CHECK(sarek_hip_vector_blit(v, 0, v, 1, 999));
  if (sarek_hip_vector_blit(v, 0, c, 10, 491) == 0) return 2;
  if (sarek_hip_vector_sub(v, 900, 101, -1, 0, &parts[0]) == 0) return 3;
  int devs[3] = {0, 0, 0};
  CHECK(sarek_hip_vector_partition(v, 3, devs, parts));
  char text[256];
  CHECK(sarek_hip_vector_to_string(g, text, sizeof(text)));
  std::printf("%s\n", text);
  CHECK(sarek_hip_vector_destroy(v));                 // the views keep the block alive
  float y = 0;
  CHECK(sarek_hip_vector_get(g, 19, &y));
  CHECK(sarek_hip_vector_set(parts[2], 332, &y));
  CHECK(sarek_hip_vector_destroy(s));
  CHECK(sarek_hip_vector_destroy(c));
  for (auto p : parts) CHECK(sarek_hip_vector_destroy(p));
  CHECK(sarek_hip_vector_get(g, 0, &y));
  CHECK(sarek_hip_vector_destroy(g));
  // a large bulk write and read: the four-thread copy
  sarek_hip_vector big;
  const long n = 9 << 20;
  CHECK(sarek_hip_vector_create(SAREK_HIP_KIND_INT32, n, 0, 0, &big));
  std::vector<int> data(n), back(n);
  for (long i = 0; i < n; ++i) data[i] = (int)(i * 2654435761u);
  CHECK(sarek_hip_vector_write(big, data.data(), 0, n));
  CHECK(sarek_hip_vector_read(big, back.data(), 0, n));
  if (std::memcmp(data.data(), back.data(), n * 4) != 0) return 4;
  CHECK(sarek_hip_vector_write(big, data.data() + 5, 3, n - 10));
  CHECK(sarek_hip_vector_read(big, back.data(), 3, n - 10));
  if (std::memcmp(data.data() + 5, back.data(), (n - 10) * 4) != 0) return 5;
  CHECK(sarek_hip_vector_destroy(big));
  std::printf("vector storage ok\n");
  return 0;
}

// Eight threads at once through everything that keeps state between calls: the lowering's caches of tagged
// texts and rebuilt-kernel entries (the same IR texts from every thread), the fusion entry points, tunables set and
// read, the device-memory counters, the persistent cache's key function, and vectors of each thread's own.  Built
// with ThreadSanitizer by the test: a data race in the library's bookkeeping is a failure.
static int threads(const char *path) {
  FILE *f = std::fopen(path, "rb");
  if (!f) return 10;
  std::string all;
  char buf[65536];
  size_t n;
  while ((n = std::fread(buf, 1, sizeof(buf), f)) > 0) all.append(buf, n);
  std::fclose(f);
  std::vector<std::string> recs;
  for (size_t at = 0; at < all.size();) {
    size_t e = all.find('\0', at);
    if (e == std::string::npos) e = all.size();
    recs.emplace_back(all.substr(at, e - at));
    at = e + 1;
  }
  std::atomic<long> lowered{0}, failed{0};
  auto work = [&](int t) {
    std::vector<char> out(1 << 18);
    const int block[3] = {256, 1, 1};
    for (size_t i = 0; i < recs.size(); ++i) {
      size_t need = 0;
      // every thread lowers every text: the caches see the same keys from all sides
      int rc = sarek_hip_generate_source(recs[i].c_str(), ((i + t) & 1) ? block : nullptr, out.data(), out.size(), &need);
      (rc == 0 ? lowered : failed).fetch_add(1);
      if (rc == 0 && (i + t) % 3 == 0) {
        size_t need2 = 0;
        std::vector<char> rebuilt(1 << 18);
        sarek_hip_rebuilt_source(recs[i].c_str(), (int)(i % 2), 0u, rebuilt.data(), rebuilt.size(), &need2);
      }
      if (i > 0 && (i + t) % 4 == 0) {
        int did = 0;
        size_t need2 = 0;
        sarek_hip_fusion_fuse(recs[i - 1].c_str(), recs[i].c_str(), "output", 3, &did, out.data(), out.size(), &need2);
      }
      sarek_hip_set_tunable("stream.nt", (int64_t)((i + t) % 3) - 1);
      sarek_hip_gpu_memory_track_alloc(64);
      sarek_hip_gpu_memory_track_free(64);
      sarek_hip_gpu_memory_stats_t st;
      sarek_hip_gpu_memory_stats(&st);
      char key[64];
      sarek_hip_cache_compute_key("device", "driver", recs[i].c_str(), key);
    }
    sarek_hip_vector v, c;
    if (sarek_hip_vector_create(SAREK_HIP_KIND_FLOAT32, 4096, 0, 0, &v) != 0) return;
    float x = (float)t;
    sarek_hip_vector_fill(v, &x);
    sarek_hip_vector_copy(v, &c);
    sarek_hip_vector_destroy(v);
    sarek_hip_vector_destroy(c);
  };
  std::vector<std::thread> pool;
  for (int t = 0; t < 8; ++t) pool.emplace_back(work, t);
  for (auto &th : pool) th.join();
  sarek_hip_set_tunable("stream.nt", -1);
  std::printf("threads ok: lowered %ld failed %ld\n", lowered.load(), failed.load());
  return 0;
}

int main(int argc, char **argv) {
  if (argc < 2) return 11;
  if (argc > 2 && std::strcmp(argv[2], "threads") == 0) return threads(argv[1]);
  if (int rc = damaged_ir(argv[1])) return rc;
  return vector_storage();
}
