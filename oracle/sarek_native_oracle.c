/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of what the reference's Native
 * (OCaml-domains) backend computes for the tiled-GEMM, stream-triad and
 * block-256 tree-reduction kernels, and for the other bench kernels that
 * have a hand-written counterpart (vector add and copy, transposes, the
 * one-thread-per-element matmul, the histogram and the two kernels of a
 * radix-sort pass).  Nothing in the shipped library links,
 * loads or calls this file; only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may.
 *
 * Arithmetic rule restated here (reference citations, paths relative to the
 * upstream tree):
 *   - A `float32` kernel value on the Native backend is an OCaml `float`,
 *     i.e. an IEEE double: `+.` and `*.` are emitted for Float32 registers
 *     (sarek/ppx/Sarek_native_gen.ml:746-821) and shared arrays are plain
 *     OCaml `float array`s (sarek/ppx/Sarek_native_gen.ml:533-539,
 *     sarek/sarek/Sarek_cpu_runtime.ml:102-109).
 *   - Values are rounded to binary32 exactly once, when they are stored
 *     into a float32 vector (Bigarray store, sarek/core/Vector.ml:139-143).
 *   - Every output element is produced by one logical thread in a fixed
 *     order, so the result does not depend on the number of worker domains
 *     (sarek/sarek/Sarek_cpu_runtime.ml:686-782, 918-1002, 1042-1174).
 *
 * Parity pins (see tests/test_oracle.py): the reference's own deterministic
 * inputs and tolerances from benchmarks/bench_matrix_mul_tiled.ml:43-52,
 * 109-112,194; benchmarks/bench_stream_triad.ml:44-49,122;
 * benchmarks/bench_reduction.ml:110-111,154-163;
 * benchmarks/bench_dot_product.ml (inputs, 1e-3 rel); a literal
 * block/thread/superstep restatement of the tiled kernel checked against the
 * closed form; float64 library GEMM cross-checks; for the later kernels the
 * benches' own inputs, CPU loops and checks (benchmarks/bench_vector_add.ml,
 * bench_vector_copy.ml, bench_transpose.ml, bench_matrix_mul.ml,
 * bench_histogram.ml, bench_radix_sort.ml): sums of f32 pairs, identity and
 * transposition, numpy's bincount, a stable sort by digit.
 *
 * The bf16 / fp16-input GEMMs and the bias+ReLU+row-sum epilogue have NO
 * counterpart in the reference (it has no 16-bit vector kinds and no fused
 * epilogue); those functions extend the rule above and are
 * "parity unpinned by the reference": they are pinned only by library
 * cross-checks and by the definition written next to each function.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_MAX_THREADS 256

/* ------------------------------------------------------------------ */
/* Thread helper: static partition of [0,total) into contiguous ranges,
 * the same shape as the reference's ThreadPool (contiguous block ranges
 * per worker, sarek/sarek/Sarek_cpu_runtime.ml:918-1002).              */
typedef void (*range_fn)(int64_t lo, int64_t hi, void *ctx);
typedef struct {
  range_fn fn;
  int64_t lo, hi;
  void *ctx;
} range_job;

static void *range_tramp(void *p) {
  range_job *j = (range_job *)p;
  j->fn(j->lo, j->hi, j->ctx);
  return NULL;
}

static void parallel_ranges(int64_t total, int threads, range_fn fn, void *ctx) {
  if (threads < 1) threads = 1;
  if (threads > ORACLE_MAX_THREADS) threads = ORACLE_MAX_THREADS;
  if ((int64_t)threads > total) threads = (int)(total > 0 ? total : 1);
  if (threads == 1) {
    fn(0, total, ctx);
    return;
  }
  pthread_t tid[ORACLE_MAX_THREADS];
  range_job jobs[ORACLE_MAX_THREADS];
  int64_t chunk = (total + threads - 1) / threads;
  for (int t = 0; t < threads; ++t) {
    jobs[t].fn = fn;
    jobs[t].ctx = ctx;
    jobs[t].lo = (int64_t)t * chunk;
    jobs[t].hi = jobs[t].lo + chunk > total ? total : jobs[t].lo + chunk;
    if (jobs[t].lo > total) jobs[t].lo = total;
    pthread_create(&tid[t], NULL, range_tramp, &jobs[t]);
  }
  for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
}

/* ------------------------------------------------------------------ */
/* Seeded synthetic inputs (counter-based, so any index can be produced
 * independently): splitmix64 of (seed + index), top 24 bits -> [0,1).   */
static inline uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

typedef struct {
  float *out;
  uint64_t seed;
  float lo, hi;
} fill_ctx;

static void fill_uniform_range(int64_t lo, int64_t hi, void *p) {
  fill_ctx *c = (fill_ctx *)p;
  for (int64_t i = lo; i < hi; ++i) {
    uint64_t r = splitmix64(c->seed * 0x100000001B3ull + (uint64_t)i);
    float u = (float)(r >> 40) * (1.0f / 16777216.0f); /* exact, [0,1) */
    c->out[i] = c->lo + (c->hi - c->lo) * u;
  }
}

/* out[i] = lo + (hi-lo)*u_i, u_i in [0,1) on a 2^-24 grid. */
void oracle_fill_uniform_f32(float *out, int64_t n, uint64_t seed, float lo, float hi,
                             int threads) {
  fill_ctx c = {out, seed, lo, hi};
  parallel_ranges(n, threads, fill_uniform_range, &c);
}

/* ------------------------------------------------------------------ */
/* Round-to-nearest-even narrowing to bf16 / fp16, result held in f32.
 * No reference counterpart (parity unpinned by the reference).          */
float oracle_round_bf16(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if ((u & 0x7F800000u) == 0x7F800000u) { /* inf / nan: truncate, keep nan */
    if (u & 0x007FFFFFu) u |= 0x00400000u;
    u &= 0xFFFF0000u;
  } else {
    u += 0x7FFFu + ((u >> 16) & 1u);
    u &= 0xFFFF0000u;
  }
  memcpy(&x, &u, 4);
  return x;
}

uint16_t oracle_bf16_bits(float x) {
  float r = oracle_round_bf16(x);
  uint32_t u;
  memcpy(&u, &r, 4);
  return (uint16_t)(u >> 16);
}

/* binary32 -> binary16 bits, round to nearest even, with subnormals,
 * overflow to inf and nan kept quiet.                                    */
uint16_t oracle_f16_bits(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t absu = u & 0x7FFFFFFFu;
  if (absu >= 0x7F800000u) /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((absu > 0x7F800000u) ? 0x0200u : 0u));
  if (absu >= 0x477FF000u) /* rounds to >= 65520: overflow to inf */
    return (uint16_t)(sign | 0x7C00u);
  if (absu < 0x38800000u) { /* below 2^-14: subnormal half or zero */
    if (absu < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
    uint32_t e = absu >> 23;                     /* biased exponent, 102..112 */
    uint32_t man = (absu & 0x007FFFFFu) | 0x00800000u;
    uint32_t shift = 126u - e;                   /* 14..24 */
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1u);
    if (rem > halfway || (rem == halfway && (q & 1u))) q += 1u;
    return (uint16_t)(sign | q);
  }
  uint32_t v = absu - 0x38000000u; /* rebias exponent 127 -> 15 */
  uint32_t q = v >> 13;
  uint32_t rem = v & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q += 1u;
  return (uint16_t)(sign | q);
}

static float f16_bits_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu, man = h & 0x3FFu, u;
  if (e == 0) {
    float f = (float)man * (1.0f / 16777216.0f); /* man * 2^-24, exact */
    memcpy(&u, &f, 4);
    u |= sign;
  } else if (e == 31) {
    u = sign | 0x7F800000u | (man << 13);
  } else {
    u = sign | ((e + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

float oracle_round_f16(float x) { return f16_bits_to_f32(oracle_f16_bits(x)); }

void oracle_round_bf16_array(const float *in, float *out, uint16_t *bits, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    float r = oracle_round_bf16(in[i]);
    if (out) out[i] = r;
    if (bits) bits[i] = oracle_bf16_bits(in[i]);
  }
}

void oracle_round_f16_array(const float *in, float *out, uint16_t *bits, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    if (out) out[i] = oracle_round_f16(in[i]);
    if (bits) bits[i] = oracle_f16_bits(in[i]);
  }
}

/* ------------------------------------------------------------------ */
/* Stream triad: a[i] = b[i] + c[i]*s for i < n
 * (benchmarks/bench_stream_triad.ml:22-32).  b, c, s widen to double, the
 * product of two binary32 values is exact in double, one addition in
 * double, one rounding to binary32 at the store.                         */
typedef struct {
  float *a;
  const float *b, *c;
  double s;
} triad_ctx;

static void triad_range(int64_t lo, int64_t hi, void *p) {
  triad_ctx *t = (triad_ctx *)p;
  for (int64_t i = lo; i < hi; ++i)
    t->a[i] = (float)((double)t->b[i] + (double)t->c[i] * t->s);
}

void oracle_triad_f32(float *a, const float *b, const float *c, float s, int64_t n,
                      int threads) {
  triad_ctx t = {a, b, c, (double)s};
  parallel_ranges(n, threads, triad_range, &t);
}

/* ------------------------------------------------------------------ */
/* Block-256 tree sum (benchmarks/bench_reduction.ml:62-96): block j owns
 * gids [256j, 256j+256); sdata[tid] = in[gid] or 0 when gid >= n; eight
 * halving supersteps 128,64,...,1 with sdata held as doubles; the partial
 * is rounded to binary32 when stored to output[j].                       */
static float block256_tree(const double *vals) {
  double s[256];
  memcpy(s, vals, sizeof(s));
  for (int half = 128; half >= 1; half >>= 1)
    for (int t = 0; t < half; ++t) s[t] = s[t] + s[t + half];
  return (float)s[0];
}

typedef struct {
  const float *x, *y; /* y == NULL: plain sum; else elementwise product */
  float *partials;
  int64_t n;
} red_ctx;

static void reduce_blocks_range(int64_t lo, int64_t hi, void *p) {
  red_ctx *r = (red_ctx *)p;
  double v[256];
  for (int64_t blk = lo; blk < hi; ++blk) {
    for (int t = 0; t < 256; ++t) {
      int64_t g = blk * 256 + t;
      if (g < r->n)
        v[t] = r->y ? (double)r->x[g] * (double)r->y[g] : (double)r->x[g];
      else
        v[t] = 0.0;
    }
    r->partials[blk] = block256_tree(v);
  }
}

/* partials must hold ceil(n/256) floats. */
void oracle_reduce_sum_block256_f32(const float *in, int64_t n, float *partials,
                                    int threads) {
  red_ctx r = {in, NULL, partials, n};
  parallel_ranges((n + 255) / 256, threads, reduce_blocks_range, &r);
}

/* Fused map+reduce of benchmarks/bench_dot_product.ml:16-54:
 * sdata[tid] = a[gid]*b[gid] (exact in double), then the same tree.      */
void oracle_dot_block256_f32(const float *a, const float *b, int64_t n, float *partials,
                             int threads) {
  red_ctx r = {a, b, partials, n};
  parallel_ranges((n + 255) / 256, threads, reduce_blocks_range, &r);
}

/* Block-256 "take the greater" tree (benchmarks/bench_reduction_max.ml:18-100):
 * sdata[tid] = in[gid], or `pad` (-1000000.0 there) when gid >= n; for half =
 * 128..1, threads tid < half do  a = sdata[tid]; b = sdata[tid+half];
 * if b > a then sdata[tid] <- b;  output[block] = sdata[0].  Shared values are
 * doubles holding binary32 values, so the comparisons equal binary32 ones.  */
void oracle_reduce_max_block256_f32(const float *in, int64_t n, double pad, float *partials) {
  const int64_t nblocks = (n + 255) / 256;
  for (int64_t blk = 0; blk < nblocks; ++blk) {
    double s[256];
    for (int t = 0; t < 256; ++t) {
      const int64_t g = blk * 256 + t;
      s[t] = g < n ? (double)in[g] : pad;
    }
    for (int half = 128; half >= 1; half >>= 1)
      for (int t = 0; t < half; ++t) {
        const double a = s[t], b = s[t + half];
        if (b > a) s[t] = b;
      }
    partials[blk] = (float)s[0];
  }
}

/* Host fold of the partials, left to right in double
 * (benchmarks/bench_reduction.ml:154-160).                               */
double oracle_fold_partials_f64(const float *partials, int64_t count) {
  double s = 0.0;
  for (int64_t i = 0; i < count; ++i) s = s + (double)partials[i];
  return s;
}

/* "Fused triad + sum" as the Native backend can express it: the fused IR
 * has no native function (sarek/sarek/Sarek_fusion.ml:756,
 * sarek/plugins/native/Native_plugin.ml:325-330), so the oracle is the
 * unfused pair: triad stores binary32 a, then the block-256 reduction of a
 * and the double fold.  Returns the sum; a and partials are outputs.      */
double oracle_triad_sum_f32(float *a, const float *b, const float *c, float s, int64_t n,
                            float *partials, int threads) {
  oracle_triad_f32(a, b, c, s, n, threads);
  oracle_reduce_sum_block256_f32(a, n, partials, threads);
  return oracle_fold_partials_f64(partials, (n + 255) / 256);
}

/* ------------------------------------------------------------------ */
/* Tiled GEMM closed form (benchmarks/bench_matrix_mul_tiled.ml:55-95):
 * C[r*N+c] = binary32( sum_{k=0}^{K-1} (double)A[r*K+k]*(double)B[k*N+c] )
 * accumulated sequentially in increasing k starting from 0.0.  Zero padded
 * tile slots add exact zeros, so the tile decomposition does not change the
 * value.  Loop order here is r,k,c (vectorisable) which keeps each
 * element's k-order.                                                      */
typedef struct {
  const float *a, *b, *bias;
  float *c, *rowsum;
  const int32_t *rows; /* optional subset of rows */
  int64_t m, n, k;
  int relu_bias;
} gemm_ctx;

static void gemm_rows_range(int64_t lo, int64_t hi, void *p) {
  gemm_ctx *g = (gemm_ctx *)p;
  const int64_t N = g->n, K = g->k;
  double *acc = (double *)malloc(sizeof(double) * (size_t)N);
  for (int64_t i = lo; i < hi; ++i) {
    int64_t r = g->rows ? g->rows[i] : i;
    for (int64_t c = 0; c < N; ++c) acc[c] = 0.0;
    const float *arow = g->a + r * K;
    for (int64_t kk = 0; kk < K; ++kk) {
      const double av = (double)arow[kk];
      const float *brow = g->b + kk * N;
      for (int64_t c = 0; c < N; ++c) acc[c] = acc[c] + av * (double)brow[c];
    }
    float *crow = g->c + i * N; /* output row i of the (sub)matrix */
    if (!g->relu_bias) {
      for (int64_t c = 0; c < N; ++c) crow[c] = (float)acc[c];
    } else {
      /* Extension (no reference counterpart): y = relu(acc + bias) in
       * double, one rounding to binary32; row sum = left-to-right double
       * fold of the stored binary32 row, one rounding.                   */
      double rs = 0.0;
      for (int64_t c = 0; c < N; ++c) {
        double y = acc[c] + (double)g->bias[c];
        if (!(y > 0.0)) y = 0.0;
        crow[c] = (float)y;
        rs = rs + (double)crow[c];
      }
      if (g->rowsum) g->rowsum[i] = (float)rs;
    }
  }
  free(acc);
}

void oracle_gemm_f32(const float *a, const float *b, float *c, int64_t m, int64_t n,
                     int64_t k, int threads) {
  gemm_ctx g = {a, b, NULL, c, NULL, NULL, m, n, k, 0};
  parallel_ranges(m, threads, gemm_rows_range, &g);
}

/* Only the listed rows of C are produced: c_rows is [nrows x n].          */
void oracle_gemm_f32_rows(const float *a, const float *b, float *c_rows,
                          const int32_t *rows, int64_t nrows, int64_t n, int64_t k,
                          int threads) {
  gemm_ctx g = {a, b, NULL, c_rows, NULL, rows, nrows, n, k, 0};
  parallel_ranges(nrows, threads, gemm_rows_range, &g);
}

/* Y = relu(A.B + bias), rowsum[r] = sum_c Y[r,c]; rows == NULL: all rows.
 * Inputs are binary32 values (already rounded to fp16/bf16 by the caller
 * when the 16-bit path is being checked).                                 */
void oracle_gemm_bias_relu_rowsum(const float *a, const float *b, const float *bias,
                                  float *y_rows, float *rowsum, const int32_t *rows,
                                  int64_t nrows, int64_t n, int64_t k, int threads) {
  gemm_ctx g = {a, b, bias, y_rows, rowsum, rows, nrows, n, k, 1};
  parallel_ranges(nrows, threads, gemm_rows_range, &g);
}

/* Literal restatement of the kernel as the Native runtime executes it: one
 * logical thread per (ty,tx) of a 16x16 block, shared tiles of doubles,
 * three supersteps per K tile, guarded loads with zero fill, guarded store
 * (benchmarks/bench_matrix_mul_tiled.ml:62-95; BSP order
 * sarek/sarek/Sarek_cpu_runtime.ml:686-782).  O(MNK) scalar work: small
 * shapes only.  Exists to pin the closed form above.                      */
void oracle_matmul_tiled_bsp(const float *a, const float *b, float *c, int m, int n, int k) {
  const int ts = 16;
  const int gx = (n + ts - 1) / ts, gy = (m + ts - 1) / ts;
  const int num_tiles = (k + ts - 1) / ts;
  for (int by = 0; by < gy; ++by)
    for (int bx = 0; bx < gx; ++bx) {
      double tile_a[256], tile_b[256], sum[256];
      for (int i = 0; i < 256; ++i) sum[i] = 0.0;
      for (int t = 0; t <= num_tiles - 1; ++t) {
        for (int ty = 0; ty < ts; ++ty) /* superstep load_a */
          for (int tx = 0; tx < ts; ++tx) {
            int row = ty + ts * by, a_col = t * ts + tx;
            tile_a[ty * ts + tx] = (row < m && a_col < k) ? (double)a[row * k + a_col] : 0.0;
          }
        for (int ty = 0; ty < ts; ++ty) /* superstep load_b */
          for (int tx = 0; tx < ts; ++tx) {
            int col = tx + ts * bx, b_row = t * ts + ty;
            tile_b[ty * ts + tx] = (b_row < k && col < n) ? (double)b[b_row * n + col] : 0.0;
          }
        for (int ty = 0; ty < ts; ++ty) /* superstep compute */
          for (int tx = 0; tx < ts; ++tx)
            for (int i = 0; i <= ts - 1; ++i)
              sum[ty * ts + tx] = sum[ty * ts + tx] + tile_a[ty * ts + i] * tile_b[i * ts + tx];
      }
      for (int ty = 0; ty < ts; ++ty)
        for (int tx = 0; tx < ts; ++tx) {
          int row = ty + ts * by, col = tx + ts * bx;
          if (row < m && col < n) c[row * n + col] = (float)sum[ty * ts + tx];
        }
    }
}

/* ------------------------------------------------------------------ */
/* The reference's other memory-bound kernels, thread by thread as its 1-D
 * launches run them (one logical thread per global id, `if tid < n`):
 * vector add (benchmarks/bench_vector_add.ml:53-61; the sum of two binary32
 * values is formed in double and rounded once at the store, which is the
 * binary32 sum), vector copy (bench_vector_copy.ml:21-27), the transpose
 * (bench_transpose.ml: col = tid mod width, row = tid / width,
 * output[col*height + row] = input[row*width + col]; bench_transpose_tiled.ml
 * computes the same matrix through a 16x17 shared tile) and the
 * one-thread-per-element matmul (bench_matrix_mul.ml:55-73: row = tid / n,
 * col = tid mod n, sum in double in increasing i, one rounding at the store).
 * `threads` is the launch size (grid * block): ids at or past the guard do
 * nothing, so elements they would own keep their old value.             */
void oracle_vector_add_f32(const float *a, const float *b, float *c, int64_t n, int64_t threads) {
  for (int64_t tid = 0; tid < threads; ++tid)
    if (tid < n) c[tid] = (float)((double)a[tid] + (double)b[tid]);
}

void oracle_vector_copy_f32(const float *a, float *b, int64_t n, int64_t threads) {
  for (int64_t tid = 0; tid < threads; ++tid)
    if (tid < n) b[tid] = a[tid];
}

/* benchmarks/bench_histogram.ml:54-84, block by block: a 256-slot block histogram, the slots below
 * min(block, num_bins) cleared, one count per thread with gid < n, the same slots added to the global
 * histogram.  Int32.rem has the sign of the key (sarek/ppx/Sarek_native_gen.ml, Mod on int32); a key whose
 * slot is outside 0..255 would index the shared array out of bounds: it is skipped and counted in the
 * return value, so a test can insist on 0.  Slots never cleared start at `stale` (any value: they are
 * never merged, so it must not show).                                                                    */
int64_t oracle_histogram_i32(const int32_t *input, int32_t *histogram, int32_t n, int32_t num_bins,
                             int32_t block, int32_t grid, int32_t stale) {
  int64_t skipped = 0;
  for (int32_t b = 0; b < grid; ++b) {
    int32_t local_hist[256];
    for (int i = 0; i < 256; ++i) local_hist[i] = stale;
    for (int32_t tid = 0; tid < block; ++tid)
      if (tid < num_bins && tid < 256) local_hist[tid] = 0;
    for (int32_t tid = 0; tid < block; ++tid) {
      const int64_t gid = (int64_t)b * block + tid;
      if (gid < n) {
        const int32_t bin = input[gid] % num_bins;
        if (bin < 0 || bin > 255) ++skipped;
        else local_hist[bin] += 1;
      }
    }
    for (int32_t tid = 0; tid < block; ++tid)
      if (tid < num_bins && tid < 256) histogram[tid] = (int32_t)((uint32_t)histogram[tid] + (uint32_t)local_hist[tid]);
  }
  return skipped;
}

/* The counting kernel of benchmarks/bench_radix_sort.ml:82-116 the same way: digit =
 * (value lsr shift) land mask, logical shift as the Native backend computes it
 * (sarek/ppx/Sarek_native_gen.ml:809-815), 256 slots.                                                    */
int64_t oracle_radix_histogram_i32(const int32_t *input, int32_t *histogram, int32_t n, int32_t shift,
                                   int32_t mask, int32_t block, int32_t grid, int32_t stale) {
  int64_t skipped = 0;
  for (int32_t b = 0; b < grid; ++b) {
    int32_t local_hist[256];
    for (int i = 0; i < 256; ++i) local_hist[i] = stale;
    for (int32_t tid = 0; tid < block; ++tid)
      if (tid < 256) local_hist[tid] = 0;
    for (int32_t tid = 0; tid < block; ++tid) {
      const int64_t gid = (int64_t)b * block + tid;
      if (gid < n) {
        const int32_t digit = (int32_t)((uint32_t)input[gid] >> shift) & mask;
        if (digit < 0 || digit > 255) ++skipped;
        else local_hist[digit] += 1;
      }
    }
    for (int32_t tid = 0; tid < block; ++tid)
      if (tid < 256) histogram[tid] = (int32_t)((uint32_t)histogram[tid] + (uint32_t)local_hist[tid]);
  }
  return skipped;
}

/* The scatter kernel of benchmarks/bench_radix_sort.ml:120-137 with its threads run in gid order (the Native
 * backend runs them one after the other): pos = counters[digit]++, output[pos] = value.  The GPU kernel's
 * order inside a digit's range is not fixed, so a device result is compared with this one digit by digit as
 * multisets, and through the counters.  Returns the number of positions outside [0, out_len) (skipped).   */
int64_t oracle_radix_scatter_i32(const int32_t *input, int32_t *output, int64_t out_len, int32_t *counters,
                                 int32_t n, int32_t shift, int32_t mask, int64_t threads) {
  int64_t outside = 0;
  for (int64_t gid = 0; gid < threads; ++gid)
    if (gid < n) {
      const int32_t value = input[gid];
      const int32_t digit = (int32_t)((uint32_t)value >> shift) & mask;
      const int32_t pos = counters[digit];
      counters[digit] = (int32_t)((uint32_t)pos + 1u);
      if (pos < 0 || pos >= out_len) ++outside;
      else output[pos] = value;
    }
  return outside;
}

void oracle_transpose_f32(const float *input, float *output, int32_t width, int32_t height, int64_t threads) {
  const int32_t n = width * height;
  for (int64_t tid = 0; tid < threads; ++tid)
    if (tid < n) {
      const int32_t col = (int32_t)tid % width, row = (int32_t)tid / width;
      output[col * height + row] = input[row * width + col];
    }
}

void oracle_matmul_naive_f32(const float *a, const float *b, float *c, int32_t m, int32_t n, int32_t k,
                             int64_t threads) {
  for (int64_t tid = 0; tid < threads; ++tid) {
    const int32_t row = (int32_t)tid / n, col = (int32_t)tid % n;
    if (row < m && col < n) {
      double sum = 0.0;
      for (int32_t i = 0; i <= k - 1; ++i) sum = sum + (double)a[row * k + i] * (double)b[i * n + col];
      c[row * n + col] = (float)sum;
    }
  }
}

/* benchmarks/bench_stencil_2d.ml:43-58, thread by thread of a 2-D launch of threads_x x threads_y
 * threads: x and y are the global thread coordinates; for 0 < x < width - 1 and 0 < y < height - 1 the
 * five neighbours are read as doubles, added in the order up, down, left, right, center, divided by 5.0
 * and rounded once at the store (float32 vectors hold OCaml floats on the Native backend); every other
 * cell of `output` keeps what it holds.                                                                 */
void oracle_stencil_2d_f32(const float *input, float *output, int32_t width, int32_t height, int64_t threads_x,
                           int64_t threads_y) {
  for (int64_t ty = 0; ty < threads_y; ++ty)
    for (int64_t tx = 0; tx < threads_x; ++tx) {
      const int32_t x = (int32_t)tx, y = (int32_t)ty;
      if (x > 0 && x < width - 1 && y > 0 && y < height - 1) {
        const int32_t idx = y * width + x;
        const double up = input[(y - 1) * width + x];
        const double down = input[(y + 1) * width + x];
        const double left = input[y * width + x - 1];
        const double right = input[y * width + x + 1];
        const double center = input[idx];
        output[idx] = (float)((up + down + left + right + center) / 5.0);
      }
    }
}

/* benchmarks/bench_conv2d.ml:49-77, thread by thread of a 1-D launch: tid < width * height owns cell
 * x = tid mod width, y = tid / width; a border cell becomes 0, any other the nine cells round it added
 * p00 + p01 + ... + p22 (rows top to bottom, left to right) in double, divided by 9.0, rounded once.   */
void oracle_conv2d_f32(const float *input, float *output, int32_t width, int32_t height, int64_t threads) {
  const int32_t n = width * height;
  for (int64_t t = 0; t < threads; ++t) {
    const int32_t tid = (int32_t)t;
    if (tid < n) {
      const int32_t x = tid % width, y = tid / width;
      if (x == 0 || x == width - 1 || y == 0 || y == height - 1) {
        output[tid] = 0.0f;
      } else {
        const double p00 = input[(y - 1) * width + x - 1], p01 = input[(y - 1) * width + x];
        const double p02 = input[(y - 1) * width + x + 1];
        const double p10 = input[y * width + x - 1], p11 = input[y * width + x], p12 = input[y * width + x + 1];
        const double p20 = input[(y + 1) * width + x - 1], p21 = input[(y + 1) * width + x];
        const double p22 = input[(y + 1) * width + x + 1];
        const double sum = p00 + p01 + p02 + p10 + p11 + p12 + p20 + p21 + p22;
        output[tid] = (float)(sum / 9.0);
      }
    }
  }
}

int oracle_abi_version(void) { return 1; }
