/* ORACLE -- test infrastructure, not product code.
 *
 * OpenMP versions of the five configurations' loops: the "all host cores" CPU baseline that
 * bench.py reports beside the sequential restatement in configs.c (the reference's own
 * multicore backend, accelerate-llvm-native, is not part of the reference tree and cannot be
 * built here).  Integer results equal the sequential ones bit for bit (wrapping sums in any
 * order); Float32 sums associate differently and are compared within the benchmark's tolerance.
 * Only tests/ and the cpu_baseline leg of bench.py may load this library.
 */
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

int oracle_omp_threads(void) { return omp_get_max_threads(); }

float oracle_omp_dotp_f32(const float* xs, const float* ys, int64_t n) {
  float r = 0.0f;
#pragma omp parallel for reduction(+ : r) schedule(static)
  for (int64_t i = 0; i < n; ++i) r += xs[i] * ys[i];
  return r;
}

/* inclusive scan in three phases: a running sum per contiguous chunk, an exclusive scan of the
 * chunk totals, the carry added to every chunk but the first */
#define OMP_SCAN(NAME, T, ADD)                                                        \
  void NAME(const T* in, int64_t n, T* out) {                                        \
    int nt = omp_get_max_threads();                                                   \
    T* tot = (T*)calloc((size_t)nt + 1, sizeof(T));                                   \
    _Pragma("omp parallel num_threads(nt)") {                                        \
      int t = omp_get_thread_num();                                                   \
      int64_t lo = n * t / nt, hi = n * (t + 1) / nt;                                 \
      T acc = 0;                                                                      \
      for (int64_t i = lo; i < hi; ++i) {                                             \
        acc = ADD(acc, in[i]);                                                        \
        out[i] = acc;                                                                 \
      }                                                                               \
      tot[t + 1] = acc;                                                               \
      _Pragma("omp barrier")                                                         \
      _Pragma("omp single") {                                                        \
        for (int k = 1; k <= nt; ++k) tot[k] = ADD(tot[k - 1], tot[k]);               \
      }                                                                               \
      T carry = tot[t];                                                               \
      if (t > 0)                                                                      \
        for (int64_t i = lo; i < hi; ++i) out[i] = ADD(carry, out[i]);                \
    }                                                                                 \
    free(tot);                                                                        \
  }
#define ADD_I64(a, b) ((int64_t)((uint64_t)(a) + (uint64_t)(b)))
#define ADD_F32(a, b) ((a) + (b))
OMP_SCAN(oracle_omp_scanl1_i64, int64_t, ADD_I64)
OMP_SCAN(oracle_omp_scanl1_f32, float, ADD_F32)

void oracle_omp_foldseg_i32(const int32_t* vals, const int32_t* offs, int64_t nseg, int32_t z, int32_t* out) {
#pragma omp parallel for schedule(dynamic, 1024)
  for (int64_t s = 0; s < nseg; ++s) {
    uint32_t acc = (uint32_t)z;
    for (int64_t i = offs[s]; i < offs[s + 1]; ++i) acc += (uint32_t)vals[i];
    out[s] = (int32_t)acc;
  }
}

void oracle_omp_histogram_i32(const int32_t* keys, int64_t n, int32_t* bins, int64_t nbins) {
  int nt = omp_get_max_threads();
  uint32_t* priv = (uint32_t*)calloc((size_t)nt * (size_t)nbins, sizeof(uint32_t));
#pragma omp parallel num_threads(nt)
  {
    uint32_t* mine = priv + (size_t)omp_get_thread_num() * (size_t)nbins;
#pragma omp for schedule(static)
    for (int64_t i = 0; i < n; ++i) mine[keys[i]] += 1u;
#pragma omp for schedule(static)
    for (int64_t b = 0; b < nbins; ++b) {
      uint32_t acc = 0;
      for (int t = 0; t < nt; ++t) acc += priv[(size_t)t * (size_t)nbins + (size_t)b];
      bins[b] = (int32_t)acc;
    }
  }
  free(priv);
}

static inline int64_t clampi(int64_t i, int64_t n) { return i < 0 ? 0 : (i >= n ? n - 1 : i); }
static void sweep(const float* in, float* out, int64_t h, int64_t w) {
#pragma omp parallel for schedule(static)
  for (int64_t y = 0; y < h; ++y) {
    const float* up = in + clampi(y - 1, h) * w;
    const float* mid = in + y * w;
    const float* dn = in + clampi(y + 1, h) * w;
    for (int64_t x = 0; x < w; ++x) {
      float t = up[x], l = mid[clampi(x - 1, w)], r = mid[clampi(x + 1, w)], b = dn[x];
      out[y * w + x] = 0.25f * (((t + l) + r) + b);
    }
  }
}
int oracle_omp_jacobi_iter_f32(float* a, float* b, int64_t h, int64_t w, int iters) {
  int where = 0;
  for (int k = 0; k < iters; ++k) {
    if (where == 0) sweep(a, b, h, w);
    else sweep(b, a, h, w);
    where ^= 1;
  }
  return where;
}
