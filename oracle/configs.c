/* ORACLE -- test infrastructure, not product code.
 *
 * Sequential C restatement of the reference interpreter's loops for the five benchmark
 * configurations, for inputs too large for oracle/interp.py.  Only tests/,
 * __graft_entry__.smoke() and the cpu_baseline leg of bench.py may load this library.
 * Built by oracle/Makefile with -ffp-contract=off -fwrapv (no fused multiply-add, wrapping
 * integers: Haskell Int32/Int64 semantics).  Each function is pinned in
 * tests/test_oracle_golden.py against oracle/interp.py on random inputs and against the
 * reference's doctest vectors.  Paths below are relative to the reference's
 * src/Data/Array/Accelerate.
 */
#include <stdint.h>

/* fold (+) 0 (zipWith (*) xs ys): foldOp (Interpreter.hs:371-377) with Shape.iter's left
 * fold from the seed (Representation/Shape.hs:127-132); the product is the fused indexD. */
float oracle_dotp_f32(const float* xs, const float* ys, int64_t n) {
  float r = 0.0f;
  for (int64_t i = 0; i < n; ++i) r = r + xs[i] * ys[i];
  return r;
}

/* fold (+) z over the innermost dimension of a rows x n matrix (Interpreter.hs:371-377). */
void oracle_fold_sum_i32(const int32_t* in, int64_t rows, int64_t n, int32_t z, int32_t* out) {
  for (int64_t r = 0; r < rows; ++r) {
    int32_t acc = z;
    for (int64_t i = 0; i < n; ++i) acc = (int32_t)((uint32_t)acc + (uint32_t)in[r * n + i]);
    out[r] = acc;
  }
}

/* scanl1 (+): scanl1Op (Interpreter.hs:427-448): out[0] = in[0], out[i] = out[i-1] + in[i]. */
void oracle_scanl1_i64(const int64_t* in, int64_t n, int64_t* out) {
  for (int64_t i = 0; i < n; ++i)
    out[i] = i == 0 ? in[0] : (int64_t)((uint64_t)out[i - 1] + (uint64_t)in[i]);
}
void oracle_scanl1_f32(const float* in, int64_t n, float* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = i == 0 ? in[0] : out[i - 1] + in[i];
}

/* scanl (+) 0 on the segment lengths: scanlOp (Interpreter.hs:451-474), n+1 results. */
void oracle_scanl_i32(const int32_t* in, int64_t n, int32_t z, int32_t* out) {
  out[0] = z;
  for (int64_t i = 1; i <= n; ++i) out[i] = (int32_t)((uint32_t)out[i - 1] + (uint32_t)in[i - 1]);
}

/* foldSeg' (+) z vals offs: foldSegOp (Interpreter.hs:390-406): left fold of
 * vals[offs[s] .. offs[s+1]) from z; an empty segment gives z. */
void oracle_foldseg_i32(const int32_t* vals, const int32_t* offs, int64_t nseg, int32_t z, int32_t* out) {
  for (int64_t s = 0; s < nseg; ++s) {
    int32_t acc = z;
    for (int64_t i = offs[s]; i < offs[s + 1]; ++i) acc = (int32_t)((uint32_t)acc + (uint32_t)vals[i]);
    out[s] = acc;
  }
}

/* permute (+) zeros (\ix -> Just (keys!ix)) ones: permuteOp (Interpreter.hs:585-624):
 * defaults copied, then out[key] = 1 + out[key] in source order. */
void oracle_histogram_i32(const int32_t* keys, int64_t n, int32_t* bins, int64_t nbins) {
  for (int64_t b = 0; b < nbins; ++b) bins[b] = 0;
  for (int64_t i = 0; i < n; ++i) {
    int64_t k = keys[i];
    bins[k] = (int32_t)(1u + (uint32_t)bins[k]);
  }
}

/* One Jacobi sweep: stencilOp with a 3x3 pattern and Clamp (Interpreter.hs:637-649,
 * 797-839); f ((_,t,_),(l,_,r),(_,b,_)) = 0.25 * (((t + l) + r) + b). */
static inline int64_t clampi(int64_t i, int64_t n) { return i < 0 ? 0 : (i >= n ? n - 1 : i); }
void oracle_jacobi_f32(const float* in, float* out, int64_t h, int64_t w) {
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

/* iters sweeps, ping-pong between a and b; returns 0 if the result is in a, 1 if in b. */
int oracle_jacobi_iter_f32(float* a, float* b, int64_t h, int64_t w, int iters) {
  int where = 0;
  for (int k = 0; k < iters; ++k) {
    if (where == 0) oracle_jacobi_f32(a, b, h, w);
    else oracle_jacobi_f32(b, a, h, w);
    where ^= 1;
  }
  return where;
}
