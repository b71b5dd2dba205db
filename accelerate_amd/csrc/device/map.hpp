// Elementwise skeleton: out[i] = produce(i) over the linear index space of the result.
// Serves Generate, Map, ZipWith, Transform, Backpermute, Replicate and Slice
// (Interpreter.hs:265-368, 627-634): the generated S::produce turns the linear index
// into a multi-dimensional one when the term needs it, applies the fused producer and
// the scalar function.  Each thread owns S::V consecutive results so that plain-array
// operands are moved with one 128-bit request per lane.  A producer that defines
// ACC_MAP_INDEXED (stencils) takes the multi-dimensional index as well.

struct MapParams {
  i64 n;     // number of results
  i64 base;  // workgroups of the launches that came before: index spaces of 2^32 threads
             // and more are covered by several launches
};

template <bool NT>
ACC_DEV void acc_map_body(const Spec::Env& env, const Spec::Out& out, const MapParams& p) {
  typedef Spec S;
  const int V = S::V;
#ifdef ACC_MAP_XCD
  // producers that read neighbouring rows / planes (stencils): every XCD works on one
  // contiguous stretch of the result, so that what neighbouring workgroups share is found
  // in that XCD's L2
  const i64 b = p.base + acc_xcd_contiguous((i64)blockIdx.x, (i64)gridDim.x);
#else
  const i64 b = p.base + (i64)blockIdx.x;
#endif
  i64 i0 = (b * ACC_BLOCK + threadIdx.x) * V;
#ifdef ACC_MAP_INDEXED
  // the producer wants the multi-dimensional index: split the linear index once per thread
  // (the divisions), then step
  if (i0 >= p.n) return;
  i64 ix[S::kRank];
  S::from_index(env, i0, ix);
#ifdef ACC_MAP_INTERIOR_RUN
  // all V results and their taps inside one row: no boundary tests, shared wide loads
  if (S::interior_run(env, ix)) {
    S::Elt r[S::V];
#pragma unroll
    for (int k = 0; k < V; ++k) r[k] = S::produce_in(env, i0 + k, ix, k);
#pragma unroll
    for (int k = 0; k < V; ++k) S::store(out, i0 + k, r[k]);
    return;
  }
#endif
  if (i0 + V <= p.n) {
    S::Elt r[S::V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
      r[k] = S::produce_at(env, i0 + k, ix);
      if (k + 1 < V) S::next_index(env, ix);
    }
#pragma unroll
    for (int k = 0; k < V; ++k) S::store(out, i0 + k, r[k]);
  } else {
    for (int k = 0; k < V && i0 + k < p.n; ++k) {
      S::store(out, i0 + k, S::produce_at(env, i0 + k, ix));
      S::next_index(env, ix);
    }
  }
#else
  if (i0 + V <= p.n) {
    S::Elt r[S::V];
#pragma unroll
    for (int k = 0; k < V; ++k) r[k] = S::produce<NT>(env, i0 + k);
#pragma unroll
    for (int k = 0; k < V; ++k) S::store<NT>(out, i0 + k, r[k]);
  } else {
    for (int k = 0; k < V; ++k)
      if (i0 + k < p.n) S::store(out, i0 + k, S::produce(env, i0 + k));
  }
#endif
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_map(Spec::Env env, Spec::Out out, MapParams p) {
  acc_map_body<false>(env, out, p);
}

#ifndef ACC_MAP_INDEXED
// the variant for launches that move far more than the last-level cache holds
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_map_stream(Spec::Env env, Spec::Out out, MapParams p) {
  acc_map_body<true>(env, out, p);
}
#endif

// The same over two-dimensional tiles of the result: a workgroup produces 32 rows x 8*V
// columns of the (outer dimensions flattened) x (innermost dimension) view, 8 lanes a row.
// For producers that permute indices (Backpermute, Transform): when the source is walked
// along another dimension than the result -- a transposition -- the 32 rows of a tile use
// whole cache lines of the source, where 256*V consecutive results would use four bytes of
// each line they touch.
struct MapTiledParams {
  i64 h, w;     // rows (outer extents multiplied) and columns (innermost extent)
  i64 tilesX;   // tiles per row of tiles
};

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_map_tiled(Spec::Env env, Spec::Out out, MapTiledParams p) {
  typedef Spec S;
  const int V = S::V;
  const i64 b = (i64)blockIdx.x;
  const i64 ty = b / p.tilesX, tx = b - ty * p.tilesX;
  const i64 row = ty * (ACC_BLOCK / 8) + threadIdx.x / 8;
  const i64 x0 = (tx * 8 + (threadIdx.x & 7)) * V;
  if (row >= p.h || x0 >= p.w) return;
  const i64 i0 = row * p.w + x0;
#ifdef ACC_MAP_INDEXED
  i64 ix[S::kRank];
  S::from_index(env, i0, ix);
  for (int k = 0; k < V && x0 + k < p.w; ++k) {
    S::store(out, i0 + k, S::produce_at(env, i0 + k, ix));
    S::next_index(env, ix);
  }
#else
  if (x0 + V <= p.w) {
    S::Elt r[S::V];
#pragma unroll
    for (int k = 0; k < V; ++k) r[k] = S::produce(env, i0 + k);
#pragma unroll
    for (int k = 0; k < V; ++k) S::store(out, i0 + k, r[k]);
  } else {
    for (int k = 0; k < V && x0 + k < p.w; ++k) S::store(out, i0 + k, S::produce(env, i0 + k));
  }
#endif
}

#ifdef ACC_MAP_XPOSE
// Index-permuting producers whose source runs along another dimension of the result than the
// innermost one -- transpositions of any rank: the result is seen as [o][a][m][w] (dimension a is
// the one the source's memory follows; o and m gather the dimensions around it), and a workgroup
// produces a 64 x 64 tile of the (a, w) plane: evaluated with the lanes along a, which walks
// the source contiguously, kept in LDS (rows 65 elements apart), written with the lanes along w.
// The choice of a is the host's guess from two evaluations of the index function and only
// decides the order of evaluation: every element is produced at its own index.
struct MapXposeParams {
  i64 na, nm, nw;   // extents of a, m, w
  i64 tilesA, tilesW;
  i64 axis;         // which dimension of the result a is
  i64 nt;           // the result leaves with the non-temporal hint
};

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_map_xpose(Spec::Env env, Spec::Out out, MapXposeParams p) {
  typedef Spec S;
  __shared__ S::Elt tile[64][65];
  i64 b = (i64)blockIdx.x;
  const i64 tw = b % p.tilesW;
  b /= p.tilesW;
  const i64 ta = b % p.tilesA;
  const i64 rest = b / p.tilesA;
  const i64 o = rest / p.nm, m = rest - o * p.nm;
  const i64 a0 = ta * 64, w0 = tw * 64;
  const int c = (int)threadIdx.x & 63, r0 = (int)threadIdx.x >> 6;
  auto linear = [&](i64 a, i64 w) { return ((o * p.na + a) * p.nm + m) * p.nw + w; };
  // the index of the tile's first element, split once; an element of the tile differs from it
  // in dimension a and in the innermost one only
  i64 ix0[S::kRank];
  S::from_index(env, linear(a0 < p.na ? a0 : 0, w0 < p.nw ? w0 : 0), ix0);
#pragma unroll 2
  for (int r = r0; r < 64; r += ACC_BLOCK / 64) {
    const i64 a = a0 + c, w = w0 + r;
    if (a < p.na && w < p.nw) {
      i64 ix[S::kRank];
#pragma unroll
      for (int d = 0; d < S::kRank; ++d) ix[d] = d == S::kRank - 1 ? w : (d == (int)p.axis ? a : ix0[d]);
      tile[r][c] = S::produce_at(env, linear(a, w), ix);
    }
  }
  __syncthreads();
  if (p.nt) {
#pragma unroll 2
    for (int r = r0; r < 64; r += ACC_BLOCK / 64) {
      const i64 a = a0 + r, w = w0 + c;
      if (a < p.na && w < p.nw) S::template store<true>(out, linear(a, w), tile[c][r]);
    }
  } else {
#pragma unroll 2
    for (int r = r0; r < 64; r += ACC_BLOCK / 64) {
      const i64 a = a0 + r, w = w0 + c;
      if (a < p.na && w < p.nw) S::store(out, linear(a, w), tile[c][r]);
    }
  }
}
#endif
