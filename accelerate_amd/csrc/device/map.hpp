// Elementwise skeleton: out[i] = produce(i) over the linear index space of the result.
// Serves Generate, Map, ZipWith, Transform, Backpermute, Replicate and Slice
// (Interpreter.hs:265-368, 627-634): the generated S::produce turns the linear index
// into a multi-dimensional one when the term needs it, applies the fused producer and
// the scalar function.  Each thread owns S::V consecutive results so that plain-array
// operands are moved with one 128-bit request per lane.  A producer that defines
// ACC_MAP_INDEXED (stencils) takes the multi-dimensional index as well.

struct MapParams {
  i64 n;  // number of results
};

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_map(Spec::Env env, Spec::Out out, MapParams p) {
  typedef Spec S;
  const int V = S::V;
#ifdef ACC_MAP_XCD
  // producers that read neighbouring rows / planes (stencils): every XCD works on one
  // contiguous stretch of the result, so that what neighbouring workgroups share is found
  // in that XCD's L2
  const i64 b = acc_xcd_contiguous((i64)blockIdx.x, (i64)gridDim.x);
#else
  const i64 b = (i64)blockIdx.x;
#endif
  i64 i0 = (b * ACC_BLOCK + threadIdx.x) * V;
#ifdef ACC_MAP_INDEXED
  // the producer wants the multi-dimensional index: split the linear index once per thread
  // (the divisions), then step
  if (i0 >= p.n) return;
  i64 ix[S::kRank];
  S::from_index(env, i0, ix);
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
    for (int k = 0; k < V; ++k) r[k] = S::produce(env, i0 + k);
#pragma unroll
    for (int k = 0; k < V; ++k) S::store(out, i0 + k, r[k]);
  } else {
    for (int k = 0; k < V; ++k)
      if (i0 + k < p.n) S::store(out, i0 + k, S::produce(env, i0 + k));
  }
#endif
}
