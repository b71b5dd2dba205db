// Elementwise skeleton: out[i] = produce(i) over the linear index space of the result.
// Serves Generate, Map, ZipWith, Transform, Backpermute, Replicate and Slice
// (Interpreter.hs:265-368, 627-634): the generated S::produce turns the linear index
// into a multi-dimensional one when the term needs it, applies the fused producer and
// the scalar function.  Each thread owns S::V consecutive results so that plain-array
// operands are moved with one 128-bit request per lane.

struct MapParams {
  i64 n;  // number of results
};

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_map(Spec::Env env, Spec::Out out, MapParams p) {
  typedef Spec S;
  const int V = S::V;
  i64 i0 = ((i64)blockIdx.x * ACC_BLOCK + threadIdx.x) * V;
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
}
