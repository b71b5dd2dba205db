// Permute skeleton (permuteOp, Interpreter.hs:585-624): the destination starts as a copy
// of the defaults; every source element whose target is `Just dst` is combined into
// out[dst] with f new old.  Sources are visited in parallel, so the result is defined for
// associative and commutative f only (AST.hs:420-423).
//
// S::target turns the linear source index into the linear destination index (false for
// Nothing); S::update applies the combination with the cheapest mechanism the generated
// code could prove correct for f and the element type:
//   store   f ignores the old value: plain store
//   atomic  f is +, min, max, and, or, xor on a 32/64-bit scalar: one hardware atomic
//   cas     any f on one 32/64-bit scalar: compare-and-swap loop on the bit pattern
//   lock    anything else (tuples, narrow scalars): per-destination spin lock
// The lock loop keeps the critical section inside the branch that won the lock, so lanes
// of one wave that contend for the same cell take turns instead of dead-locking.

struct PermuteParams {
  i64 n;       // number of source elements
  u32* locks;  // one word per destination element, zero when free (lock mode only)
};

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_permute(Spec::Env env, Spec::Out out, PermuteParams p) {
  typedef Spec S;
  const i64 stride = (i64)gridDim.x * ACC_BLOCK;
  for (i64 i = (i64)blockIdx.x * ACC_BLOCK + threadIdx.x; i < p.n; i += stride) {
    i64 j;
    if (S::target(env, i, j)) {
      S::Elt x = S::in_linear(env, i);
      S::update(env, out, j, x, p.locks);
    }
  }
}
