// Permute skeleton (permuteOp, Interpreter.hs:585-624): the destination starts as a copy
// of the defaults; every source element whose target is `Just dst` is combined into
// out[dst] with f new old.  Sources are visited in parallel, so the result is defined for
// associative and commutative f only (AST.hs:420-423).
//
// S::target turns the linear source index into the linear destination index (0 for Nothing,
// 2 for an index outside the destination, which the skeleton drops and reports); S::update applies the combination with the cheapest mechanism the generated
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
  u32* err;    // host-visible word: 2 = a target outside the destination, 4 = a lock never came free
};

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_permute(Spec::Env env, Spec::Out out, PermuteParams p) {
  typedef Spec S;
  const i64 stride = (i64)gridDim.x * ACC_BLOCK;
  bool bad = false;
  for (i64 i = (i64)blockIdx.x * ACC_BLOCK + threadIdx.x; i < p.n; i += stride) {
    i64 j;
    const int t = S::target(env, i, j);
    if (t == 1) {
      S::Elt x = S::in_linear(env, i);
      S::update(env, out, j, x, p.locks, p.err);
    }
    bad = bad || t == 2;
  }
  if (bad) __hip_atomic_store(p.err, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

#ifdef ACC_PERMUTE_LDS
// Privatised variant for combination functions that are a single hardware atomic (+, min,
// max, and, or, xor on a 32/64-bit scalar) and destinations of at most a few LDS-fuls.
// Contended destinations (a histogram over skewed keys) serialise in the memory-side atomic
// units; here a workgroup first combines its share of the sources into a private copy of one
// destination range held in LDS (LDS atomics), then adds what it found to the real
// destination with one global atomic per touched element.
//
// Measured on 2^26 keys into 2^16 Int32 bins (two ranges): streaming the keys alone takes
// 45 us, the LDS atomics add 40 us whether the keys are uniform or Zipf-distributed, adding
// the private copies to the destination 12 us; sorted keys or a single key serialise in the
// LDS atomic unit (440 us).  Issuing the key loads of the next step before the LDS updates of
// the current one changed nothing (101 us against 100 us).
//
// Dealing the destination to the workgroups in blocks of 2^4 .. 2^10 elements instead of
// contiguous ranges (so that the popular elements of a skewed distribution do not all land in
// one range) changed nothing for Zipf keys and cost the uniform ones a third through the
// extra index arithmetic: the update loop is bound by its instructions.
//
// The destination is cut into `nparts` ranges of `part` elements (part <= S::kPart, the
// elements that fit 128 KiB of LDS; a tuple element has one private array per component).  The sources are cut into `groups` chunks; workgroup b serves chunk
// (b / (8 * nparts)) * 8 + b % 8 and range (b / 8) % nparts: workgroups are dealt to the 8
// XCDs round-robin, so the nparts workgroups that read the same chunk run on the same XCD
// and share its L2 -- the sources come from HBM once.
#define ACC_PERMUTE_LDS_BLOCK 1024
#ifndef ACC_PERMUTE_UNROLL
#define ACC_PERMUTE_UNROLL 4
#endif

struct PermuteLdsParams {
  i64 n;       // number of source elements
  i64 chunk;   // sources per chunk (multiple of 4)
  i64 nparts;  // destination ranges
  i64 part;    // elements per range
  i64 dst_n;   // destination elements
  u32* err;    // host-visible word: 2 = a target outside the destination, 4 = a lock never came free
};

extern "C" __global__ void __launch_bounds__(ACC_PERMUTE_LDS_BLOCK)
acc_permute_lds(Spec::Env env, Spec::Out out, PermuteLdsParams p) {
  typedef Spec S;
  __shared__ S::Priv priv;
  const i64 b = (i64)blockIdx.x;
  const i64 range = (b / 8) % p.nparts;
  const i64 chunkId = (b / (8 * p.nparts)) * 8 + (b % 8);
  const i64 lo = range * p.part;
  const i64 hi = lo + p.part < p.dst_n ? lo + p.part : p.dst_n;
  for (int i = threadIdx.x; i < (int)(hi - lo); i += ACC_PERMUTE_LDS_BLOCK) S::lds_init(priv, i);
  __syncthreads();
  const i64 begin = chunkId * p.chunk;
  const i64 end = begin + p.chunk < p.n ? begin + p.chunk : p.n;
  // ACC_PERMUTE_UNROLL groups of 4 consecutive sources per thread and step: all targets of
  // a step are computed (their loads issued) before the first update, which keeps enough
  // loads in flight for a single resident workgroup per CU to stream at HBM speed
  const i64 step = (i64)ACC_PERMUTE_LDS_BLOCK * 4 * ACC_PERMUTE_UNROLL;
  bool bad = false;  // a target outside the destination was met (reported once, at the end)
  for (i64 base = begin; base < end; base += step) {
    if (base + step <= end) {
      i64 j[ACC_PERMUTE_UNROLL][4];
      bool ok[ACC_PERMUTE_UNROLL][4];
#pragma unroll
      for (int g = 0; g < ACC_PERMUTE_UNROLL; ++g) {
        const i64 i0 = base + ((i64)g * ACC_PERMUTE_LDS_BLOCK + threadIdx.x) * 4;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int t = S::target(env, i0 + k, j[g][k]);
          ok[g][k] = t == 1;
          bad = bad || t == 2;
        }
      }
#pragma unroll
      for (int g = 0; g < ACC_PERMUTE_UNROLL; ++g) {
        const i64 i0 = base + ((i64)g * ACC_PERMUTE_LDS_BLOCK + threadIdx.x) * 4;
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (ok[g][k] && j[g][k] >= lo && j[g][k] < hi) S::lds_update(priv, (int)(j[g][k] - lo), S::in_linear(env, i0 + k));
      }
    } else {
      for (i64 i = base + threadIdx.x; i < end; i += ACC_PERMUTE_LDS_BLOCK) {
        i64 j;
        const int t = S::target(env, i, j);
        if (t == 1 && j >= lo && j < hi) S::lds_update(priv, (int)(j - lo), S::in_linear(env, i));
        bad = bad || t == 2;
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < (int)(hi - lo); i += ACC_PERMUTE_LDS_BLOCK) {
    S::lds_flush(priv, i, out, lo + i);  // components that still hold the identity are skipped
  }
  if (bad) __hip_atomic_store(p.err, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
#endif
