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
  // counting variant: where the workgroups leave their counters for acc_permute_count_reduce,
  // [nparts][groups][32768 + 16] words (null: every workgroup adds its counters to the destination itself);
  // combinations that need the lock: where they leave their private copies, [nparts][groups] of Spec::Priv
  u32* partials;
  i64 groups;  // source chunks
  // != 0: the destination holds nothing yet; its elements all start from one constant, which
  // acc_permute_count_reduce writes together with the counts (Spec::count_set), and nothing else
  // may touch it
  i64 fresh;
};

// (a combination that needs the lock also needs the environment, for the function, and the error word)
#ifdef ACC_PERMUTE_LDS_LOCKED
#define ACC_LDS_UPDATE(idx, x) S::lds_update(env, priv, idx, x, p.err)
#else
#define ACC_LDS_UPDATE(idx, x) S::lds_update(priv, idx, x)
#endif

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
          if (ok[g][k] && j[g][k] >= lo && j[g][k] < hi) ACC_LDS_UPDATE((int)(j[g][k] - lo), S::in_linear(env, i0 + k));
      }
    } else {
      for (i64 i = base + threadIdx.x; i < end; i += ACC_PERMUTE_LDS_BLOCK) {
        i64 j;
        const int t = S::target(env, i, j);
        if (t == 1 && j >= lo && j < hi) ACC_LDS_UPDATE((int)(j - lo), S::in_linear(env, i));
        bad = bad || t == 2;
      }
    }
  }
  __syncthreads();
#ifdef ACC_PERMUTE_LDS_LOCKED
  // the private copy goes to memory as it is; acc_permute_lds_merge combines the copies of a range
  S::Priv* mine = (S::Priv*)p.partials + (range * p.groups + chunkId);
  for (int i = threadIdx.x; i < (int)(hi - lo); i += ACC_PERMUTE_LDS_BLOCK) S::lds_spill(priv, i, mine);
#else
  for (int i = threadIdx.x; i < (int)(hi - lo); i += ACC_PERMUTE_LDS_BLOCK) {
    S::lds_flush(priv, i, out, lo + i);  // components that still hold the identity are skipped
  }
#endif
  if (bad) __hip_atomic_store(p.err, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

#ifdef ACC_PERMUTE_LDS_LOCKED
// Second launch for combinations that need the lock: a thread per destination element combines
// what the workgroups' private copies hold for it, then the element itself -- alone, so without
// the lock.  (Through the global locks instead, every workgroup asking for every element of a
// small destination at the same time, 2^24 pairs into 384 elements took 7 ms and into 4096 elements
// 20 ms, against 6.4 s and 0.54 s without private copies.)
extern "C" __global__ void __launch_bounds__(256)
acc_permute_lds_merge(Spec::Env env, Spec::Out out, PermuteLdsParams p) {
  typedef Spec S;
  const i64 perRange = (p.part + 255) / 256;
  const i64 range = (i64)blockIdx.x / perRange;
  const i64 i = ((i64)blockIdx.x - range * perRange) * 256 + threadIdx.x;
  const i64 j = range * p.part + i;
  if (i >= p.part || j >= p.dst_n) return;
  S::lds_merge(env, out, j, (const S::Priv*)p.partials + range * p.groups, p.groups, (int)i);
}
#endif
#endif

#ifdef ACC_PERMUTE_COUNT
// Counting variant: the combination is an integer sum and every source contributes the same
// constant, so a workgroup only has to count the sources per destination element -- in 16-bit
// counters, which lets one LDS-ful (128 KiB) cover 65536 destination elements whatever their
// width.  For the histogram of 2^16 bins one workgroup per source chunk then serves all bins:
// the keys are read once, and each key costs one LDS atomic instead of one in each of two
// workgroups.  Measured on 2^26 Zipf(1.1) keys into 2^16 Int32 bins: 59 us for this kernel and
// 6.5 us for the sum of the workgroups' counters, against 98 us for acc_permute_lds; streaming
// the keys through the same loop without touching LDS takes 50 us.  With a branch around every
// update (a lane whose source does not count, a counter that needs relief) the loads of the next
// step were waited for before the first update and the updates ran one by one: 110 us.
//
// Element e of the range lives in half (e >> 15) of word (e & 32767): neighbouring elements --
// the popular ones of a skewed distribution are neighbours -- fall into different words and banks.
// A counter must not run over into its neighbour: the update returns the word's old value, and
// the one lane that takes a counter from T - 1 to T (T = 32768) at once subtracts T again and adds
// T * constant to the destination.  Between two workgroup barriers the workgroup handles at most
// M = 32768 sources, so a counter below T at a barrier stays below T + M = 65536 until the next
// one, crosses T at most once in between, and is below M <= T again at that barrier, all
// corrections having landed by then.
#ifndef ACC_COUNT_UNROLL
#define ACC_COUNT_UNROLL 4
#endif
#ifndef ACC_COUNT_DEPTH
#define ACC_COUNT_DEPTH 2
#endif
#define ACC_COUNT_WORDS 32768
// words a workgroup leaves for acc_permute_count_reduce: its counters, then the list of the
// elements whose counter it relieved of ACC_COUNT_T (their number first, at most 15 of them)
#define ACC_COUNT_STRIDE (ACC_COUNT_WORDS + 16)
#define ACC_COUNT_T 32768u

// ONE: the destination is one range (range 0 starts at element 0 and covers all of it)
template <bool ONE>
ACC_DEV void acc_permute_count_body(const Spec::Env& env, const Spec::Out& out, const PermuteLdsParams& p, u32* cnt) {
  typedef Spec S;
  const i64 b = (i64)blockIdx.x;
  const i64 range = ONE ? 0 : (b / 8) % p.nparts;
  const i64 chunkId = ONE ? b : (b / (8 * p.nparts)) * 8 + (b % 8);
  const i64 lo = range * p.part;
  const i64 hi = lo + p.part < p.dst_n ? lo + p.part : p.dst_n;
  const u64 span = (u64)(hi - lo);  // <= 65536
  __shared__ u32 relieved[16];  // [0]: how many elements follow
  for (int i = threadIdx.x; i < (ACC_COUNT_WORDS + ACC_WAVE) / 4; i += ACC_PERMUTE_LDS_BLOCK)
    reinterpret_cast<uint4*>(cnt)[i] = make_uint4(0u, 0u, 0u, 0u);
  if (threadIdx.x < 16) relieved[threadIdx.x] = 0u;
  __syncthreads();
  const i64 begin = chunkId * p.chunk;
  const i64 end = begin + p.chunk < p.n ? begin + p.chunk : p.n;
  const u32 NONE = 0xffffffffu;
  const u32 spare = ACC_COUNT_WORDS + (u32)acc_lane();
  bool bad = false;
#ifdef ACC_PERMUTE_TARGET32
  // The index function widens an integer of at most 32 bits and the destination has fewer than
  // 2^31 elements (at most 128 ranges of 65536): everything per source stays in 32 bits, and one
  // comparison decides both "inside the destination" and "inside this range", because a target
  // outside either is at least span away from the range's first element.  A source that does not
  // count adds 0 to whatever word its number falls on.  (The 64-bit version below spends 17
  // vector instructions per source, this one 10: 23.8 M against 11.7 M wave instructions for 2^26
  // sources, 58 against 52 us.)  What is fetched is kept as it comes from the index function and
  // examined only when it is counted: a comparison at fetch time is a wait for the load.
  (void)spare;
  const u32 dstN = (u32)p.dst_n;
  auto locate = [&](i64 i, bool& tag) -> u32 {
    u32 j;
    tag = S::target32(env, i, j) != 0;
    return j;
  };
  auto bump = [&](u32 j, bool tag, u32& sh) -> bool {
    const u32 e = ONE ? j : j - (u32)lo;
    const bool valid = tag && e < (u32)span;
    bad = bad || (tag && (ONE ? e >= (u32)span : j >= dstN));
    sh = (e >> 11) & 16u;
    const u32 old = __hip_atomic_fetch_add(&cnt[e & (ACC_COUNT_WORDS - 1)], valid ? 1u << sh : 0u, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP);
    return valid && ((old >> sh) & 0xffffu) == ACC_COUNT_T - 1u;
  };
#define ACC_COUNT_ELEMENT(j) (ONE ? (j) : (j) - (u32)lo)
#else
  // the element of this range a source goes to, or NONE
  auto locate = [&](i64 i, bool& tag) -> u32 {
    i64 j;
    const int t = S::target(env, i, j);
    bad = bad || t == 2;
    tag = true;
    // t == 1 says 0 <= j < dst_n, which fits 32 bits (at most 128 ranges of 65536): a target below
    // this range wraps to something far beyond span
    const u32 e = (u32)j - (u32)lo;
    return t == 1 && e < (u32)span ? e : NONE;
  };
  // one more source for element e (or none, for NONE): returns whether this lane took the counter to T
  auto bump = [&](u32 e, bool, u32& sh) -> bool {
    const bool valid = e != NONE;
    sh = (e >> 11) & 16u;
    const u32 old = __hip_atomic_fetch_add(&cnt[valid ? (e & (ACC_COUNT_WORDS - 1)) : spare], valid ? 1u << sh : 0u,
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return ((old >> sh) & 0xffffu) == ACC_COUNT_T - 1u;  // (a spare word reads 0)
  };
#define ACC_COUNT_ELEMENT(e) (e)
#endif
  // A destination that holds nothing yet cannot take the relief: the element is noted in the
  // workgroup's list instead (a relief uses up ACC_COUNT_T of the workgroup's sources, and the host
  // gives a workgroup fewer than 15 * ACC_COUNT_T), for acc_permute_count_reduce to add.
  auto relieve = [&](u32 e, u32 sh) {
    (void)__hip_atomic_fetch_sub(&cnt[e & (ACC_COUNT_WORDS - 1)], ACC_COUNT_T << sh, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_WORKGROUP);
    if (p.fresh) {
      const u32 at = __hip_atomic_fetch_add(&relieved[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) + 1u;
      if (at < 16u) relieved[at] = e;
      else __hip_atomic_store(p.err, 5u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    } else {
      S::count_flush(out, lo + (i64)e, ACC_COUNT_T);
    }
  };
  // ACC_COUNT_UNROLL groups of 4 consecutive sources per thread and step.  The loop body is free
  // of branches up to the rare relief of a counter: the targets of the next step are computed
  // (their loads issued) in the same stretch of code as the updates of the current one, which do
  // not depend on them and are all issued before the first result is looked at.
  const i64 step = (i64)ACC_PERMUTE_LDS_BLOCK * 4 * ACC_COUNT_UNROLL;
  // steps between two barriers: as many as handle at most T sources (a power of two)
  constexpr int kSync = ACC_COUNT_T / (ACC_PERMUTE_LDS_BLOCK * 4 * ACC_COUNT_UNROLL);
  static_assert(kSync >= 1 && (kSync & (kSync - 1)) == 0, "a step must not handle more than T sources");
  struct Batch {
    u32 e[ACC_COUNT_UNROLL][4];
    bool tag[ACC_COUNT_UNROLL][4];
  };
  Batch batch[ACC_COUNT_DEPTH];
  auto fetch = [&](i64 base, Batch& b) {
#pragma unroll
    for (int g = 0; g < ACC_COUNT_UNROLL; ++g) {
      const i64 i0 = base + ((i64)g * ACC_PERMUTE_LDS_BLOCK + threadIdx.x) * 4;
#pragma unroll
      for (int k = 0; k < 4; ++k) b.e[g][k] = locate(i0 + k, b.tag[g][k]);
    }
  };
  auto countAll = [&](const Batch& b) {
    u32 sh[ACC_COUNT_UNROLL][4];
    bool hit[ACC_COUNT_UNROLL][4];
    bool any = false;
#pragma unroll
    for (int g = 0; g < ACC_COUNT_UNROLL; ++g)
#pragma unroll
      for (int k = 0; k < 4; ++k) hit[g][k] = bump(b.e[g][k], b.tag[g][k], sh[g][k]);
#pragma unroll
    for (int g = 0; g < ACC_COUNT_UNROLL; ++g)
#pragma unroll
      for (int k = 0; k < 4; ++k) any = any || hit[g][k];
    if (any) {
#pragma unroll
      for (int g = 0; g < ACC_COUNT_UNROLL; ++g)
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (hit[g][k]) relieve(ACC_COUNT_ELEMENT(b.e[g][k]), sh[g][k]);
    }
  };
  const i64 nsteps = end > begin ? (end - begin) / step : 0;  // whole steps of the chunk
  auto stepBase = [&](i64 s) { return begin + (s < nsteps ? s : nsteps - 1) * step; };
  if (nsteps > 0) {
#pragma unroll
    for (int d = 0; d < ACC_COUNT_DEPTH - 1; ++d) fetch(stepBase(d), batch[d]);
  }
  for (i64 s0 = 0; s0 < nsteps; s0 += ACC_COUNT_DEPTH) {
#pragma unroll
    for (int d = 0; d < ACC_COUNT_DEPTH; ++d) {
      const i64 s = s0 + d;
      if (s < nsteps) {  // (uniform: begin and end are the workgroup's)
        fetch(stepBase(s + ACC_COUNT_DEPTH - 1), batch[(d + ACC_COUNT_DEPTH - 1) % ACC_COUNT_DEPTH]);
        countAll(batch[d]);
        if ((s & (kSync - 1)) == kSync - 1) __syncthreads();
      }
    }
  }
  // what is left of the chunk: fewer sources than a step, an interval of its own
  __syncthreads();
  for (i64 i = begin + nsteps * step + threadIdx.x; i < end; i += ACC_PERMUTE_LDS_BLOCK) {
    u32 sh;
    bool tag;
    const u32 e = locate(i, tag);
    if (bump(e, tag, sh)) relieve(ACC_COUNT_ELEMENT(e), sh);
  }
  __syncthreads();
  if (p.partials) {
    // A global atomic per counter and workgroup is what this kernel would spend half its time on
    // (2^16 counters in each of 256 workgroups: 58 us against 52 us for the counting itself); the
    // counters are left in memory as they are, 128 KiB of coalesced stores per workgroup, and summed by
    // acc_permute_count_reduce.
    u32* mine = p.partials + ((u64)range * (u64)p.groups + (u64)chunkId) * ACC_COUNT_STRIDE;
    uint4* dst = reinterpret_cast<uint4*>(mine);
    for (int i = threadIdx.x; i < ACC_COUNT_WORDS / 4; i += ACC_PERMUTE_LDS_BLOCK) dst[i] = reinterpret_cast<const uint4*>(cnt)[i];
    if (threadIdx.x < 16) mine[ACC_COUNT_WORDS + threadIdx.x] = relieved[threadIdx.x];
  } else {
    for (int i = threadIdx.x; i < ACC_COUNT_WORDS; i += ACC_PERMUTE_LDS_BLOCK) {
      const u32 w = cnt[i];
      if (w & 0xffffu) S::count_flush(out, lo + i, w & 0xffffu);
      if (w >> 16) S::count_flush(out, lo + ACC_COUNT_WORDS + i, w >> 16);
    }
  }
  if (bad) __hip_atomic_store(p.err, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

extern "C" __global__ void __launch_bounds__(ACC_PERMUTE_LDS_BLOCK)
acc_permute_count(Spec::Env env, Spec::Out out, PermuteLdsParams p) {
  // the counters, and one spare word per lane: a source that does not count adds 0 to its lane's
  // spare word, so that the update needs no branch
  __shared__ __attribute__((aligned(16))) u32 cnt[ACC_COUNT_WORDS + ACC_WAVE];
  if (p.nparts == 1) acc_permute_count_body<true>(env, out, p, cnt);
  else acc_permute_count_body<false>(env, out, p, cnt);
}

// Sums the counters the workgroups of acc_permute_count left.  A workgroup takes 128 neighbouring
// words (256 counters) of one range: lane pairs (column of 4 words, one of 8 slices of the groups)
// sum their share, the slices are added through LDS, and every counter goes to the destination
// with one addition.  grid: nparts * 256 workgroups of 256 threads.
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_permute_count_reduce(Spec::Env env, Spec::Out out, PermuteLdsParams p) {
  typedef Spec S;
  __shared__ __attribute__((aligned(16))) u32 part[8 * 256];
  const int blocksPerPart = ACC_COUNT_WORDS / 128;
  const i64 b = (i64)blockIdx.x;
  const i64 range = b / blocksPerPart;
  const int wbase = (int)(b % blocksPerPart) * 128;
  const i64 lo = range * p.part;
  const int col = (int)threadIdx.x & 31, sl = (int)threadIdx.x >> 5;
  const u32* mine0 = p.partials + (u64)range * (u64)p.groups * ACC_COUNT_STRIDE;
  const uint4* src = reinterpret_cast<const uint4*>(mine0 + wbase + col * 4);
  u32 sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // low halves of the 4 words, then their high halves
  auto take = [&](const uint4& v) {
    const u32 w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      sum[k] += w[k] & 0xffffu;
      sum[4 + k] += w[k] >> 16;
    }
  };
  i64 g = sl;
  for (; g + 24 < p.groups; g += 32) {
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = src[(u64)(g + 8 * u) * (ACC_COUNT_STRIDE / 4)];
#pragma unroll
    for (int u = 0; u < 4; ++u) take(v[u]);
  }
  for (; g < p.groups; g += 8) take(src[(u64)g * (ACC_COUNT_STRIDE / 4)]);
  uint4* mine = reinterpret_cast<uint4*>(part + sl * 256 + col * 8);
  mine[0] = make_uint4(sum[0], sum[1], sum[2], sum[3]);
  mine[1] = make_uint4(sum[4], sum[5], sum[6], sum[7]);
  __syncthreads();
  u32 total = 0;
#pragma unroll
  for (int q = 0; q < 8; ++q) total += part[q * 256 + threadIdx.x];
  const int c2 = (int)threadIdx.x >> 3, v = (int)threadIdx.x & 7;
  const u32 e = (u32)((v >> 2) * ACC_COUNT_WORDS + wbase + c2 * 4 + (v & 3));  // this thread's element of the range
#ifdef ACC_PERMUTE_COUNT_SET
  if (p.fresh) {
    // what the workgroups relieved their counters of: a thread reads the list of one workgroup
    // (of every 256th) and adds, in LDS, for each of its entries that falls among this
    // workgroup's 256 elements
    __shared__ u32 extra[256];
    extra[threadIdx.x] = 0u;
    __syncthreads();
    for (i64 g = threadIdx.x; g < p.groups; g += ACC_BLOCK) {
      const uint4* l = reinterpret_cast<const uint4*>(mine0 + (u64)g * ACC_COUNT_STRIDE + ACC_COUNT_WORDS);
      uint4 q[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) q[i] = l[i];
      const u32 w[16] = {q[0].x, q[0].y, q[0].z, q[0].w, q[1].x, q[1].y, q[1].z, q[1].w,
                         q[2].x, q[2].y, q[2].z, q[2].w, q[3].x, q[3].y, q[3].z, q[3].w};
#pragma unroll
      for (int k = 1; k < 16; ++k) {
        const u32 rel = (w[k] & (ACC_COUNT_WORDS - 1)) - (u32)wbase;  // (an element's word, from this workgroup's first)
        if ((u32)k <= w[0] && rel < 128u)
          (void)__hip_atomic_fetch_add(&extra[(rel >> 2) * 8 + ((w[k] >> 15) << 2) + (rel & 3u)], ACC_COUNT_T, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
    __syncthreads();
    total += extra[threadIdx.x];
    const i64 j = lo + (i64)e;
    if ((i64)e < p.part && j < p.dst_n) S::count_set(out, j, total);
    return;
  }
#endif
  if (total) S::count_flush(out, lo + (i64)e, total);
}
#endif
