// Fold / Fold1 skeleton: reduction of the innermost dimension, one result per outer row.
// Reference semantics: foldOp / fold1Op (Interpreter.hs:371-387) with Shape.iter's left
// fold seeded once by z (Representation/Shape.hs:127-132).
//
// A row is cut into `bpr` contiguous chunks, one per workgroup; a chunk is cut into one
// contiguous span per wave.  Each lane reads S::V consecutive elements per step (one
// 128-bit request when the source is a plain array) so that a wave's step is one fully
// coalesced tile of 64*V elements.
//   commutative operator: lanes keep private accumulators over all their tiles and one
//     wave reduction runs at the end;
//   otherwise: every tile is reduced in lane order and chained onto a carry in lane 0,
//     which keeps operands strictly left to right (associativity only).
// Wave results meet in LDS and are combined in wave order.  With bpr > 1 the chunk
// results go to `tmp` (rows x bpr) and acc_fold_final reduces them, again in order, and
// applies the seed exactly once on the left.
// A fold of a single row needs no second launch: every workgroup publishes its chunk's result
// as self-validating words (acc_publish of scan.hpp: value and the launch's tag in one relaxed
// 64-bit store, no fence); the workgroup of the row's last chunk, which the hardware starts last,
// then reads the others' words -- valid exactly when they carry this launch's tag, polled under
// the same bounded wait as the scans' look-back -- and reduces them in order.  It waits for
// nobody who needs its place: a fold launches at most `fold_target` workgroups.  (Measured and
// rejected: a counter of finished workgroups, whose last increment elects the reducer -- 2048
// atomics on one address cost more than the launch they save, dotp over 2^24 elements 23 -> 40
// us; and before that a release / acquire pair around such a count: the fences write back and
// invalidate the XCD's whole L2 under the streaming workgroups, 2^28 elements 0.37 -> 0.44 ms.)

#ifndef ACC_FOLD_ROWS
#define ACC_FOLD_ROWS 1  // 0: commutative operators read a contiguous span per wave too
#endif

struct FoldParams {
  i64 rows;   // number of outer rows
  i64 n;      // extent of the innermost dimension
  i64 bpr;    // workgroups per row
  i64 chunk;  // elements per workgroup (multiple of ACC_WAVES * 64 * V)
  i64 first;  // number of the launch's first workgroup: more workgroups than a launch holds take several
  // one launch for a single row (null desc: chunk results go to tmp for acc_fold_final)
  u64* desc;        // bpr descriptors of AccWords<Elt>::N words
  u64 epoch;        // tag of this launch
  u64 spin_limit;   // polls after which the last workgroup stops waiting for a chunk's words
  u32* err;         // host-visible word: 3 = it gave up
};

// tiles the ordered fold turns over in LDS at a time: 128 bytes of elements per lane, none for
// elements so large that the staging area of a workgroup would pass 40 KiB
#ifndef ACC_FOLD_STAGE_BYTES
#define ACC_FOLD_STAGE_BYTES 128
#endif
template <class S> struct AccFoldStage {
  enum { kRun = S::V * (int)sizeof(typename S::Elt),
         K = S::kCommutative || kRun > 64 ? 1 : ACC_FOLD_STAGE_BYTES / kRun };
};

template <class S, class Src, bool STAGE = false>
ACC_DEV bool acc_fold_span(const typename S::Env& env, const Src& src, i64 off, i64 lo, i64 hi,
                           typename S::Elt& result) {
  typedef typename S::Elt Elt;
  const int V = S::V;
  const i64 T = (i64)ACC_WAVE * V;
  const int lane = acc_lane();
  Elt acc;
  bool have = false;
  if (S::kCommutative) {
    i64 base = lo;
    bool full = false;
    if (base + T <= hi) {
      i64 p = off + base + (i64)lane * V;
      acc = src(p);
#pragma unroll
      for (int k = 1; k < V; ++k) acc = S::combine(env, acc, src(p + k));
      base += T;
      full = true;
#pragma unroll 4
      for (; base + T <= hi; base += T) {
        i64 q = off + base + (i64)lane * V;
        Elt x[S::V];
#pragma unroll
        for (int k = 0; k < V; ++k) x[k] = src(q + k);
#pragma unroll
        for (int k = 0; k < V; ++k) acc = S::combine(env, acc, x[k]);
      }
    }
    have = full;
    i64 p0 = base + (i64)lane * V;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (p0 + k < hi) {
        Elt x = src(off + p0 + k);
        acc = have ? S::combine(env, acc, x) : x;
        have = true;
      }
    }
    i64 cnt = hi - base;
    int nvalid = full ? ACC_WAVE : (cnt <= 0 ? 0 : (int)((cnt + V - 1) / V));
    acc = acc_wave_reduce<S>(env, acc, lane, nvalid);
    result = acc;
    return nvalid > 0;
  } else {
    Elt carry;
    i64 base = lo;
    // Blocks of K tiles, for as long as they last: the wave loads them tile by tile (one load
    // instruction covers consecutive memory, K of them in flight per lane) and turns them over in
    // LDS, so that a lane gets K * V consecutive elements to combine in order, and the wave joins
    // its lanes once per block instead of once per tile -- the join is what a tile costs (a single
    // row of 2^27 Int64 under "the last value that is not zero": 3.1 TB/s tile by tile).  A lane's
    // stretch is padded by one element, which keeps its reads off the banks of its neighbours'.
    // (the staging area costs occupancy, so only the kernels launched for long chunks have it)
    constexpr int K = STAGE && Src::kBulk ? AccFoldStage<S>::K : 1;
    if constexpr (K > 1) {
      constexpr int R = K * V;  // elements a lane combines per block
      __shared__ Elt sh_stage[ACC_WAVES][ACC_WAVE * (R + 1)];
      Elt* st = sh_stage[acc_wave()];
      for (; base + K * T <= hi; base += K * T) {
        const i64 q = off + base + (i64)lane * V;
        Elt x[K][S::V];
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int v = 0; v < V; ++v) x[k][v] = src(q + (i64)k * T + v);
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int v = 0; v < V; ++v) {
            const int e = k * (int)T + lane * V + v;
            st[e + e / R] = x[k][v];
          }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        Elt t = st[lane * (R + 1)];
#pragma unroll
        for (int j = 1; j < R; ++j) t = S::combine(env, t, st[lane * (R + 1) + j]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        t = acc_wave_reduce<S>(env, t, lane, ACC_WAVE);
        carry = have ? S::combine(env, carry, t) : t;
        have = true;
      }
    }
    // full tiles: V unconditional loads per lane (one wide request), all lanes take part
    for (; base + T <= hi; base += T) {
      const i64 q = off + base + (i64)lane * V;
      Elt x[S::V];
#pragma unroll
      for (int k = 0; k < V; ++k) x[k] = src(q + k);
      Elt t = x[0];
#pragma unroll
      for (int k = 1; k < V; ++k) t = S::combine(env, t, x[k]);
      t = acc_wave_reduce<S>(env, t, lane, ACC_WAVE);
      carry = have ? S::combine(env, carry, t) : t;
      have = true;
    }
    for (; base < hi; base += T) {
      i64 cnt = hi - base < T ? hi - base : T;
      int nl = (int)((cnt + V - 1) / V);
      i64 p0 = base + (i64)lane * V;
      Elt t;
      if (p0 < hi) {
        t = src(off + p0);
#pragma unroll
        for (int k = 1; k < V; ++k)
          if (p0 + k < hi) t = S::combine(env, t, src(off + p0 + k));
      }
      t = acc_wave_reduce<S>(env, t, lane, nl);
      carry = have ? S::combine(env, carry, t) : t;
      have = true;
    }
    result = carry;
    return have;
  }
}

// The wave's share of [lo, hi) for a commutative operator, where the order of the operands is
// free: the workgroup goes over the chunk row by row, a row being ACC_BLOCK lanes x V elements,
// so that one load instruction of the workgroup covers 4 KiB of consecutive addresses.  (Two
// Float32 arrays of 2^28 elements read this way by a bare kernel: 7.0 TB/s for any number of
// workgroups from 1024 to 16384; with a contiguous span per wave, as below for the other
// operators, 6.0 to 6.7 depending on how the spans fall onto the memory channels.)
template <class S, class Src>
ACC_DEV bool acc_fold_rows_of_block(const typename S::Env& env, const Src& src, i64 off, i64 lo, i64 hi,
                                    typename S::Elt& result) {
  typedef typename S::Elt Elt;
  const int V = S::V;
  const i64 T = (i64)ACC_BLOCK * V;
  const int lane = acc_lane();
  Elt acc;
  i64 base = lo;
  bool full = false;
  if (base + T <= hi) {
    const i64 p = off + base + (i64)threadIdx.x * V;
    acc = src(p);
#pragma unroll
    for (int k = 1; k < V; ++k) acc = S::combine(env, acc, src(p + k));
    base += T;
    full = true;
#pragma unroll 4
    for (; base + T <= hi; base += T) {
      const i64 q = off + base + (i64)threadIdx.x * V;
      Elt x[S::V];
#pragma unroll
      for (int k = 0; k < V; ++k) x[k] = src(q + k);
#pragma unroll
      for (int k = 0; k < V; ++k) acc = S::combine(env, acc, x[k]);
    }
  }
  bool have = full;
  const i64 p0 = base + (i64)threadIdx.x * V;
#pragma unroll
  for (int k = 0; k < V; ++k) {
    if (p0 + k < hi) {
      Elt x = src(off + p0 + k);
      acc = have ? S::combine(env, acc, x) : x;
      have = true;
    }
  }
  // lanes that hold something come first in the workgroup
  const i64 cnt = hi - base;
  i64 holders = full ? (i64)ACC_BLOCK : (cnt <= 0 ? 0 : (cnt + V - 1) / V);
  holders -= (i64)acc_wave() * ACC_WAVE;
  const int nvalid = holders <= 0 ? 0 : (holders > ACC_WAVE ? ACC_WAVE : (int)holders);
  acc = acc_wave_reduce<S>(env, acc, lane, nvalid);
  result = acc;
  return nvalid > 0;
}

// Reduce [lo, hi) of one row with the whole workgroup; the result is valid in thread 0.
template <class S, class Src, bool STAGE = false>
ACC_DEV bool acc_fold_block(const typename S::Env& env, const Src& src, i64 off, i64 lo, i64 hi,
                            typename S::Elt& result) {
  typedef typename S::Elt Elt;
  __shared__ Elt sh_v[ACC_WAVES];
  __shared__ int sh_ok[ACC_WAVES];
  const i64 T = (i64)ACC_WAVE * S::V;
  i64 span = hi - lo;
  i64 wlen = (span + ACC_WAVES - 1) / ACC_WAVES;
  wlen = (wlen + T - 1) / T * T;
  const int w = acc_wave();
  i64 wlo = lo + (i64)w * wlen;
  i64 whi = wlo + wlen < hi ? wlo + wlen : hi;
  Elt r;
  bool ok;
  if constexpr (S::kCommutative && ACC_FOLD_ROWS) ok = acc_fold_rows_of_block<S>(env, src, off, lo, hi, r);
  else ok = acc_fold_span<S, Src, STAGE>(env, src, off, wlo, whi, r);
  if (acc_lane() == 0) {
    sh_v[w] = r;
    sh_ok[w] = ok ? 1 : 0;
  }
  __syncthreads();
  bool have = false;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 0; k < ACC_WAVES; ++k) {
      if (sh_ok[k]) {
        result = have ? S::combine(env, result, sh_v[k]) : sh_v[k];
        have = true;
      }
    }
  }
  return have;
}

template <class S, bool NT = false> struct AccFoldSrcIn {
  static constexpr bool kBulk = true;  // the operand itself: worth staging blocks of it in LDS
  const typename S::Env& env;
  __device__ __forceinline__ typename S::Elt operator()(i64 i) const { return S::template in_linear<NT>(env, i); }
};
template <class S> struct AccFoldSrcTmp {
  static constexpr bool kBulk = false;
  const typename S::Out& tmp;
  __device__ __forceinline__ typename S::Elt operator()(i64 i) const { return S::load(tmp, i); }
};

// chunk results published by the workgroups of this launch: waits (bounded) until the words carry the launch's tag
template <class S> struct AccFoldSrcDesc {
  static constexpr bool kBulk = false;
  const u64* desc;
  u64 epoch, limit;
  u32* err;
  __device__ __forceinline__ typename S::Elt operator()(i64 i) const {
    typename S::Elt v;
    u64 polls = 0;
    while (acc_try_read<typename S::Elt>(desc + i * AccWords<typename S::Elt>::N, v, epoch) == 0) {
      if (++polls >= limit) {
        __hip_atomic_store(err, 3u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    return v;
  }
};

template <class S>
ACC_DEV void acc_fold_finish(const typename S::Env& env, const typename S::Out& out, i64 row, bool have,
                             const typename S::Elt& r) {
  if (threadIdx.x != 0) return;
  if (S::kSeeded) {
    typename S::Elt z = S::seed(env);
    S::store(out, row, have ? S::combine(env, z, r) : z);
  } else if (have) {
    S::store(out, row, r);
  }
}

template <bool NT, bool STAGE = false>
ACC_DEV void acc_fold_main_body(const Spec::Env& env, const Spec::Out& out, const Spec::Out& tmp, const FoldParams& p) {
  typedef Spec S;
  i64 bid = p.first + (i64)blockIdx.x;
  i64 row = bid / p.bpr;
  i64 b = bid - row * p.bpr;
  i64 lo = b * p.chunk;
  i64 hi = lo + p.chunk < p.n ? lo + p.chunk : p.n;
  AccFoldSrcIn<S, NT> src{env};
  S::Elt r;
  bool have = acc_fold_block<S, AccFoldSrcIn<S, NT>, STAGE>(env, src, row * p.n, lo, hi, r);
  if (p.bpr == 1) {
    acc_fold_finish<S>(env, out, row, have, r);
  } else if (p.desc) {
    // a single row, one launch (every chunk holds elements: `have` is true in thread 0)
    const int W = AccWords<S::Elt>::N;
    if (threadIdx.x == 0) acc_publish<S::Elt>(p.desc + b * W, r, p.epoch, 1);
    if (b == p.bpr - 1) {
      __syncthreads();  // (the reduction below reuses the LDS of the one above)
      AccFoldSrcDesc<S> parts{p.desc, p.epoch, p.spin_limit, p.err};
      S::Elt t;
      const bool any = acc_fold_block<S>(env, parts, 0, 0, p.bpr, t);
      acc_fold_finish<S>(env, out, row, any, t);
    }
  } else if (threadIdx.x == 0 && have) {
    S::store(tmp, bid, r);
  }
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_fold_main(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldParams p) {
  acc_fold_main_body<false>(env, out, tmp, p);
}

// the variant for sources far larger than the last-level cache: reads at the row's own
// linear index are marked non-temporal
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_fold_main_stream(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldParams p) {
  acc_fold_main_body<true>(env, out, tmp, p);
}

// the same for operators that are not commutative and chunks of 64 KiB and more: blocks of tiles
// turned over in LDS (acc_fold_span)
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_fold_main_staged(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldParams p) {
  acc_fold_main_body<false, (AccFoldStage<Spec>::K > 1)>(env, out, tmp, p);
}
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_fold_main_staged_stream(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldParams p) {
  acc_fold_main_body<true, (AccFoldStage<Spec>::K > 1)>(env, out, tmp, p);
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_fold_final(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldParams p) {
  typedef Spec S;
  i64 row = (i64)blockIdx.x;
  AccFoldSrcTmp<S> src{tmp};
  S::Elt r;
  bool have = acc_fold_block<S>(env, src, row * p.bpr, 0, p.bpr, r);
  acc_fold_finish<S>(env, out, row, have, r);
}

// Rows of at most half a tile of the scan machinery: a workgroup reduces rpt whole rows at
// once as a scan of (head flag, value) pairs over the row-major stream (acc_rows_tile); the
// lane that holds the last element of a row writes the row's result.  One workgroup per row
// would leave all but a few lanes idle.
struct FoldRowsParams {
  i64 rows;
  i64 n;    // 1 <= n, rpt * n <= TILE
  i64 rpt;  // rows per workgroup
};

extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK)
acc_fold_rows(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldRowsParams p) {
  typedef Spec S;
  typedef S::Elt Elt;
  const i64 row0 = (i64)blockIdx.x * p.rpt;
  const i64 nrows = p.rows - row0 < p.rpt ? p.rows - row0 : p.rpt;
  const int n = (int)p.n;
  auto load = [&](int idx, int r, int t) -> Elt {
    Elt v = S::in_linear(env, row0 * p.n + idx);
    if (S::kSeeded && t == 0) v = S::combine(env, S::seed(env), v);
    return v;
  };
  auto store = [&](int idx, int r, int t, const Elt& y) {
    if (t == n - 1) S::store(out, row0 + r, y);
  };
  acc_rows_tile<S>(env, (int)(nrows * p.n), n, load, store);
}

// Many rows of up to a few thousand elements under a commutative operator: a row belongs to
// `lanes` neighbouring lanes of a wave (a power of two: as many as the row has runs of V
// elements, 64 at most), a wave works on 64 / lanes rows at a time and a workgroup on `rpg`
// rows in all.  A lane adds up its runs (run c of the row goes to lane c mod lanes, so one load
// instruction of the wave covers consecutive memory, rows following each other as they do in
// memory), the lanes of a row combine through shuffles, the first one writes.  No LDS, no
// barrier.  (2^28 Float32 as rows of 4 ... 2048 elements: 3.6 - 5.4 TB/s through acc_fold_rows
// and acc_fold_main, whose tiles such rows do not fill.)
struct FoldWaveRowsParams {
  i64 rows;
  i64 n;      // elements per row, >= 1
  i64 lanes;  // lanes per row: 1, 2, 4, .. 64
  i64 rpg;    // rows per workgroup, a multiple of ACC_WAVES * (64 / lanes)
};

// a lane's value on its way through the wave: bit 0 of f marks the first lane of a row, bit 1 a
// lane that holds a value at all (rows of fewer runs than lanes, rows beyond the last one)
struct AccFoldRowLanes {
  typedef Spec::Env Env;
  struct Elt {
    Spec::Elt v;
    u32 f;
  };
  ACC_DEV Elt combine(const Env& env, const Elt& a, const Elt& b) {
    if constexpr (sizeof(Spec::Elt) <= 8) {
      if (b.f & 1u) return b;
      Elt r;
      if ((a.f & 2u) && (b.f & 2u)) r.v = Spec::combine(env, a.v, b.v);
      else if (b.f & 2u) r.v = b.v;
      else r.v = a.v;
      r.f = (a.f & 1u) | ((a.f | b.f) & 2u);
      return r;
    }
    // (larger values: the one kept is chosen word by word, see acc_pick; the function is only
    // applied to two values that exist: it may read tables with them)
    Elt r;
    const bool head = (b.f & 1u) != 0u, ha = (a.f & 2u) != 0u, hb = (b.f & 2u) != 0u;
    u32 wr[AccWords<Spec::Elt>::N];
    acc_to_words(acc_pick(head || hb, b.v, a.v), wr);
    if (!head && ha && hb) acc_to_words(Spec::combine(env, a.v, b.v), wr);
    r.v = acc_from_words<Spec::Elt>(wr);
    r.f = head ? b.f : ((a.f & 1u) | ((a.f | b.f) & 2u));
    return r;
  }
};

template <bool NT>
ACC_DEV void acc_fold_wrows_body(const Spec::Env& env, const Spec::Out& out, const FoldWaveRowsParams& p) {
  typedef Spec S;
  const int V = S::V;
  const int L = (int)p.lanes;
  const int lane = acc_lane();
  const int sub = lane & (L - 1), slot = lane / L;
  const int perStep = ACC_WAVE / L;  // rows a wave works on at a time
  AccFoldSrcIn<S, NT> src{env};
  const i64 first = (i64)blockIdx.x * p.rpg;
  const i64 last = first + p.rpg < p.rows ? first + p.rpg : p.rows;
  const i64 step = (i64)L * V;
  // joins the lanes of each row of a step and writes the rows' results
  auto finishRows = [&](i64 row, bool valid, S::Elt acc, bool have) {
    if (L > 1) {
      // through the wave's ordered scan (data-parallel moves only): a row's last lane ends up
      // with all of it
      AccFoldRowLanes::Elt t;
      t.v = acc;
      t.f = (sub == 0 ? 1u : 0u) | (have ? 2u : 0u);
      t = acc_wave_scan<AccFoldRowLanes>(env, t, lane);
      acc = t.v;
      have = (t.f & 2u) != 0u;
    }
    if (valid && sub == L - 1) {
      if (S::kSeeded) {
        const S::Elt z = S::seed(env);
        S::store(out, row, have ? S::combine(env, z, acc) : z);
      } else if (have) {
        S::store(out, row, acc);
      }
    }
  };
  i64 rw = first + (i64)acc_wave() * perStep;
  if (p.n <= step) {
    // a row is one run per lane at most: four steps of rows at a time, so that a lane has four
    // loads in flight
    const i64 stride = (i64)ACC_WAVES * perStep;
    const i64 e0 = (i64)sub * V;
    for (; rw + 3 * stride < last; rw += 4 * stride) {
      S::Elt acc[4];
      bool have[4], ok[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) ok[u] = rw + u * stride + slot < last;
      if (e0 + V <= p.n) {
        S::Elt x[4][S::V];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const i64 off = (ok[u] ? rw + u * stride + slot : first) * p.n;  // (a row that exists, for the lanes beyond the last)
#pragma unroll
          for (int k = 0; k < V; ++k) x[u][k] = src(off + e0 + k);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          acc[u] = x[u][0];
#pragma unroll
          for (int k = 1; k < V; ++k) acc[u] = S::combine(env, acc[u], x[u][k]);
          have[u] = ok[u];
        }
      } else {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          have[u] = false;
          if (ok[u])
            for (i64 e = e0; e < p.n; ++e) {
              const S::Elt y = src((rw + u * stride + slot) * p.n + e);
              acc[u] = have[u] ? S::combine(env, acc[u], y) : y;
              have[u] = true;
            }
        }
      }
      // (all lanes of the wave together: the join moves values between them)
#pragma unroll
      for (int u = 0; u < 4; ++u) finishRows(rw + u * stride + slot, ok[u], acc[u], have[u]);
    }
  }
  for (; rw < last; rw += (i64)ACC_WAVES * perStep) {
    const i64 row = rw + slot;
    const bool valid = row < last;
    const i64 off = row * p.n;
    S::Elt acc;
    bool have = false;
    if (valid) {
      // A commutative operator lets a lane take every L-th run of V elements, so that the wave's
      // loads cover consecutive memory; any other needs the row in order: a lane takes one stretch
      // of consecutive elements (a whole number of runs), and the join below, which goes through
      // the lanes in order, keeps the stretches in theirs.
      i64 e0 = (i64)sub * V, end = p.n, stp = step;
      if (!S::kCommutative) {
        const i64 stretch = ((p.n + L - 1) / L + V - 1) / V * V;
        e0 = (i64)sub * stretch;
        end = e0 + stretch < p.n ? e0 + stretch : p.n;
        stp = V;
      }
      // four runs at a time, their loads together
      for (; e0 + 3 * stp + V <= end; e0 += 4 * stp) {
        S::Elt x[4][S::V];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int k = 0; k < V; ++k) x[u][k] = src(off + e0 + u * stp + k);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int k = 0; k < V; ++k) {
            acc = have ? S::combine(env, acc, x[u][k]) : x[u][k];
            have = true;
          }
      }
      for (; e0 + V <= end; e0 += stp) {
        S::Elt x[S::V];
#pragma unroll
        for (int k = 0; k < V; ++k) x[k] = src(off + e0 + k);
#pragma unroll
        for (int k = 0; k < V; ++k) {
          acc = have ? S::combine(env, acc, x[k]) : x[k];
          have = true;
        }
      }
      for (i64 e = e0; e < end; ++e) {  // the ragged end of the row (or of the stretch), in one lane
        const S::Elt x = src(off + e);
        acc = have ? S::combine(env, acc, x) : x;
        have = true;
      }
    }
    finishRows(row, valid, acc, have);
  }
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_fold_wrows(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldWaveRowsParams p) {
  acc_fold_wrows_body<false>(env, out, p);
}
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_fold_wrows_stream(Spec::Env env, Spec::Out out, Spec::Out tmp, FoldWaveRowsParams p) {
  acc_fold_wrows_body<true>(env, out, p);
}
