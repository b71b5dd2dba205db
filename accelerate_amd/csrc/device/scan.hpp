// Scan skeleton: scanl, scanl1, scanl', scanr, scanr1, scanr' along the innermost dimension,
// independently per outer row (Interpreter.hs:427-582), as a single pass over the data
// with decoupled look-back between tiles.
//
// Everything is phrased in traversal order t = 0..n-1 (left scans: t is the position;
// right scans: t = n-1-position) with S::combine(earlier, later); for right scans the
// generated combine swaps its operands, which gives the reference's `f input accumulated`.
// With incl[t] the running combination of the inputs up to t and val[t] = z (+) incl[t]
// when seeded:
//   kind 0 (scanl1/scanr1):  out[t] = incl[t]
//   kind 1 (scanl/scanr):    out has n+1 entries: entry 0 = z, entry t+1 = val[t]
//   kind 2 (scanl'/scanr'):  out has n entries: entry 0 = z, entry t+1 = val[t] (t+1 < n);
//                            tot[row] = val[n-1], or z when n = 0
// (entry u lives at position u for left scans and at the mirrored position for right scans).
//
// Tile layout: a workgroup has 16 waves (1024 threads) and a tile is 16 * G * 64 * V
// consecutive elements of one row.  Wave w
// owns G consecutive groups; in a group, lane l owns V consecutive elements, so every
// load and store of a wave is one coalesced run of 64 * V elements (128 bits per lane for
// plain arrays).  Order of work: lane-local scan, ordered wave scan per group, chain of
// group totals inside the wave, wave totals through LDS, then the tile's exclusive prefix
// from its predecessors by look-back.
//
// Look-back: tiles take their number from an atomic ticket, so a tile only ever waits for
// tiles that have already started.  Each tile publishes its aggregate, looks back, and
// publishes its inclusive prefix.  One round trip to a predecessor's descriptor costs on
// the order of a microsecond on this part (device-scope loads cross the XCDs), and the
// prefix can only advance along the row by (descriptors inspected per round trip) per
// round trip.  Large tiles (1024 threads x 192 bytes) keep the number of tiles, and with it
// the number of round trips on the critical path, small; with one workgroup resident per
// CU the nearest inclusive prefix is a few dozen tiles away, so one wave polling a window of
// 64 predecessors (one lane each) resolves it in one round trip.  ACC_SCAN_LBWAVES waves can
// poll further windows in parallel; measured on MI355X more polling only costs.  A published value is cut into 32-bit words, each stored with a relaxed
// device-scope 64-bit atomic next to the launch's epoch: a word is valid exactly when its
// upper half equals the epoch, so no fence or initialisation pass is needed, values of
// any size can be exchanged, and descriptors left by earlier launches read as "not yet".

struct ScanParams {
  i64 rows;
  i64 n;            // extent of the innermost dimension
  i64 tpr;          // tiles per row (>= 1)
  u64* desc;        // [rows * tpr][W] descriptor words
  u64* ticket;      // monotonically increasing counter shared by all launches of a context
  u64 ticket_base;  // value of the counter when this launch starts
  u64 epoch;        // tag of this launch, 1 .. 2^30 - 1
  u64 spin_limit;   // polls of one window after which a tile stops waiting for its predecessors
  u32* err;         // host-visible word: 3 = a tile gave up waiting, or took a ticket outside the launch
  i64 tpr_full;     // tiles per row that lie completely inside the row (the pipelined kernel's share)
};

#ifndef ACC_SCAN_BLOCK
#define ACC_SCAN_BLOCK 1024  // threads per workgroup; the generated code may set another size
#endif
#define ACC_SCAN_WAVES (ACC_SCAN_BLOCK / ACC_WAVE)
#ifndef ACC_SCAN_MINWAVES
#define ACC_SCAN_MINWAVES 4  // waves per SIMD the register allocation must leave room for
#endif

template <class S> struct AccScanCfg {
  enum {
    V = S::V,
    G = S::G,
    W = AccWords<typename S::Elt>::N,
    GROUP = ACC_WAVE * V,
    TILE = ACC_SCAN_WAVES * G * GROUP
  };
};

// Descriptor words.  A tile owns W 64-bit words; word k carries the k-th 32-bit word of the
// published value in its lower half and (epoch << 2 | state) in its upper half, state 1 =
// the tile's aggregate, 2 = its inclusive prefix (which overwrites the aggregate).  A read
// is valid when all W words carry the same tag of this launch.
#ifndef ACC_SCAN_LBWAVES
#define ACC_SCAN_LBWAVES 1   // waves of the workgroup that poll predecessors (64 each)
#endif
#ifndef ACC_SCAN_SLEEP
#define ACC_SCAN_SLEEP 16    // s_sleep argument between two polls of the same window
#endif
#ifndef ACC_SCAN_SETTLE
#define ACC_SCAN_SETTLE 32   // s_sleep argument before the first poll of a tile in a long launch
#endif
#ifndef ACC_SCAN_SETTLE_TILES
#define ACC_SCAN_SETTLE_TILES 4096  // a launch of at least this many tiles is a long one
#endif

// Two descriptor words moved as one 16-byte access at device scope.  Values of an even number
// of words travel this way: a poll of 64 predecessors of an Int64 scan is then one load
// instruction over 8 cache lines instead of two, and what a poll waits for is its slowest
// request (2^28 Int64 through the pipelined kernel: 779 -> 715 us).  Each 8-byte half still
// validates itself, so it does not matter whether the 16 bytes arrive as one piece.  The load
// waits for the wave's outstanding memory operations: a polling wave has none but its polls.
typedef u32 acc_u32x4 __attribute__((ext_vector_type(4)));
ACC_DEV void acc_store16(u64* slot, u64 w0, u64 w1) {
  acc_u32x4 v = {(u32)w0, (u32)(w0 >> 32), (u32)w1, (u32)(w1 >> 32)};
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(slot), "v"(v) : "memory");
}
ACC_DEV void acc_load16(const u64* slot, u64& w0, u64& w1) {
  acc_u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(slot) : "memory");
  w0 = (u64)v[0] | ((u64)v[1] << 32);
  w1 = (u64)v[2] | ((u64)v[3] << 32);
}

template <class E> ACC_DEV void acc_publish(u64* slot, const E& v, u64 epoch, u64 state) {
  constexpr int N = AccWords<E>::N;
  u32 w[N];
  acc_to_words(v, w);
  const u64 tag = ((epoch << 2) | state) << 32;
  if constexpr (N % 2 == 0) {
#pragma unroll
    for (int k = 0; k < N; k += 2) acc_store16(slot + k, tag | (u64)w[k], tag | (u64)w[k + 1]);
  } else {
#pragma unroll
    for (int k = 0; k < N; ++k)
      __hip_atomic_store(slot + k, tag | (u64)w[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// 0: nothing valid yet, 1: aggregate, 2: inclusive prefix
template <class E> ACC_DEV int acc_try_read(const u64* slot, E& v, u64 epoch) {
  u32 w[AccWords<E>::N];
  u64 tag0 = 0;
  bool same = true;
  if constexpr (AccWords<E>::N % 2 == 0) {
#pragma unroll
    for (int k = 0; k < AccWords<E>::N; k += 2) {
      u64 x, y;
      acc_load16(slot + k, x, y);
      if (k == 0) tag0 = x >> 32;
      same = same && ((x >> 32) == tag0) && ((y >> 32) == tag0);
      w[k] = (u32)x;
      w[k + 1] = (u32)y;
    }
  } else {
#pragma unroll
    for (int k = 0; k < AccWords<E>::N; ++k) {
      u64 x = __hip_atomic_load(slot + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (k == 0) tag0 = x >> 32;
      same = same && ((x >> 32) == tag0);
      w[k] = (u32)x;
    }
  }
  if (!same || (tag0 >> 2) != epoch) return 0;
  const int st = (int)(tag0 & 3);
  if (st != 1 && st != 2) return 0;
  v = acc_from_words<E>(w);
  return st;
}

// a (+) b where either side may be absent
template <class S>
ACC_DEV bool acc_join(const typename S::Env& env, bool ha, const typename S::Elt& a, bool hb, const typename S::Elt& b,
                      typename S::Elt& r) {
  if (ha && hb) r = S::combine(env, a, b);
  else if (ha) r = a;
  else if (hb) r = b;
  return ha || hb;
}

// One wave resolves the window of 64 predecessors ending at tile index `look` (lane 0
// looks at `look`, lane l at look - l).  It polls until it sees, from the nearest
// predecessor outwards, only aggregates up to the first predecessor that ends the walk (an
// inclusive prefix, or the start of the row), or 64 aggregates.  On return lane 0 holds in
// `r` the ordered combination of the `nv` values found (nv may be 0) and `terminal` says
// whether the walk ends inside this window.
//
// The wait is bounded: every tile takes its number from the ticket, so all tiles it waits for
// have started and the wait is short; should the host's idea of the ticket counter ever be
// wrong (tiles then carry numbers their predecessors never get), the wave gives up after
// `limit` polls, reports through `err` and returns as if the walk had ended with nothing
// found, so that every workgroup still finishes and the next wait on the stream raises the
// error instead of the launch never ending.
template <class S>
ACC_DEV void acc_window(const typename S::Env& env, const u64* rowDesc, i64 look, u64 epoch, u64 limit, u32* err,
                        typename S::Elt& r, int& nv, bool& terminal) {
  typedef typename S::Elt Elt;
  const int W = AccScanCfg<S>::W;
  const int lane = acc_lane();
  const i64 idx = look - lane;
  int st;  // 0 not yet, 1 aggregate, 2 inclusive prefix, 3 before the row
  Elt val;
  int first;
  u64 polls = 0;
  for (;;) {
    st = idx < 0 ? 3 : acc_try_read<Elt>(rowDesc + idx * W, val, epoch);
    if (st == 1 && S::stops(val)) st = 2;  // nothing before this aggregate can matter
    const u64 mEnd = __ballot(st >= 2);
    const u64 mInv = __ballot(st == 0);
    first = mEnd ? __builtin_ctzll(mEnd) : ACC_WAVE;
    const u64 need = first >= 63 ? ~0ull : ((2ull << first) - 1);
    if ((mInv & need) == 0) break;
    if (++polls >= limit) {
      if (lane == 0) __hip_atomic_store(err, 3u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      nv = 0;
      terminal = true;
      return;
    }
    __builtin_amdgcn_s_sleep(ACC_SCAN_SLEEP);
  }
  nv = ACC_WAVE;
  terminal = first < ACC_WAVE;
  if (terminal) {
    const int stEnd = __shfl(st, first, ACC_WAVE);
    if (stEnd == 3) {
      if (S::kSeeded) {
        if (lane == first) val = S::seed(env);
        nv = first + 1;
      } else {
        nv = first;
      }
    } else {
      nv = first + 1;
    }
  }
  // earlier tiles sit in higher lanes: fold them in from the left
  r = val;
#pragma unroll
  for (int d = 1; d < ACC_WAVE; d <<= 1) {
    Elt o = acc_shfl_down(r, d);
    if (lane + d < nv) r = S::combine(env, o, r);
  }
}

// Exclusive prefix of tile `tile` (> 0) of a row whose descriptors start at `rowDesc`.
// Called by all threads of the workgroup; the result is valid in thread 0.
template <class S>
ACC_DEV bool acc_lookback(const typename S::Env& env, const u64* rowDesc, i64 tile, u64 epoch, bool settle, u64 limit,
                          u32* err, typename S::Elt& excl) {
  typedef typename S::Elt Elt;
  enum { LB = ACC_SCAN_LBWAVES < ACC_SCAN_WAVES ? ACC_SCAN_LBWAVES : ACC_SCAN_WAVES };
  __shared__ Elt sh_win[LB];
  __shared__ int sh_nv[LB];
  __shared__ int sh_term[LB];
  __shared__ int sh_done;
  const int w = acc_wave();
  bool have = false;
  Elt running;
  i64 look = tile - 1;
  // In a long launch the nearest predecessors have published a little less than one trip to
  // their descriptors ago, so a poll sent at once finds them a moment too early and costs a
  // whole further round trip; one sent 2048 cycles later mostly succeeds (2^28 Int64: 0.770 ->
  // 0.757 ms).  Short launches, where every tile's wait is on the critical path, poll at once.
  // (the condition goes through a scalar register: under a mere lane mask the scalar s_sleep
  // would run whether or not any lane is enabled)
  if (__builtin_amdgcn_readfirstlane((int)(settle && w < LB))) __builtin_amdgcn_s_sleep(ACC_SCAN_SETTLE);
  for (;;) {
    if (w < LB) {
      Elt r;
      int nv;
      bool term;
      acc_window<S>(env, rowDesc, look - (i64)w * ACC_WAVE, epoch, limit, err, r, nv, term);
      if (acc_lane() == 0) {
        sh_win[w] = r;
        sh_nv[w] = nv;
        sh_term[w] = term ? 1 : 0;
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int done = 0;
      for (int k = 0; k < LB && !done; ++k) {  // nearest window first
        if (sh_nv[k] > 0) {
          running = have ? S::combine(env, sh_win[k], running) : sh_win[k];
          have = true;
        }
        done = sh_term[k];
      }
      sh_done = done;
    }
    __syncthreads();
    if (sh_done) break;
    look -= (i64)LB * ACC_WAVE;
  }
  excl = running;
  return have;
}

// Exclusive prefixes of the 64 * G values t[g] that the lanes of a wave hold, taken in the
// order (g, lane), by raking: the values go to the wave's stretch of LDS (`mine`, room for
// 64 * (G + 1) + 1 elements), every lane scans G consecutive ones serially, one ordered wave
// scan joins the 64 chunks, and every lane reads the prefix of each of its values back.  One
// wave scan instead of G, which were most of the vector instructions of these kernels.  A
// chunk takes G + 1 slots so that the lanes' reads of their chunks spread over the banks.
// Only the first `entries` values (in that order) hold data.  pre[g] is undefined for the
// very first value (g = 0 in lane 0); total is their combination, valid when entries > 0.
template <class S, int G>
ACC_DEV void acc_rake(const typename S::Env& env, typename S::Elt* mine, const typename S::Elt (&t)[G], int lane,
                      int entries, typename S::Elt (&pre)[G], typename S::Elt& total) {
  typedef typename S::Elt Elt;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int e = g * ACC_WAVE + lane;
    mine[(e / G) * (G + 1) + e % G] = t[g];
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  Elt c[G];
#pragma unroll
  for (int j = 0; j < G; ++j) c[j] = mine[lane * (G + 1) + j];
#pragma unroll
  for (int j = 1; j < G; ++j) c[j] = S::combine(env, c[j - 1], c[j]);  // inclusive inside the chunk
  Elt ts = acc_wave_scan<S>(env, c[G - 1], lane);
  Elt chunkPre = acc_prev_lane(ts);  // everything before this lane's chunk (lane > 0)
  // the total is the inclusive value of the last value that holds data
  if (entries > 0 && (entries - 1) / G == lane) {
    const int jl = (entries - 1) % G;
    Elt v = c[0];
#pragma unroll
    for (int j = 1; j < G; ++j)
      if (j == jl) v = c[j];
    mine[ACC_WAVE * (G + 1)] = lane > 0 ? S::combine(env, chunkPre, v) : v;
  }
  // exclusive prefixes go back in place
  if (lane > 0) mine[lane * (G + 1)] = chunkPre;
#pragma unroll
  for (int j = 1; j < G; ++j) mine[lane * (G + 1) + j] = lane > 0 ? S::combine(env, chunkPre, c[j - 1]) : c[j - 1];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int e = g * ACC_WAVE + lane;
    if (e > 0) pre[g] = mine[(e / G) * (G + 1) + e % G];
  }
  if (entries > 0) total = mine[ACC_WAVE * (G + 1)];
}

// One tile of a scan over a sequence of n elements: load(t) yields element t, store(t, y)
// receives val[t] (the inclusive combination up to t, seed included when S::kSeeded).
// `desc` holds the descriptors of this sequence's tiles.  Called by all threads of the
// workgroup (ACC_SCAN_BLOCK threads).  When `plain` holds, a tile that lies completely inside
// the sequence hands the V consecutive values of a lane to storeRun(t0, y) instead, which
// can move them with one wide request: a caller whose store tests for a special position
// (the total of scan', which is the sequence's last value) sets it for the tiles that cannot hold
// that position; in the tile that can, only the run that reaches the end goes value by value.  `settle` delays
// the first look at the predecessors (see acc_lookback).
template <class S, class Load, class Store, class StoreRun>
ACC_DEV void acc_scan_tile(const typename S::Env& env, u64* desc, i64 tiles, i64 tile, i64 n, u64 epoch, u64 limit,
                           u32* err, const Load& load, const Store& store, const StoreRun& storeRun, bool plain,
                           bool settle) {
  typedef typename S::Elt Elt;
  typedef AccScanCfg<S> C;
  const int V = C::V, G = C::G, W = C::W;
  __shared__ Elt sh_wave[ACC_SCAN_WAVES];   // wave totals, then inclusive prefixes of the wave totals
  __shared__ Elt sh_excl;
  __shared__ int sh_has_excl;
  const int lane = acc_lane(), w = acc_wave();
  const i64 tlo = tile * (i64)C::TILE;
  const i64 wlo = tlo + (i64)w * G * C::GROUP;

  // load + lane-local scan; trailing invalid slots repeat the last valid value so that
  // x[g][V-1] is always the lane's total.  A tile that lies completely inside the sequence
  // takes the branch without bounds tests, which lets the V consecutive accesses of a lane
  // become one wide request.
  Elt x[C::G][C::V];
  Elt filler;
  const bool full = tlo + (i64)C::TILE <= n;
  if (full) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
      Elt e[C::V];
#pragma unroll
      for (int k = 0; k < V; ++k) e[k] = load(t0 + k);
      x[g][0] = e[0];
#pragma unroll
      for (int k = 1; k < V; ++k) x[g][k] = S::combine(env, x[g][k - 1], e[k]);
    }
    filler = x[0][0];
  } else {
    // Slots past the end repeat a real element (the tile's first one), and so do the totals
    // of waves without data: the wave scans and the raking below apply the combination
    // function to every lane, and that function may only ever see values of the array (it
    // may index a table by its operands, or loop on them).  Nothing of this is stored.
    // A wave's group that lies inside the sequence is loaded like those of a full tile (the test
    // is the same for all its lanes): of a row that fills three quarters of its tile, only the
    // one group that holds the row's end goes element by element.
    filler = tlo < n ? load(tlo) : S::seed(env);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
      if (wlo + (i64)(g + 1) * C::GROUP <= n) {
        Elt e[C::V];
#pragma unroll
        for (int k = 0; k < V; ++k) e[k] = load(t0 + k);
        x[g][0] = e[0];
#pragma unroll
        for (int k = 1; k < V; ++k) x[g][k] = S::combine(env, x[g][k - 1], e[k]);
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) {
          const i64 t = t0 + k;
          if (t < n) {
            Elt e = load(t);
            x[g][k] = k == 0 ? e : S::combine(env, x[g][k - 1], e);
          } else {
            if (k > 0) x[g][k] = x[g][k - 1];
          else x[g][k] = filler;
          }
        }
      }
    }
  }

  Elt waveTot = filler;
  bool hasWaveTot = false;
#ifdef ACC_SCAN_RAKE
  // prefixes of the lane totals by raking (acc_rake), applied to the elements at once, so
  // that only x stays live across the look-back
  {
    __shared__ Elt sh_rake[ACC_SCAN_WAVES][ACC_WAVE * (C::G + 1) + 1];
    i64 wcnt = n - wlo;  // elements of the sequence from this wave's start on
    wcnt = wcnt < 0 ? 0 : (wcnt > (i64)G * C::GROUP ? (i64)G * C::GROUP : wcnt);
    const int entries = (int)((wcnt + V - 1) / V);  // lane totals that hold data; they come first
    Elt tl[C::G], pre[C::G];
#pragma unroll
    for (int g = 0; g < G; ++g) tl[g] = x[g][V - 1];
    acc_rake<S, C::G>(env, sh_rake[w], tl, lane, entries, pre, waveTot);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g * ACC_WAVE + lane > 0) {
#pragma unroll
        for (int k = 0; k < V; ++k) x[g][k] = S::combine(env, pre[g], x[g][k]);
      }
    }
    hasWaveTot = entries > 0;
  }
#else
  // Wave scan per group, chained over the groups of this wave; the prefix inside the wave
  // is applied to the elements at once, so that only x stays live across the look-back.
#pragma unroll
  for (int g = 0; g < G; ++g) {
    i64 cnt = n - (wlo + (i64)g * C::GROUP);
    cnt = cnt < 0 ? 0 : (cnt > C::GROUP ? C::GROUP : cnt);
    Elt ts = acc_wave_scan<S>(env, x[g][V - 1], lane);
    Elt lanePre = acc_prev_lane(ts);  // exclusive prefix of the lane inside its group (lane > 0)
    const int last = cnt > 0 ? (int)((cnt - 1) / V) : 0;
    Elt gt = acc_readlane(ts, last);
    Elt pre;
    if (acc_join<S>(env, hasWaveTot, waveTot, lane > 0, lanePre, pre)) {
#pragma unroll
      for (int k = 0; k < V; ++k) x[g][k] = S::combine(env, pre, x[g][k]);
    }
    if (cnt > 0) {
      waveTot = hasWaveTot ? S::combine(env, waveTot, gt) : gt;
      hasWaveTot = true;
    }
  }
#endif
  if (lane == 0) sh_wave[w] = waveTot;
  __syncthreads();

  // a wave has data only if all earlier waves are full, so validity follows from counts
  const i64 tcnt = n - tlo;  // elements from the tile's start to the end (may exceed TILE)
  const i64 perWave = (i64)G * C::GROUP;
  i64 wd = tcnt <= 0 ? 0 : (tcnt + perWave - 1) / perWave;
  const int wavesWithData = wd > ACC_SCAN_WAVES ? ACC_SCAN_WAVES : (int)wd;
  const bool successors = tile + 1 < tiles;

  // the first wave scans the wave totals (ordered) and publishes the tile's aggregate
  if (w == 0) {
    Elt t = sh_wave[lane < ACC_SCAN_WAVES ? lane : 0];
    t = acc_wave_scan<S>(env, t, lane);
    if (lane < ACC_SCAN_WAVES) sh_wave[lane] = t;
    if (lane == wavesWithData - 1 && tile > 0 && successors) acc_publish<Elt>(desc + tile * W, t, epoch, 1);
  }
  __syncthreads();

  Elt excl;
  bool hasExcl = false;
  if (tile == 0) {
    if (S::kSeeded) {
      excl = S::seed(env);
      hasExcl = true;
    }
  } else {
    hasExcl = acc_lookback<S>(env, desc, tile, epoch, settle, limit, err, excl);  // valid in thread 0
  }
  if (threadIdx.x == 0) {
    if (successors && wavesWithData > 0) {
      Elt inc;
      acc_join<S>(env, hasExcl, excl, true, sh_wave[wavesWithData - 1], inc);
      acc_publish<Elt>(desc + tile * W, inc, epoch, 2);
    }
    sh_excl = excl;
    sh_has_excl = hasExcl ? 1 : 0;
  }
  __syncthreads();

  // prefix of everything before this wave
  Elt base;
  const bool hasWavePre = w > 0 && w <= wavesWithData;
  Elt wavePre = sh_wave[w > 0 ? w - 1 : 0];
  bool hasBase = acc_join<S>(env, sh_has_excl != 0, sh_excl, hasWavePre, wavePre, base);
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
    if (full || wlo + (i64)(g + 1) * C::GROUP <= n) {
      Elt y[C::V];
#pragma unroll
      for (int k = 0; k < V; ++k) y[k] = hasBase ? S::combine(env, base, x[g][k]) : x[g][k];
      if (plain || t0 + V < n) {  // (the special position is the sequence's last)
        storeRun(t0, y);
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) store(t0 + k, y[k]);
      }
    } else {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const i64 t = t0 + k;
        if (t < n) store(t, hasBase ? S::combine(env, base, x[g][k]) : x[g][k]);
      }
    }
  }
}

// Values paired with a head flag: the scan of such pairs under
//     (fa, a) (+) (fb, b) = fb ? (1, b) : (fa, a (+) b)
// restarts at every head and is associative whenever (+) is.
template <class S> struct AccSegSpec {
  typedef typename S::Env Env;
  struct Elt {
    typename S::Elt v;
    u32 f;
  };
  enum { V = S::V, G = S::G };
  static constexpr bool kSeeded = false;  // z is applied when a segment's value is written
  ACC_DEV Elt combine(const Env& env, const Elt& a, const Elt& b) {
    // (the value goes through its words, so that `b or the combination` is a choice between
    // values and not between the addresses of two objects: see acc_pick)
    Elt r;
    u32 wr[AccWords<typename S::Elt>::N];
    acc_to_words(b.v, wr);
    if (!b.f) acc_to_words(S::combine(env, a.v, b.v), wr);
    r.v = acc_from_words<typename S::Elt>(wr);
    r.f = b.f ? b.f : a.f;
    return r;
  }
  ACC_DEV Elt seed(const Env&) {
    Elt r{};
    return r;
  }
  // an aggregate that contains a segment head hides everything before it: the look-back
  // of a later tile may stop there
  ACC_DEV bool stops(const Elt& a) { return a.f != 0; }
};

// Many rows shorter than a tile: a workgroup takes `cnt` consecutive elements of the
// row-major stream that are a whole number of rows of n elements (cnt <= TILE) and scans
// them as (head flag, value) pairs with a head at the start of every row, so that no lane
// idles however short the rows are and nothing is exchanged between workgroups.
// load(idx, r, t) yields the element at stream position idx of the tile = row r of the
// tile, traversal position t; store(idx, r, t, y) receives the running combination of
// row r up to t.  Called by all threads of the workgroup.
template <class S, class Load, class Store>
ACC_DEV void acc_rows_tile(const typename S::Env& env, int cnt, int n, const Load& load, const Store& store) {
  typedef AccSegSpec<S> SS;
  typedef typename SS::Elt P;
  typedef AccScanCfg<S> C;
  const int V = C::V, G = C::G;
  __shared__ P sh_wave[ACC_SCAN_WAVES];
  const int lane = acc_lane(), w = acc_wave();
  const int wlo = w * G * C::GROUP;
  P x[C::G][C::V];
  P filler;
  bool haveFiller = false;
  int r0[C::G], t0[C::G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int idx0 = wlo + (g * ACC_WAVE + lane) * V;
    int r = idx0 / n, t = idx0 - r * n;
    r0[g] = r;
    t0[g] = t;
    if (wlo + (g + 1) * C::GROUP <= cnt) {
      // the whole group lies inside (wave-uniform): no tests, so that the V loads of a lane
      // can become one wide request
      P e[C::V];
#pragma unroll
      for (int k = 0; k < V; ++k) {
        e[k].v = load(idx0 + k, r, t);
        e[k].f = t == 0 ? 1u : 0u;
        if (++t == n) {
          t = 0;
          ++r;
        }
      }
      x[g][0] = e[0];
#pragma unroll
      for (int k = 1; k < V; ++k) x[g][k] = SS::combine(env, x[g][k - 1], e[k]);
    } else {
      // slots past the end repeat the first element of the stretch (see acc_scan_tile)
      if (!haveFiller) {
        filler.v = load(0, 0, 0);
        filler.f = 1u;
        haveFiller = true;
      }
#pragma unroll
      for (int k = 0; k < V; ++k) {
        if (idx0 + k < cnt) {
          P e;
          e.v = load(idx0 + k, r, t);
          e.f = t == 0 ? 1u : 0u;
          x[g][k] = k == 0 ? e : SS::combine(env, x[g][k - 1], e);
        } else {
          if (k > 0) x[g][k] = x[g][k - 1];
          else x[g][k] = filler;
        }
        if (++t == n) {
          t = 0;
          ++r;
        }
      }
    }
  }
  // (not `haveFiller ? filler : x[0][0]`: a choice between two objects is a choice between two
  // addresses, and values of 16 bytes then live in scratch memory -- the rows kernels ran at
  // 0.84 TB/s for 8-byte elements)
  P waveTot = x[0][0];
  if (haveFiller) waveTot = filler;
  bool hasWaveTot = false;
#ifdef ACC_ROWS_RAKE
  {
    // prefixes of the lane totals by raking (acc_rake)
    __shared__ P sh_rake[ACC_SCAN_WAVES][ACC_WAVE * (C::G + 1) + 1];
    int wcnt = cnt - wlo;
    wcnt = wcnt < 0 ? 0 : (wcnt > G * C::GROUP ? G * C::GROUP : wcnt);
    const int entries = (wcnt + V - 1) / V;
    P tl[C::G], pre[C::G];
#pragma unroll
    for (int g = 0; g < G; ++g) tl[g] = x[g][V - 1];
    acc_rake<SS, C::G>(env, sh_rake[w], tl, lane, entries, pre, waveTot);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g * ACC_WAVE + lane > 0) {
#pragma unroll
        for (int k = 0; k < V; ++k) x[g][k] = SS::combine(env, pre[g], x[g][k]);
      }
    }
    hasWaveTot = entries > 0;
  }
#else
  {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      int c = cnt - (wlo + g * C::GROUP);
      c = c < 0 ? 0 : (c > C::GROUP ? C::GROUP : c);
      P ts = acc_wave_scan<SS>(env, x[g][V - 1], lane);
      P lanePre = acc_prev_lane(ts);
      const int last = c > 0 ? (c - 1) / V : 0;
      P gt = acc_readlane(ts, last);
      P pre;
      if (acc_join<SS>(env, hasWaveTot, waveTot, lane > 0, lanePre, pre)) {
#pragma unroll
        for (int k = 0; k < V; ++k) x[g][k] = SS::combine(env, pre, x[g][k]);
      }
      if (c > 0) {
        waveTot = hasWaveTot ? SS::combine(env, waveTot, gt) : gt;
        hasWaveTot = true;
      }
    }
  }
#endif
  if (lane == 0) sh_wave[w] = waveTot;
  __syncthreads();
  const int perWave = G * C::GROUP;
  int wavesWithData = (cnt + perWave - 1) / perWave;
  if (wavesWithData > ACC_SCAN_WAVES) wavesWithData = ACC_SCAN_WAVES;
  if (w == 0) {
    P t = sh_wave[lane < ACC_SCAN_WAVES ? lane : 0];
    t = acc_wave_scan<SS>(env, t, lane);
    if (lane < ACC_SCAN_WAVES) sh_wave[lane] = t;
  }
  __syncthreads();
  const bool hasBase = w > 0 && w <= wavesWithData;
  const P base = sh_wave[w > 0 ? w - 1 : 0];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int idx0 = wlo + (g * ACC_WAVE + lane) * V;
    int r = r0[g], t = t0[g];
    if (wlo + (g + 1) * C::GROUP <= cnt) {
      typename S::Elt y[C::V];
#pragma unroll
      for (int k = 0; k < V; ++k) y[k] = (hasBase ? SS::combine(env, base, x[g][k]) : x[g][k]).v;
#pragma unroll
      for (int k = 0; k < V; ++k) {
        store(idx0 + k, r, t, y[k]);
        if (++t == n) {
          t = 0;
          ++r;
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        if (idx0 + k < cnt) {
          const P y = hasBase ? SS::combine(env, base, x[g][k]) : x[g][k];
          store(idx0 + k, r, t, y.v);
        }
        if (++t == n) {
          t = 0;
          ++r;
        }
      }
    }
  }
}

ACC_DEV i64 acc_take_ticket(u64* ticket, u64 base) {
  __shared__ i64 sh_tile;
  if (threadIdx.x == 0)
    sh_tile = (i64)(__hip_atomic_fetch_add(ticket, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - base);
  __syncthreads();
  return sh_tile;
}
