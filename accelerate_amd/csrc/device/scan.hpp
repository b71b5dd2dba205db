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
// Tile layout: a tile is ACC_WAVES * G * 64 * V consecutive elements of one row.  Wave w
// owns G consecutive groups; in a group, lane l owns V consecutive elements, so every
// load and store of a wave is one coalesced run of 64 * V elements (128 bits per lane for
// plain arrays).  Order of work: lane-local scan, ordered wave scan per group, chain of
// group totals inside the wave, wave totals through LDS, then the tile's exclusive prefix
// from its predecessors by look-back.
//
// Look-back: tiles take their number from an atomic ticket, so a tile only ever waits for
// tiles that have already started.  Each tile publishes its aggregate, looks back over
// windows of 64 predecessors with one lane per predecessor, and publishes its inclusive
// prefix.  A published value is cut into 32-bit words, each stored with a relaxed
// device-scope 64-bit atomic next to the launch's epoch: a word is valid exactly when its
// upper half equals the epoch, so no fence or initialisation pass is needed, values of
// any size can be exchanged, and descriptors left by earlier launches read as "not yet".

struct ScanParams {
  i64 rows;
  i64 n;            // extent of the innermost dimension
  i64 tpr;          // tiles per row (>= 1)
  u64* desc;        // [rows * tpr][2][W] words: aggregate, inclusive prefix
  u64* ticket;      // monotonically increasing counter shared by all launches of a context
  u64 ticket_base;  // value of the counter when this launch starts
  u64 epoch;        // tag of this launch, never 0
};

template <class S> struct AccScanCfg {
  enum {
    V = S::V,
    G = S::G,
    W = AccWords<typename S::Elt>::N,
    GROUP = ACC_WAVE * V,
    TILE = ACC_WAVES * G * GROUP
  };
};

template <class E> ACC_DEV void acc_publish(u64* slot, const E& v, u64 epoch) {
  u32 w[AccWords<E>::N];
  acc_to_words(v, w);
#pragma unroll
  for (int k = 0; k < AccWords<E>::N; ++k)
    __hip_atomic_store(slot + k, (epoch << 32) | (u64)w[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <class E> ACC_DEV bool acc_try_read(const u64* slot, E& v, u64 epoch) {
  u32 w[AccWords<E>::N];
  bool ok = true;
#pragma unroll
  for (int k = 0; k < AccWords<E>::N; ++k) {
    u64 x = __hip_atomic_load(slot + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ok = ok && ((x >> 32) == epoch);
    w[k] = (u32)x;
  }
  if (ok) v = acc_from_words<E>(w);
  return ok;
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

// Exclusive prefix of tile `tile` (> 0) of a row whose descriptors start at `rowDesc`;
// run by all lanes of one wave, result valid in lane 0.
template <class S>
ACC_DEV bool acc_lookback(const typename S::Env& env, const u64* rowDesc, i64 tile, u64 epoch, typename S::Elt& excl) {
  typedef typename S::Elt Elt;
  const int W = AccScanCfg<S>::W;
  const int lane = acc_lane();
  bool have = false;
  Elt running;
  i64 look = tile - 1;
  for (;;) {
    const i64 idx = look - lane;  // lane 0 looks at the nearest predecessor
    int st;                       // 0 not yet, 1 aggregate, 2 inclusive prefix, 3 before the row
    Elt val;
    int first;
    for (;;) {
      st = 0;
      if (idx < 0) st = 3;
      else if (acc_try_read<Elt>(rowDesc + (idx * 2 + 1) * W, val, epoch)) st = 2;
      else if (acc_try_read<Elt>(rowDesc + (idx * 2 + 0) * W, val, epoch)) st = 1;
      const u64 mEnd = __ballot(st >= 2);
      const u64 mInv = __ballot(st == 0);
      first = mEnd ? __builtin_ctzll(mEnd) : ACC_WAVE;
      const u64 need = first >= 63 ? ~0ull : ((2ull << first) - 1);
      if ((mInv & need) == 0) break;
      __builtin_amdgcn_s_sleep(1);
    }
    int nv = ACC_WAVE;
    if (first < ACC_WAVE) {
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
    Elt r = val;
#pragma unroll
    for (int d = 1; d < ACC_WAVE; d <<= 1) {
      Elt o = acc_shfl_down(r, d);
      if (lane + d < nv) r = S::combine(env, o, r);
    }
    if (nv > 0) {
      running = have ? S::combine(env, r, running) : r;
      have = true;
    }
    if (first < ACC_WAVE) break;
    look -= ACC_WAVE;
  }
  excl = running;
  return have;
}

// One tile of a scan over a sequence of n elements: load(t) yields element t, store(t, y)
// receives val[t] (the inclusive combination up to t, seed included when S::kSeeded).
// `desc` holds the descriptors of this sequence's tiles.  Called by all threads of the
// workgroup.
template <class S, class Load, class Store>
ACC_DEV void acc_scan_tile(const typename S::Env& env, u64* desc, i64 tiles, i64 tile, i64 n, u64 epoch,
                           const Load& load, const Store& store) {
  typedef typename S::Elt Elt;
  typedef AccScanCfg<S> C;
  const int V = C::V, G = C::G, W = C::W;
  __shared__ Elt sh_wave[ACC_WAVES];
  __shared__ Elt sh_excl;
  __shared__ int sh_has_excl;
  const int lane = acc_lane(), w = acc_wave();
  const i64 tlo = tile * (i64)C::TILE;
  const i64 wlo = tlo + (i64)w * G * C::GROUP;

  // load + lane-local scan; trailing invalid slots repeat the last valid value so that
  // x[g][V-1] is always the lane's total
  Elt x[C::G][C::V];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      const i64 t = t0 + k;
      if (t < n) {
        Elt e = load(t);
        x[g][k] = k == 0 ? e : S::combine(env, x[g][k - 1], e);
      } else if (k > 0) {
        x[g][k] = x[g][k - 1];
      }
    }
  }

  // wave scan per group, then chain the groups of this wave
  Elt lanePre[C::G];   // exclusive prefix of the lane inside its group (lane > 0)
  Elt groupPre[C::G];  // exclusive prefix of the group inside its wave
  bool hasGroupPre[C::G];
  Elt waveTot;
  bool hasWaveTot = false;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    i64 cnt = n - (wlo + (i64)g * C::GROUP);
    cnt = cnt < 0 ? 0 : (cnt > C::GROUP ? C::GROUP : cnt);
    Elt ts = acc_wave_scan<S>(env, x[g][V - 1], lane);
    lanePre[g] = acc_shfl_up(ts, 1);
    const int last = cnt > 0 ? (int)((cnt - 1) / V) : 0;
    Elt gt = acc_shfl(ts, last);
    groupPre[g] = waveTot;
    hasGroupPre[g] = hasWaveTot;
    if (cnt > 0) {
      waveTot = hasWaveTot ? S::combine(env, waveTot, gt) : gt;
      hasWaveTot = true;
    }
  }
  if (lane == 0) sh_wave[w] = waveTot;
  __syncthreads();

  // a wave has data only if all earlier waves are full, so validity follows from counts
  const i64 tcnt = n - tlo;  // elements from the tile's start to the end (may exceed TILE)
  const i64 perWave = (i64)G * C::GROUP;
  i64 wd = tcnt <= 0 ? 0 : (tcnt + perWave - 1) / perWave;
  const int wavesWithData = wd > ACC_WAVES ? ACC_WAVES : (int)wd;
  Elt wavePre;
  bool hasWavePre = false;
#pragma unroll
  for (int k = 0; k < ACC_WAVES; ++k) {
    if (k < w && k < wavesWithData) {
      wavePre = hasWavePre ? S::combine(env, wavePre, sh_wave[k]) : sh_wave[k];
      hasWavePre = true;
    }
  }

  if (w == 0) {
    Elt agg;
    bool hasAgg = false;
#pragma unroll
    for (int k = 0; k < ACC_WAVES; ++k) {
      if (k < wavesWithData) {
        agg = hasAgg ? S::combine(env, agg, sh_wave[k]) : sh_wave[k];
        hasAgg = true;
      }
    }
    const bool successors = tile + 1 < tiles;
    Elt excl;
    bool hasExcl = false;
    if (tile == 0) {
      if (S::kSeeded) {
        excl = S::seed(env);
        hasExcl = true;
      }
    } else {
      if (lane == 0 && successors && hasAgg) acc_publish<Elt>(desc + (tile * 2 + 0) * W, agg, epoch);
      hasExcl = acc_lookback<S>(env, desc, tile, epoch, excl);
    }
    if (lane == 0) {
      if (successors && hasAgg) {
        Elt inc;
        acc_join<S>(env, hasExcl, excl, hasAgg, agg, inc);
        acc_publish<Elt>(desc + (tile * 2 + 1) * W, inc, epoch);
      }
      sh_excl = excl;
      sh_has_excl = hasExcl ? 1 : 0;
    }
  }
  __syncthreads();

  // prefix of everything before this wave
  Elt base;
  bool hasBase = acc_join<S>(env, sh_has_excl != 0, sh_excl, hasWavePre, wavePre, base);
#pragma unroll
  for (int g = 0; g < G; ++g) {
    Elt gb;
    bool hasGb = acc_join<S>(env, hasBase, base, hasGroupPre[g], groupPre[g], gb);
    Elt lp;
    bool hasLp = acc_join<S>(env, hasGb, gb, lane > 0, lanePre[g], lp);
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      const i64 t = t0 + k;
      if (t < n) store(t, hasLp ? S::combine(env, lp, x[g][k]) : x[g][k]);
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
