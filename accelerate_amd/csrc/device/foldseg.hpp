// FoldSeg / Fold1Seg skeleton (foldSegOp, Interpreter.hs:390-424): per outer row, segment
// s reduces the elements [offs[s], offs[s+1]) of the row, seeded once with z; an empty
// segment yields z.  The node receives offsets (Prelude.hs:710-717), not lengths.
//
// Load balance does not depend on segment lengths: the rows are laid end to end into one
// stream of rows*n elements which is cut into equal tiles, exactly as for a scan, and a
// tile computes a segmented inclusive scan of its elements, i.e. a scan of (head flag,
// value) pairs under
//     (fa, a) (+) (fb, b) = fb ? (1, b) : (fa, a (+) b)
// which is associative whenever (+) is.  Segments that cross tile borders get their
// carry through the same decoupled look-back as a plain scan.  The value of a segment is
// the scan value at its last element; it is written by the lane that holds that element.
//
// Boundaries: row r contributes S+1 boundaries at stream positions r*n + offs[s],
// s = 0..S (S segments per row).  Boundary number j = r*(S+1) + s starts segment (r, s)
// when s < S; what lies between boundary (r, S) and boundary (r+1, 0) belongs to no
// segment and is discarded.  A partition kernel finds, for every tile border, how many
// boundaries lie before it (binary search in the offsets), so a tile knows which
// boundaries fall inside it and marks them in LDS: sh_first[p] = first boundary at
// position p of the tile.  Empty segments are recognised while marking (two equal
// consecutive offsets) and get z directly.

struct FoldSegParams {
  i64 rows;
  i64 n;       // elements per row
  i64 nseg;    // segments per row (S)
  i64 total;   // rows * n
  i64 tiles;   // >= 1
  i64* part;   // [tiles + 1]: boundaries before each tile border; part[tiles] = rows * (S + 1)
  u64* desc;
  u64* ticket;
  u64 ticket_base;
  u64 epoch;
};

template <class S> struct AccSegSpec {
  typedef typename S::Env Env;
  struct Elt {
    typename S::Elt v;
    u32 f;
  };
  enum { V = S::V, G = S::G };
  static constexpr bool kSeeded = false;  // z is applied when a segment's value is written
  ACC_DEV Elt combine(const Env& env, const Elt& a, const Elt& b) {
    Elt r;
    if (b.f) {
      r = b;
    } else {
      r.v = S::combine(env, a.v, b.v);
      r.f = a.f;
    }
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

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_foldseg_partition(Spec::Env env, Spec::Out out, FoldSegParams p) {
  typedef AccScanCfg<AccSegSpec<Spec>> C;
  const i64 t = (i64)blockIdx.x * ACC_BLOCK + threadIdx.x;
  if (t > p.tiles) return;
  const i64 sp1 = p.nseg + 1;
  if (t == p.tiles) {
    p.part[t] = p.rows * sp1;
    return;
  }
  if (p.n <= 0) {
    p.part[t] = 0;
    return;
  }
  const i64 pos = t * (i64)C::TILE;
  const i64 row = pos / p.n;
  const i64 within = pos - row * p.n;
  i64 lo = 0, hi = sp1;  // first s with offs[s] >= within
  while (lo < hi) {
    const i64 mid = (lo + hi) >> 1;
    if (Spec::seg_at(env, mid) < within) lo = mid + 1;
    else hi = mid;
  }
  p.part[t] = row * sp1 + lo;
}

// One tile.  A lane owns, per group, a run of V consecutive elements and reduces it in
// order, starting afresh at every head.  A segment end whose segment began inside the run
// is written at once; the first end of a run that has seen no head yet still lacks what
// precedes the run, and is kept as the run's pending end (at most one per run).  The runs'
// aggregates (head seen, value since the last head) go through the ordered wave scan and
// the wave totals through LDS, exactly as in a plain scan, but only pending ends receive
// the prefix: a prefix that contains a head closes them inside the wave, the others wait
// for the tile's exclusive prefix from the look-back.
extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK)
acc_foldseg(Spec::Env env, Spec::Out out, FoldSegParams p) {
  typedef Spec S;
  typedef AccSegSpec<Spec> SS;
  typedef AccScanCfg<SS> C;
  typedef SS::Elt P;
  const int V = C::V, G = C::G, W = C::W;
  const int NONE = 0x7fffffff;
  __shared__ __attribute__((aligned(16))) int sh_first[C::TILE + 4];
  __shared__ P sh_wave[ACC_SCAN_WAVES];
  __shared__ P sh_excl;
  __shared__ int sh_has_excl;

  const i64 tile = acc_take_ticket(p.ticket, p.ticket_base);
  const i64 tlo = tile * (i64)C::TILE;
  const i64 sp1 = p.nseg + 1;
  const i64 j0 = p.part[tile], j1 = p.part[tile + 1];
  const int lane = acc_lane(), w = acc_wave();
  const i64 n = p.total;
  const i64 wlo = tlo + (i64)w * G * C::GROUP;
  const bool full = tlo + (i64)C::TILE <= n;
  // all loads of the tile are issued first: they depend on nothing but the tile number, and
  // could not be moved past the stores further down
  S::Elt x[C::G][C::V];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
    if (full) {
#pragma unroll
      for (int k = 0; k < V; ++k) x[g][k] = S::in_linear(env, t0 + k);
    } else {
#pragma unroll
      for (int k = 0; k < V; ++k)
        if (t0 + k < n) x[g][k] = S::in_linear(env, t0 + k);
    }
  }
  for (int i = threadIdx.x; i < C::TILE / 4 + 1; i += ACC_SCAN_BLOCK)
    reinterpret_cast<int4*>(sh_first)[i] = make_int4(NONE, NONE, NONE, NONE);
  __syncthreads();
  for (i64 j = j0 + threadIdx.x; j < j1; j += ACC_SCAN_BLOCK) {
    const i64 row = p.rows == 1 ? 0 : acc_quot(j, sp1), s = j - row * sp1;
    const i64 o = S::seg_at(env, s);
    const i64 rel = row * p.n + o - tlo;
    if (rel >= 0 && rel <= C::TILE) atomicMin(&sh_first[rel], (int)(j - j0));
    if (S::kSeeded && s < p.nseg && S::seg_at(env, s + 1) == o) S::store(out, row * p.nseg + s, S::seed(env));
  }
  if (threadIdx.x == 0 && tile + 1 < p.tiles && j1 < p.rows * sp1) {
    // a boundary sitting exactly on this tile's upper border belongs to the next tile
    const i64 row = j1 / sp1, s = j1 - row * sp1;
    if (row * p.n + S::seg_at(env, s) - tlo == C::TILE) sh_first[C::TILE] = (int)(j1 - j0);
  }
  __syncthreads();

  // the segment that ends where boundary j0 + idx sits
  auto emit = [&](int idx, const S::Elt& v) {
    const i64 j = j0 + idx;
    const i64 row = p.rows == 1 ? 0 : acc_quot(j, sp1), s = j - row * sp1;
    if (s == 0) return;  // what precedes a row's first boundary belongs to no segment
    S::store(out, row * p.nseg + s - 1, S::kSeeded ? S::combine(env, S::seed(env), v) : v);
  };

  P waveTot;
  bool hasWaveTot = false;
  S::Elt pendVal[C::G];
  int pendIdx[C::G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
    const int rel0 = (int)(t0 - tlo);
    int m[C::V + 1];
#pragma unroll
    for (int k = 0; k <= V; ++k) m[k] = sh_first[rel0 + k];
    i64 c = n - t0;
    c = c < 0 ? 0 : (c > V ? V : c);
    const S::Elt* e = x[g];
    P a{};
    bool has = false;
    pendIdx[g] = NONE;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (full || k < c) {
        if (m[k] != NONE) {
          a.v = e[k];
          a.f = 1u;
        } else {
          a.v = has ? S::combine(env, a.v, e[k]) : e[k];
        }
        has = true;
        if (m[k + 1] != NONE) {
          if (a.f) {
            emit(m[k + 1], a.v);
          } else {
            pendVal[g] = a.v;
            pendIdx[g] = m[k + 1];
          }
        }
      }
    }

    i64 cnt = n - (wlo + (i64)g * C::GROUP);
    cnt = cnt < 0 ? 0 : (cnt > C::GROUP ? C::GROUP : cnt);
    P ts = acc_wave_scan<SS>(env, a, lane);
    P lanePre = acc_prev_lane(ts);  // exclusive prefix of the run inside its group (lane > 0)
    const int last = cnt > 0 ? (int)((cnt - 1) / V) : 0;
    P gt = acc_readlane(ts, last);
    P pre;
    if (acc_join<SS>(env, hasWaveTot, waveTot, lane > 0, lanePre, pre) && pendIdx[g] != NONE) {
      pendVal[g] = S::combine(env, pre.v, pendVal[g]);
      if (pre.f) {
        emit(pendIdx[g], pendVal[g]);
        pendIdx[g] = NONE;
      }
    }
    if (cnt > 0) {
      waveTot = hasWaveTot ? SS::combine(env, waveTot, gt) : gt;
      hasWaveTot = true;
    }
  }
  if (lane == 0) sh_wave[w] = waveTot;
  __syncthreads();

  // a wave has data only if all earlier waves are full, so validity follows from counts
  const i64 tcnt = n - tlo;
  const i64 perWave = (i64)G * C::GROUP;
  i64 wd = tcnt <= 0 ? 0 : (tcnt + perWave - 1) / perWave;
  const int wavesWithData = wd > ACC_SCAN_WAVES ? ACC_SCAN_WAVES : (int)wd;
  const bool successors = tile + 1 < p.tiles;
  if (w == 0) {
    P t = sh_wave[lane < ACC_SCAN_WAVES ? lane : 0];
    t = acc_wave_scan<SS>(env, t, lane);
    if (lane < ACC_SCAN_WAVES) sh_wave[lane] = t;
    if (lane == wavesWithData - 1 && tile > 0 && successors) acc_publish<P>(p.desc + tile * W, t, p.epoch, 1);
  }
  __syncthreads();

  P excl;
  bool hasExcl = false;
  if (tile > 0) hasExcl = acc_lookback<SS>(env, p.desc, tile, p.epoch, excl);  // valid in thread 0
  if (threadIdx.x == 0) {
    if (successors && wavesWithData > 0) {
      P inc;
      acc_join<SS>(env, hasExcl, excl, true, sh_wave[wavesWithData - 1], inc);
      acc_publish<P>(p.desc + tile * W, inc, p.epoch, 2);
    }
    sh_excl = excl;
    sh_has_excl = hasExcl ? 1 : 0;
  }
  __syncthreads();

  // ends still pending have seen no head since the start of the tile
  P base;
  const bool hasWavePre = w > 0 && w <= wavesWithData;
  P wavePre = sh_wave[w > 0 ? w - 1 : 0];
  const bool hasBase = acc_join<SS>(env, sh_has_excl != 0, sh_excl, hasWavePre, wavePre, base);
#pragma unroll
  for (int g = 0; g < G; ++g)
    if (pendIdx[g] != NONE) emit(pendIdx[g], hasBase ? S::combine(env, base.v, pendVal[g]) : pendVal[g]);
}
