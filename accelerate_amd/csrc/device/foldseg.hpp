// FoldSeg / Fold1Seg skeleton (foldSegOp, Interpreter.hs:390-424): per outer row, segment
// s reduces the elements [offs[s], offs[s+1]) of the row, seeded once with z; an empty
// segment yields z.  The node receives offsets (Prelude.hs:710-717), not lengths.
//
// Load balance does not depend on segment lengths: the rows are laid end to end into one
// stream of rows*n elements which is cut into equal tiles, and a tile reduces its elements
// as (head flag, value) pairs under
//     (fa, a) (+) (fb, b) = fb ? (1, b) : (fa, a (+) b)
// which is associative whenever (+) is.  Tiles do not wait for each other: a tile publishes its
// carry (head seen, value since the last head) and the one segment end that no head of the tile
// precedes as tagged descriptor words.  The launch has a few workgroups more than tiles; they are
// dispatched last, and complete those ends from the carries of the tiles before (acc_foldseg_fix),
// most of which were published long before.  Measured on 2^27 values in 2^20 segments, against
// 111 us for the three launches scan, partition, tiles + completion: a tile that completes its own
// end at its close, by looking back itself, keeps its slot on the CU for a further round trip to
// memory (+10 us and more); the borders numbered by workgroups in front of the tiles of the same launch
// and read by the tiles as tagged words cost every tile a slower first load and a barrier
// (+3 us); the borders left by the scan that produces the offsets, as it stores them, lengthen
// that scan, whose few hundred workgroups are one dependent chain each, by as much as the
// partition kernel takes (8.5 -> 13.7 us).
//
// Boundaries: row r contributes S+1 boundaries at stream positions r*n + offs[s],
// s = 0..S (S segments per row).  Boundary number j = r*(S+1) + s starts segment (r, s)
// when s < S; what lies between boundary (r, S) and boundary (r+1, 0) belongs to no
// segment and is discarded.  acc_foldseg_partition finds, for every tile border, how many
// boundaries lie before it, so a tile knows which boundaries fall inside it and marks them
// in LDS: sh_first[p] = first boundary at position p of the tile.  Empty segments (two equal
// consecutive offsets) get z from the partition kernel.

#ifndef ACC_FOLDSEG_STAGE
#define ACC_FOLDSEG_STAGE 1024  // segment results a tile collects in LDS before it writes them (a multiple of 32)
#endif

struct FoldSegParams {
  i64 rows;
  i64 n;       // elements per row
  i64 nseg;    // segments per row (S)
  i64 total;   // rows * n
  i64 tiles;   // >= 1
  i64* part;   // [tiles + 1]: boundaries before each tile border; part[tiles] = rows * (S + 1)
  u64* desc;   // [tiles] descriptors: a tile's carry, state 2 when the tile holds a head (or is the first), else 1
  u64 epoch;   // tag of this launch in the descriptors
  u64 spin_limit;  // polls after which a wait for a predecessor's carry gives up (reported as 3 through err)
  u32* err;       // host-visible word: 1 = "empty segment" (what the reference's boundsCheck reports)
};

// The carries as a scan sees them: the value since the tile's last head, combined in order; a
// carry whose tile holds a head ends the walk like an inclusive prefix does.
struct AccSegCarrySpec {
  typedef Spec::Env Env;
  typedef Spec::Elt Elt;
  enum { V = AccSegSpec<Spec>::V, G = AccSegSpec<Spec>::G };
  static constexpr bool kSeeded = false;
  ACC_DEV Elt combine(const Env& env, const Elt& a, const Elt& b) { return Spec::combine(env, a, b); }
  ACC_DEV Elt seed(const Env&) {
    Elt r_{};
    return r_;
  }
  ACC_DEV bool stops(const Elt&) { return false; }
};

ACC_DEV void acc_foldseg_publish(const FoldSegParams& p, i64 tile, const AccSegSpec<Spec>::Elt& carry) {
  acc_publish<Spec::Elt>(p.desc + tile * AccWords<Spec::Elt>::N, carry.v, p.epoch, carry.f || tile == 0 ? 2 : 1);
}

// A tile's pending end: boundary number and the tile's share of the value; state 2 when the tile
// has one, 1 when not.  The records follow the carries in the descriptor memory.
struct AccSegPend {
  Spec::Elt v;
  i64 j;
};
ACC_DEV u64* acc_foldseg_pend_desc(const FoldSegParams& p, i64 tile) {
  const i64 carries = (p.tiles * AccWords<Spec::Elt>::N + 1) & ~(i64)1;  // 16-byte aligned
  return p.desc + carries + tile * AccWords<AccSegPend>::N;
}
ACC_DEV void acc_foldseg_publish_pend(const FoldSegParams& p, i64 tile, bool has, i64 j, const Spec::Elt& v) {
  AccSegPend r{};
  if (has) {
    r.v = v;
    r.j = j;
  }
  acc_publish<AccSegPend>(acc_foldseg_pend_desc(p, tile), r, p.epoch, has ? 2 : 1);
}

// Completes the end at boundary j whose value so far is v, from the carries of the tiles before
// `tile`, 64 a step: called by a whole wave.  Those tiles were dispatched before the caller, so
// their carries arrive without its help; the wait is bounded all the same (acc_window).
ACC_DEV void acc_foldseg_pending(const Spec::Env& env, const Spec::Out& out, const FoldSegParams& p, i64 tile, i64 j, Spec::Elt v) {
  typedef Spec S;
  bool have = false;
  S::Elt run;
  i64 look = tile - 1;
  while (look >= 0) {
    S::Elt r;
    int nv;
    bool term;
    acc_window<AccSegCarrySpec>(env, p.desc, look, p.epoch, p.spin_limit, p.err, r, nv, term);
    if (nv > 0) {
      run = have ? S::combine(env, r, run) : r;
      have = true;
    }
    if (term) break;
    look -= ACC_WAVE;
  }
  if (acc_lane() != 0) return;
  if (have) v = S::combine(env, run, v);
  const i64 sp1 = p.nseg + 1;
  const i64 row = p.rows == 1 ? 0 : acc_quot(j, sp1), s = j - row * sp1;
  if (s == 0) return;  // what precedes a row's first boundary belongs to no segment
  S::store(out, row * p.nseg + s - 1, S::kSeeded ? S::combine(env, S::seed(env), v) : v);
}

// The workgroups behind the tiles: one lane per tile.  Nearly every pending end needs just the
// carry of the tile before it (that tile holds a head), which the lanes fetch side by side; an
// end whose segment began further back is walked by the whole wave.
ACC_DEV void acc_foldseg_fix(const Spec::Env& env, const Spec::Out& out, const FoldSegParams& p, i64 group) {
  typedef Spec S;
  enum { NP = AccWords<AccSegPend>::N, NC = AccWords<Spec::Elt>::N };
  const i64 t = group * (i64)ACC_SCAN_BLOCK + threadIdx.x;
  const bool valid = t < p.tiles;
  // the tile's record and the carry of the tile before it are asked for together: one trip to
  // memory for nearly every lane (each word validates itself, so the words may arrive singly)
  auto check = [&](const u64* x, int n) -> int {
    const u64 tag0 = x[0] >> 32;
    for (int q = 1; q < n; ++q)
      if ((x[q] >> 32) != tag0) return 0;
    if ((tag0 >> 2) != p.epoch) return 0;
    const int st = (int)(tag0 & 3);
    return st == 1 || st == 2 ? st : 0;
  };
  AccSegPend pr{};
  S::Elt c{};
  int st = valid ? 0 : 1, sc = 0;
  for (u64 polls = 0; valid; ) {
    u64 xa[NP], xb[NC];
    const u64* pd = acc_foldseg_pend_desc(p, t);
    const u64* cd = p.desc + (t > 0 ? t - 1 : 0) * NC;
#pragma unroll
    for (int q = 0; q < NP; ++q) xa[q] = __hip_atomic_load(pd + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int q = 0; q < NC; ++q) xb[q] = __hip_atomic_load(cd + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    st = check(xa, NP);
    sc = check(xb, NC);
    if (st == 1 || (st == 2 && (t == 0 || sc != 0))) {
      u32 wa[NP], wb[NC];
#pragma unroll
      for (int q = 0; q < NP; ++q) wa[q] = (u32)xa[q];
#pragma unroll
      for (int q = 0; q < NC; ++q) wb[q] = (u32)xb[q];
      pr = acc_from_words<AccSegPend>(wa);
      c = acc_from_words<S::Elt>(wb);
      break;
    }
    if (++polls >= p.spin_limit) {
      __hip_atomic_store(p.err, 3u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      st = 1;
      break;
    }
    __builtin_amdgcn_s_sleep(32);  // the last tiles are still at work: ask again in a microsecond
  }
  const bool has = st == 2;
  bool done = !has || t == 0;
  S::Elt v = pr.v;
  if (has && t > 0) {
    v = S::combine(env, c, v);
    done = sc == 2;
  }
  if (has && done) {
    const i64 sp1 = p.nseg + 1;
    const i64 row = p.rows == 1 ? 0 : acc_quot(pr.j, sp1), s = pr.j - row * sp1;
    if (s != 0) S::store(out, row * p.nseg + s - 1, S::kSeeded ? S::combine(env, S::seed(env), v) : v);
  }
  u64 m = __ballot(has && !done);
  while (m) {
    const int src = __builtin_ctzll(m);
    m &= m - 1;
    acc_foldseg_pending(env, out, p, acc_shfl(t, src) - 1, acc_shfl(pr.j, src), acc_shfl(v, src));
  }
}

// part[t] = number of boundaries that lie before position t * TILE of the stream.  One
// thread per boundary j: the borders t * TILE in (position of boundary j-1, position of
// boundary j] have exactly j boundaries before them.  The offsets are read once, coalesced,
// and no thread waits for a chain of dependent loads as a search per border would.
// A range of more than a few borders (a segment that spans many tiles, the tail behind the
// last boundary) is filled by the whole wave, 64 borders a step.
ACC_DEV void acc_fill_borders(i64* part, bool valid, i64 lo, i64 hi, i64 value) {
  const int lane = acc_lane();
  const bool big = valid && hi - lo >= 4;
  if (valid && !big)
    for (i64 t = lo; t <= hi; ++t) part[t] = value;
  u64 m = __ballot(big);
  while (m) {
    const int src = __builtin_ctzll(m);
    m &= m - 1;
    const i64 l = acc_shfl(lo, src), h = acc_shfl(hi, src), v = acc_shfl(value, src);
    for (i64 t = l + lane; t <= h; t += ACC_WAVE) part[t] = v;
  }
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_foldseg_partition(Spec::Env env, Spec::Out out, FoldSegParams p) {
  typedef AccScanCfg<AccSegSpec<Spec>> C;
  const i64 sp1 = p.nseg + 1;
  const i64 nb = p.rows * sp1;
  const i64 j = (i64)blockIdx.x * ACC_BLOCK + threadIdx.x;
  const bool valid = j < nb;
  i64 lo = 0, hi = -1;  // borders in (previous boundary, this boundary]
  if (valid) {
    const i64 row = p.rows == 1 ? 0 : acc_quot(j, sp1), s = j - row * sp1;
    const i64 pos = row * p.n + Spec::seg_at(env, s);
    if (j > 0) {
      const i64 prev = s > 0 ? row * p.n + Spec::seg_at(env, s - 1) : (row - 1) * p.n + Spec::seg_at(env, p.nseg);
      lo = prev < 0 ? 0 : prev / (i64)C::TILE + 1;
      // an empty segment yields z; it is written here, where every boundary has a thread of its own
      if (Spec::kSeeded && s > 0 && prev == pos) Spec::store(out, row * p.nseg + s - 1, Spec::seed(env));
      // foldSeg: offsets must not decrease; fold1Seg: every segment needs an element
      // (Interpreter.hs:407, 424)
      if (s > 0 && (prev > pos || (!Spec::kSeeded && prev == pos)))
        __hip_atomic_store(p.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    hi = pos < 0 ? -1 : pos / (i64)C::TILE;
    if (hi > p.tiles - 1) hi = p.tiles - 1;
  }
  acc_fill_borders(p.part, valid, lo, hi, j);
  // the borders behind the last boundary, and the end marker
  const bool last = valid && j == nb - 1;
  acc_fill_borders(p.part, last, (hi < lo - 1 ? lo - 1 : hi) + 1, p.tiles - 1, nb);
  if (last) p.part[p.tiles] = nb;
}

// One tile.  A lane owns, per group, a run of V consecutive elements and reduces it in
// order, starting afresh at every head.  A segment end whose segment began inside the run
// is written at once; the first end of a run that has seen no head yet still lacks what
// precedes the run, and is kept as the run's pending end (at most one per run).  The runs'
// aggregates (head seen, value since the last head) go through the ordered wave scan and
// the wave totals through LDS, exactly as in a plain scan, but only pending ends receive
// the prefix: a prefix that contains a head closes them inside the wave, the others wait
// for what the earlier waves of the tile contribute; the one end of a tile that no head of
// the tile precedes is left to the fix-up kernel together with the tile's carry.
//
// ONE_ROW: the stream is a single row, so boundary j is segment boundary j of that row and
// no division is needed.  FULL: the tile lies completely inside the stream.
template <bool ONE_ROW, bool FULL>
ACC_DEV void acc_foldseg_tile(const Spec::Env& env, const Spec::Out& out, const FoldSegParams& p, unsigned short* sh_first,
                              AccSegSpec<Spec>::Elt* sh_wave, AccSegSpec<Spec>::Elt* sh_rake, Spec::Elt& sh_pend, int& sh_pend_at,
                              Spec::Elt* sh_stage, u32* sh_staged) {
  typedef Spec S;
  typedef AccSegSpec<Spec> SS;
  typedef AccScanCfg<SS> C;
  typedef SS::Elt P;
  const int V = C::V, G = C::G;
  // marks are 16 bits: the boundary number relative to the tile's first, NONE, or LOOKUP
  // (a boundary sits here, its number must be searched: crowded tiles only)
  const int NONE = 0xffff, LOOKUP = 0xfffe;
  const int NOPEND = 0x7fffffff;
  const i64 tile = blockIdx.x;
  const i64 tlo = tile * (i64)C::TILE;
  const i64 sp1 = p.nseg + 1;
  // (clamped: offsets that do not ascend leave entries of part unwritten)
  const i64 nb = p.rows * sp1;
  i64 j0 = p.part[tile], j1 = p.part[tile + 1];
  j0 = j0 < 0 ? 0 : (j0 > nb ? nb : j0);
  j1 = j1 < j0 ? j0 : (j1 > nb ? nb : j1);
  const int lane = acc_lane(), w = acc_wave();
  const i64 n = p.total;
  const i64 wlo = tlo + (i64)w * G * C::GROUP;
  // all loads of the tile are issued first: they depend on nothing but the tile number, and
  // could not be moved past the stores further down
  S::Elt x[C::G][C::V];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
    if (FULL) {
#pragma unroll
      for (int k = 0; k < V; ++k) x[g][k] = S::in_linear(env, t0 + k);
    } else {
#pragma unroll
      for (int k = 0; k < V; ++k)
        if (t0 + k < n) x[g][k] = S::in_linear(env, t0 + k);
    }
  }
  // Boundaries are marked four per thread and step so that their offsets are loaded
  // together; the loads of the first step are issued before the marks are cleared, so that
  // they travel while the workgroup waits at the barrier.  A boundary at the same position
  // as its predecessor (an empty segment before it, or the previous row's last boundary) is
  // not the first at its position and is skipped, so every mark has exactly one writer.  The first boundary of the next tile is looked at too: it may sit exactly on this
  // tile's upper border, where it ends a segment of this tile.
  const bool crowded = j1 - j0 > (4 * (i64)C::TILE < 65000 ? 4 * (i64)C::TILE : 65000);
  const i64 jend = tile + 1 < p.tiles && j1 < nb ? j1 + 1 : j1;
  i64 row[4], sg[4], o[4], before[4];
  auto loadBatch = [&](i64 jb) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const i64 j = jb + (i64)u * ACC_SCAN_BLOCK + threadIdx.x;
      if (j < jend) {
        row[u] = ONE_ROW ? 0 : acc_quot(j, sp1);
        sg[u] = j - row[u] * sp1;
        o[u] = S::seg_at(env, sg[u]);
        // position of the boundary before it, relative to this row's start
        before[u] = sg[u] > 0 ? S::seg_at(env, sg[u] - 1) : (row[u] > 0 ? S::seg_at(env, p.nseg) - p.n : -1);
      }
    }
  };
  auto markBatch = [&](i64 jb) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const i64 j = jb + (i64)u * ACC_SCAN_BLOCK + threadIdx.x;
      if (j < jend && o[u] != before[u]) {
        const i64 rel = row[u] * p.n + o[u] - tlo;
        if (rel >= 0 && rel <= C::TILE) sh_first[rel] = (unsigned short)(j - j0);  // the only writer of this mark
      }
    }
  };
  if (!crowded) loadBatch(j0);
  for (int i = threadIdx.x; i < C::TILE / 8 + 1; i += ACC_SCAN_BLOCK)
    reinterpret_cast<int4*>(sh_first)[i] = make_int4(-1, -1, -1, -1);
  for (int i = threadIdx.x; i < ACC_FOLDSEG_STAGE / 32; i += ACC_SCAN_BLOCK) sh_staged[i] = 0u;
  __syncthreads();
  if (crowded) {
    // far more boundaries than positions (long runs of empty segments): every position
    // looks for its first boundary by binary search instead
    auto position = [&](i64 j) {
      const i64 r = ONE_ROW ? 0 : acc_quot(j, sp1);
      return r * p.n + S::seg_at(env, j - r * sp1);
    };
    for (int q = threadIdx.x; q <= C::TILE; q += ACC_SCAN_BLOCK) {
      i64 a = j0, b = jend;  // first boundary at a position >= tlo + q
      while (a < b) {
        const i64 mid = (a + b) >> 1;
        if (position(mid) < tlo + q) a = mid + 1;
        else b = mid;
      }
      if (a < jend && position(a) == tlo + q) sh_first[q] = (unsigned short)LOOKUP;
    }
  } else {
    markBatch(j0);
    for (i64 jb = j0 + (i64)ACC_SCAN_BLOCK * 4; jb < jend; jb += (i64)ACC_SCAN_BLOCK * 4) {
      loadBatch(jb);
      markBatch(jb);
    }
  }
  __syncthreads();

  // boundary number (relative to j0) behind the mark found at position pos of the stream
  auto resolve = [&](int mark, i64 pos) -> int {
    if (mark != LOOKUP) return mark;
    i64 a = j0, b = j1 + 1 < nb ? j1 + 1 : nb;
    while (a < b) {
      const i64 mid = (a + b) >> 1;
      const i64 r = ONE_ROW ? 0 : acc_quot(mid, sp1);
      if (r * p.n + S::seg_at(env, mid - r * sp1) < pos) a = mid + 1;
      else b = mid;
    }
    return (int)(a - j0);
  };
  // the segment that ends where boundary j0 + idx sits: written to the result
  auto write = [&](int idx, const S::Elt& v) {
    const i64 j = j0 + idx;
    const i64 row = ONE_ROW ? 0 : acc_quot(j, sp1), s = j - row * sp1;
    if (s == 0) return;  // what precedes a row's first boundary belongs to no segment
    S::store(out, row * p.nseg + s - 1, S::kSeeded ? S::combine(env, S::seed(env), v) : v);
  };
  // A finished segment waits in LDS under its boundary's number: neighbouring boundaries are
  // neighbouring segments, so the workgroup writes them to the result side by side at the end,
  // instead of one scattered store (and one index division) where each segment happens to
  // end.  Boundaries beyond the staging area (a tile crowded with short segments) are written at once.
  auto emit = [&](int idx, const S::Elt& v) {
    if (idx < ACC_FOLDSEG_STAGE) {
      sh_stage[idx] = v;
      (void)__hip_atomic_fetch_or(&sh_staged[idx >> 5], 1u << (idx & 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    } else {
      write(idx, v);
    }
  };

  P waveTot;
  bool hasWaveTot = false;
  S::Elt pendVal[C::G];
  int pendIdx[C::G];
  P agg[C::G];
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
    // a run past the end of the stream stands for a real element without a head: the raking
    // below applies the combination function to every run, and that function may only ever
    // see values of the array
    if (!FULL && c == 0 && n > 0) a.v = S::in_linear(env, tlo);
    bool has = false;
    pendIdx[g] = NOPEND;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      if (FULL || k < c) {
        if (m[k] != NONE) {
          a.v = e[k];
          a.f = 1u;
        } else {
          a.v = has ? S::combine(env, a.v, e[k]) : e[k];
        }
        has = true;
        if (m[k + 1] != NONE) {
          const int idx = resolve(m[k + 1], t0 + k + 1);
          if (a.f) {
            emit(idx, a.v);
          } else {
            pendVal[g] = a.v;
            pendIdx[g] = idx;
          }
        }
      }
    }

    agg[g] = a;
  }
  // exclusive prefixes of the runs' aggregates inside the wave, by raking (acc_rake); a prefix
  // that contains a head closes a pending end here
  {
    i64 wcnt = n - wlo;
    wcnt = wcnt < 0 ? 0 : (wcnt > (i64)G * C::GROUP ? (i64)G * C::GROUP : wcnt);
    const int entries = (int)((wcnt + V - 1) / V);
    P pre[C::G];
    acc_rake<SS, C::G>(env, sh_rake + w * (ACC_WAVE * (C::G + 1) + 1), agg, lane, entries, pre, waveTot);
    hasWaveTot = entries > 0;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g * ACC_WAVE + lane > 0 && pendIdx[g] != NOPEND) {
        pendVal[g] = S::combine(env, pre[g].v, pendVal[g]);
        if (pre[g].f) {
          emit(pendIdx[g], pendVal[g]);
          pendIdx[g] = NOPEND;
        }
      }
    }
  }
  if (lane == 0) sh_wave[w] = waveTot;
  if (threadIdx.x == 0) sh_pend_at = NOPEND;
  __syncthreads();

  // a wave has data only if all earlier waves are full, so validity follows from counts
  const i64 tcnt = n - tlo;
  const i64 perWave = (i64)G * C::GROUP;
  i64 wd = tcnt <= 0 ? 0 : (tcnt + perWave - 1) / perWave;
  const int wavesWithData = wd > ACC_SCAN_WAVES ? ACC_SCAN_WAVES : (int)wd;
  if (w == 0) {
    P t = sh_wave[lane < ACC_SCAN_WAVES ? lane : 0];
    t = acc_wave_scan<SS>(env, t, lane);
    if (lane < ACC_SCAN_WAVES) sh_wave[lane] = t;
    if (lane == wavesWithData - 1) acc_foldseg_publish(p, tile, t);
  }
  __syncthreads();

  // an end still pending has seen no head since the start of its wave; if none of the
  // earlier waves has one either it is the tile's pending end (there is at most one)
  const bool hasWavePre = w > 0 && w <= wavesWithData;
  const P wavePre = sh_wave[w > 0 ? w - 1 : 0];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (pendIdx[g] != NOPEND) {
      const S::Elt v = hasWavePre ? S::combine(env, wavePre.v, pendVal[g]) : pendVal[g];
      if (hasWavePre && wavePre.f) {
        emit(pendIdx[g], v);
      } else {
        sh_pend_at = pendIdx[g];
        sh_pend = v;
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) acc_foldseg_publish_pend(p, tile, sh_pend_at != NOPEND, j0 + sh_pend_at, sh_pend);
  // the staged segments, in the order of their boundaries
  {
    const i64 inTile = jend - j0 + 1;  // boundary numbers the tile can have met, relative to j0
    const int top = inTile < ACC_FOLDSEG_STAGE ? (int)inTile : ACC_FOLDSEG_STAGE;
    for (int idx = threadIdx.x; idx < top; idx += ACC_SCAN_BLOCK)
      if ((sh_staged[idx >> 5] >> (idx & 31)) & 1u) write(idx, sh_stage[idx]);
  }
}

// The same tile for the ordinary case (at most 4 boundaries per position on average, so that
// every boundary of the tile has a 16-bit number), arranged so that the pass over the elements
// has no branches: next to the marks a bitmap says which positions hold a boundary, a run reads
// its 9 bits at once and computes, with selects only, the running value after each of its
// elements.  Segment ends are dealt with once, after the prefix of every run inside the tile is
// known (raking inside the wave, wave totals through LDS): a lane that has none skips them
// together, an end reads its boundary's number from the marks then, and its value is the
// running value, preceded by the prefix unless the run itself holds the segment's head.
// the tile's elements: lane l of wave w holds, per group g, the V consecutive elements from
// position tile * TILE + ((w * G + g) * 64 + l) * V on
template <bool FULL>
ACC_DEV void acc_foldseg_load(const Spec::Env& env, i64 tile, i64 n,
                              Spec::Elt (&x)[AccScanCfg<AccSegSpec<Spec>>::G][AccScanCfg<AccSegSpec<Spec>>::V]) {
  typedef AccScanCfg<AccSegSpec<Spec>> C;
  const i64 wlo = tile * (i64)C::TILE + (i64)acc_wave() * C::G * C::GROUP;
#pragma unroll
  for (int g = 0; g < C::G; ++g) {
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + acc_lane()) * C::V;
    if (FULL) {
#pragma unroll
      for (int k = 0; k < C::V; ++k) x[g][k] = Spec::in_linear(env, t0 + k);
    } else {
#pragma unroll
      for (int k = 0; k < C::V; ++k)
        if (t0 + k < n) x[g][k] = Spec::in_linear(env, t0 + k);
    }
  }
}

template <bool ONE_ROW, bool FULL>
ACC_DEV void acc_foldseg_tile_fast(const Spec::Env& env, const Spec::Out& out, const FoldSegParams& p, i64 j0, i64 j1,
                                   unsigned short* sh_first, u32* sh_head, AccSegSpec<Spec>::Elt* sh_wave,
                                   AccSegSpec<Spec>::Elt* sh_rake, Spec::Elt& sh_pend, int& sh_pend_at, Spec::Elt* sh_stage,
                                   u32* sh_staged) {
  typedef Spec S;
  typedef AccSegSpec<Spec> SS;
  typedef AccScanCfg<SS> C;
  typedef SS::Elt P;
  const int V = C::V, G = C::G;
  static_assert(C::V <= 24, "a run's boundary bits are taken from two words of the bitmap");
  const int NOPEND = 0x7fffffff;
  const i64 tile = blockIdx.x;
  const i64 tlo = tile * (i64)C::TILE;
  const i64 sp1 = p.nseg + 1;
  const i64 nb = p.rows * sp1;
  const int lane = acc_lane(), w = acc_wave();
  const i64 n = p.total;
  const i64 wlo = tlo + (i64)w * G * C::GROUP;
  // marks and bitmap: four boundaries per thread and step, their offsets loaded together; a
  // boundary at the position of its predecessor is not the first there and is skipped, so every
  // mark has one writer.  The next tile's first boundary is looked at too: it may sit on this
  // tile's upper border, where it ends a segment of this tile.
  const i64 jend = tile + 1 < p.tiles && j1 < nb ? j1 + 1 : j1;
  i64 row[4], sg[4], o[4], before[4];
  auto loadBatch = [&](i64 jb) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const i64 j = jb + (i64)u * ACC_SCAN_BLOCK + threadIdx.x;
      if (j < jend) {
        row[u] = ONE_ROW ? 0 : acc_quot(j, sp1);
        sg[u] = j - row[u] * sp1;
        o[u] = S::seg_at(env, sg[u]);
        before[u] = sg[u] > 0 ? S::seg_at(env, sg[u] - 1) : (row[u] > 0 ? S::seg_at(env, p.nseg) - p.n : -1);
      }
    }
  };
  auto markBatch = [&](i64 jb) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const i64 j = jb + (i64)u * ACC_SCAN_BLOCK + threadIdx.x;
      if (j < jend && o[u] != before[u]) {
        const i64 rel = row[u] * p.n + o[u] - tlo;
        if (rel >= 0 && rel <= C::TILE) {
          sh_first[rel] = (unsigned short)(j - j0);
          (void)__hip_atomic_fetch_or(&sh_head[rel >> 5], 1u << (rel & 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
  };
  // The offsets of the first boundaries are asked for before the elements: a wave's loads
  // come back in the order they were issued, and the marks, which everything else waits for,
  // would otherwise queue behind the tile's 32 KiB of elements.
  loadBatch(j0);
  S::Elt x[C::G][C::V];
  acc_foldseg_load<FULL>(env, tile, n, x);
  for (int i = threadIdx.x; i < C::TILE / 32 + 2; i += ACC_SCAN_BLOCK) sh_head[i] = 0u;
  for (int i = threadIdx.x; i < ACC_FOLDSEG_STAGE / 32; i += ACC_SCAN_BLOCK) sh_staged[i] = 0u;
  if (threadIdx.x == 0) sh_pend_at = NOPEND;
  __syncthreads();
  markBatch(j0);
  for (i64 jb = j0 + (i64)ACC_SCAN_BLOCK * 4; jb < jend; jb += (i64)ACC_SCAN_BLOCK * 4) {
    loadBatch(jb);
    markBatch(jb);
  }
  __syncthreads();

  // the pass over the elements: s[g][k] = value of the segment piece that ends with element k of
  // the run (starting afresh at every head), bits[g] = boundaries at the run's V + 1 positions
  u32 bits[C::G];
  P agg[C::G];
  S::Elt firstEnd[C::G];  // running value at the run's first boundary that lies behind an element
#pragma unroll
  for (int g = 0; g < G; ++g) {  // (all reads of the bitmap in flight together)
    const int rel0 = (int)(wlo - tlo) + (g * ACC_WAVE + lane) * V;
    const u32 w0 = sh_head[rel0 >> 5], w1 = sh_head[(rel0 >> 5) + 1];
    bits[g] = (u32)((((u64)w1 << 32) | (u64)w0) >> (rel0 & 31)) & ((2u << V) - 1u);
  }
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const i64 t0 = wlo + ((i64)g * ACC_WAVE + lane) * V;
    const u32 b = bits[g];
    i64 c = n - t0;
    c = c < 0 ? 0 : (c > V ? V : c);
    S::Elt* e = x[g];
    if (!FULL && c == 0) {  // a run past the end stands for a real element (none exists in an empty stream)
      S::Elt none{};
      e[0] = n > 0 ? S::in_linear(env, tlo) : none;
    }
    // Most of a stream of long segments has no boundary for hundreds of elements: when none of
    // the wave's runs of this group has one, a run is a plain fold (wave-uniform test, so the
    // branch costs no divergence) and its running values are never looked at.
    if (FULL && __ballot(b != 0u) == 0ull) {
      S::Elt v = e[0];
#pragma unroll
      for (int k = 1; k < V; ++k) v = S::combine(env, v, e[k]);
      agg[g].v = v;
      agg[g].f = 0u;
      firstEnd[g] = v;
    } else {
#pragma unroll
      for (int k = 1; k < V; ++k) {
        if (FULL || k < c) {
          const S::Elt joined = S::combine(env, e[k - 1], e[k]);
          if (!((b >> k) & 1u)) e[k] = joined;  // a head starts afresh
        } else {
          e[k] = e[k - 1];
        }
      }
      agg[g].v = e[V - 1];
      agg[g].f = (b & ((1u << V) - 1u)) != 0u ? 1u : 0u;
      const u32 eb = b >> 1, lowest = eb & (0u - eb);  // the first end, one bit
      S::Elt fe = e[0];
#pragma unroll
      for (int k = 1; k < V; ++k)
        if ((lowest >> k) & 1u) fe = e[k];
      firstEnd[g] = fe;
    }
  }
  // prefixes of the runs inside the wave by raking, wave totals through LDS
  P pre[C::G], waveTot;
  {
    i64 wcnt = n - wlo;
    wcnt = wcnt < 0 ? 0 : (wcnt > (i64)G * C::GROUP ? (i64)G * C::GROUP : wcnt);
    const int entries = (int)((wcnt + V - 1) / V);
    waveTot = agg[0];
    acc_rake<SS, C::G>(env, sh_rake + w * (ACC_WAVE * (C::G + 1) + 1), agg, lane, entries, pre, waveTot);
  }
  if (lane == 0) sh_wave[w] = waveTot;
  __syncthreads();
  const i64 tcnt = n - tlo;
  const i64 perWave = (i64)G * C::GROUP;
  i64 wd = tcnt <= 0 ? 0 : (tcnt + perWave - 1) / perWave;
  const int wavesWithData = wd > ACC_SCAN_WAVES ? ACC_SCAN_WAVES : (int)wd;
  // every wave joins the totals of the waves in front of it by itself (a few combinations,
  // the same in all lanes): a second barrier with one wave scanning in between costs more
  const bool hasWavePre = w > 0 && w <= wavesWithData;
  P wavePre = sh_wave[0];
  for (int i = 1; i < w; ++i) wavePre = SS::combine(env, wavePre, sh_wave[i]);
  if (w == wavesWithData - 1 && lane == 0) acc_foldseg_publish(p, tile, w > 0 ? SS::combine(env, wavePre, waveTot) : waveTot);

  auto write = [&](int idx, const S::Elt& v) {
    const i64 j = j0 + idx;
    const i64 row = ONE_ROW ? 0 : acc_quot(j, sp1), s = j - row * sp1;
    if (s == 0) return;  // what precedes a row's first boundary belongs to no segment
    S::store(out, row * p.nseg + s - 1, S::kSeeded ? S::combine(env, S::seed(env), v) : v);
  };
  // The segment ends.  Nearly every wave has, in each of its groups, a few lanes whose run
  // holds a boundary, and hardly any lane has two: the first end of every run is therefore
  // prepared by all lanes without a branch (the G reads of boundary numbers are in flight
  // together; a lane without an end reads the tile's first mark and ignores it), and what is
  // rare -- further ends in the same run, an end nothing of the tile precedes, a boundary
  // number beyond the staging area -- goes through a branch afterwards.
  int endIdx[C::G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const u32 eb = bits[g] >> 1;
    const int rel0 = (int)(wlo - tlo) + (g * ACC_WAVE + lane) * V;
    endIdx[g] = sh_first[eb != 0u ? rel0 + __builtin_ctz(eb) + 1 : 0];
  }
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const u32 b = bits[g], eb = b >> 1;
    const bool has = eb != 0u;
    // everything of the tile in front of the run
    P fore;
    const bool hasFore = acc_join<SS>(env, hasWavePre, wavePre, g * ACC_WAVE + lane > 0, pre[g], fore);
    const bool local = (b & 1u) != 0u;  // the segment's head is the run's first position
    const S::Elt v = !local && hasFore ? S::combine(env, fore.v, firstEnd[g]) : firstEnd[g];
    const bool finished = local || (hasFore && fore.f);
    const int idx = endIdx[g];
    // finished: it waits in LDS under its boundary's number and is written with its neighbours
    const bool stage = has && finished && idx < ACC_FOLDSEG_STAGE;
    if (stage) {
      sh_stage[idx] = v;
      (void)__hip_atomic_fetch_or(&sh_staged[idx >> 5], 1u << (idx & 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (has && (!stage || (eb & (eb - 1u)) != 0u)) {
      if (!stage) {
        if (finished) {
          write(idx, v);  // beyond the staging area: written at once
        } else {
          sh_pend_at = idx;  // no head of the tile precedes it: at most one such end per tile
          sh_pend = v;
        }
      }
      // the run's further ends: their segments began in the run
      const int rel0 = (int)(wlo - tlo) + (g * ACC_WAVE + lane) * V;
      const u32 rest = eb & (eb - 1u);
#pragma unroll
      for (int k = 1; k < V; ++k) {
        if ((rest >> k) & 1u) {
          const int idx2 = sh_first[rel0 + k + 1];
          if (idx2 < ACC_FOLDSEG_STAGE) {
            sh_stage[idx2] = x[g][k];
            (void)__hip_atomic_fetch_or(&sh_staged[idx2 >> 5], 1u << (idx2 & 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          } else {
            write(idx2, x[g][k]);
          }
        }
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) acc_foldseg_publish_pend(p, tile, sh_pend_at != NOPEND, j0 + sh_pend_at, sh_pend);
  {
    const i64 inTile = jend - j0 + 1;
    const int top = inTile < ACC_FOLDSEG_STAGE ? (int)inTile : ACC_FOLDSEG_STAGE;
    for (int idx = threadIdx.x; idx < top; idx += ACC_SCAN_BLOCK)
      if ((sh_staged[idx >> 5] >> (idx & 31)) & 1u) write(idx, sh_stage[idx]);
  }
}

extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK)
acc_foldseg(Spec::Env env, Spec::Out out, FoldSegParams p) {
  typedef AccScanCfg<AccSegSpec<Spec>> C;
  // sh_first[q]: first boundary (relative to the tile's first) at position q of the tile
  __shared__ __attribute__((aligned(16))) unsigned short sh_first[C::TILE + 8];
  __shared__ u32 sh_head[C::TILE / 32 + 2];
  __shared__ AccSegSpec<Spec>::Elt sh_wave[ACC_SCAN_WAVES];
  __shared__ AccSegSpec<Spec>::Elt sh_rake[ACC_SCAN_WAVES * (ACC_WAVE * (C::G + 1) + 1)];
  __shared__ Spec::Elt sh_pend;
  __shared__ int sh_pend_at;
  __shared__ Spec::Elt sh_stage[ACC_FOLDSEG_STAGE];
  __shared__ u32 sh_staged[ACC_FOLDSEG_STAGE / 32];
  if ((i64)blockIdx.x >= p.tiles) {
    acc_foldseg_fix(env, out, p, (i64)blockIdx.x - p.tiles);
    return;
  }
  const bool full = ((i64)blockIdx.x + 1) * (i64)C::TILE <= p.total;
  // (clamped: offsets that do not ascend leave entries of part unwritten)
  const i64 nb = p.rows * (p.nseg + 1);
  i64 j0 = p.part[blockIdx.x], j1 = p.part[blockIdx.x + 1];
  j0 = j0 < 0 ? 0 : (j0 > nb ? nb : j0);
  j1 = j1 < j0 ? j0 : (j1 > nb ? nb : j1);
  // far more boundaries than positions (long runs of empty segments): the tile that numbers
  // its boundaries by searching
  const bool crowded = j1 - j0 > (4 * (i64)C::TILE < 65000 ? 4 * (i64)C::TILE : 65000);
  if (crowded) {
    if (p.rows == 1) acc_foldseg_tile<true, false>(env, out, p, sh_first, sh_wave, sh_rake, sh_pend, sh_pend_at, sh_stage, sh_staged);
    else acc_foldseg_tile<false, false>(env, out, p, sh_first, sh_wave, sh_rake, sh_pend, sh_pend_at, sh_stage, sh_staged);
  } else if (p.rows == 1) {
    if (full) acc_foldseg_tile_fast<true, true>(env, out, p, j0, j1, sh_first, sh_head, sh_wave, sh_rake, sh_pend, sh_pend_at, sh_stage, sh_staged);
    else acc_foldseg_tile_fast<true, false>(env, out, p, j0, j1, sh_first, sh_head, sh_wave, sh_rake, sh_pend, sh_pend_at, sh_stage, sh_staged);
  } else {
    if (full) acc_foldseg_tile_fast<false, true>(env, out, p, j0, j1, sh_first, sh_head, sh_wave, sh_rake, sh_pend, sh_pend_at, sh_stage, sh_staged);
    else acc_foldseg_tile_fast<false, false>(env, out, p, j0, j1, sh_first, sh_head, sh_wave, sh_rake, sh_pend, sh_pend_at, sh_stage, sh_staged);
  }
}

// the same completion as a launch of its own (the knob that compares the two)
extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK)
acc_foldseg_fixup(Spec::Env env, Spec::Out out, FoldSegParams p) {
  acc_foldseg_fix(env, out, p, (i64)blockIdx.x);
}
