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

extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK)
acc_foldseg(Spec::Env env, Spec::Out out, FoldSegParams p) {
  typedef Spec S;
  typedef AccSegSpec<Spec> SS;
  typedef AccScanCfg<SS> C;
  const int NONE = 0x7fffffff;
  __shared__ int sh_first[C::TILE + 1];

  const i64 tile = acc_take_ticket(p.ticket, p.ticket_base);
  const i64 tlo = tile * (i64)C::TILE;
  const i64 sp1 = p.nseg + 1;
  const i64 j0 = p.part[tile], j1 = p.part[tile + 1];
  for (int i = threadIdx.x; i <= C::TILE; i += ACC_SCAN_BLOCK) sh_first[i] = NONE;
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

  auto load = [&](i64 t) -> SS::Elt {
    SS::Elt e;
    e.v = S::in_linear(env, t);
    e.f = sh_first[t - tlo] != NONE ? 1u : 0u;
    return e;
  };
  auto store = [&](i64 t, const SS::Elt& y) {
    const int nxt = sh_first[t - tlo + 1];
    if (nxt == NONE) return;
    const i64 j = j0 + nxt;
    const i64 row = p.rows == 1 ? 0 : acc_quot(j, sp1), s = j - row * sp1;
    if (s == 0) return;  // what precedes a row's first boundary belongs to no segment
    S::store(out, row * p.nseg + s - 1, S::kSeeded ? S::combine(env, S::seed(env), y.v) : y.v);
  };
  acc_scan_tile<SS>(env, p.desc, p.tiles, tile, p.total, p.epoch, load, store);
}
