// Entry point of the scan skeleton: one workgroup per tile, tiles numbered by ticket in
// row-major (row, tile-in-row) order; the tile machinery lives in scan.hpp.

extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK, ACC_SCAN_MINWAVES)
acc_scan(Spec::Env env, Spec::Out out, Spec::Out tot, ScanParams p) {
  typedef Spec S;
  typedef S::Elt Elt;
  const int W = AccScanCfg<S>::W;
  // (no counter: the launch holds no more tiles than the device holds workgroups at a time)
  const i64 gtile = p.ticket ? acc_take_ticket(p.ticket, p.ticket_base) : (i64)blockIdx.x;
  // a ticket outside the launch means that the host's count of tickets is off: touch nothing
  if (gtile < 0 || gtile >= p.rows * p.tpr) {
    if (threadIdx.x == 0) __hip_atomic_store(p.err, 3u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    return;
  }
  const i64 row = gtile / p.tpr;
  const i64 tile = gtile - row * p.tpr;
  const i64 n = p.n;
  const i64 inBase = row * n;
  const i64 m = S::kKind == 1 ? n + 1 : n;  // entries per output row
  const i64 outBase = row * m;
  u64* rowDesc = p.desc + (u64)row * (u64)p.tpr * W;

  auto load = [&](i64 t) -> Elt { return S::in_linear(env, inBase + (S::kRight ? n - 1 - t : t)); };
  auto store = [&](i64 t, const Elt& y) {
    if (S::kKind == 0) {
      S::store(out, outBase + (S::kRight ? n - 1 - t : t), y);
    } else {
      const i64 u = t + 1;
      if (S::kKind == 2 && u == n) S::store(tot, row, y);
      else S::store(out, outBase + (S::kRight ? m - 1 - u : u), y);
    }
  };
  // the V consecutive values of a lane, moved with one wide request per leaf (a right scan
  // writes them in reverse).  scan' keeps the row's total apart: only the row's last tile can
  // hold it, the others need no test.
  auto storeRun = [&](i64 t0, const Elt* y) {
    const i64 shift = S::kKind == 0 ? 0 : 1;
    if (!S::kRight) {
      S::store_run(out, outBase + t0 + shift, y);
    } else {
      Elt z[S::V];
#pragma unroll
      for (int k = 0; k < S::V; ++k) z[k] = y[S::V - 1 - k];
      S::store_run(out, outBase + (m - 1 - shift) - (t0 + S::V - 1), z);
    }
  };
  acc_scan_tile<S>(env, rowDesc, p.tpr, tile, n, p.epoch, p.spin_limit, p.err, load, store, storeRun, S::kKind != 2 || tile + 1 < p.tpr,
                   p.rows * p.tpr >= ACC_SCAN_SETTLE_TILES);

  if (S::kKind != 0 && tile == 0 && threadIdx.x == 0) {
    Elt z = S::seed(env);
    if (S::kKind == 2 && n == 0) S::store(tot, row, z);
    else S::store(out, outBase + (S::kRight ? m - 1 : 0), z);
  }
}

// Rows of at most half a tile: a workgroup scans rpt whole rows at once (acc_rows_tile).
struct ScanRowsParams {
  i64 rows;
  i64 n;    // 1 <= n, rpt * n <= TILE
  i64 rpt;  // rows per workgroup
};

// the rows kernel's own tile size (values carry a head flag there: half the elements per lane)
#ifndef ACC_ROWS_G
#define ACC_ROWS_G Spec::G
#endif
struct AccRowsSpec : Spec {
  static constexpr int G = ACC_ROWS_G;
};

extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK, ACC_SCAN_MINWAVES)
acc_scan_rows(Spec::Env env, Spec::Out out, Spec::Out tot, ScanRowsParams p) {
  typedef Spec S;
  typedef S::Elt Elt;
  const i64 row0 = (i64)blockIdx.x * p.rpt;
  const i64 nrows = p.rows - row0 < p.rpt ? p.rows - row0 : p.rpt;
  const int n = (int)p.n;
  const i64 m = S::kKind == 1 ? p.n + 1 : p.n;  // entries per output row
  auto load = [&](int idx, int r, int t) -> Elt {
    Elt v = S::in_linear(env, S::kRight ? (row0 + r) * p.n + (n - 1 - t) : row0 * p.n + idx);
    if (S::kSeeded && t == 0) v = S::combine(env, S::seed(env), v);
    return v;
  };
  auto store = [&](int idx, int r, int t, const Elt& y) {
    const i64 row = row0 + r;
    if (S::kKind == 0) {
      S::store(out, S::kRight ? row * p.n + (n - 1 - t) : row0 * p.n + idx, y);
    } else {
      const i64 outBase = row * m;
      if (t == 0) S::store(out, outBase + (S::kRight ? m - 1 : 0), S::seed(env));
      const i64 u = (i64)t + 1;
      if (S::kKind == 2 && u == p.n) S::store(tot, row, y);
      else S::store(out, outBase + (S::kRight ? m - 1 - u : u), y);
    }
  };
  acc_rows_tile<AccRowsSpec>(env, (int)(nrows * p.n), n, load, store);
}
