// Rank-2 stencil skeleton with LDS halo tiles (stencilOp, Interpreter.hs:637-649; taps as
// stencilAccess builds them, :670-794; out-of-range taps as `bounded` resolves them,
// :797-839).
//
// A workgroup of 256 threads produces a tile of ACC_ST_H x ACC_ST_W results (the code
// generator chooses the size).  It first
// stages the tile plus a halo of S::HY rows and S::HX columns in LDS, one array per scalar
// leaf of the source element; the staged value is the *result* of the (possibly fused)
// source at that position, with the boundary condition already applied, so a delayed
// producer runs once per staged element instead of once per tap and the stencil function
// itself never sees an index outside the tile.  Tiles that lie completely inside the array
// (with their halo) take a branch without any boundary code.  Lanes of a wave walk along
// x, so LDS reads are conflict-free and global accesses are contiguous runs of a row.
// Workgroups are numbered so that neighbouring tiles run on the same XCD: the halo columns
// of a tile are the border columns of its neighbours and are then found in that XCD's L2
// (measured: half the fetch traffic of the round-robin numbering).

#ifndef ACC_ST_W
#define ACC_ST_W 64
#endif
#ifndef ACC_ST_H
#define ACC_ST_H 16
#endif
#define ACC_ST_PW (ACC_ST_W + 2 * Spec::HX)
#define ACC_ST_PH (ACC_ST_H + 2 * Spec::HY)

struct Stencil2dParams {
  i64 h, w;     // extent of the result (= extent of the source)
  i64 tilesX;   // tiles per row of tiles
  i64 tilesY;   // rows of tiles
  i64 chain;    // tiles (consecutive in y) one workgroup works through, >= 1
};

// A workgroup walks down `chain` tiles of one column of tiles.  The loads of the next tile
// are issued before the current tile is computed from LDS, so that a workgroup has global
// loads in flight all the time instead of only at its start.  (Two tiles ahead was measured
// too: 106 us against 98 us per 8192 x 8192 sweep; the second set of staging registers
// costs a wave per SIMD and the waits still drain both sets together.)  INSIDE: every tile of the
// chain lies, with its halo, completely inside the array, and no boundary code is needed;
// the two cases are separate loops so that each has exactly one way of loading.
template <bool INSIDE>
ACC_DEV void acc_stencil2d_chain(const Spec::Env& env, const Spec::Out& out, const Stencil2dParams& p, Spec::Tile& tile,
                                 i64 x0, i64 ty, i64 tyEnd) {
  typedef Spec S;
  const int PW = ACC_ST_PW, PH = ACC_ST_PH;
  const int ITER = (ACC_ST_PW * ACC_ST_PH + ACC_BLOCK - 1) / ACC_BLOCK;
  // element idx of the padded tile ty, for every idx this thread stages
  auto fetch = [&](i64 t, S::SrcElt (&v)[ITER]) {
    const i64 y0 = t * ACC_ST_H;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int idx = it * ACC_BLOCK + threadIdx.x;
      const int ry = idx / PW, rx = idx - ry * PW;
      const i64 gy = y0 - S::HY + ry, gx = x0 - S::HX + rx;
      if (INSIDE) {
        if (idx < PW * PH) v[it] = S::src_in(env, gy, gx);
      } else {
        // positions further out than the halo of the last row / column are never read
        if (idx < PW * PH && gy < p.h + S::HY && gx < p.w + S::HX) v[it] = S::src_at(env, gy, gx);
      }
    }
  };
  const int lx = threadIdx.x & (ACC_ST_W - 1);
  const int lyBase = threadIdx.x / ACC_ST_W;
  S::SrcElt v[ITER];
  fetch(ty, v);
  for (; ty < tyEnd; ++ty) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int idx = it * ACC_BLOCK + threadIdx.x;
      if (idx < PW * PH) S::stage(tile, idx, v[it]);
    }
    __syncthreads();
    if (ty + 1 < tyEnd) fetch(ty + 1, v);
    const i64 y0 = ty * ACC_ST_H;
#pragma unroll
    for (int k = 0; k < ACC_ST_H / (ACC_BLOCK / ACC_ST_W); ++k) {
      const int ly = lyBase + k * (ACC_BLOCK / ACC_ST_W);
      const i64 gy = y0 + ly, gx = x0 + lx;
      if (INSIDE || (gy < p.h && gx < p.w))
        S::store(out, gy * p.w + gx, S::apply(env, tile, (ly + S::HY) * PW + lx + S::HX, gy, gx));
    }
    __syncthreads();
  }
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_stencil2d(Spec::Env env, Spec::Out out, Stencil2dParams p) {
  typedef Spec S;
  __shared__ S::Tile tile;
  const i64 b = acc_xcd_contiguous((i64)blockIdx.x, (i64)gridDim.x);
  const i64 cy = b / p.tilesX, tx = b - cy * p.tilesX;
  const i64 x0 = tx * ACC_ST_W;
  const i64 ty = cy * p.chain;
  const i64 tyEnd = ty + p.chain < p.tilesY ? ty + p.chain : p.tilesY;
  const bool inside = x0 >= S::HX && x0 + ACC_ST_W + S::HX <= p.w && ty * ACC_ST_H >= S::HY &&
                      tyEnd * ACC_ST_H + S::HY <= p.h;
  if (inside) acc_stencil2d_chain<true>(env, out, p, tile, x0, ty, tyEnd);
  else acc_stencil2d_chain<false>(env, out, p, tile, x0, ty, tyEnd);
}
