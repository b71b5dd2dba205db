// Rank-2 stencil skeleton with LDS halo tiles (stencilOp, Interpreter.hs:637-649; taps as
// stencilAccess builds them, :670-794; out-of-range taps as `bounded` resolves them,
// :797-839).
//
// A workgroup of 256 threads produces a tile of ACC_ST_H x ACC_ST_W results (32 x 64 by
// default: measured best of 8/16/32/64 rows on the 8192 x 8192 Jacobi sweep).  It first
// stages the tile plus a halo of S::HY rows and S::HX columns in LDS, one array per scalar
// leaf of the source element; the staged value is the *result* of the (possibly fused)
// source at that position, with the boundary condition already applied, so a delayed
// producer runs once per staged element instead of once per tap and the stencil function
// itself never sees an index outside the tile.  Tiles that lie completely inside the array
// (with their halo) take a branch without any boundary code.  Lanes of a wave walk along
// x, so LDS reads are conflict-free and global accesses are contiguous runs of a row.

#define ACC_ST_W 64
#ifndef ACC_ST_H
#define ACC_ST_H 16
#endif
#define ACC_ST_PW (ACC_ST_W + 2 * Spec::HX)
#define ACC_ST_PH (ACC_ST_H + 2 * Spec::HY)

struct Stencil2dParams {
  i64 h, w;     // extent of the result (= extent of the source)
  i64 tilesX;   // tiles per row of tiles
};

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_stencil2d(Spec::Env env, Spec::Out out, Stencil2dParams p) {
  typedef Spec S;
  __shared__ S::Tile tile;
  const i64 b = (i64)blockIdx.x;
  const i64 ty = b / p.tilesX, tx = b - ty * p.tilesX;
  const i64 y0 = ty * ACC_ST_H, x0 = tx * ACC_ST_W;
  const bool interior = y0 >= S::HY && x0 >= S::HX && y0 + ACC_ST_H + S::HY <= p.h && x0 + ACC_ST_W + S::HX <= p.w;
  const int PW = ACC_ST_PW, PH = ACC_ST_PH;
  const int ITER = (ACC_ST_PW * ACC_ST_PH + ACC_BLOCK - 1) / ACC_BLOCK;
  if (interior) {
    // fixed trip count, fully unrolled: all loads of a thread are in flight together
    S::SrcElt v[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int idx = it * ACC_BLOCK + threadIdx.x;
      const int ry = idx / PW, rx = idx - ry * PW;
      if (idx < PW * PH) v[it] = S::src_in(env, y0 - S::HY + ry, x0 - S::HX + rx);
    }
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int idx = it * ACC_BLOCK + threadIdx.x;
      if (idx < PW * PH) S::stage(tile, idx, v[it]);
    }
  } else {
    for (int idx = threadIdx.x; idx < PW * PH; idx += ACC_BLOCK) {
      const int ry = idx / PW, rx = idx - ry * PW;
      const i64 gy = y0 - S::HY + ry, gx = x0 - S::HX + rx;
      // positions further out than the halo of the last row / column are never read
      if (gy < p.h + S::HY && gx < p.w + S::HX) S::stage(tile, idx, S::src_at(env, gy, gx));
    }
  }
  __syncthreads();
  const int lx = threadIdx.x & (ACC_ST_W - 1);
  const int lyBase = threadIdx.x / ACC_ST_W;
#pragma unroll
  for (int k = 0; k < ACC_ST_H / (ACC_BLOCK / ACC_ST_W); ++k) {
    const int ly = lyBase + k * (ACC_BLOCK / ACC_ST_W);
    const i64 gy = y0 + ly, gx = x0 + lx;
    if (interior || (gy < p.h && gx < p.w))
      S::store(out, gy * p.w + gx, S::apply(env, tile, (ly + S::HY) * PW + lx + S::HX, gy, gx));
  }
}
