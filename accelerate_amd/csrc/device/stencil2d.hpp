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
// x, four columns each, so LDS reads are conflict-free and global accesses are contiguous
// runs of a row.
// Workgroups are numbered so that neighbouring tiles run on the same XCD: the halo columns
// of a tile are the border columns of its neighbours and are then found in that XCD's L2
// (measured: half the fetch traffic of the round-robin numbering).

#ifndef ACC_ST_W
#define ACC_ST_W 128
#endif
#ifndef ACC_ST_H
#define ACC_ST_H 8
#endif
// A staged row: HXP columns of left halo (the halo proper, right-aligned in a pad of a
// multiple of 4 columns), ACC_ST_W columns of results, HXP columns of right halo.  The pad
// keeps every group of 4 result columns 16-byte aligned in LDS.
#define ACC_ST_PW (ACC_ST_W + 2 * Spec::HXP)
#define ACC_ST_PH (ACC_ST_H + 2 * Spec::HY)
#define ACC_ST_GROUPS (ACC_ST_W / 4)   // groups of 4 result columns per row

struct Stencil2dParams {
  i64 h, w;     // extent of the result (= extent of the source)
  i64 tilesX;   // tiles per row of tiles
  i64 tilesY;   // rows of tiles
  i64 chain;    // tiles (consecutive in y) one workgroup works through, >= 1
};

// A workgroup walks down `chain` tiles of one column of tiles (normally one), issuing the
// loads of the next tile before the current tile is computed from LDS.  A thread stages and
// produces groups of 4 consecutive columns, so that plain-array sources, LDS and the result
// are all moved 128 bits at a time; the halo columns are staged one by one.  INSIDE: every
// tile of the chain lies, with its halo, completely inside the array, and no boundary code
// is needed; the two cases are separate loops so that each has exactly one way of loading.
// Measured on the 8192 x 8192 Jacobi sweep: staging and producing one column per thread and
// access took 123 us with one tile per workgroup and 98 us with chains of 4; 128-bit
// accesses take 92 us with one tile per workgroup, and chains (103 / 107 us for 2 / 4, 106 us
// with two tiles ahead) no longer pay.
template <bool INSIDE>
ACC_DEV void acc_stencil2d_chain(const Spec::Env& env, const Spec::Out& out, const Stencil2dParams& p, Spec::Tile& tile,
                                 i64 x0, i64 ty, i64 tyEnd) {
  typedef Spec S;
  const int PW = ACC_ST_PW, PH = ACC_ST_PH, NG = ACC_ST_GROUPS;
  const int NI = PH * NG;                                   // groups of 4 interior columns to stage
  const int NH = PH * 2 * S::HX;                            // halo elements to stage
  const int ITER_I = (NI + ACC_BLOCK - 1) / ACC_BLOCK;
  const int ITER_H = (NH + ACC_BLOCK - 1) / ACC_BLOCK;
  struct Staged {
    S::SrcElt in[ITER_I][4];
    S::SrcElt halo[ITER_H > 0 ? ITER_H : 1];
  };
  // source element at (gy, gx) of the array, for a position of the padded tile
  auto at = [&](i64 gy, i64 gx, S::SrcElt& v) {
    if (INSIDE) v = S::src_in(env, gy, gx);
    // positions further out than the halo of the last row / column are never read
    else if (gy < p.h + S::HY && gx < p.w + S::HX) v = S::src_at(env, gy, gx);
  };
  auto fetch = [&](i64 t, Staged& v) {
    const i64 y0 = t * ACC_ST_H;
#pragma unroll
    for (int it = 0; it < ITER_I; ++it) {
      const int id = it * ACC_BLOCK + threadIdx.x;
      const int ry = id / NG, g = id - ry * NG;
      if (id < NI) {
#pragma unroll
        for (int k = 0; k < 4; ++k) at(y0 - S::HY + ry, x0 + 4 * g + k, v.in[it][k]);
      }
    }
#pragma unroll
    for (int it = 0; it < ITER_H; ++it) {
      const int id = it * ACC_BLOCK + threadIdx.x;
      const int ry = id / (2 * S::HX), c = id - ry * (2 * S::HX);
      if (id < NH) at(y0 - S::HY + ry, c < S::HX ? x0 - S::HX + c : x0 + ACC_ST_W + (c - S::HX), v.halo[it]);
    }
  };
  auto stage = [&](const Staged& v) {
#pragma unroll
    for (int it = 0; it < ITER_I; ++it) {
      const int id = it * ACC_BLOCK + threadIdx.x;
      const int ry = id / NG, g = id - ry * NG;
      if (id < NI) {
#pragma unroll
        for (int k = 0; k < 4; ++k) S::stage(tile, ry * PW + S::HXP + 4 * g + k, v.in[it][k]);
      }
    }
#pragma unroll
    for (int it = 0; it < ITER_H; ++it) {
      const int id = it * ACC_BLOCK + threadIdx.x;
      const int ry = id / (2 * S::HX), c = id - ry * (2 * S::HX);
      if (id < NH) S::stage(tile, ry * PW + (c < S::HX ? S::HXP - S::HX + c : S::HXP + ACC_ST_W + (c - S::HX)), v.halo[it]);
    }
  };
  Staged v;
  fetch(ty, v);
  for (; ty < tyEnd; ++ty) {
    stage(v);
    __syncthreads();
    if (ty + 1 < tyEnd) fetch(ty + 1, v);
    const i64 y0 = ty * ACC_ST_H;
#pragma unroll
    for (int q = 0; q < (ACC_ST_H * NG + ACC_BLOCK - 1) / ACC_BLOCK; ++q) {
      const int id = q * ACC_BLOCK + threadIdx.x;
      const int ly = id / NG, g = id - ly * NG;
      const i64 gy = y0 + ly, gx = x0 + 4 * g;
      const int c = (ly + S::HY) * PW + S::HXP + 4 * g;
      if (id < ACC_ST_H * NG) {
        if (INSIDE || (gy < p.h && gx + 4 <= p.w)) {
          S::Elt r[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) r[k] = S::apply(env, tile, c + k, gy, gx + k);
#pragma unroll
          for (int k = 0; k < 4; ++k) S::store(out, gy * p.w + gx + k, r[k]);
        } else if (gy < p.h) {
          for (int k = 0; k < 4 && gx + k < p.w; ++k) S::store(out, gy * p.w + gx + k, S::apply(env, tile, c + k, gy, gx + k));
        }
      }
    }
    __syncthreads();
  }
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_stencil2d(Spec::Env env, Spec::Out out, Stencil2dParams p) {
  typedef Spec S;
  __shared__ __attribute__((aligned(16))) S::Tile tile;
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
