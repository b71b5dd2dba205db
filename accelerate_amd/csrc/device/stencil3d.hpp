// Rank-3 stencil skeleton (stencilOp, Interpreter.hs:637-649; taps as stencilAccess builds
// them, :670-794; out-of-range taps as `bounded` resolves them, :797-839).
//
// A direct evaluation reads every tap from global memory: the planes z-1, z, z+1 of a large
// array do not stay in an XCD's L2 between their uses, and every element comes from HBM
// several times.  Here a workgroup of 256 threads owns a column of ACC_ST_H x ACC_ST_W
// results in (y, x) and marches along z: LDS holds a ring of 2*HZ+1 planes of the column,
// each with its halo in y and x, so every step stages one new plane (boundary condition
// applied while staging, delayed sources evaluated once per staged element) and produces
// one plane of results from LDS.  The loads of the next plane are issued before the current
// one is computed.  Columns are numbered so that neighbours run on the same XCD.  (Staging
// and producing groups of 4 columns with 128-bit accesses, which pays for rank 2, was
// measured here too: 270-330 us against 210-230 us for the 7-point stencil on 512^3.)

#ifndef ACC_ST_W
#define ACC_ST_W 128
#endif
#ifndef ACC_ST_H
#define ACC_ST_H 8
#endif
#define ACC_ST_PW (ACC_ST_W + 2 * Spec::HX)
#define ACC_ST_PH (ACC_ST_H + 2 * Spec::HY)
#define ACC_ST_PLANE (ACC_ST_PW * ACC_ST_PH)
#define ACC_ST_NP (2 * Spec::HZ + 1)

struct Stencil3dParams {
  i64 d, h, w;          // extent of the result (= extent of the source), outermost first
  i64 tilesX, tilesY;   // columns per row / rows of columns
  i64 chain;            // planes a workgroup produces, >= 1
};

template <bool INSIDE>
ACC_DEV void acc_stencil3d_chain(const Spec::Env& env, const Spec::Out& out, const Stencil3dParams& p,
                                 Spec::Tile& tile, i64 x0, i64 y0, i64 z0, i64 zEnd) {
  typedef Spec S;
  const int PW = ACC_ST_PW, PLANE = ACC_ST_PLANE, NP = ACC_ST_NP;
  const int ITER = (ACC_ST_PLANE + ACC_BLOCK - 1) / ACC_BLOCK;
  // element idx of the padded plane z of this column, for every idx this thread stages
  auto fetch = [&](i64 z, S::SrcElt (&v)[ITER]) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int idx = it * ACC_BLOCK + threadIdx.x;
      const int ry = idx / PW, rx = idx - ry * PW;
      const i64 gy = y0 - S::HY + ry, gx = x0 - S::HX + rx;
      if (INSIDE) {
        if (idx < PLANE) v[it] = S::src_in(env, z, gy, gx);
      } else {
        // positions further out than the halo of the last row / column are never read
        if (idx < PLANE && gy < p.h + S::HY && gx < p.w + S::HX) v[it] = S::src_at(env, z, gy, gx);
      }
    }
  };
  auto stage = [&](int slot, const S::SrcElt (&v)[ITER]) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int idx = it * ACC_BLOCK + threadIdx.x;
      if (idx < PLANE) S::stage(tile, slot * PLANE + idx, v[it]);
    }
  };
  const int lx = threadIdx.x & (ACC_ST_W - 1);
  const int lyBase = threadIdx.x / ACC_ST_W;
  S::SrcElt v[ITER];
  // the planes below the first result
  for (int q = 0; q < 2 * S::HZ; ++q) {
    fetch(z0 - S::HZ + q, v);
    stage(q, v);
  }
  int slot = NP - 1;  // ring slot that receives plane z + HZ
  fetch(z0 + S::HZ, v);
  for (i64 z = z0; z < zEnd; ++z) {
    stage(slot, v);
    __syncthreads();
    if (z + 1 < zEnd) fetch(z + 1 + S::HZ, v);
    int pl[ACC_ST_NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) pl[q] = ((slot + 1 + q) % NP) * PLANE;  // plane z - HZ + q
#pragma unroll
    for (int k = 0; k < ACC_ST_H / (ACC_BLOCK / ACC_ST_W); ++k) {
      const int ly = lyBase + k * (ACC_BLOCK / ACC_ST_W);
      const i64 gy = y0 + ly, gx = x0 + lx;
      if (INSIDE || (gy < p.h && gx < p.w))
        S::store(out, (z * p.h + gy) * p.w + gx, S::apply(env, tile, pl, (ly + S::HY) * PW + lx + S::HX));
    }
    __syncthreads();
    slot = slot + 1 == NP ? 0 : slot + 1;
  }
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
acc_stencil3d(Spec::Env env, Spec::Out out, Stencil3dParams p) {
  typedef Spec S;
  __shared__ S::Tile tile;
  const i64 b = acc_xcd_contiguous((i64)blockIdx.x, (i64)gridDim.x);
  const i64 perSlab = p.tilesX * p.tilesY;
  const i64 cz = b / perSlab, rest = b - cz * perSlab;
  const i64 ty = rest / p.tilesX, tx = rest - ty * p.tilesX;
  const i64 x0 = tx * ACC_ST_W, y0 = ty * ACC_ST_H;
  const i64 z0 = cz * p.chain;
  const i64 zEnd = z0 + p.chain < p.d ? z0 + p.chain : p.d;
  const bool inside = x0 >= S::HX && x0 + ACC_ST_W + S::HX <= p.w && y0 >= S::HY && y0 + ACC_ST_H + S::HY <= p.h &&
                      z0 >= S::HZ && zEnd + S::HZ <= p.d;
  if (inside) acc_stencil3d_chain<true>(env, out, p, tile, x0, y0, z0, zEnd);
  else acc_stencil3d_chain<false>(env, out, p, tile, x0, y0, z0, zEnd);
}
