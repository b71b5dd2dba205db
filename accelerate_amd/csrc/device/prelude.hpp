// Device-side prelude shared by every generated kernel (gfx950, wave64).
// Compiled at run time by hipRTC together with the generated scalar code and one
// skeleton; nothing here is host code.

typedef signed char i8;
typedef short i16;
typedef int i32;
typedef long long i64;
typedef unsigned char u8;
typedef unsigned short u16;
typedef unsigned int u32;
typedef unsigned long long u64;
typedef _Float16 f16;
typedef float f32;
typedef double f64;

// SIMD vector element types Vec n t: n components side by side, aligned like one of them
template <class T, int N> struct acc_vec { T e[N]; };
#define ACC_VEC_TYPES(T)                                                                          \
  typedef acc_vec<T, 2> v2##T; typedef acc_vec<T, 3> v3##T; typedef acc_vec<T, 4> v4##T;           \
  typedef acc_vec<T, 8> v8##T; typedef acc_vec<T, 16> v16##T;
ACC_VEC_TYPES(i8) ACC_VEC_TYPES(i16) ACC_VEC_TYPES(i32) ACC_VEC_TYPES(i64)
ACC_VEC_TYPES(u8) ACC_VEC_TYPES(u16) ACC_VEC_TYPES(u32) ACC_VEC_TYPES(u64)
ACC_VEC_TYPES(f16) ACC_VEC_TYPES(f32) ACC_VEC_TYPES(f64)

// N values that lie side by side in memory, aligned like one of them: assigning through a
// pointer to it moves them with one request
template <class T, int N> struct __attribute__((packed, aligned(alignof(T)))) acc_run { T e[N]; };

#define ACC_DEV static __device__ __forceinline__
#define ACC_WAVE 64
#ifndef ACC_LOCK_SPIN_LIMIT
#define ACC_LOCK_SPIN_LIMIT (1u << 26)  // rounds in a row without any lane of the wave winning its lock, after which a locked permute gives up
#endif
#define ACC_BLOCK 256
#define ACC_WAVES (ACC_BLOCK / ACC_WAVE)

// Index arithmetic is 64-bit in the source language (Int); array extents almost always
// fit 32 bits, where the hardware divide is several times cheaper.
ACC_DEV i64 acc_quot(i64 a, i64 b) {
  if ((((u64)a | (u64)b) >> 32) == 0) return (i64)((u32)a / (u32)b);
  return a / b;
}
ACC_DEV i64 acc_rem(i64 a, i64 b) {
  if ((((u64)a | (u64)b) >> 32) == 0) return (i64)((u32)a % (u32)b);
  return a % b;
}

// Workgroups are handed to the 8 XCDs (each with its own L2) round-robin by workgroup
// number.  This renumbering gives every XCD one contiguous range of the nb work items, so
// that neighbouring items, which share cache lines at their borders, meet in the same L2.
ACC_DEV i64 acc_xcd_contiguous(i64 b, i64 nb) {
  const i64 q = nb >> 3, r = nb & 7;
  const i64 xcd = b & 7, k = b >> 3;
  return xcd * q + (xcd < r ? xcd : r) + k;
}

// Streaming accesses.  A launch that moves several times what the last-level cache holds
// gains from telling the caches that an operand is touched once (the `nt` hint): map over
// 2^28 Float32 348 -> 331 us, dotp 370 -> 340 us.  A launch whose operands fit the cache
// loses (the next kernel finds less of them there), so the host picks the variant by size.
// The generated functions that read at the skeleton's own linear index, and the plain
// stores, are templates over kStream; everywhere else the name refers to this constant.
static constexpr bool kStream = false;
template <bool NT, class T> ACC_DEV T acc_ld(const T* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT, class T> ACC_DEV void acc_st(T* p, const T& v) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

template <bool NT, class T, int N> ACC_DEV acc_vec<T, N> acc_ld(const acc_vec<T, N>* p) {
  acc_vec<T, N> r;
#pragma unroll
  for (int k = 0; k < N; ++k) r.e[k] = acc_ld<NT>(&p->e[k]);
  return r;
}
template <bool NT, class T, int N> ACC_DEV void acc_st(acc_vec<T, N>* p, const acc_vec<T, N>& v) {
#pragma unroll
  for (int k = 0; k < N; ++k) acc_st<NT>(&p->e[k], v.e[k]);
}

ACC_DEV int acc_lane() { return (int)(threadIdx.x & (ACC_WAVE - 1)); }
ACC_DEV int acc_wave() { return (int)(threadIdx.x / ACC_WAVE); }

// Word-wise cross-lane movement of any trivially copyable value.
template <class T> struct AccWords { enum { N = (sizeof(T) + 3) / 4 }; };

template <class T> ACC_DEV void acc_to_words(const T& v, u32* w) {
  for (int k = 0; k < AccWords<T>::N; ++k) w[k] = 0;
  __builtin_memcpy(w, &v, sizeof(T));
}
template <class T> ACC_DEV T acc_from_words(const u32* w) {
  T r;
  __builtin_memcpy(&r, w, sizeof(T));
  return r;
}

// c ? x : y, word by word.  (A choice between two objects of more than 8 bytes, however it is
// written, may be compiled as a choice between their addresses, and both then live in scratch
// memory: the rows kernels of folds and scans ran at 0.84 - 1.9 TB/s for such elements.)
template <class T> ACC_DEV T acc_pick(bool c, const T& x, const T& y) {
  u32 wx[AccWords<T>::N], wy[AccWords<T>::N];
  acc_to_words(x, wx);
  acc_to_words(y, wy);
#pragma unroll
  for (int k = 0; k < AccWords<T>::N; ++k) wx[k] = c ? wx[k] : wy[k];
  return acc_from_words<T>(wx);
}

template <class T> ACC_DEV T acc_shfl_up(const T& v, int delta) {
  u32 w[AccWords<T>::N];
  acc_to_words(v, w);
#pragma unroll
  for (int k = 0; k < AccWords<T>::N; ++k) w[k] = (u32)__shfl_up((int)w[k], delta, ACC_WAVE);
  return acc_from_words<T>(w);
}
template <class T> ACC_DEV T acc_shfl_down(const T& v, int delta) {
  u32 w[AccWords<T>::N];
  acc_to_words(v, w);
#pragma unroll
  for (int k = 0; k < AccWords<T>::N; ++k) w[k] = (u32)__shfl_down((int)w[k], delta, ACC_WAVE);
  return acc_from_words<T>(w);
}
template <class T> ACC_DEV T acc_shfl(const T& v, int src) {
  u32 w[AccWords<T>::N];
  acc_to_words(v, w);
#pragma unroll
  for (int k = 0; k < AccWords<T>::N; ++k) w[k] = (u32)__shfl((int)w[k], src, ACC_WAVE);
  return acc_from_words<T>(w);
}

// Data-parallel-primitive moves (VALU, no LDS traffic).  Controls of the gfx9 family:
// row_shr:n = 0x110 + n (shift right by n inside each row of 16 lanes), wave_shr:1 = 0x138
// (whole wave shifted by one lane), row_bcast:15 = 0x142 (lane 15 of each row to the next
// row), row_bcast:31 = 0x143 (lane 31 to rows 2 and 3).  Lanes without a source, or in
// rows the row mask disables, keep their own value.
template <int CTRL, int ROW_MASK, class T> ACC_DEV T acc_dpp(const T& v) {
  u32 w[AccWords<T>::N];
  acc_to_words(v, w);
#pragma unroll
  for (int k = 0; k < AccWords<T>::N; ++k)
    w[k] = (u32)__builtin_amdgcn_update_dpp((int)w[k], (int)w[k], CTRL, ROW_MASK, 0xf, false);
  return acc_from_words<T>(w);
}

// value held by lane `src` (wave-uniform) of the wave
template <class T> ACC_DEV T acc_readlane(const T& v, int src) {
  u32 w[AccWords<T>::N];
  acc_to_words(v, w);
  const int s = __builtin_amdgcn_readfirstlane(src);
#pragma unroll
  for (int k = 0; k < AccWords<T>::N; ++k) w[k] = (u32)__builtin_amdgcn_readlane((int)w[k], s);
  return acc_from_words<T>(w);
}

// Ordered reduction of the values held by lanes [0, nvalid) of a wave: the result, valid in
// lane 0, is v0 (+) v1 (+) .. with operands kept left to right, so the operator need
// only be associative.  Inside each row of 16 lanes the partner's value comes through
// row_shl (a lane receives from the lane n places above it); the four row results are read
// with readlane and combined in order.
template <class S> ACC_DEV typename S::Elt acc_wave_reduce(const typename S::Env& env, typename S::Elt v, int lane, int nvalid) {
  typedef typename S::Elt Elt;
  const int col = lane & 15;
  {
    Elt o = acc_dpp<0x101, 0xf>(v);
    if (col + 1 < 16 && lane + 1 < nvalid) v = S::combine(env, v, o);
  }
  {
    Elt o = acc_dpp<0x102, 0xf>(v);
    if (col + 2 < 16 && lane + 2 < nvalid) v = S::combine(env, v, o);
  }
  {
    Elt o = acc_dpp<0x104, 0xf>(v);
    if (col + 4 < 16 && lane + 4 < nvalid) v = S::combine(env, v, o);
  }
  {
    Elt o = acc_dpp<0x108, 0xf>(v);
    if (col + 8 < 16 && lane + 8 < nvalid) v = S::combine(env, v, o);
  }
  Elt r = acc_readlane(v, 0);
  if (nvalid > 16) r = S::combine(env, r, acc_readlane(v, 16));
  if (nvalid > 32) r = S::combine(env, r, acc_readlane(v, 32));
  if (nvalid > 48) r = S::combine(env, r, acc_readlane(v, 48));
  return r;
}


// Ordered inclusive scan across the lanes of a wave (valid lanes must form a prefix):
// four shifts inside the rows of 16 lanes, then the row totals are handed to the next row
// and the half totals to the upper half.  Operands stay in lane order, so the operator need
// only be associative.
template <class S> ACC_DEV typename S::Elt acc_wave_scan(const typename S::Env& env, typename S::Elt v, int lane) {
  typedef typename S::Elt Elt;
  const int rl = lane & 15;
#define ACC_SCAN_STEP(CTRL, ROWS, COND)             \
  {                                                 \
    Elt o_ = acc_dpp<CTRL, ROWS>(v);                \
    Elt r_ = S::combine(env, o_, v);                \
    if (COND) v = r_;                               \
  }
  ACC_SCAN_STEP(0x111, 0xf, rl >= 1)
  ACC_SCAN_STEP(0x112, 0xf, rl >= 2)
  ACC_SCAN_STEP(0x114, 0xf, rl >= 4)
  ACC_SCAN_STEP(0x118, 0xf, rl >= 8)
  ACC_SCAN_STEP(0x142, 0xa, (lane & 16) != 0)
  ACC_SCAN_STEP(0x143, 0xc, lane >= 32)
#undef ACC_SCAN_STEP
  return v;
}

// value of the previous lane (lane 0 keeps its own)
template <class T> ACC_DEV T acc_prev_lane(const T& v) { return acc_dpp<0x138, 0xf>(v); }
