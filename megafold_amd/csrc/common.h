// Shared device helpers for the gfx950 kernels: fragment types for the 32x32 MFMA family,
// vector loads/stores, and LDS fragment reads (plain and transposing).
//
// Conventions used by every kernel in this directory
// --------------------------------------------------
// A wavefront has 64 lanes; lane l is written (x, g) with x = l & 31 and g = l >> 5.
// One "mma step" contracts 16 slots.  Slot (g, e), e = 0..7, is element e of the
// 8-element fragment held by a lane whose half is g.  For an A operand lane (x, g) holds
// row x of the 32-row tile, for a B operand it holds column x.  The accumulator tile is
// 32x32 fp32: lane (x, g) register r holds row  8*(r>>2) + 4*g + (r&3)  of column x.
// The same slot convention is used for bf16/fp16 (one v_mfma_f32_32x32x16) and for fp32
// (eight v_mfma_f32_32x32x2, MFMA t taking element t of every fragment).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mf {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

#define MF_LOG2E 1.4426950408889634f
#define MF_LN2 0.6931471805599453f

// Element-type codes shared with the C ABI (include/megafold_amd.h).
enum { MF_F32 = 0, MF_F16 = 1, MF_BF16 = 2, MF_BOOL = 3 };

template <typename T> struct Frag;
template <> struct Frag<bf16_t> { typedef bf16x8 type; typedef bf16x4 half; };
template <> struct Frag<f16_t> { typedef f16x8 type; typedef f16x4 half; };
template <> struct Frag<float> { typedef f32x8 type; typedef f32x4 half; };
template <typename T> using frag_t = typename Frag<T>::type;

template <typename T> __device__ __forceinline__ frag_t<T> frag_zero() {
  frag_t<T> f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (T)0.0f;
  return f;
}

__device__ __forceinline__ f32x16 acc_zero() {
  f32x16 c;
#pragma unroll
  for (int r = 0; r < 16; ++r) c[r] = 0.0f;
  return c;
}

// ---- matrix multiply-accumulate on one 32x32 tile over 16 contraction slots -------------
__device__ __forceinline__ f32x16 mma(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mma(f16x8 a, f16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mma(f32x8 a, f32x8 b, f32x16 c) {
#pragma unroll
  for (int t = 0; t < 8; ++t) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], c, 0, 0, 0);
  return c;
}

// ---- 8-element (fragment sized) global / LDS access --------------------------------------
// 16-bit types move as one 16-byte vector, fp32 as two.  Addresses must be 16-byte aligned.
template <typename T> __device__ __forceinline__ frag_t<T> ld8(const T* p);
template <> __device__ __forceinline__ bf16x8 ld8<bf16_t>(const bf16_t* p) {
  u32x4 v = *reinterpret_cast<const u32x4*>(p);
  return __builtin_bit_cast(bf16x8, v);
}
template <> __device__ __forceinline__ f16x8 ld8<f16_t>(const f16_t* p) {
  u32x4 v = *reinterpret_cast<const u32x4*>(p);
  return __builtin_bit_cast(f16x8, v);
}
template <> __device__ __forceinline__ f32x8 ld8<float>(const float* p) {
  f32x4 a = *reinterpret_cast<const f32x4*>(p);
  f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
  f32x8 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) { r[e] = a[e]; r[e + 4] = b[e]; }
  return r;
}
template <typename T> __device__ __forceinline__ void st8(T* p, frag_t<T> v);
template <> __device__ __forceinline__ void st8<bf16_t>(bf16_t* p, bf16x8 v) {
  *reinterpret_cast<u32x4*>(p) = __builtin_bit_cast(u32x4, v);
}
template <> __device__ __forceinline__ void st8<f16_t>(f16_t* p, f16x8 v) {
  *reinterpret_cast<u32x4*>(p) = __builtin_bit_cast(u32x4, v);
}
template <> __device__ __forceinline__ void st8<float>(float* p, f32x8 v) {
  f32x4 a, b;
#pragma unroll
  for (int e = 0; e < 4; ++e) { a[e] = v[e]; b[e] = v[e + 4]; }
  *reinterpret_cast<f32x4*>(p) = a;
  *reinterpret_cast<f32x4*>(p + 4) = b;
}

// fp32 values -> fragment of T (round to nearest even for the 16-bit types).
template <typename T> __device__ __forceinline__ frag_t<T> cvt8(float v0, float v1, float v2, float v3, float v4,
                                                               float v5, float v6, float v7) {
  frag_t<T> f;
  f[0] = (T)v0; f[1] = (T)v1; f[2] = (T)v2; f[3] = (T)v3;
  f[4] = (T)v4; f[5] = (T)v5; f[6] = (T)v6; f[7] = (T)v7;
  return f;
}
// Registers 8u..8u+7 of an accumulator tile as a fragment (the accumulator-to-operand move
// that needs no data movement: register index is the contraction slot).
template <typename T> __device__ __forceinline__ frag_t<T> acc_half(const f32x16& c, int u) {
  return u == 0 ? cvt8<T>(c[0], c[1], c[2], c[3], c[4], c[5], c[6], c[7])
                : cvt8<T>(c[8], c[9], c[10], c[11], c[12], c[13], c[14], c[15]);
}
template <typename T> __device__ __forceinline__ frag_t<T> scale8(frag_t<T> f, float s) {
  frag_t<T> o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (T)((float)f[e] * s);
  return o;
}

// ---- transposing fragment read from a row-major LDS tile ---------------------------------
// The tile is X[k][n] with n contiguous and `stride` elements between rows.  The calling lane
// (x, g) receives the 8 values X[k0 + 8*g + e][own_col], e = 0..7.
// For 16-bit types this is two ds_read_b64_tr_b16.  That instruction works on groups of 16
// lanes: inside a group lane i = 4*a + c supplies the address of 4 consecutive elements of row a
// and receives, as element e, element (i & 3) of what lane 4*e + (i >> 2) addressed.  So when
// lane 4*a + c addresses row a at the 4-aligned column run chunk_col(c), lane i receives column
// chunk_col(i >> 2) + (i & 3) of rows 0..3.  The caller passes `chunk_col` evaluated for its own
// c = l & 3 (and its own 16-lane group) and `own_col`, the column it ends up holding; the two
// must describe the same map.  fp32 has no transposing read and uses eight scalar reads of
// `own_col`.
template <typename T> struct TrRead {
  static __device__ __forceinline__ frag_t<T> read(const T* tile, int stride, int k0, int g, int l, int chunk_col,
                                                   int own_col) {
    const int a = (l >> 2) & 3;
    const T* p0 = tile + (k0 + 8 * g + a) * stride + chunk_col;
    const T* p1 = p0 + 4 * stride;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p0));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p1));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    s16x8 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[e + 4] = hi[e]; }
    return __builtin_bit_cast(frag_t<T>, v);
  }
};
template <> struct TrRead<float> {
  static __device__ __forceinline__ f32x8 read(const float* tile, int stride, int k0, int g, int l, int chunk_col,
                                               int own_col) {
    f32x8 v;
    const float* p = tile + (k0 + 8 * g) * stride + own_col;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = p[e * stride];
    return v;
  }
};

// Column (inside a DP-wide tile) whose values a lane must hold when the tile's columns are the
// rows of an A operand and the accumulator must come out with DP/2 contiguous columns per lane:
// accumulator register r of d-tile dt in lane half g  <->  column (DP/2)*g + 16*dt + r.
template <int DP> __device__ __forceinline__ int dsel(int dt, int x) {
  return (DP / 2) * ((x >> 2) & 1) + 16 * dt + 4 * (x >> 3) + (x & 3);
}
// Same map expressed for the transposing read: 4-aligned column run that pointing-lane l must
// address so that lane (x, .) receives column dsel<DP>(dt, x).
template <int DP> __device__ __forceinline__ int dsel_chunk(int dt, int l) {
  const int c = l & 3, q1 = (l >> 4) & 1;
  return (DP / 2) * (c & 1) + 16 * dt + 8 * q1 + 4 * (c >> 1);
}
// Plain column map (lane x receives column n0 + x): run addressed by pointing-lane l.
__device__ __forceinline__ int plain_chunk(int l) { return 16 * ((l >> 4) & 1) + 4 * (l & 3); }

// Row permutation that makes accumulator registers contiguous: storing tile row kk (0..31) at
// A-operand row perm32(kk) makes register r of lane half g hold row 16*g + r.
__device__ __forceinline__ int perm32(int kk) { return 2 * (kk & 12) + ((kk >> 4) << 2) + (kk & 3); }
// Inverse: A-operand row m holds tile row unperm32(m).
__device__ __forceinline__ int unperm32(int m) { return 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Load one element of a mask / bias tensor whose dtype is only known at run time.
__device__ __forceinline__ float load_any(const void* p, int dtype, int64_t idx) {
  switch (dtype) {
    case MF_F32: return reinterpret_cast<const float*>(p)[idx];
    case MF_F16: return (float)reinterpret_cast<const f16_t*>(p)[idx];
    case MF_BF16: return (float)reinterpret_cast<const bf16_t*>(p)[idx];
    default: return reinterpret_cast<const uint8_t*>(p)[idx] ? 0.0f : -__builtin_inff();
  }
}

// Split an additive mask value into (hi, lo) with hi + lo == v to ~2^-17 relative in T, so that
// it can ride through a 16-bit MFMA operand.  Infinite values keep lo = 0.
template <typename T> __device__ __forceinline__ void split_hi_lo(float v, T& hi, T& lo) {
  hi = (T)v;
  float h = (float)hi;
  float r = v - h;
  lo = (h - h == 0.0f) ? (T)r : (T)0.0f;  // h - h is NaN when h is +-inf
}
template <> __device__ __forceinline__ void split_hi_lo<float>(float v, float& hi, float& lo) {
  hi = v;
  lo = 0.0f;
}

}  // namespace mf
