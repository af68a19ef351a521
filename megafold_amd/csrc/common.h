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

// ---- LDS tile of DP-wide rows ----------------------------------------------------------------------
// 16-bit element types: rows are stored unpadded (DP*2 bytes) with their 16-byte chunks XOR-swizzled
// by the row number, which keeps both fragment reads (one row per lane, same chunk) and transposing
// reads free of bank conflicts and — unlike padding — is compatible with direct global->LDS loads,
// whose destination is "lane i writes 16 bytes at base + 16*i".  fp32 keeps padded rows and is staged
// through registers.
template <typename T, int DP> struct Tile {
  static constexpr bool kAsync = sizeof(T) == 2;
  static constexpr int CPR = DP * (int)sizeof(T) / 16;          // 16-byte chunks per row
  static constexpr int EPC = 16 / (int)sizeof(T);               // elements per chunk
  static constexpr int RP = CPR >= 8 ? 1 : 8 / CPR;             // rows per 128 bytes
  static constexpr int STRIDE = kAsync ? DP : DP + 4;           // elements between rows
  static __device__ __forceinline__ int swz(int row) { return kAsync ? (row / RP) % (CPR < 8 ? CPR : 8) : 0; }
  // element offset of (row, col); col must not cross a chunk together with the access width
  static __device__ __forceinline__ int off(int row, int col) {
    if (kAsync) return row * DP + ((((col / EPC) ^ swz(row))) * EPC) + (col % EPC);
    return row * STRIDE + col;
  }
  // the 8 values X[k0 + 8*g + e][own_col], e = 0..7 (see TrRead for the lane protocol)
  static __device__ __forceinline__ frag_t<T> tr_read(const T* tile, int k0, int g, int l, int chunk_col, int own_col) {
    if constexpr (kAsync) {
      const int a = (l >> 2) & 3;
      const int r0 = k0 + 8 * g + a, r1 = r0 + 4;
      const T* p0 = tile + off(r0, chunk_col);
      const T* p1 = tile + off(r1, chunk_col);
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p0));
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p1));
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      s16x8 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[e + 4] = hi[e]; }
      return __builtin_bit_cast(frag_t<T>, v);
    } else {
      frag_t<T> v;
      const T* p = tile + (k0 + 8 * g) * STRIDE + own_col;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = p[e * STRIDE];
      return v;
    }
  }
};

// Direct global->LDS copy of 16 bytes per lane: lane i's data lands at lds_base + 16*i (lds_base must
// be wave-uniform).  Completion is tracked by vmcnt like any vector memory load.
__device__ __forceinline__ void async_copy16(const void* gsrc, void* lds_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                   (__attribute__((address_space(3))) void*)lds_base, 16, 0, 0);
}
// Work-group barrier without the memory fence __syncthreads() implies (which would drain every
// outstanding direct-to-LDS load): wait for this wavefront's LDS traffic and all but the newest
// `VM` vector-memory operations, then synchronise.
template <int VM> __device__ __forceinline__ void barrier_keep_vm() {
  static_assert(VM >= 0 && VM < 64, "vmcnt range");
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(((VM & 15) | ((VM >> 4) << 14)) | (7 << 4) | (0 << 8));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// ---- carrier fragments: scalars riding through one extra MFMA contraction step -------------------
// 16-bit types: a 32-bit word holds two slots (value split as hi + lo, or the pair (1, 1)); a carrier
// fragment is {w0, w1, 0, 0} = slots (w0.lo, w0.hi, w1.lo, w1.hi, 0, 0, 0, 0).  fp32: a word is one
// slot, the fragment is {w0, w1, 0, ...}.  Pairing A = {ones, -x} with B = {y, ones} adds y - x to
// every element of the tile exactly (to ~2^-17 relative for the split 16-bit values).
template <typename T> __device__ __forceinline__ frag_t<T> make_aug(unsigned w0, unsigned w1) {
  u32x4 v = {w0, w1, 0u, 0u};
  return __builtin_bit_cast(frag_t<T>, v);
}
template <> __device__ __forceinline__ f32x8 make_aug<float>(unsigned w0, unsigned w1) {
  f32x8 f = {__builtin_bit_cast(float, w0), __builtin_bit_cast(float, w1), 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  return f;
}
template <typename T> __device__ __forceinline__ unsigned pack_split(float m) {
  T hi, lo;
  split_hi_lo<T>(m, hi, lo);
  typedef T pair_t __attribute__((ext_vector_type(2)));
  pair_t pr = {hi, lo};
  return __builtin_bit_cast(unsigned, pr);
}
template <> __device__ __forceinline__ unsigned pack_split<float>(float m) { return __builtin_bit_cast(unsigned, m); }
template <typename T> __device__ __forceinline__ unsigned ones_word() {
  typedef T pair_t __attribute__((ext_vector_type(2)));
  pair_t pr = {(T)1.0f, (T)1.0f};
  return __builtin_bit_cast(unsigned, pr);
}
template <> __device__ __forceinline__ unsigned ones_word<float>() { return __builtin_bit_cast(unsigned, 1.0f); }

}  // namespace mf

// Sum over aligned groups of W consecutive lanes (W = 2, 4, 8, 16 or 32); every lane of a group gets
// the group's total.  Up to 16 lanes this is pure DPP (quad permutes, then the half-row and row
// mirrors, which pair up lanes that already hold equal partial sums): no LDS traffic, unlike
// __shfl_xor, which goes through ds_bpermute and costs an LDS round trip per step.
template <int W> __device__ __forceinline__ float group_sum(float v) {
  static_assert(W == 1 || W == 2 || W == 4 || W == 8 || W == 16 || W == 32, "group width");
  auto dpp_add = [](float a, int ctrl) {
    const int moved = ctrl == 0xB1   ? __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), 0xB1, 0xF, 0xF, true)
                      : ctrl == 0x4E ? __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), 0x4E, 0xF, 0xF, true)
                      : ctrl == 0x141 ? __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), 0x141, 0xF, 0xF, true)
                                      : __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), 0x140, 0xF, 0xF, true);
    return a + __builtin_bit_cast(float, moved);
  };
  if (W >= 2) v = dpp_add(v, 0xB1);     // quad_perm [1,0,3,2]
  if (W >= 4) v = dpp_add(v, 0x4E);     // quad_perm [2,3,0,1]
  if (W >= 8) v = dpp_add(v, 0x141);    // row_half_mirror
  if (W >= 16) v = dpp_add(v, 0x140);   // row_mirror
  if (W >= 32) v += __shfl_xor(v, 16);
  return v;
}

// Force a value to be computed where this statement stands.  The optimiser otherwise sinks arithmetic
// on loaded registers towards its first use, which can carry it past the issue of the NEXT batch of
// loads: the in-order vector-memory counter then makes the old value wait for the new loads.
template <typename V> __device__ __forceinline__ void pin(V& v) { asm volatile("" : "+v"(v)); }

// ---- development aid: per-phase cycle stamps ------------------------------------------------------
// Compiled in only with -DMF_TIMELINE.  MF_TL(p, slot) makes lane 0 of every wavefront of the chosen
// work-group store the shader clock at p.tl[slot]; the caller supplies the buffer address through the
// environment variable MF_TL_PTR (hex) and the work-group through MF_TL_BLOCK.
#ifdef MF_TIMELINE
#define MF_TL(p, slot)                                                                              \
  do {                                                                                              \
    if ((p).tl && (int)blockIdx.x == (p).tl_block && (threadIdx.x & 63) == 0)                       \
      (p).tl[(slot)] = (unsigned)__builtin_readcyclecounter();                                      \
  } while (0)
#else
#define MF_TL(p, slot) do { } while (0)
#endif
