// MSA pair-weighted averaging (Algorithm 10 of AlphaFold 3), the contraction part of the reference's
// MSAPairWeightedAveraging.forward (megafold/model/megafold.py:868-902):
//
//     w[b,h,i,:]     = softmax_j(logits[b,i,j,h] + mask[b,j])                      megafold.py:884-890
//     y[b,s,i,h,:]   = (sum_j w[b,h,i,j] x[b,s,j,h,:]) * sigmoid(g[b,s,i,h,:])     megafold.py:892-893
//
// The weights do not depend on the MSA row s: the softmax is taken ONCE per (b, h, i) and stored (16-bit,
// zero padded to whole 32 x 32 tiles); the averaging is then a product of the [n, n] weight matrix of a head
// with the [n, s * d] matrix of that head's values, organised so that a wavefront keeps its 32 weight rows in
// registers for all the MSA rows it walks over, the value rows of an MSA row travel as whole 128-byte lines
// (two heads) straight into LDS, and the gate is applied to the accumulators before they are stored.
// Backward (the gate's own backward aside):
//     dx[b,s,j,h,:]  = sum_i w[b,h,i,j] dy[b,s,i,h,:]          the same kernel on the transposed weights
//     dw[b,h,i,j]    = sum_{s,d} dy[b,s,i,h,d] x[b,s,j,h,d]     pwa_dw_kernel: patches of dw stay in registers
//                                                               while the MSA rows stream by (row chunks write
//                                                               partial buffers)
//     dlogits        = w * (dw - sum_j w dw)                    pwa_softmax_bwd_kernel, which also sums the partials
// Shapes: 16-bit element types, 8 heads of 32 channels (a row of logits and a head's channels are 16 / 64
// bytes), n <= 384 for the averaging kernel (the weight rows of a wavefront must fit its registers).
#include "../../include/megafold_amd.h"
#include "capi_common.h"
#include "common.h"

namespace mf {
namespace {

struct PwaParams {
  int B, S, N, H, NP, n_chunks, rows_per_chunk;
  const void* logits; int64_t ld_logits;
  const unsigned char* mask;
  void* w;
  const void* x; int64_t ldx;
  const void* g; int64_t ldg;
  void* y; int64_t ldy;
  const void* dy; int64_t lddy;
  float* dw_part;
  void* dlogits; int64_t ld_dlogits;
};

__device__ __forceinline__ void dma16(unsigned voff, const void* sbase, unsigned lds) {
  asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "{m0}"(lds) : "memory");
}
template <int VM> __device__ __forceinline__ void wait_vm() {
  static_assert(VM >= 0 && VM < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt(((VM & 15) | ((VM >> 4) << 14)) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
template <typename T> __device__ __forceinline__ void unpack8(u32x4 c, float (&f)[8]) {
  const frag_t<T> v = __builtin_bit_cast(frag_t<T>, c);
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (float)v[e];
}

// ---- softmax of the logits, once per (b, h, i): one work-group per row i, one wavefront per head ----------------
template <typename T>
__global__ void __launch_bounds__(512) pwa_softmax_fwd_kernel(const PwaParams p) {
  const int l = threadIdx.x & 63, h = threadIdx.x >> 6;
  const int64_t row = blockIdx.x;
  const int b = (int)(row / p.NP), i = (int)(row % p.NP);
  const int N = p.N, NP = p.NP;
  T* wrow = reinterpret_cast<T*>(p.w) + (((int64_t)b * 8 + h) * NP + i) * NP;
  if (i >= N) {                                                             // padding rows: zeros
    for (int j = l; j < NP; j += 64) wrow[j] = (T)0.0f;
    return;
  }
  const T* lrow = reinterpret_cast<const T*>(p.logits) + ((int64_t)b * N + i) * N * p.ld_logits + h;
  const unsigned char* mk = p.mask ? p.mask + (int64_t)b * N : nullptr;
  auto load = [&](int j) {
    const float f = (float)lrow[(int64_t)j * p.ld_logits];
    return (mk && !mk[j]) ? -__builtin_inff() : f;
  };
  float m = -__builtin_inff(), sum = 0.0f;
  for (int j = l; j < N; j += 64) m = fmaxf(m, load(j));
  m = wave_max(m);
  for (int j = l; j < N; j += 64) {
    const float f = load(j);
    sum += f == -__builtin_inff() ? 0.0f : __expf(f - m);
  }
  sum = wave_sum(sum);
  sum = sum > 0.0f ? 1.0f / sum : 0.0f;      // every key masked: zero weights
  for (int j = l; j < NP; j += 64) {
    const float f = j < N ? load(j) : -__builtin_inff();
    wrow[j] = (T)(f != -__builtin_inff() ? __expf(f - m) * sum : 0.0f);
  }
}

// ---- dlogits = w * (dw - sum_j w dw), dw = sum of the partial buffers: one work-group per row i, one wavefront per
// head; the eight heads' results meet in LDS and leave as whole 16-byte rows of the logits' layout
template <typename T>
__global__ void __launch_bounds__(512) pwa_softmax_bwd_kernel(const PwaParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);                   // [N][8]
  const int l = threadIdx.x & 63, h = threadIdx.x >> 6;
  const int64_t row = blockIdx.x;
  const int b = (int)(row / p.N), i = (int)(row % p.N);
  const int N = p.N, NP = p.NP;
  const int64_t part = (int64_t)p.B * 8 * NP * NP;
  const int64_t off = (((int64_t)b * 8 + h) * NP + i) * NP;
  const T* wrow = reinterpret_cast<const T*>(p.w) + off;
  const float* drow = p.dw_part + off;
  auto dw_of = [&](int j) {
    float s = 0.0f;
    for (int c = 0; c < p.n_chunks; ++c) s += drow[c * part + j];    // fixed order
    return s;
  };
  // the row's dw values stay in registers when the row is short enough, else they are summed again
  float dwv[8];
  float r = 0.0f;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int j = l + 64 * t;
    dwv[t] = j < N ? dw_of(j) : 0.0f;
    if (j < N) r += (float)wrow[j] * dwv[t];
  }
  for (int j = l + 512; j < N; j += 64) r += (float)wrow[j] * dw_of(j);
  r = wave_sum(r);
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int j = l + 64 * t;
    if (j < N) tile[j * 8 + h] = (T)((float)wrow[j] * (dwv[t] - r));
  }
  for (int j = l + 512; j < N; j += 64) tile[j * 8 + h] = (T)((float)wrow[j] * (dw_of(j) - r));
  __syncthreads();
  T* out = reinterpret_cast<T*>(p.dlogits) + ((int64_t)b * N + i) * N * p.ld_dlogits;
  for (int j = threadIdx.x; j < N; j += 512)
    *reinterpret_cast<u32x4*>(out + (int64_t)j * p.ld_dlogits) = *reinterpret_cast<const u32x4*>(tile + j * 8);
}

// ---- y[s, i, h, :] = (sum_j w[h, i, j] x[s, j, h, :]) (* sigmoid(g[s, i, h, :])) --------------------------------
// Work-group: eight wavefronts = (head of a pair) x (four tiles of 32 rows i); it walks over a chunk of the MSA
// rows.  NK = 16-key steps of the contraction (2 per 32 x 32 tile of w).
constexpr int APPLY_NBUF = 3;
template <typename T, int NK>
__global__ void __launch_bounds__(512, 1) pwa_apply_kernel(const PwaParams p, const int IB, const int SC) {
  using frag = frag_t<T>;
  constexpr int ROWS = NK * 16;                     // LDS rows of a value tile (>= NP)
  constexpr int RND = (ROWS * 8 + 511) / 512;       // direct loads per thread and MSA row
  constexpr int SLOT = RND * 8192;
  extern __shared__ __align__(16) unsigned char smem[];
  const int t512 = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(t512 >> 6);
  const int l = t512 & 63, x = l & 31, g = l >> 5;
  const int hs = wv >> 2, w = wv & 3;
  int bid = blockIdx.x;
  const int sc = bid % SC; bid /= SC;
  const int ib = bid % IB; bid /= IB;
  const int pair = bid % 4;
  const int b = bid / 4;
  const int h = 2 * pair + hs;
  const int N = p.N, NP = p.NP;
  const int s0 = sc * p.rows_per_chunk, s1 = min(p.S, s0 + p.rows_per_chunk);
  if (s0 >= s1) return;

  // this wavefront's 32 rows of w: B operands (column = row i, contraction slots = keys), resident
  const int i = ib * 128 + 32 * w + x;
  const int ic = i < NP ? i : NP - 1;
  frag wf[NK];
  {
    const T* wrow = reinterpret_cast<const T*>(p.w) + (((int64_t)b * 8 + h) * NP + ic) * NP + 8 * g;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) wf[ks] = 16 * ks < NP ? ld8<T>(wrow + 16 * ks) : frag_zero<T>();
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) pin(wf[ks]);
  }

  // direct loads of a value tile: LDS row m = key m (clamped), 16-byte chunk c of the pair line at c ^ (m & 7)
  unsigned voff[RND];
#pragma unroll
  for (int rd = 0; rd < RND; ++rd) {
    const int q = rd * 512 + t512, m = q >> 3, pos = q & 7;
    const int j = m < N ? m : N - 1;
    voff[rd] = (unsigned)((int64_t)j * p.ldx * 2 + pair * 128 + ((pos ^ (m & 7)) << 4));
  }
  const unsigned lds0 = (unsigned)(unsigned long)((__attribute__((address_space(3))) unsigned char*)smem);
  const char* xb = reinterpret_cast<const char*>(p.x) + ((int64_t)b * p.S + s0) * N * p.ldx * 2;
  const int64_t x_step = (int64_t)N * p.ldx * 2;
  auto issue = [&](int buf) {
#pragma unroll
    for (int rd = 0; rd < RND; ++rd) dma16(voff[rd], xb, lds0 + buf * SLOT + rd * 8192 + wv * 1024);
    xb += x_step;
  };
  // transposing reads: the 8 values x[16 ks + 8 g + e][d], d = the column this lane's accumulator rows need
  const int a = (l >> 2) & 3;
  const int col = dsel_chunk<32>(0, l);
  const int r0 = 8 * g + a, r1 = r0 + 4;
  const int ta0 = r0 * 128 + (((hs * 4 + (col >> 3)) ^ (r0 & 7)) << 4) + (col & 7) * 2;
  const int ta1 = r1 * 128 + (((hs * 4 + (col >> 3)) ^ (r1 & 7)) << 4) + (col & 7) * 2;

  const int S_rows = s1 - s0;
  issue(0);
  if (S_rows > 1) issue(1);
  const bool gate = p.g != nullptr;
  const int64_t orow0 = ((int64_t)b * p.S + s0) * N + (i < N ? i : N - 1);
  for (int r = 0; r < S_rows; ++r) {
    const int buf = r % APPLY_NBUF;
    // row r has arrived (the newest RND requests, row r + 1, may still travel)
    if (r + 1 < S_rows) wait_vm<RND>(); else wait_vm<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F);           // lgkmcnt(0): this wavefront's LDS reads of the slot reused next
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    u32x4 g0 = {0u, 0u, 0u, 0u}, g1 = {0u, 0u, 0u, 0u};
    if (gate) {
      const T* gp = reinterpret_cast<const T*>(p.g) + (orow0 + (int64_t)r * N) * p.ldg + h * 32 + 16 * g;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(g0) : "v"(gp) : "memory");
      asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(g1) : "v"(gp) : "memory");
    }
    if (r + 2 < S_rows) issue((r + 2) % APPLY_NBUF);
    const unsigned char* tile = smem + buf * SLOT;
    f32x16 acc = acc_zero();
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + ta0 + ks * 2048));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + ta1 + ks * 2048));
      s16x8 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[e + 4] = hi[e]; }
      acc = mma(__builtin_bit_cast(frag, v), wf[ks], acc);      // rows = channels d, columns = rows i
    }
    // lane (x = row i, g) holds the 16 contiguous channels 16 g .. 16 g + 15 of head h
    if (gate) {
      if (r + 2 < S_rows) wait_vm<RND>(); else wait_vm<0>();   // the gate values (requested before the newest row)
      pin(g0); pin(g1);
      float gv[8];
      unpack8<T>(g0, gv);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] *= 1.0f / (1.0f + __expf(-gv[e]));
      unpack8<T>(g1, gv);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[8 + e] *= 1.0f / (1.0f + __expf(-gv[e]));
    }
    if (i < N) {
      T* yp = reinterpret_cast<T*>(p.y) + (orow0 + (int64_t)r * N) * p.ldy + h * 32 + 16 * g;
      st8<T>(yp, acc_half<T>(acc, 0));
      st8<T>(yp + 8, acc_half<T>(acc, 1));
    }
  }
}

// ---- dw[h, i, j] = sum over (s, d) of dy[s, i, h, d] x[s, j, h, d] --------------------------------------------------
// Work-group: eight wavefronts = (head of a pair) x (four tiles of 32 rows i), patch 128 i x 192 j per head (six
// key tiles per wavefront: the larger the patch, the fewer bytes travel per product), over a chunk of the MSA
// rows; the rows of dy and x travel as whole pair lines into a ring of three LDS slots.
constexpr int DW_TJ = 6;                                // key tiles per patch
constexpr int DW_XR = (DW_TJ * 32 * 8) / 512;           // direct loads per thread for the x rows
constexpr int DW_OPS = 2 + DW_XR;
constexpr int DW_SLOT = 16384 + DW_TJ * 4096;           // dy: 128 rows of 128 bytes, x: 192 rows
template <typename T>
__global__ void __launch_bounds__(512, 1) pwa_dw_kernel(const PwaParams p, const int IB, const int JB) {
  using frag = frag_t<T>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int t512 = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(t512 >> 6);
  const int l = t512 & 63, x = l & 31, g = l >> 5;
  const int hs = wv >> 2, w = wv & 3;
  int bid = blockIdx.x;
  const int chunk = bid % p.n_chunks; bid /= p.n_chunks;
  const int ib = bid % IB; bid /= IB;
  const int jb = bid % JB; bid /= JB;
  const int pair = bid % 4;
  const int b = bid / 4;
  const int h = 2 * pair + hs;
  const int N = p.N, NP = p.NP;
  const int s0 = chunk * p.rows_per_chunk, s1 = min(p.S, s0 + p.rows_per_chunk);
  const int R = s1 - s0;

  // direct loads: chunk c of LDS row m at position c ^ ((m >> 1) & 7) (conflict-free 16-byte fragment reads)
  const int m = t512 >> 3, pos = t512 & 7, cg = pos ^ ((m >> 1) & 7);
  unsigned yoff[2], xoff[DW_XR];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    int ii = ib * 128 + 64 * q + m;
    ii = ii < N ? ii : N - 1;
    yoff[q] = (unsigned)((int64_t)ii * p.lddy * 2 + pair * 128 + cg * 16);
  }
#pragma unroll
  for (int q = 0; q < DW_XR; ++q) {
    const int mm = 64 * q + m;                                               // operand row of the patch
    int jj = jb * (DW_TJ * 32) + (mm & ~31) + unperm32(mm & 31);             // row m of a key tile holds key unperm32(m)
    jj = jj < N ? jj : N - 1;
    xoff[q] = (unsigned)((int64_t)jj * p.ldx * 2 + pair * 128 + cg * 16);
  }
  const unsigned lds0 = (unsigned)(unsigned long)((__attribute__((address_space(3))) unsigned char*)smem);
  const char* yb = reinterpret_cast<const char*>(p.dy) + ((int64_t)b * p.S + s0) * N * p.lddy * 2;
  const char* xb = reinterpret_cast<const char*>(p.x) + ((int64_t)b * p.S + s0) * N * p.ldx * 2;
  const int64_t y_step = (int64_t)N * p.lddy * 2, x_step = (int64_t)N * p.ldx * 2;
  auto issue = [&](int buf) {
    const unsigned sb = lds0 + buf * DW_SLOT + wv * 1024;
    dma16(yoff[0], yb, sb);
    dma16(yoff[1], yb, sb + 8192);
#pragma unroll
    for (int q = 0; q < DW_XR; ++q) dma16(xoff[q], xb, sb + 16384 + q * 8192);
    yb += y_step; xb += x_step;
  };
  int ya[2], xa[2];
  const int qrow = 32 * w + x;
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const int c = hs * 4 + 2 * g + ks;
    ya[ks] = qrow * 128 + ((c ^ ((qrow >> 1) & 7)) << 4);
    xa[ks] = 16384 + x * 128 + ((c ^ ((x >> 1) & 7)) << 4);
  }
  f32x16 acc[DW_TJ];
#pragma unroll
  for (int t = 0; t < DW_TJ; ++t) acc[t] = acc_zero();
  if (R > 0) {
    issue(0);
    if (R > 1) issue(1);
    for (int r = 0; r < R; ++r) {
      if (r + 1 < R) wait_vm<DW_OPS>(); else wait_vm<0>();
      __builtin_amdgcn_s_waitcnt(0xC07F);
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (r + 2 < R) issue((r + 2) % 3);
      const unsigned char* sb = smem + (r % 3) * DW_SLOT;
      frag yf[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) yf[ks] = ld8<T>(reinterpret_cast<const T*>(sb + ya[ks]));
#pragma unroll
      for (int t = 0; t < DW_TJ; ++t)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
          acc[t] = mma(ld8<T>(reinterpret_cast<const T*>(sb + xa[ks] + t * 4096)), yf[ks], acc[t]);
    }
  }
  // lane (x = row i, g) owns keys 16 g .. 16 g + 15 of each key tile
  const int i = ib * 128 + qrow;
  if (i < NP) {
    float* dst = p.dw_part + (((int64_t)chunk * p.B + b) * 8 + h) * NP * NP + (int64_t)i * NP;
#pragma unroll
    for (int t = 0; t < DW_TJ; ++t) {
      const int j = jb * (DW_TJ * 32) + 32 * t + 16 * g;
      if (j < NP) {
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          f32x4 v = {acc[t][4 * c4], acc[t][4 * c4 + 1], acc[t][4 * c4 + 2], acc[t][4 * c4 + 3]};
          *reinterpret_cast<f32x4*>(dst + j + 4 * c4) = v;
        }
      }
    }
  }
}

int num_cu() {
  int dev = 0, n = 0;
  return (hipGetDevice(&dev) == hipSuccess &&
          hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
}

int check_pwa(const mf_pwa_args* a, bool need_x) {
  clear_error();
  if (!a) return fail(MF_ERR_NULL, "args is NULL");
  if (a->B <= 0 || a->S <= 0 || a->N <= 0) return fail(MF_ERR_SHAPE, "B, S, N must be positive (got %d %d %d)", a->B, a->S, a->N);
  if (a->H != 8 || a->D != 32) return fail(MF_ERR_SHAPE, "H=%d, D=%d unsupported: 8 heads of 32 channels", a->H, a->D);
  if (a->dtype != MF_DTYPE_F16 && a->dtype != MF_DTYPE_BF16) return fail(MF_ERR_DTYPE, "dtype %d unsupported: f16 / bf16", a->dtype);
  if (!a->w || !aligned16(a->w)) return fail(MF_ERR_NULL, "w is NULL or not 16-byte aligned");
  if (need_x) {
    if (!a->x || !aligned16(a->x)) return fail(MF_ERR_NULL, "x is NULL or not 16-byte aligned");
    if (a->ldx < 256 || a->ldx % 8 != 0) return fail(MF_ERR_STRIDE, "ldx=%lld: need a multiple of 8, at least 256", (long long)a->ldx);
    if ((int64_t)a->N * a->ldx * 2 + 256 >= (1LL << 31)) return fail(MF_ERR_SHAPE, "N * ldx too large");
  }
  return 0;
}

PwaParams params_of(const mf_pwa_args* a) {
  PwaParams p{};
  p.B = a->B; p.S = a->S; p.N = a->N; p.H = a->H; p.NP = (a->N + 31) / 32 * 32;
  p.n_chunks = a->n_chunks; p.rows_per_chunk = a->S;
  p.logits = a->logits; p.ld_logits = a->ld_logits;
  p.mask = static_cast<const unsigned char*>(a->mask);
  p.w = a->w;
  p.x = a->x; p.ldx = a->ldx;
  p.g = a->g; p.ldg = a->ldg;
  p.y = a->y; p.ldy = a->ldy;
  p.dy = a->dy; p.lddy = a->lddy;
  p.dw_part = a->dw_part;
  p.dlogits = a->dlogits; p.ld_dlogits = a->ld_dlogits;
  return p;
}

template <typename T, int NK> hipError_t launch_apply(PwaParams p, hipStream_t stream) {
  const int IB = (p.N + 127) / 128;
  // MSA-row chunks: enough work-groups for the device, at least two rows each where there are that many
  const long long groups = (long long)p.B * 4 * IB;
  int SC = (int)(num_cu() / groups);          // one work-group per compute unit: never more than one round
  if (SC > p.S) SC = p.S;
  if (SC < 1) SC = 1;
  p.rows_per_chunk = (p.S + SC - 1) / SC;
  SC = (p.S + p.rows_per_chunk - 1) / p.rows_per_chunk;
  constexpr int RND = (NK * 16 * 8 + 511) / 512;
  const size_t smem = (size_t)APPLY_NBUF * RND * 8192;
  auto kern = pwa_apply_kernel<T, NK>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3((unsigned)(groups * SC)), dim3(512), smem, stream, p, IB, SC);
  return hipGetLastError();
}
template <typename T> hipError_t launch_apply_n(const PwaParams& p, hipStream_t stream) {
  const int nk = p.NP / 16;
  if (nk <= 8) return launch_apply<T, 8>(p, stream);
  if (nk <= 16) return launch_apply<T, 16>(p, stream);
  return launch_apply<T, 24>(p, stream);
}

int dw_chunks(const mf_pwa_args* a) {
  const int IB = (a->N + 127) / 128, JB = (a->N + DW_TJ * 32 - 1) / (DW_TJ * 32);
  const long long patches = (long long)a->B * 4 * IB * JB;
  long long c = num_cu() / patches;              // one work-group per compute unit, one round
  if (c > 16) c = 16;
  if (c > a->S) c = a->S;
  if (c < 1) c = 1;
  const int rows = (int)((a->S + c - 1) / c);
  return (a->S + rows - 1) / rows;
}

}  // namespace
}  // namespace mf

using namespace mf;

extern "C" int mf_pwa_softmax_fwd(const mf_pwa_args* a) {
  int rc = check_pwa(a, false);
  if (rc) return rc;
  if (!a->logits || !aligned16(a->logits)) return fail(MF_ERR_NULL, "logits is NULL or not 16-byte aligned");
  if (a->ld_logits < 8 || a->ld_logits % 8 != 0) return fail(MF_ERR_STRIDE, "ld_logits=%lld: need a multiple of 8", (long long)a->ld_logits);
  const PwaParams p = params_of(a);
  const int64_t rows = (int64_t)p.B * p.NP;
  if (rows > 0x7fffffffLL) return fail(MF_ERR_SHAPE, "B * N too large");
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  if (a->dtype == MF_DTYPE_BF16)
    hipLaunchKernelGGL(pwa_softmax_fwd_kernel<bf16_t>, dim3((unsigned)rows), dim3(512), 0, stream, p);
  else
    hipLaunchKernelGGL(pwa_softmax_fwd_kernel<f16_t>, dim3((unsigned)rows), dim3(512), 0, stream, p);
  return (int)hipGetLastError();
}

extern "C" int mf_pwa_apply(const mf_pwa_args* a) {
  int rc = check_pwa(a, true);
  if (rc) return rc;
  if (a->N > 384) return fail(MF_ERR_SHAPE, "N=%d unsupported: at most 384", a->N);
  if (!a->y || !aligned16(a->y)) return fail(MF_ERR_NULL, "y is NULL or not 16-byte aligned");
  if (a->ldy < 256 || a->ldy % 8 != 0) return fail(MF_ERR_STRIDE, "ldy=%lld: need a multiple of 8, at least 256", (long long)a->ldy);
  if (a->g && (!aligned16(a->g) || a->ldg < 256 || a->ldg % 8 != 0)) return fail(MF_ERR_STRIDE, "g: need 16-byte alignment and ldg a multiple of 8, at least 256");
  const PwaParams p = params_of(a);
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  return (int)(a->dtype == MF_DTYPE_BF16 ? launch_apply_n<bf16_t>(p, stream) : launch_apply_n<f16_t>(p, stream));
}

extern "C" int mf_pwa_dw_chunks(const mf_pwa_args* a) {
  if (!a || a->B <= 0 || a->S <= 0 || a->N <= 0) return 0;
  return dw_chunks(a);
}

extern "C" int mf_pwa_dw(const mf_pwa_args* a) {
  int rc = check_pwa(a, true);
  if (rc) return rc;
  if (!a->dy || !aligned16(a->dy)) return fail(MF_ERR_NULL, "dy is NULL or not 16-byte aligned");
  if (a->lddy < 256 || a->lddy % 8 != 0) return fail(MF_ERR_STRIDE, "lddy=%lld: need a multiple of 8, at least 256", (long long)a->lddy);
  if ((int64_t)a->N * a->lddy * 2 + 256 >= (1LL << 31)) return fail(MF_ERR_SHAPE, "N * lddy too large");
  if (!a->dw_part || !aligned16(a->dw_part)) return fail(MF_ERR_NULL, "dw_part is NULL or not 16-byte aligned");
  if (a->n_chunks != dw_chunks(a)) return fail(MF_ERR_WORKSPACE, "n_chunks=%d: mf_pwa_dw_chunks says %d", a->n_chunks, dw_chunks(a));
  PwaParams p = params_of(a);
  p.rows_per_chunk = (p.S + p.n_chunks - 1) / p.n_chunks;
  const int IB = (p.N + 127) / 128, JB = (p.N + DW_TJ * 32 - 1) / (DW_TJ * 32);
  const long long blocks = (long long)p.B * 4 * IB * JB * p.n_chunks;
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  const size_t smem = 3 * DW_SLOT;
  auto launch = [&](auto kern) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(512), smem, stream, p, IB, JB);
    return hipGetLastError();
  };
  return (int)(a->dtype == MF_DTYPE_BF16 ? launch(pwa_dw_kernel<bf16_t>) : launch(pwa_dw_kernel<f16_t>));
}

extern "C" int mf_pwa_softmax_bwd(const mf_pwa_args* a) {
  int rc = check_pwa(a, false);
  if (rc) return rc;
  if (!a->dw_part || a->n_chunks < 1 || a->n_chunks > 16) return fail(MF_ERR_NULL, "dw_part is NULL or n_chunks=%d out of range", a->n_chunks);
  if (!a->dlogits || !aligned16(a->dlogits)) return fail(MF_ERR_NULL, "dlogits is NULL or not 16-byte aligned");
  if (a->ld_dlogits < 8 || a->ld_dlogits % 8 != 0) return fail(MF_ERR_STRIDE, "ld_dlogits=%lld: need a multiple of 8", (long long)a->ld_dlogits);
  const PwaParams p = params_of(a);
  const int64_t rows = (int64_t)p.B * p.N;
  if (rows > 0x7fffffffLL || p.N > 4096) return fail(MF_ERR_SHAPE, "B * N too large, or N > 4096");
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  const size_t smem = (size_t)p.N * 16;      // at most 64 KiB: within the default limit of dynamic LDS
  if (a->dtype == MF_DTYPE_BF16)
    hipLaunchKernelGGL(pwa_softmax_bwd_kernel<bf16_t>, dim3((unsigned)rows), dim3(512), smem, stream, p);
  else
    hipLaunchKernelGGL(pwa_softmax_bwd_kernel<f16_t>, dim3((unsigned)rows), dim3(512), smem, stream, p);
  return (int)hipGetLastError();
}
