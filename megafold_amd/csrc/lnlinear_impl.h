// LayerNorm -> Linear (and LayerNorm -> SwiGLU) for gfx950.
//
//   mu, r = mean(x), 1/sqrt(var(x) + eps)      x_hat = (x - mu) r      y = x_hat * gamma + beta
//   out = y W + b                                (reference: fused_layernorm_linear.py:109-218)
//
// Forward.  With W' = gamma (.) W (rows scaled),  cs[n] = sum_k W'[k, n]  and
// b'[n] = sum_k beta[k] W[k, n] + b[n]:
//       out[m, n] = r[m] * (x[m, :] W'[:, n]) - r[m] mu[m] cs[n] + b'[n]
// so the MFMA runs on the RAW 16-bit x (no rounding of the normalised activations, no vector-ALU
// work per input element) and LayerNorm becomes two fused multiply-adds per OUTPUT element.  The row
// statistics are computed while the x tile is staged into LDS (two-pass variance, fp32) — the
// "prologue" of the GEMM — and saved as fp32 for the backward.  Each wavefront keeps its slice of
// W'^T in registers for the whole kernel and walks over row blocks (persistent work-groups), so the
// only streams are x in and out out.  The SwiGLU variant gives a wavefront matching value/gate
// column tiles and writes only h = silu(gate) * value.
//
// Backward (fused_layernorm_linear.py:226-348, closed forms at 281-306, 345), two kernels, no atomics:
//   dx:  w = gamma (.) (dOut W^T) (contraction over N on the MFMA with the weights as stored, W chunks through
//        LDS, dOut straight from global; gamma multiplies the fp32 products, as in the reference, so the
//        rounding of W' never enters the gradient), then c1 = mean(x_hat w), c2 = mean(w),
//        dx = (w - x_hat c1 - c2) r in registers: a lane owns one row, so the two means are register sums
//        plus one lane exchange.
//   dW:  G = x_hat^T dOut and s = colsum(dOut) per row range (contraction over the rows: both
//        operands are staged row-major and reach the MFMA through transposing LDS reads), then a small
//        kernel sums the ranges in a fixed order and forms
//        dW = gamma G + beta s,  dgamma = rowsum(W (.) G),  dbeta = W s,  db = s.
#pragma once
#include <cstdlib>
#include "common.h"
#include "lnlinear.h"

namespace mf {

template <typename T> __device__ __forceinline__ float to_f(T v) { return (float)v; }

// =================================================================================================
// forward
// =================================================================================================
template <typename T, int KP> struct LnLayout {
  static constexpr int UNIT = 16 / (int)sizeof(T);
  static constexpr int XSTR = ((KP / UNIT) % 2 == 0) ? KP + UNIT : KP;
};

__device__ __forceinline__ float sigmoidf_fast(float g) {
  return __builtin_amdgcn_rcpf(1.0f + fast_exp2(-g * MF_LOG2E));
}

// Column of W handled by A-operand row m of tile t (see the layout note in common.h): the
// accumulator of lane half g then holds TILES*16 contiguous columns.
template <int NTW, int ACT> __device__ __forceinline__ int ln_col(int t, int gm, int rr, int base, int Nhalf) {
  if (ACT == LN_ACT_NONE) return base + (NTW * 16) * gm + 16 * t + rr;
  constexpr int TH = NTW / 2;
  const int th = t % TH, half = t / TH;
  return half * Nhalf + base + (TH * 16) * gm + 16 * th + rr;
}

template <int NTW, int ACT> __device__ __forceinline__ bool ln_col_ok(int t, int gm, int rr, int base, int N, int Nhalf) {
  if (ACT == LN_ACT_NONE) return base + (NTW * 16) * gm + 16 * t + rr < N;
  constexpr int TH = NTW / 2;
  return base + (TH * 16) * gm + 16 * (t % TH) + rr < Nhalf;
}

// Rows of more than 256 bytes double the resident weight fragments and the staged rows: those variants get the whole register file
// (one work-group per compute unit) instead of spilling at two.
template <typename T, int KP, int NTW, int ACT, int WN>
__global__ void __launch_bounds__(256, KP * sizeof(T) > 256 ? 1 : 2) ln_fwd_kernel(const LnParams p) {
  using L = LnLayout<T, KP>;
  using frag = frag_t<T>;
  constexpr int KS = KP / 16, CPR = KP / 8;
  constexpr int TH = NTW / 2;
  constexpr int OUTW = (ACT == LN_ACT_NONE) ? NTW * 32 : TH * 32;   // output columns per wavefront
  constexpr int WR = 4 / WN, RB = 32 * WR;

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Xs = reinterpret_cast<T*>(smem_raw);                          // [2][RB][XSTR]
  float* meanL = reinterpret_cast<float*>(Xs + 2 * RB * L::XSTR);  // [2][RB]
  float* rstdL = meanL + 2 * RB;                                   // [2][RB]
  float* csL = rstdL + 2 * RB;                                     // [4 * NTW * 32]
  float* bpL = csL + 4 * NTW * 32;
  // per-wavefront output tile(s), row-major: results leave the registers with one row per lane and
  // are stored from here with consecutive lanes on consecutive 16-byte chunks (whole cache lines)
  constexpr int OSTR = OUTW + 16 / (int)sizeof(T);
  constexpr int OTILES = (ACT == LN_ACT_SWIGLU_BWD) ? 2 : 1;
  T* Os = reinterpret_cast<T*>(bpL + 4 * NTW * 32) + (threadIdx.x >> 6) * (OTILES * 32 * OSTR);

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int wn = w % WN, wr = w / WN;
  const int Nhalf = p.N / 2;
  const int NOUT = (ACT == LN_ACT_NONE) ? p.N : Nhalf;             // width of the output / dout
  const int base = (blockIdx.y * WN + wn) * OUTW;                  // first output column of this wavefront
  const T* Wt = reinterpret_cast<const T*>(p.Wt);
  const T* X = reinterpret_cast<const T*>(p.x);

  // ---- this wavefront's slice of W'^T, resident in registers -----------------------------------
  // Fetched by the whole work-group with consecutive lanes on consecutive 16-byte chunks of a row
  // (whole cache lines; a lane-per-row gather of the same bytes takes four times as many L1 requests)
  // and handed to the owning lanes through LDS, one tile of 32 rows per wavefront at a time.
  frag af[NTW][KS];
  {
    T* Wst = reinterpret_cast<T*>(bpL + 4 * NTW * 32);     // [4 * 32][XSTR], aliases the output tiles
    constexpr int WITEMS = 128 * CPR, WPF = WITEMS / 256;   // 16-byte chunks per staged tile / per thread
    // all tiles are requested up front where the registers allow it (K <= 128), else tile by tile
    constexpr bool kBatch = KP <= 128;
    frag wtmp[kBatch ? NTW : 1][WPF];
    auto request = [&](int t, frag* dst) {
#pragma unroll
      for (int i = 0; i < WPF; ++i) {
        const int item = tid + 256 * i;
        const int r = item / CPR, dc = item % CPR;          // staged row: wavefront r / 32, lane row r % 32
        const int xx = r & 31, wq = r >> 5;
        const int gm = (xx >> 2) & 1, rr = 4 * (xx >> 3) + (xx & 3);
        const int b2 = (blockIdx.y * WN + wq % WN) * OUTW;
        const int col = ln_col<NTW, ACT>(t, gm, rr, b2, Nhalf);
        const bool ok = ln_col_ok<NTW, ACT>(t, gm, rr, b2, p.N, Nhalf);
        dst[i] = ld8<T>(Wt + (int64_t)(ok ? col : 0) * KP + 8 * dc);
      }
    };
    if constexpr (kBatch) {
#pragma unroll
      for (int t = 0; t < NTW; ++t) request(t, wtmp[t]);
    }
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      if constexpr (!kBatch) request(t, wtmp[0]);
      const frag* src = wtmp[kBatch ? t : 0];
#pragma unroll
      for (int i = 0; i < WPF; ++i) {
        const int item = tid + 256 * i;
        const int r = item / CPR, dc = item % CPR;
        const int xx = r & 31, wq = r >> 5;
        const int gm = (xx >> 2) & 1, rr = 4 * (xx >> 3) + (xx & 3);
        const int b2 = (blockIdx.y * WN + wq % WN) * OUTW;
        const bool ok = ln_col_ok<NTW, ACT>(t, gm, rr, b2, p.N, Nhalf);
        st8<T>(Wst + r * L::XSTR + 8 * dc, ok ? src[i] : frag_zero<T>());
      }
      __syncthreads();
#pragma unroll
      for (int s = 0; s < KS; ++s) af[t][s] = ld8<T>(Wst + (w * 32 + x) * L::XSTR + (KP / 2) * g + 8 * s);
      __syncthreads();
    }
  }
  // column constants of the work-group's columns: index ((wn * NTW + t) * 2 + g) * 16 + rr
  for (int i = tid; i < WN * NTW * 32; i += 256) {
    const int rr = i & 15, gg = (i >> 4) & 1, t = (i >> 5) % NTW, wn2 = (i >> 5) / NTW;
    const int b2 = (blockIdx.y * WN + wn2) * OUTW;
    const int col = ln_col<NTW, ACT>(t, gg, rr, b2, Nhalf);
    const bool ok = ln_col_ok<NTW, ACT>(t, gg, rr, b2, p.N, Nhalf);
    csL[i] = ok ? p.colsum[col] : 0.0f;
    bpL[i] = ok ? p.bprime[col] : 0.0f;
  }

  // ---- staging of one block of rows: x -> LDS, statistics on the way ---------------------------
  // fetch() only issues loads (clamped addresses, nothing touches the results); stash() consumes
  // them one iteration later, applies the zero padding and forms the row statistics.
  constexpr int items = RB * CPR;
  constexpr int PFMAX = (items + 255) / 256;
  frag xr[PFMAX];
  auto fetch = [&](int64_t rb) {
#pragma unroll
    for (int i = 0; i < PFMAX; ++i) {
      const int item = tid + 256 * i;
      const int row = (item < items ? item : 0) / CPR, dc = item % CPR;
      int64_t m = rb * RB + row;
      m = m < p.M ? m : p.M - 1;
      xr[i] = ld8<T>(X + m * p.K + (8 * dc < p.K ? 8 * dc : 0));
    }
  };
  auto stash = [&](int64_t rb, int buf, bool valid) {
    T* xd = Xs + buf * RB * L::XSTR;
    float mu_s[PFMAX], rs_s[PFMAX];
#pragma unroll
    for (int i = 0; i < PFMAX; ++i) {
      const int item = tid + 256 * i;
      mu_s[i] = 0.0f; rs_s[i] = 0.0f;
      if (items % 256 == 0 || item < items) {   // compile-time true for whole multiples: no branch
        const int row = item / CPR, dc = item % CPR;
        const int64_t m = rb * RB + row;
        const bool live = m < p.M && 8 * dc < p.K;
        const frag xv = live ? xr[i] : frag_zero<T>();
        st8<T>(xd + row * L::XSTR + 8 * dc, xv);
        float s = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s += to_f(xv[e]);
        s = group_sum<CPR>(s);
        const float mu = s / (float)p.K;
        float d = 0.0f;
        if (8 * dc < p.K) {
#pragma unroll
          for (int e = 0; e < 8; ++e) { const float c = to_f(xv[e]) - mu; d += c * c; }
        }
        d = group_sum<CPR>(d);
        const float rs = __builtin_amdgcn_rsqf(d / (float)p.K + p.eps);
        mu_s[i] = mu; rs_s[i] = rs;
        if (dc == 0) {
          meanL[buf * RB + row] = mu;
          rstdL[buf * RB + row] = rs;
        }
      }
    }
    // the statistics go to global memory only after every staged register has been consumed: a store
    // issued between two of them would have to be acknowledged before the second one may be read
    if (ACT != LN_ACT_SWIGLU_BWD && blockIdx.y == 0 && valid) {
#pragma unroll
      for (int i = 0; i < PFMAX; ++i) {
        const int item = tid + 256 * i;
        const int64_t m = rb * RB + item / CPR;
        if (item < items && item % CPR == 0 && m < p.M) { p.mean[m] = mu_s[i]; p.rstd[m] = rs_s[i]; }
      }
    }
  };

  // SwiGLU backward: the incoming gradient of a block is requested one iteration ahead (coalesced:
  // lane l takes chunk l % DCH of rows l / DCH + j * DRPI) and consumed in that block's epilogue
  constexpr int DCH = OUTW / 8, DRPI = 64 / DCH, DNL = (ACT == LN_ACT_SWIGLU_BWD) ? 32 / DRPI : 1;
  frag dpre[DNL];
  auto fetch_dh = [&](int64_t rbx) {
    if constexpr (ACT == LN_ACT_SWIGLU_BWD) {
      const T* dsrc = reinterpret_cast<const T*>(p.dout);
      const int ch = l % DCH, r0 = l / DCH;
      const int col = base + 8 * ch < Nhalf ? base + 8 * ch : 0;
#pragma unroll
      for (int j = 0; j < DNL; ++j) {
        int64_t mm = rbx * RB + wr * 32 + r0 + j * DRPI;
        mm = mm < p.M ? mm : p.M - 1;
        dpre[j] = ld8<T>(dsrc + mm * Nhalf + col);
      }
    }
  };
  // flush of one staged output tile: lane l takes chunk l % CH of rows l / CH + j * (64 / CH)
  auto flush = [&](int64_t rbx, const T* tile, T* gbase, int64_t ld, int col_base, int col_limit) {
    constexpr int CH = OUTW / 8, RPI = 64 / CH;
    const int ch = l % CH, r0 = l / CH;
#pragma unroll 2
    for (int j = 0; j < 32 / RPI; ++j) {
      const int row = r0 + j * RPI;
      const int64_t mm = rbx * RB + wr * 32 + row;
      const frag v = ld8<T>(tile + row * OSTR + 8 * ch);
      if (mm < p.M && col_base + 8 * ch < col_limit) st8<T>(gbase + mm * ld + col_base + 8 * ch, v);
    }
  };
  // The results of a block stay in the wavefront's LDS tile and are stored one iteration later,
  // right after the loads of the block after next have been requested: see the loop.
  auto flush_block = [&](int64_t rbx) {
    if constexpr (ACT == LN_ACT_NONE) {
      flush(rbx, Os, reinterpret_cast<T*>(p.out), p.N, base, p.N);
    } else if constexpr (ACT == LN_ACT_SWIGLU) {
      flush(rbx, Os, reinterpret_cast<T*>(p.out), Nhalf, base, Nhalf);
    } else {
      flush(rbx, Os, reinterpret_cast<T*>(p.du), p.N, base, Nhalf);
      flush(rbx, Os + 32 * OSTR, reinterpret_cast<T*>(p.du) + Nhalf, p.N, base, Nhalf);
    }
  };

  // Iteration order (G = gridDim.x row blocks apart): the block of this iteration is already in LDS;
  // after its matrix products the NEXT block's registers (requested one iteration ago, just before
  // that iteration's output stores) are stashed, the block after that is requested, and only then the
  // outputs are stored.  The single point that waits for vector memory therefore only ever waits for
  // loads and stores that are a whole iteration old.
  const int64_t nrb = (p.M + RB - 1) / RB;
  const int64_t G = gridDim.x;
  int64_t rb = blockIdx.x;
  if (rb < nrb) { fetch(rb); stash(rb, 0, true); }
  if (rb + G < nrb) fetch(rb + G);
  if (rb < nrb) fetch_dh(rb);
  // One-time drain: the resident W' registers were loaded above and are first used inside the loop;
  // without this the compiler guards that use with a wait for ALL vector memory in every iteration.
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0), other counters untouched
  int it = 0;
  for (; rb < nrb; rb += G, ++it) {
    const int buf = it & 1;
    // LDS hand-over only.  __syncthreads() would also wait for the output stores of the previous
    // iteration to be acknowledged, which nothing here depends on.
    barrier_keep_vm<63>();

    const T* xt = Xs + buf * RB * L::XSTR + (wr * 32 + x) * L::XSTR;
    f32x16 acc[NTW];
#pragma unroll
    for (int t = 0; t < NTW; ++t) acc[t] = acc_zero();
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const frag bf = ld8<T>(xt + (KP / 2) * g + 8 * s);
#pragma unroll
      for (int t = 0; t < NTW; ++t) acc[t] = mma(af[t][s], bf, acc[t]);
    }
    const float mu_cur = meanL[buf * RB + wr * 32 + x], rs_cur = rstdL[buf * RB + wr * 32 + x];
    // unconditional (past the end it moves stale registers into a buffer nobody reads): a branch here
    // would leave the staged registers "possibly still in flight" for everything that follows
    stash(rb + G, buf ^ 1, rb + G < nrb);
    frag dcur[DNL];
#pragma unroll
    for (int j = 0; j < DNL; ++j) dcur[j] = dpre[j];
    if (rb + 2 * G < nrb) fetch(rb + 2 * G);
    if (rb + G < nrb) fetch_dh(rb + G);
    if (it > 0) flush_block(rb - G);

    const int64_t m = rb * RB + wr * 32 + x;
    const float mu = mu_cur, rs = rs_cur;
    const float c0 = -rs * mu;
    const float* csw = csL + (wn * NTW) * 32 + 16 * g;
    const float* bpw = bpL + (wn * NTW) * 32 + 16 * g;
    if constexpr (ACT == LN_ACT_NONE) {
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        float v[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
          v[r] = __builtin_fmaf(acc[t][r], rs, __builtin_fmaf(c0, csw[t * 32 + r], bpw[t * 32 + r]));
        T* orow = Os + x * OSTR + (NTW * 16) * g + 16 * t;
        st8<T>(orow, cvt8<T>(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]));
        st8<T>(orow + 8, cvt8<T>(v[8], v[9], v[10], v[11], v[12], v[13], v[14], v[15]));
      }
    } else {
      frag dh[2 * TH];
      if constexpr (ACT == LN_ACT_SWIGLU_BWD) {
        // incoming gradient of h: through the second tile, read back one row per lane
        const int ch = l % DCH, r0 = l / DCH;
        T* dtile = Os + 32 * OSTR;
#pragma unroll
        for (int j = 0; j < DNL; ++j) st8<T>(dtile + (r0 + j * DRPI) * OSTR + 8 * ch, dcur[j]);
#pragma unroll
        for (int th = 0; th < TH; ++th) {
          dh[2 * th] = ld8<T>(dtile + x * OSTR + (TH * 16) * g + 16 * th);
          dh[2 * th + 1] = ld8<T>(dtile + x * OSTR + (TH * 16) * g + 16 * th + 8);
        }
      }
#pragma unroll
      for (int th = 0; th < TH; ++th) {
        float a[16], gt[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          a[r] = __builtin_fmaf(acc[th][r], rs, __builtin_fmaf(c0, csw[th * 32 + r], bpw[th * 32 + r]));
          gt[r] = __builtin_fmaf(acc[TH + th][r], rs, __builtin_fmaf(c0, csw[(TH + th) * 32 + r], bpw[(TH + th) * 32 + r]));
        }
        const int lcol = (TH * 16) * g + 16 * th;          // column inside this wavefront's tile
        if constexpr (ACT == LN_ACT_SWIGLU) {
          float h[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) h[r] = a[r] * gt[r] * sigmoidf_fast(gt[r]);
          st8<T>(Os + x * OSTR + lcol, cvt8<T>(h[0], h[1], h[2], h[3], h[4], h[5], h[6], h[7]));
          st8<T>(Os + x * OSTR + lcol + 8, cvt8<T>(h[8], h[9], h[10], h[11], h[12], h[13], h[14], h[15]));
        } else {
          // SwiGLU backward on the recomputed pre-activation (fused_transition.py:44-47)
          float da[16], dg[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float dhv = to_f(r < 8 ? dh[2 * th][r & 7] : dh[2 * th + 1][r & 7]);
            const float sg = sigmoidf_fast(gt[r]);
            const float silu = gt[r] * sg;
            da[r] = dhv * silu;
            dg[r] = dhv * a[r] * (sg + silu * (1.0f - sg));
          }
          T* t0 = Os + x * OSTR + lcol;
          T* t1 = Os + 32 * OSTR + x * OSTR + lcol;
          st8<T>(t0, cvt8<T>(da[0], da[1], da[2], da[3], da[4], da[5], da[6], da[7]));
          st8<T>(t0 + 8, cvt8<T>(da[8], da[9], da[10], da[11], da[12], da[13], da[14], da[15]));
          st8<T>(t1, cvt8<T>(dg[0], dg[1], dg[2], dg[3], dg[4], dg[5], dg[6], dg[7]));
          st8<T>(t1 + 8, cvt8<T>(dg[8], dg[9], dg[10], dg[11], dg[12], dg[13], dg[14], dg[15]));
        }
      }
    }
  }
  if (it > 0) flush_block(rb - G);
}

// Compute units of the current device, asked at every launch: a process may drive devices of different sizes.
static inline int num_cu() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
    return n;
  return 256;
}

template <typename T, int KP, int NTW, int ACT, int WN>
static hipError_t launch_fwd_w(const LnParams& p, hipStream_t stream) {
  using L = LnLayout<T, KP>;
  constexpr int OUTW = (ACT == LN_ACT_NONE) ? NTW * 32 : (NTW / 2) * 32;
  constexpr int RB = 32 * (4 / WN);
  const int NOUT = (ACT == LN_ACT_NONE) ? p.N : p.N / 2;
  const int gy = (NOUT + WN * OUTW - 1) / (WN * OUTW);
  const int64_t nrb = (p.M + RB - 1) / RB;
  int64_t gx = (KP * sizeof(T) > 256 ? 1LL : 2LL) * num_cu() / gy;     // resident work-groups per compute unit: see the launch bounds
  if (gx < 1) gx = 1;
  if (gx > nrb) gx = nrb;
  constexpr int OSTR = OUTW + 16 / (int)sizeof(T);
  constexpr int OTILES = (ACT == LN_ACT_SWIGLU_BWD) ? 2 : 1;
  // the output tiles share their space with the staging area of the resident weights (128 rows)
  constexpr size_t tail_elems = (size_t)4 * OTILES * 32 * OSTR > (size_t)128 * L::XSTR ? (size_t)4 * OTILES * 32 * OSTR
                                                                                        : (size_t)128 * L::XSTR;
  const size_t smem = (size_t)2 * RB * L::XSTR * sizeof(T) + (size_t)4 * RB * 4 + (size_t)2 * 4 * NTW * 32 * 4 +
                      tail_elems * sizeof(T);
  if (smem > 160 * 1024) return hipErrorInvalidValue;   // not reached: launch_fwd_k picks forms that fit
  auto kern = ln_fwd_kernel<T, KP, NTW, ACT, WN>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)gx, (unsigned)gy), dim3(256), smem, stream, p);
  return hipGetLastError();
}

// Tiles per wavefront (NTW) and wavefronts along the columns (WN) by output width; the remaining
// wavefronts of the work-group take further 32-row blocks.
template <typename T, int KP, int ACT> static hipError_t launch_fwd_k(const LnParams& p, hipStream_t stream) {
  const int NOUT = (ACT == LN_ACT_NONE) ? p.N : p.N / 2;
  constexpr bool wide = sizeof(T) == 4 || KP > 128;   // fragments twice as large: halve the resident slice
  if constexpr (ACT == LN_ACT_NONE) {
    // one column tile, four row blocks per work-group: two staged blocks of 128 rows of 512 bytes would not
    // fit the LDS next to the weight staging area, such rows take the two-by-two form
    if constexpr (KP * sizeof(T) <= 256)
      if (NOUT <= 32) return launch_fwd_w<T, KP, 1, ACT, 1>(p, stream);
    if (NOUT <= 128) return launch_fwd_w<T, KP, 2, ACT, 2>(p, stream);
    if constexpr (wide) {
      return launch_fwd_w<T, KP, 2, ACT, 4>(p, stream);
    } else {
      if (NOUT <= 256) return launch_fwd_w<T, KP, 2, ACT, 4>(p, stream);
      // 512-column slabs, unless 256-column slabs pad N up by less and their last slab is at least a quarter
      // full (measured at M = 147456, K = 128: N = 640 70 against 78 us; N = 520 is better off with 512)
      const int pad512 = (NOUT + 511) / 512 * 512, pad256 = (NOUT + 255) / 256 * 256;
      if (pad256 < pad512 && NOUT - (pad256 - 256) >= 64) return launch_fwd_w<T, KP, 2, ACT, 4>(p, stream);
      return launch_fwd_w<T, KP, 4, ACT, 4>(p, stream);
    }
  } else {
    if (NOUT <= 64) return launch_fwd_w<T, KP, 2, ACT, 2>(p, stream);
    // the backward form also holds the incoming gradient and two outputs per column: with four tiles
    // per wavefront it would spill registers
    if constexpr (wide || ACT == LN_ACT_SWIGLU_BWD) {
      return launch_fwd_w<T, KP, 2, ACT, 4>(p, stream);
    } else {
      if (NOUT <= 128) return launch_fwd_w<T, KP, 2, ACT, 4>(p, stream);
      return launch_fwd_w<T, KP, 4, ACT, 4>(p, stream);
    }
  }
}

template <typename T, int KP> static hipError_t launch_fwd_a(const LnParams& p, int act, hipStream_t stream) {
  switch (act) {
    case LN_ACT_NONE: return launch_fwd_k<T, KP, LN_ACT_NONE>(p, stream);
    case LN_ACT_SWIGLU: return launch_fwd_k<T, KP, LN_ACT_SWIGLU>(p, stream);
    case LN_ACT_SWIGLU_BWD: return launch_fwd_k<T, KP, LN_ACT_SWIGLU_BWD>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

template <typename T> hipError_t ln_fwd_dispatch(const LnParams& p, int act, hipStream_t stream) {
  switch (p.KP) {
    case 16: return launch_fwd_a<T, 16>(p, act, stream);
    case 32: return launch_fwd_a<T, 32>(p, act, stream);
    case 64: return launch_fwd_a<T, 64>(p, act, stream);
    case 128: return launch_fwd_a<T, 128>(p, act, stream);
    case 256: return launch_fwd_a<T, 256>(p, act, stream);
    default: return hipErrorInvalidValue;
  }
}




// =================================================================================================
// backward: dx
// =================================================================================================
// RTW row tiles (of 32 rows) per wavefront share every W fragment read from LDS, and the work-group
// streams the whole of W once per 128 * RTW rows: that stream (from L2, through L1) is as large as
// dOut itself at RTW = 1, so two tiles per wavefront are used where the registers allow it.
template <typename T, int KP, int RTW>
__global__ void __launch_bounds__(256, KP * sizeof(T) > 256 ? 1 : 2) ln_bwd_dx_kernel(const LnParams p, const T* __restrict__ dY) {
  using frag = frag_t<T>;
  constexpr int KPT = KP < 32 ? 32 : KP;       // rows of the W operand, padded to whole tiles
  constexpr int KT = KPT / 32;
  constexpr int NC = 64;                       // columns of N per staged chunk
  constexpr int UNIT = 16 / (int)sizeof(T);
  constexpr int WSTR = ((NC / UNIT) % 2 == 0) ? NC + UNIT : NC;
  constexpr int WITEMS = KPT * (NC / 8);
  constexpr int PF = (WITEMS + 255) / 256;
  constexpr int RBW = 128 * RTW;               // rows per work-group block

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Ws = reinterpret_cast<T*>(smem_raw);      // [2][KPT][WSTR]

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const T* Wsrc = reinterpret_cast<const T*>(p.W);   // the weights as stored; gamma multiplies the fp32 products below
  const T* gam = reinterpret_cast<const T*>(p.gamma);
  const T* X = reinterpret_cast<const T*>(p.x);
  T* dX = reinterpret_cast<T*>(p.dx);
  const int N = p.N, K = p.K;
  const int nchunks = (N + NC - 1) / NC;

  // W chunk staging: loads are only issued here (clamped addresses), padding is applied at the stash
  frag wr_[PF];
  auto fetch_w = [&](int c) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int item = tid + 256 * i;
      const int k = (item < WITEMS ? item : 0) / (NC / 8), nc = item % (NC / 8);
      const int n = c * NC + 8 * nc;
      wr_[i] = ld8<T>(Wsrc + (int64_t)(k < K ? k : 0) * N + (n < N ? n : 0));
    }
  };
  auto stash_w = [&](int c, int buf) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int item = tid + 256 * i;
      if (WITEMS % 256 == 0 || item < WITEMS) {
        const int k = item / (NC / 8), nc = item % (NC / 8);
        const bool ok = k < K && c * NC + 8 * nc < N;
        st8<T>(Ws + (buf * KPT + k) * WSTR + 8 * nc, ok ? wr_[i] : frag_zero<T>());
      }
    }
  };

  const int64_t nrb = (p.M + RBW - 1) / RBW;
  for (int64_t rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    int64_t m[RTW], mc[RTW];
    const T* dyrow[RTW];
    f32x16 acc[RTW][KT];
#pragma unroll
    for (int j = 0; j < RTW; ++j) {
      m[j] = rb * RBW + (j * 4 + w) * 32 + x;
      mc[j] = m[j] < p.M ? m[j] : p.M - 1;      // rows past the end work on a copy of the last row, store nothing
      dyrow[j] = dY + mc[j] * N;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) acc[j][kt] = acc_zero();
    }

    frag yb[RTW][4];
    auto fetch_y = [&](int c) {
#pragma unroll
      for (int j = 0; j < RTW; ++j)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const int n = c * NC + 32 * g + 8 * s;
          yb[j][s] = ld8<T>(dyrow[j] + (n < N ? n : 0));
        }
    };
    __syncthreads();          // the previous row block is done with both W buffers
    fetch_w(0);
    fetch_y(0);
    stash_w(0, 0);
    __syncthreads();
    for (int c = 0; c < nchunks; ++c) {
      const int buf = c & 1;
      frag yc[RTW][4];
#pragma unroll
      for (int j = 0; j < RTW; ++j)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const bool ok = c * NC + 32 * g + 8 * s < N;     // only the last chunk of a ragged N
          yc[j][s] = ok ? yb[j][s] : frag_zero<T>();
          pin(yc[j][s]);
        }
      const int cn = c + 1 < nchunks ? c + 1 : c;          // the last chunk is requested twice: no branch
      fetch_w(cn);
      fetch_y(cn);
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const T* wrow = Ws + (buf * KPT + dsel<KPT>(kt, x)) * WSTR + 32 * g;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const frag wf = ld8<T>(wrow + 8 * s);
#pragma unroll
          for (int j = 0; j < RTW; ++j) acc[j][kt] = mma(wf, yc[j][s], acc[j][kt]);
        }
      }
      stash_w(cn, buf ^ 1);
      __syncthreads();
    }

    // ---- LayerNorm backward on the rows this lane owns: register r of tile kt <-> k = (KPT/2) g + 16 kt + r
#pragma unroll
    for (int j = 0; j < RTW; ++j) {
      const float mu = p.mean[mc[j]], rs = p.rstd[mc[j]];
      float xh[KT][16];
      float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int k0 = (KPT / 2) * g + 16 * kt + 8 * u;
          const frag xv = k0 < K ? ld8<T>(X + mc[j] * K + k0) : frag_zero<T>();
          const frag gv = k0 < K ? ld8<T>(gam + k0) : frag_zero<T>();
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float v = k0 < K ? (to_f(xv[e]) - mu) * rs : 0.0f;
            xh[kt][8 * u + e] = v;
            acc[j][kt][8 * u + e] *= to_f(gv[e]);            // dOut W^T times gamma, in fp32
            s1 += v * acc[j][kt][8 * u + e];
            s2 += acc[j][kt][8 * u + e];
          }
        }
      }
      s1 += __shfl_xor(s1, 32);
      s2 += __shfl_xor(s2, 32);
      const float c1 = s1 / (float)K, c2 = s2 / (float)K;
      if (m[j] < p.M) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int k0 = (KPT / 2) * g + 16 * kt + 8 * u;
            if (k0 < K) {
              float o[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) o[e] = (acc[j][kt][8 * u + e] - (xh[kt][8 * u + e] * c1 + c2)) * rs;
              st8<T>(dX + m[j] * K + k0, cvt8<T>(o[0], o[1], o[2], o[3], o[4], o[5], o[6], o[7]));
            }
          }
      }
    }
  }
}

// -------------------------------------------------------------------------------------------------
// dx for K <= 128 (four k tiles of 32), N <= 16 * NSTEPS * NH <= 1024 and 16-bit element types.  A
// wavefront owns one k tile and one of NH halves of N and keeps that slice of W in registers for the
// whole kernel (A operand), so the only streams are dOut and x in and dx out.  dOut and x rows are
// fetched coalesced one block ahead, staged in LDS and read by all wavefronts; with NH = 2 the two
// halves of a k tile are added through LDS; the LayerNorm backward needs row sums over all K, which the
// k tiles exchange through LDS; dx leaves through an LDS tile so that it is stored in whole lines.
// ADD: the rows of LnParams::dx_add are staged beside x and added to dx before its rounding (a compile-time
// variant: the widest shapes have no registers to spare for a run-time one).
template <typename T, int NSTEPS, int NH, bool ADD>
__global__ void __launch_bounds__(256 * NH, 2 / NH) ln_bwd_dx_res_kernel(const LnParams p, const T* __restrict__ dY) {
  using frag = frag_t<T>;
  static_assert(sizeof(T) == 2, "16-bit element types only");
  constexpr int NTHR = 256 * NH;
  constexpr int NP = 16 * NSTEPS * NH;         // padded N
  constexpr int YSTR = NP + 8, XSTR = 128 + 8;
  constexpr int YCH = NP / 8;                  // 16-byte chunks per dOut row
  constexpr int YPF = 32 * YCH / NTHR;         // staged dOut chunks per thread
  constexpr int XPF = 512 / NTHR;              // staged x chunks per thread
  static_assert(32 * YCH % NTHR == 0, "whole number of chunks per thread");

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Ys = reinterpret_cast<T*>(smem_raw);      // [32][YSTR]  dOut block (also used to hand out W)
  T* Xs = Ys + 32 * YSTR;                      // [32][XSTR]  x block
  T* Os = Xs + 32 * XSTR;                      // [32][XSTR]  dx block
  T* Rs = Os + 32 * XSTR;                      // [32][XSTR]  rows of dx_add (the gradient that skips the operator; ADD only)
  float* part = reinterpret_cast<float*>(Os + (ADD ? 2 : 1) * 32 * XSTR);   // [4][32][2] per-k-tile row sums
  float* pair = part + 4 * 32 * 2;                          // [4][16][64] second half's accumulators (NH = 2)
  T* gl = reinterpret_cast<T*>(pair + (NH == 2 ? 4 * 16 * 64 : 0));   // [128] gamma, zero past K

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int kt = w & 3, nh = w >> 2;
  const int N = p.N, K = p.K;
  const T* Wraw = reinterpret_cast<const T*>(p.W);
  const T* gam = reinterpret_cast<const T*>(p.gamma);
  const T* X = reinterpret_cast<const T*>(p.x);
  T* dX = reinterpret_cast<T*>(p.dx);
  const T* DR = ADD ? reinterpret_cast<const T*>(p.dx_add) : nullptr;

  if (tid < 16) st8<T>(gl + 8 * tid, 8 * tid < K ? ld8<T>(gam + 8 * tid) : frag_zero<T>());   // published by the barriers below

  // ---- resident slice of W (rows 32 kt .. 32 kt + 31, columns of half nh), handed out through the
  // dOut staging area one k tile at a time
  frag af[NSTEPS];
  for (int ww = 0; ww < 4; ++ww) {
    frag tmp[YPF];
#pragma unroll
    for (int i = 0; i < YPF; ++i) {
      const int item = tid + NTHR * i;
      const int r = item / YCH, c = item % YCH;
      const int k = 32 * ww + r;
      const bool ok = k < K && 8 * c < N;
      // the weights as stored: gamma multiplies the fp32 products (below), as the reference applies it
      tmp[i] = ld8<T>(Wraw + (int64_t)(ok ? k : 0) * N + (ok ? 8 * c : 0));
    }
#pragma unroll
    for (int i = 0; i < YPF; ++i) {
      const int item = tid + NTHR * i;
      const int r = item / YCH, c = item % YCH;
      const bool ok = 32 * ww + r < K && 8 * c < N;
      st8<T>(Ys + r * YSTR + 8 * c, ok ? tmp[i] : frag_zero<T>());
    }
    __syncthreads();
    if (kt == ww) {
      // operand row x holds tile row unperm32(x): accumulator register i of half g <-> k = 32 kt + 16 g + i
#pragma unroll
      for (int s = 0; s < NSTEPS; ++s)
        af[s] = ld8<T>(Ys + unperm32(x) * YSTR + nh * (16 * NSTEPS) + 16 * s + 8 * g);
    }
    __syncthreads();
  }

  // ---- staging registers: dOut and x chunks of the next block, mean / rstd of the lane's row --------
  frag yr[YPF], xr[XPF], rr[ADD ? XPF : 1];
  float mu_n = 0.0f, rs_n = 0.0f;
  auto fetch = [&](int64_t rb) {
#pragma unroll
    for (int i = 0; i < YPF; ++i) {
      const int item = tid + NTHR * i;
      const int r = item / YCH, c = item % YCH;
      int64_t m = rb * 32 + r;
      m = m < p.M ? m : p.M - 1;
      yr[i] = ld8<T>(dY + m * N + (8 * c < N ? 8 * c : 0));
    }
#pragma unroll
    for (int i = 0; i < XPF; ++i) {
      const int item = tid + NTHR * i;
      const int r = item >> 4, c = item & 15;
      int64_t m = rb * 32 + r;
      m = m < p.M ? m : p.M - 1;
      xr[i] = ld8<T>(X + m * K + (8 * c < K ? 8 * c : 0));
      if constexpr (ADD) rr[i] = ld8<T>(DR + m * K + (8 * c < K ? 8 * c : 0));
    }
    int64_t m = rb * 32 + x;
    m = m < p.M ? m : p.M - 1;
    mu_n = p.mean[m];
    rs_n = p.rstd[m];
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < YPF; ++i) {
      const int item = tid + NTHR * i;
      const int r = item / YCH, c = item % YCH;
      st8<T>(Ys + r * YSTR + 8 * c, 8 * c < N ? yr[i] : frag_zero<T>());
    }
#pragma unroll
    for (int i = 0; i < XPF; ++i) {
      const int item = tid + NTHR * i;
      const int r = item >> 4, c = item & 15;
      st8<T>(Xs + r * XSTR + 8 * c, 8 * c < K ? xr[i] : frag_zero<T>());
      if constexpr (ADD) st8<T>(Rs + r * XSTR + 8 * c, rr[i]);
    }
  };
  // dx block of the previous iteration: consecutive lanes take consecutive 16-byte chunks (whole lines)
  auto flush = [&](int64_t rb) {
#pragma unroll
    for (int i = 0; i < XPF; ++i) {
      const int item = tid + NTHR * i;
      const int r = item >> 4, c = item & 15;
      const int64_t m = rb * 32 + r;
      const frag v = ld8<T>(Os + r * XSTR + 8 * c);
      if (m < p.M && 8 * c < K) st8<T>(dX + m * K + 8 * c, v);
    }
  };

  const int64_t nrb = (p.M + 31) / 32;
  const int64_t G = gridDim.x;
  int64_t rb = blockIdx.x;
  if (rb < nrb) fetch(rb);
  __builtin_amdgcn_s_waitcnt(0x0F70);   // one-time drain: nothing older than the staged block is in flight
  int it = 0;
  for (; rb < nrb; rb += G, ++it) {
    // (A) everybody is done with the LDS blocks of the previous iteration
    barrier_keep_vm<63>();
    stash();
    const float mu = mu_n, rs = rs_n;
    fetch(rb + G < nrb ? rb + G : rb);          // the tail repeats the last block rather than branching
    if (it > 0) flush(rb - G);
    // (B) this iteration's dOut / x are visible
    barrier_keep_vm<63>();

    f32x16 acc = acc_zero();
    const T* yrow = Ys + x * YSTR + nh * (16 * NSTEPS) + 8 * g;
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s) acc = mma(af[s], ld8<T>(yrow + 16 * s), acc);

    if constexpr (NH == 2) {
      // the upper half of N hands its partial products to the lower half's wavefront of the same k tile
      if (nh == 1) {
#pragma unroll
        for (int i = 0; i < 16; ++i) pair[(kt * 16 + i) * 64 + l] = acc[i];
      }
      barrier_keep_vm<63>();
      if (nh == 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] += pair[(kt * 16 + i) * 64 + l];
      }
    }

    // LayerNorm backward: a lane of half 0 holds w[m][32 kt + 16 g + 0..15]
    float s1 = 0.0f, s2 = 0.0f;
    if (nh == 0) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        // dOut W^T times gamma in fp32, formed where it is used (here and below) instead of once in place (rewriting
        // the accumulator block costs the compiler a second copy of it); four columns at a time, so that the
        // operands of one quarter are all that is in registers beside the accumulators
        using half = typename Frag<T>::half;
        const int k0 = 32 * kt + 16 * g + 4 * q;
        const half xq = *reinterpret_cast<const half*>(Xs + x * XSTR + k0);
        const half gq = *reinterpret_cast<const half*>(gl + k0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = k0 + e < K ? (to_f(xq[e]) - mu) * rs : 0.0f;
          const float wg = acc[4 * q + e] * to_f(gq[e]);
          s1 += v * wg;
          s2 += wg;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      s1 += __shfl_xor(s1, 32);
      s2 += __shfl_xor(s2, 32);
      if (g == 0) { part[(kt * 32 + x) * 2] = s1; part[(kt * 32 + x) * 2 + 1] = s2; }
    }
    // (C) row sums of all four k tiles
    barrier_keep_vm<63>();
    if (nh == 0) {
      float t1 = 0.0f, t2 = 0.0f;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) { t1 += part[(ww * 32 + x) * 2]; t2 += part[(ww * 32 + x) * 2 + 1]; }
      const float c1 = t1 / (float)K, c2 = t2 / (float)K;
      T* orow = Os + x * XSTR + 32 * kt + 16 * g;
#pragma unroll
      for (int q = 0; q < 4; ++q) {                // four columns at a time, as above; x_hat is formed again from the
        using half = typename Frag<T>::half;       // staged row rather than kept in sixteen registers across the barrier
        const int k0 = 32 * kt + 16 * g + 4 * q;
        const half xq = *reinterpret_cast<const half*>(Xs + x * XSTR + k0);
        const half gq = *reinterpret_cast<const half*>(gl + k0);
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = k0 + e < K ? (to_f(xq[e]) - mu) * rs : 0.0f;
          o[e] = (acc[4 * q + e] * to_f(gq[e]) - (v * c1 + c2)) * rs;
        }
        if constexpr (ADD) {                       // summed in fp32, rounded once below
          const half rq = *reinterpret_cast<const half*>(Rs + x * XSTR + 32 * kt + 16 * g + 4 * q);
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] += to_f(rq[e]);
        }
        half oq;
#pragma unroll
        for (int e = 0; e < 4; ++e) oq[e] = (T)o[e];
        *reinterpret_cast<half*>(orow + 4 * q) = oq;
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  barrier_keep_vm<63>();
  if (it > 0) flush(rb - G);
}

template <typename T, int NSTEPS, int NH, bool ADD>
static hipError_t launch_dx_res_a(const LnParams& p, const void* dY, hipStream_t stream) {
  constexpr int NP = 16 * NSTEPS * NH;
  const size_t smem = (size_t)(32 * (NP + 8) + (ADD ? 3 : 2) * 32 * (128 + 8)) * sizeof(T) + 4 * 32 * 2 * 4 +
                      (NH == 2 ? (size_t)4 * 16 * 64 * 4 : 0) + 128 * sizeof(T);
  const int64_t nrb = (p.M + 31) / 32;
  int64_t gx = (2LL / NH) * num_cu();
  if (gx > nrb) gx = nrb;
  auto kern = ln_bwd_dx_res_kernel<T, NSTEPS, NH, ADD>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)gx), dim3(256 * NH), smem, stream, p, reinterpret_cast<const T*>(dY));
  return hipGetLastError();
}

template <typename T, int NSTEPS, int NH>
static hipError_t launch_dx_res(const LnParams& p, const void* dY, hipStream_t stream) {
  return p.dx_add ? launch_dx_res_a<T, NSTEPS, NH, true>(p, dY, stream) : launch_dx_res_a<T, NSTEPS, NH, false>(p, dY, stream);
}

template <typename T, int KP, int RTW>
static hipError_t launch_dx_r(const LnParams& p, const void* dY, hipStream_t stream) {
  constexpr int KPT = KP < 32 ? 32 : KP;
  constexpr int UNIT = 16 / (int)sizeof(T);
  constexpr int WSTR = ((64 / UNIT) % 2 == 0) ? 64 + UNIT : 64;
  const size_t smem = (size_t)2 * KPT * WSTR * sizeof(T);
  const int64_t nrb = (p.M + 128 * RTW - 1) / (128 * RTW);
  int64_t gx = (KP * sizeof(T) > 256 ? 1LL : 2LL) * num_cu();
  if (gx > nrb) gx = nrb;
  auto kern = ln_bwd_dx_kernel<T, KP, RTW>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)gx), dim3(256), smem, stream, p, reinterpret_cast<const T*>(dY));
  return hipGetLastError();
}

// Two row tiles per wavefront halve the W stream but double the block: the grid runs in whole rounds
// of 2 * CUs resident work-groups, so the larger block only pays when it does not add a partly
// filled round (a double block is priced at 1.7 single ones).
template <typename T, int KP> static hipError_t launch_dx_t(const LnParams& p, const void* dY, hipStream_t stream) {
  if constexpr (sizeof(T) == 2 && KP == 128) {
    // register-resident W: K in (64, 128], 64 <= N <= 1024
    if (p.N >= 64) {
      if (p.N <= 128) return launch_dx_res<T, 8, 1>(p, dY, stream);
      if (p.N <= 256) return launch_dx_res<T, 16, 1>(p, dY, stream);
      if (p.N <= 512) return launch_dx_res<T, 32, 1>(p, dY, stream);
      // eight wavefronts, N split in halves; 640 columns cover the pair stack's 520- and 640-wide projections
      // without running the products over 1024 padded columns
      if (p.N <= 640) return launch_dx_res<T, 20, 2>(p, dY, stream);
      if (p.N <= 1024) return launch_dx_res<T, 32, 2>(p, dY, stream);
    }
  }
  if constexpr (sizeof(T) == 2 && KP <= 128) {
    const int64_t slots = 2LL * num_cu();
    const int64_t r1 = ((p.M + 127) / 128 + slots - 1) / slots, r2 = ((p.M + 255) / 256 + slots - 1) / slots;
    if (1.7 * (double)r2 < (double)r1) return launch_dx_r<T, KP, 2>(p, dY, stream);
  }
  return launch_dx_r<T, KP, 1>(p, dY, stream);
}

template <typename T> hipError_t ln_dx_dispatch(const LnParams& p, const void* dY, hipStream_t stream) {
  switch (p.KP) {
    case 16: return launch_dx_t<T, 16>(p, dY, stream);
    case 32: return launch_dx_t<T, 32>(p, dY, stream);
    case 64: return launch_dx_t<T, 64>(p, dY, stream);
    case 128: return launch_dx_t<T, 128>(p, dY, stream);
    case 256: return launch_dx_t<T, 256>(p, dY, stream);
    default: return hipErrorInvalidValue;
  }
}


// =================================================================================================
// backward: G = x_hat^T dOut, s = colsum(dOut), then dW / dgamma / dbeta / db
// =================================================================================================
// Row stride (elements) of the dW kernel's LDS tiles.  The tiles are read with transposing reads: a group of 16
// lanes touches 32 contiguous bytes in each of four consecutive rows, so the rows must start 8 banks (32 bytes modulo
// 256) apart or further; a stride of 4 banks (widths that are multiples of 128 16-bit elements, padded by one
// 16-byte unit) made every such read a two-way bank conflict.
template <typename T> constexpr int dw_tile_stride(int width) {
  constexpr int UNIT = 16 / (int)sizeof(T);
  int stride = ((width / UNIT) % 2 == 0) ? width + UNIT : width;
  if (sizeof(T) == 2 && (stride * (int)sizeof(T) / 4) % 64 == 4) stride += UNIT;
  return stride;
}

template <int KP> struct DwShape {
  static constexpr int KPT = KP < 32 ? 32 : KP;
  static constexpr int WK = KPT >= 256 ? 4 : (KPT >= 64 ? 2 : 1);   // wavefronts along k
  static constexpr int KTW = KPT / (32 * WK);                        // k tiles per wavefront
  static constexpr int WNN = 4 / WK;                                  // wavefronts along n
  static constexpr int NTW = WNN == 4 ? 1 : 2;                        // n tiles per wavefront
  static constexpr int CW = WNN * NTW * 32;                           // columns per work-group
};

template <typename T, int KP>
__global__ void __launch_bounds__(256, 2) ln_bwd_dw_kernel(const LnParams p, const T* __restrict__ dY) {
  using frag = frag_t<T>;
  using Sh = DwShape<KP>;
  constexpr int KPT = Sh::KPT, KTW = Sh::KTW, WNN = Sh::WNN, NTW = Sh::NTW, CW = Sh::CW;
  constexpr int RT = 64;                       // rows per staged tile
  constexpr int UNIT = 16 / (int)sizeof(T);
  constexpr int XSTR = dw_tile_stride<T>(KPT);
  constexpr int YSTR = dw_tile_stride<T>(CW);
  constexpr int XI = RT * (KPT / 8), YI = RT * (CW / 8);
  constexpr int PFX = (XI + 255) / 256, PFY = (YI + 255) / 256;
  static_assert(256 % (CW / 8) == 0, "a thread must keep one column chunk");

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Xs = reinterpret_cast<T*>(smem_raw);      // [2][RT][XSTR]  normalised rows
  T* Ys = Xs + 2 * RT * XSTR;                  // [2][RT][YSTR]

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int wk = w / WNN, wn = w % WNN;
  const int range = blockIdx.x, cb = blockIdx.y * CW;
  const int64_t m_begin = (int64_t)range * p.rows_per_range;
  const int64_t m_end = m_begin + p.rows_per_range < p.M ? m_begin + p.rows_per_range : p.M;
  const T* X = reinterpret_cast<const T*>(p.x);
  const int K = p.K, N = p.N;

  f32x16 acc[KTW][NTW];
#pragma unroll
  for (int a = 0; a < KTW; ++a)
#pragma unroll
    for (int b = 0; b < NTW; ++b) acc[a][b] = acc_zero();
  float colsum[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) colsum[e] = 0.0f;

  // fetch() only issues loads (clamped addresses, nothing touches the results); stash() consumes them
  // one tile later and applies the padding
  frag xr[PFX], yr[PFY];
  float mur[PFX], rsr[PFX];
  auto fetch = [&](int64_t m0) {
#pragma unroll
    for (int i = 0; i < PFX; ++i) {
      const int item = tid + 256 * i;
      const int row = (item < XI ? item : 0) / (KPT / 8), dc = item % (KPT / 8);
      int64_t m = m0 + row;
      m = m < m_end ? m : m_end - 1;
      xr[i] = ld8<T>(X + m * K + (8 * dc < K ? 8 * dc : 0));
      mur[i] = p.mean[m];
      rsr[i] = p.rstd[m];
    }
#pragma unroll
    for (int i = 0; i < PFY; ++i) {
      const int item = tid + 256 * i;
      const int row = (item < YI ? item : 0) / (CW / 8), cc = item % (CW / 8);
      int64_t m = m0 + row;
      m = m < m_end ? m : m_end - 1;
      const int n = cb + 8 * cc;
      yr[i] = ld8<T>(dY + m * N + (n < N ? n : 0));
    }
  };
  auto stash = [&](int64_t m0, int buf) {
#pragma unroll
    for (int i = 0; i < PFX; ++i) {
      const int item = tid + 256 * i;
      if (XI % 256 == 0 || item < XI) {
        const int row = item / (KPT / 8), dc = item % (KPT / 8);
        const bool live = m0 + row < m_end && 8 * dc < K;
        const float rs = live ? rsr[i] : 0.0f;            // rows / columns past the end: zero
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (to_f(xr[i][e]) - mur[i]) * rs;
        st8<T>(Xs + (buf * RT + row) * XSTR + 8 * dc, cvt8<T>(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]));
      }
    }
#pragma unroll
    for (int i = 0; i < PFY; ++i) {
      const int item = tid + 256 * i;
      if (YI % 256 == 0 || item < YI) {
        const int row = item / (CW / 8), cc = item % (CW / 8);
        const bool live = m0 + row < m_end && cb + 8 * cc < N;
        const frag yv = live ? yr[i] : frag_zero<T>();
        st8<T>(Ys + (buf * RT + row) * YSTR + 8 * cc, yv);
#pragma unroll
        for (int e = 0; e < 8; ++e) colsum[e] += to_f(yv[e]);
      }
    }
  };

  if (m_begin < m_end) fetch(m_begin);
  int it = 0;
  for (int64_t m0 = m_begin; m0 < m_end; m0 += RT, ++it) {
    const int buf = it & 1;
    stash(m0, buf);
    barrier_keep_vm<63>();                              // LDS hand-over only (double-buffered tiles)
    fetch(m0 + RT < m_end ? m0 + RT : m0);              // the tail repeats the last tile: no branch around loads
    __builtin_amdgcn_sched_barrier(0);                  // keep the requests here: the scheduler would sink them to their use
    const T* xs = Xs + buf * RT * XSTR;
    const T* ys = Ys + buf * RT * YSTR;
#pragma unroll
    for (int st = 0; st < RT / 16; ++st) {
      frag bf[NTW];
#pragma unroll
      for (int b = 0; b < NTW; ++b) {
        const int nb = (wn * NTW + b) * 32;
        bf[b] = TrRead<T>::read(ys, YSTR, 16 * st, g, l, nb + plain_chunk(l), nb + x);
      }
#pragma unroll
      for (int a = 0; a < KTW; ++a) {
        const int kb = (wk * KTW + a) * 32;
        const frag af = TrRead<T>::read(xs, XSTR, 16 * st, g, l, kb + plain_chunk(l), kb + x);
#pragma unroll
        for (int b = 0; b < NTW; ++b) acc[a][b] = mma(af, bf[b], acc[a][b]);
      }
    }
  }

  // ---- partial G: natural accumulator layout, lane = column n, registers = rows k ----------------
  float* Gp = p.Gpart + (int64_t)range * K * N;
#pragma unroll
  for (int a = 0; a < KTW; ++a)
#pragma unroll
    for (int b = 0; b < NTW; ++b) {
      const int n = cb + (wn * NTW + b) * 32 + x;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int k = (wk * KTW + a) * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (k < K && n < N) Gp[(int64_t)k * N + n] = acc[a][b][r];
      }
    }
  // ---- partial column sums: threads with the same column chunk are 256 / (CW/8) apart ------------
  __syncthreads();
  float* red = reinterpret_cast<float*>(smem_raw);       // [256][8]
#pragma unroll
  for (int e = 0; e < 8; ++e) red[tid * 8 + e] = colsum[e];
  __syncthreads();
  if (tid < CW) {
    const int cc = tid / 8, e = tid % 8;
    float s = 0.0f;
    for (int j = cc; j < 256; j += CW / 8) s += red[j * 8 + e];
    const int n = cb + tid;
    if (n < N) p.spart[(int64_t)range * N + n] = s;
  }
}

// Sum of the per-range partials in a fixed order, first level.  A work-group owns 256 consecutive
// float4 groups (4 KiB per range: long contiguous reads) of the flattened [K, N] matrix and one of
// LN_RED_GROUPS interleaved sets of ranges; it adds ranges rq, rq + 8, ... and overwrites range rq.  The
// finalize kernel adds the remaining (at most 8) ranges.  Work-groups past the matrix sum the column
// sums completely.
constexpr int LN_RED_GROUPS = 8;
template <typename T>
__global__ void __launch_bounds__(256) ln_bwd_reduce_kernel(float* __restrict__ Gpart, float* __restrict__ spart,
                                                            int64_t kn, int N, int R, int g_blocks) {
  const int tid = threadIdx.x;
  if ((int)blockIdx.x < g_blocks * LN_RED_GROUPS) {
    const int cb = (int)blockIdx.x / LN_RED_GROUPS, rq = (int)blockIdx.x % LN_RED_GROUPS;
    const int64_t e = ((int64_t)cb * 256 + tid) * 4;
    if (e < kn && rq < R) {
      f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 8
      for (int r = rq; r < R; r += LN_RED_GROUPS) acc += *reinterpret_cast<const f32x4*>(Gpart + (int64_t)r * kn + e);
      *reinterpret_cast<f32x4*>(Gpart + (int64_t)rq * kn + e) = acc;
    }
  } else {
    const int n = ((int)blockIdx.x - g_blocks * LN_RED_GROUPS) * 256 + tid;
    if (n < N) {
      // sixteen independent loads at a time (a one-by-one loop would pay the memory latency R times)
      float sacc = 0.0f;
      int r = 0;
      for (; r + 16 <= R; r += 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = spart[(int64_t)(r + u) * N + n];
#pragma unroll
        for (int u = 0; u < 16; ++u) sacc += v[u];
      }
      for (; r < R; ++r) sacc += spart[(int64_t)r * N + n];
      spart[n] = sacc;
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) ln_bwd_finalize_kernel(const LnParams p) {
  const int k = blockIdx.x, tid = threadIdx.x;
  const T* W = reinterpret_cast<const T*>(p.W);
  const float gam = to_f(reinterpret_cast<const T*>(p.gamma)[k]);
  const float bet = p.beta ? to_f(reinterpret_cast<const T*>(p.beta)[k]) : 0.0f;
  // the parameter gradients leave in fp32 or already rounded to the element type (one conversion here instead
  // of one more pass over each of them)
  auto put = [&](void* base, int64_t i, float v) {
    if (p.grads_as_x) reinterpret_cast<T*>(base)[i] = (T)v;
    else reinterpret_cast<float*>(base)[i] = v;
  };
  float dg = 0.0f, dbt = 0.0f;
  for (int n = tid; n < p.N; n += 256) {
    const int64_t kn = (int64_t)p.K * p.N;
    const int nr = p.R < LN_RED_GROUPS ? p.R : LN_RED_GROUPS;
    // all loads first (independent), then the sum in its fixed order: a load-add chain would pay the
    // memory latency once per range
    float gv[LN_RED_GROUPS];
#pragma unroll
    for (int r = 0; r < LN_RED_GROUPS; ++r)
      gv[r] = r < nr ? p.Gpart[(int64_t)r * kn + (int64_t)k * p.N + n] : 0.0f;
    float G = 0.0f;
#pragma unroll
    for (int r = 0; r < LN_RED_GROUPS; ++r) G += gv[r];
    const float s = p.spart[n];
    const float wv = to_f(W[(int64_t)k * p.N + n]);
    put(p.dW, (int64_t)k * p.N + n, gam * G + bet * s);
    dg += wv * G;
    dbt += wv * s;
    if (k == 0 && p.db) put(p.db, n, s);
  }
  __shared__ float r1[256], r2[256];
  r1[tid] = dg; r2[tid] = dbt;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (tid < o) { r1[tid] += r1[tid + o]; r2[tid] += r2[tid + o]; }
    __syncthreads();
  }
  if (tid == 0) {
    put(p.dgamma, k, r1[0]);
    if (p.dbeta) put(p.dbeta, k, r2[0]);
  }
}

template <typename T> static hipError_t launch_dw_reduce(const LnParams& p, hipStream_t stream);

template <typename T, int KP> static hipError_t launch_dw_t(const LnParams& p, const void* dY, hipStream_t stream) {
  using Sh = DwShape<KP>;
  constexpr int UNIT = 16 / (int)sizeof(T);
  constexpr int XSTR = dw_tile_stride<T>(Sh::KPT);
  constexpr int YSTR = dw_tile_stride<T>(Sh::CW);
  size_t smem = (size_t)2 * 64 * (XSTR + YSTR) * sizeof(T);
  if (smem < 256 * 8 * 4) smem = 256 * 8 * 4;
  const int gy = (p.N + Sh::CW - 1) / Sh::CW;
  auto kern = ln_bwd_dw_kernel<T, KP>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)p.R, (unsigned)gy), dim3(256), smem, stream, p, reinterpret_cast<const T*>(dY));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  return launch_dw_reduce<T>(p, stream);
}

// Fixed-order sum of the per-range partials, then dW / dgamma / dbeta / db.
template <typename T> static hipError_t launch_dw_reduce(const LnParams& p, hipStream_t stream) {
  hipError_t e;
  const int64_t kn = (int64_t)p.K * p.N;
  const int g_blocks = (int)((kn / 4 + 255) / 256);
  const int s_blocks = (p.N + 255) / 256;
  hipLaunchKernelGGL(ln_bwd_reduce_kernel<T>, dim3((unsigned)(g_blocks * LN_RED_GROUPS + s_blocks)), dim3(256), 0, stream,
                     p.Gpart, p.spart, kn, p.N, p.R, g_blocks);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ln_bwd_finalize_kernel<T>, dim3((unsigned)p.K), dim3(256), 0, stream, p);
  return hipGetLastError();
}

template <typename T> hipError_t ln_dw_dispatch(const LnParams& p, const void* dY, hipStream_t stream) {
  switch (p.KP) {
    case 16: return launch_dw_t<T, 16>(p, dY, stream);
    case 32: return launch_dw_t<T, 32>(p, dY, stream);
    case 64: return launch_dw_t<T, 64>(p, dY, stream);
    case 128: return launch_dw_t<T, 128>(p, dY, stream);
    case 256: return launch_dw_t<T, 256>(p, dY, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mf

#include "lnlinear_swiglu_bwd.h"

namespace mf {

// SwiGLU backward in three kernels: the fused pass (weight-gradient partials, and each column block's share of
// dU W^T in place of dU itself), the reduction of the partials, and dx from the shares (times gamma).  Returns
// hipErrorNotSupported for shapes the fused kernel does not take (the caller then runs the separate kernels).
// With MF_LN_DU_FORM the fused pass writes dU and the general dx kernel reads it back (kept for comparison).
template <typename T> hipError_t ln_swiglu_bwd_fused_dispatch(const LnParams& p, hipStream_t stream) {
  if constexpr (sizeof(T) != 2) {
    return hipErrorNotSupported;
  } else {
    if (!swiglu_bwd_fused_ok<T>(p)) return hipErrorNotSupported;
#ifdef MF_LN_DU_FORM
    constexpr bool PARTS = false;
#else
    constexpr bool PARTS = true;
#endif
    hipError_t e;
    switch (p.KP) {
      case 32: e = launch_swiglu_bwd_fused_k<T, 32, PARTS>(p, stream); break;
      case 64: e = launch_swiglu_bwd_fused_k<T, 64, PARTS>(p, stream); break;
      case 128: e = launch_swiglu_bwd_fused_k<T, 128, PARTS>(p, stream); break;
      default: return hipErrorNotSupported;
    }
    if (e != hipSuccess) return e;
    e = launch_dw_reduce<T>(p, stream);
    if (e != hipSuccess) return e;
    if constexpr (PARTS) {
      switch (p.KP) {
        case 32: return launch_dx_parts_k<T, 32>(p, stream);
        case 64: return launch_dx_parts_k<T, 64>(p, stream);
        default: return launch_dx_parts_k<T, 128>(p, stream);
      }
    } else {
      return ln_dx_dispatch<T>(p, p.du, stream);
    }
  }
}

}  // namespace mf
