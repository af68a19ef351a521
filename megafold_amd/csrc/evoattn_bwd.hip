// Backward pass of the pair-biased, key-masked attention for gfx950.
//
// With P = exp(z - LSE) recomputed from the saved logsumexp (the S x S scores are never stored):
//   delta[i] = sum_d dO[i, d] O[i, d]          dP = dO V^T          dS = P * (dP - delta)
//   dV = P^T dO      dK = scale * dS^T Q      dQ = scale * dS K      dBias[h, i, j] = sum_n dS
// Same mathematics as the reference kernels _attn_bwd_preprocess, _attn_bwd_dk_dv and _attn_bwd_dq
// (megafold/model/FusedEvoAttention/evoattention.py:272-301, 514-686, 325-490), organised differently:
//
//  * evo_bwd_dqkv_kernel computes dQ, dK and dV in ONE pass over the score tiles (5 matrix products
//    per tile instead of the reference's 7) and also produces delta.  A work-group owns one (b, n, h);
//    each wavefront owns TPW key tiles whose dK/dV accumulate in registers while the group walks over
//    the query tiles; the per-wavefront partial dQ of a query tile is summed through LDS in a fixed
//    order, so the result is bitwise reproducible.
//  * evo_bwd_dbias_kernel replaces the reference's N-way contended fp32 atomic adds
//    (evoattention.py:465): a wavefront owns a 32 x (TR*32) patch of the [S, S] bias gradient of one
//    head, keeps it in registers and walks over a chunk of the N rows; the few per-chunk partial
//    patches are added by a small reduction kernel.  No atomics, fixed summation order.
#include <cstdlib>
#include "common.h"
#include "evoattn.h"

namespace mf {

template <typename T, int DP> struct BwdLayout {
  static constexpr int UNIT = 16 / (int)sizeof(T);
  static constexpr int KRAW = DP + 16;
  static constexpr int KSTR = ((KRAW / UNIT) % 2 == 0) ? KRAW + UNIT : KRAW;   // K rows + mask carrier
  static constexpr int QSTR = ((DP / UNIT) % 2 == 0) ? DP + UNIT : DP;         // Q / dO / V rows
  static constexpr int TSTR = ((32 / UNIT) % 2 == 0) ? 32 + UNIT : 32;         // dS tile rows
  static constexpr int SSTR = DP + 4;                                          // fp32 dQ slab rows
  static constexpr int TR_BYTES = 32 * TSTR * (int)sizeof(T);
  static constexpr int SLAB_BYTES = 32 * SSTR * 4;
  static constexpr int WAVE_BYTES = TR_BYTES > SLAB_BYTES ? TR_BYTES : SLAB_BYTES;  // per-wave scratch (aliased)
  static constexpr int STAGE_ELEMS = 2 * 32 * QSTR;                            // Q tile + dO tile
};

// =================================================================================================
// dQ, dK, dV (+ delta)
// =================================================================================================
template <typename T, int DP, int TPW, int MAXT>
__global__ void __launch_bounds__(MAXT) evo_bwd_dqkv_kernel(const EvoParams p) {
  using L = BwdLayout<T, DP>;
  using frag = frag_t<T>;
  constexpr int KS = DP / 16, DT = DP / 32, CPR = DP / 8;
  constexpr int QITEMS = 32 * CPR;               // 8-element chunks in one 32-row tile
  constexpr int PF = (QITEMS + 255) / 256;       // staged chunks per thread (block has >= 256 threads)

  const int nthr = blockDim.x, NW = nthr >> 6;
  const int KC = NW * TPW * 32;                  // keys per chunk

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Kc = reinterpret_cast<T*>(smem_raw);                                   // [KC][KSTR]
  T* Stage = Kc + KC * L::KSTR;                                             // [2][Q tile | dO tile]
  float* Lv = reinterpret_cast<float*>(Stage + 2 * L::STAGE_ELEMS);         // [2][32] LSE * log2(e)
  float* Dv = Lv + 64;                                                      // [2][32] delta
  unsigned char* Wv = reinterpret_cast<unsigned char*>(Dv + 64);            // [NW][WAVE_BYTES]

  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  const int bn = (kq / p.H) * 8 + xcd;
  if (bn >= p.B * p.N) return;
  const int h = kq % p.H;
  const int b = bn / p.N, n = bn % p.N;

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int S = p.S, D = p.D;
  const int NT = (S + 31) >> 5;

  const T* Qg = reinterpret_cast<const T*>(p.q.ptr) + b * p.q.sb + n * p.q.sn + h * p.q.sh;
  const T* Kg = reinterpret_cast<const T*>(p.k.ptr) + b * p.k.sb + n * p.k.sn + h * p.k.sh;
  const T* Vg = reinterpret_cast<const T*>(p.v.ptr) + b * p.v.sb + n * p.v.sn + h * p.v.sh;
  const T* Og = reinterpret_cast<const T*>(p.o.ptr) + b * p.o.sb + n * p.o.sn + h * p.o.sh;
  const T* dOg = reinterpret_cast<const T*>(p.dO.ptr) + b * p.dO.sb + n * p.dO.sn + h * p.dO.sh;
  T* dQg = reinterpret_cast<T*>(p.dq.ptr) + b * p.dq.sb + n * p.dq.sn + h * p.dq.sh;
  T* dKg = reinterpret_cast<T*>(p.dk.ptr) + b * p.dk.sb + n * p.dk.sn + h * p.dk.sh;
  T* dVg = reinterpret_cast<T*>(p.dv.ptr) + b * p.dv.sb + n * p.dv.sn + h * p.dv.sh;
  const float* biasg = p.bias + b * p.bias_sb + h * p.bias_sh;
  const int64_t mask_base = b * p.mask_sb + n * p.mask_sn;
  const int64_t row_base = (((int64_t)b * p.N + n) * p.H + h) * S;   // into lse / delta

  T* Trw = reinterpret_cast<T*>(Wv + w * L::WAVE_BYTES);
  float* Slw = reinterpret_cast<float*>(Wv + w * L::WAVE_BYTES);

  frag qaugA = frag_zero<T>();   // Q side of the mask-carrier step (A operand here)
  if (g == 0) { qaugA[0] = (T)1.0f; qaugA[1] = (T)1.0f; }

  const float cexp = p.scale * MF_LOG2E;   // the accumulator holds z / scale (unscaled q.k + bias/scale + mask/scale)
  const float inv_scale = 1.0f / p.scale;

  // ---- staging of one query tile: Q, dO, LSE, delta --------------------------------------------
  frag sq[PF], sdo[PF];
  float sdelta[PF], slse[PF];
  auto fetch_q = [&](int it) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int item = tid + i * nthr;
      sdelta[i] = 0.0f; slse[i] = __builtin_inff();
      sq[i] = frag_zero<T>(); sdo[i] = frag_zero<T>();
      if (item < QITEMS) {
        const int row = item / CPR, dc = item % CPR;
        const int qi = it * 32 + row;
        const bool ok = qi < S && 8 * dc < D;
        frag of = frag_zero<T>();
        if (ok) {
          sq[i] = ld8<T>(Qg + (int64_t)qi * p.q.ss + 8 * dc);
          sdo[i] = ld8<T>(dOg + (int64_t)qi * p.dO.ss + 8 * dc);
          of = ld8<T>(Og + (int64_t)qi * p.o.ss + 8 * dc);
        }
        float part = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) part += (float)sdo[i][e] * (float)of[e];
#pragma unroll
        for (int m = 1; m < CPR; m <<= 1) part += __shfl_xor(part, m);
        sdelta[i] = part;
        if (dc == 0 && qi < S) {
          const float lse = p.lse[row_base + qi];
          // fully masked row: LSE = -inf; +inf makes every recomputed probability exactly 0
          slse[i] = (lse == -__builtin_inff()) ? __builtin_inff() : lse * MF_LOG2E;
        }
      }
    }
  };
  auto stash_q = [&](int it, int buf, bool write_delta) {
    T* qd = Stage + buf * L::STAGE_ELEMS;
    T* dod = qd + 32 * L::QSTR;
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int item = tid + i * nthr;
      if (item < QITEMS) {
        const int row = item / CPR, dc = item % CPR;
        st8<T>(qd + row * L::QSTR + 8 * dc, sq[i]);
        st8<T>(dod + row * L::QSTR + 8 * dc, sdo[i]);
        if (dc == 0) {
          Lv[buf * 32 + row] = slse[i];
          Dv[buf * 32 + row] = sdelta[i];
          const int qi = it * 32 + row;
          if (write_delta && qi < S) p.delta[row_base + qi] = sdelta[i];
        }
      }
    }
  };

  const int nchunks = (NT + NW * TPW - 1) / (NW * TPW);
  for (int kc = 0; kc < nchunks; ++kc) {
    const int tile0 = kc * NW * TPW;
    // ---- stage this chunk's K rows (plain order) with the mask carrier columns ------------------
    for (int c = tid; c < KC * CPR; c += nthr) {
      const int kk = c / CPR, dc = c % CPR;
      const int j = tile0 * 32 + kk;
      const bool ok = j < S && 8 * dc < D;
      st8<T>(Kc + kk * L::KSTR + 8 * dc, ok ? ld8<T>(Kg + (int64_t)j * p.k.ss + 8 * dc) : frag_zero<T>());
    }
    for (int kk = tid; kk < KC; kk += nthr) {
      const int j = tile0 * 32 + kk;
      const float mv = j < S ? load_any(p.mask, p.mask_dtype, mask_base + (int64_t)j * p.mask_sj) * inv_scale
                             : -__builtin_inff();
      frag a = frag_zero<T>();
      T hi, lo;
      split_hi_lo<T>(mv, hi, lo);
      a[0] = hi; a[1] = lo;
      st8<T>(Kc + kk * L::KSTR + DP, a);
      st8<T>(Kc + kk * L::KSTR + DP + 8, frag_zero<T>());
    }
    // V fragments of this wavefront's tiles (B operand of dP = dO V^T): lane (x, g) <-> key j0 + x
    frag vf[TPW][KS];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int j = (tile0 + w * TPW + t) * 32 + x;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = (DP / 2) * g + 8 * s;
        vf[t][s] = (j < S && d0 < D) ? ld8<T>(Vg + (int64_t)j * p.v.ss + d0) : frag_zero<T>();
      }
    }
    f32x16 dk[TPW][DT], dv[TPW][DT];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) { dk[t][dt] = acc_zero(); dv[t][dt] = acc_zero(); }

    // bias/scale tile of the next (query tile, key tile) step, loaded one step ahead.  The copy in
    // the workspace is zero padded to whole tiles, so no bounds checks: register i of half g <->
    // query 32*it + 16*g + i, lane x <-> key j0 + x.
    const float* bias_t[TPW];
    bool tile_ok[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int j0 = (tile0 + w * TPW + t) * 32;
      tile_ok[t] = j0 < S;
      bias_t[t] = biasg + (int64_t)(16 * g) * p.bias_ld + (tile_ok[t] ? j0 : 0) + x;
    }
    f32x16 bzn;
    auto load_bias = [&](int it, const float* base) {
      const float* bp = base + (int64_t)it * 32 * p.bias_ld;
#pragma unroll
      for (int i = 0; i < 16; ++i) bzn[i] = bp[(int64_t)i * p.bias_ld];
    };
    if (tile_ok[0]) load_bias(0, bias_t[0]);

    fetch_q(0);
    stash_q(0, 0, kc == 0);
    __syncthreads();

    for (int it = 0; it < NT; ++it) {
      const int buf = it & 1;
      const bool more = it + 1 < NT;
      if (more) fetch_q(it + 1);

      const T* qs = Stage + buf * L::STAGE_ELEMS;
      const T* dos = qs + 32 * L::QSTR;
      const int i0 = it * 32;

      // per-register row constants: register r of half g <-> query i0 + 16*g + r
      float l2v[16], dlv[16];
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(Lv + buf * 32 + 16 * g + 4 * c4);
        const f32x4 d = *reinterpret_cast<const f32x4*>(Dv + buf * 32 + 16 * g + 4 * c4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { l2v[4 * c4 + e] = a[e]; dlv[4 * c4 + e] = d[e]; }
      }
      // A operands of S = Q K^T and dP = dO V^T: operand row x holds tile row unperm32(x)
      frag qA[KS], doA[KS];
      const int arow = unperm32(x);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        qA[s] = ld8<T>(qs + arow * L::QSTR + (DP / 2) * g + 8 * s);
        doA[s] = ld8<T>(dos + arow * L::QSTR + (DP / 2) * g + 8 * s);
      }
      f32x16 dq[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) dq[dt] = acc_zero();

#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        const int tl = w * TPW + t;            // tile inside the chunk
        const int j0 = (tile0 + tl) * 32;
        if (j0 < S) {                          // wave-uniform
          const T* krow = Kc + (tl * 32 + x) * L::KSTR;
          f32x16 z = mma(qaugA, ld8<T>(krow + DP + 8 * g), bzn);
          if (t + 1 < TPW && tile_ok[t + 1 < TPW ? t + 1 : 0]) load_bias(it, bias_t[t + 1 < TPW ? t + 1 : 0]);
          else if (more) load_bias(it + 1, bias_t[0]);
#pragma unroll
          for (int s = 0; s < KS; ++s) z = mma(qA[s], ld8<T>(krow + (DP / 2) * g + 8 * s), z);
          f32x16 dp = acc_zero();
#pragma unroll
          for (int s = 0; s < KS; ++s) dp = mma(doA[s], vf[t][s], dp);
          f32x16 ds;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float pr = fast_exp2(__builtin_fmaf(z[r], cexp, -l2v[r]));
            z[r] = pr;
            ds[r] = pr * (dp[r] - dlv[r]);
          }
          frag dsf[2];
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const frag pf = acc_half<T>(z, u);
            dsf[u] = acc_half<T>(ds, u);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
              const frag doT = TrRead<T>::read(dos, L::QSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(dt, l), dsel<DP>(dt, x));
              dv[t][dt] = mma(doT, pf, dv[t][dt]);
              const frag qT = TrRead<T>::read(qs, L::QSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(dt, l), dsel<DP>(dt, x));
              dk[t][dt] = mma(qT, dsf[u], dk[t][dt]);
            }
          }
          // dS tile, rows = keys, through this wavefront's LDS scratch, read back transposed
          st8<T>(Trw + x * L::TSTR + 16 * g, dsf[0]);
          st8<T>(Trw + x * L::TSTR + 16 * g + 8, dsf[1]);
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const frag dsT = TrRead<T>::read(Trw, L::TSTR, 8 * u + 8 * g, g, l, plain_chunk(l), x);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
              const frag kT = TrRead<T>::read(Kc, L::KSTR, tl * 32 + 8 * u + 8 * g, g, l, dsel_chunk<DP>(dt, l),
                                              dsel<DP>(dt, x));
              dq[dt] = mma(kT, dsT, dq[dt]);
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
        }
      }

      // this wavefront's partial dQ^T -> its slab: lane (x = query, g) owns DP/2 contiguous columns
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          f32x4 v;
          v[0] = dq[dt][4 * c4]; v[1] = dq[dt][4 * c4 + 1]; v[2] = dq[dt][4 * c4 + 2]; v[3] = dq[dt][4 * c4 + 3];
          *reinterpret_cast<f32x4*>(Slw + x * L::SSTR + (DP / 2) * g + 16 * dt + 4 * c4) = v;
        }
      if (more) stash_q(it + 1, buf ^ 1, kc == 0);
      __syncthreads();

      // fixed-order sum of the NW slabs, scale, store (or add to what earlier key chunks stored)
      for (int item = tid; item < 8 * DP; item += nthr) {
        const int row = item / (DP / 4), c4 = item % (DP / 4);
        f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int ww = 0; ww < NW; ++ww) {
          const float* sl = reinterpret_cast<const float*>(Wv + ww * L::WAVE_BYTES);
          sum += *reinterpret_cast<const f32x4*>(sl + row * L::SSTR + 4 * c4);
        }
        const int qi = i0 + row;
        if (qi < S && 4 * c4 < D) {
          T* dst = dQg + (int64_t)qi * p.dq.ss + 4 * c4;
          float o4[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) o4[e] = sum[e] * p.scale;
          if (kc > 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) o4[e] += (float)dst[e];
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) dst[e] = (T)o4[e];
        }
      }
      __syncthreads();
    }

    // ---- dK, dV of this wavefront's tiles: lane (x = key, g) owns DP/2 contiguous columns --------
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int j = (tile0 + w * TPW + t) * 32 + x;
      if (j < S) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int d0 = (DP / 2) * g + 16 * dt + 8 * u;
            if (d0 < D) {
              f32x16 dks = dk[t][dt];
#pragma unroll
              for (int i = 0; i < 16; ++i) dks[i] *= p.scale;
              st8<T>(dKg + (int64_t)j * p.dk.ss + d0, acc_half<T>(dks, u));
              st8<T>(dVg + (int64_t)j * p.dv.ss + d0, acc_half<T>(dv[t][dt], u));
            }
          }
      }
    }
  }
}

template <typename T, int DP, int TPW> static size_t dqkv_smem(int NW) {
  using L = BwdLayout<T, DP>;
  return (size_t)NW * TPW * 32 * L::KSTR * sizeof(T) + (size_t)2 * L::STAGE_ELEMS * sizeof(T) + 128 * 4 +
         (size_t)NW * L::WAVE_BYTES;
}

template <typename T, int DP, int TPW, int MAXT>
static hipError_t launch_dqkv_t(const EvoParams& p, int NW, hipStream_t stream) {
  const size_t smem = dqkv_smem<T, DP, TPW>(NW);
  if (smem > 160 * 1024) return hipErrorInvalidValue;
  const long long blocks = (long long)round_up(p.B * p.N, 8) * p.H;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kern = evo_bwd_dqkv_kernel<T, DP, TPW, MAXT>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(64 * NW), smem, stream, p);
  return hipGetLastError();
}

// Wavefronts per work-group (NW) and key tiles per wavefront (TPW).  Preference order: fewest key
// chunks (one chunk means dQ is written once, never read back), then fewest idle tile slots, then
// the larger TPW (more reuse of the staged query tile).  A configuration must fit the 160 KiB LDS.
// MF_DQKV_NW / MF_DQKV_TPW override the choice (tuning aid).
template <typename T, int DP> static hipError_t launch_dqkv_d(const EvoParams& p, hipStream_t stream) {
  const int NT = (p.S + 31) / 32;
  constexpr int max_tpw = (sizeof(T) == 4 || DP > 32) ? 1 : 3;
  int best_nw = 4, best_tpw = 1;
  long long best_cost = -1;
  for (int tpw = 1; tpw <= max_tpw; ++tpw) {
    const int max_nw = tpw == 1 ? 16 : 8;
    for (int nw = 4; nw <= max_nw; ++nw) {
      const size_t smem = tpw == 1 ? dqkv_smem<T, DP, 1>(nw) : tpw == 2 ? dqkv_smem<T, DP, 2>(nw) : dqkv_smem<T, DP, 3>(nw);
      if (tpw > max_tpw) continue;
      if (smem > 160 * 1024) continue;
      const int slots = nw * tpw;
      const int chunks = (NT + slots - 1) / slots;
      const long long cost = ((long long)chunks << 40) + ((long long)(chunks * slots - NT) << 20) + (16 - tpw) * 32 + nw;
      if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_nw = nw; best_tpw = tpw; }
    }
  }
  if (best_cost < 0) return hipErrorInvalidValue;
  if (const char* e = getenv("MF_DQKV_TPW")) { const int v = atoi(e); if (v >= 1 && v <= max_tpw) best_tpw = v; }
  if (const char* e = getenv("MF_DQKV_NW")) { const int v = atoi(e); if (v >= 4 && v <= (best_tpw == 1 ? 16 : 8)) best_nw = v; }
  if (best_tpw == 1) {
    return best_nw <= 8 ? launch_dqkv_t<T, DP, 1, 512>(p, best_nw, stream) : launch_dqkv_t<T, DP, 1, 1024>(p, best_nw, stream);
  }
  if constexpr (max_tpw >= 3) {
    if (best_tpw == 2) return launch_dqkv_t<T, DP, 2, 512>(p, best_nw, stream);
    return launch_dqkv_t<T, DP, 3, 512>(p, best_nw, stream);
  }
  return hipErrorInvalidValue;
}

template <typename T> static hipError_t launch_dqkv_s(const EvoParams& p, hipStream_t stream) {
  if (p.D <= 32) return launch_dqkv_d<T, 32>(p, stream);
  if (p.D <= 64) return launch_dqkv_d<T, 64>(p, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_evo_bwd_dqkv(const EvoParams& p, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return launch_dqkv_s<bf16_t>(p, stream);
    case MF_F16: return launch_dqkv_s<f16_t>(p, stream);
    case MF_F32: return launch_dqkv_s<float>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

// =================================================================================================
// dBias
// =================================================================================================
template <typename T, int DP, int TR>
__global__ void __launch_bounds__(256, 2) evo_bwd_dbias_kernel(const EvoParams p, const int IB, const int JB) {
  using L = BwdLayout<T, DP>;
  using frag = frag_t<T>;
  constexpr int KS = DP / 16, CPR = DP / 8;
  constexpr int ROWS = TR * 32;
  constexpr int ITEMS = ROWS * CPR;
  constexpr int PF = (ITEMS + 255) / 256;

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Ks = reinterpret_cast<T*>(smem_raw);       // [2][ROWS][KSTR]
  T* Vs = Ks + 2 * ROWS * L::KSTR;              // [2][ROWS][QSTR]

  const int R = IB * JB;
  const int G = p.B * p.H * p.n_chunks;
  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  const int grp = (kq / R) * 8 + xcd;
  if (grp >= G) return;
  const int reg = kq % R;
  const int ib = reg % IB, jb = reg / IB;
  const int chunk = grp % p.n_chunks;
  const int bh = grp / p.n_chunks;
  const int h = bh % p.H, b = bh / p.H;

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int S = p.S, D = p.D;
  const int n_begin = chunk * p.rows_per_chunk;
  const int n_end = min(p.N, n_begin + p.rows_per_chunk);

  const int qi = ib * 128 + w * 32 + x;
  const int qi_c = qi < S ? qi : S - 1;
  const int jt0 = jb * TR;                    // first key tile of the patch

  const T* Qg = reinterpret_cast<const T*>(p.q.ptr) + b * p.q.sb + h * p.q.sh + (int64_t)qi_c * p.q.ss;
  const T* dOg = reinterpret_cast<const T*>(p.dO.ptr) + b * p.dO.sb + h * p.dO.sh + (int64_t)qi_c * p.dO.ss;
  const T* Kg = reinterpret_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh;
  const T* Vg = reinterpret_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh;
  const float* biasg = p.bias + b * p.bias_sb + h * p.bias_sh;

  const float cexp = p.scale * MF_LOG2E;   // the accumulator holds z / scale
  const float inv_scale = 1.0f / p.scale;
  // the bias patch is the same for every row n: keep it in registers as the accumulator seed
  f32x16 bz[TR], acc[TR];
#pragma unroll
  for (int t = 0; t < TR; ++t) {
    acc[t] = acc_zero();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = (jt0 + t) * 32 + 16 * g + r;
      bz[t][r] = j < p.bias_ld ? biasg[(int64_t)qi_c * p.bias_ld + j] : 0.0f;
    }
  }
  frag qaug = frag_zero<T>();
  if (g == 0) { qaug[0] = (T)1.0f; qaug[1] = (T)1.0f; }

  frag kreg[PF], vreg[PF];
  float mreg = 0.0f;
  frag qf[KS], dof[KS];
  float l2 = 0.0f, dl = 0.0f;
  auto fetch = [&](int n) {
    const T* kn = Kg + (int64_t)n * p.k.sn;
    const T* vn = Vg + (int64_t)n * p.v.sn;
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int c = tid + 256 * i;
      kreg[i] = frag_zero<T>(); vreg[i] = frag_zero<T>();
      if (c < ITEMS) {
        const int kk = c / CPR, dc = c % CPR;
        const int j = jt0 * 32 + kk;
        if (j < S && 8 * dc < D) {
          kreg[i] = ld8<T>(kn + (int64_t)j * p.k.ss + 8 * dc);
          vreg[i] = ld8<T>(vn + (int64_t)j * p.v.ss + 8 * dc);
        }
      }
    }
    if (tid < ROWS) {
      const int j = jt0 * 32 + tid;
      mreg = j < S ? load_any(p.mask, p.mask_dtype, b * p.mask_sb + n * p.mask_sn + (int64_t)j * p.mask_sj) * inv_scale
                   : -__builtin_inff();
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int d0 = (DP / 2) * g + 8 * s;
      const bool ok = qi < S && d0 < D;
      qf[s] = ok ? ld8<T>(Qg + (int64_t)n * p.q.sn + d0) : frag_zero<T>();
      dof[s] = ok ? ld8<T>(dOg + (int64_t)n * p.dO.sn + d0) : frag_zero<T>();
    }
    const int64_t ridx = (((int64_t)b * p.N + n) * p.H + h) * S + qi_c;
    const float lse = p.lse[ridx];
    l2 = (qi < S && lse != -__builtin_inff()) ? lse * MF_LOG2E : __builtin_inff();
    dl = p.delta[ridx];
  };
  auto stash = [&](int buf) {
    T* kd = Ks + buf * ROWS * L::KSTR;
    T* vd = Vs + buf * ROWS * L::QSTR;
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int c = tid + 256 * i;
      if (c < ITEMS) {
        const int kk = c / CPR, dc = c % CPR;
        const int row = (kk & ~31) + perm32(kk & 31);
        st8<T>(kd + row * L::KSTR + 8 * dc, kreg[i]);
        st8<T>(vd + row * L::QSTR + 8 * dc, vreg[i]);
      }
    }
    if (tid < ROWS) {
      const int row = (tid & ~31) + perm32(tid & 31);
      frag a = frag_zero<T>();
      T hi, lo;
      split_hi_lo<T>(mreg, hi, lo);
      a[0] = hi; a[1] = lo;
      st8<T>(kd + row * L::KSTR + DP, a);
      st8<T>(kd + row * L::KSTR + DP + 8, frag_zero<T>());
    }
  };

  if (n_begin < n_end) {
    fetch(n_begin);
    for (int n = n_begin; n < n_end; ++n) {
      const int buf = (n - n_begin) & 1;
      // operands of this row move from the staging registers to their working copies
      frag qc[KS], doc[KS];
#pragma unroll
      for (int s = 0; s < KS; ++s) { qc[s] = qf[s]; doc[s] = dof[s]; }
      const float l2c = l2, dlc = dl;
      stash(buf);
      __syncthreads();
      if (n + 1 < n_end) fetch(n + 1);

      const T* kt = Ks + buf * ROWS * L::KSTR;
      const T* vt = Vs + buf * ROWS * L::QSTR;
#pragma unroll
      for (int t = 0; t < TR; ++t) {
        if ((jt0 + t) * 32 < S) {
          const T* krow = kt + (32 * t + x) * L::KSTR;
          const T* vrow = vt + (32 * t + x) * L::QSTR;
          f32x16 z = mma(ld8<T>(krow + DP + 8 * g), qaug, bz[t]);
          f32x16 dp = acc_zero();
#pragma unroll
          for (int s = 0; s < KS; ++s) {
            z = mma(ld8<T>(krow + (DP / 2) * g + 8 * s), qc[s], z);
            dp = mma(ld8<T>(vrow + (DP / 2) * g + 8 * s), doc[s], dp);
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float pr = fast_exp2(__builtin_fmaf(z[r], cexp, -l2c));
            acc[t][r] = __builtin_fmaf(pr, dp[r] - dlc, acc[t][r]);
          }
        }
      }
    }
  }

  // ---- store the patch: lane (x = query, g) owns 16 contiguous keys per tile ---------------------
  float* dst = (p.n_chunks > 1 ? p.dbias_part + (int64_t)chunk * p.B * p.H * S * S : p.dbias) +
               ((int64_t)b * p.H + h) * S * S;
  if (qi < S) {
#pragma unroll
    for (int t = 0; t < TR; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = (jt0 + t) * 32 + 16 * g + r;
        if (j < S) dst[(int64_t)qi * S + j] = acc[t][r];
      }
  }
}

__global__ void __launch_bounds__(256) dbias_reduce_kernel(const float* part, float* out, int64_t n, int chunks) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    float s = 0.0f;
    for (int c = 0; c < chunks; ++c) s += part[(int64_t)c * n + i];
    out[i] = s;
  }
}

// Key tiles per wavefront patch: limited by the registers the patch and its bias seed occupy.
static int dbias_tr(int dtype, int D) { (void)D; return dtype == MF_F32 ? 1 : 2; }

int evo_dbias_chunks(int B, int N, int S, int H, int D, int dtype) {
  const int TR = dbias_tr(dtype, D);
  const int NT = (S + 31) / 32;
  const int IB = (S + 127) / 128, JB = (NT + TR - 1) / TR;
  const long long regions = (long long)B * H * IB * JB;
  long long want = (768 + regions - 1) / regions;   // ~3 work-groups per compute unit
  if (want > 8) want = 8;                           // bounds the partial-sum workspace
  if (want > N) want = N;
  if (want < 1) want = 1;
  const int rows = (int)((N + want - 1) / want);
  return (N + rows - 1) / rows;
}

template <typename T, int DP, int TR> static hipError_t launch_dbias_t(const EvoParams& p, hipStream_t stream) {
  using L = BwdLayout<T, DP>;
  const int NT = (p.S + 31) / 32;
  const int IB = (p.S + 127) / 128, JB = (NT + TR - 1) / TR;
  const size_t smem = (size_t)2 * TR * 32 * (L::KSTR + L::QSTR) * sizeof(T);
  const long long G = (long long)p.B * p.H * p.n_chunks;
  const long long blocks = (G + 7) / 8 * 8 * IB * JB;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kern = evo_bwd_dbias_kernel<T, DP, TR>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), smem, stream, p, IB, JB);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (p.n_chunks > 1) {
    const int64_t n = (int64_t)p.B * p.H * p.S * p.S;
    int64_t rb = (n + 255) / 256;
    if (rb > 2048) rb = 2048;
    hipLaunchKernelGGL(dbias_reduce_kernel, dim3((unsigned)rb), dim3(256), 0, stream, p.dbias_part, p.dbias, n,
                       p.n_chunks);
    e = hipGetLastError();
  }
  return e;
}

template <typename T> static hipError_t launch_dbias_s(const EvoParams& p, hipStream_t stream) {
  constexpr bool wide = sizeof(T) == 4;
  if (p.D <= 32) return launch_dbias_t<T, 32, wide ? 1 : 2>(p, stream);
  if (p.D <= 64) return launch_dbias_t<T, 64, wide ? 1 : 2>(p, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_evo_bwd_dbias(const EvoParams& p, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return launch_dbias_s<bf16_t>(p, stream);
    case MF_F16: return launch_dbias_s<f16_t>(p, stream);
    case MF_F32: return launch_dbias_s<float>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mf
