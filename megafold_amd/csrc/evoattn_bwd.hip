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
#include "evoattn_bwd_layout.h"

namespace mf {

// =================================================================================================
// dQ, dK, dV (+ delta)
// =================================================================================================
// Per (query tile, key tile) step, with everything additive riding through carrier MFMA steps:
//   z' = <q, k> + bias/s + mask/s - LSE/s      (5 = 1 carrier + DP/16 MFMAs for D = 32: 3)
//   P  = exp2(c z'),  c = s log2 e
//   d' = <dO, v> - delta                        (1 carrier + DP/16 MFMAs)
//   dS = P d'
//   dV += P^T dO,  dK += dS^T Q  (operands: P, dS straight from the accumulator registers; dO^T, Q^T
//        through transposing LDS reads),  dQ += dS K (dS through a per-wavefront LDS tile, K^T through
//        transposing reads)
// so the vector ALU does one multiply, one exp2, one multiply and two packed converts per logit.
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
  T* Kc = reinterpret_cast<T*>(smem_raw);                                   // [KC][QSTR]
  T* Stage = Kc + KC * L::QSTR;                                             // [2][Q tile | dO tile]
  unsigned* Lpk = reinterpret_cast<unsigned*>(Stage + 2 * L::STAGE_ELEMS);  // [2][32] packed -LSE/scale
  unsigned* Dpk = Lpk + 64;                                                 // [2][32] packed -delta
  unsigned char* Wv = reinterpret_cast<unsigned char*>(Dpk + 64);           // [NW][WAVE_BYTES]
  constexpr int WAVE_BYTES = L::wave_bytes(TPW);

  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  const int bn = (kq / p.H) * 8 + xcd;
  if (bn >= p.B * p.N) return;
  const int h = kq % p.H;
  const int b = bn / p.N, n = bn % p.N;

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int S = p.S, D = p.D;
  const int NT = (S + 31) >> 5;
  const float cexp = p.scale * MF_LOG2E;   // the accumulator holds z / scale
  const float inv_scale = 1.0f / p.scale;

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

  T* Trw = reinterpret_cast<T*>(Wv + w * WAVE_BYTES);
  float* Slw = reinterpret_cast<float*>(Wv + w * WAVE_BYTES);

  const unsigned ones_g = g == 0 ? ones_word<T>() : 0u;     // carrier slots live in the lower lane half only
  const frag vaugB = make_aug<T>(ones_g, 0u);                // B side of the delta carrier

  // ---- staging of one query tile: Q, dO, packed -LSE/scale and -delta ----------------------------
  // Rows past S are clamped for the loads; their LSE is +inf, which makes every probability exactly 0.
  frag sq[PF], sdo[PF];
  float sdelta[PF], sls[PF];
  auto fetch_q = [&](int it) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int item = tid + i * nthr;
      if (item < QITEMS) {
        const int row = item / CPR, dc = item % CPR;
        const int qi = it * 32 + row;
        const int qc = qi < S ? qi : S - 1;
        const bool dok = 8 * dc < D;
        sq[i] = dok ? ld8<T>(Qg + (int64_t)qc * p.q.ss + 8 * dc) : frag_zero<T>();
        sdo[i] = dok ? ld8<T>(dOg + (int64_t)qc * p.dO.ss + 8 * dc) : frag_zero<T>();
        const frag of = dok ? ld8<T>(Og + (int64_t)qc * p.o.ss + 8 * dc) : frag_zero<T>();
        float part = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) part += (float)sdo[i][e] * (float)of[e];
        part = group_sum<CPR>(part);
        sdelta[i] = part;
        sls[i] = __builtin_inff();
        if (dc == 0 && qi < S) {
          const float lse = p.lse[row_base + qi];
          sls[i] = (lse == -__builtin_inff()) ? __builtin_inff() : lse * inv_scale;
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
          Lpk[buf * 32 + row] = pack_split<T>(-sls[i]);
          Dpk[buf * 32 + row] = pack_split<T>(-sdelta[i]);
          const int qi = it * 32 + row;
          if (write_delta && qi < S) p.delta[row_base + qi] = sdelta[i];
        }
      }
    }
  };

  const int nchunks = (NT + NW * TPW - 1) / (NW * TPW);
  for (int kc = 0; kc < nchunks; ++kc) {
    const int tile0 = kc * NW * TPW;
    // ---- stage this chunk's K rows (keys past S clamped: their mask is -inf) ----------------------
    for (int c = tid; c < KC * CPR; c += nthr) {
      const int kk = c / CPR, dc = c % CPR;
      int j = tile0 * 32 + kk;
      j = j < S ? j : S - 1;
      st8<T>(Kc + kk * L::QSTR + 8 * dc, 8 * dc < D ? ld8<T>(Kg + (int64_t)j * p.k.ss + 8 * dc) : frag_zero<T>());
    }
    // this wavefront's key tiles: V fragments (B operand of dO V^T), packed mask/scale, bias pointers
    frag vf[TPW][KS];
    unsigned mk[TPW];
    const float* bias_t[TPW];
    bool tile_ok[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int j0 = (tile0 + w * TPW + t) * 32;
      const int j = j0 + x;
      const int jc = j < S ? j : S - 1;
      tile_ok[t] = j0 < S;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = (DP / 2) * g + 8 * s;
        vf[t][s] = d0 < D ? ld8<T>(Vg + (int64_t)jc * p.v.ss + d0) : frag_zero<T>();
      }
      const float mv = j < S ? load_any(p.mask, p.mask_dtype, mask_base + (int64_t)j * p.mask_sj) * inv_scale
                             : -__builtin_inff();
      mk[t] = g == 0 ? pack_split<T>(mv) : 0u;
      // column of bias tiles of this key tile (backward layout, see EvoParams::bias): register i of half g
      // <-> query 32*it + 16*g + i
      bias_t[t] = biasg + (int64_t)(tile_ok[t] ? j0 >> 5 : 0) * p.bias_nt * 1024 + 4 * l;
    }
    f32x16 dk[TPW][DT], dv[TPW][DT];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) { dk[t][dt] = acc_zero(); dv[t][dt] = acc_zero(); }

    // bias/scale tile of the next (query tile, key tile) step, loaded one step ahead
    f32x16 bzn;
    auto load_bias = [&](int it, const float* base) {
      const float* bp = base + it * 1024;
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(bp + 256 * c4);
        bzn[4 * c4] = v[0]; bzn[4 * c4 + 1] = v[1]; bzn[4 * c4 + 2] = v[2]; bzn[4 * c4 + 3] = v[3];
      }
    };
    load_bias(0, bias_t[0]);   // idle tile slots read (and ignore) column block 0

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

      // A operands of S = Q K^T and dP = dO V^T: operand row x holds tile row unperm32(x), so that
      // accumulator register i of half g belongs to query i0 + 16*g + i
      const int arow = unperm32(x);
      frag qA[KS], doA[KS];
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        qA[s] = ld8<T>(qs + arow * L::QSTR + (DP / 2) * g + 8 * s);
        doA[s] = ld8<T>(dos + arow * L::QSTR + (DP / 2) * g + 8 * s);
      }
      const frag qaugA = make_aug<T>(ones_g, g == 0 ? Lpk[buf * 32 + arow] : 0u);
      const frag doaugA = make_aug<T>(g == 0 ? Dpk[buf * 32 + arow] : 0u, 0u);

      f32x16 dq[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) dq[dt] = acc_zero();

#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        const int tl = w * TPW + t;            // tile inside the chunk
        {   // key tiles past S run on clamped keys with mask -inf: they contribute exact zeros
          const T* krow = Kc + (tl * 32 + x) * L::QSTR;
          f32x16 z = mma(qaugA, make_aug<T>(mk[t], ones_g), bzn);
          if (t + 1 < TPW && tile_ok[t + 1 < TPW ? t + 1 : 0]) load_bias(it, bias_t[t + 1 < TPW ? t + 1 : 0]);
          else if (more) load_bias(it + 1, bias_t[0]);
#pragma unroll
          for (int s = 0; s < KS; ++s) z = mma(qA[s], ld8<T>(krow + (DP / 2) * g + 8 * s), z);
          f32x16 dp = mma(doaugA, vaugB, acc_zero());
#pragma unroll
          for (int s = 0; s < KS; ++s) dp = mma(doA[s], vf[t][s], dp);
          f32x16 ds;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float pr = fast_exp2(z[i] * cexp);
            z[i] = pr;
            ds[i] = pr * dp[i];
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
          // dS tile, rows = keys, through this wavefront's LDS scratch (one tile per t, so the tiles of
          // a query step do not serialise on it), read back transposed.  LDS operations of one
          // wavefront execute in program order, which is all the ordering this exchange needs.
          T* trt = Trw + t * 32 * L::TSTR;
          st8<T>(trt + x * L::TSTR + 16 * g, dsf[0]);
          st8<T>(trt + x * L::TSTR + 16 * g + 8, dsf[1]);
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const frag dsT = TrRead<T>::read(trt, L::TSTR, 8 * u + 8 * g, g, l, plain_chunk(l), x);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
              const frag kT = TrRead<T>::read(Kc, L::QSTR, tl * 32 + 8 * u + 8 * g, g, l, dsel_chunk<DP>(dt, l),
                                              dsel<DP>(dt, x));
              dq[dt] = mma(kT, dsT, dq[dt]);
            }
          }
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
      barrier_keep_vm<63>();   // LDS hand-over only: global loads / stores stay in flight

      // fixed-order sum of the NW slabs, scale, store (or add to what earlier key chunks stored)
      for (int item = tid; item < 8 * DP; item += nthr) {
        const int row = item / (DP / 4), c4 = item % (DP / 4);
        f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int ww = 0; ww < NW; ++ww) {
          const float* sl = reinterpret_cast<const float*>(Wv + ww * WAVE_BYTES);
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
          typedef T out4_t __attribute__((ext_vector_type(4)));
          out4_t ov = {(T)o4[0], (T)o4[1], (T)o4[2], (T)o4[3]};
          *reinterpret_cast<out4_t*>(dst) = ov;
        }
      }
      barrier_keep_vm<63>();
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

// -------------------------------------------------------------------------------------------------
// Variant for the 16-bit element types and D <= 32 (the configurations training runs on): one key tile
// per wavefront, whose K, K^T and V fragments stay in registers for the whole walk over the query
// tiles, so that the only LDS round trip on a step's critical path is the transposition of dS.  The
// query-tile operands (Q, dO, Q^T, dO^T) are read at the top of the step, before the matrix products
// that hide their latency.  The per-wavefront partial dQ goes to one of two alternating fp32 slabs,
// which leaves ONE work-group barrier per step: the fixed-order sum of the slabs of step `it` runs
// after that barrier while faster wavefronts already work on step it + 1.
template <typename T> struct RkLayout {
  using L = BwdLayout<T, 32>;
  static constexpr int WAVE_BYTES = L::TR_BYTES + 2 * L::SLAB_BYTES;
  // K chunk, two staged (Q | dO) tiles, the packed -LSE/scale and -delta of every query row, and the
  // per-wavefront dS tile + dQ slabs
  static size_t smem(int NW, int NT) {
    return (size_t)NW * 32 * L::QSTR * sizeof(T) + (size_t)2 * L::STAGE_ELEMS * sizeof(T) + (size_t)NT * 64 * 4 +
           (size_t)NW * WAVE_BYTES;
  }
};

template <typename T, int MAXT, int MINW>
__global__ void __launch_bounds__(MAXT, MINW) evo_bwd_dqkv_rk_kernel(const EvoParams p) {
  constexpr int DP = 32, KS = 2, CPR = 4, QITEMS = 128;
  using L = BwdLayout<T, DP>;
  using frag = frag_t<T>;
  static_assert(sizeof(T) == 2, "16-bit element types only");

  const int nthr = blockDim.x, NW = nthr >> 6;
  const int KC = NW * 32;

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Kc = reinterpret_cast<T*>(smem_raw);                                   // [KC][QSTR]
  T* Stage = Kc + KC * L::QSTR;                                             // [2][Q tile | dO tile]
  const int NT = (p.S + 31) >> 5;
  unsigned* Lpk = reinterpret_cast<unsigned*>(Stage + 2 * L::STAGE_ELEMS);  // [NT * 32] packed -LSE/scale
  unsigned* Dpk = Lpk + NT * 32;                                            // [NT * 32] packed -delta
  unsigned char* Wv = reinterpret_cast<unsigned char*>(Dpk + NT * 32);      // [NW][WAVE_BYTES]
  constexpr int WAVE_BYTES = RkLayout<T>::WAVE_BYTES;

  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  const int bn = (kq / p.H) * 8 + xcd;
  if (bn >= p.B * p.N) return;
  const int h = kq % p.H;
  const int b = bn / p.N, n = bn % p.N;

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int S = p.S, D = p.D;
  const float cexp = p.scale * MF_LOG2E;
  const float inv_scale = 1.0f / p.scale;

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
  const int64_t row_base = (((int64_t)b * p.N + n) * p.H + h) * S;

  T* Trw = reinterpret_cast<T*>(Wv + w * WAVE_BYTES);
  float* Slw = reinterpret_cast<float*>(Wv + w * WAVE_BYTES + L::TR_BYTES);   // [2][32][SSTR]

  const unsigned ones_g = g == 0 ? ones_word<T>() : 0u;
  const frag vaugB = make_aug<T>(ones_g, 0u);

  // ---- once per work-group: delta = <dO, O> and the packed carrier words of every query row -----
  // Four threads per row (one 8-element chunk each).  Rows past S and fully masked rows (LSE = -inf)
  // get LSE = +inf: every probability of such a row becomes exactly 0.
  {
    constexpr int PB = 4;                          // rows in flight per thread
    const int items = NT * 32 * CPR;
    const int c = tid % CPR;
    const int cd0 = 8 * c < D ? 8 * c : 0;
    for (int base = 0; base < items; base += PB * nthr) {
      frag a[PB], o[PB];
      float ls[PB];
#pragma unroll
      for (int u = 0; u < PB; ++u) {
        const int row = (base + u * nthr + tid) / CPR;
        const unsigned rc = (unsigned)(row < S ? row : S - 1);
        a[u] = ld8<T>(dOg + __umul24(rc, (unsigned)p.dO.ss) + cd0);
        o[u] = ld8<T>(Og + __umul24(rc, (unsigned)p.o.ss) + cd0);
        ls[u] = p.lse[row_base + rc];
      }
#pragma unroll
      for (int u = 0; u < PB; ++u) {
        const int row = (base + u * nthr + tid) / CPR;
        float part = 0.0f;
        if (8 * c < D) {
#pragma unroll
          for (int e = 0; e < 8; ++e) part += (float)a[u][e] * (float)o[u][e];
        }
        part = group_sum<CPR>(part);
        if (c == 0 && row < NT * 32) {
          const float l2 = (row >= S || ls[u] == -__builtin_inff()) ? __builtin_inff() : ls[u] * inv_scale;
          Lpk[row] = pack_split<T>(-l2);
          Dpk[row] = pack_split<T>(-part);
          if (row < S) p.delta[row_base + row] = part;
        }
      }
    }
  }

  // Staging of one query tile: threads 0..127 move Q, threads 128..255 move dO (one 8-element chunk
  // of one row each).  Loads are issued two steps ahead into two alternating registers (tile t uses
  // register t & 1) and nothing touches a loaded register before its stash: by then the wait for the
  // bias tile of the step, which was requested later, has already covered it.
  frag sa0, sa1;
  const int sgrp = tid >> 7;                    // 0: Q, 1: dO, >= 2: no staging work
  const int srow = (tid & 127) / CPR, sdc = tid % CPR;
  const int sd0 = 8 * sdc < D ? 8 * sdc : 0;
  // Row strides as 24-bit unsigned values (checked by the launcher): row * stride is then one
  // full-rate multiply instead of a 64-bit product.
  const T* const src_a = (sgrp != 1 ? Qg : dOg) + sd0;
  const unsigned str_a = (unsigned)(sgrp != 1 ? p.q.ss : p.dO.ss);
  const unsigned dq_ss = (unsigned)p.dq.ss;
  auto fetch_q = [&](int it, frag& sa) {
    const int qi = (it < NT ? it : NT - 1) * 32 + srow;
    const int qc = qi < S ? qi : S - 1;
    sa = ld8<T>(src_a + __umul24((unsigned)qc, str_a));
  };
  auto stash_q = [&](int buf, const frag& sa) {
    if (sgrp < 2) {
      T* qd = Stage + buf * L::STAGE_ELEMS + sgrp * 32 * L::QSTR;
      st8<T>(qd + srow * L::QSTR + 8 * sdc, 8 * sdc < D ? sa : frag_zero<T>());
    }
  };

  const int nchunks = (NT + NW - 1) / NW;
  for (int kc = 0; kc < nchunks; ++kc) {
    const int tile0 = kc * NW;
    for (int c = tid; c < KC * CPR; c += nthr) {
      const int kk = c / CPR, dc = c % CPR;
      int j = tile0 * 32 + kk;
      j = j < S ? j : S - 1;
      st8<T>(Kc + kk * L::QSTR + 8 * dc, 8 * dc < D ? ld8<T>(Kg + (int64_t)j * p.k.ss + 8 * dc) : frag_zero<T>());
    }
    // this wavefront's key tile.  Tiles past S run on clamped keys with mask -inf: exact zeros.
    const int j0 = (tile0 + w) * 32;
    const int j = j0 + x;
    const int jc = j < S ? j : S - 1;
    frag vf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int d0 = 16 * g + 8 * s;
      vf[s] = d0 < D ? ld8<T>(Vg + (int64_t)jc * p.v.ss + d0) : frag_zero<T>();
    }
    const float mv = j < S ? load_any(p.mask, p.mask_dtype, mask_base + (int64_t)j * p.mask_sj) * inv_scale
                           : -__builtin_inff();
    const frag maugB = make_aug<T>(g == 0 ? pack_split<T>(mv) : 0u, ones_g);
    // bias/scale copy is zero padded to whole tiles: register i of half g <-> query 32*it + 16*g + i
    const float* bias_t = biasg + (int64_t)(j0 < S ? j0 >> 5 : 0) * p.bias_nt * 1024 + 4 * l;
    f32x16 bzn;
    auto load_bias = [&](int it) {
      const float* bp = bias_t + it * 1024;
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(bp + 256 * c4);
        bzn[4 * c4] = v[0]; bzn[4 * c4 + 1] = v[1]; bzn[4 * c4 + 2] = v[2]; bzn[4 * c4 + 3] = v[3];
      }
    };
    load_bias(0);

    fetch_q(0, sa0);
    fetch_q(1, sa1);
    stash_q(0, sa0);
    fetch_q(2, sa0);
    __syncthreads();

    frag kf[KS], kT[2];
#pragma unroll
    for (int s = 0; s < KS; ++s) kf[s] = ld8<T>(Kc + (w * 32 + x) * L::QSTR + 16 * g + 8 * s);
#pragma unroll
    for (int u = 0; u < 2; ++u)
      kT[u] = TrRead<T>::read(Kc, L::QSTR, w * 32 + 8 * u + 8 * g, g, l, dsel_chunk<DP>(0, l), dsel<DP>(0, x));

    f32x16 dk = acc_zero(), dv = acc_zero();

    // Fixed-order sum of the NW slabs of step `it`, scale, store (or add to what earlier key chunks
    // stored).  Runs one step late, after the loads of the following step have been requested, so
    // that neither its LDS reads nor its global store sit on the critical path; for the same reason
    // the earlier chunks' dQ values are requested a step ahead (fetch_dq_old).
    typedef T out4_t __attribute__((ext_vector_type(4)));
    const int rrow = tid >> 3, rc4 = tid & 7;           // threads 0..255: one 4-column run of one row
    const bool reducer = tid < 8 * DP;
    out4_t dq_old = {(T)0.0f, (T)0.0f, (T)0.0f, (T)0.0f};
    auto fetch_dq_old = [&](int it) {
      if (kc > 0 && reducer) {
        const int qi = it * 32 + rrow;
        dq_old = *reinterpret_cast<const out4_t*>(dQg + __umul24((unsigned)(qi < S ? qi : S - 1), dq_ss) + (4 * rc4 < D ? 4 * rc4 : 0));
      }
    };
    // reduce_load requests the four first slabs' values of step `it` at the top of the following step,
    // together with that step's operand reads; reduce_dq finishes the sum after the step's loads
    // have been issued.
    f32x4 part[4];
    auto reduce_load = [&](int it) {
      if (reducer) {
        const float* sl0 = reinterpret_cast<const float*>(Wv + L::TR_BYTES) + (it & 1) * (32 * L::SSTR) + rrow * L::SSTR + 4 * rc4;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) part[ww] = *reinterpret_cast<const f32x4*>(sl0 + ww * (WAVE_BYTES / 4));
      }
    };
    auto reduce_dq = [&](int it) {
      if (reducer) {
        const float* sl0 = reinterpret_cast<const float*>(Wv + L::TR_BYTES) + (it & 1) * (32 * L::SSTR) + rrow * L::SSTR + 4 * rc4;
        f32x4 sum = part[0];
#pragma unroll
        for (int ww = 1; ww < 4; ++ww) sum += part[ww];
        for (int ww = 4; ww < NW; ++ww) sum += *reinterpret_cast<const f32x4*>(sl0 + ww * (WAVE_BYTES / 4));
        const int qi = it * 32 + rrow;
        if (qi < S && 4 * rc4 < D) {
          float o4[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) o4[e] = sum[e] * p.scale;
          if (kc > 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) o4[e] += (float)dq_old[e];
          }
          out4_t ov = {(T)o4[0], (T)o4[1], (T)o4[2], (T)o4[3]};
          *reinterpret_cast<out4_t*>(dQg + __umul24((unsigned)qi, dq_ss) + 4 * rc4) = ov;
        }
      }
    };

    auto step = [&](const int it, frag& sa) {
      const int buf = it & 1;
      const bool more = it + 1 < NT;
#ifdef MF_TIMELINE
      const int tls = ((kc * NW + w) * NT + it) * 8;
#endif
      MF_TL(p, tls + 0);

      const T* qs = Stage + buf * L::STAGE_ELEMS;
      const T* dos = qs + 32 * L::QSTR;
      const int arow = unperm32(x);
      frag qA[KS], doA[KS], qT[2], doT[2];
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        qA[s] = ld8<T>(qs + arow * L::QSTR + 16 * g + 8 * s);
        doA[s] = ld8<T>(dos + arow * L::QSTR + 16 * g + 8 * s);
      }
      const frag qaugA = make_aug<T>(ones_g, g == 0 ? Lpk[it * 32 + arow] : 0u);
      const frag doaugA = make_aug<T>(g == 0 ? Dpk[it * 32 + arow] : 0u, 0u);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        doT[u] = TrRead<T>::read(dos, L::QSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(0, l), dsel<DP>(0, x));
        qT[u] = TrRead<T>::read(qs, L::QSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(0, l), dsel<DP>(0, x));
      }
      if (it > 0) reduce_load(it - 1);
      f32x16 z = mma(qaugA, maugB, bzn);
      MF_TL(p, tls + 1);
      // Everything for the following steps is requested here, AFTER the last use of the bias registers.
      // The vector-memory counter retires in order, so the order of issue is chosen such that the
      // only wait of a step is the one for its bias tile (top of the step): the dQ store of the
      // previous step first, then the read-back of earlier chunks' dQ (used a step later, after the
      // next bias wait), the next bias tile, and last the query-tile load that has two steps to land.
      __builtin_amdgcn_sched_barrier(0);
      MF_TL(p, tls + 2);
      if (it > 0) reduce_dq(it - 1);
      MF_TL(p, tls + 3);
      // staging: `sa` holds query tile it + 1, requested two steps ago; publish it for the next step
      // and request tile it + 3 into the same register
      if (more) stash_q(buf ^ 1, sa);
      fetch_dq_old(it);
      load_bias(more ? it + 1 : it);
      fetch_q(it + 3, sa);
      __builtin_amdgcn_sched_barrier(0);
      f32x16 dp = mma(doaugA, vaugB, acc_zero());
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        z = mma(qA[s], kf[s], z);
        dp = mma(doA[s], vf[s], dp);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pr = fast_exp2(z[i] * cexp);
        z[i] = pr;
        dp[i] = pr * dp[i];
      }
      frag pf[2], dsf[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) { pf[u] = acc_half<T>(z, u); dsf[u] = acc_half<T>(dp, u); }
      MF_TL(p, tls + 4);
      // dS, rows = keys, through this wavefront's LDS tile and back transposed.  LDS operations of one
      // wavefront execute in program order, which is all the ordering this exchange needs; the dV / dK
      // products run while it is in flight.
      st8<T>(Trw + x * L::TSTR + 16 * g, dsf[0]);
      st8<T>(Trw + x * L::TSTR + 16 * g + 8, dsf[1]);
      frag dsT[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) dsT[u] = TrRead<T>::read(Trw, L::TSTR, 8 * u + 8 * g, g, l, plain_chunk(l), x);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        dv = mma(doT[u], pf[u], dv);
        dk = mma(qT[u], dsf[u], dk);
      }
      __builtin_amdgcn_sched_barrier(0);
      MF_TL(p, tls + 5);
      f32x16 dq = mma(kT[0], dsT[0], acc_zero());
      dq = mma(kT[1], dsT[1], dq);

      // partial dQ^T -> this step's slab: lane (x = query, g) owns 16 contiguous columns
      float* slab = Slw + buf * (32 * L::SSTR);
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        f32x4 v;
        v[0] = dq[4 * c4]; v[1] = dq[4 * c4 + 1]; v[2] = dq[4 * c4 + 2]; v[3] = dq[4 * c4 + 3];
        *reinterpret_cast<f32x4*>(slab + x * L::SSTR + 16 * g + 4 * c4) = v;
      }
      MF_TL(p, tls + 6);
      barrier_keep_vm<63>();   // LDS hand-over only: global loads / stores stay in flight
      MF_TL(p, tls + 7);
    };
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0) once: the loop's own wait counts stay exact
    // two steps per trip, so that each staging register is named statically; an odd last step runs
    // after the loop
    for (int it = 0; it + 1 < NT; it += 2) {
      step(it, sa1);                       // publishes tile it + 1, requests tile it + 3
      step(it + 1, sa0);
    }
    if (NT & 1) step(NT - 1, sa1);
    reduce_load(NT - 1);
    reduce_dq(NT - 1);

    if (j < S) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int d0 = 16 * g + 8 * u;
        if (d0 < D) {
          f32x16 dks = dk;
#pragma unroll
          for (int i = 0; i < 16; ++i) dks[i] *= p.scale;
          st8<T>(dKg + (int64_t)j * p.dk.ss + d0, acc_half<T>(dks, u));
          st8<T>(dVg + (int64_t)j * p.dv.ss + d0, acc_half<T>(dv, u));
        }
      }
    }
    __syncthreads();   // the next chunk restages K and the first query tile
  }
}

template <typename T, int MAXT, int MINW>
static hipError_t launch_dqkv_rk_t(const EvoParams& p, int NW, hipStream_t stream) {
  const size_t smem = RkLayout<T>::smem(NW, (p.S + 31) / 32);
  if (smem > 160 * 1024) return hipErrorInvalidValue;
  const long long blocks = (long long)round_up(p.B * p.N, 8) * p.H;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kern = evo_bwd_dqkv_rk_kernel<T, MAXT, MINW>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(64 * NW), smem, stream, p);
  return hipGetLastError();
}

// Wavefronts per work-group for the register-resident variant.  A compute unit holds 8 of its
// wavefronts (2 per SIMD), i.e. floor(8 / NW) work-groups; the estimate of the time per (b, n, h) is
// (key chunks * NW) / (resident wavefronts).  Ties go to fewer chunks.
template <typename T> static hipError_t launch_dqkv_rk(const EvoParams& p, hipStream_t stream) {
  const int NT = (p.S + 31) / 32;
  int best_nw = 4;
  long long best_cost = -1;
  for (int nw = 4; nw <= 8; ++nw) {
    if (nw > 4 && RkLayout<T>::smem(nw, NT) > 160 * 1024) continue;   // four wavefronts fit: the caller has checked
    const int chunks = (NT + nw - 1) / nw;
    const int resident = nw * (8 / nw);
    const long long cost = ((long long)chunks * nw * 840 / resident) * 64 + chunks;
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_nw = nw; }
  }
  if (best_nw == 4) return launch_dqkv_rk_t<T, 256, 2>(p, 4, stream);
  return launch_dqkv_rk_t<T, 512, 1>(p, best_nw, stream);
}

template <typename T, int DP, int TPW> static size_t dqkv_smem(int NW) {
  using L = BwdLayout<T, DP>;
  return (size_t)NW * TPW * 32 * L::QSTR * sizeof(T) + (size_t)2 * L::STAGE_ELEMS * sizeof(T) + 128 * 4 +
         (size_t)NW * L::wave_bytes(TPW);
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

// Wavefronts per work-group (NW) of the general kernel, one key tile per wavefront.  Preference order:
// fewest key chunks (one chunk means dQ is written once, never read back), then fewest idle tile
// slots, then the smaller group.  fp32 with D > 32 needs more than 256 registers per lane and runs
// with four wavefronts (one per SIMD).
template <typename T, int DP> static hipError_t launch_dqkv_d(const EvoParams& p, hipStream_t stream) {
  const int NT = (p.S + 31) / 32;
  constexpr bool kWide = sizeof(T) == 4 && DP > 32;
  const int max_nw = kWide ? 4 : 8;
  int best_nw = 4;
  long long best_cost = -1;
  for (int nw = 4; nw <= max_nw; ++nw) {
    if (dqkv_smem<T, DP, 1>(nw) > 160 * 1024) continue;
    const int chunks = (NT + nw - 1) / nw;
    const long long cost = ((long long)chunks << 40) + ((long long)(chunks * nw - NT) << 20) + nw;
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_nw = nw; }
  }
  if (best_cost < 0) return hipErrorInvalidValue;
  if constexpr (kWide) return launch_dqkv_t<T, DP, 1, 256>(p, 4, stream);
  else return launch_dqkv_t<T, DP, 1, 512>(p, best_nw, stream);
}

static int dbias_num_cu();

template <typename T> static hipError_t launch_dqkv_s(const EvoParams& p, hipStream_t stream) {
  if (evo_bwd_dqkv_pw_supported(p)) return launch_evo_bwd_dqkv_pw(p, dbias_num_cu(), stream);
  if constexpr (sizeof(T) == 2) {
    // the register-resident variant forms row offsets with 24-bit multiplies
    auto fits = [&](int64_t ss) { return ss < (1 << 24) && (int64_t)p.S * ss < (1LL << 31); };
    const bool lds_ok = RkLayout<T>::smem(4, (p.S + 31) / 32) <= 80 * 1024;   // two work-groups per compute unit
    if (p.D <= 32 && lds_ok && fits(p.q.ss) && fits(p.dO.ss) && fits(p.o.ss) && fits(p.dq.ss))
      return launch_dqkv_rk<T>(p, stream);
  }
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
// HP = heads per work-group.  With H * D 16-bit values per position two neighbouring heads share every
// 128-byte line of Q, K, V and dO, and the L1 fetches whole lines: a work-group that handles one head
// moves twice the bytes it uses (this kernel is bound by exactly that L2 -> L1 stream).  With HP = 2 the
// work-group has eight wavefronts, four per head of a pair, working on the same patch and row in step, so
// the second head finds its half of every line in the L1.
template <typename T, int DP, int TR, int HP>
__global__ void __launch_bounds__(256 * HP, HP == 2 ? 1 : ((sizeof(T) == 4 && DP > 32) ? 1 : 2))
evo_bwd_dbias_kernel(const EvoParams p, const int IB, const int JB) {
  constexpr int AHEAD = DP <= 32 ? 2 : 1;
  using L = BwdLayout<T, DP>;
  using frag = frag_t<T>;
  constexpr int KS = DP / 16, CPR = DP / 8;
  constexpr int ROWS = TR * 32;
  constexpr int ITEMS = ROWS * CPR;
  constexpr int PF = (ITEMS + 255) / 256;

  const int tid = threadIdx.x & 255, hs = threadIdx.x >> 8;      // hs: head inside the pair (HP = 2)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  // per head: K [2][ROWS][KSTR], V [2][ROWS][QSTR] and, with HP = 2, the query-side tiles Q, dO [2][128][QSTR]
  constexpr int QT_ELEMS = HP == 2 ? 2 * 128 * L::QSTR : 0;
  constexpr int HEAD_ELEMS = 2 * ROWS * (L::KSTR + L::QSTR) + 2 * QT_ELEMS;
  T* const lds0 = reinterpret_cast<T*>(smem_raw);
  T* Ks = lds0 + hs * HEAD_ELEMS;
  T* Vs = Ks + 2 * ROWS * L::KSTR;
  T* Qs = Vs + 2 * ROWS * L::QSTR;              // HP = 2 only
  T* dOs = Qs + QT_ELEMS;

  const int R = IB * JB;
  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  int h, b, chunk, reg;
  if (HP == 2) {
    // (b, head pair, chunk) groups of R patches, dealt out evenly: XCD x takes the contiguous run
    // [x * per_xcd, (x + 1) * per_xcd) of the (group, patch) list, so that a group's patches (which share
    // Q, K, V, dO) stay in at most two L2s while every XCD gets the same number of work-groups
    const int64_t total = (int64_t)p.B * (p.H / 2) * p.n_chunks * R;
    const int64_t per_xcd = (total + 7) / 8;
    const int64_t q = xcd * per_xcd + kq;
    if (kq >= per_xcd || q >= total) return;
    const int grp = (int)(q / R);
    reg = (int)(q % R);
    chunk = grp % p.n_chunks;
    const int hb = grp / p.n_chunks;
    h = (hb % (p.H / 2)) * 2 + hs;
    b = hb / (p.H / 2);
  } else {
    const int G = p.B * p.H * p.n_chunks;
    // Each XCD takes a contiguous run of groups (b, head pair, chunk, head in pair): the two heads of a
    // pair share every 128-byte line, so they should at least meet in one L2.  With an odd run length
    // some pairs straddle two XCDs; the run length is what balances the device.
    const int hp = (p.H & 1) ? 1 : 2;
    const int gpx = (G + 7) / 8;                             // groups per XCD
    const int grp = xcd * gpx + kq / R;
    if (grp >= G) return;
    reg = kq % R;
    // grp = ((b * (H / hp) + head pair) * n_chunks + chunk) * hp + head inside the pair
    const int hsub = grp % hp;
    chunk = (grp / hp) % p.n_chunks;
    const int hb = grp / hp / p.n_chunks;
    h = (hb % (p.H / hp)) * hp + hsub;
    b = hb / (p.H / hp);
  }
  const int ib = reg % IB, jb = reg / IB;

  const int w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
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
  // HP = 2: the eight wavefronts stage both heads together, one whole 128-byte line (2 heads x 32 values)
  // per eight lanes, so the pointers below address head 2 * pair; the launcher has checked that the head
  // stride of Q, K, V, dO is D = 32 elements.
  const int t512 = threadIdx.x;
  const int c8 = t512 & 7;                               // 16-byte chunk of the pair line: head c8 >> 2, chunk c8 & 3
  const T* Kp = reinterpret_cast<const T*>(p.k.ptr) + b * p.k.sb + (h - hs) * p.k.sh + 8 * c8;
  const T* Vp = reinterpret_cast<const T*>(p.v.ptr) + b * p.v.sb + (h - hs) * p.v.sh + 8 * c8;
  const T* Qp = reinterpret_cast<const T*>(p.q.ptr) + b * p.q.sb + (h - hs) * p.q.sh + 8 * c8;
  const T* dOp = reinterpret_cast<const T*>(p.dO.ptr) + b * p.dO.sb + (h - hs) * p.dO.sh + 8 * c8;

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
      // element (query qi, key j) of the backward-layout tile (j / 32, qi / 32)
      const int qq = qi_c & 31;
      bz[t][r] = j < 32 * p.bias_nt
                     ? biasg[((int64_t)(j >> 5) * p.bias_nt + (qi_c >> 5)) * 1024 + (((qq & 15) >> 2) * 64 + 32 * (qq >> 4) + (j & 31)) * 4 + (qq & 3)]
                     : 0.0f;
    }
  }
  frag qaug = frag_zero<T>();
  if (g == 0) { qaug[0] = (T)1.0f; qaug[1] = (T)1.0f; }

  // Staging registers, AHEAD sets: the row consumed in iteration n was requested in iteration
  // n - AHEAD (two rows of loads in flight where the registers allow it).  fetch() only ISSUES loads (clamped addresses, no
  // arithmetic on the results); zeroing of padded columns / rows and every conversion happens where
  // the set is consumed, two iterations later.
  struct Staged {
    frag k[PF], v[PF];
    unsigned mraw;
    frag q[KS], dO[KS];
    float lraw, draw;
  };
  Staged sA, sB;
  const int mask_es = p.mask_dtype == MF_F32 ? 4 : (p.mask_dtype == MF_F16 || p.mask_dtype == MF_BF16) ? 2 : 1;
  const int mj = jt0 * 32 + tid < S ? jt0 * 32 + tid : S - 1;     // mask column of the threads tid < ROWS
  auto fetch = [&](int n, Staged& st) {
    if constexpr (HP == 2) {
      int j = jt0 * 32 + (t512 >> 3);                    // 64 key rows x 8 chunks = 512 threads
      j = j < S ? j : S - 1;
      st.k[0] = ld8<T>(Kp + (int64_t)n * p.k.sn + (int64_t)j * p.k.ss);
      st.v[0] = ld8<T>(Vp + (int64_t)n * p.v.sn + (int64_t)j * p.v.ss);
    } else {
      const T* kn = Kg + (int64_t)n * p.k.sn;
      const T* vn = Vg + (int64_t)n * p.v.sn;
#pragma unroll
      for (int i = 0; i < PF; ++i) {
        const int c = tid + 256 * i;
        const int kk = (c < ITEMS ? c : 0) / CPR, dc = c % CPR;
        int j = jt0 * 32 + kk;
        j = j < S ? j : S - 1;
        const int d0 = 8 * dc < D ? 8 * dc : 0;
        st.k[i] = ld8<T>(kn + (int64_t)j * p.k.ss + d0);
        st.v[i] = ld8<T>(vn + (int64_t)j * p.v.ss + d0);
      }
    }
    {
      const unsigned char* mp = reinterpret_cast<const unsigned char*>(p.mask) +
                                (b * p.mask_sb + n * p.mask_sn + (int64_t)mj * p.mask_sj) * mask_es;
      if (mask_es == 4) st.mraw = *reinterpret_cast<const unsigned*>(mp);
      else if (mask_es == 2) st.mraw = *reinterpret_cast<const unsigned short*>(mp);
      else st.mraw = *mp;
    }
    if constexpr (HP == 2) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {                      // 128 query rows x 8 chunks = 2 x 512 threads
        int qr = ib * 128 + 64 * i + (t512 >> 3);
        qr = qr < S ? qr : S - 1;
        st.q[i] = ld8<T>(Qp + (int64_t)n * p.q.sn + (int64_t)qr * p.q.ss);
        st.dO[i] = ld8<T>(dOp + (int64_t)n * p.dO.sn + (int64_t)qr * p.dO.ss);
      }
    } else {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = (DP / 2) * g + 8 * s;
        const int dcl = d0 < D ? d0 : 0;
        st.q[s] = ld8<T>(Qg + (int64_t)n * p.q.sn + dcl);
        st.dO[s] = ld8<T>(dOg + (int64_t)n * p.dO.sn + dcl);
      }
    }
    const int64_t ridx = (((int64_t)b * p.N + n) * p.H + h) * S + qi_c;
    st.lraw = p.lse[ridx];
    st.draw = p.delta[ridx];
  };
  auto stash = [&](int buf, const Staged& st) {
    T* kd = Ks + buf * ROWS * L::KSTR;
    T* vd = Vs + buf * ROWS * L::QSTR;
    if constexpr (HP == 2) {
      // this thread's chunk belongs to head c8 >> 2: write it into that head's tiles
      T* const hb = lds0 + (c8 >> 2) * HEAD_ELEMS;
      const int dc = c8 & 3;
      {
        const int kk = t512 >> 3;
        const int row = (kk & ~31) + perm32(kk & 31);
        const bool ok = jt0 * 32 + kk < S;
        st8<T>(hb + (buf * ROWS + row) * L::KSTR + 8 * dc, ok ? st.k[0] : frag_zero<T>());
        st8<T>(hb + 2 * ROWS * L::KSTR + (buf * ROWS + row) * L::QSTR + 8 * dc, ok ? st.v[0] : frag_zero<T>());
      }
      T* const qb = hb + 2 * ROWS * (L::KSTR + L::QSTR) + buf * 128 * L::QSTR;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = 64 * i + (t512 >> 3);
        const bool ok = ib * 128 + row < S;
        st8<T>(qb + row * L::QSTR + 8 * dc, ok ? st.q[i] : frag_zero<T>());
        st8<T>(qb + QT_ELEMS + row * L::QSTR + 8 * dc, ok ? st.dO[i] : frag_zero<T>());
      }
    } else {
#pragma unroll
      for (int i = 0; i < PF; ++i) {
        const int c = tid + 256 * i;
        if (c < ITEMS) {
          const int kk = c / CPR, dc = c % CPR;
          const int row = (kk & ~31) + perm32(kk & 31);
          const bool ok = jt0 * 32 + kk < S && 8 * dc < D;
          st8<T>(kd + row * L::KSTR + 8 * dc, ok ? st.k[i] : frag_zero<T>());
          st8<T>(vd + row * L::QSTR + 8 * dc, ok ? st.v[i] : frag_zero<T>());
        }
      }
    }
    if (tid < ROWS) {
      float mv;
      if (mask_es == 4) mv = __builtin_bit_cast(float, st.mraw);
      else if (p.mask_dtype == MF_F16) mv = (float)__builtin_bit_cast(f16_t, (unsigned short)st.mraw);
      else if (p.mask_dtype == MF_BF16) mv = __builtin_bit_cast(float, st.mraw << 16);
      else mv = st.mraw ? 0.0f : -__builtin_inff();
      mv = jt0 * 32 + tid < S ? mv * inv_scale : -__builtin_inff();
      const int row = (tid & ~31) + perm32(tid & 31);
      frag a = frag_zero<T>();
      T hi, lo;
      split_hi_lo<T>(mv, hi, lo);
      a[0] = hi; a[1] = lo;
      st8<T>(kd + row * L::KSTR + DP, a);
      st8<T>(kd + row * L::KSTR + DP + 8, frag_zero<T>());
    }
  };

  // one row n: consume the staged set, publish K / V, request row n + AHEAD into the same set, compute
  auto row_step = [&](int n, int buf, Staged& st) {
    frag qc[KS], doc[KS];
    if constexpr (HP != 2) {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const bool ok = qi < S && (DP / 2) * g + 8 * s < D;
        qc[s] = ok ? st.q[s] : frag_zero<T>();
        doc[s] = ok ? st.dO[s] : frag_zero<T>();
      }
    }
    float l2p = (qi < S && st.lraw != -__builtin_inff()) ? st.lraw * MF_LOG2E : __builtin_inff();
    float dlc = st.draw;
    if constexpr (HP != 2) {
#pragma unroll
      for (int s = 0; s < KS; ++s) { pin(qc[s]); pin(doc[s]); }
    }
    pin(l2p); pin(dlc);
    stash(buf, st);
    __syncthreads();
    fetch(n + AHEAD < n_end ? n + AHEAD : n_end - 1, st);   // the tail repeats the last row rather than branching around loads
    if constexpr (HP == 2) {
      // this lane's query row of its own head, staged by the whole work-group
      const T* qrow = Qs + (buf * 128 + w * 32 + x) * L::QSTR + (DP / 2) * g;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        qc[s] = ld8<T>(qrow + 8 * s);
        doc[s] = ld8<T>(qrow + QT_ELEMS + 8 * s);
      }
    }

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
          const float pr = fast_exp2(__builtin_fmaf(z[r], cexp, -l2p));
          acc[t][r] = __builtin_fmaf(pr, dp[r] - dlc, acc[t][r]);
        }
      }
    }
  };

  if (n_begin < n_end) {
    if constexpr (AHEAD == 2) {
      fetch(n_begin, sA);
      fetch(n_begin + 1 < n_end ? n_begin + 1 : n_begin, sB);
      int n = n_begin;
      for (; n + 1 < n_end; n += 2) {     // both halves unconditional: the loop-carried load order is fixed
        row_step(n, 0, sA);
        row_step(n + 1, 1, sB);
      }
      if (n < n_end) row_step(n, 0, sA);
    } else {
      fetch(n_begin, sA);
      for (int n = n_begin; n < n_end; ++n) row_step(n, (n - n_begin) & 1, sA);
    }
  }

  // ---- store the patch: lane (x = query, g) owns 16 contiguous keys per tile ---------------------
  // chunk 0 writes into dbias itself, the others into the partial buffers that the reduction adds to it
  float* dst = (chunk > 0 ? p.dbias_part + (int64_t)(chunk - 1) * p.B * p.H * S * S : p.dbias) +
               ((int64_t)b * p.H + h) * S * S;
  if (qi < S) {
    const bool vec = (S & 3) == 0;     // rows of the gradient are 16-byte aligned
#pragma unroll
    for (int t = 0; t < TR; ++t)
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const int j = (jt0 + t) * 32 + 16 * g + 4 * c4;
        float* d4 = dst + (int64_t)qi * S + j;
        if (vec && j + 3 < S) {
          f32x4 v = {acc[t][4 * c4], acc[t][4 * c4 + 1], acc[t][4 * c4 + 2], acc[t][4 * c4 + 3]};
          *reinterpret_cast<f32x4*>(d4) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (j + e < S) d4[e] = acc[t][4 * c4 + e];
        }
      }
  }
}

// out += sum over the partial buffers part[0 .. parts), in that order (out holds the first chunk's sum); four
// elements per thread when `vec` (n a multiple of 4).
__global__ void __launch_bounds__(256) dbias_reduce_kernel(const float* part, float* out, int64_t n, int parts, int vec) {
  if (vec) {
    const int64_t n4 = n >> 2;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
      // parts <= 7: all loads are issued together, the sum keeps its fixed order
      f32x4 v[8];
      v[0] = *reinterpret_cast<const f32x4*>(out + 4 * i);
#pragma unroll
      for (int c = 1; c < 8; ++c) {
        const f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
        v[c] = c <= parts ? *reinterpret_cast<const f32x4*>(part + (int64_t)(c - 1) * n + 4 * i) : z;
      }
      f32x4 s = v[0];
#pragma unroll
      for (int c = 1; c < 8; ++c) s += v[c];
      *reinterpret_cast<f32x4*>(out + 4 * i) = s;
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
      float v[8];
      v[0] = out[i];
#pragma unroll
      for (int c = 1; c < 8; ++c) v[c] = c <= parts ? part[(int64_t)(c - 1) * n + i] : 0.0f;
      float s = v[0];
#pragma unroll
      for (int c = 1; c < 8; ++c) s += v[c];
      out[i] = s;
    }
  }
}

// Key tiles per wavefront patch: limited by the registers the patch and its bias seed occupy.
static int dbias_tr(int dtype, int D) { return (dtype == MF_F32 || D > 32) ? 1 : 2; }

// Compute units of the CURRENT device, asked on every call: a process may drive several devices, and the
// answer decides grids and workspace sizes (256 when no device can be queried, e.g. without a GPU).
static int dbias_num_cu() {
  int dev = 0, n = 0;
  return (hipGetDevice(&dev) == hipSuccess &&
          hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
}

// Number of chunks the N rows are split into.  Work-groups of one (b, h, chunk) group are placed on
// one XCD (they share Q, dO, K, V in its L2) and two work-groups fit a compute unit, so the busiest XCD
// runs ceil(groups / 8) * regions work-groups in rounds of 2 * CUs / 8, each round lasting
// ceil(N / chunks) row steps.  Every chunk also costs one partial [B, H, S, S] buffer that is written
// and read back, priced in row steps (about 1.4 us) at about 2 TB/s so that near-ties go to the
// smaller workspace.  Pick the chunk count with the smallest estimate.
// Two heads per work-group (see the kernel) for the 16-bit types at D <= 32 when the heads pair up.
static bool dbias_pairs_heads(int dtype, int D, int H) { return dtype != MF_F32 && D <= 32 && (H & 1) == 0; }

int evo_num_cu() { return dbias_num_cu(); }

int evo_dbias_chunks(int B, int N, int S, int H, int D, int dtype) {
  const int TR = dbias_tr(dtype, D);
  const int NT = (S + 31) / 32;
  const int IB = (S + 127) / 128, JB = (NT + TR - 1) / TR;
  const long long regions = (long long)IB * JB;
  const bool pairs = dbias_pairs_heads(dtype, D, H);
  const long long cu_xcd = dbias_num_cu() / 8 > 0 ? dbias_num_cu() / 8 : 1;
  const long long slots_xcd = pairs ? cu_xcd : 2 * cu_xcd;          // eight-wavefront groups: one per compute unit
  const double part_cost = (double)B * H * S * S * 8.0 / 2.0e12 / 1.4e-6;
  int best = 1;
  double best_cost = -1.0;
  for (int c = 1; c <= 8 && c <= N; ++c) {     // at most 8 partial buffers: they count as activation memory
    const int rows = (N + c - 1) / c;
    if ((N + rows - 1) / rows != c) continue;
    // work-groups of the busiest XCD: whole groups per XCD, or (paired heads) an even split of all patches
    const long long wg_xcd = pairs ? ((long long)B * (H / 2) * c * regions + 7) / 8
                                   : (((long long)B * H * c + 7) / 8) * regions;
    const long long rounds = (wg_xcd + slots_xcd - 1) / slots_xcd;
    const double cost = (double)rounds * rows + (c > 1 ? c * part_cost : 0.0);
    if (best_cost < 0.0 || cost < best_cost) { best_cost = cost; best = c; }
  }
  return best;
}

// Fixed-order sum of the chunks' partial buffers (nothing to do with one chunk: the kernel wrote dbias itself).
static hipError_t launch_dbias_reduce(const EvoParams& p, hipStream_t stream) {
  if (p.n_chunks <= 1) return hipSuccess;
  const int64_t n = (int64_t)p.B * p.H * p.S * p.S;
  const int vec = (n & 3) == 0;     // partial buffers and dbias are 16-byte aligned
  int64_t rb = ((vec ? n >> 2 : n) + 255) / 256;
  if (rb > 2048) rb = 2048;
  hipLaunchKernelGGL(dbias_reduce_kernel, dim3((unsigned)rb), dim3(256), 0, stream, p.dbias_part, p.dbias, n,
                     p.n_chunks - 1, vec);
  return hipGetLastError();
}

template <typename T, int DP, int TR, int HP> static hipError_t launch_dbias_t(const EvoParams& p, hipStream_t stream) {
  using L = BwdLayout<T, DP>;
  const int NT = (p.S + 31) / 32;
  const int IB = (p.S + 127) / 128, JB = (NT + TR - 1) / TR;
  const size_t smem = (size_t)HP * (2 * TR * 32 * (L::KSTR + L::QSTR) + (HP == 2 ? 4 * 128 * L::QSTR : 0)) * sizeof(T);
  long long blocks;
  if (HP == 2) blocks = ((long long)p.B * (p.H / 2) * p.n_chunks * IB * JB + 7) / 8 * 8;
  else blocks = ((long long)p.B * p.H * p.n_chunks + 7) / 8 * 8 * IB * JB;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kern = evo_bwd_dbias_kernel<T, DP, TR, HP>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256 * HP), smem, stream, p, IB, JB);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  return launch_dbias_reduce(p, stream);
}

template <typename T> static hipError_t launch_dbias_s(const EvoParams& p, hipStream_t stream) {
  constexpr bool wide = sizeof(T) == 4;
  if constexpr (!wide) {
    // whole-line staging of a head pair needs the two heads side by side in memory (D = 32 exactly)
    if (dbias_pairs_heads(p.dtype, p.D, p.H) && p.D == 32 && p.q.sh == 32 && p.k.sh == 32 && p.v.sh == 32 &&
        p.dO.sh == 32) {
#ifndef MF_NO_DBIAS_RING
      if (evo_bwd_dbias_ring_supported(p)) {
        const hipError_t e = launch_evo_bwd_dbias_ring(p, stream);
        return e != hipSuccess ? e : launch_dbias_reduce(p, stream);
      }
#endif
      return launch_dbias_t<T, 32, 2, 2>(p, stream);
    }
  }
  if (p.D <= 32) return launch_dbias_t<T, 32, wide ? 1 : 2, 1>(p, stream);
  if (p.D <= 64) return launch_dbias_t<T, 64, 1, 1>(p, stream);
  return hipErrorInvalidValue;
}

// delta[b, n, h, s] = sum_d dO[b, n, s, h, d] O[b, n, s, h, d] on its own (evoattention.py:272-301): D / 8 lanes per
// (s, h), consecutive lanes on consecutive 16-byte chunks of a position's H * D values.  The dQ/dK/dV kernels form
// delta themselves; this kernel serves the order in which the bias gradient runs before them.
template <typename T>
__global__ void __launch_bounds__(256) evo_delta_kernel(const EvoParams p) {
  const int CPR = p.D / 8;                                   // lanes per (s, h): 1, 2, 4 or 8
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)p.B * p.N * p.S * p.H * CPR;
  const int64_t it = item < total ? item : total - 1;        // whole groups stay together: no early exit
  const int dc = (int)(it % CPR);
  int64_t r = it / CPR;
  const int h = (int)(r % p.H); r /= p.H;
  const int s = (int)(r % p.S); r /= p.S;
  const int n = (int)(r % p.N);
  const int64_t b = r / p.N;
  const T* dO = reinterpret_cast<const T*>(p.dO.ptr) + b * p.dO.sb + n * p.dO.sn + s * p.dO.ss + h * p.dO.sh + 8 * dc;
  const T* O = reinterpret_cast<const T*>(p.o.ptr) + b * p.o.sb + n * p.o.sn + s * p.o.ss + h * p.o.sh + 8 * dc;
  const frag_t<T> a = ld8<T>(dO), c = ld8<T>(O);
  float part = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) part += (float)a[e] * (float)c[e];
  if (CPR >= 2) part += __shfl_xor(part, 1);
  if (CPR >= 4) part += __shfl_xor(part, 2);
  if (CPR >= 8) part += __shfl_xor(part, 4);
  if (dc == 0 && item < total) p.delta[((b * p.N + n) * p.H + h) * p.S + s] = part;
}

hipError_t launch_evo_delta(const EvoParams& p, hipStream_t stream) {
  const int64_t total = (int64_t)p.B * p.N * p.S * p.H * (p.D / 8);
  const int64_t blocks = (total + 255) / 256;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  switch (p.dtype) {
    case MF_BF16: hipLaunchKernelGGL(evo_delta_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, p); break;
    case MF_F16: hipLaunchKernelGGL(evo_delta_kernel<f16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, p); break;
    case MF_F32: hipLaunchKernelGGL(evo_delta_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
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
