// Forward pass of the pair-biased, key-masked attention for gfx950.
//
//   z[i, j] = scale * <Q[i, :], K[j, :]> + bias[i, j] + mask[j]
//   O[i, :] = softmax_j(z[i, :]) V          LSE[i] = logsumexp_j z[i, j]
//
// Follows the arithmetic of the reference kernel _attn_fwd / _attn_fwd_inner
// (megafold/model/FusedEvoAttention/evoattention.py:10-98, 122-261) and of the eager form in
// tests/test_evoattention.py:45-56, but reads and writes the API layout [B, N, S, H, D] directly.
//
// Work decomposition.  A work-group (4 wavefronts) owns 128 query positions of one head and R
// consecutive rows n; a wavefront owns 32 query positions.  The pair-bias tile of a (query strip,
// key block) is the same for every row n, so it is loaded ONCE into registers and used as the
// read-only accumulator input of the score MFMAs of all R rows: the bias, which is the largest
// operand of the op after the row batching of the model (N times re-read), costs 1/R of its traffic
// and no vector-ALU instruction.  The host hands the kernels bias/scale, so the accumulator holds
// z/scale = <q, k> + bias/scale + mask/scale from UNSCALED 16-bit q and k — the softmax scale is
// applied in fp32 inside the exponent's fused multiply-add and is exact (the reference rounds
// q*scale to the input type, evoattention.py:39).
//
// The score tile is computed transposed (rows = keys, columns = queries) so that a lane owns one
// query: online-softmax reductions are register-local, and the exponentiated accumulator registers
// are, without any data movement, the B operand of the P.V product.  K and V of one (key block, row)
// stage are staged row-major in LDS (double buffered); V reaches the MFMA through transposing LDS
// reads.  The additive key mask rides through one extra MFMA step (K side: mask/scale split in two
// 16-bit halves, Q side: ones).
#include <cstdlib>
#include "common.h"
#include "evoattn.h"

namespace mf {

template <typename T, int DP> struct FwdLayout {
  static constexpr int UNIT = 16 / (int)sizeof(T);
  static constexpr int KSTR = ((DP / UNIT) % 2 == 0) ? DP + UNIT : DP;   // K and V rows (odd number of 16-byte units)
};

// A query's logits sit in two lanes (l and l ^ 32); this combines the two halves.
__device__ __forceinline__ float max_across_halves(float v) { return fmaxf(v, __shfl_xor(v, 32)); }
__device__ __forceinline__ float sum_across_halves(float v) { return v + __shfl_xor(v, 32); }

// The mask carrier fragment: (hi, lo, 0, ...) from one packed 32-bit word (16-bit types) or the fp32
// value itself.
template <typename T> __device__ __forceinline__ frag_t<T> aug_frag(unsigned w) {
  u32x4 v = {w, 0u, 0u, 0u};
  return __builtin_bit_cast(frag_t<T>, v);
}
template <> __device__ __forceinline__ f32x8 aug_frag<float>(unsigned w) {
  f32x8 f = {__builtin_bit_cast(float, w), 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  return f;
}
template <typename T> __device__ __forceinline__ unsigned pack_mask(float m) {
  T hi, lo;
  split_hi_lo<T>(m, hi, lo);
  typedef T pair_t __attribute__((ext_vector_type(2)));
  pair_t pr = {hi, lo};
  return __builtin_bit_cast(unsigned, pr);
}
template <> __device__ __forceinline__ unsigned pack_mask<float>(float m) { return __builtin_bit_cast(unsigned, m); }

// Softmax bookkeeping.  Every query keeps an offset m (in accumulator units) and accumulates
// p = exp2(c (z - m)); ANY offset gives the same softmax as long as nothing overflows, so the
// offset is only refreshed — maximum search, lane exchange, rescaling of the running sum and of the
// output accumulators — when a stage's probabilities come out larger than 2^16 (or overflow), which
// after the first stage practically never happens.  The common path is fma, exp2, add and one
// packed convert per logit.  The offset starts hugely negative so the first finite logit forces a
// refresh; masked logits (-inf) give exactly 0 under every offset.
#define MF_M_INIT (-1.0e30f)
// Refresh threshold on the sum of a lane's 16 probabilities of a stage.  The probabilities are converted to
// the element type for the P.V product: for float16 every one of them must stay below 65504, which a sum
// below 2^15 guarantees; bfloat16 and float32 have the range of fp32 and only need the sums to stay finite.
template <typename T> struct PLimit { static constexpr float value = 1048576.0f; };     /* 16 logits x 2^16 */
template <> struct PLimit<f16_t> { static constexpr float value = 32768.0f; };

template <typename T, int DP, int R, int WPE>
__global__ void __launch_bounds__(256, WPE) evo_fwd_kernel(const EvoParams p, const int QB, const int NG) {
  using L = FwdLayout<T, DP>;
  using frag = frag_t<T>;
  constexpr int KS = DP / 16;       // contraction steps of Q.K^T
  constexpr int DT = DP / 32;       // 32-row tiles of the transposed output
  constexpr int CPR = DP / 8;       // 8-element chunks per row
  constexpr int ITEMS = R * 32 * CPR;            // chunks of one stage (one 32-key tile, R rows), per tensor
  constexpr int NCH = (ITEMS + 255) / 256;
  constexpr int STG = R * 32 * L::KSTR;          // elements of one staged tensor

  const int S = p.S, D = p.D;
  const int NT = (S + 31) >> 5;

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Ks = reinterpret_cast<T*>(smem_raw);        // [2][R][32][KSTR]
  T* Vs = Ks + 2 * STG;                          // [2][R][32][KSTR]
  unsigned* Ma = reinterpret_cast<unsigned*>(Vs + 2 * STG);   // [R][NT*32] packed mask/scale, then 1 zero word

  // ---- which (b, row group, h, query block) is ours.  Work-groups are dealt round-robin to the 8
  // XCDs; all work-groups of one (b, row group) are placed on the same XCD so the K/V rows they
  // share hit its L2.
  const int per_grp = p.H * QB;
  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  const int grp = (kq / per_grp) * 8 + xcd;
  if (grp >= p.B * NG) return;
  const int inner = kq % per_grp;
  const int h = inner % p.H, qb = inner / p.H;
  const int b = grp / NG, n0 = (grp % NG) * R;

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const float cexp = p.scale * MF_LOG2E;     // exponent multiplier on the unscaled accumulator
  const float inv_scale = 1.0f / p.scale;

  const int qrow = qb * 128 + w * 32 + x;
  const int qrow_c = qrow < S ? qrow : S - 1;

  // ---- Q fragments of the R rows (B operand): lane (x, g) holds Q[qrow][(DP/2)*g + 8*s + e].
  // Rows past N are clamped: computed, never stored.
  frag qf[R][KS];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = n0 + r < p.N ? n0 + r : p.N - 1;
    const T* Qg = reinterpret_cast<const T*>(p.q.ptr) + b * p.q.sb + n * p.q.sn + h * p.q.sh + (int64_t)qrow_c * p.q.ss;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int d0 = (DP / 2) * g + 8 * s;
      qf[r][s] = d0 < D ? ld8<T>(Qg + d0) : frag_zero<T>();
    }
  }
  frag qaug = frag_zero<T>();
  if (g == 0) { qaug[0] = (T)1.0f; qaug[1] = (T)1.0f; }

  // ---- mask/scale of all keys of the R rows, packed once; keys past S are -inf ---------------------
  for (int i = tid; i < R * NT * 32; i += 256) {
    const int r = i / (NT * 32), j = i % (NT * 32);
    const int n = n0 + r < p.N ? n0 + r : p.N - 1;
    const float mv = j < S ? load_any(p.mask, p.mask_dtype, b * p.mask_sb + n * p.mask_sn + (int64_t)j * p.mask_sj) * inv_scale
                           : -__builtin_inff();
    Ma[i] = pack_mask<T>(mv);
  }
  if (tid == 0) Ma[R * NT * 32] = 0u;
  // the upper lane half carries no mask: it reads the zero word
  const unsigned* mask_lane = g == 0 ? Ma + unperm32(x) : Ma + R * NT * 32;
  const int mask_step = g == 0 ? 32 : 0;

  // bias/scale rows are zero padded to whole tiles: no bounds checks on the loads
  // this wavefront's row of bias tiles (forward layout, see EvoParams::bias); query tiles past S are
  // clamped, their rows are never stored
  const int qt = qb * 4 + w < p.bias_nt ? qb * 4 + w : p.bias_nt - 1;
  const float* biasp = p.bias + b * p.bias_sb + h * p.bias_sh + (int64_t)qt * p.bias_nt * 1024 + 4 * l;

  // ---- staging of one stage.  Source pointers advance by 32 keys per stage; keys past S are
  // clamped to the last key (their logits are -inf through the mask, and P = 0 times a finite V is 0).
  // Chunks that only pad D up to DP are zeroed once and never touched again.
  const T* ksrc[NCH];
  const T* vsrc[NCH];
  int kdst[NCH], vdst[NCH], kkey[NCH];
  bool live[NCH];
  frag kreg[NCH], vreg[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = tid + 256 * i;
    const int r = (c / (32 * CPR)) % R, kk = (c / CPR) % 32, dc = c % CPR;
    const int n = n0 + r < p.N ? n0 + r : p.N - 1;
    live[i] = c < ITEMS && 8 * dc < D;
    kkey[i] = kk;
    ksrc[i] = reinterpret_cast<const T*>(p.k.ptr) + b * p.k.sb + h * p.k.sh + (int64_t)n * p.k.sn + 8 * dc;
    vsrc[i] = reinterpret_cast<const T*>(p.v.ptr) + b * p.v.sb + h * p.v.sh + (int64_t)n * p.v.sn + 8 * dc;
    kdst[i] = (r * 32 + perm32(kk)) * L::KSTR + 8 * dc;
    vdst[i] = (r * 32 + kk) * L::KSTR + 8 * dc;
    if (c < ITEMS && !live[i]) {
#pragma unroll
      for (int bb = 0; bb < 2; ++bb) {
        st8<T>(Ks + bb * STG + kdst[i], frag_zero<T>());
        st8<T>(Vs + bb * STG + vdst[i], frag_zero<T>());
      }
    }
  }
  auto fetch = [&](int jt) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (live[i]) {
        int j = jt * 32 + kkey[i];
        j = j < S ? j : S - 1;
        kreg[i] = ld8<T>(ksrc[i] + (int64_t)j * p.k.ss);
        vreg[i] = ld8<T>(vsrc[i] + (int64_t)j * p.v.ss);
      }
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (live[i]) {
        st8<T>(Ks + buf * STG + kdst[i], kreg[i]);
        st8<T>(Vs + buf * STG + vdst[i], vreg[i]);
      }
    }
  };

  f32x16 o[R][DT];
  float m_use[R], nm[R], lsum[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    m_use[r] = MF_M_INIT;
    nm[r] = -MF_M_INIT * cexp;
    lsum[r] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[r][dt] = acc_zero();
  }

  auto load_bias = [&](int jt, f32x16& dst) {
    const float* bp = biasp + jt * 1024;
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(bp + 256 * c4);
      dst[4 * c4 + 0] = v[0]; dst[4 * c4 + 1] = v[1]; dst[4 * c4 + 2] = v[2]; dst[4 * c4 + 3] = v[3];
    }
  };

  // one stage: key tile jt of all R rows; `bz` is this tile's bias/scale, `bznext` receives the next
  auto stage = [&](int jt, const f32x16& bz, f32x16& bznext) {
    const int buf = jt & 1;
    const bool more = jt + 1 < NT;
    if (more) {
      fetch(jt + 1);
      load_bias(jt + 1, bznext);
    }
    const T* kt = Ks + buf * STG;
    const T* vt = Vs + buf * STG;
    const unsigned* mrow = mask_lane + jt * mask_step;

#pragma unroll
    for (int r = 0; r < R; ++r) {
      // scores / scale, transposed: z[i] <-> key 32*jt + 16*g + i, query qrow
      const T* krow = kt + (r * 32 + x) * L::KSTR;
      const frag ma = aug_frag<T>(mrow[g == 0 ? r * NT * 32 : 0]);
      auto scores = [&]() {
        f32x16 zz = mma(ma, qaug, bz);
#pragma unroll
        for (int s = 0; s < KS; ++s) zz = mma(ld8<T>(krow + (DP / 2) * g + 8 * s), qf[r][s], zz);
        return zz;
      };
      float e[16];
      float rs = 0.0f;
      {
        const f32x16 z = scores();
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          e[i] = fast_exp2(__builtin_fmaf(z[i], cexp, nm[r]));
          rs += e[i];
        }
      }
      if (__builtin_amdgcn_ballot_w64(!(rs < PLimit<T>::value)) != 0) {       // wave-uniform; rare after the first stage
        const f32x16 z = scores();                       // recomputed: keeps the common path's register need low
        float mx = fmaxf(z[0], z[1]);
#pragma unroll
        for (int i = 2; i < 16; ++i) mx = fmaxf(mx, z[i]);
        mx = max_across_halves(mx);
        const float m_new = fmaxf(m_use[r], mx);       // mx = -inf (all masked) keeps the offset
        const float alpha = fast_exp2((m_use[r] - m_new) * cexp);
        m_use[r] = m_new;
        nm[r] = -m_new * cexp;
        lsum[r] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[r][dt][i] *= alpha;
        rs = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          e[i] = fast_exp2(__builtin_fmaf(z[i], cexp, nm[r]));
          rs += e[i];
        }
      }
      lsum[r] += rs;

      // O^T += V^T P^T : A operand = V^T through transposing reads, B operand = P from registers
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const frag pf = cvt8<T>(e[8 * u], e[8 * u + 1], e[8 * u + 2], e[8 * u + 3], e[8 * u + 4], e[8 * u + 5],
                                e[8 * u + 6], e[8 * u + 7]);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const frag vf = TrRead<T>::read(vt + r * 32 * L::KSTR, L::KSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(dt, l),
                                          dsel<DP>(dt, x));
          o[r][dt] = mma(vf, pf, o[r][dt]);
        }
      }
    }

    if (more) stash(buf ^ 1);
    // Everything requested at the top of this stage (the next tile's K/V and bias) is a whole stage old
    // here.  Draining it explicitly tells the compiler that nothing is in flight at the loop head;
    // without that it makes the first use of the bias registers wait for ALL outstanding loads,
    // including the ones the next stage has only just issued.
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0), other counters untouched
    __syncthreads();
  };

  f32x16 bzA, bzB;
  fetch(0);
  load_bias(0, bzA);
  stash(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): see the end of stage()
  __syncthreads();

  for (int jt = 0; jt < NT; jt += 2) {
    stage(jt, bzA, bzB);
    if (jt + 1 < NT) stage(jt + 1, bzB, bzA);
  }

  // ---- epilogue: normalise, store O (DP/2 contiguous columns per lane) and the logsumexp
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = n0 + r;
    const float l_tot = sum_across_halves(lsum[r]);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (qrow < S && n < p.N) {
      T* orow = reinterpret_cast<T*>(p.o.ptr) + b * p.o.sb + n * p.o.sn + h * p.o.sh + (int64_t)qrow * p.o.ss;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int d0 = (DP / 2) * g + 16 * dt + 8 * u;
          if (d0 < D) {
            const f32x16& c = o[r][dt];
            const frag f = u == 0 ? cvt8<T>(c[0] * inv, c[1] * inv, c[2] * inv, c[3] * inv, c[4] * inv, c[5] * inv,
                                            c[6] * inv, c[7] * inv)
                                  : cvt8<T>(c[8] * inv, c[9] * inv, c[10] * inv, c[11] * inv, c[12] * inv,
                                            c[13] * inv, c[14] * inv, c[15] * inv);
            st8<T>(orow + d0, f);
          }
        }
      if (g == 0) {
        const float lse = l_tot > 0.0f ? m_use[r] * p.scale + __builtin_logf(l_tot) : -__builtin_inff();
        p.lse[(((int64_t)b * p.N + n) * p.H + h) * S + qrow] = lse;
      }
    }
  }
}

// LDS of a work-group with R rows: K / V tiles of the rows, double buffered, and the rows' mask values
template <typename T, int DP> static size_t fwd_smem(int R, int NT) {
  using L = FwdLayout<T, DP>;
  return (size_t)4 * R * 32 * L::KSTR * sizeof(T) + ((size_t)R * NT * 32 + 4) * 4;
}

template <typename T, int DP, int R, int WPE> static hipError_t launch_fwd_t(const EvoParams& p, hipStream_t stream) {
  const int NT = (p.S + 31) / 32;
  const size_t smem = fwd_smem<T, DP>(R, NT);
  if (smem > 160 * 1024) return hipErrorInvalidValue;   // not reached: launch_fwd_d lowers R until the rows fit
  const int QB = (p.S + 127) / 128;
  const int NG = (p.N + R - 1) / R;
  const long long blocks = (long long)round_up(p.B * NG, 8) * p.H * QB;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kern = evo_fwd_kernel<T, DP, R, WPE>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), smem, stream, p, QB, NG);
  return hipGetLastError();
}

// Rows n per work-group (R).  More rows share one pair-bias tile, but the grid runs in whole rounds of
// resident work-groups (3 per compute unit for R = 2, 2 for R = 3 and 4), and a stage costs about
// 7 + R units of time, so the best R is the one with the smallest rounds * (7 + R) (fitted to
// measurements at S = 384 and S = 768).  Small problems use fewer rows to keep the device busy.
template <typename T> static hipError_t launch_fwd_d(const EvoParams& p, hipStream_t stream) {
  constexpr bool wide = sizeof(T) == 4;
  const long long QB = (p.S + 127) / 128;
  const int num_cu = evo_num_cu();
  int rows = 4;
  double best = -1.0;
  for (int r = 2; r <= 4; ++r) {
    const long long wgs = (long long)round_up(p.B * ((p.N + r - 1) / r), 8) * p.H * QB;
    const long long slots = (long long)(r == 2 ? 3 : 2) * num_cu;
    const double cost = (double)((wgs + slots - 1) / slots) * (7.0 + r);
    if (best < 0.0 || cost < best) { best = cost; rows = r; }
  }
  const long long groups1 = (long long)p.B * p.N * p.H * QB;
  if (groups1 < 2048) rows = rows > 2 ? 2 : rows;   // small problems: keep enough work-groups
  if (groups1 < 1024 || p.N == 1) rows = 1;
  // very long sequences: the rows' mask values (4 R S bytes) must fit the LDS next to the tiles; one row always
  // does for the sequence lengths the C ABI admits
  const int NT = (p.S + 31) / 32;
  while (rows > 1 && (p.D <= 32 ? fwd_smem<T, 32>(rows, NT) : fwd_smem<T, 64>(rows, NT)) > 160 * 1024) --rows;
  if constexpr (wide) {
    if (p.D <= 32) return rows >= 2 ? launch_fwd_t<T, 32, 2, 2>(p, stream) : launch_fwd_t<T, 32, 1, 2>(p, stream);
    if (p.D <= 64) return launch_fwd_t<T, 64, 1, 2>(p, stream);
  } else {
    if (p.D <= 32) {
      if (rows >= 4) return launch_fwd_t<T, 32, 4, 2>(p, stream);
      if (rows == 3) return launch_fwd_t<T, 32, 3, 2>(p, stream);
      if (rows >= 2) return launch_fwd_t<T, 32, 2, 3>(p, stream);
      return launch_fwd_t<T, 32, 1, 4>(p, stream);
    }
    if (p.D <= 64) return rows >= 2 ? launch_fwd_t<T, 64, 2, 2>(p, stream) : launch_fwd_t<T, 64, 1, 3>(p, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_evo_fwd(const EvoParams& p, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return launch_fwd_d<bf16_t>(p, stream);
    case MF_F16: return launch_fwd_d<f16_t>(p, stream);
    case MF_F32: return launch_fwd_d<float>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

// ---- pair bias of any float dtype / strides -> tiled fp32 copy times `mult`, zero padded ------------
// A work-group takes one 32 x 32 tile (query block ti, key block tj) of one (b, h): 8 threads read the 32
// consecutive keys of a query row, the tile goes through LDS, and every thread writes one float4 of the layout
// described at EvoParams::bias — of the forward's order (tile (ti, tj): lane = query, registers = keys), of the
// backward's (tile (tj, ti): lane = key, registers = queries), or of both from the one read.
__global__ void __launch_bounds__(256) bias_prep_kernel(const void* src, int dtype, int64_t sb, int64_t sh, int64_t si,
                                                        int64_t sj, float* dst_fwd, float* dst_bwd, int H, int S, int nt,
                                                        float mult) {
  __shared__ float tile[32][33];
  const int t = threadIdx.x;
  const int64_t tidx = blockIdx.x;
  const int tj = (int)(tidx % nt);
  const int64_t r1 = tidx / nt;
  const int ti = (int)(r1 % nt);
  const int64_t bh = r1 / nt;
  const int h = (int)(bh % H);
  const int64_t b = bh / H;
  {
    const int r = t >> 3, c = (t & 7) * 4;
    const int i = 32 * ti + r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int j = 32 * tj + c + e;
      tile[r][c + e] = (i < S && j < S) ? load_any(src, dtype, b * sb + h * sh + i * si + j * sj) * mult : 0.0f;
    }
  }
  __syncthreads();
  // float4 number t of a tile: lane l = t & 63 (x = l & 31, g = l >> 5), chunk c4 = t >> 6; value e is column / row
  // 16 g + 4 c4 + e against row / column x
  const int l = t & 63, c4 = t >> 6, x = l & 31, g = l >> 5, k0 = 16 * g + 4 * c4;
  if (dst_fwd) {
    const f32x4 v = {tile[x][k0], tile[x][k0 + 1], tile[x][k0 + 2], tile[x][k0 + 3]};
    *reinterpret_cast<f32x4*>(dst_fwd + ((bh * nt + ti) * nt + tj) * 1024 + 4 * t) = v;
  }
  if (dst_bwd) {
    const f32x4 v = {tile[k0][x], tile[k0 + 1][x], tile[k0 + 2][x], tile[k0 + 3][x]};
    *reinterpret_cast<f32x4*>(dst_bwd + ((bh * nt + tj) * nt + ti) * 1024 + 4 * t) = v;
  }
}

hipError_t launch_bias_prep(const void* src, int dtype, int64_t sb, int64_t sh, int64_t si, int64_t sj, float* dst,
                            int B, int H, int S, float mult, bool backward_layout, hipStream_t stream, float* dst_bwd) {
  const int nt = (S + 31) / 32;
  const int64_t tiles = (int64_t)B * H * nt * nt;
  if (tiles == 0) return hipSuccess;
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(bias_prep_kernel, dim3((unsigned)tiles), dim3(256), 0, stream, src, dtype, sb, sh, si, sj,
                     backward_layout ? nullptr : dst, backward_layout ? dst : dst_bwd, H, S, nt, mult);
  return hipGetLastError();
}

}  // namespace mf
