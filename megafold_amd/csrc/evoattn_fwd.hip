// Forward pass of the pair-biased, key-masked attention for gfx950.
//
//   z[i, j] = scale * <Q[i, :], K[j, :]> + bias[i, j] + mask[j]
//   O[i, :] = softmax_j(z[i, :]) V          LSE[i] = logsumexp_j z[i, j]
//
// Follows the arithmetic of the reference kernel _attn_fwd / _attn_fwd_inner
// (megafold/model/FusedEvoAttention/evoattention.py:10-98, 122-261) and of the eager form in
// tests/test_evoattention.py:45-56, but reads and writes the API layout [B, N, S, H, D] directly.
//
// One work-group (4 wavefronts) owns 128 query rows of one (b, n, h); each wavefront owns 32 rows.
// The score tile is computed transposed (rows = keys, columns = queries) so that a lane owns one
// query: the online-softmax reductions are register-local, and the exponentiated accumulator
// registers are, without any data movement, the B operand of the P.V product.  K and V blocks are
// staged row-major in LDS (double buffered); V reaches the MFMA through transposing LDS reads.
// The additive key mask rides through one extra MFMA step (K side: mask split in two 16-bit
// halves, Q side: ones) and the pair bias is the initial value of the accumulator, so neither
// costs a vector-ALU instruction per score.
#include "common.h"
#include "evoattn.h"

namespace mf {

template <typename T, int DP> struct FwdLayout {
  static constexpr int UNIT = 16 / (int)sizeof(T);
  static constexpr int KRAW = DP + 16;  // data columns + 16 mask-carrier columns
  static constexpr int KSTR = ((KRAW / UNIT) % 2 == 0) ? KRAW + UNIT : KRAW;
  static constexpr int VSTR = ((DP / UNIT) % 2 == 0) ? DP + UNIT : DP;
};

template <typename T, int DP, int KT, int WPE>
__global__ void __launch_bounds__(256, WPE) evo_fwd_kernel(const EvoParams p, const int QB) {
  using L = FwdLayout<T, DP>;
  using frag = frag_t<T>;
  constexpr int KS = DP / 16;       // contraction steps of Q.K^T
  constexpr int DT = DP / 32;       // 32-row tiles of the transposed output
  constexpr int KB = KT * 32;       // keys per staged block
  constexpr int CPR = DP / 8;       // 8-element chunks per row
  constexpr int NCH = KB * CPR / 256;  // chunks per thread per tensor
  static_assert(KB * CPR % 256 == 0, "block must split evenly over 256 threads");
  static_assert(KB <= 256, "one thread per key for the mask");

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Ks = reinterpret_cast<T*>(smem_raw);   // [2][KB][KSTR]
  T* Vs = Ks + 2 * KB * L::KSTR;            // [2][KB][VSTR]

  // ---- which (b, n, h, query block) is ours.  Work-groups are dealt round-robin to the 8 XCDs;
  // all work-groups of one (b, n) are placed on the same XCD so the rows they share hit its L2.
  const int per_bn = p.H * QB;
  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  const int bn = (kq / per_bn) * 8 + xcd;
  if (bn >= p.B * p.N) return;
  const int inner = kq % per_bn;
  const int h = inner % p.H, qb = inner / p.H;
  const int b = bn / p.N, n = bn % p.N;

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const int S = p.S, D = p.D;

  const T* Qg = reinterpret_cast<const T*>(p.q.ptr) + b * p.q.sb + n * p.q.sn + h * p.q.sh;
  const T* Kg = reinterpret_cast<const T*>(p.k.ptr) + b * p.k.sb + n * p.k.sn + h * p.k.sh;
  const T* Vg = reinterpret_cast<const T*>(p.v.ptr) + b * p.v.sb + n * p.v.sn + h * p.v.sh;
  T* Og = reinterpret_cast<T*>(p.o.ptr) + b * p.o.sb + n * p.o.sn + h * p.o.sh;
  const float* biasg = p.bias + b * p.bias_sb + h * p.bias_sh;
  const int64_t mask_base = b * p.mask_sb + n * p.mask_sn;

  const int qrow = qb * 128 + w * 32 + x;
  const int qrow_c = qrow < S ? qrow : S - 1;

  // ---- Q fragments (B operand): lane (x, g) holds Q[qrow][(DP/2)*g + 8*s + e], pre-scaled in T
  // like the reference does (evoattention.py:39).
  frag qf[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int d0 = (DP / 2) * g + 8 * s;
    qf[s] = d0 < D ? scale8<T>(ld8<T>(Qg + (int64_t)qrow_c * p.q.ss + d0), p.scale) : frag_zero<T>();
  }
  frag qaug = frag_zero<T>();
  if (g == 0) { qaug[0] = (T)1.0f; qaug[1] = (T)1.0f; }

  // ---- staging registers for the next K/V block
  frag kreg[NCH], vreg[NCH];
  float mreg = 0.0f;
  auto fetch = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = tid + 256 * i;
      const int kk = c / CPR, dc = c % CPR;
      const int j = kb * KB + kk;
      const bool ok = j < S && 8 * dc < D;
      kreg[i] = ok ? ld8<T>(Kg + (int64_t)j * p.k.ss + 8 * dc) : frag_zero<T>();
      vreg[i] = ok ? ld8<T>(Vg + (int64_t)j * p.v.ss + 8 * dc) : frag_zero<T>();
    }
    if (tid < KB) {
      const int j = kb * KB + tid;
      mreg = j < S ? load_any(p.mask, p.mask_dtype, mask_base + (int64_t)j * p.mask_sj) : -__builtin_inff();
    }
  };
  auto stash = [&](int buf) {
    T* kd = Ks + buf * KB * L::KSTR;
    T* vd = Vs + buf * KB * L::VSTR;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = tid + 256 * i;
      const int kk = c / CPR, dc = c % CPR;
      const int krow = (kk & ~31) + perm32(kk & 31);
      st8<T>(kd + krow * L::KSTR + 8 * dc, kreg[i]);
      st8<T>(vd + kk * L::VSTR + 8 * dc, vreg[i]);
    }
    if (tid < KB) {
      const int krow = (tid & ~31) + perm32(tid & 31);
      frag a = frag_zero<T>();
      T hi, lo;
      split_hi_lo<T>(mreg, hi, lo);
      a[0] = hi; a[1] = lo;
      st8<T>(kd + krow * L::KSTR + DP, a);
      st8<T>(kd + krow * L::KSTR + DP + 8, frag_zero<T>());
    }
  };

  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = acc_zero();
  float m_run = -__builtin_inff(), lsum = 0.0f;

  const int nkb = (S + KB - 1) / KB;
  fetch(0);
  stash(0);
  __syncthreads();

  for (int kb = 0; kb < nkb; ++kb) {
    const int buf = kb & 1;
    const bool more = kb + 1 < nkb;
    if (more) fetch(kb + 1);

    const T* kt = Ks + buf * KB * L::KSTR;
    const T* vt = Vs + buf * KB * L::VSTR;

    // scores, transposed: z[t][r] <-> key kb*KB + 32*t + 16*g + r, query qrow
    f32x16 z[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int key0 = kb * KB + 32 * t + 16 * g;
      if (key0 < S) {
        const float* bp = biasg + (int64_t)qrow_c * p.bias_ld + key0;
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          f32x4 v = *reinterpret_cast<const f32x4*>(bp + 4 * c4);
          z[t][4 * c4 + 0] = v[0]; z[t][4 * c4 + 1] = v[1]; z[t][4 * c4 + 2] = v[2]; z[t][4 * c4 + 3] = v[3];
        }
      } else {
        z[t] = acc_zero();
      }
    }
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      const T* krow = kt + (32 * t + x) * L::KSTR;
      z[t] = mma(ld8<T>(krow + DP + 8 * g), qaug, z[t]);
#pragma unroll
      for (int s = 0; s < KS; ++s) z[t] = mma(ld8<T>(krow + (DP / 2) * g + 8 * s), qf[s], z[t]);
    }

    // online softmax over this block (lane-local except one exchange between the two halves)
    float mx = z[0][0];
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, z[t][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == -__builtin_inff()) ? 0.0f : m_new;
    const float alpha = fast_exp2((m_run - m_use) * MF_LOG2E);
    const float nm = -m_use * MF_LOG2E;
    float rs = 0.0f;
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = fast_exp2(__builtin_fmaf(z[t][r], MF_LOG2E, nm));
        z[t][r] = e;
        rs += e;
      }
    lsum = lsum * alpha + rs;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;

    // O^T += V^T P^T : A operand = V^T through transposing reads, B operand = P from registers
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const frag pf = acc_half<T>(z[t], u);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const frag vf = TrRead<T>::read(vt, L::VSTR, 32 * t + 8 * u + 8 * g, g, l, dsel_chunk<DP>(dt, l),
                                          dsel<DP>(dt, x));
          o[dt] = mma(vf, pf, o[dt]);
        }
      }

    if (more) stash(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, store O (DP/2 contiguous columns per lane) and the logsumexp
  const float l_tot = lsum + __shfl_xor(lsum, 32);
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  if (qrow < S) {
    T* orow = Og + (int64_t)qrow * p.o.ss;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int d0 = (DP / 2) * g + 16 * dt + 8 * u;
        if (d0 < D) {
          const f32x16& c = o[dt];
          const frag f = u == 0 ? cvt8<T>(c[0] * inv, c[1] * inv, c[2] * inv, c[3] * inv, c[4] * inv, c[5] * inv,
                                          c[6] * inv, c[7] * inv)
                                : cvt8<T>(c[8] * inv, c[9] * inv, c[10] * inv, c[11] * inv, c[12] * inv, c[13] * inv,
                                          c[14] * inv, c[15] * inv);
          st8<T>(orow + d0, f);
        }
      }
    if (g == 0) {
      const float lse = l_tot > 0.0f ? m_run + __builtin_logf(l_tot) : -__builtin_inff();
      p.lse[(((int64_t)b * p.N + n) * p.H + h) * S + qrow] = lse;
    }
  }
}

template <typename T, int DP, int KT, int WPE> static hipError_t launch_fwd_t(const EvoParams& p, hipStream_t stream) {
  using L = FwdLayout<T, DP>;
  constexpr int KB = KT * 32;
  const size_t smem = (size_t)2 * KB * (L::KSTR + L::VSTR) * sizeof(T);
  const int QB = (p.S + 127) / 128;
  const int bn8 = round_up(p.B * p.N, 8);
  const long long blocks = (long long)bn8 * p.H * QB;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kern = evo_fwd_kernel<T, DP, KT, WPE>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), smem, stream, p, QB);
  return hipGetLastError();
}

template <typename T> static hipError_t launch_fwd_d(const EvoParams& p, hipStream_t stream) {
  // keys per staged block and the occupancy the register allocator is asked to reach
  constexpr bool wide = sizeof(T) == 4;
  if (p.D <= 32) return launch_fwd_t<T, 32, 4, wide ? 2 : 3>(p, stream);
  if (p.D <= 64) return launch_fwd_t<T, 64, 2, 2>(p, stream);
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

// ---- pair bias of any float dtype / strides -> fp32 [B, H, S, ld], zero padded for j >= S --------
__global__ void __launch_bounds__(256) bias_to_f32_kernel(const void* src, int dtype, int64_t sb, int64_t sh, int64_t si,
                                                          int64_t sj, float* dst, int H, int S, int ld, int64_t total) {
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
    const int j = (int)(idx % ld);
    const int64_t r = idx / ld;
    const int i = (int)(r % S);
    const int64_t bh = r / S;
    const int h = (int)(bh % H);
    const int64_t b = bh / H;
    dst[idx] = j < S ? load_any(src, dtype, b * sb + h * sh + i * si + j * sj) : 0.0f;
  }
}

hipError_t launch_bias_to_f32(const void* src, int dtype, int64_t sb, int64_t sh, int64_t si, int64_t sj, float* dst,
                              int B, int H, int S, int ld, hipStream_t stream) {
  const int64_t total = (int64_t)B * H * S * ld;
  if (total == 0) return hipSuccess;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(bias_to_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, dtype, sb, sh, si, sj, dst,
                     H, S, ld, total);
  return hipGetLastError();
}

}  // namespace mf
