// Element-type dispatch, weight preparation and the stand-alone SwiGLU kernels of the
// LayerNorm->Linear family (the GEMM kernels live in lnlinear_impl.h, one translation unit per type).
#include "lnlinear_impl.h"

namespace mf {

template <typename T> hipError_t ln_fwd_dispatch(const LnParams& p, int act, hipStream_t stream);
template <typename T> hipError_t ln_dx_dispatch(const LnParams& p, const void* dY, hipStream_t stream);
template <typename T> hipError_t ln_dw_dispatch(const LnParams& p, const void* dY, hipStream_t stream);
template <typename T> hipError_t ln_swiglu_bwd_fused_dispatch(const LnParams& p, hipStream_t stream);
extern template hipError_t ln_swiglu_bwd_fused_dispatch<bf16_t>(const LnParams&, hipStream_t);
extern template hipError_t ln_swiglu_bwd_fused_dispatch<f16_t>(const LnParams&, hipStream_t);
extern template hipError_t ln_swiglu_bwd_fused_dispatch<float>(const LnParams&, hipStream_t);
extern template hipError_t ln_fwd_dispatch<bf16_t>(const LnParams&, int, hipStream_t);
extern template hipError_t ln_fwd_dispatch<f16_t>(const LnParams&, int, hipStream_t);
extern template hipError_t ln_fwd_dispatch<float>(const LnParams&, int, hipStream_t);
extern template hipError_t ln_dx_dispatch<bf16_t>(const LnParams&, const void*, hipStream_t);
extern template hipError_t ln_dx_dispatch<f16_t>(const LnParams&, const void*, hipStream_t);
extern template hipError_t ln_dx_dispatch<float>(const LnParams&, const void*, hipStream_t);
extern template hipError_t ln_dw_dispatch<bf16_t>(const LnParams&, const void*, hipStream_t);
extern template hipError_t ln_dw_dispatch<f16_t>(const LnParams&, const void*, hipStream_t);
extern template hipError_t ln_dw_dispatch<float>(const LnParams&, const void*, hipStream_t);

hipError_t launch_ln_fwd(const LnParams& p, int act, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return ln_fwd_dispatch<bf16_t>(p, act, stream);
    case MF_F16: return ln_fwd_dispatch<f16_t>(p, act, stream);
    case MF_F32: return ln_fwd_dispatch<float>(p, act, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_ln_swiglu_bwd_fused(const LnParams& p, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return ln_swiglu_bwd_fused_dispatch<bf16_t>(p, stream);
    case MF_F16: return ln_swiglu_bwd_fused_dispatch<f16_t>(p, stream);
    default: return hipErrorNotSupported;
  }
}

// Elements of LnParams::du the SwiGLU backward needs: the column blocks' shares of dU W'^T where the fused pass
// takes the shape (the condition of swiglu_bwd_fused_ok), all of dU otherwise.
uint64_t ln_swiglu_bwd_scratch_elems(int dtype, int64_t M, int K, int N) {
  const int KP = ln_padded_k(K);
#ifndef MF_LN_DU_FORM
  if ((dtype == MF_BF16 || dtype == MF_F16) && KP >= 32 && KP <= 128 && (N / 2) % 128 == 0)
    return (uint64_t)(N / 256) * (uint64_t)M * (uint64_t)KP;
#endif
  return (uint64_t)M * (uint64_t)N;
}

hipError_t launch_ln_bwd_dx(const LnParams& p, const void* dY, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return ln_dx_dispatch<bf16_t>(p, dY, stream);
    case MF_F16: return ln_dx_dispatch<f16_t>(p, dY, stream);
    case MF_F32: return ln_dx_dispatch<float>(p, dY, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_ln_bwd_dw(const LnParams& p, const void* dY, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return ln_dw_dispatch<bf16_t>(p, dY, stream);
    case MF_F16: return ln_dw_dispatch<f16_t>(p, dY, stream);
    case MF_F32: return ln_dw_dispatch<float>(p, dY, stream);
    default: return hipErrorInvalidValue;
  }
}

// =================================================================================================
// weight preparation:  W' = gamma (.) W in both layouts, column sums of W', folded bias
// =================================================================================================
// One work-group owns 32 columns of W and all K rows.  A thread moves 8 consecutive columns (16 bytes for
// the 16-bit types) of every 64th row, so four neighbouring threads read and write 64 contiguous bytes of
// the [K, N] layout; the transposed [N, KP] copy goes through LDS so that its rows are written whole.
template <typename T>
__global__ void __launch_bounds__(256) ln_prep_kernel(const LnParams p) {
  constexpr int CW = 32;                      // columns per work-group
  __shared__ float tile[CW][257];             // [n][k], K <= 256
  __shared__ float red_cs[64][CW + 1], red_bp[64][CW + 1];
  const int tid = threadIdx.x, c8 = tid & 3, kr = tid >> 2;
  const int n0 = blockIdx.x * CW + 8 * c8;    // first of this thread's 8 columns (N is a multiple of 8)
  const T* W = reinterpret_cast<const T*>(p.W);
  const T* gamma = reinterpret_cast<const T*>(p.gamma);
  const T* beta = reinterpret_cast<const T*>(p.beta);
  T* Wt = reinterpret_cast<T*>(p.Wt);
  float cs[8], bp[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { cs[e] = 0.0f; bp[e] = 0.0f; }
  for (int k = kr; k < p.KP; k += 64) {
    float gwf[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) gwf[e] = 0.0f;
    if (k < p.K && n0 < p.N) {
      const frag_t<T> w = ld8<T>(W + (int64_t)k * p.N + n0);
      const float gk = to_f(gamma[k]), bk = beta ? to_f(beta[k]) : 0.0f;
      frag_t<T> gw;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        gw[e] = (T)(gk * to_f(w[e]));
        gwf[e] = to_f(gw[e]);
        cs[e] += gwf[e];
        bp[e] += bk * to_f(w[e]);
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) tile[8 * c8 + e][k] = gwf[e];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) { red_cs[kr][8 * c8 + e] = cs[e]; red_bp[kr][8 * c8 + e] = bp[e]; }
  __syncthreads();
  if (tid < CW) {
    const int n2 = blockIdx.x * CW + tid;
    float a = 0.0f, b2 = 0.0f;
    for (int j = 0; j < 64; ++j) { a += red_cs[j][tid]; b2 += red_bp[j][tid]; }   // fixed order
    if (n2 < p.N) {
      if (p.colsum) p.colsum[n2] = a;
      if (p.bprime) p.bprime[n2] = b2 + (p.b ? to_f(reinterpret_cast<const T*>(p.b)[n2]) : 0.0f);
    }
  }
  if (Wt) {
    // eight consecutive k per thread: whole 16-byte (fp32: 32-byte) pieces of a transposed row
    const int k8 = p.KP / 8;
    for (int i = tid; i < CW * k8; i += 256) {
      const int r = i / k8, k = (i % k8) * 8;
      const int n2 = blockIdx.x * CW + r;
      if (n2 < p.N) {
        const float* src = &tile[r][k];
        st8<T>(Wt + (int64_t)n2 * p.KP + k, cvt8<T>(src[0], src[1], src[2], src[3], src[4], src[5], src[6], src[7]));
      }
    }
  }
}

hipError_t launch_ln_prep(const LnParams& p, bool forward, hipStream_t stream) {
  (void)forward;
  const unsigned blocks = (unsigned)((p.N + 31) / 32);
  switch (p.dtype) {
    case MF_BF16: hipLaunchKernelGGL(ln_prep_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, p); break;
    case MF_F16: hipLaunchKernelGGL(ln_prep_kernel<f16_t>, dim3(blocks), dim3(256), 0, stream, p); break;
    case MF_F32: hipLaunchKernelGGL(ln_prep_kernel<float>, dim3(blocks), dim3(256), 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// The register-resident dx kernel (ln_bwd_dx_res_kernel) is the one that adds LnParams::dx_add: 16-bit element
// types, padded K = 128, 64 <= N <= 1024 (the condition of launch_dx_t).
bool ln_bwd_takes_dx_add(int dtype, int K, int N) {
  return (dtype == MF_BF16 || dtype == MF_F16) && ln_padded_k(K) == 128 && N >= 64 && N <= 1024;
}

int ln_padded_k(int K) {
  if (K <= 0 || K % 8 != 0) return 0;
  for (int kp = 16; kp <= 256; kp *= 2)
    if (K <= kp) return kp;
  return 0;
}

int ln_row_ranges(int64_t M, int K, int N) {
  // The weight-gradient kernel runs (ranges x column blocks) work-groups, two resident per compute unit:
  // the number of ranges is chosen so that the grid is ONE round of resident work-groups (a grid of 1.25
  // rounds costs two), with at least 256 rows per range.
  const int KP = ln_padded_k(K);
  const int cw = KP > 128 ? 64 : 128;                    // columns per work-group (DwShape<KP>::CW)
  const int gy = (N + cw - 1) / cw;
  int64_t r = 2LL * num_cu() / (gy > 0 ? gy : 1);
  if (r > M / 256) r = M / 256;
  if (r > 1024) r = 1024;
  if (r < 1) r = 1;
  return (int)r;
}

// =================================================================================================
// stand-alone SwiGLU (fused_transition.py:11-52)
// =================================================================================================
template <typename T>
__global__ void __launch_bounds__(256) swiglu_fwd_kernel(const T* __restrict__ xin, T* __restrict__ y, int64_t M, int Dh) {
  const int cpr = Dh / 8;
  const int64_t total = M * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / cpr;
    const int c = (int)(i % cpr) * 8;
    const frag_t<T> a = ld8<T>(xin + m * 2 * Dh + c);
    const frag_t<T> gt = ld8<T>(xin + m * 2 * Dh + Dh + c);
    float h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { const float gv = to_f(gt[e]); h[e] = gv * sigmoidf_fast(gv) * to_f(a[e]); }
    st8<T>(y + m * Dh + c, cvt8<T>(h[0], h[1], h[2], h[3], h[4], h[5], h[6], h[7]));
  }
}

template <typename T>
__global__ void __launch_bounds__(256) swiglu_bwd_kernel(const T* __restrict__ dy, const T* xin, T* dxo, int64_t M, int Dh) {
  const int cpr = Dh / 8;
  const int64_t total = M * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / cpr;
    const int c = (int)(i % cpr) * 8;
    const frag_t<T> a = ld8<T>(xin + m * 2 * Dh + c);
    const frag_t<T> gt = ld8<T>(xin + m * 2 * Dh + Dh + c);
    const frag_t<T> d = ld8<T>(dy + m * Dh + c);
    float da[8], dg[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gv = to_f(gt[e]), dh = to_f(d[e]);
      const float sg = sigmoidf_fast(gv), silu = gv * sg;
      da[e] = dh * silu;
      dg[e] = dh * (silu * (1.0f - sg) + sg) * to_f(a[e]);
    }
    st8<T>(dxo + m * 2 * Dh + c, cvt8<T>(da[0], da[1], da[2], da[3], da[4], da[5], da[6], da[7]));
    st8<T>(dxo + m * 2 * Dh + Dh + c, cvt8<T>(dg[0], dg[1], dg[2], dg[3], dg[4], dg[5], dg[6], dg[7]));
  }
}

static unsigned ew_blocks(int64_t total) {
  int64_t b = (total + 255) / 256;
  const int64_t cap = 16LL * num_cu();
  return (unsigned)(b > cap ? cap : (b < 1 ? 1 : b));
}

hipError_t launch_swiglu_fwd(const void* x, void* y, int64_t M, int Dh, int dtype, hipStream_t stream) {
  const unsigned blocks = ew_blocks(M * (Dh / 8));
  switch (dtype) {
    case MF_BF16: hipLaunchKernelGGL(swiglu_fwd_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)x, (bf16_t*)y, M, Dh); break;
    case MF_F16: hipLaunchKernelGGL(swiglu_fwd_kernel<f16_t>, dim3(blocks), dim3(256), 0, stream, (const f16_t*)x, (f16_t*)y, M, Dh); break;
    case MF_F32: hipLaunchKernelGGL(swiglu_fwd_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, (float*)y, M, Dh); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_swiglu_bwd(const void* dy, const void* x, void* dx, int64_t M, int Dh, int dtype, hipStream_t stream) {
  const unsigned blocks = ew_blocks(M * (Dh / 8));
  switch (dtype) {
    case MF_BF16: hipLaunchKernelGGL(swiglu_bwd_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)dy, (const bf16_t*)x, (bf16_t*)dx, M, Dh); break;
    case MF_F16: hipLaunchKernelGGL(swiglu_bwd_kernel<f16_t>, dim3(blocks), dim3(256), 0, stream, (const f16_t*)dy, (const f16_t*)x, (f16_t*)dx, M, Dh); break;
    case MF_F32: hipLaunchKernelGGL(swiglu_bwd_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)dy, (const float*)x, (float*)dx, M, Dh); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace mf
