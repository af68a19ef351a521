// Parameter block and launch entry points of the LayerNorm->Linear (and LayerNorm->SwiGLU) kernels.
// Replaces the Triton kernels of the reference:
//   megafold/model/FusedLayernormLinear/fused_layernorm_linear.py
//     _first_forward_kernel :109-140, _second_forward_kernel :147-218,
//     _first_backward_kernel :226-308, _second_backward_kernel :311-348
//   megafold/model/FusedTransition/fused_transition.py  _swiglu_forward_kernel :11-26,
//     _swiglu_backward_kernel :29-52
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mf {

enum { LN_ACT_NONE = 0, LN_ACT_SWIGLU = 1, LN_ACT_SWIGLU_BWD = 2 };

struct LnParams {
  int64_t M;
  int K, N;        // N = columns of W (for SwiGLU the output has N/2 columns)
  int KP;          // K rounded up to the kernel's padded width
  int dtype;
  float eps;
  const void* x;       // [M, K]
  const void* gamma;   // [K]
  const void* beta;    // [K] or null
  const void* W;       // [K, N]
  const void* b;       // [N] or null
  void* out;           // [M, N] (or [M, N/2] with SwiGLU)
  float* mean;         // [M]
  float* rstd;         // [M]
  // prepared weights (workspace)
  void* Wt;            // [N, KP]  gamma[k] * W[k, n], transposed, element type of x   (forward)
  float* colsum;       // [N] sum_k Wt[n, k]
  float* bprime;       // [N] sum_k beta[k] W[k, n] + b[n]
  // backward
  const void* dout;    // [M, N] (or [M, N/2] with SwiGLU)
  void* dx;            // [M, K]
  const void* dx_add;  // [M, K] or null: added to dx (residual dx kernel only, see ln_bwd_takes_dx_add)
  void* du;            // SwiGLU backward scratch, ln_swiglu_bwd_scratch_elems elements: [N / 256, M, KP] shares of
                       // dU W^T (fused pass) or [M, N] gradient of the pre-activation
  void* dW;            // [K, N]   parameter gradients: float, or the element type of x when grads_as_x
  void* db;            // [N] or null
  void* dgamma;        // [K]
  void* dbeta;         // [K] or null
  int grads_as_x;
  float* Gpart;        // [R, K, N] partial x_hat^T dOut
  float* spart;        // [R, N]   partial column sums of dOut
#ifdef MF_TIMELINE
  unsigned* tl;        // development aid: cycle stamps of one work-group (see MF_TL in common.h)
  int tl_block;
#endif
  int R;               // number of row ranges (partials)
  int64_t rows_per_range;
};

// Whether the dx kernel of this element type and shape adds LnParams::dx_add.
bool ln_bwd_takes_dx_add(int dtype, int K, int N);
hipError_t launch_ln_prep(const LnParams& p, bool forward, hipStream_t stream);
hipError_t launch_ln_fwd(const LnParams& p, int act, hipStream_t stream);
// SwiGLU backward, complete (dx and the weight / LayerNorm parameter gradients; p.du is scratch);
// hipErrorNotSupported when the shape needs the separate kernels (launch_ln_fwd with LN_ACT_SWIGLU_BWD, then
// launch_ln_bwd_dx and launch_ln_bwd_dw on p.du).
hipError_t launch_ln_swiglu_bwd_fused(const LnParams& p, hipStream_t stream);
uint64_t ln_swiglu_bwd_scratch_elems(int dtype, int64_t M, int K, int N);   // elements of p.du that backward needs
hipError_t launch_ln_bwd_dx(const LnParams& p, const void* dY, hipStream_t stream);
hipError_t launch_ln_bwd_dw(const LnParams& p, const void* dY, hipStream_t stream);
hipError_t launch_swiglu_fwd(const void* x, void* y, int64_t M, int Dh, int dtype, hipStream_t stream);
hipError_t launch_swiglu_bwd(const void* dy, const void* x, void* dx, int64_t M, int Dh, int dtype, hipStream_t stream);

int ln_padded_k(int K);                 // padded K of the kernels, 0 if K is unsupported
int ln_row_ranges(int64_t M, int K, int N);    // R for the weight-gradient partials

}  // namespace mf
