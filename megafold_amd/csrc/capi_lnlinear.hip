// C-ABI entry points of LayerNorm->Linear, LayerNorm->SwiGLU and stand-alone SwiGLU: argument
// validation before any launch, workspace carving and kernel sequencing.
// Host side of the reference being replaced: layernorm_linear_forward / _backward
// (megafold/model/FusedLayernormLinear/fused_layernorm_linear.py:351-405, 408-474) and swiglu_forward /
// swiglu_backward (megafold/model/FusedTransition/fused_transition.py:55-93).
#include "../../include/megafold_amd.h"
#include <cstdlib>
#include "capi_common.h"
#include "common.h"
#include "lnlinear.h"

using namespace mf;

namespace {

struct LnPlan {
  int KP, R;
  int64_t rows_per_range;
  uint64_t off_wt, off_cs, off_bp, off_g, off_s, off_du, total;
};

LnPlan make_plan(const mf_lnlinear_args* a, bool backward) {
  LnPlan pl{};
  const uint64_t es = dtype_size(a->dtype);
  pl.KP = ln_padded_k(a->K);
  const bool swiglu = a->act == MF_ACT_SWIGLU;
  uint64_t off = 0;
  if (!backward || swiglu) {
    pl.off_wt = off; off += align256((uint64_t)a->N * pl.KP * es);
    pl.off_cs = off; off += align256((uint64_t)a->N * 4);
    pl.off_bp = off; off += align256((uint64_t)a->N * 4);
  }
  if (backward) {
    pl.R = ln_row_ranges(a->M, a->K, a->N);
    pl.rows_per_range = (a->M + pl.R - 1) / pl.R;
    pl.off_g = off; off += align256((uint64_t)pl.R * a->K * a->N * 4);
    pl.off_s = off; off += align256((uint64_t)pl.R * a->N * 4);
    if (swiglu) { pl.off_du = off; off += align256(ln_swiglu_bwd_scratch_elems(a->dtype, a->M, a->K, a->N) * es); }
  }
  pl.total = off;
  return pl;
}

int check(const mf_lnlinear_args* a, bool backward) {
  clear_error();
  if (!a) return fail(MF_ERR_NULL, "args is NULL");
  if (a->M <= 0 || a->K <= 0 || a->N <= 0)
    return fail(MF_ERR_SHAPE, "M, K, N must be positive (got %lld %d %d)", (long long)a->M, a->K, a->N);
  if (a->dtype != MF_DTYPE_F32 && a->dtype != MF_DTYPE_F16 && a->dtype != MF_DTYPE_BF16)
    return fail(MF_ERR_DTYPE, "dtype %d unsupported", a->dtype);
  if (ln_padded_k(a->K) == 0)
    return fail(MF_ERR_SHAPE, "K=%d unsupported: need a multiple of 8, at most 256", a->K);
  if (a->dtype == MF_DTYPE_F32 && a->K > 128)
    return fail(MF_ERR_SHAPE, "K=%d unsupported for fp32: rows of at most 512 bytes (K <= 128)", a->K);
  if (a->act != MF_ACT_NONE && a->act != MF_ACT_SWIGLU) return fail(MF_ERR_SHAPE, "act %d unknown", a->act);
  if (a->N % 8 != 0 || (a->act == MF_ACT_SWIGLU && a->N % 16 != 0))
    return fail(MF_ERR_SHAPE, "N=%d unsupported: need a multiple of %d", a->N, a->act == MF_ACT_SWIGLU ? 16 : 8);
  if (a->act == MF_ACT_SWIGLU && a->b) return fail(MF_ERR_SHAPE, "the SwiGLU form takes no linear bias");
  const void* need[] = {a->x, a->gamma, a->W, a->mean, a->rstd};
  const char* names[] = {"x", "gamma", "W", "mean", "rstd"};
  for (int i = 0; i < 5; ++i)
    if (!need[i]) return fail(MF_ERR_NULL, "%s is NULL", names[i]);
  if (!backward && !a->out) return fail(MF_ERR_NULL, "out is NULL");
  if (backward) {
    if (!a->dout) return fail(MF_ERR_NULL, "dout is NULL");
    if (!a->dx) return fail(MF_ERR_NULL, "dx is NULL");
    if (!a->dW) return fail(MF_ERR_NULL, "dW is NULL");
    if (!a->dgamma) return fail(MF_ERR_NULL, "dgamma is NULL");
    if (a->param_grad_dtype != 0 && a->param_grad_dtype != 1)
      return fail(MF_ERR_DTYPE, "param_grad_dtype must be 0 (float) or 1 (the dtype of x)");
    if (a->dx_add && !ln_bwd_takes_dx_add(a->dtype, a->K, a->N))
      return fail(MF_ERR_SHAPE, "dx_add is not supported for dtype %d, K=%d, N=%d (see mf_lnlinear_bwd_takes_dx_add)",
                  a->dtype, a->K, a->N);
  }
  const void* al[] = {a->x, a->W, a->out, a->dout, a->dx, a->workspace, backward ? a->dx_add : nullptr};
  const char* aln[] = {"x", "W", "out", "dout", "dx", "workspace", "dx_add"};
  for (int i = 0; i < 7; ++i)
    if (al[i] && !aligned16(al[i])) return fail(MF_ERR_ALIGN, "%s is not 16-byte aligned", aln[i]);
  const LnPlan pl = make_plan(a, backward);
  if (!a->workspace || a->workspace_bytes < pl.total)
    return fail(MF_ERR_WORKSPACE, "%s needs %llu workspace bytes, got %llu", backward ? "backward" : "forward",
                (unsigned long long)pl.total, (unsigned long long)(a->workspace ? a->workspace_bytes : 0));
  return 0;
}

LnParams fill(const mf_lnlinear_args* a, const LnPlan& pl, bool backward) {
  LnParams p{};
#ifdef MF_TIMELINE
  { const char* e = getenv("MF_TL_PTR"); p.tl = e ? reinterpret_cast<unsigned*>(strtoull(e, nullptr, 16)) : nullptr;
    const char* f = getenv("MF_TL_BLOCK"); p.tl_block = f ? atoi(f) : 0; }
#endif
  p.M = a->M; p.K = a->K; p.N = a->N; p.KP = pl.KP; p.dtype = a->dtype; p.eps = a->eps;
  p.x = a->x; p.gamma = a->gamma; p.beta = a->beta; p.W = a->W; p.b = a->b;
  p.out = a->out; p.mean = a->mean; p.rstd = a->rstd;
  unsigned char* ws = static_cast<unsigned char*>(a->workspace);
  const bool swiglu = a->act == MF_ACT_SWIGLU;
  if (!backward || swiglu) {
    p.Wt = ws + pl.off_wt;
    p.colsum = reinterpret_cast<float*>(ws + pl.off_cs);
    p.bprime = reinterpret_cast<float*>(ws + pl.off_bp);
  }
  if (backward) {
    p.Gpart = reinterpret_cast<float*>(ws + pl.off_g);
    p.spart = reinterpret_cast<float*>(ws + pl.off_s);
    p.R = pl.R; p.rows_per_range = pl.rows_per_range;
    p.dout = a->dout; p.dx = a->dx; p.dx_add = a->dx_add; p.dW = a->dW; p.db = a->db; p.dgamma = a->dgamma; p.dbeta = a->dbeta;
    p.grads_as_x = a->param_grad_dtype == 1;
    if (swiglu) p.du = ws + pl.off_du;
  }
  return p;
}

}  // namespace

extern "C" uint64_t mf_lnlinear_fwd_workspace_bytes(const mf_lnlinear_args* a) {
  if (!a || a->M <= 0 || a->K <= 0 || a->N <= 0 || ln_padded_k(a->K) == 0 || dtype_size(a->dtype) == 0) return 0;
  return make_plan(a, false).total;
}
extern "C" uint64_t mf_lnlinear_bwd_workspace_bytes(const mf_lnlinear_args* a) {
  if (!a || a->M <= 0 || a->K <= 0 || a->N <= 0 || ln_padded_k(a->K) == 0 || dtype_size(a->dtype) == 0) return 0;
  return make_plan(a, true).total;
}

extern "C" int mf_lnlinear_bwd_takes_dx_add(const mf_lnlinear_args* a) {
  return a && a->K > 0 && a->N > 0 && ln_bwd_takes_dx_add(a->dtype, a->K, a->N) ? 1 : 0;
}

extern "C" int mf_lnlinear_fwd(const mf_lnlinear_args* a) {
  int rc = check(a, false);
  if (rc) return rc;
  const LnPlan pl = make_plan(a, false);
  const LnParams p = fill(a, pl, false);
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  hipError_t e = launch_ln_prep(p, true, stream);
  if (e != hipSuccess) return (int)e;
  return (int)launch_ln_fwd(p, a->act == MF_ACT_SWIGLU ? LN_ACT_SWIGLU : LN_ACT_NONE, stream);
}

extern "C" int mf_lnlinear_bwd(const mf_lnlinear_args* a) {
  int rc = check(a, true);
  if (rc) return rc;
  const LnPlan pl = make_plan(a, true);
  const LnParams p = fill(a, pl, true);
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  hipError_t e = hipSuccess;
  // The dx kernels multiply dOut by the weights as stored and apply gamma to the fp32 products, as the reference does
  // (fused_layernorm_linear.py:281-306): only the SwiGLU form, which recomputes the pre-activation with the
  // forward's prepared operands, needs the preparation kernel.
  if (a->act == MF_ACT_SWIGLU) {
    e = launch_ln_prep(p, false, stream);
    if (e != hipSuccess) return (int)e;
  }
  const void* dY = a->dout;
  if (a->act == MF_ACT_SWIGLU) {
    // recompute the pre-activation tile by tile and turn dh into dU = [da, dg]; where the shape allows it one pass
    // forms the weight-gradient partials and dU W^T per column block, and dU never reaches memory
    e = launch_ln_swiglu_bwd_fused(p, stream);
    if (e != hipErrorNotSupported) return (int)e;
    e = launch_ln_fwd(p, LN_ACT_SWIGLU_BWD, stream);
    if (e != hipSuccess) return (int)e;
    dY = p.du;
  }
  e = launch_ln_bwd_dx(p, dY, stream);
  if (e != hipSuccess) return (int)e;
  return (int)launch_ln_bwd_dw(p, dY, stream);
}

extern "C" int mf_swiglu_fwd(const void* x, void* y, int64_t M, int32_t Dh, int32_t dtype, void* stream) {
  clear_error();
  if (!x || !y) return fail(MF_ERR_NULL, "x or y is NULL");
  if (M <= 0 || Dh <= 0 || Dh % 8 != 0) return fail(MF_ERR_SHAPE, "need M > 0 and Dh a positive multiple of 8 (got %lld, %d)", (long long)M, Dh);
  if (dtype != MF_DTYPE_F32 && dtype != MF_DTYPE_F16 && dtype != MF_DTYPE_BF16) return fail(MF_ERR_DTYPE, "dtype %d unsupported", dtype);
  if (!aligned16(x) || !aligned16(y)) return fail(MF_ERR_ALIGN, "x / y not 16-byte aligned");
  return (int)launch_swiglu_fwd(x, y, M, Dh, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int mf_swiglu_bwd(const void* dy, const void* x, void* dx, int64_t M, int32_t Dh, int32_t dtype, void* stream) {
  clear_error();
  if (!dy || !x || !dx) return fail(MF_ERR_NULL, "dy, x or dx is NULL");
  if (M <= 0 || Dh <= 0 || Dh % 8 != 0) return fail(MF_ERR_SHAPE, "need M > 0 and Dh a positive multiple of 8 (got %lld, %d)", (long long)M, Dh);
  if (dtype != MF_DTYPE_F32 && dtype != MF_DTYPE_F16 && dtype != MF_DTYPE_BF16) return fail(MF_ERR_DTYPE, "dtype %d unsupported", dtype);
  if (!aligned16(dy) || !aligned16(x) || !aligned16(dx)) return fail(MF_ERR_ALIGN, "dy / x / dx not 16-byte aligned");
  return (int)launch_swiglu_bwd(dy, x, dx, M, Dh, dtype, static_cast<hipStream_t>(stream));
}
