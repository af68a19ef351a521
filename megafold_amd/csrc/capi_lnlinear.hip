// placeholder until the LayerNorm->Linear kernels land: every entry point rejects its call.
#include "../../include/megafold_amd.h"
#include "capi_common.h"
using namespace mf;
extern "C" uint64_t mf_lnlinear_fwd_workspace_bytes(const mf_lnlinear_args*) { return 0; }
extern "C" uint64_t mf_lnlinear_bwd_workspace_bytes(const mf_lnlinear_args*) { return 0; }
extern "C" int mf_lnlinear_fwd(const mf_lnlinear_args*) { return fail(MF_ERR_SHAPE, "not implemented"); }
extern "C" int mf_lnlinear_bwd(const mf_lnlinear_args*) { return fail(MF_ERR_SHAPE, "not implemented"); }
extern "C" int mf_swiglu_fwd(const void*, void*, int64_t, int32_t, int32_t, void*) { return fail(MF_ERR_SHAPE, "not implemented"); }
extern "C" int mf_swiglu_bwd(const void*, const void*, void*, int64_t, int32_t, int32_t, void*) { return fail(MF_ERR_SHAPE, "not implemented"); }
