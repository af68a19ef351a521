// C-ABI entry points of the attention path: argument validation (before any launch, so it can be
// exercised without a GPU), workspace carving and kernel sequencing.
// Host side of the reference being replaced: EvoformerAttention.forward / .backward
// (megafold/model/FusedEvoAttention/evoattention.py:688-779, 782-903).
#include "../../include/megafold_amd.h"
#include <atomic>
#include <cstdlib>
#include "capi_common.h"
#include "common.h"
#include "evoattn.h"

using namespace mf;

namespace {

struct Plan {
  int bias_nt;              // 32 x 32 tiles per side of the fp32 bias/scale copy the kernels read
  uint64_t off_bias, off_delta, off_part, dq_scratch_bytes, part_bytes, total;
  int n_chunks, rows_per_chunk;
};

Plan make_plan(const mf_evoattn_args* a, bool backward) {
  Plan pl{};
  pl.bias_nt = (a->S + 31) / 32;
  uint64_t off = 0;
  pl.off_bias = off;
  // the backward reads the tiles a forward call left in bias_tiles_bwd, if the caller kept them
  if (!(backward && a->bias_tiles_bwd)) off += align256((uint64_t)a->B * a->H * pl.bias_nt * pl.bias_nt * 4096);
  pl.n_chunks = 1;
  pl.rows_per_chunk = a->N;
  if (backward) {
    pl.off_delta = off;
    off += align256((uint64_t)a->B * a->N * a->H * a->S * 4);
    pl.off_part = off;
    uint64_t part_bytes = 0;
    if (a->dbias) {
      pl.n_chunks = evo_dbias_chunks(a->B, a->N, a->S, a->H, a->D, a->dtype);
      pl.rows_per_chunk = (a->N + pl.n_chunks - 1) / pl.n_chunks;
      // the first chunk writes into dbias itself
      if (pl.n_chunks > 1) part_bytes = (uint64_t)(pl.n_chunks - 1) * a->B * a->H * a->S * a->S * 4;
    }
    // the multi-pass dQ array of the dQ/dK/dV kernel is dead before the bias-gradient kernel starts: one region.
    // In the memory-lean order the partial sums live in the dq buffer instead.
    pl.part_bytes = part_bytes;
    if (a->dbias && (a->phases & MF_EVO_BWD_LEAN)) part_bytes = 0;
    pl.dq_scratch_bytes = evo_bwd_dqkv_pw_scratch_bytes(a->dtype, a->S, a->D, evo_num_cu());
    off += align256(part_bytes > pl.dq_scratch_bytes ? part_bytes : pl.dq_scratch_bytes);
  }
  pl.total = off;
  return pl;
}

int check_tensor(const char* name, const void* p, const int64_t* st, int esize) {
  if (!p) return fail(MF_ERR_NULL, "%s is NULL", name);
  if (!aligned16(p)) return fail(MF_ERR_ALIGN, "%s is not 16-byte aligned", name);
  const int unit = 16 / esize;
  for (int i = 0; i < 4; ++i)
    if (st[i] % unit != 0 || st[i] < 0)
      return fail(MF_ERR_STRIDE, "%s stride[%d]=%lld is not a non-negative multiple of %d elements", name, i,
                  (long long)st[i], unit);
  return 0;
}

int check_common(const mf_evoattn_args* a) {
  clear_error();
  if (!a) return fail(MF_ERR_NULL, "args is NULL");
  if (a->B <= 0 || a->N <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0)
    return fail(MF_ERR_SHAPE, "B, N, S, H, D must be positive (got %d %d %d %d %d)", a->B, a->N, a->S, a->H, a->D);
  if (a->D % 8 != 0 || a->D > 64) return fail(MF_ERR_SHAPE, "D=%d unsupported: need a multiple of 8, at most 64", a->D);
  // the forward keeps the mask values of a row (4 S bytes) in LDS next to its tiles
  if (a->S > MF_EVOATTN_MAX_S) return fail(MF_ERR_SHAPE, "S=%d unsupported: at most %d", a->S, MF_EVOATTN_MAX_S);
  if (a->dtype != MF_DTYPE_F32 && a->dtype != MF_DTYPE_F16 && a->dtype != MF_DTYPE_BF16)
    return fail(MF_ERR_DTYPE, "dtype %d unsupported for q/k/v", a->dtype);
  if (a->bias_dtype != MF_DTYPE_F32 && a->bias_dtype != MF_DTYPE_F16 && a->bias_dtype != MF_DTYPE_BF16)
    return fail(MF_ERR_DTYPE, "bias_dtype %d unsupported", a->bias_dtype);
  if (a->mask_dtype < MF_DTYPE_F32 || a->mask_dtype > MF_DTYPE_BOOL)
    return fail(MF_ERR_DTYPE, "mask_dtype %d unsupported", a->mask_dtype);
  const int es = dtype_size(a->dtype);
  int rc;
  if ((rc = check_tensor("q", a->q, a->q_stride, es))) return rc;
  if ((rc = check_tensor("k", a->k, a->k_stride, es))) return rc;
  if ((rc = check_tensor("v", a->v, a->v_stride, es))) return rc;
  if ((rc = check_tensor("o", a->o, a->o_stride, es))) return rc;
  if (!a->bias) return fail(MF_ERR_NULL, "bias is NULL");
  if (!a->mask) return fail(MF_ERR_NULL, "mask is NULL");
  if (!a->lse) return fail(MF_ERR_NULL, "lse is NULL");
  return 0;
}

EvoTensor tens(const void* p, const int64_t* st) {
  return EvoTensor{const_cast<void*>(p), st[0], st[1], st[2], st[3]};
}

int fill_params(const mf_evoattn_args* a, const Plan& pl, EvoParams& p, hipStream_t stream, bool prep, bool backward) {
  p = EvoParams{};
  p.B = a->B; p.N = a->N; p.S = a->S; p.H = a->H; p.D = a->D;
  p.dtype = a->dtype;
  p.scale = a->scale;
  p.q = tens(a->q, a->q_stride); p.k = tens(a->k, a->k_stride); p.v = tens(a->v, a->v_stride);
  p.o = tens(a->o, a->o_stride);
  p.mask = a->mask; p.mask_dtype = a->mask_dtype;
  p.mask_sb = a->mask_stride[0]; p.mask_sn = a->mask_stride[1]; p.mask_sj = a->mask_stride[2];
  p.lse = a->lse;
  unsigned char* ws = static_cast<unsigned char*>(a->workspace);
  float* b32 = reinterpret_cast<float*>(ws + pl.off_bias);
  if (a->scale <= 0.0f) return fail(MF_ERR_SHAPE, "scale must be positive (got %g)", (double)a->scale);
  if (a->bias_tiles_bwd && !aligned16(a->bias_tiles_bwd)) return fail(MF_ERR_ALIGN, "bias_tiles_bwd is not 16-byte aligned");
  if (backward && a->bias_tiles_bwd) {
    b32 = static_cast<float*>(a->bias_tiles_bwd);          // prepared by the forward: nothing to do here
  } else if (prep) {
    hipError_t e = launch_bias_prep(a->bias, a->bias_dtype, a->bias_stride[0], a->bias_stride[1], a->bias_stride[2],
                                    a->bias_stride[3], b32, a->B, a->H, a->S, 1.0f / a->scale, backward, stream,
                                    backward ? nullptr : static_cast<float*>(a->bias_tiles_bwd));
    if (e != hipSuccess) return (int)e;
  }
  p.bias = b32;
  p.bias_sb = (int64_t)a->H * pl.bias_nt * pl.bias_nt * 1024;
  p.bias_sh = (int64_t)pl.bias_nt * pl.bias_nt * 1024;
  p.bias_nt = pl.bias_nt;
  return 0;
}

}  // namespace

extern "C" int mf_version(void) { return 101; }
extern "C" const char* mf_last_error(void) { return last_error_buf(); }

extern "C" uint64_t mf_evoattn_fwd_workspace_bytes(const mf_evoattn_args* a) {
  if (!a || a->B <= 0 || a->N <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0) return 0;
  return make_plan(a, false).total;
}
extern "C" uint64_t mf_evoattn_bias_tiles_bytes(const mf_evoattn_args* a) {
  if (!a || a->B <= 0 || a->S <= 0 || a->H <= 0) return 0;
  const uint64_t nt = ((uint64_t)a->S + 31) / 32;
  return align256((uint64_t)a->B * a->H * nt * nt * 4096);
}
namespace {
// The memory-lean order keeps the bias gradient's partial sums in the dq buffer: it must be one contiguous
// [B, N, S, H, D] array and large enough.
bool lean_ok(const mf_evoattn_args* a, const Plan& pl) {
  if (!a->dbias || !a->dq) return false;
  const int64_t D = a->D, H = a->H, S = a->S, N = a->N;
  if (a->dq_stride[3] != D || a->dq_stride[2] != H * D || a->dq_stride[1] != S * H * D || a->dq_stride[0] != N * S * H * D)
    return false;
  return pl.part_bytes <= (uint64_t)a->B * N * S * H * D * dtype_size(a->dtype);
}
}  // namespace
extern "C" int mf_evoattn_bwd_lean_ok(const mf_evoattn_args* a) {
  if (!a || a->B <= 0 || a->N <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0 || dtype_size(a->dtype) == 0) return 0;
  return lean_ok(a, make_plan(a, true)) ? 1 : 0;
}
extern "C" uint64_t mf_evoattn_bwd_workspace_bytes(const mf_evoattn_args* a) {
  if (!a || a->B <= 0 || a->N <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0) return 0;
  return make_plan(a, true).total;
}

namespace {

// Forward with the workspace at `ws` (already checked to be large enough and aligned).
int forward_with_workspace(const mf_evoattn_args* a, const Plan& pl, void* ws) {
  mf_evoattn_args b = *a;
  b.workspace = ws;
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  EvoParams p;
  int rc = fill_params(&b, pl, p, stream, true, false);
  if (rc) return rc;
  return (int)launch_evo_fwd(p, stream);
}

}  // namespace

extern "C" int mf_evoattn_fwd(const mf_evoattn_args* a) {
  int rc = check_common(a);
  if (rc) return rc;
  const Plan pl = make_plan(a, false);
  if (!a->workspace || a->workspace_bytes < pl.total)
    return fail(MF_ERR_WORKSPACE, "forward needs %llu workspace bytes, got %llu", (unsigned long long)pl.total,
                (unsigned long long)(a->workspace ? a->workspace_bytes : 0));
  if (!aligned16(a->workspace)) return fail(MF_ERR_ALIGN, "workspace is not 16-byte aligned");
  return forward_with_workspace(a, pl, a->workspace);
}

// ---- forward without any allocation ---------------------------------------------------------------
// The forward's only scratch memory is the tiled fp32 copy of the pair bias.  For callers that can neither
// allocate nor bring a workspace it lives in a fixed device array of this library; every GPU the library
// runs on holds its own copy of the array (at its own address) until the process ends.
namespace {

__device__ __align__(256) unsigned char scratch[MF_EVOATTN_NOALLOC_MAX_WORKSPACE];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_addr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.  The array's name is only
// a host-side handle: kernels and memory calls must be given this address.
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return fail(MF_ERR_SHAPE, "device ordinal %d not supported", dev);
  void* ptr = g_scratch_addr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return fail(MF_ERR_NULL, "no device address for the scratch array");
    g_scratch_addr[dev].store(ptr, std::memory_order_release);   // every thread finds the same address
  }
  *out = ptr;
  return 0;
}

}  // namespace

extern "C" int mf_evoattn_fwd_noalloc(const mf_evoattn_args* a) {
  int rc = check_common(a);
  if (rc) return rc;
  const Plan pl = make_plan(a, false);
  if (pl.total > MF_EVOATTN_NOALLOC_MAX_WORKSPACE)
    return fail(MF_ERR_WORKSPACE, "forward needs %llu scratch bytes, the built-in array holds %llu (B*H*ceil(S/32)^2 <= %llu)",
                (unsigned long long)pl.total, (unsigned long long)MF_EVOATTN_NOALLOC_MAX_WORKSPACE,
                (unsigned long long)(MF_EVOATTN_NOALLOC_MAX_WORKSPACE / 4096));
  void* ws = nullptr;
  rc = scratch_address(&ws);
  if (rc) return rc;
  return forward_with_workspace(a, pl, ws);
}

extern "C" int mf_evoattn_bwd(const mf_evoattn_args* a) {
  int rc = check_common(a);
  if (rc) return rc;
  const int es = dtype_size(a->dtype);
  if ((rc = check_tensor("dO", a->dO, a->do_stride, es))) return rc;
  if ((rc = check_tensor("dq", a->dq, a->dq_stride, es))) return rc;
  if ((rc = check_tensor("dk", a->dk, a->dk_stride, es))) return rc;
  if ((rc = check_tensor("dv", a->dv, a->dv_stride, es))) return rc;
  if (a->dbias && !aligned16(a->dbias)) return fail(MF_ERR_ALIGN, "dbias is not 16-byte aligned");
  if (a->phases < 0 || a->phases > (MF_EVO_BWD_DQKV | MF_EVO_BWD_DBIAS | MF_EVO_BWD_PREP | MF_EVO_BWD_LEAN))
    return fail(MF_ERR_SHAPE, "phases %d unknown", a->phases);
  const Plan pl = make_plan(a, true);
  const bool lean = (a->phases & MF_EVO_BWD_LEAN) != 0;
  if (lean && !lean_ok(a, pl))
    return fail(MF_ERR_SHAPE, "MF_EVO_BWD_LEAN needs dbias, a contiguous dq and a dq buffer of at least %llu bytes "
                "(see mf_evoattn_bwd_lean_ok)", (unsigned long long)pl.part_bytes);
  if (!a->workspace || a->workspace_bytes < pl.total)
    return fail(MF_ERR_WORKSPACE, "backward needs %llu workspace bytes, got %llu", (unsigned long long)pl.total,
                (unsigned long long)(a->workspace ? a->workspace_bytes : 0));
  if (!aligned16(a->workspace)) return fail(MF_ERR_ALIGN, "workspace is not 16-byte aligned");
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  const int which = a->phases & ~MF_EVO_BWD_LEAN;
  const int phases = which == 0 ? (MF_EVO_BWD_PREP | MF_EVO_BWD_DQKV | MF_EVO_BWD_DBIAS) : which;
  EvoParams p;
  rc = fill_params(a, pl, p, stream, (phases & MF_EVO_BWD_PREP) != 0, true);
  if (rc) return rc;
  unsigned char* ws = static_cast<unsigned char*>(a->workspace);
  p.dO = tens(a->dO, a->do_stride);
  p.dq = tens(a->dq, a->dq_stride); p.dk = tens(a->dk, a->dk_stride); p.dv = tens(a->dv, a->dv_stride);
  p.delta = reinterpret_cast<float*>(ws + pl.off_delta);
  p.dbias = a->dbias;
  p.n_chunks = pl.n_chunks;
#ifdef MF_TIMELINE
  { const char* e = getenv("MF_TL_PTR"); p.tl = e ? reinterpret_cast<unsigned*>(strtoull(e, nullptr, 16)) : nullptr;
    const char* f = getenv("MF_TL_BLOCK"); p.tl_block = f ? atoi(f) : 0; }
#endif
  p.rows_per_chunk = pl.rows_per_chunk;
  p.dbias_part = pl.n_chunks > 1 ? reinterpret_cast<float*>(lean ? a->dq : ws + pl.off_part) : nullptr;
  p.dq_scratch = pl.dq_scratch_bytes ? reinterpret_cast<float*>(ws + pl.off_part) : nullptr;
  hipError_t e = hipSuccess;
  if (lean && (phases & MF_EVO_BWD_DBIAS)) {      // bias gradient first: its partial sums are in the dq buffer
    e = launch_evo_delta(p, stream);
    if (e != hipSuccess) return (int)e;
    e = launch_evo_bwd_dbias(p, stream);
    if (e != hipSuccess) return (int)e;
  }
  if (phases & MF_EVO_BWD_DQKV) {
    e = launch_evo_bwd_dqkv(p, stream);
    if (e != hipSuccess) return (int)e;
  }
  if (!lean && (phases & MF_EVO_BWD_DBIAS) && a->dbias) e = launch_evo_bwd_dbias(p, stream);
  return (int)e;
}
