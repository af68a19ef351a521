// Layout kernels of the triangle-multiplication block and their C-ABI entry points.
// Reference statements being replaced (megafold/model/megafold.py:474-483):
//     left, right = glu(combined[..., :4*dh]).chunk(2, dim=-1);  left, right *= mask
//     out = einsum(left, right, "... i k d, ... j k d -> ... i j d")      ("outgoing"; "incoming" contracts over the first index)
// The contraction is a batch of dh independent n x n x n products, one per channel, while every tensor
// around it is channel-last.  These kernels move between the two layouts with the elementwise work fused
// into the move, so that the products themselves can run as one batched GEMM on row-major matrices:
//     pack   : channel-last rows -> channel-first matrices  P[c][o][q]   (GLU and pair mask applied on the way)
//     unpack : channel-first matrices -> channel-last rows               (GLU backward applied on the way)
// A thread moves an 8 x 8 block (8 channels x 8 consecutive positions of the inner axis) through registers:
// 16-byte accesses on both sides; eight neighbouring lanes cover 128 contiguous bytes of a channel-last row
// when reading and 128 contiguous bytes of a channel-first row when writing (and vice versa).
#include "../../include/megafold_amd.h"
#include "capi_common.h"
#include "common.h"

namespace mf {
namespace {

__device__ __forceinline__ float tm_sigmoid(float g) { return __builtin_amdgcn_rcpf(1.0f + fast_exp2(-g * MF_LOG2E)); }

struct TmParams {
  int B, n, np, C;            // C channels per row move (2*dh for the GLU forms, dh for the plain forms)
  int dh;                     // channels of one operand (channel c < dh is "left", c >= dh is "right")
  int transposed, swap;       // see mf_trimul_args
  const void* y; int64_t ldy; // channel-last source (pack) or GLU input (unpack with GLU backward)
  void* dy; int64_t lddy;     // channel-last destination (unpack)
  const unsigned char* mask;  // [B, n] bool or NULL
  void* p;                    // channel-first matrices [C / dh][B][dh][np][np]
};

// GLU forms: value column c, gate column 2*dh + c of the same row.
template <typename T, bool GLU>
__global__ void __launch_bounds__(256) tm_pack_kernel(const TmParams a) {
  const int CB = a.C / 8;                       // 8-channel blocks: 8 per wavefront
  const int wpc = CB / 8;                       // wavefronts that cover the channels (1, 2 or 4)
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int ib = (l & 7) + 8 * (w / wpc) + (4 / wpc) * 8 * blockIdx.x;     // 8-position block of the inner axis
  const int cb = (l >> 3) + 8 * (w % wpc);
  const int o = blockIdx.y, b = blockIdx.z;
  const int q0 = ib * 8;
  if (q0 >= a.np) return;
  const T* Y = reinterpret_cast<const T*>(a.y);
  T* P = reinterpret_cast<T*>(a.p);
  const int c0 = cb * 8;
  const bool mo = a.mask ? a.mask[b * a.n + o] != 0 : true;
  frag_t<T> in[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int q = q0 + e;
    const int qc = q < a.n ? q : a.n - 1;
    const int64_t row = ((int64_t)b * a.n + (a.transposed ? qc : o)) * a.n + (a.transposed ? o : qc);
    const frag_t<T> v = ld8<T>(Y + row * a.ldy + c0);
    const bool keep = q < a.n && mo && (a.mask ? a.mask[b * a.n + qc] != 0 : true);
    if (GLU) {
      const frag_t<T> g = ld8<T>(Y + row * a.ldy + 2 * a.dh + c0);
      float r[8];
#pragma unroll
      for (int f = 0; f < 8; ++f) r[f] = keep ? (float)v[f] * tm_sigmoid((float)g[f]) : 0.0f;
      in[e] = cvt8<T>(r[0], r[1], r[2], r[3], r[4], r[5], r[6], r[7]);
    } else {
      in[e] = keep ? v : frag_zero<T>();
    }
  }
#pragma unroll
  for (int f = 0; f < 8; ++f) {
    const int c = c0 + f;
    const int which = (c / a.dh) ^ a.swap, d = c % a.dh;
    frag_t<T> out;
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = in[e][f];
    st8<T>(P + ((((int64_t)which * a.B + b) * a.dh + d) * a.np + o) * a.np + q0, out);
  }
}

// Plain form: channel-first -> channel-last.  GLU form: the channel-first values are the gradients of
// (left | right); with the row's value v and gate g of the forward input, the gradients of the value and
// gate columns are  dv = dl * s * m,  dg = dl * v * s * (1 - s) * m  (s = sigmoid(g), m = pair mask).
template <typename T, bool GLU>
__global__ void __launch_bounds__(256) tm_unpack_kernel(const TmParams a) {
  const int CB = a.C / 8;
  const int wpc = CB / 8;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int ib = (l & 7) + 8 * (w / wpc) + (4 / wpc) * 8 * blockIdx.x;
  const int cb = (l >> 3) + 8 * (w % wpc);
  const int o = blockIdx.y, b = blockIdx.z;
  const int q0 = ib * 8;
  if (q0 >= a.n) return;
  const T* P = reinterpret_cast<const T*>(a.p);
  const T* Y = reinterpret_cast<const T*>(a.y);
  T* DY = reinterpret_cast<T*>(a.dy);
  const int c0 = cb * 8;
  const bool mo = a.mask ? a.mask[b * a.n + o] != 0 : true;
  frag_t<T> in[8];
#pragma unroll
  for (int f = 0; f < 8; ++f) {
    const int c = c0 + f;
    const int which = (c / a.dh) ^ a.swap, d = c % a.dh;
    in[f] = ld8<T>(P + ((((int64_t)which * a.B + b) * a.dh + d) * a.np + o) * a.np + q0);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int q = q0 + e;
    if (q < a.n) {
      const int64_t row = ((int64_t)b * a.n + (a.transposed ? q : o)) * a.n + (a.transposed ? o : q);
      frag_t<T> t;
#pragma unroll
      for (int f = 0; f < 8; ++f) t[f] = in[f][e];
      if (GLU) {
        const bool keep = mo && (a.mask ? a.mask[b * a.n + q] != 0 : true);
        const frag_t<T> v = ld8<T>(Y + row * a.ldy + c0);
        const frag_t<T> g = ld8<T>(Y + row * a.ldy + 2 * a.dh + c0);
        float dv[8], dg[8];
#pragma unroll
        for (int f = 0; f < 8; ++f) {
          const float s = tm_sigmoid((float)g[f]);
          const float dl = keep ? (float)t[f] : 0.0f;
          dv[f] = dl * s;
          dg[f] = dl * (float)v[f] * (s * (1.0f - s));
        }
        st8<T>(DY + row * a.lddy + c0, cvt8<T>(dv[0], dv[1], dv[2], dv[3], dv[4], dv[5], dv[6], dv[7]));
        st8<T>(DY + row * a.lddy + 2 * a.dh + c0, cvt8<T>(dg[0], dg[1], dg[2], dg[3], dg[4], dg[5], dg[6], dg[7]));
      } else {
        st8<T>(DY + row * a.lddy + c0, t);
      }
    }
  }
}

int check_tm(const mf_trimul_args* a, bool glu, bool unpack, TmParams& p) {
  clear_error();
  if (!a) return fail(MF_ERR_NULL, "args is NULL");
  if (a->B <= 0 || a->n <= 0 || a->dh <= 0) return fail(MF_ERR_SHAPE, "B, n, dh must be positive (got %d %d %d)", a->B, a->n, a->dh);
  const int C = glu ? 2 * a->dh : a->dh;
  if (C != 64 && C != 128 && C != 256)
    return fail(MF_ERR_SHAPE, "dh=%d unsupported: the moved row must hold 64, 128 or 256 channels", a->dh);
  if (a->np < a->n || a->np % 8 != 0) return fail(MF_ERR_SHAPE, "np=%d must be a multiple of 8 and >= n", a->np);
  if (a->B > 65535 || a->n > 65535) return fail(MF_ERR_SHAPE, "B and n are limited to 65535");
  if (a->dtype != MF_DTYPE_F32 && a->dtype != MF_DTYPE_F16 && a->dtype != MF_DTYPE_BF16)
    return fail(MF_ERR_DTYPE, "dtype %d unsupported", a->dtype);
  const int es = dtype_size(a->dtype), unit = 16 / es;
  const int need = glu ? 4 * a->dh : a->dh;
  if (!a->p) return fail(MF_ERR_NULL, "p is NULL");
  if (!aligned16(a->p)) return fail(MF_ERR_ALIGN, "p is not 16-byte aligned");
  const bool need_y = !unpack || glu;
  if (need_y) {
    if (!a->y) return fail(MF_ERR_NULL, "y is NULL");
    if (!aligned16(a->y)) return fail(MF_ERR_ALIGN, "y is not 16-byte aligned");
    if (a->ldy < need || a->ldy % unit != 0)
      return fail(MF_ERR_STRIDE, "y row stride %lld must be >= %d and a multiple of %d elements", (long long)a->ldy, need, unit);
  }
  if (unpack) {
    if (!a->dy) return fail(MF_ERR_NULL, "dy is NULL");
    if (!aligned16(a->dy)) return fail(MF_ERR_ALIGN, "dy is not 16-byte aligned");
    if (a->lddy < need || a->lddy % unit != 0)
      return fail(MF_ERR_STRIDE, "dy row stride %lld must be >= %d and a multiple of %d elements", (long long)a->lddy, need, unit);
  }
  p = TmParams{a->B, a->n, a->np, C, a->dh, a->transposed ? 1 : 0, (glu && a->swap) ? 1 : 0, a->y, a->ldy, a->dy, a->lddy,
               reinterpret_cast<const unsigned char*>(a->mask), a->p};
  return 0;
}

template <bool GLU, bool UNPACK> int launch_tm(const mf_trimul_args* a) {
  TmParams p;
  int rc = check_tm(a, GLU, UNPACK, p);
  if (rc) return rc;
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  const int per_block = (4 / (p.C / 64)) * 64;              // inner positions one work-group covers
  const int extent = UNPACK ? p.n : p.np;
  const dim3 grid((unsigned)((extent + per_block - 1) / per_block), (unsigned)p.n, (unsigned)p.B);
  switch (a->dtype) {
    case MF_DTYPE_BF16:
      if (UNPACK) hipLaunchKernelGGL((tm_unpack_kernel<bf16_t, GLU>), grid, dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((tm_pack_kernel<bf16_t, GLU>), grid, dim3(256), 0, stream, p);
      break;
    case MF_DTYPE_F16:
      if (UNPACK) hipLaunchKernelGGL((tm_unpack_kernel<f16_t, GLU>), grid, dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((tm_pack_kernel<f16_t, GLU>), grid, dim3(256), 0, stream, p);
      break;
    default:
      if (UNPACK) hipLaunchKernelGGL((tm_unpack_kernel<float, GLU>), grid, dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((tm_pack_kernel<float, GLU>), grid, dim3(256), 0, stream, p);
      break;
  }
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace mf

extern "C" int mf_trimul_pack_fwd(const mf_trimul_args* a) { return mf::launch_tm<true, false>(a); }
extern "C" int mf_trimul_pack_bwd(const mf_trimul_args* a) { return mf::launch_tm<true, true>(a); }
extern "C" int mf_channels_last_to_first(const mf_trimul_args* a) { return mf::launch_tm<false, false>(a); }
extern "C" int mf_channels_first_to_last(const mf_trimul_args* a) { return mf::launch_tm<false, true>(a); }
