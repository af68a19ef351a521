/*
 * megafold_amd — C ABI of the MI355X (gfx950) kernels that replace MegaFold's three fused
 * training kernels.  Plain pointers and sizes only; every pointer that names tensor data is a
 * DEVICE pointer, every stride is in ELEMENTS.  Nothing here allocates, frees or synchronises:
 * outputs and workspaces are caller-owned, work is enqueued on the caller's stream (a hipStream_t
 * passed as void*; NULL = the default stream).
 *
 * Return value of every int function: 0 = enqueued; < 0 = argument rejected before anything was
 * launched (MF_ERR_*, text in mf_last_error()); > 0 = the hipError_t a launch returned.
 *
 * Reference interfaces replaced (paths relative to the MegaFold repository):
 *   mf_evoattn_fwd        EvoformerAttention.forward   megafold/model/FusedEvoAttention/evoattention.py:688-779
 *   mf_evoattn_bwd        EvoformerAttention.backward  megafold/model/FusedEvoAttention/evoattention.py:782-903
 *   mf_lnlinear_fwd       layernorm_linear_forward     megafold/model/FusedLayernormLinear/fused_layernorm_linear.py:351-405
 *   mf_lnlinear_bwd       layernorm_linear_backward    megafold/model/FusedLayernormLinear/fused_layernorm_linear.py:408-474
 *   mf_swiglu_fwd / _bwd  swiglu_forward / _backward   megafold/model/FusedTransition/fused_transition.py:55-93
 *   mf_sigmoid_gate_fwd / _bwd
 *                         out * gates.sigmoid() of Attention.forward and its autograd backward
 *                                                      megafold/model/attention.py:199-203
 *   mf_trimul_pack_fwd / _bwd, mf_channels_last_to_first / _first_to_last
 *                         glu, chunk, mask and the operand layouts of the einsum in TriangleMultiplication.forward
 *                                                      megafold/model/megafold.py:474-483
 *   mf_permute_0213       the layout of einsum(a, b, "b s i d, b s j e -> b i j d e") of OuterProductMean.forward
 *                                                      megafold/model/megafold.py:795, 807, 812
 *   mf_lnlinear_* with act = MF_ACT_SWIGLU
 *                         LayernormLinear + FusedSwiGLU of FusedTransition.ff[0:2]
 *                                                      megafold/model/FusedTransition/fused_transition.py:128-131
 */
#ifndef MEGAFOLD_AMD_H
#define MEGAFOLD_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types */
#define MF_DTYPE_F32 0
#define MF_DTYPE_F16 1
#define MF_DTYPE_BF16 2
#define MF_DTYPE_BOOL 3 /* 1 byte per element; only for the attention key mask (true = keep) */

/* argument errors */
#define MF_ERR_NULL (-1)      /* required pointer is NULL */
#define MF_ERR_SHAPE (-2)     /* non-positive or unsupported dimension */
#define MF_ERR_DTYPE (-3)     /* unknown / unsupported element type */
#define MF_ERR_STRIDE (-4)    /* stride not supported (alignment) */
#define MF_ERR_ALIGN (-5)     /* pointer not 16-byte aligned */
#define MF_ERR_WORKSPACE (-6) /* workspace missing or too small */

int mf_version(void);
/* Text of the last argument error on the calling thread ("" if none). */
const char* mf_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * Pair-biased, key-masked attention ("EvoAttention").
 *   q, k, v, o, dO, dq, dk, dv : [B, N, S, H, D], element type `dtype`, D contiguous;
 *                                *_stride = element strides of the (B, N, S, H) axes.
 *   bias  : [B, 1, H, S, S] of bias_dtype, bias_stride = strides of (B, H, S_query, S_key).
 *   mask  : [B, N, 1, 1, S] of mask_dtype, ADDED to the logits (0 / -1e9 / -inf ...);
 *           mask_stride = strides of (B, N, S_key); stride 0 broadcasts.  MF_DTYPE_BOOL is a
 *           keep-mask: true -> 0, false -> -inf.
 *   lse   : [B, N, H, S] fp32, written by fwd, read by bwd.
 *   dbias : [B, H, S, S] fp32 contiguous, written by bwd; NULL = the bias needs no gradient.
 * Supported: D multiple of 8, D <= 64; S <= MF_EVOATTN_MAX_S; dtype f32 / f16 / bf16; strides of
 * q..dv multiples of 16 bytes; pointers 16-byte aligned.  Anything else: MF_ERR_SHAPE / _DTYPE / _STRIDE with a
 * message (mf_last_error), before anything is launched.
 * A query row whose keys are all masked with -inf yields o = 0, lse = -inf and zero gradients.
 * ---------------------------------------------------------------------------------------------- */
/* Backward phases.  MF_EVO_BWD_PREP copies the pair bias into the workspace (scaled, padded, fp32);
 * MF_EVO_BWD_DQKV needs that copy, writes dq, dk, dv and leaves rowsum(dO * o) in the workspace;
 * MF_EVO_BWD_DBIAS needs both and writes dbias.  A call with a subset of the phases must therefore
 * follow calls for the earlier ones on the same stream with the same workspace.  phases = 0 runs
 * all of them (DBIAS only when dbias != NULL).
 * The workspace size depends on the shape, on whether dbias is requested and on the number of compute units of
 * the CURRENT device: query it with the arguments of the call and with the device of the call current. */
#define MF_EVOATTN_MAX_S 16384
#define MF_EVO_BWD_DQKV 1
#define MF_EVO_BWD_DBIAS 2
#define MF_EVO_BWD_PREP 4
/* Modifier bit: memory-lean order.  The bias gradient runs BEFORE dq, dk, dv: rowsum(dO * o) comes from a kernel of
 * its own and the partial sums of the bias gradient live in the dq buffer, which nothing has written yet, instead of
 * in the workspace (smaller workspace: query it with this bit set).  Costs one more pass over dO and o.  Needs
 * dbias != NULL, a contiguous dq ([B, N, S, H, D]) and a dq buffer at least as large as the partial sums
 * (mf_evoattn_bwd_lean_ok reports both; MF_ERR_SHAPE otherwise).  With split phases the order of the calls is PREP,
 * DBIAS, DQKV, each with this bit. */
#define MF_EVO_BWD_LEAN 8

typedef struct mf_evoattn_args {
  int32_t B, N, S, H, D;
  int32_t dtype, bias_dtype, mask_dtype;
  float scale; /* softmax scale; the reference uses D^-0.5 */
  int32_t phases; /* backward only: 0 = everything; else a mask of MF_EVO_BWD_* (see below) */
  const void *q, *k, *v;
  const void* bias;
  const void* mask;
  void* o;
  float* lse;
  int64_t q_stride[4], k_stride[4], v_stride[4], o_stride[4];
  int64_t bias_stride[4];
  int64_t mask_stride[3];
  /* backward only */
  const void* dO;
  void *dq, *dk, *dv;
  float* dbias;
  int64_t do_stride[4], dq_stride[4], dk_stride[4], dv_stride[4];
  /* scratch */
  void* workspace;
  uint64_t workspace_bytes;
  void* stream;
  /* optional, NULL = unused: mf_evoattn_bias_tiles_bytes() bytes, 16-byte aligned.  The forward then also leaves
   * the pair bias in the tiled fp32 order the backward reads (one launch prepares both orders); a backward
   * call given the same buffer reads it instead of preparing its own copy, needs a smaller workspace and no
   * MF_EVO_BWD_PREP phase.  The buffer is an activation the caller keeps between the two calls (the reference
   * keeps the bias itself, evoattention.py:777); scale, shape and bias must be those of the forward call. */
  void* bias_tiles_bwd;
} mf_evoattn_args;

uint64_t mf_evoattn_fwd_workspace_bytes(const mf_evoattn_args* a);
uint64_t mf_evoattn_bwd_workspace_bytes(const mf_evoattn_args* a);
uint64_t mf_evoattn_bias_tiles_bytes(const mf_evoattn_args* a);
int mf_evoattn_bwd_lean_ok(const mf_evoattn_args* a); /* 1 if MF_EVO_BWD_LEAN can be used with these arguments */
int mf_evoattn_fwd(const mf_evoattn_args* a);
int mf_evoattn_bwd(const mf_evoattn_args* a);

/* mf_evoattn_fwd for callers that can neither allocate nor provide a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * `workspace` / `workspace_bytes` of the arguments are ignored: the scratch memory of the forward (the tiled
 * fp32 copy of the pair bias) is a fixed device array inside the library, MF_EVOATTN_NOALLOC_MAX_WORKSPACE
 * bytes on every GPU the library is used on; a problem that needs more (B * H * ceil(S/32)^2 > 4096, e.g.
 * S > 1024 at B = 1, H = 4) is rejected with MF_ERR_WORKSPACE.  The call allocates and frees nothing.  All
 * calls on one GPU share the array, so calls that overlap on one GPU (two streams, two threads) race; calls
 * on one stream are ordered.  Results are identical to mf_evoattn_fwd. */
#define MF_EVOATTN_NOALLOC_MAX_WORKSPACE (16u << 20)
int mf_evoattn_fwd_noalloc(const mf_evoattn_args* a);

/* ------------------------------------------------------------------------------------------------
 * LayerNorm -> Linear:  out = LayerNorm(x; gamma, beta, eps) @ W (+ b)
 *   x     : [M, K] contiguous, element type `dtype`
 *   gamma : [K], beta : [K] or NULL, W : [K, N] contiguous (the reference's `linear_weight`,
 *           i.e. nn.Linear.weight transposed), b : [N] or NULL; all of element type `dtype`
 *   out   : [M, N] contiguous; mean, rstd : [M] fp32 (saved for backward)
 * Backward: dout [M, N] -> dx [M, K] (dtype); dW [K, N], db [N] (may be NULL), dgamma [K],
 * dbeta [K] (may be NULL) are fp32.
 * With act == MF_ACT_SWIGLU (N even): out and dout are [M, N/2] and
 *   out = silu(u[:, N/2:]) * u[:, :N/2]   with u = LayerNorm(x) @ W   (b must be NULL);
 * the backward recomputes u, nothing of shape [M, N] is saved.
 * Supported: K a multiple of 8 with rows of at most 512 bytes (K <= 256 for f16 / bf16, K <= 128 for f32);
 * N a multiple of 8 (16 with MF_ACT_SWIGLU).
 * ---------------------------------------------------------------------------------------------- */
#define MF_ACT_NONE 0
#define MF_ACT_SWIGLU 1

typedef struct mf_lnlinear_args {
  int64_t M;
  int32_t K, N;
  int32_t dtype;
  int32_t act;
  float eps;
  int32_t param_grad_dtype; /* backward: 0 = dW, db, dgamma, dbeta are float arrays; 1 = arrays of x's dtype (the
                               reference returns them cast to x's dtype, fused_layernorm_linear.py:470-472) */
  const void* x;
  const void* gamma;
  const void* beta;
  const void* W;
  const void* b;
  void* out;
  float* mean;
  float* rstd;
  /* backward only */
  const void* dout;
  void* dx;
  const void* dx_add; /* optional [M, K] of x's dtype, added to dx before its single rounding: the gradient that
                         reaches x around the operator when the caller computes x + f(x).  Only where
                         mf_lnlinear_bwd_takes_dx_add() says so; NULL otherwise. */
  void* dW;      /* [K, N] */
  void* db;      /* [N] or NULL */
  void* dgamma;  /* [K] */
  void* dbeta;   /* [K] or NULL */
  /* scratch */
  void* workspace;
  uint64_t workspace_bytes;
  void* stream;
} mf_lnlinear_args;

uint64_t mf_lnlinear_fwd_workspace_bytes(const mf_lnlinear_args* a);
uint64_t mf_lnlinear_bwd_workspace_bytes(const mf_lnlinear_args* a);
int mf_lnlinear_fwd(const mf_lnlinear_args* a);
int mf_lnlinear_bwd(const mf_lnlinear_args* a);
/* 1 if the backward of this dtype / K / N adds dx_add inside its dx kernel (16-bit types, 64 < K <= 128,
 * 64 <= N <= 1024), else 0: such callers add the skip gradient themselves.  No counterpart in the reference, whose
 * residual adds are separate PyTorch operations (megafold/model/megafold.py:742-747). */
int mf_lnlinear_bwd_takes_dx_add(const mf_lnlinear_args* a);

/* ------------------------------------------------------------------------------------------------
 * SwiGLU on its own (FusedTransition with include_ln=False or use_layernormlinear=False):
 *   x [M, 2*Dh] contiguous -> y [M, Dh],  y = silu(x[:, Dh:]) * x[:, :Dh]
 *   backward: dy [M, Dh], x -> dx [M, 2*Dh] = [dy * silu(g), dy * a * (sig(g) + silu(g)(1 - sig(g)))]
 * dx may alias x (the reference overwrites its saved input, fused_transition.py:49-52).
 * ---------------------------------------------------------------------------------------------- */
int mf_swiglu_fwd(const void* x, void* y, int64_t M, int32_t Dh, int32_t dtype, void* stream);
int mf_swiglu_bwd(const void* dy, const void* x, void* dx, int64_t M, int32_t Dh, int32_t dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Sigmoid output gate of the attention block (megafold/model/attention.py:199-203):
 *   forward : a = o * sigmoid(g)  (+ res, if given: the block's residual x + f(x), megafold.py:742-743, summed
 *             in fp32 and rounded once)
 *   backward: d_o = da * s,  dg = da * o * s * (1 - s),  a = o * s  (s = sigmoid(g); a may be NULL)
 * Every operand is a matrix of M rows and C columns (C a multiple of 8) with its own row stride in
 * elements (>= C, 16-byte multiples), so that g / dg can be column slices of the wider matrix the fused
 * projections produce.  Outputs must not overlap inputs other than element-for-element.
 * ---------------------------------------------------------------------------------------------- */
typedef struct {
  int64_t M;
  int32_t C;
  int32_t dtype;
  const void* o;   int64_t ldo;   /* attention output, heads merged */
  const void* g;   int64_t ldg;   /* gate pre-activations */
  void* a;         int64_t lda;   /* o * sigmoid(g): output of forward, optional output of backward */
  const void* res; int64_t ldres; /* forward only, optional: added to a */
  /* backward only */
  const void* da;  int64_t ldda;  /* gradient of a */
  void* d_o;       int64_t lddo;  /* gradient of o */
  void* dg;        int64_t lddg;  /* gradient of g */
  void* stream;
} mf_gate_args;

int mf_sigmoid_gate_fwd(const mf_gate_args* a);
int mf_sigmoid_gate_bwd(const mf_gate_args* a);

/* ------------------------------------------------------------------------------------------------
 * Layout moves of the triangle-multiplication block (megafold/model/megafold.py:474-483).  The
 * contraction  out[i,j,c] = sum_k left[i,k,c] * right[j,k,c]  ("outgoing";  "incoming" is
 * sum_k left[k,j,c] * right[k,i,c])  is a batch of dh independent n x n x n products, so its operands are
 * moved from channel-last rows to channel-first matrices  p[which][b][c][o][q]  with row stride and row
 * count np (a multiple of 8, >= n; positions q >= n of written rows are zero, rows o >= n are not
 * touched).  With  out_c = p[0][b][c] * p[1][b][c]^T  as the batched product:
 *   outgoing: transposed = 0, swap = 0   p[0][c][i][k] = left[i,k,c],  p[1][c][j][k] = right[j,k,c]
 *   incoming: transposed = 1, swap = 1   p[0][c][i][k] = right[k,i,c], p[1][c][j][k] = left[k,j,c]
 * i.e. the channel-last row of position (o, q) is row o*n + q (transposed = 0) or q*n + o (transposed = 1),
 * and swap exchanges which of the two channel halves lands in p[0].
 *
 *   mf_trimul_pack_fwd        y [B*n*n, ldy >= 4*dh]: columns [0,2dh) values, [2dh,4dh) gates;
 *                             (left | right) = y[:, :2dh] * sigmoid(y[:, 2dh:4dh]) * mask[b,o] * mask[b,q] -> p
 *   mf_trimul_pack_bwd        p holds the gradients of the two matrices; writes the gradients of the value
 *                             and gate columns into dy [B*n*n, lddy >= 4*dh] (y as in forward)
 *   mf_channels_last_to_first y [B*n*n, ldy >= dh] -> p[0] (one matrix set; mask, if given, is applied)
 *   mf_channels_first_to_last p[0] -> dy [B*n*n, lddy >= dh]
 * dh must make the moved row 64, 128 or 256 channels wide (2*dh for the pack forms, dh for the plain ones).
 * mask: [B, n] bytes (non-zero = keep) or NULL.
 * ---------------------------------------------------------------------------------------------- */
typedef struct {
  int32_t B, n, np, dh;
  int32_t dtype;
  int32_t transposed;
  int32_t swap;
  int32_t reserved0;
  const void* y;  int64_t ldy;
  void* dy;       int64_t lddy;
  const void* mask;
  void* p;
  void* stream;
} mf_trimul_args;

int mf_trimul_pack_fwd(const mf_trimul_args* a);
int mf_trimul_pack_bwd(const mf_trimul_args* a);
int mf_channels_last_to_first(const mf_trimul_args* a);
int mf_channels_first_to_last(const mf_trimul_args* a);

/* ------------------------------------------------------------------------------------------------
 * MSA pair-weighted averaging (Algorithm 10), the contraction part of MSAPairWeightedAveraging.forward
 * (megafold/model/megafold.py:868-902): the weights  w[b,h,i,:] = softmax_j(logits[b,i,j,h] + mask[b,j])  do not
 * depend on the MSA row, so they are formed once and applied to every row:
 *   y[b,s,i,h,:] = (sum_j w[b,h,i,j] x[b,s,j,h,:]) * sigmoid(g[b,s,i,h,:])
 * 16-bit element types, H = 8 heads of D = 32 channels.
 *   logits, dlogits : rows [B*N*N] of H elements, ld_* elements apart (a multiple of 8)
 *   mask            : [B, N] bytes, non-zero = keep, or NULL; a row whose keys are all masked gets zero weights
 *   w               : [B, H, NP, NP], NP = N rounded up to 32, zero outside [N, N]
 *   x, g, y, dy     : rows [B*S*N] of H*D elements (channels of head h at 32 h), ld* elements apart (multiples
 *                     of 8, >= 256): column slices of wider matrices are fine
 *   dw_part         : [n_chunks, B, H, NP, NP] fp32, n_chunks = mf_pwa_dw_chunks(args)
 * mf_pwa_softmax_fwd   logits, mask -> w
 * mf_pwa_apply         w, x (, g) -> y; N <= 384.  With the transposed weights as w and dy as x it computes
 *                      dx[b,s,j,h,:] = sum_i w[b,h,i,j] dy[b,s,i,h,:]
 * mf_pwa_dw            dy, x -> dw_part: partial sums over chunks of the MSA rows of
 *                      dw[b,h,i,j] = sum_{s,d} dy[b,s,i,h,d] x[b,s,j,h,d]
 * mf_pwa_softmax_bwd   w, dw_part -> dlogits = w * (dw - sum_j w dw), dw = the sum of the partial buffers
 * ---------------------------------------------------------------------------------------------- */
typedef struct {
  int32_t B, S, N, H, D;
  int32_t dtype;
  int32_t n_chunks;
  int32_t reserved0;
  const void* logits; int64_t ld_logits;
  const void* mask;
  void* w;
  const void* x;  int64_t ldx;
  const void* g;  int64_t ldg;
  void* y;        int64_t ldy;
  const void* dy; int64_t lddy;
  float* dw_part;
  void* dlogits;  int64_t ld_dlogits;
  void* stream;
} mf_pwa_args;

int mf_pwa_softmax_fwd(const mf_pwa_args* a);
int mf_pwa_apply(const mf_pwa_args* a);
int mf_pwa_dw_chunks(const mf_pwa_args* a);
int mf_pwa_dw(const mf_pwa_args* a);
int mf_pwa_softmax_bwd(const mf_pwa_args* a);

/* ------------------------------------------------------------------------------------------------
 * Outer product mean (Algorithm 9), the contraction part of OuterProductMean.forward
 * (megafold/model/megafold.py:795-823) in one kernel, without the [n, n, dh*dh] tensor:
 *   out[b,i,j,:] = sum_{d,e} w[:, e*32 + d] * (sum_s a[b, i*32 + d, s] * b[b, j*32 + e, s]) + bias
 *   a, b : [B, n*32, 128] (hidden dimension 32; the MSA rows s along the contiguous axis, zero padded to 128;
 *          masks and the division by the number of rows already applied)
 *   w    : [128, 1024]: the projection weight with its two hidden indices exchanged (column e*32 + d holds
 *          the reference's column d*32 + e); bias : [128] or NULL; out : [B, n, n, 128]
 * 16-bit element types.
 * ---------------------------------------------------------------------------------------------- */
int mf_opm_fused_fwd(const void* a, const void* b, const void* w, const void* bias, void* out, int32_t B, int32_t n,
                     int32_t dtype, void* stream);

/* The two operands of mf_opm_fused_fwd from the hidden projection, and the way back for their gradients
 * (megafold/model/megafold.py:788-807: MSA-row mask and the division by the number of rows as row_scale, the pair
 * mask as a position mask on either side):
 *   unpack = 0:  a[b, i*32 + d, s] = hidden[b, s, i, d] * row_scale[b, s] * pos[b, i]   (rounded once)
 *                b[b, i*32 + e, s] = hidden[b, s, i, 32 + e] * pos[b, i];  columns S..127 are written as zero
 *   unpack = 1:  hidden[b, s, i, d] = a[...] * row_scale[b, s] * pos[b, i],  hidden[b, s, i, 32 + e] = b[...] * pos[b, i]
 *   hidden : [B, S, n, ldh >= 64] (ldh = element stride of a position); row_scale : [B, S] float;
 *   pos : [B, n] bytes (0 = masked) or NULL; a, b : [B, n*32, 128]; S <= 128; 16-bit element types. */
int mf_opm_pack(void* hidden, int64_t ldh, const float* row_scale, const void* pos, void* a, void* b, int32_t B, int32_t S,
                int32_t n, int32_t unpack, int32_t dtype, void* stream);

/* Gradient of that projection weight, the outer blocks formed again tile by tile and never stored
 * (autograd of megafold/model/megafold.py:807-812 with respect to to_pairwise_repr.weight):
 *   dwt[e*32 + d, c] = sum_{b,i,j} (sum_s a[b, i*32 + d, s] * b[b, j*32 + e, s]) * dout[b, i, j, c]
 *   a, b as above; dout : [B, n, n, 128] (element type of a); dwt : [1024, 128] float, in the index order of w
 *   transposed; workspace : mf_opm_dw_workspace_bytes(B, n) bytes, 16-byte aligned.  Fixed summation order. */
uint64_t mf_opm_dw_workspace_bytes(int32_t B, int32_t n);
int mf_opm_dw(const void* a, const void* b, const void* dout, float* dwt, void* workspace, uint64_t workspace_bytes,
              int32_t B, int32_t n, int32_t dtype, void* stream);

/* Gradient of one of the two operands, likewise without the [n, n, dh*dh] tensor (autograd of
 * megafold/model/megafold.py:795-812 with respect to a or b):
 *   res[b, o*32 + f, s] = sum_{t,h} (sum_c dout[b, pair(o,t), c] * wt[f*32 + h, c]) * opnd[b, t*32 + h, s]
 *   transposed = 0: pair(o,t) = (o, t): res = da with opnd = b and wt[d*32 + e, c] = W[c, d*32 + e];
 *   transposed = 1: pair(o,t) = (t, o): res = db with opnd = a and wt[e*32 + d, c] = W[c, d*32 + e].
 *   dout : [B, n, n, 128]; wt : [1024, 128]; opnd, res : [B, n*32, 128] (all the element type `dtype`, 16 bits);
 *   workspace : mf_opm_dab_workspace_bytes(B, n) bytes, 16-byte aligned.  Fixed summation order. */
uint64_t mf_opm_dab_workspace_bytes(int32_t B, int32_t n);
int mf_opm_dab(const void* dout, const void* wt, const void* opnd, void* res, void* workspace, uint64_t workspace_bytes,
               int32_t B, int32_t n, int32_t transposed, int32_t dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * y[a][c][b][:] = x[a][b][c][:] for contiguous arrays of rows of `row_bytes` bytes (a multiple of 16, at most
 * 256): the layout move between the [(i d), (j e)] result of OuterProductMean's contraction and the
 * "b i j (d e)" rows its projection reads (megafold/model/megafold.py:795, 807, 812), and the inverse move for
 * the gradient (call it with B and C exchanged).  A <= 65535, B <= 65535 * 32.
 * ---------------------------------------------------------------------------------------------- */
int mf_permute_0213(const void* x, void* y, int64_t A, int64_t B, int64_t C, int32_t row_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MEGAFOLD_AMD_H */
