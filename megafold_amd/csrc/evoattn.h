// Parameter blocks and launch entry points of the pair-biased, key-masked attention kernels.
// Replaces the Triton kernels of the reference: megafold/model/FusedEvoAttention/evoattention.py
// (_attn_fwd :122-261, _attn_bwd_preprocess :272-301, _attn_bwd_dk_dv :514-686, _attn_bwd_dq :325-490).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mf {

// Tensors are addressed in the API layout [B, N, S, H, D] (D contiguous) through four element
// strides (b, n, s, h), so views of a fused projection output can be consumed without copies.
struct EvoTensor {
  void* ptr;
  int64_t sb, sn, ss, sh;
};

struct EvoParams {
  int B, N, S, H, D;
  int dtype;       // MF_F32 / MF_F16 / MF_BF16: element type of q, k, v, o, dO, dq, dk, dv
  float scale;     // softmax scale, D^-0.5 in the reference (evoattention.py:705)
  EvoTensor q, k, v, o;
  // Pair bias DIVIDED BY scale as fp32 [B, H, Sr, bias_ld] with Sr = round_up(S, 32) rows and
  // bias_ld = round_up(S, 64) columns, zero padded (built in the workspace by launch_bias_prep), so
  // the kernels read it without bounds checks; row (b, h, i) starts at
  // bias + b*bias_sb + h*bias_sh + i*bias_ld.
  const float* bias;
  int64_t bias_sb, bias_sh, bias_ld;
  // Additive key mask [B, N, S] in its own dtype (MF_BOOL: keep-mask, true -> 0, false -> -inf).
  const void* mask;
  int mask_dtype;
  int64_t mask_sb, mask_sn, mask_sj;
  float* lse;      // [B, N, H, S] fp32, natural-log logsumexp of the masked, biased logits
  // backward only
  EvoTensor dO, dq, dk, dv;
  float* delta;    // [B, N, H, S] fp32 rowsum(dO * O)
  float* dbias;    // [B, H, S, S] fp32 or nullptr
  float* dbias_part;  // [n_chunks, B, H, S, S] fp32 partial sums (nullptr when n_chunks == 1)
#ifdef MF_TIMELINE
  unsigned* tl;    // development aid: cycle stamps of one work-group (see MF_TL in common.h)
  int tl_block;
#endif
  int n_chunks;    // number of N-chunks the bias-gradient kernel splits the rows into
  int rows_per_chunk;
};

// All launchers return hipSuccess or the launch error.  They never allocate or synchronise.
hipError_t launch_evo_fwd(const EvoParams& p, hipStream_t stream);
hipError_t launch_evo_bwd_dqkv(const EvoParams& p, hipStream_t stream);
hipError_t launch_evo_bwd_dbias(const EvoParams& p, hipStream_t stream);
// bias (any float dtype, any strides) * mult -> fp32 [B, H, Sr, ld], zero padded for i >= S or j >= S.
hipError_t launch_bias_prep(const void* src, int dtype, int64_t sb, int64_t sh, int64_t si, int64_t sj, float* dst,
                            int B, int H, int S, int Sr, int ld, float mult, hipStream_t stream);

// Number of rows of N one work-group of the bias-gradient kernel walks over, chosen so the grid
// fills the device while the partial-sum workspace stays small.
int evo_dbias_chunks(int B, int N, int S, int H, int D, int dtype);

static inline int round_up(int a, int b) { return (a + b - 1) / b * b; }

}  // namespace mf
