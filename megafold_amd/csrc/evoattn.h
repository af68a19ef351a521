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
  // Pair bias DIVIDED BY scale, fp32, zero padded to whole 32 x 32 tiles and stored tile by tile in the
  // order the consuming lanes hold it (built in the workspace by launch_bias_prep), so that a tile is
  // four perfectly coalesced 1 KiB loads and can be used directly as the C operand of the score MFMA.
  // With nt = ceil(S / 32), l = 32 g + x the lane and c4 = 0..3 the load:
  //   forward layout   tile (qt, jt) at ((qt nt + jt) 1024), float4 (c4 64 + l) =
  //                    bias[32 qt + x][32 jt + 16 g + 4 c4 + 0..3]          (lane = query, registers = keys)
  //   backward layout  tile (jt, it) at ((jt nt + it) 1024), float4 (c4 64 + l) =
  //                    bias[32 it + 16 g + 4 c4 + 0..3][32 jt + x]          (lane = key, registers = queries)
  // bias_sb / bias_sh are the element strides of the batch and head dimensions.
  const float* bias;
  int64_t bias_sb, bias_sh;
  int bias_nt;
  // Additive key mask [B, N, S] in its own dtype (MF_BOOL: keep-mask, true -> 0, false -> -inf).
  const void* mask;
  int mask_dtype;
  int64_t mask_sb, mask_sn, mask_sj;
  float* lse;      // [B, N, H, S] fp32, natural-log logsumexp of the masked, biased logits
  // backward only
  EvoTensor dO, dq, dk, dv;
  float* delta;    // [B, N, H, S] fp32 rowsum(dO * O)
  float* dbias;    // [B, H, S, S] fp32 or nullptr
  float* dbias_part;  // [n_chunks - 1, B, H, S, S] fp32 partial sums of the chunks 1.. (chunk 0 writes dbias; nullptr when n_chunks == 1)
  float* dq_scratch;  // fp32 dQ of the sequences the persistent dQ/dK/dV kernel walks in several passes: one
                      // [ceil(S/32) * 32, 32] array per work-group (evo_bwd_dqkv_pw_scratch_bytes), else nullptr
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
hipError_t launch_evo_delta(const EvoParams& p, hipStream_t stream);   // p.delta = rowsum(dO * O) by its own kernel
// Bias-gradient kernel that streams its rows through an LDS ring with direct loads (16-bit, D = 32, paired heads;
// evoattn_bwd_dbias_ring.hip): whether it handles the problem, and its launcher (same grid and chunking as
// the paired-head form of evo_bwd_dbias_kernel; the caller sums the partial buffers).
bool evo_bwd_dbias_ring_supported(const EvoParams& p);
hipError_t launch_evo_bwd_dbias_ring(const EvoParams& p, hipStream_t stream);
// Persistent form of the dQ/dK/dV kernel (16-bit element types, D <= 32; evoattn_bwd_pw.hip): whether it
// handles the problem, and its launcher (num_cu = compute units of the device).
// Compute units of the current device (256 when no device can be queried).
int evo_num_cu();
bool evo_bwd_dqkv_pw_supported(const EvoParams& p);
// Bytes of EvoParams::dq_scratch the persistent kernel needs for this shape (0: one pass, or not its shape).
uint64_t evo_bwd_dqkv_pw_scratch_bytes(int dtype, int S, int D, int num_cu);
hipError_t launch_evo_bwd_dqkv_pw(const EvoParams& p, int num_cu, hipStream_t stream);
// bias (any float dtype, any strides) * mult -> the tiled fp32 copy described at EvoParams::bias;
// `backward_layout` selects which of the two orders is written.
hipError_t launch_bias_prep(const void* src, int dtype, int64_t sb, int64_t sh, int64_t si, int64_t sj, float* dst,
                            int B, int H, int S, float mult, bool backward_layout, hipStream_t stream,
                            float* dst_bwd = nullptr);   // dst_bwd: the backward's order too, in the same launch

// Number of rows of N one work-group of the bias-gradient kernel walks over, chosen so the grid
// fills the device while the partial-sum workspace stays small.
int evo_dbias_chunks(int B, int N, int S, int H, int D, int dtype);

static inline int round_up(int a, int b) { return (a + b - 1) / b * b; }

}  // namespace mf
