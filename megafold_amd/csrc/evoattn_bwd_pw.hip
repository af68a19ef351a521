// dQ, dK, dV of the pair-biased attention backward for the 16-bit element types at D <= 32:
// persistent work-groups, several key tiles per wavefront, software-pipelined over the score tiles.
//
// Same mathematics as the reference kernels _attn_bwd_preprocess, _attn_bwd_dk_dv and _attn_bwd_dq
// (megafold/model/FusedEvoAttention/evoattention.py:272-301, 514-686, 325-490) in ONE pass over the score
// tiles (5 matrix products per tile), organised around what limits this op at D = 32 on gfx950:
//
//  * A 32 x 32 score tile costs 12 MFMAs (390 cycles of the matrix pipe) and about 420 cycles of vector
//    ALU work (exp2, two multiplies, the packed converts).  One tile at a time is a long dependent chain
//    (scores -> exp -> convert -> products), so the loop is a software pipeline over tiles: while the vector
//    ALU turns the scores of tile i into P and dS, the matrix pipe computes the scores of tile i + 1 and
//    the dV / dK / dQ products of tile i - 1.  The interleaving is written out (one MFMA between pairs of
//    score elements) and pinned with scheduling barriers.
//  * A wavefront owns TPW key tiles (K, K^T, V fragments and the dK / dV accumulators stay in registers)
//    and walks over the query tiles.  The query-side operands are read from LDS once per step and used
//    for TPW tiles, the partial dQ of a step is summed over the wavefront's tiles in registers before it
//    goes to the fixed-order LDS reduction: less than half the LDS traffic per tile of a one-tile form.
//  * The register file is used as two halves: the accumulators dK, dV, dQ and the operands that only the
//    matrix pipe reads live in accumulation registers (the products that update them are issued as
//    inline assembly, because the compiler picks ONE register form for all MFMA builtins of a kernel);
//    scores and dP are ordinary vector registers, where the vector ALU reads them without copies.
//  * With four wavefronts of TPW = 3 tiles a work-group covers 384 keys: at S <= 384 every query tile is
//    read once and dQ is written once.  Longer sequences run in passes of 4 * TPW key tiles; the running
//    dQ then stays, in fp32 (no rounding between passes), in an array of the work-group's own in global memory
//    (EvoParams::dq_scratch: one [ceil(S/32) * 32, 32] array per work-group, so its size, and with it the
//    backward's workspace, follows the compute-unit count of the device the launch runs on).
//  * One work-group per compute unit, looping over its share of the (b, n, h) problems: all heads of a
//    row n are handled by the same XCD at the same time, because two heads share every 128-byte line of
//    Q, K, V, dO.
#include "common.h"
#include "evoattn.h"
#include "evoattn_bwd_layout.h"

namespace mf {

template <typename T> struct PwLayout {
  using L = BwdLayout<T, 32>;
  static constexpr int NW = 4;
  static constexpr int KV_BYTES = 32 * L::QSTR * (int)sizeof(T);        // one K or V tile
  // per wavefront: dS tile, two dQ slabs, then the K and V tiles it owns
  static constexpr int wave_bytes(int tpw) { return L::TR_BYTES + 2 * L::SLAB_BYTES + 2 * tpw * KV_BYTES; }
  static constexpr int REC_BYTES = 12 * 32;                             // address records (see AddrRec)
  static size_t smem(int tpw) {
    return (size_t)REC_BYTES + 2 * L::STAGE_ELEMS * sizeof(T) + 128 * 4 + (size_t)NW * wave_bytes(tpw);
  }
};

// Every MFMA of the loop is issued as inline assembly, which fixes both its place in the instruction
// stream and the register file of each operand ("a": accumulation register, "v": vector register):
//   acc_av / acc_aa   c (acc. regs) += A * B with B in vector / accumulation registers
//   zero_av           c (acc. regs)  = A * B (the register keeps its place: c is tied)
//   *_last            followed by enough idle cycles that the next instruction may read the result; the
//                     compiler cannot see into the assembly, so it would not wait by itself
//   v_set / v_zero / v_acc   the same with the result in vector registers (scores and dP, read by the
//                     vector ALU one slot later, after at least two further MFMAs have been issued)
// An operand register written by the vector ALU (a convert, a move between the register files) must not be
// read by the matrix pipe in the next two issue slots, and the compiler does not know that the assembly is
// an MFMA: operands are therefore produced well ahead of their product (the words of P and dS a slot
// earlier, the constant fragments once per pass through to_acc()), and csrc/check_pw_hazards.py verifies
// this on the generated code at build time.
template <typename T> struct AsmMma;
// MF_PRE: two idle issue slots in front of every MFMA.  The register allocator may place a copy of an
// operand (between the two register files, or of a tied accumulator) directly in front of an assembly
// statement, and a register written by the vector ALU must not be read by the matrix pipe in the next two
// slots.
#ifndef MF_PW_NO_PRE_NOP
#define MF_PRE "s_nop 1\n "
#else
#define MF_PRE
#endif
#define MF_ASM_MMA(T, MNEM)                                                                                   \
  template <> struct AsmMma<T> {                                                                              \
    using frag = frag_t<T>;                                                                                   \
    static __device__ __forceinline__ void acc_av(f32x16& c, const frag& a, const frag& b) {                  \
      asm volatile(MF_PRE MNEM " %0, %1, %2, %0" : "+a"(c) : "a"(a), "v"(b));                                        \
    }                                                                                                         \
    static __device__ __forceinline__ void acc_aa(f32x16& c, const frag& a, const frag& b) {                  \
      asm volatile(MF_PRE MNEM " %0, %1, %2, %0" : "+a"(c) : "a"(a), "a"(b));                                        \
    }                                                                                                         \
    static __device__ __forceinline__ void zero_av(f32x16& c, const frag& a, const frag& b) {                 \
      asm volatile(MF_PRE MNEM " %0, %1, %2, 0" : "+a"(c) : "a"(a), "v"(b));                                         \
    }                                                                                                         \
    static __device__ __forceinline__ void acc_av_last(f32x16& c, const frag& a, const frag& b) {             \
      asm volatile(MF_PRE MNEM " %0, %1, %2, %0\n s_nop 15\n s_nop 3" : "+a"(c) : "a"(a), "v"(b));                   \
    }                                                                                                         \
    static __device__ __forceinline__ void v_set(f32x16& d, const frag& a, const frag& b, const f32x16& c) {  \
      asm volatile(MF_PRE MNEM " %0, %1, %2, %3" : "=&v"(d) : "a"(a), "a"(b), "v"(c));                               \
    }                                                                                                         \
    static __device__ __forceinline__ void v_zero(f32x16& d, const frag& a, const frag& b) {                  \
      asm volatile(MF_PRE MNEM " %0, %1, %2, 0" : "=&v"(d) : "a"(a), "a"(b));                                        \
    }                                                                                                         \
    static __device__ __forceinline__ void v_acc(f32x16& c, const frag& a, const frag& b) {                   \
      asm volatile(MF_PRE MNEM " %0, %1, %2, %0" : "+v"(c) : "a"(a), "a"(b));                                        \
    }                                                                                                         \
    static __device__ __forceinline__ void v_acc_last(f32x16& c, const frag& a, const frag& b) {              \
      asm volatile(MF_PRE MNEM " %0, %1, %2, %0\n s_nop 15\n s_nop 3" : "+v"(c) : "a"(a), "a"(b));                   \
    }                                                                                                         \
  };
MF_ASM_MMA(bf16_t, "v_mfma_f32_32x32x16_bf16")
MF_ASM_MMA(f16_t, "v_mfma_f32_32x32x16_f16")
#undef MF_ASM_MMA

// The same fragment held in accumulation registers: one copy here instead of one per use (an operand with
// the "a" constraint whose value lives in vector registers is copied in front of every assembly statement).
template <typename F> __device__ __forceinline__ F to_acc(const F& f) {
  F r;
  asm volatile("" : "=a"(r) : "0"(f));
  return r;
}

// <a, b> of four 16-bit elements held in two words each, accumulated in fp32.
template <typename T> __device__ __forceinline__ float dot4(u32x2 a, u32x2 b) {
  typedef T vec4_t __attribute__((ext_vector_type(4)));
  const vec4_t x = __builtin_bit_cast(vec4_t, a), y = __builtin_bit_cast(vec4_t, b);
  float s = (float)x[0] * (float)y[0];
  s = __builtin_fmaf((float)x[1], (float)y[1], s);
  s = __builtin_fmaf((float)x[2], (float)y[2], s);
  return __builtin_fmaf((float)x[3], (float)y[3], s);
}

template <typename T> __device__ __forceinline__ unsigned pack2(float a, float b) {
  typedef T pair_t __attribute__((ext_vector_type(2)));
  pair_t pr = {(T)a, (T)b};
  return __builtin_bit_cast(unsigned, pr);
}
template <typename T> __device__ __forceinline__ frag_t<T> words_frag(unsigned w0, unsigned w1, unsigned w2, unsigned w3) {
  u32x4 v = {w0, w1, w2, w3};
  return __builtin_bit_cast(frag_t<T>, v);
}

#define MF_FENCE() __builtin_amdgcn_sched_barrier(0)
// development aid (see MF_TL in common.h): stamp k of slot (query tile, key tile) of this wavefront, first pass only
#define MF_TLI(q, t, k) ((pass == 0 ? ((w * 64 + (q)) * TPW + (t)) : 4 * 64 * TPW) * 8 + (k))

// One per-problem address of the kernel: base + ((b * sb + n * sn + h * sh) << shift).  The twelve records sit in
// LDS; lane i of a wavefront evaluates record i, so the addresses of a problem cost three multiply-adds for
// all tensors together instead of a chain of 64-bit scalar multiplies per tensor.
struct __attribute__((aligned(32))) AddrRec {
  unsigned long long base;
  int sb, sn, sh, shift;
};
// A pointer made from an integer is a flat pointer to the compiler (flat loads count on both memory counters);
// going through the global address space keeps the accesses global.
template <typename U> __device__ __forceinline__ U* as_global(unsigned long long a) {
  return (U*)reinterpret_cast<U __attribute__((address_space(1)))*>(a);
}
enum { REC_Q, REC_DO, REC_O, REC_K, REC_V, REC_DQ, REC_DK, REC_DV, REC_LSE, REC_DELTA, REC_MASK, REC_BIAS, REC_COUNT };

// MP: sequences of more than NW * TPW key tiles, walked in several passes per problem (a compile-time variant:
// the one-pass kernel of the common lengths carries none of its code).
template <typename T, int TPW, bool MP>
__global__ void __launch_bounds__(256, 1) evo_bwd_dqkv_pw_kernel(const EvoParams p, const int nchunks, const int slots) {
  constexpr int DP = 32, KS = 2, NW = 4;
  constexpr int LAST = TPW - 1;
  static_assert(TPW >= 2, "the pipeline needs distinct first and last tiles of a step");
  using L = BwdLayout<T, DP>;
  using frag = frag_t<T>;
  using AM = AsmMma<T>;
  static_assert(sizeof(T) == 2, "16-bit element types only");
  constexpr int WAVE_BYTES = PwLayout<T>::wave_bytes(TPW);

  const int S = p.S, D = p.D;
  const int NT = (S + 31) >> 5;

  extern __shared__ __align__(16) unsigned char smem_raw[];
  AddrRec* Recs = reinterpret_cast<AddrRec*>(smem_raw);                     // [12]
  T* Stage = reinterpret_cast<T*>(smem_raw + PwLayout<T>::REC_BYTES);       // [2][Q tile | dO tile]
  unsigned* Lpk = reinterpret_cast<unsigned*>(Stage + 2 * L::STAGE_ELEMS);  // [2][32] packed -LSE/scale
  unsigned* Dpk = Lpk + 64;                                                 // [2][32] packed -delta
  unsigned char* Wv = reinterpret_cast<unsigned char*>(Dpk + 64);           // [NW][WAVE_BYTES]
  // Sequences of more than NW * TPW key tiles take several passes per problem; the fp32 dQ of the passes so far
  // lives in this work-group's own array in global memory (it would not fit the LDS next to the key tiles) and
  // stays in the L2: every thread re-reads exactly what it wrote one pass earlier, one step ahead of its use.
  // (the one-pass variant is launched with nchunks = 1 and never touches the array; it keeps the run-time test
  // and an LDS address only because the register allocation of the hand-scheduled loop is sensitive to both)
  float* DQacc = MP ? p.dq_scratch + (size_t)blockIdx.x * NT * 1024                       // [NT * 32][32]
                    : reinterpret_cast<float*>(Wv + NW * WAVE_BYTES);
  f32x4 accpre = {0.0f, 0.0f, 0.0f, 0.0f};

  // ---- this work-group's share of the problems ---------------------------------------------------
  // XCD x owns the rows bn = 8 r + x; its problems are (row r, head h) in the order r * H + h, dealt
  // round-robin to the `slots` work-groups of the XCD: neighbouring work-groups run the heads of one
  // row at the same time.
  const int bid = blockIdx.x;
  const int xcd = bid & 7, slot = bid >> 3;
  const int BN = p.B * p.N;
  const int rows_x = BN > xcd ? (BN - xcd + 7) >> 3 : 0;
  const int items_x = rows_x * p.H;
  if (slot >= items_x) return;
  const int nk = (items_x - slot + slots - 1) / slots;
  const int npasses = nk * nchunks;

  const int tid = threadIdx.x, l = tid & 63, x = l & 31, g = l >> 5;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const float cexp = p.scale * MF_LOG2E;
  const float inv_scale = 1.0f / p.scale;

  T* Trw = reinterpret_cast<T*>(Wv + w * WAVE_BYTES);
  float* Slw = reinterpret_cast<float*>(Wv + w * WAVE_BYTES + L::TR_BYTES);   // [2][32][SSTR]
  T* Kw = reinterpret_cast<T*>(Wv + w * WAVE_BYTES + L::TR_BYTES + 2 * L::SLAB_BYTES);   // [TPW][32][QSTR]
  T* Vw = Kw + TPW * 32 * L::QSTR;                                                       // [TPW][32][QSTR]

  const unsigned ones_g = g == 0 ? ones_word<T>() : 0u;
  const frag vaugB = to_acc(make_aug<T>(ones_g, 0u));

  // ---- staging of query tiles: every thread moves one 4-element run (8 bytes) of Q, dO and O of one row,
  // eight threads per row, so that all wavefronts do the same work; delta = <dO, O> is summed over the eight
  // threads of a row with DPP.  Loads are requested two steps ahead into two alternating register sets and
  // nothing touches a loaded register before its stash.
  struct Stg { u32x2 q, d, o; float lse; };
  const int srow = tid >> 3, shc = tid & 7;
  const int sc0 = 4 * shc < D ? 4 * shc : 0;
  const bool sdok = 4 * shc < D;

  // Base addresses of one (b, n, h) problem and the pass over it.  The batch / row / head strides fit 32 bits
  // (checked by the launcher).
  struct Item {
    const T *q, *dO, *o, *k, *v;
    T *dq, *dk, *dv;
    const float* lse;
    float* delta;
    int64_t mask_base;
    int obias, chunk;
  };
  if (tid < REC_COUNT) {
    AddrRec rc;
    auto tensor = [&](const EvoTensor& t, int shift) {
      rc.base = reinterpret_cast<unsigned long long>(t.ptr); rc.sb = (int)t.sb; rc.sn = (int)t.sn; rc.sh = (int)t.sh; rc.shift = shift;
    };
    auto rows = [&](const void* ptr) {   // [B, N, H, S] fp32
      rc.base = reinterpret_cast<unsigned long long>(ptr); rc.sb = p.N * p.H * S; rc.sn = p.H * S; rc.sh = S; rc.shift = 2;
    };
    constexpr int es = sizeof(T) == 2 ? 1 : 2;
    switch (tid) {
      case REC_Q: tensor(p.q, es); break;
      case REC_DO: tensor(p.dO, es); break;
      case REC_O: tensor(p.o, es); break;
      case REC_K: tensor(p.k, es); break;
      case REC_V: tensor(p.v, es); break;
      case REC_DQ: tensor(p.dq, es); break;
      case REC_DK: tensor(p.dk, es); break;
      case REC_DV: tensor(p.dv, es); break;
      case REC_LSE: rows(p.lse); break;
      case REC_DELTA: rows(p.delta); break;
      case REC_MASK: rc.base = 0; rc.sb = (int)p.mask_sb; rc.sn = (int)p.mask_sn; rc.sh = 0; rc.shift = 0; break;
      default: rc.base = 0; rc.sb = (int)p.bias_sb; rc.sn = 0; rc.sh = (int)p.bias_sh; rc.shift = 0; break;
    }
    Recs[tid] = rc;
  }
  __syncthreads();
  auto decode = [&](int pass) {
    Item it;
    const int k = pass / nchunks;
    it.chunk = pass - k * nchunks;
    const int j = slot + k * slots;
    const int r = j / p.H, h = j - r * p.H;
    const int bn = r * 8 + xcd;
    const int b = bn / p.N, n = bn - b * p.N;
    const AddrRec rc = Recs[l < REC_COUNT ? l : 0];
    const long long off = (long long)b * rc.sb + (long long)n * rc.sn + (long long)h * rc.sh;
    const unsigned long long a = rc.base + ((unsigned long long)off << rc.shift);
    const int alo = (int)(unsigned)a, ahi = (int)(unsigned)(a >> 32);
    auto lane = [&](int i) {
      const unsigned lo = (unsigned)__builtin_amdgcn_readlane(alo, i), hi = (unsigned)__builtin_amdgcn_readlane(ahi, i);
      return ((unsigned long long)hi << 32) | lo;
    };
    it.q = as_global<const T>(lane(REC_Q));
    it.dO = as_global<const T>(lane(REC_DO));
    it.o = as_global<const T>(lane(REC_O));
    it.k = as_global<const T>(lane(REC_K));
    it.v = as_global<const T>(lane(REC_V));
    it.dq = as_global<T>(lane(REC_DQ));
    it.dk = as_global<T>(lane(REC_DK));
    it.dv = as_global<T>(lane(REC_DV));
    it.lse = as_global<const float>(lane(REC_LSE));
    it.delta = as_global<float>(lane(REC_DELTA));
    it.mask_base = (int64_t)lane(REC_MASK);
    it.obias = __builtin_amdgcn_readlane(alo, REC_BIAS);
    return it;
  };

  const unsigned str_q = (unsigned)p.q.ss, str_d = (unsigned)p.dO.ss;
  const unsigned str_o = (unsigned)p.o.ss;
  const unsigned dq_ss = (unsigned)p.dq.ss;

  typedef T out4_t __attribute__((ext_vector_type(4)));
  const int rrow = tid >> 3, rc4 = tid & 7;     // slab reduction: one 4-column run of one row per thread
  const int arow = unperm32(x);

  // ---- what a pass needs before its first product, requested one pass ahead (while the preceding pass
  // stores its results): the K / V rows and mask values of this wavefront's key tiles, the first bias tiles
  // and the first two query tiles.  Tiles past S run on clamped keys with mask -inf (exact zeros) and read
  // bias column block 0.
  frag kpre[TPW][KS], vpre[TPW][KS];
  unsigned mraw[TPW];       // raw mask elements: nothing computes on a requested value before the pass starts
  const int mask_es = p.mask_dtype == MF_F32 ? 4 : (p.mask_dtype == MF_F16 || p.mask_dtype == MF_BF16) ? 2 : 1;
  unsigned bias_off[TPW];
  f32x16 bzn[TPW];
  Stg sa0, sa1;
  auto fetch_q_of = [&](const Item& im, int it, Stg& st) {
    const int qi = (it < NT ? it : NT - 1) * 32 + srow;
    const unsigned qc = (unsigned)(qi < S ? qi : S - 1);
    st.q = *reinterpret_cast<const u32x2*>(im.q + sc0 + __umul24(qc, str_q));
    st.d = *reinterpret_cast<const u32x2*>(im.dO + sc0 + __umul24(qc, str_d));
    st.o = *reinterpret_cast<const u32x2*>(im.o + sc0 + __umul24(qc, str_o));
    st.lse = im.lse[qc];
  };
  auto load_bias = [&](int t, int it) {
    const float* bp = p.bias + bias_off[t] + (it < NT ? it : NT - 1) * 1024;
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(bp + 256 * c4);
      bzn[t][4 * c4] = v[0]; bzn[t][4 * c4 + 1] = v[1]; bzn[t][4 * c4 + 2] = v[2]; bzn[t][4 * c4 + 3] = v[3];
    }
  };
  auto request_pass = [&](const Item& im) {
    const int tile0 = im.chunk * NW * TPW + w * TPW;
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int j0 = (tile0 + t) * 32;
      const int j = j0 + x;
      const int jc = j < S ? j : S - 1;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = 16 * g + 8 * s;
        const int dcl = d0 < D ? d0 : 0;
        kpre[t][s] = ld8<T>(im.k + (int64_t)jc * p.k.ss + dcl);
        vpre[t][s] = ld8<T>(im.v + (int64_t)jc * p.v.ss + dcl);
      }
      {
        const unsigned char* mp = reinterpret_cast<const unsigned char*>(p.mask) +
                                  (im.mask_base + (int64_t)jc * p.mask_sj) * mask_es;
        if (mask_es == 4) mraw[t] = *reinterpret_cast<const unsigned*>(mp);
        else if (mask_es == 2) mraw[t] = *reinterpret_cast<const unsigned short*>(mp);
        else mraw[t] = *mp;
      }
      bias_off[t] = (unsigned)(im.obias + (int64_t)(j0 < S ? j0 >> 5 : 0) * p.bias_nt * 1024 + 4 * l);
    }
#pragma unroll
    for (int t = 0; t < TPW; ++t) load_bias(t, 0);
    fetch_q_of(im, 0, sa0);
    fetch_q_of(im, 1, sa1);
  };

  Item nx = decode(0);
  request_pass(nx);

  for (int pass = 0; pass < npasses; ++pass) {
    const Item im = nx;
    const bool last_chunk = im.chunk == nchunks - 1;
    const int tile0 = im.chunk * NW * TPW + w * TPW;      // first key tile of this wavefront

    auto fetch_q = [&](int it, Stg& st) { fetch_q_of(im, it, st); };
    auto stash_q = [&](int it, const Stg& st) {
      const int buf = it & 1;
      T* qd = Stage + buf * L::STAGE_ELEMS + srow * L::QSTR + 4 * shc;
      const u32x2 zero2 = {0u, 0u};
      *reinterpret_cast<u32x2*>(qd) = sdok ? st.q : zero2;
      *reinterpret_cast<u32x2*>(qd + 32 * L::QSTR) = sdok ? st.d : zero2;
      float part = sdok ? dot4<T>(st.d, st.o) : 0.0f;
      part = group_sum<8>(part);
      const int qi = it * 32 + srow;
      const float l2 = (qi >= S || st.lse == -__builtin_inff()) ? __builtin_inff() : st.lse * inv_scale;
      // the eight threads of a row write the same words
      Lpk[buf * 32 + srow] = pack_split<T>(-l2);
      Dpk[buf * 32 + srow] = pack_split<T>(-part);
      if (shc == 0 && qi < S && im.chunk == 0) im.delta[qi] = part;
    };
    // fp32 dQ of the earlier passes: device-scope loads (the line may sit in this compute unit's L1 since an
    // earlier problem; the value was written through to the L2 one pass ago by this very thread)
    auto load_acc = [&](const float* src) {
      f32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = __hip_atomic_load(src + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return v;
    };
    if constexpr (MP) {
      if (im.chunk > 0) accpre = load_acc(DQacc + rrow * 32 + 4 * rc4);                // query tile 0
    }
    // fixed-order sum of the NW slabs of query tile `it`, scale, store (or keep in the work-group's fp32 array)
    auto reduce_dq = [&](int it) {
      const float* sl0 = reinterpret_cast<const float*>(Wv + L::TR_BYTES) + (it & 1) * (32 * L::SSTR) + rrow * L::SSTR + 4 * rc4;
      f32x4 part4[NW];
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) part4[ww] = *reinterpret_cast<const f32x4*>(sl0 + ww * (WAVE_BYTES / 4));
      f32x4 sum = part4[0];
#pragma unroll
      for (int ww = 1; ww < NW; ++ww) sum += part4[ww];
      const int qi = it * 32 + rrow;
      if (nchunks > 1) {
        float* acc = DQacc + qi * 32 + 4 * rc4;
        if (im.chunk > 0) {
          if constexpr (MP) {
            sum += accpre;
            if (it + 1 < NT) accpre = load_acc(acc + 1024);  // the next tile's, a step ahead of its use
          } else {
            sum += *reinterpret_cast<const f32x4*>(acc);
          }
        }
        if (!last_chunk) { *reinterpret_cast<f32x4*>(acc) = sum; return; }
      }
      if (qi < S && 4 * rc4 < D) {
        out4_t ov = {(T)(sum[0] * p.scale), (T)(sum[1] * p.scale), (T)(sum[2] * p.scale), (T)(sum[3] * p.scale)};
        *reinterpret_cast<out4_t*>(im.dq + __umul24((unsigned)qi, dq_ss) + 4 * rc4) = ov;
      }
    };

    // ---- this pass's key tiles: K and V rows into the wavefront's LDS tiles (fragments are read from there
    // slot by slot), mask carrier
    frag maugB[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = 16 * g + 8 * s;
        st8<T>(Kw + (t * 32 + x) * L::QSTR + d0, d0 < D ? kpre[t][s] : frag_zero<T>());
        st8<T>(Vw + (t * 32 + x) * L::QSTR + d0, d0 < D ? vpre[t][s] : frag_zero<T>());
      }
      float mv;
      if (mask_es == 4) mv = __builtin_bit_cast(float, mraw[t]);
      else if (p.mask_dtype == MF_F16) mv = (float)__builtin_bit_cast(f16_t, (unsigned short)mraw[t]);
      else if (p.mask_dtype == MF_BF16) mv = __builtin_bit_cast(float, mraw[t] << 16);
      else mv = mraw[t] ? 0.0f : -__builtin_inff();
      mv = (tile0 + t) * 32 + x < S ? mv * inv_scale : -__builtin_inff();
      maugB[t] = to_acc(make_aug<T>(g == 0 ? pack_split<T>(mv) : 0u, ones_g));
    }

    stash_q(0, sa0);
    fetch_q(2, sa0);
    __syncthreads();

    // operands of the current step: A operands of the score / dP products (row-major fragments and the
    // carriers of -LSE/scale and -delta), and Q^T / dO^T for the dK / dV products
    frag qA[KS], doA[KS], qaugA, doaugA, qT[2], doT[2];
    auto read_a_operands = [&](int it) {
      const int buf = it & 1;
      const T* qs = Stage + buf * L::STAGE_ELEMS;
      const T* dos = qs + 32 * L::QSTR;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        qA[s] = ld8<T>(qs + arow * L::QSTR + 16 * g + 8 * s);
        doA[s] = ld8<T>(dos + arow * L::QSTR + 16 * g + 8 * s);
      }
      qaugA = to_acc(make_aug<T>(ones_g, g == 0 ? Lpk[buf * 32 + arow] : 0u));
      doaugA = to_acc(make_aug<T>(g == 0 ? Dpk[buf * 32 + arow] : 0u, 0u));
    };
    auto read_t_operands = [&](int it) {
      const T* qs = Stage + (it & 1) * L::STAGE_ELEMS;
      const T* dos = qs + 32 * L::QSTR;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        doT[u] = TrRead<T>::read(dos, L::QSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(0, l), dsel<DP>(0, x));
        qT[u] = TrRead<T>::read(qs, L::QSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(0, l), dsel<DP>(0, x));
      }
    };
    // fragments of one of this wavefront's key tiles
    auto read_kv = [&](int t, frag (&kf)[KS], frag (&vf)[KS]) {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        kf[s] = ld8<T>(Kw + (t * 32 + x) * L::QSTR + 16 * g + 8 * s);
        vf[s] = ld8<T>(Vw + (t * 32 + x) * L::QSTR + 16 * g + 8 * s);
      }
    };
    auto read_kt = [&](int t, frag (&kT)[2]) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
        kT[u] = TrRead<T>::read(Kw + t * 32 * L::QSTR, L::QSTR, 8 * u + 8 * g, g, l, dsel_chunk<DP>(0, l), dsel<DP>(0, x));
    };

    f32x16 dk[TPW], dv[TPW], dq;
    {
      // cleared by products of zero operands: one instruction per accumulator instead of sixteen register writes
      const frag zf_a = to_acc(frag_zero<T>()), zf_v = frag_zero<T>();
#pragma unroll
      for (int t = 0; t < TPW; ++t) { AM::zero_av(dk[t], zf_a, zf_v); AM::zero_av(dv[t], zf_a, zf_v); }
      AM::zero_av(dq, zf_a, zf_v);
    }

    // Two sets of score registers (the tile being exponentiated and the one being computed), one set of
    // P / dS words: a word is rewritten only after the product that reads its old value has been issued.
    f32x16 zA, dpA, zB, dpB;
    u32x4 pw[2], dw[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) { pw[i] = u32x4{0u, 0u, 0u, 0u}; dw[i] = u32x4{0u, 0u, 0u, 0u}; }
    // transposed dS of the preceding tile; before the first tile: zeros, read from the (zeroed) LDS tile so
    // that the registers are only ever written by LDS reads
    frag dsT[2];
    st8<T>(Trw + x * L::TSTR + 16 * g, frag_zero<T>());
    st8<T>(Trw + x * L::TSTR + 16 * g + 8, frag_zero<T>());

    // prologue: operands of step 0, scores of tile (0, 0)
    read_a_operands(0);
    read_t_operands(0);
    {
      frag kf[KS], vf[KS];
      read_kv(0, kf, vf);
      AM::v_set(zA, qaugA, maugB[0], bzn[0]);
      AM::v_zero(dpA, doaugA, vaugB);
      asm volatile("s_nop 15\n s_nop 15" : "+v"(bzn[0]));   // the C operand is read while the product runs
      load_bias(0, 1);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        AM::v_acc(zA, qA[s], kf[s]);
        if (s + 1 < KS) AM::v_acc(dpA, doA[s], vf[s]); else AM::v_acc_last(dpA, doA[s], vf[s]);
      }
    }

    // One slot of the pipeline = one (query tile it, key tile t) pair.  In the slot the vector ALU turns
    // the scores zc / dpc of tile (it, t) into the words of P and dS, while the matrix pipe computes the
    // products of the preceding tile (whose words are consumed just before they are rewritten; its
    // transposed dS is in dsT) and the scores zn / dpn of the following tile.
    // The exponentiation of a tile is done in two octets (eight accumulator registers = one operand
    // fragment) and five stages per octet, each stage a run of independent instructions whose results are
    // first used a stage later: a single wavefront has nobody else to hide the latency of a dependent
    // instruction.  The scores are overwritten in place; the empty statements keep each stage where it is
    // written (between two MFMAs).
    auto st_scale = [&](const int o, f32x16& z) {
#pragma unroll
      for (int i = 8 * o; i < 8 * o + 8; ++i) z[i] *= cexp;
      asm volatile("" : "+v"(z));
    };
    auto st_exp = [&](const int o, f32x16& z) {
#pragma unroll
      for (int i = 8 * o; i < 8 * o + 8; ++i) z[i] = fast_exp2(z[i]);
      asm volatile("" : "+v"(z));
    };
    auto st_pack_p = [&](const int o, const f32x16& z) {
#pragma unroll
      for (int k = 0; k < 4; ++k) pw[o][k] = pack2<T>(z[8 * o + 2 * k], z[8 * o + 2 * k + 1]);
      asm volatile("" : "+v"(pw[o]));
    };
    auto st_ds = [&](const int o, const f32x16& z, f32x16& dp) {
#pragma unroll
      for (int i = 8 * o; i < 8 * o + 8; ++i) dp[i] *= z[i];
      asm volatile("" : "+v"(dp));
    };
    auto st_pack_ds = [&](const int o, const f32x16& dp) {
#pragma unroll
      for (int k = 0; k < 4; ++k) dw[o][k] = pack2<T>(dp[8 * o + 2 * k], dp[8 * o + 2 * k + 1]);
      asm volatile("" : "+v"(dw[o]));
    };

#define MF_SLOT(TT, IT, ZC, DPC, ZN, DPN, SA)                                                                     \
    {                                                                                                          \
      constexpr int t = (TT);                                                                                  \
      constexpr int tn = (t + 1) % TPW, tp = (t + TPW - 1) % TPW;                                              \
      const int qs_ = (IT);                                                                                     \
      const int qn_ = t == LAST ? qs_ + 1 : qs_;          /* query tile of the following tile */                 \
      if (t == LAST) {                                                                                         \
        MF_TL(p, MF_TLI(qs_, t, 3));                                                                         \
        barrier_keep_vm<63>();                                                         \
        read_a_operands(qs_ + 1);                                                                               \
        if (qs_ > 0) reduce_dq(qs_ - 1);                                                 \
      }                                                                                                        \
      MF_TL(p, MF_TLI(qs_, t, 0));                                                                           \
      frag kfn[KS], vfn[KS], kTp[2];                                                                           \
      read_kt(tp, kTp);                                                                                        \
      /* first half: products of the preceding tile, first octet of this tile */                             \
      MF_FENCE(); AM::acc_av(dv[tp], doT[0], __builtin_bit_cast(frag, pw[0])); MF_FENCE();                   \
      st_scale(0, ZC);                                                                                       \
      kfn[0] = ld8<T>(Kw + (tn * 32 + x) * L::QSTR + 16 * g);                                                \
      MF_FENCE(); AM::acc_av(dk[tp], qT[0], __builtin_bit_cast(frag, dw[0])); MF_FENCE();                    \
      st_exp(0, ZC);                                                                                         \
      kfn[1] = ld8<T>(Kw + (tn * 32 + x) * L::QSTR + 16 * g + 8);                                            \
      MF_FENCE(); AM::acc_av(dv[tp], doT[1], __builtin_bit_cast(frag, pw[1])); MF_FENCE();                   \
      st_pack_p(0, ZC);                                                                                      \
      /* dS of the preceding tile, transposed: its rows were written half a slot and more ago (an LDS read  \
         queued right behind a write of the same wavefront stalls the wavefront for ~200 cycles) */          \
      _Pragma("unroll") for (int u = 0; u < 2; ++u)                                                            \
        dsT[u] = TrRead<T>::read(Trw, L::TSTR, 8 * u + 8 * g, g, l, plain_chunk(l), x);                        \
      vfn[0] = ld8<T>(Vw + (tn * 32 + x) * L::QSTR + 16 * g);                                                \
      MF_FENCE(); AM::acc_av(dk[tp], qT[1], __builtin_bit_cast(frag, dw[1])); MF_FENCE();                    \
      st_ds(0, ZC, DPC);                                                                                     \
      vfn[1] = ld8<T>(Vw + (tn * 32 + x) * L::QSTR + 16 * g + 8);                                            \
      MF_FENCE();                                                                                            \
      if (tp == 0) AM::zero_av(dq, kTp[0], dsT[0]); else AM::acc_av(dq, kTp[0], dsT[0]);                     \
      MF_FENCE();                                                                                            \
      st_pack_ds(0, DPC);                                                                                    \
      MF_FENCE(); AM::acc_av(dq, kTp[1], dsT[1]); MF_FENCE();                                                \
      st_scale(1, ZC);                                                                                       \
      if (t == 0) {                                                                                            \
        /* the preceding tile closed query tile qs_ - 1: its partial dQ^T goes to the slab (lane (x = query,   \
           g) owns 16 contiguous columns; at qs_ = 0 this is a dummy of zeros); then this step's transposed     \
           operands and the staging */                                                                         \
        MF_TL(p, MF_TLI(qs_, t, 5));                                                                         \
        read_t_operands(qs_);                                                                                   \
        MF_TL(p, MF_TLI(qs_, t, 6));                                                                         \
        stash_q(qs_ + 1, SA);                                                          \
        MF_TL(p, MF_TLI(qs_, t, 7));                                                                         \
        fetch_q(qs_ + 3, SA);                                                          \
        /* the partial dQ^T is stored last: the products that wrote it are more than 18 issue slots old */   \
        MF_FENCE();                                                                                          \
        MF_TL(p, MF_TLI(qs_, t, 4));                                                                         \
        float* slab = Slw + ((qs_ - 1) & 1) * (32 * L::SSTR);                                                   \
        _Pragma("unroll") for (int c4 = 0; c4 < 4; ++c4) {                                                   \
          f32x4 v;                                                                                             \
          v[0] = dq[4 * c4]; v[1] = dq[4 * c4 + 1]; v[2] = dq[4 * c4 + 2]; v[3] = dq[4 * c4 + 3];              \
          *reinterpret_cast<f32x4*>(slab + x * L::SSTR + 16 * g + 4 * c4) = v;         \
        }                                                                                                      \
      }                                                                                                        \
      /* first half of this tile's dS, rows = keys, into the wavefront's LDS tile (the transposed reads of  \
         the preceding tile have been consumed by the dQ products above) */                                  \
      st8<T>(Trw + x * L::TSTR + 16 * g, __builtin_bit_cast(frag, dw[0]));                           \
      MF_TL(p, MF_TLI(qs_, t, 1));                                                                           \
      /* second half: scores and dP of the following tile, second octet of this tile (its stages run one   \
         product early so that the last dS words are in LDS two products before the slot ends) */            \
      MF_FENCE(); AM::v_set(ZN, qaugA, maugB[tn], bzn[tn]); MF_FENCE();                                      \
      st_exp(1, ZC);                                                                                         \
      MF_FENCE(); AM::v_zero(DPN, doaugA, vaugB); MF_FENCE();                                                \
      st_pack_p(1, ZC);                                                                                      \
      /* The matrix pipe reads the bias tile (the C operand) while the product runs: its registers must      \
         not be rewritten, or reused by the compiler, in the first 13 issue slots after the MFMA.  The empty \
         statement keeps them allocated until here; only then is the next bias tile requested. */            \
      asm volatile("" : "+v"(bzn[tn]));                                                                      \
      load_bias(tn, qn_ + 1);                                                          \
      MF_FENCE(); AM::v_acc(ZN, qA[0], kfn[0]); MF_FENCE();                                                  \
      st_ds(1, ZC, DPC);                                                                                     \
      MF_FENCE(); AM::v_acc(DPN, doA[0], vfn[0]); MF_FENCE();                                                \
      st_pack_ds(1, DPC);                                                                                    \
      MF_FENCE(); AM::v_acc(ZN, qA[1], kfn[1]); MF_FENCE();                                                  \
      st8<T>(Trw + x * L::TSTR + 16 * g + 8, __builtin_bit_cast(frag, dw[1]));                       \
      /* After the last slot of a pass these scores belong to no tile, and the code behind the walk reuses  \
         their registers: the last product of a step is followed by idle slots, so that no instruction can    \
         rewrite a register an MFMA in flight is about to write. */                                            \
      MF_FENCE();                                                                                              \
      if (t == LAST) AM::v_acc_last(DPN, doA[1], vfn[1]); else AM::v_acc(DPN, doA[1], vfn[1]);                 \
      MF_FENCE();                                                                                              \
      MF_TL(p, MF_TLI(qs_, t, 2));                                                                           \
    }

    // one query tile = TPW slots; the score register sets alternate from slot to slot
#define MF_STEP_EVEN(IT, SA)                                                                              \
    MF_SLOT(0, IT, zA, dpA, zB, dpB, SA)                                                                  \
    MF_SLOT(1, IT, zB, dpB, zA, dpA, SA)                                                                  \
    if constexpr (TPW == 3) { MF_SLOT(2, IT, zA, dpA, zB, dpB, SA) }
#define MF_STEP_ODD(IT, SA)                                                                               \
    MF_SLOT(0, IT, zB, dpB, zA, dpA, SA)                                                                  \
    MF_SLOT(1, IT, zA, dpA, zB, dpB, SA)                                                                  \
    if constexpr (TPW == 3) { MF_SLOT(2, IT, zB, dpB, zA, dpA, SA) }

    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0) once: the loop's own wait counts stay exact
    // With TPW = 2 a step leaves the score register sets where it found them; with TPW = 3 two steps do.
    int it = 0;
    if constexpr (TPW == 2) {
      for (; it + 1 < NT; it += 2) {
        MF_STEP_EVEN(it, sa1)
        MF_STEP_EVEN(it + 1, sa0)
      }
      if (it < NT) { MF_STEP_EVEN(it, sa1) }
    } else {
      for (; it + 1 < NT; it += 2) {
        MF_STEP_EVEN(it, sa1)
        MF_STEP_ODD(it + 1, sa0)
      }
      if (it < NT) { MF_STEP_EVEN(it, sa1) }
    }
#undef MF_STEP_EVEN
#undef MF_STEP_ODD
#undef MF_SLOT
    // the next pass's first operands travel while this pass's results are reduced and stored
    if (pass + 1 < npasses) {
      nx = decode(pass + 1);
      request_pass(nx);
    }
    // drain: products of the last tile
    {
      frag kTp[2];
      read_kt(LAST, kTp);
      AM::acc_av(dv[LAST], doT[0], __builtin_bit_cast(frag, pw[0]));
      AM::acc_av(dk[LAST], qT[0], __builtin_bit_cast(frag, dw[0]));
      AM::acc_av(dv[LAST], doT[1], __builtin_bit_cast(frag, pw[1]));
      AM::acc_av(dk[LAST], qT[1], __builtin_bit_cast(frag, dw[1]));
#pragma unroll
      for (int u = 0; u < 2; ++u) dsT[u] = TrRead<T>::read(Trw, L::TSTR, 8 * u + 8 * g, g, l, plain_chunk(l), x);
      AM::acc_av(dq, kTp[0], dsT[0]);
      AM::acc_av_last(dq, kTp[1], dsT[1]);
    }
    {
      float* slab = Slw + ((NT - 1) & 1) * (32 * L::SSTR);
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        f32x4 v;
        v[0] = dq[4 * c4]; v[1] = dq[4 * c4 + 1]; v[2] = dq[4 * c4 + 2]; v[3] = dq[4 * c4 + 3];
        *reinterpret_cast<f32x4*>(slab + x * L::SSTR + 16 * g + 4 * c4) = v;
      }
    }
    __syncthreads();
    reduce_dq(NT - 1);

    // ---- dK, dV of this wavefront's tiles: lane (x = key, g) owns 16 contiguous columns -------------
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int j = (tile0 + t) * 32 + x;
      if (j < S) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int d0 = 16 * g + 8 * u;
          if (d0 < D) {
            f32x16 dks = dk[t];
#pragma unroll
            for (int i = 0; i < 16; ++i) dks[i] *= p.scale;
            st8<T>(im.dk + (int64_t)j * p.dk.ss + d0, acc_half<T>(dks, u));
            st8<T>(im.dv + (int64_t)j * p.dv.ss + d0, acc_half<T>(dv[t], u));
          }
        }
      }
    }
    __syncthreads();   // the next pass restages the first query tile and reuses the slabs
  }
}
#undef MF_FENCE

template <typename T, int TPW>
static hipError_t launch_pw_t(const EvoParams& p, int nchunks, int num_cu, hipStream_t stream) {
  const int NT = (p.S + 31) / 32;
  const size_t smem = PwLayout<T>::smem(TPW);
  if (smem > 160 * 1024) return hipErrorInvalidValue;
  // work-groups per XCD: one per compute unit, fewer when there are fewer problems
  const long long BN = (long long)p.B * p.N;
  const long long items_x = ((BN + 7) / 8) * p.H;
  int slots = num_cu / 8 > 0 ? num_cu / 8 : 1;
  if (items_x < slots) slots = (int)items_x;
  auto kern = nchunks > 1 ? evo_bwd_dqkv_pw_kernel<T, TPW, true> : evo_bwd_dqkv_pw_kernel<T, TPW, false>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(8 * slots)), dim3(256), smem, stream, p, nchunks, slots);
  return hipGetLastError();
}

// Key tiles per wavefront and passes for a sequence of NT key tiles (four wavefronts per work-group).
static void pw_shape(int NT, int& tpw, int& nchunks) {
  tpw = NT <= 8 ? 2 : 3;
  nchunks = (NT + 4 * tpw - 1) / (4 * tpw);
}

// True when the persistent kernel handles this problem: 16-bit types, D <= 32, more than four key tiles
// (shorter sequences leave wavefronts idle here), row strides that fit the 24-bit multiplies, bias offsets
// that fit 32 bits, LDS for the fp32 dQ array of multi-pass sequences.
template <typename T> static bool pw_supported(const EvoParams& p) {
  if (sizeof(T) != 2 || p.D > 32) return false;
  auto fits = [&](int64_t ss) { return ss < (1 << 24) && (int64_t)p.S * ss < (1LL << 31); };
  if (!(fits(p.q.ss) && fits(p.dO.ss) && fits(p.o.ss) && fits(p.dq.ss))) return false;
  // batch / row / head strides as 32-bit factors of the per-problem offsets
  auto s32 = [](int64_t v) { return v >= 0 && v < (1LL << 31); };
  for (const EvoTensor* t : {&p.q, &p.k, &p.v, &p.dO, &p.o, &p.dq, &p.dk, &p.dv})
    if (!(s32(t->sb) && s32(t->sn) && s32(t->sh))) return false;
  if (!(s32(p.mask_sb) && s32(p.mask_sn))) return false;
  if ((int64_t)p.B * p.N * p.H * p.S >= (1LL << 31)) return false;        // row offsets of LSE / delta as 32-bit factors
  const int NT = (p.S + 31) / 32;
  if (NT <= 4) return false;
  if ((int64_t)p.B * p.bias_sb + 64 * 4 >= (1LL << 31)) return false;
  int tpw, nchunks;
  pw_shape(NT, tpw, nchunks);
  if (nchunks > 1 && !p.dq_scratch) return false;
  return PwLayout<T>::smem(tpw) <= 160 * 1024;
}

template <typename T> static hipError_t launch_pw(const EvoParams& p, int num_cu, hipStream_t stream) {
  int tpw, nchunks;
  pw_shape((p.S + 31) / 32, tpw, nchunks);
  if (tpw == 2) return launch_pw_t<T, 2>(p, nchunks, num_cu, stream);
  return launch_pw_t<T, 3>(p, nchunks, num_cu, stream);
}

uint64_t evo_bwd_dqkv_pw_scratch_bytes(int dtype, int S, int D, int num_cu) {
  if ((dtype != MF_BF16 && dtype != MF_F16) || D > 32) return 0;
  int tpw, nchunks;
  pw_shape((S + 31) / 32, tpw, nchunks);
  if (nchunks <= 1) return 0;
  const uint64_t groups = 8ull * (uint64_t)(num_cu / 8 > 0 ? num_cu / 8 : 1);   // the most work-groups launch_pw_t starts
  return groups * (uint64_t)((S + 31) / 32) * 1024 * 4;
}

bool evo_bwd_dqkv_pw_supported(const EvoParams& p) {
  switch (p.dtype) {
    case MF_BF16: return pw_supported<bf16_t>(p);
    case MF_F16: return pw_supported<f16_t>(p);
    default: return false;
  }
}

hipError_t launch_evo_bwd_dqkv_pw(const EvoParams& p, int num_cu, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return launch_pw<bf16_t>(p, num_cu, stream);
    case MF_F16: return launch_pw<f16_t>(p, num_cu, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mf
