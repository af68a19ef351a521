// Bias gradient of the pair-biased attention for the 16-bit element types at D = 32 with paired heads:
// dBias[b, h, i, j] = sum over rows n of dS[b, n, h, i, j], the sum the reference forms with fp32 atomics
// (megafold/model/FusedEvoAttention/evoattention.py:459-465, tl.atomic_add on d_pair_bias).
//
// Same decomposition as evo_bwd_dbias_kernel<T, 32, 2, 2> (evoattn_bwd.hip): a work-group of eight wavefronts
// owns the patch (128 queries x 64 keys) of a head PAIR and walks over a chunk of the rows n; wavefront
// (head, query tile) keeps its 32 x 64 piece of the sum and the matching bias seed in registers.  What differs
// is how a row travels and how its work is ordered:
//
//  * The operands of a row (K, V of the 64 keys, Q, dO of the 128 queries, both heads: whole 128-byte lines;
//    LSE and delta of the queries) go from global memory straight into LDS (global_load_lds), three rows deep:
//    no staging registers, no LDS stores, no selects in the wavefronts' instruction streams, and a row is
//    requested two row steps before its first use.  The destination of such a load is fixed (lane i writes 16
//    bytes at base + 16 i), so the row permutation of the key tiles and the XOR swizzle of the 16-byte chunks
//    (conflict-free fragment reads) are applied on the global side: each lane fetches the chunk that belongs
//    where its data lands.  Rows or keys past S are clamped to S - 1: a clamped key carries mask -inf (an
//    exact zero), a clamped query is never stored.
//  * One barrier per row, in the MIDDLE of a row step: first the products of (row n, key tile 1) are issued
//    while the vector ALU turns the scores of (row n, tile 0) into probabilities, then the barrier publishes
//    row n + 1 and frees row n's slot for row n + 3, then the products of (row n + 1, tile 0) are issued while
//    the vector ALU works on (row n, tile 1).  A wavefront's matrix products are always one tile ahead of
//    its exponentials, so neither waits for the other.
//  * The key mask rides through a third contraction step of the score product (hi + lo 16-bit words written to
//    LDS by the first wavefront one row ahead), -delta through one of the dP product: per logit the vector
//    ALU does a multiply-add, an exponential and a multiply-add.
//
// All vector-memory instructions of the row loop are inline assembly and the waits are written out: the
// compiler would otherwise wait for EVERY outstanding load before an LDS read that may alias a direct load.
#include <type_traits>
#include "common.h"
#include "evoattn.h"

namespace mf {

namespace {

// LDS: three row slots, the key side of all slots first (so that every key-side read of a lane is one address
// register plus an immediate), then the query side.  Byte offsets:
constexpr int KS_BYTES = 16640;  // key side of one slot
constexpr int KS_K = 0;          //   [64 key rows][2 heads x 64 bytes], chunk c of row m at position c ^ ((m >> 1) & 7)
constexpr int KS_V = 8192;
constexpr int KS_MK = 16384;     //   [64 key rows] packed (hi, lo) of mask / scale
constexpr int QS_BASE = 3 * KS_BYTES;
constexpr int QS_BYTES = 34816;  // query side of one slot
constexpr int QS_LSE = 0;        //   [2 heads][128] fp32
constexpr int QS_DL = 1024;      //   [2 heads][128] fp32
constexpr int QS_Q = 2048;       //   [128 query rows][2 heads x 64 bytes], same swizzle as the key rows
constexpr int QS_DO = 18432;
constexpr int RING_BYTES = QS_BASE + 3 * QS_BYTES;
constexpr int RING = 3;
#ifdef MF_RING_KO_DO      // timing experiment, wrong results: dO is not loaded
constexpr int ROW_OPS = 5;
#else
constexpr int ROW_OPS = 7;       // direct-to-LDS loads per wavefront and row
#endif

#define MF_SB() __builtin_amdgcn_sched_barrier(0)

__device__ __forceinline__ void dma16(unsigned voff, const void* sbase, unsigned lds) {
  asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "{m0}"(lds) : "memory");
}
__device__ __forceinline__ void dma4(unsigned voff, const void* sbase, unsigned lds) {
  asm volatile("global_load_lds_dword %0, %1" ::"v"(voff), "s"(sbase), "{m0}"(lds) : "memory");
}
// vmcnt(N), nothing else
template <int VM> __device__ __forceinline__ void wait_vm() {
  static_assert(VM >= 0 && VM < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt(((VM & 15) | ((VM >> 4) << 14)) | (7 << 4) | (15 << 8));
}

// The products are issued as inline assembly: that fixes their place between the runs of vector-ALU
// instructions (the compiler moves builtin MFMAs and the arithmetic around them freely, and did: with builtins
// the exponentials of three row steps ended up behind the third barrier, a hundred registers spilled).  Two idle
// slots in front of every product cover an operand written by the vector ALU just before (the mask and delta
// carriers); results are first read a tile step later.  csrc/check_pw_hazards.py checks both on the generated code.
template <typename T> struct RingMma;
#define MF_RING_MMA(T, MNEM)                                                                                   \
  template <> struct RingMma<T> {                                                                              \
    using frag = frag_t<T>;                                                                                    \
    static __device__ __forceinline__ void set(f32x16& d, const frag& a, const frag& b, const f32x16& c) {     \
      asm volatile("s_nop 1\n " MNEM " %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));                   \
    }                                                                                                          \
    static __device__ __forceinline__ void zero(f32x16& d, const frag& a, const frag& b) {                     \
      asm volatile("s_nop 1\n " MNEM " %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));                            \
    }                                                                                                          \
    static __device__ __forceinline__ void acc(f32x16& c, const frag& a, const frag& b) {                      \
      asm volatile("s_nop 1\n " MNEM " %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));                            \
    }                                                                                                          \
  };
MF_RING_MMA(bf16_t, "v_mfma_f32_32x32x16_bf16")
MF_RING_MMA(f16_t, "v_mfma_f32_32x32x16_f16")
#undef MF_RING_MMA

template <typename T> __device__ __forceinline__ frag_t<T> lds_frag(const unsigned char* p) {
  return ld8<T>(reinterpret_cast<const T*>(p));
}

}  // namespace

// MES: bytes of a mask element (4: fp32, 2: fp16 / bf16, 1: bool keep-mask)
template <typename T, int MES>
__global__ void __launch_bounds__(512, 1) evo_bwd_dbias_ring_kernel(const EvoParams p, const int IB, const int JB) {
  using frag = frag_t<T>;
  extern __shared__ __align__(16) unsigned char smem[];

  const int t512 = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(t512 >> 6);
  const int l = t512 & 63, x = l & 31, g = l >> 5;
  const int hs = wv >> 2, w = wv & 3;            // head inside the pair, query tile

  // (b, head pair, chunk) groups of R patches, dealt out evenly: XCD x takes the contiguous run
  // [x * per_xcd, (x + 1) * per_xcd) of the (group, patch) list
  const int Rg = IB * JB;
  const int bid = blockIdx.x;
  const int xcd = bid & 7, kq = bid >> 3;
  const int64_t total = (int64_t)p.B * (p.H / 2) * p.n_chunks * Rg;
  const int64_t per_xcd = (total + 7) / 8;
  const int64_t qidx = xcd * per_xcd + kq;
  if (kq >= per_xcd || qidx >= total) return;
  const int grp = (int)(qidx / Rg);
  const int reg = (int)(qidx % Rg);
  const int chunk = grp % p.n_chunks;
  const int hb = grp / p.n_chunks;
  const int h0 = (hb % (p.H / 2)) * 2;           // first head of the pair
  const int h = h0 + hs;
  const int b = hb / (p.H / 2);
  const int ib = reg % IB, jb = reg / IB;

  const int S = p.S;
  const int n_begin = chunk * p.rows_per_chunk;
  const int n_end = min(p.N, n_begin + p.rows_per_chunk);
  const int R = n_end - n_begin;
  const int jt0 = jb * 2;                        // first key tile of the patch
  const int qrow = w * 32 + x;                   // this lane's query row inside the patch
  const int qi = ib * 128 + qrow;
  const int qi_c = qi < S ? qi : S - 1;

  const float cexp = p.scale * MF_LOG2E;         // the accumulator holds z / scale
  const float inv_scale = 1.0f / p.scale;

  // ---- the bias patch is the same for every row n: it stays in registers as the seed of the score product
  f32x16 bz[2], acc[2];
  {
    const float* biasg = p.bias + b * p.bias_sb + h * p.bias_sh;
    const int qq = qi_c & 31;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      acc[t] = acc_zero();
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = (jt0 + t) * 32 + 16 * g + r;
        // element (query qi, key j) of the backward-layout tile (j / 32, qi / 32), see EvoParams::bias
        bz[t][r] = j < 32 * p.bias_nt
                       ? biasg[((int64_t)(j >> 5) * p.bias_nt + (qi_c >> 5)) * 1024 + (((qq & 15) >> 2) * 64 + 32 * (qq >> 4) + (j & 31)) * 4 + (qq & 3)]
                       : 0.0f;
      }
    }
    pin(bz[0]); pin(bz[1]);                      // loaded before the first direct load is issued
  }
  if (R <= 0) return;

  // ---- per-lane byte offsets of the direct loads (relative to the row's base address) ------------------
  const int es = (int)sizeof(T);
  const int m = t512 >> 3, pos = t512 & 7, cg = pos ^ ((m >> 1) & 7);   // LDS row, position, global chunk that lands there
  unsigned koff, voff, qoff[2], dooff[2];
  {
    int key = jt0 * 32 + (m & 32) + unperm32(m & 31);
    key = key < S ? key : S - 1;
    koff = (unsigned)((int64_t)key * p.k.ss * es + cg * 16);
    voff = (unsigned)((int64_t)key * p.v.ss * es + cg * 16);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int q = ib * 128 + 64 * i + m;
      q = q < S ? q : S - 1;
      qoff[i] = (unsigned)((int64_t)q * p.q.ss * es + cg * 16);
      dooff[i] = (unsigned)((int64_t)q * p.dO.ss * es + cg * 16);
    }
  }
  // LSE (wavefronts 0-3) / delta (4-7): wavefront ww = (head, half of the 128 queries), one value per lane
  unsigned ldoff;
  {
    const int ww = wv & 3;
    int q = ib * 128 + 64 * (ww & 1) + l;
    q = q < S ? q : S - 1;
    ldoff = (unsigned)(((ww >> 1) * S + q) * 4);
  }
  unsigned moff;
  {
    int key = jt0 * 32 + l;
    key = key < S ? key : S - 1;
    moff = (unsigned)((int64_t)key * p.mask_sj * MES);
  }

  // running base addresses of the next row to request (uniform)
  const char* kb = reinterpret_cast<const char*>(p.k.ptr) + (b * p.k.sb + h0 * p.k.sh + (int64_t)n_begin * p.k.sn) * es;
  const char* vb = reinterpret_cast<const char*>(p.v.ptr) + (b * p.v.sb + h0 * p.v.sh + (int64_t)n_begin * p.v.sn) * es;
  const char* qb = reinterpret_cast<const char*>(p.q.ptr) + (b * p.q.sb + h0 * p.q.sh + (int64_t)n_begin * p.q.sn) * es;
  const char* dob = reinterpret_cast<const char*>(p.dO.ptr) + (b * p.dO.sb + h0 * p.dO.sh + (int64_t)n_begin * p.dO.sn) * es;
  const int64_t row0 = (((int64_t)b * p.N + n_begin) * p.H + h0) * S;
  const char* ldb = reinterpret_cast<const char*>(wv < 4 ? p.lse : p.delta) + row0 * 4;
  const char* mb = reinterpret_cast<const char*>(p.mask) + (b * p.mask_sb + (int64_t)n_begin * p.mask_sn) * MES;
  const int64_t k_step = p.k.sn * es, v_step = p.v.sn * es, q_step = p.q.sn * es, do_step = p.dO.sn * es;
  const int64_t ld_step = (int64_t)p.H * S * 4, m_step = p.mask_sn * MES;
  int rows_left = R - 1, mrows_left = R - 1;     // rows after the one the pointers stand on

  const unsigned lds0 = (unsigned)(unsigned long)((__attribute__((address_space(3))) unsigned char*)smem);   // LDS byte address of the ring
  const unsigned wslot = (unsigned)wv * 1024;
  const unsigned ldst = QS_BASE + (wv < 4 ? QS_LSE : QS_DL) + (unsigned)(wv & 3) * 256;

  // Request of one row into ring slot `slot`, in seven parts (one instruction each) so that the requests can be
  // spread over a row step: a wavefront that issues them in one burst sits in the memory pipeline's queue for
  // hundreds of cycles.  Past the chunk's last row the last row is requested again.
  auto issue_part = [&](int slot, int part) {
    const unsigned ks = lds0 + (unsigned)slot * KS_BYTES + wslot;
    const unsigned qs = lds0 + QS_BASE + (unsigned)slot * QS_BYTES + wslot;
    switch (part) {
      case 0: dma16(koff, kb, ks + KS_K); break;
      case 1: dma16(voff, vb, ks + KS_V); break;
      case 2: dma16(qoff[0], qb, qs + QS_Q); break;
      case 3: dma16(qoff[1], qb, qs + QS_Q + 8192); break;
#ifndef MF_RING_KO_DO
      case 4: dma16(dooff[0], dob, qs + QS_DO); break;
      case 5: dma16(dooff[1], dob, qs + QS_DO + 8192); break;
#endif
      case 6:
        dma4(ldoff, ldb, lds0 + (unsigned)slot * QS_BYTES + ldst);
        if (rows_left > 0) {
          kb += k_step; vb += v_step; qb += q_step; dob += do_step; ldb += ld_step;
        }
        --rows_left;
        break;
      default: break;
    }
  };
  auto issue_row = [&](int slot) {
#pragma unroll
    for (int part = 0; part < 7; ++part) issue_part(slot, part);
  };
  // the 64 mask elements of a row, raw, one per lane (every wavefront requests them so that all wavefronts
  // count the same number of outstanding loads; the first one converts and publishes them)
  unsigned mraw;
  auto issue_mask = [&]() {
    if constexpr (MES == 4) asm volatile("global_load_dword %0, %1, %2" : "=v"(mraw) : "v"(moff), "s"(mb) : "memory");
    else if constexpr (MES == 2) asm volatile("global_load_ushort %0, %1, %2" : "=v"(mraw) : "v"(moff), "s"(mb) : "memory");
    else asm volatile("global_load_ubyte %0, %1, %2" : "=v"(mraw) : "v"(moff), "s"(mb) : "memory");
    if (mrows_left > 0) mb += m_step;
    --mrows_left;
  };
  const int mk_row = (l & 32) + perm32(l & 31);                  // operand row of key l of the patch
  const bool key_ok = jt0 * 32 + l < S;
  const bool mask_f16 = p.mask_dtype == MF_F16;
  auto publish_mask = [&](int slot) {
    if (wv == 0) {
      pin(mraw);
      float mv;
      if constexpr (MES == 4) mv = __builtin_bit_cast(float, mraw);
      else if constexpr (MES == 2)
        mv = mask_f16 ? (float)__builtin_bit_cast(f16_t, (unsigned short)mraw) : __builtin_bit_cast(float, mraw << 16);
      else mv = (mraw & 0xff) ? 0.0f : -__builtin_inff();
      mv = key_ok ? mv * inv_scale : -__builtin_inff();
      *reinterpret_cast<unsigned*>(smem + slot * KS_BYTES + KS_MK + 4 * mk_row) = pack_split<T>(mv);
    }
  };

  // ---- per-lane LDS read offsets ---------------------------------------------------------------------------
  int qa[2], ka[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const int c = hs * 4 + 2 * g + s;            // 16-byte chunk of the pair line: head hs, d = 16 g + 8 s
    qa[s] = QS_BASE + QS_Q + qrow * 128 + ((c ^ ((qrow >> 1) & 7)) << 4);
    ka[s] = KS_K + x * 128 + ((c ^ ((x >> 1) & 7)) << 4);
  }
  const int la = QS_BASE + QS_LSE + (hs * 128 + qrow) * 4;

  const unsigned ones_g = g == 0 ? ones_word<T>() : 0u;
  const frag ones_aug = make_aug<T>(ones_g, 0u);

  // query-side state of the row being worked on
  frag qc[2], doc[2];
  u32x4 dB4 = {0u, 0u, 0u, 0u}, mk4 = {0u, 0u, 0u, 0u};   // carrier fragments: only the first word ever changes
  float l2p;
  auto read_query_side = [&](int slot) {
    const unsigned char* sb = smem + slot * QS_BYTES;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      qc[s] = lds_frag<T>(sb + qa[s]);
      doc[s] = lds_frag<T>(sb + qa[s] + (QS_DO - QS_Q));
    }
    const float lraw = *reinterpret_cast<const float*>(sb + la);
    const float draw = *reinterpret_cast<const float*>(sb + la + (QS_DL - QS_LSE));
    l2p = (qi < S && lraw != -__builtin_inff()) ? lraw * MF_LOG2E : __builtin_inff();
    dB4[0] = g == 0 ? pack_split<T>(-draw) : 0u;
  };
  // One tile step: the matrix pipe computes the scores / scale (seeded with the bias, mask through the carrier) and
  // dP - delta of key tile `tn` of the row in `slot` into (zn, dpn) while the vector ALU turns the finished tile
  // (zc, dpc) into probabilities and adds P (dP - delta) to patch `tc`.  Six products, six runs of eight
  // independent vector-ALU instructions, one run behind each product; the empty statements keep every run where
  // it is written.  COMPUTE = false: products only (the very first tile).
  using MM = RingMma<T>;
  auto tile_step = [&](int slot, int tn, f32x16& zn, f32x16& dpn, auto compute_c, int tc, f32x16& zc, f32x16& dpc, float l2, auto&& hook) {
    constexpr bool COMPUTE = decltype(compute_c)::value;
    const unsigned char* sb = smem + slot * KS_BYTES + tn * 4096;
    const unsigned mw = *reinterpret_cast<const unsigned*>(smem + slot * KS_BYTES + KS_MK + (32 * tn + x) * 4);
    const frag k0 = lds_frag<T>(sb + ka[0]), k1 = lds_frag<T>(sb + ka[1]);
    const frag v0 = lds_frag<T>(sb + ka[0] + (KS_V - KS_K)), v1 = lds_frag<T>(sb + ka[1] + (KS_V - KS_K));
    mk4[0] = g == 0 ? mw : 0u;
    const frag mfrag = __builtin_bit_cast(frag, mk4), dB = __builtin_bit_cast(frag, dB4);
    auto st_arg = [&](const int o) {
      if constexpr (COMPUTE) {
#pragma unroll
        for (int i = 8 * o; i < 8 * o + 8; ++i) zc[i] = __builtin_fmaf(zc[i], cexp, -l2);
        asm volatile("" : "+v"(zc));
      }
    };
    auto st_exp = [&](const int o) {
      if constexpr (COMPUTE) {
#pragma unroll
        for (int i = 8 * o; i < 8 * o + 8; ++i) zc[i] = fast_exp2(zc[i]);
        asm volatile("" : "+v"(zc));
      }
    };
    auto st_acc = [&](const int o) {
      if constexpr (COMPUTE) {
#pragma unroll
        for (int i = 8 * o; i < 8 * o + 8; ++i) acc[tc][i] = __builtin_fmaf(zc[i], dpc[i], acc[tc][i]);
        asm volatile("" : "+v"(acc[tc]));
      }
    };
#ifdef MF_RING_KO_MFMA   // timing experiment, wrong results
    asm volatile("" : "=v"(zn), "=v"(dpn) : "v"(mfrag), "v"(dB), "v"(k0), "v"(k1), "v"(v0), "v"(v1));
    st_arg(0); hook(0); st_exp(0); hook(1); st_acc(0); hook(2); st_arg(1); hook(3); st_exp(1); hook(4); st_acc(1); hook(5);
#else
    MM::set(zn, mfrag, ones_aug, bz[tn]);
    st_arg(0);
    hook(0);
    MM::zero(dpn, ones_aug, dB);
    st_exp(0);
    hook(1);
    MM::acc(zn, k0, qc[0]);
    st_acc(0);
    hook(2);
    MM::acc(dpn, v0, doc[0]);
    st_arg(1);
    hook(3);
    MM::acc(zn, k1, qc[1]);
    st_exp(1);
    hook(4);
    MM::acc(dpn, v1, doc[1]);
    st_acc(1);
    hook(5);
#endif
  };
#ifdef MF_RING_KO_VALU    // timing experiment, wrong results
  using yes = std::integral_constant<bool, false>;
#else
  using yes = std::integral_constant<bool, true>;
#endif
  using no = std::integral_constant<bool, false>;

  // ---- prologue: rows 0, 1, 2 requested, mask of row 0 published, products of (row 0, tile 0) --------------
  f32x16 zA, dpA, zB, dpB;
  auto no_hook = [](int) {};
  issue_mask();
  issue_row(0);
  issue_row(1);
  wait_vm<2 * ROW_OPS>();
  publish_mask(0);
  issue_mask();
  issue_part(2, 0); issue_part(2, 1); issue_part(2, 2);      // the rest of row 2 follows in the first row step
  barrier_keep_vm<ROW_OPS + 1 + 3>();
  read_query_side(0);
  tile_step(0, 0, zA, dpA, no(), 0, zB, dpB, 0.0f, no_hook);
  asm volatile("s_nop 15\n s_nop 15" : "+v"(zA), "+v"(dpA));   // no vector-ALU run sits between these products and their first use

#ifdef MF_TIMELINE
  // development aid: shader-clock stamps of rows 20..35 of the chosen work-group, logged in LDS behind the ring
  unsigned* tlog = reinterpret_cast<unsigned*>(smem + RING_BYTES);
  int tl_row = 0;
#define MF_RTL(k)                                                                                      \
  do {                                                                                                 \
    if (p.tl && (int)blockIdx.x == p.tl_block && l == 0 && tl_row >= 20 && tl_row < 36)                \
      tlog[((tl_row - 20) * 8 + wv) * 8 + (k)] = (unsigned)__builtin_readcyclecounter();               \
  } while (0)
#else
#define MF_RTL(k) do { } while (0)
#endif
  // One row step.  SL = ring slot of row n; the barrier in the middle publishes row n + 1 (slot NS) and frees SL.
  auto row_step = [&](auto slot_c) {
    constexpr int SL = decltype(slot_c)::value, NS = (SL + 1) % RING, PS = (SL + 2) % RING;
    float l2 = l2p;
    pin(l2);
    MF_RTL(0);
    // parts 3..6 of row n + 2 (its slot is the one before SL), one behind every other product
    tile_step(SL, 1, zB, dpB, yes(), 0, zA, dpA, l2, [&](int stage) {
#ifndef MF_RING_KO_DMA
      if (stage == 0) issue_part(PS, 3);
      if (stage == 1) issue_part(PS, 4);
      if (stage == 3) issue_part(PS, 5);
      if (stage == 5) issue_part(PS, 6);
#endif
    });
    MF_RTL(1);
    wait_vm<ROW_OPS>();                          // row n + 1 and its mask have arrived, row n + 2 still travels
    MF_RTL(2);
    publish_mask(NS);
    barrier_keep_vm<ROW_OPS>();
    MF_RTL(3);
#ifndef MF_RING_KO_DMA     // timing experiment, wrong results
    issue_mask();                                // row n + 2
#endif
    pin(l2);                                     // the second tile's vector-ALU work stays behind the barrier
    MF_RTL(4);
    read_query_side(NS);
    // parts 0..2 of row n + 3 go into the slot the barrier has just freed
    tile_step(NS, 0, zA, dpA, yes(), 1, zB, dpB, l2, [&](int stage) {
#ifndef MF_RING_KO_DMA
      if (stage == 0) issue_part(SL, 0);
      if (stage == 2) issue_part(SL, 1);
      if (stage == 4) issue_part(SL, 2);
#endif
    });
    MF_RTL(5);
#ifdef MF_TIMELINE
    ++tl_row;
#endif
  };
  {
    int r = 0;
    for (; r + 2 < R; r += 3) {
      row_step(std::integral_constant<int, 0>());
      row_step(std::integral_constant<int, 1>());
      row_step(std::integral_constant<int, 2>());
    }
    if (r < R) {
      row_step(std::integral_constant<int, 0>());
      if (r + 1 < R) row_step(std::integral_constant<int, 1>());
    }
  }
  // The last step's products belong to no row, and the seeds are dead behind their last product as far as the
  // compiler knows: keep all of them allocated until the matrix pipe has drained, or a register an MFMA in flight
  // reads or writes is handed to the store code below.
  asm volatile("s_nop 15\n s_nop 15" : "+v"(zA), "+v"(dpA), "+v"(bz[0]), "+v"(bz[1]));
#ifdef MF_TIMELINE
  __syncthreads();
  if (p.tl && (int)blockIdx.x == p.tl_block)
    for (int i = t512; i < 16 * 8 * 8; i += 512) p.tl[i] = tlog[i];
#endif
  wait_vm<0>();                                  // nothing of this work-group may still travel towards its LDS

  // ---- store the patch: lane (x = query, g) owns 16 contiguous keys per tile ---------------------
  // chunk 0 writes into dbias itself, the others into the partial buffers that the reduction adds to it
  float* dst = (chunk > 0 ? p.dbias_part + (int64_t)(chunk - 1) * p.B * p.H * S * S : p.dbias) +
               ((int64_t)b * p.H + h) * S * S;
  if (qi < S) {
    const bool vec = (S & 3) == 0;     // rows of the gradient are 16-byte aligned
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const int j = (jt0 + t) * 32 + 16 * g + 4 * c4;
        float* d4 = dst + (int64_t)qi * S + j;
        if (vec && j + 3 < S) {
          f32x4 v = {acc[t][4 * c4], acc[t][4 * c4 + 1], acc[t][4 * c4 + 2], acc[t][4 * c4 + 3]};
          *reinterpret_cast<f32x4*>(d4) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (j + e < S) d4[e] = acc[t][4 * c4 + e];
        }
      }
  }
}

// True when the ring kernel handles the problem: 16-bit elements, D = 32 exactly, an even head count with the
// two heads of a pair side by side in memory (whole 128-byte lines), per-lane byte offsets that fit 32 bits.
bool evo_bwd_dbias_ring_supported(const EvoParams& p) {
  if (p.dtype != MF_BF16 && p.dtype != MF_F16) return false;
  if (p.D != 32 || (p.H & 1)) return false;
  if (p.q.sh != 32 || p.k.sh != 32 || p.v.sh != 32 || p.dO.sh != 32) return false;
  auto fits = [&](int64_t ss) { return ss > 0 && (int64_t)p.S * ss * 2 + 128 < (1LL << 31); };
  if (!(fits(p.q.ss) && fits(p.k.ss) && fits(p.v.ss) && fits(p.dO.ss))) return false;
  if ((int64_t)p.S * 8 + 4 >= (1LL << 31)) return false;
  if (p.mask_sj < 0 || (int64_t)p.S * p.mask_sj * 4 >= (1LL << 31)) return false;
  return true;
}

template <typename T, int MES> static hipError_t launch_ring_t(const EvoParams& p, hipStream_t stream) {
  const int NT = (p.S + 31) / 32;
  const int IB = (p.S + 127) / 128, JB = (NT + 1) / 2;
#ifdef MF_TIMELINE
  const size_t smem = (size_t)RING_BYTES + 4096;
#else
  const size_t smem = (size_t)RING_BYTES;
#endif
  const long long blocks = ((long long)p.B * (p.H / 2) * p.n_chunks * IB * JB + 7) / 8 * 8;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kern = evo_bwd_dbias_ring_kernel<T, MES>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(512), smem, stream, p, IB, JB);
  return hipGetLastError();
}
template <typename T> static hipError_t launch_ring_m(const EvoParams& p, hipStream_t stream) {
  switch (p.mask_dtype) {
    case MF_F32: return launch_ring_t<T, 4>(p, stream);
    case MF_F16: case MF_BF16: return launch_ring_t<T, 2>(p, stream);
    default: return launch_ring_t<T, 1>(p, stream);
  }
}

hipError_t launch_evo_bwd_dbias_ring(const EvoParams& p, hipStream_t stream) {
  switch (p.dtype) {
    case MF_BF16: return launch_ring_m<bf16_t>(p, stream);
    case MF_F16: return launch_ring_m<f16_t>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

#undef MF_SB
#undef MF_RTL

}  // namespace mf
