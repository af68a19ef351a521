// Outer product mean (Algorithm 9 of AlphaFold 3), the contraction part of the reference's
// OuterProductMean.forward (megafold/model/megafold.py:795-823):
//
//     outer[b,i,j,d,e] = sum_s a[b,s,i,d] b[b,s,j,e]                 megafold.py:795, 807   (a, b already masked / scaled)
//     out[b,i,j,:]     = W[:, (d e)] . outer[b,i,j,(d e)] + bias      megafold.py:812, 823
//
// in ONE kernel: the [n, n, dh * dh] tensor (302 MB at n = 384, dh = 32) never exists.  With the operands as
// matrices A[(i d), s] and B[(j e), s] (s contiguous), the 32 x 32 accumulator tile of rows (i, .) and columns
// (j, .) of A B^T IS the outer block of the position pair (i, j); it is rounded to 16 bits, laid into LDS as one
// row of 1024 values per pair, and 32 such rows are then multiplied with the projection weight, which every
// wavefront keeps in registers (a quarter of the output channels times half of the 1024 products each) for all
// the pair tiles its work-group walks over.
//   work-group  = eight wavefronts, persistent over a contiguous run of pair tiles (8 rows i x 4 columns j)
//   stage 1     wavefront w: the four outer blocks (i0 + w, j0 .. j0 + 3); A rows from global memory (reloaded
//               only when i0 changes), B rows of the tile from LDS (direct loads, double buffered)
//   stage 2     wavefront (channel tile ct, half kh): out[32 pairs, 32 channels] over its 512 products; the two
//               halves meet in LDS, bias added, 32-byte runs stored
// 16-bit element types, dh = 32, 128 output channels, s <= 128 (the operands are zero padded to 128 columns).
#include "../../include/megafold_amd.h"
#include "capi_common.h"
#include "common.h"
#include <type_traits>

namespace mf {
namespace {

struct OpmParams {
  int B, n, tiles_j, tiles, per_group;
  const void* a;      // [B, n * 32, 128]
  const void* b;      // [B, n * 32, 128]
  const void* w;      // [128, 1024], column e * 32 + d (the reference's weight with d and e exchanged)
  const void* bias;   // [128] or nullptr
  void* out;          // [B, n, n, 128]
};

constexpr int OB_STRIDE = 2048 + 16;            // bytes between pair rows of the outer-block buffer
constexpr int LDS_B = 0;                        // two B tiles of 128 rows x 256 bytes
constexpr int LDS_O = 2 * 32768;                // 32 pair rows
constexpr int LDS_P = LDS_O + 32 * OB_STRIDE;   // partial sums of the second half: [4 channel tiles][64 lanes][16] fp32
constexpr int LDS_BYTES = LDS_P + 4 * 64 * 16 * 4;

__device__ __forceinline__ void dma16(unsigned voff, const void* sbase, unsigned lds) {
  asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "{m0}"(lds) : "memory");
}
template <int VM> __device__ __forceinline__ void wait_vm() {
  __builtin_amdgcn_s_waitcnt(((VM & 15) | ((VM >> 4) << 14)) | (7 << 4) | (15 << 8));
}

template <typename T>
__global__ void __launch_bounds__(512, 1) opm_fused_kernel(const OpmParams p) {
  using frag = frag_t<T>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int t512 = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(t512 >> 6);
  const int l = t512 & 63, x = l & 31, g = l >> 5;
  const int ct = wv & 3, kh = wv >> 2;
  const int n = p.n;

  const int t_begin = blockIdx.x * p.per_group;
  const int t_end = min(p.tiles, t_begin + p.per_group);
  if (t_begin >= t_end) return;

  // ---- the projection weight of this wavefront: A operands of stage 2 (rows = channels, permuted so that an
  // accumulator holds 16 consecutive channels per lane), 32 steps of 16 products, resident
  frag wf[32];
  {
    const T* wrow = reinterpret_cast<const T*>(p.w) + (int64_t)(ct * 32 + unperm32(x)) * 1024 + kh * 512 + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 32; ++ks) wf[ks] = ld8<T>(wrow + 16 * ks);
#pragma unroll
    for (int ks = 0; ks < 32; ++ks) pin(wf[ks]);
  }
  float bias_c[16];
  {
    frag b0 = frag_zero<T>(), b1 = frag_zero<T>();
    if (p.bias) {
      b0 = ld8<T>(reinterpret_cast<const T*>(p.bias) + ct * 32 + 16 * g);
      b1 = ld8<T>(reinterpret_cast<const T*>(p.bias) + ct * 32 + 16 * g + 8);
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) { bias_c[r] = (float)b0[r]; bias_c[8 + r] = (float)b1[r]; }
  }

  // ---- direct loads of a B tile: LDS row r (0..127) = row (j0 * 32 + r) of the operand, 16-byte chunk c of a row
  // at position c ^ (r & 15) (conflict-free fragment reads)
  const unsigned lds0 = (unsigned)(unsigned long)((__attribute__((address_space(3))) unsigned char*)smem);
  auto issue_b = [&](int tile, int buf) {
    const int bb = tile / (p.tiles / p.B), rem = tile % (p.tiles / p.B);
    const int j0 = (rem % p.tiles_j) * 4;
    const char* base = reinterpret_cast<const char*>(p.b) + (int64_t)bb * n * 32 * 256;
#pragma unroll
    for (int rd = 0; rd < 4; ++rd) {
      const int q = rd * 512 + t512, row = q >> 4, pos = q & 15;
      int grow = j0 * 32 + row;
      grow = grow < n * 32 ? grow : n * 32 - 1;
      dma16((unsigned)(grow * 256 + ((pos ^ (row & 15)) << 4)), base, lds0 + LDS_B + buf * 32768 + rd * 8192 + wv * 1024);
    }
  };

  unsigned char* Ob = smem + LDS_O;
  float* Pp = reinterpret_cast<float*>(smem + LDS_P);
  frag af[8];
  int cur_i0 = -1, cur_b = -1;
  issue_b(t_begin, 0);
  for (int tile = t_begin; tile < t_end; ++tile) {
    const int buf = (tile - t_begin) & 1;
    const int bb = tile / (p.tiles / p.B), rem = tile % (p.tiles / p.B);
    const int i0 = (rem / p.tiles_j) * 8, j0 = (rem % p.tiles_j) * 4;
    // ---- stage 1: A rows of row i0 + wv (B operands of the product: columns = d, permuted), once per i0
    if (i0 != cur_i0 || bb != cur_b) {
      int i = i0 + wv;
      i = i < n ? i : n - 1;
      const T* arow = reinterpret_cast<const T*>(p.a) + ((int64_t)bb * n * 32 + i * 32 + unperm32(x)) * 128 + 8 * g;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) af[ks] = ld8<T>(arow + 16 * ks);
      cur_i0 = i0; cur_b = bb;
    }
    wait_vm<0>();                                  // this tile's B rows (and the A rows) have arrived
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();                  // ... for every wavefront; the other B slot and the outer-block
    asm volatile("" ::: "memory");                 // buffer are free (their readers are past the preceding tile)
    if (tile + 1 < t_end) issue_b(tile + 1, buf ^ 1);
    const unsigned char* Bt = smem + LDS_B + buf * 32768;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      f32x16 acc = acc_zero();
      const int row = jj * 32 + x;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const frag bf = ld8<T>(reinterpret_cast<const T*>(Bt + row * 256 + (((2 * ks + g) ^ (row & 15)) << 4)));
        acc = mma(af[ks], bf, acc);                // rows = d (16 g + r in register r), columns = e
      }
      // pair row (wv * 4 + jj) of the buffer: product index e * 32 + d, 16-byte chunk q at q ^ ((q >> 4) & 3)
      unsigned char* orow = Ob + (wv * 4 + jj) * OB_STRIDE;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int q = 4 * x + 2 * g + u;
        st8<T>(reinterpret_cast<T*>(orow + ((q ^ ((q >> 4) & 3)) << 4)), acc_half<T>(acc, u));
      }
    }
    barrier_keep_vm<63>();                         // LDS hand-over only: the next B tile keeps travelling
    // ---- stage 2: out[pair, 32 channels of tile ct] over this wavefront's 512 products
    f32x16 o = acc_zero();
#pragma unroll
    for (int ks = 0; ks < 32; ++ks) {
      const int q = kh * 64 + 2 * ks + g;
      const frag of = ld8<T>(reinterpret_cast<const T*>(Ob + x * OB_STRIDE + ((q ^ ((q >> 4) & 3)) << 4)));
      o = mma(wf[ks], of, o);                      // rows = channels (16 g + r in register r), columns = pairs
    }
    if (kh == 1) {
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        f32x4 v = {o[4 * c4], o[4 * c4 + 1], o[4 * c4 + 2], o[4 * c4 + 3]};
        *reinterpret_cast<f32x4*>(Pp + ((ct * 4 + c4) * 64 + l) * 4) = v;
      }
    }
    barrier_keep_vm<63>();                         // LDS hand-over only: the next B tile keeps travelling
    if (kh == 0) {
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(Pp + ((ct * 4 + c4) * 64 + l) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[4 * c4 + e] += v[e] + bias_c[4 * c4 + e];
      }
      const int i = i0 + (x >> 2), j = j0 + (x & 3);     // lane x = pair row of the buffer
      if (i < n && j < n) {
        T* op = reinterpret_cast<T*>(p.out) + (((int64_t)bb * n + i) * n + j) * 128 + ct * 32 + 16 * g;
        st8<T>(op, acc_half<T>(o, 0));
        st8<T>(op + 8, acc_half<T>(o, 1));
      }
    }
  }
}


// ================================================================================================
// Gradient of the projection weight:  dWt[e * 32 + d, c] = sum_{b,i,j} outer[b,i,j,d,e] dOut[b,i,j,c]
// with the outer blocks recomputed tile by tile as in the forward, never stored.  The accumulators of all
// 1024 x 128 products would fill a compute unit's register file, so a work-group owns a QUARTER of the products
// (e in [8 q, 8 q + 8): 256 rows of dWt) and forms only those columns of the outer blocks:
//   stage 1   wavefronts 0-3, wavefront w: the two 32 x 32 tiles  rows d  x  columns (4 positions j, 8 values e)  of rows
//             i0 + 2 w and i0 + 2 w + 1 over the MSA rows; laid into LDS as pair rows of 256 products (e_local * 32 + d)
//   stage 2   wavefronts 4-7, wavefront (kt2, ch): dWt_q[128 products, 64 channels] += O^T dOut over the 32 pairs of the
//             tile, both operands through transposing LDS reads (rows = pairs)
// A tile's operand rows of b (32 rows of 256 bytes) and its 32 rows of dOut arrive by direct loads, double
// buffered.  Work-group (q, group) walks over a contiguous run of pair tiles and writes its sums to
// part[group][q]; opm_dw_reduce_kernel adds the groups in a fixed order.
constexpr int DW_OSTR = 512 + 32;               // bytes between pair rows of the outer-block buffer
constexpr int DW_LDS_B = 0;                     // two tiles of 32 operand rows x 256 bytes
constexpr int DW_LDS_D = 2 * 8192;              // two tiles of 32 dOut rows x 256 bytes
constexpr int DW_LDS_O = 4 * 8192;
constexpr int DW_LDS_BYTES = DW_LDS_O + 2 * 32 * DW_OSTR;   // two outer-block buffers

struct OpmDwParams {
  int B, n, tiles_j, tiles, per_group, groups;
  const void* a;      // [B, n * 32, 128]
  const void* b;      // [B, n * 32, 128]
  const void* dout;   // [B, n, n, 128]
  float* part;        // [groups][4][256][128]
  float* dwt;         // [1024][128]
};

template <typename T>
__global__ void __launch_bounds__(512, 1) opm_dw_kernel(const OpmDwParams p) {
  using frag = frag_t<T>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int t512 = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(t512 >> 6);
  const int l = t512 & 63, x = l & 31, g = l >> 5;
  const int n = p.n;
  const int q = blockIdx.x & 3, group = blockIdx.x >> 2;
  const int t_begin = group * p.per_group;
  const int t_end = min(p.tiles, t_begin + p.per_group);
  if (t_begin >= t_end) return;

  const unsigned lds0 = (unsigned)(unsigned long)((__attribute__((address_space(3))) unsigned char*)smem);
  // one direct load per thread and operand: LDS row r = t512 >> 4 (0..31), 16-byte position pos = t512 & 15 holds
  // chunk pos ^ (r & 15) of the row.  b: row (j0 + (r >> 3)) * 32 + 8 q + (r & 7); dOut: pair (i0 + (r >> 2), j0 + (r & 3))
  auto issue_b = [&](int tile, int buf) {
    const int bb = tile / (p.tiles / p.B), rem = tile % (p.tiles / p.B);
    const int j0 = (rem % p.tiles_j) * 4;
    const int r = t512 >> 4, pos = t512 & 15, chunk = (pos ^ (r & 15)) << 4;
    int j = j0 + (r >> 3);
    j = j < n ? j : n - 1;
    const char* bbase = reinterpret_cast<const char*>(p.b) + (int64_t)bb * n * 32 * 256;
    dma16((unsigned)((j * 32 + 8 * q + (r & 7)) * 256 + chunk), bbase, lds0 + DW_LDS_B + buf * 8192 + wv * 1024);
  };
  auto issue_d = [&](int tile, int buf) {
    const int bb = tile / (p.tiles / p.B), rem = tile % (p.tiles / p.B);
    const int i0 = (rem / p.tiles_j) * 8, j0 = (rem % p.tiles_j) * 4;
    const int r = t512 >> 4, pos = t512 & 15, chunk = (pos ^ (r & 15)) << 4;
    int i = i0 + (r >> 2), jd = j0 + (r & 3);
    i = i < n ? i : n - 1;
    jd = jd < n ? jd : n - 1;
    const char* dbase = reinterpret_cast<const char*>(p.dout) + (int64_t)bb * n * n * 256;
    dma16((unsigned)((i * n + jd) * 256 + chunk), dbase, lds0 + DW_LDS_D + buf * 8192 + wv * 1024);
  };

  // Roles: wavefronts 0-3 form the outer blocks (wavefront w: rows i0 + 2 w and i0 + 2 w + 1), wavefronts 4-7 contract
  // them with dOut (wavefront (kt2, ch): 128 products x 64 channels in registers).  Between two barriers the second
  // group works on tile t while the first prepares tile t + 1 in the other outer-block buffer.  Separate loops with the
  // same barriers and direct loads, so that each role's registers are only live in its own loop.
  const int cw = wv & 3, kt2 = cw & 1, ch = cw >> 1;
  auto run = [&](auto role) {
    constexpr bool A = decltype(role)::value;      // true: stage 1 wavefront
    frag af[A ? 2 : 1][8];
    f32x16 acc[4][2];
    if constexpr (!A) {
#pragma unroll
      for (int a = 0; a < 4; ++a) { acc[a][0] = acc_zero(); acc[a][1] = acc_zero(); }
    }
    int cur_i0 = -1, cur_b = -1;
    auto stage1 = [&](int tile, int bbuf, int ob) {
      if constexpr (A) {
        const int bb = tile / (p.tiles / p.B), rem = tile % (p.tiles / p.B);
        const int i0 = (rem / p.tiles_j) * 8, j0 = (rem % p.tiles_j) * 4;
        if (i0 != cur_i0 || bb != cur_b) {         // rows d of the two positions (columns of the blocks: permuted)
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            int i = i0 + 2 * cw + u;
            i = i < n ? i : n - 1;
            const T* arow = reinterpret_cast<const T*>(p.a) + ((int64_t)bb * n * 32 + i * 32 + unperm32(x)) * 128 + 8 * g;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) af[u][ks] = ld8<T>(arow + 16 * ks);
          }
          cur_i0 = i0; cur_b = bb;
          wait_vm<0>();
        }
        const unsigned char* Bt = smem + DW_LDS_B + bbuf * 8192;
        f32x16 o[2] = {acc_zero(), acc_zero()};
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const frag bf = ld8<T>(reinterpret_cast<const T*>(Bt + x * 256 + (((2 * ks + g) ^ (x & 15)) << 4)));
          o[0] = mma(af[0][ks], bf, o[0]);         // rows = d (16 g + r in register r), columns = (j, e_local) = lane x
          o[1] = mma(af[1][ks], bf, o[1]);
        }
        const int jj = x >> 3, el = x & 7;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int il = 2 * cw + u;
          const bool live = i0 + il < n && j0 + jj < n;        // pairs past the edge contribute nothing
          unsigned char* orow = smem + DW_LDS_O + ob * 32 * DW_OSTR + (il * 4 + jj) * DW_OSTR + (el * 32 + 16 * g) * 2;
          st8<T>(reinterpret_cast<T*>(orow), live ? acc_half<T>(o[u], 0) : frag_zero<T>());
          st8<T>(reinterpret_cast<T*>(orow + 16), live ? acc_half<T>(o[u], 1) : frag_zero<T>());
        }
      }
    };
    auto stage2 = [&](int dbuf, int ob) {
      if constexpr (!A) {
        const unsigned char* Dt = smem + DW_LDS_D + dbuf * 8192;
        const T* Ob = reinterpret_cast<const T*>(smem + DW_LDS_O + ob * 32 * DW_OSTR);
        const int a4 = (l >> 2) & 3;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          frag df[2];
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            // dOut rows are swizzled: the two 8-byte runs a lane points at lie in rows r0 and r0 + 4
            const int col = ch * 64 + u * 32 + plain_chunk(l);               // element column of the run
            const int r0 = 16 * st + 8 * g + a4, r1 = r0 + 4;
            const unsigned char* p0 = Dt + r0 * 256 + ((((col >> 3) ^ (r0 & 15)) << 4) | ((col & 4) << 1));
            const unsigned char* p1 = Dt + r1 * 256 + ((((col >> 3) ^ (r1 & 15)) << 4) | ((col & 4) << 1));
            s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p0));
            s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p1));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            s16x8 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[e + 4] = hi[e]; }
            df[u] = __builtin_bit_cast(frag, v);
          }
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            const int k0 = kt2 * 128 + a * 32;
            const frag of = TrRead<T>::read(Ob, DW_OSTR / 2, 16 * st, g, l, k0 + plain_chunk(l), k0 + x);
            acc[a][0] = mma(of, df[0], acc[a][0]);               // rows = products, columns = channels
            acc[a][1] = mma(of, df[1], acc[a][1]);
          }
        }
      }
    };

    // prologue: operand rows of the first two tiles and dOut rows of the first, then the first tile's outer blocks
    issue_b(t_begin, 0);
    issue_d(t_begin, 0);
    if (t_begin + 1 < t_end) issue_b(t_begin + 1, 1);
    wait_vm<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    stage1(t_begin, 0, 0);
    for (int tile = t_begin; tile < t_end; ++tile) {
      const int k = (tile - t_begin) & 1;
      wait_vm<0>();                                // dOut rows of this tile, operand rows of the next have arrived
      __builtin_amdgcn_s_waitcnt(0xC07F);
      __builtin_amdgcn_s_barrier();                // ... for every wavefront, and this tile's outer blocks are complete;
      asm volatile("" ::: "memory");               // the buffers requested below were last read before this barrier
      if (tile + 2 < t_end) issue_b(tile + 2, k);
      if (tile + 1 < t_end) issue_d(tile + 1, k ^ 1);
      if (tile + 1 < t_end) stage1(tile + 1, k ^ 1, k ^ 1);
      stage2(k, k);
    }
    // ---- this work-group's sums: register r of lane (x, g) is row 8 (r >> 2) + 4 g + (r & 3), column x of its tile
    if constexpr (!A) {
      float* dst = p.part + ((int64_t)group * 4 + q) * 256 * 128;
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = kt2 * 128 + a * 32 + 8 * (r >> 2) + 4 * g + (r & 3), col = ch * 64 + c * 32 + x;
            dst[row * 128 + col] = acc[a][c][r];
          }
    }
  };
  if (wv < 4) run(std::true_type{});
  else run(std::false_type{});
}

// dwt[q * 256 + row][c] = sum over the groups, in their order
__global__ void __launch_bounds__(256) opm_dw_reduce_kernel(const OpmDwParams p) {
  const int idx = blockIdx.x * 256 + threadIdx.x;          // float4 index into [1024][128]
  if (idx >= 1024 * 128 / 4) return;
  // eight independent loads at a time (a load-add chain would pay the memory latency once per group), fixed order
  f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
  const float* src = p.part + (int64_t)idx * 4;
  int gidx = 0;
  for (; gidx + 8 <= p.groups; gidx += 8) {
    f32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const f32x4*>(src + (int64_t)(gidx + u) * 1024 * 128);
#pragma unroll
    for (int u = 0; u < 8; ++u) s += v[u];
  }
  for (; gidx < p.groups; ++gidx) s += *reinterpret_cast<const f32x4*>(src + (int64_t)gidx * 1024 * 128);
  *reinterpret_cast<f32x4*>(p.dwt + (int64_t)idx * 4) = s;
}


// ================================================================================================
// Gradients of the two operands.  With o the position on the side of the result (i for da, j for db), t the
// other position, f / h the hidden indices that go with them:
//     dO[o,t,f,h]    = sum_c dOut[pair(o,t), c] wt[f * 32 + h, c]          the gradient of the outer block
//     res[(o f), s]  = sum_{t,h} dO[o,t,f,h] opnd[(t h), s]
// again without the [n, n, dh * dh] tensor: a tile of dO lives in LDS between two matrix products.
//   unit        = (batch, block of 8 positions o, half of the 32 values f); its 128 x 128 result stays in registers
//   job         = a unit and a tile of 4 positions t; a work-group walks over a contiguous run of jobs and writes one
//                 partial piece per unit it touches (at most two); opm_dab_reduce_kernel adds the pieces of a unit
//   stage A     wavefronts 0-3, wavefront w: dO rows (f_local = 4 w .. 4 w + 3) x 32 h for the 32 pairs of the tile, wt
//               resident in registers (A operand), dOut rows from LDS; laid into LDS as pair rows of 512 values
//   stage B     wavefronts 4-7, wavefront (rt2, sh): rows (4 positions o, 16 f) x 64 values s, contraction over
//               (t, h) = 128: dO rows as plain fragments, the operand rows through transposing LDS reads
// The tile's 128 operand rows and 32 dOut rows arrive by direct loads, double buffered, and so is the dO tile: between
// two barriers the work-group runs stage B of job j and stage A of job j + 1, whose chains are independent (one
// barrier per job, and each stage covers the LDS latencies of the other).
constexpr int DAB_OSTR = 1024 + 16;             // bytes between pair rows of the dO tile
constexpr int DAB_LDS_P = 0;                    // two tiles of 128 operand rows x 256 bytes
constexpr int DAB_LDS_D = 2 * 32768;            // two tiles of 32 dOut rows x 256 bytes
constexpr int DAB_LDS_O = DAB_LDS_D + 2 * 8192;
constexpr int DAB_LDS_BYTES = DAB_LDS_O + 2 * 32 * DAB_OSTR;   // two dO tiles

struct OpmDabParams {
  int B, n, tiles_t, units_per_batch, jobs, per_group, groups, transposed;
  const void* dout;   // [B, n, n, 128]
  const void* wt;     // [1024][128], row f * 32 + h
  const void* opnd;   // [B, n * 32, 128]
  float* part;        // [groups][2][128][128]
  void* res;          // [B, n * 32, 128]
};

template <typename T>
__global__ void __launch_bounds__(512, 1) opm_dab_kernel(const OpmDabParams p) {
  using frag = frag_t<T>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int t512 = threadIdx.x;
  const int wv = __builtin_amdgcn_readfirstlane(t512 >> 6);
  const int l = t512 & 63, x = l & 31, g = l >> 5;
  const int n = p.n;
  const int j_begin = blockIdx.x * p.per_group;
  const int j_end = min(p.jobs, j_begin + p.per_group);
  if (j_begin >= j_end) return;

  const unsigned lds0 = (unsigned)(unsigned long)((__attribute__((address_space(3))) unsigned char*)smem);
  auto decode = [&](int job, int& bb, int& o0, int& fh, int& t0) {
    const int unit = job / p.tiles_t;
    t0 = (job % p.tiles_t) * 4;
    bb = unit / p.units_per_batch;
    const int u = unit % p.units_per_batch;
    o0 = (u >> 1) * 8;
    fh = u & 1;
  };
  // direct loads of a job's tiles: LDS row r, 16-byte position pos holds chunk pos ^ (r & 15) of the row
  auto issue_p = [&](int job, int buf) {           // the 128 operand rows
    int bb, o0, fh, t0;
    decode(job, bb, o0, fh, t0);
    const char* pbase = reinterpret_cast<const char*>(p.opnd) + (int64_t)bb * n * 32 * 256;
#pragma unroll
    for (int rd = 0; rd < 4; ++rd) {
      const int q = rd * 512 + t512, row = q >> 4, pos = q & 15;
      int grow = t0 * 32 + row;
      grow = grow < n * 32 ? grow : n * 32 - 1;
      dma16((unsigned)(grow * 256 + ((pos ^ (row & 15)) << 4)), pbase, lds0 + DAB_LDS_P + buf * 32768 + rd * 8192 + wv * 1024);
    }
  };
  auto issue_d = [&](int job, int buf) {           // the 32 dOut rows
    int bb, o0, fh, t0;
    decode(job, bb, o0, fh, t0);
    const int r = t512 >> 4, pos = t512 & 15;
    int o = o0 + (r >> 2), t = t0 + (r & 3);
    o = o < n ? o : n - 1;
    t = t < n ? t : n - 1;
    const char* dbase = reinterpret_cast<const char*>(p.dout) + (int64_t)bb * n * n * 256;
    const int pair = p.transposed ? t * n + o : o * n + t;
    dma16((unsigned)(pair * 256 + ((pos ^ (r & 15)) << 4)), dbase, lds0 + DAB_LDS_D + buf * 8192 + wv * 1024);
  };

  // Roles: wavefronts 0-3 run stage A (wavefront w: four values f, wt resident), wavefronts 4-7 stage B (wavefront
  // (rt2, sh2): 64 rows x 64 columns of the unit's result in registers).  Larger tiles per wavefront than with all
  // eight on both stages: a third less LDS traffic, which bounds this kernel.  The two roles run separate loops with
  // the same barriers and the same direct loads, so that each role's registers are only live in its own loop.
  const int cw = wv & 3, rt2 = cw & 1, sh2 = cw >> 1;
  auto run = [&](auto role) {
    constexpr bool A = decltype(role)::value;      // true: stage A wavefront
    frag wf[A ? 4 : 1][8];
    f32x16 acc[2][2];
    if constexpr (!A) {
#pragma unroll
      for (int a = 0; a < 2; ++a) { acc[a][0] = acc_zero(); acc[a][1] = acc_zero(); }
    }
    int cur_unit = -1, cur_fh = -1, piece = 0;
    auto flush = [&](int pc) {                     // register r of lane (x, g): row 8 (r >> 2) + 4 g + (r & 3), column x
      if constexpr (!A) {
        float* dst = p.part + ((int64_t)blockIdx.x * 2 + pc) * 128 * 128;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              dst[((2 * rt2 + a) * 32 + 8 * (r >> 2) + 4 * g + (r & 3)) * 128 + sh2 * 64 + c * 32 + x] = acc[a][c][r];
      }
    };
    // stage A of a job: dO rows of the tile's 32 pairs into dO tile `ob`
    auto stage_a = [&](int job, int db, int ob) {
      if constexpr (A) {
        int bb, o0, fh, t0;
        decode(job, bb, o0, fh, t0);
        if (fh != cur_fh) {                        // rows f * 32 + h of wt for this wavefront's four values f, h permuted
          cur_fh = fh;                             // so that a register holds 16 g + r
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            const T* wrow = reinterpret_cast<const T*>(p.wt) + (int64_t)((fh * 16 + 4 * cw + a) * 32 + unperm32(x)) * 128 + 8 * g;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) wf[a][ks] = ld8<T>(wrow + 16 * ks);
          }
          wait_vm<0>();
        }
        const unsigned char* Dt = smem + DAB_LDS_D + db * 8192;
        frag df[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) df[ks] = ld8<T>(reinterpret_cast<const T*>(Dt + x * 256 + (((2 * ks + g) ^ (x & 15)) << 4)));
        const bool live = t0 + (x & 3) < n;        // pairs past the edge contribute nothing
        unsigned char* orow = smem + DAB_LDS_O + ob * 32 * DAB_OSTR + x * DAB_OSTR;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          f32x16 o[2] = {acc_zero(), acc_zero()};
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) {
            o[0] = mma(wf[2 * half][ks], df[ks], o[0]);        // rows = h (16 g + r in register r), columns = pairs
            o[1] = mma(wf[2 * half + 1][ks], df[ks], o[1]);
          }
#pragma unroll
          for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
              const int q = 4 * (4 * cw + 2 * half + a) + 2 * g + u;   // 16-byte chunk (f_local * 32 + 16 g + 8 u) / 8
              st8<T>(reinterpret_cast<T*>(orow + ((q ^ ((q >> 4) & 3)) << 4)), live ? acc_half<T>(o[a], u) : frag_zero<T>());
            }
        }
      }
    };
    // stage B of a job: its dO tile `ob` against its operand rows `pb`
    auto stage_b = [&](int pb, int ob) {
      if constexpr (!A) {
        const unsigned char* Pt = smem + DAB_LDS_P + pb * 32768;
        const unsigned char* Ob = smem + DAB_LDS_O + ob * 32 * DAB_OSTR;
        const int a4 = (l >> 2) & 3;
        const int fl = x & 15;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const int q = 4 * fl + 2 * (ks & 1) + g;
          frag of[2];
#pragma unroll
          for (int a = 0; a < 2; ++a) {
            const int ol = 2 * (2 * rt2 + a) + (x >> 4);
            of[a] = ld8<T>(reinterpret_cast<const T*>(Ob + (ol * 4 + (ks >> 1)) * DAB_OSTR + ((q ^ ((q >> 4) & 3)) << 4)));
          }
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const int col = sh2 * 64 + c * 32 + plain_chunk(l);
            const int r0 = 16 * ks + 8 * g + a4, r1 = r0 + 4;
            const unsigned char* p0 = Pt + r0 * 256 + ((((col >> 3) ^ (r0 & 15)) << 4) | ((col & 4) << 1));
            const unsigned char* p1 = Pt + r1 * 256 + ((((col >> 3) ^ (r1 & 15)) << 4) | ((col & 4) << 1));
            s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p0));
            s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p1));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            s16x8 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[e + 4] = hi[e]; }
            const frag pf = __builtin_bit_cast(frag, v);
            acc[0][c] = mma(of[0], pf, acc[0][c]);               // rows = (o, f), columns = s
            acc[1][c] = mma(of[1], pf, acc[1][c]);
          }
        }
      }
    };

    // prologue: the first job's tiles and the second job's dOut rows, then stage A of the first job
    issue_d(j_begin, 0);
    issue_p(j_begin, 0);
    if (j_begin + 1 < j_end) issue_d(j_begin + 1, 1);
    wait_vm<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    stage_a(j_begin, 0, 0);
    for (int job = j_begin; job < j_end; ++job) {
      const int k = (job - j_begin) & 1;
      const int unit = job / p.tiles_t;
      if (unit != cur_unit) {
        if (cur_unit >= 0) {
          flush(piece);
          ++piece;
          if constexpr (!A) {
#pragma unroll
            for (int a = 0; a < 2; ++a) { acc[a][0] = acc_zero(); acc[a][1] = acc_zero(); }
          }
        }
        cur_unit = unit;
      }
      wait_vm<0>();                                // operand rows of this job, dOut rows of the next have arrived
      __builtin_amdgcn_s_waitcnt(0xC07F);
      __builtin_amdgcn_s_barrier();                // ... for every wavefront, and this job's dO tile is complete; the
      asm volatile("" ::: "memory");               // buffers requested below were last read before this barrier
      if (job + 1 < j_end) issue_p(job + 1, k ^ 1);
      if (job + 2 < j_end) issue_d(job + 2, k);
      if (job + 1 < j_end) stage_a(job + 1, k ^ 1, k ^ 1);
      stage_b(k, k);
    }
    flush(piece);
  };
  if (wv < 4) run(std::true_type{});
  else run(std::false_type{});
}

// res[b][(o0 + R >> 4) * 32 + fh * 16 + (R & 15)][s] = sum of the unit's pieces, in the order of the work-groups
template <typename T>
__global__ void __launch_bounds__(256) opm_dab_reduce_kernel(const OpmDabParams p) {
  const int unit = blockIdx.x >> 4;
  const int idx = (blockIdx.x & 15) * 256 + threadIdx.x;      // float4 index into [128][128]
  const int R = idx >> 5, s4 = (idx & 31) * 4;
  const int bb = unit / p.units_per_batch, u = unit % p.units_per_batch;
  const int o = (u >> 1) * 8 + (R >> 4), f = (u & 1) * 16 + (R & 15);
  if (o >= p.n) return;
  const int jb = unit * p.tiles_t, je = jb + p.tiles_t - 1;
  f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int k = jb / p.per_group; k <= je / p.per_group; ++k) {
    const int pc = (k * p.per_group) / p.tiles_t == unit ? 0 : 1;   // piece 0 belongs to the unit of the group's first job
    sum += *reinterpret_cast<const f32x4*>(p.part + (((int64_t)k * 2 + pc) * 128 + R) * 128 + s4);
  }
  T* dst = reinterpret_cast<T*>(p.res) + (((int64_t)bb * p.n + o) * 32 + f) * 128 + s4;
  dst[0] = (T)sum[0]; dst[1] = (T)sum[1]; dst[2] = (T)sum[2]; dst[3] = (T)sum[3];
}


// ================================================================================================
// Operands of the kernels above from the hidden projection, and the way back for the gradients.
//   pack    a[b, i*32 + d, s] = hidden[b, s, i, d] * row_scale[b, s] * pos[b, i]        (one rounding)
//           b[b, i*32 + e, s] = hidden[b, s, i, 32 + e] * pos[b, i]                      s >= S: zero (128 columns)
//   unpack  dhidden[b, s, i, d] = da[b, i*32 + d, s] * row_scale[b, s] * pos[b, i],  dhidden[b, s, i, 32 + e] = db[...] * pos
// (megafold.py:788-807: the MSA-row mask and the division by the number of rows as row_scale, the pair mask as the
// position mask on either side).  A work-group moves 8 positions x 32 MSA rows through an LDS tile.
struct OpmPackParams {
  int B, S, n, unpack;
  void* hidden; int64_t ldh;          // [B, S, n, ldh >= 64] (element stride of a position)
  const float* row_scale;             // [B, S]
  const unsigned char* pos;           // [B, n] or nullptr
  void* a; void* b;                   // [B, n * 32, 128]
};

template <typename T>
__global__ void __launch_bounds__(256) opm_pack_kernel(const OpmPackParams p) {
  __shared__ T tile[8 * 64][32 + 2];                          // [(i_local, channel)][s_local]
  const int t = threadIdx.x;
  const int s0 = blockIdx.x * 32, i0 = blockIdx.y * 8, bb = blockIdx.z;
  T* H = reinterpret_cast<T*>(p.hidden);
  T* Aop = reinterpret_cast<T*>(p.a);
  T* Bop = reinterpret_cast<T*>(p.b);
  if (!p.unpack) {
    // in: 8 threads per (s, i) row of 64 channels
    for (int item = t; item < 32 * 8 * 8; item += 256) {
      const int ch = item & 7, i_l = (item >> 3) & 7, s_l = item >> 6;
      const int sidx = s0 + s_l, i = i0 + i_l;
      frag_t<T> v = frag_zero<T>();
      float f = 0.0f;
      if (sidx < p.S && i < p.n) {
        v = ld8<T>(H + (((int64_t)bb * p.S + sidx) * p.n + i) * p.ldh + 8 * ch);
        f = p.pos ? (p.pos[(int64_t)bb * p.n + i] ? 1.0f : 0.0f) : 1.0f;
        if (ch < 4) f *= p.row_scale[(int64_t)bb * p.S + sidx];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) tile[i_l * 64 + 8 * ch + e][s_l] = (T)((float)v[e] * f);
    }
    __syncthreads();
    // out: 4 threads per operand row (32 MSA rows = 64 bytes)
    for (int item = t; item < 8 * 64 * 4; item += 256) {
      const int c4 = item & 3, row = item >> 2, i_l = row >> 6, c = row & 63;
      const int i = i0 + i_l;
      if (i < p.n) {
        frag_t<T> v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = tile[row][8 * c4 + e];
        T* dst = (c < 32 ? Aop : Bop) + (((int64_t)bb * p.n + i) * 32 + (c & 31)) * 128 + s0 + 8 * c4;
        st8<T>(dst, v);
      }
    }
  } else {
    for (int item = t; item < 8 * 64 * 4; item += 256) {
      const int c4 = item & 3, row = item >> 2, i_l = row >> 6, c = row & 63;
      const int i = i0 + i_l;
      frag_t<T> v = frag_zero<T>();
      if (i < p.n) v = ld8<T>((c < 32 ? Aop : Bop) + (((int64_t)bb * p.n + i) * 32 + (c & 31)) * 128 + s0 + 8 * c4);
#pragma unroll
      for (int e = 0; e < 8; ++e) tile[row][8 * c4 + e] = v[e];
    }
    __syncthreads();
    for (int item = t; item < 32 * 8 * 8; item += 256) {
      const int ch = item & 7, i_l = (item >> 3) & 7, s_l = item >> 6;
      const int sidx = s0 + s_l, i = i0 + i_l;
      if (sidx < p.S && i < p.n) {
        float f = p.pos ? (p.pos[(int64_t)bb * p.n + i] ? 1.0f : 0.0f) : 1.0f;
        if (ch < 4) f *= p.row_scale[(int64_t)bb * p.S + sidx];
        frag_t<T> v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (T)((float)tile[i_l * 64 + 8 * ch + e][s_l] * f);
        st8<T>(H + (((int64_t)bb * p.S + sidx) * p.n + i) * p.ldh + 8 * ch, v);
      }
    }
  }
}

}  // namespace
}  // namespace mf

using namespace mf;

extern "C" int mf_opm_fused_fwd(const void* a, const void* b, const void* w, const void* bias, void* out, int32_t B,
                                int32_t n, int32_t dtype, void* stream) {
  clear_error();
  if (!a || !b || !w || !out) return fail(MF_ERR_NULL, "a, b, w or out is NULL");
  if (!aligned16(a) || !aligned16(b) || !aligned16(w) || !aligned16(out)) return fail(MF_ERR_ALIGN, "operands must be 16-byte aligned");
  if (B <= 0 || n <= 0) return fail(MF_ERR_SHAPE, "B, n must be positive (got %d, %d)", B, n);
  if ((int64_t)n * 32 * 256 >= (1LL << 31)) return fail(MF_ERR_SHAPE, "n=%d too large", n);
  if (dtype != MF_DTYPE_F16 && dtype != MF_DTYPE_BF16) return fail(MF_ERR_DTYPE, "dtype %d unsupported: f16 / bf16", dtype);
  OpmParams p{};
  p.B = B; p.n = n;
  p.tiles_j = (n + 3) / 4;
  const int64_t tiles = (int64_t)B * ((n + 7) / 8) * p.tiles_j;
  if (tiles > 0x7fffffffLL) return fail(MF_ERR_SHAPE, "too many pair tiles");
  p.tiles = (int)tiles;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  p.per_group = (int)((tiles + cus - 1) / cus);
  const int groups = (int)((tiles + p.per_group - 1) / p.per_group);
  p.a = a; p.b = b; p.w = w; p.bias = bias; p.out = out;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kern) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)groups), dim3(512), LDS_BYTES, s, p);
    return hipGetLastError();
  };
  return (int)(dtype == MF_DTYPE_BF16 ? launch(opm_fused_kernel<bf16_t>) : launch(opm_fused_kernel<f16_t>));
}

static int opm_dw_groups() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  return cus >= 4 ? cus / 4 : 1;
}

extern "C" uint64_t mf_opm_dw_workspace_bytes(int32_t B, int32_t n) {
  if (B <= 0 || n <= 0) return 0;
  return (uint64_t)opm_dw_groups() * 1024 * 128 * 4;
}

extern "C" int mf_opm_dw(const void* a, const void* b, const void* dout, float* dwt, void* workspace, uint64_t workspace_bytes,
                         int32_t B, int32_t n, int32_t dtype, void* stream) {
  clear_error();
  if (!a || !b || !dout || !dwt || !workspace) return fail(MF_ERR_NULL, "a, b, dout, dwt or workspace is NULL");
  if (!aligned16(a) || !aligned16(b) || !aligned16(dout) || !aligned16(dwt) || !aligned16(workspace))
    return fail(MF_ERR_ALIGN, "operands must be 16-byte aligned");
  if (B <= 0 || n <= 0) return fail(MF_ERR_SHAPE, "B, n must be positive (got %d, %d)", B, n);
  if ((int64_t)n * 32 * 256 >= (1LL << 31) || (int64_t)n * n * 256 >= (1LL << 31)) return fail(MF_ERR_SHAPE, "n=%d too large", n);
  if (dtype != MF_DTYPE_F16 && dtype != MF_DTYPE_BF16) return fail(MF_ERR_DTYPE, "dtype %d unsupported: f16 / bf16", dtype);
  OpmDwParams p{};
  p.B = B; p.n = n;
  p.tiles_j = (n + 3) / 4;
  const int64_t tiles = (int64_t)B * ((n + 7) / 8) * p.tiles_j;
  if (tiles > 0x7fffffffLL) return fail(MF_ERR_SHAPE, "too many pair tiles");
  p.tiles = (int)tiles;
  const int max_groups = opm_dw_groups();
  p.per_group = (int)((tiles + max_groups - 1) / max_groups);
  p.groups = (int)((tiles + p.per_group - 1) / p.per_group);
  if (workspace_bytes < (uint64_t)p.groups * 1024 * 128 * 4)
    return fail(MF_ERR_WORKSPACE, "mf_opm_dw needs %llu workspace bytes, got %llu", (unsigned long long)p.groups * 1024 * 128 * 4,
                (unsigned long long)workspace_bytes);
  p.a = a; p.b = b; p.dout = dout; p.part = static_cast<float*>(workspace); p.dwt = dwt;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kern) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, DW_LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.groups * 4)), dim3(512), DW_LDS_BYTES, s, p);
    return hipGetLastError();
  };
  hipError_t e = dtype == MF_DTYPE_BF16 ? launch(opm_dw_kernel<bf16_t>) : launch(opm_dw_kernel<f16_t>);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(opm_dw_reduce_kernel, dim3(1024 * 128 / 4 / 256), dim3(256), 0, s, p);
  return (int)hipGetLastError();
}

static void opm_dab_plan(OpmDabParams& p, int B, int n) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  p.B = B; p.n = n;
  p.tiles_t = (n + 3) / 4;
  p.units_per_batch = ((n + 7) / 8) * 2;
  const int64_t jobs = (int64_t)B * p.units_per_batch * p.tiles_t;
  p.jobs = (int)jobs;
  int per = (int)((jobs + cus - 1) / cus);
  if (per > p.tiles_t) per = p.tiles_t;            // a work-group then touches at most two units
  p.per_group = per;
  p.groups = (int)((jobs + per - 1) / per);
}

extern "C" uint64_t mf_opm_dab_workspace_bytes(int32_t B, int32_t n) {
  if (B <= 0 || n <= 0 || (int64_t)B * (((int64_t)n + 7) / 8) * 2 * (((int64_t)n + 3) / 4) > 0x7fffffffLL) return 0;
  OpmDabParams p{};
  opm_dab_plan(p, B, n);
  return (uint64_t)p.groups * 2 * 128 * 128 * 4;
}

extern "C" int mf_opm_dab(const void* dout, const void* wt, const void* opnd, void* res, void* workspace, uint64_t workspace_bytes,
                          int32_t B, int32_t n, int32_t transposed, int32_t dtype, void* stream) {
  clear_error();
  if (!dout || !wt || !opnd || !res || !workspace) return fail(MF_ERR_NULL, "dout, wt, opnd, res or workspace is NULL");
  if (!aligned16(dout) || !aligned16(wt) || !aligned16(opnd) || !aligned16(res) || !aligned16(workspace))
    return fail(MF_ERR_ALIGN, "operands must be 16-byte aligned");
  if (B <= 0 || n <= 0) return fail(MF_ERR_SHAPE, "B, n must be positive (got %d, %d)", B, n);
  if ((int64_t)n * 32 * 256 >= (1LL << 31) || (int64_t)n * n * 256 >= (1LL << 31)) return fail(MF_ERR_SHAPE, "n=%d too large", n);
  if ((int64_t)B * (((int64_t)n + 7) / 8) * 2 * (((int64_t)n + 3) / 4) > 0x7fffffffLL) return fail(MF_ERR_SHAPE, "too many jobs");
  if (dtype != MF_DTYPE_F16 && dtype != MF_DTYPE_BF16) return fail(MF_ERR_DTYPE, "dtype %d unsupported: f16 / bf16", dtype);
  OpmDabParams p{};
  opm_dab_plan(p, B, n);
  const uint64_t need = (uint64_t)p.groups * 2 * 128 * 128 * 4;
  if (workspace_bytes < need)
    return fail(MF_ERR_WORKSPACE, "mf_opm_dab needs %llu workspace bytes, got %llu", (unsigned long long)need, (unsigned long long)workspace_bytes);
  p.transposed = transposed ? 1 : 0;
  p.dout = dout; p.wt = wt; p.opnd = opnd; p.part = static_cast<float*>(workspace); p.res = res;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kern, auto red) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, DAB_LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.groups), dim3(512), DAB_LDS_BYTES, s, p);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(red, dim3((unsigned)(B * p.units_per_batch * 16)), dim3(256), 0, s, p);
    return hipGetLastError();
  };
  return (int)(dtype == MF_DTYPE_BF16 ? launch(opm_dab_kernel<bf16_t>, opm_dab_reduce_kernel<bf16_t>)
                                      : launch(opm_dab_kernel<f16_t>, opm_dab_reduce_kernel<f16_t>));
}

extern "C" int mf_opm_pack(void* hidden, int64_t ldh, const float* row_scale, const void* pos, void* a, void* b, int32_t B,
                           int32_t S, int32_t n, int32_t unpack, int32_t dtype, void* stream) {
  clear_error();
  if (!hidden || !row_scale || !a || !b) return fail(MF_ERR_NULL, "hidden, row_scale, a or b is NULL");
  if (!aligned16(hidden) || !aligned16(a) || !aligned16(b)) return fail(MF_ERR_ALIGN, "operands must be 16-byte aligned");
  if (B <= 0 || n <= 0 || S <= 0 || S > 128) return fail(MF_ERR_SHAPE, "need B, n > 0 and 0 < S <= 128 (got %d, %d, %d)", B, n, S);
  if (ldh < 64 || ldh % 8 != 0) return fail(MF_ERR_STRIDE, "ldh=%lld: need a multiple of 8, at least 64", (long long)ldh);
  if (dtype != MF_DTYPE_F16 && dtype != MF_DTYPE_BF16) return fail(MF_ERR_DTYPE, "dtype %d unsupported: f16 / bf16", dtype);
  if (B > 65535 || (n + 7) / 8 > 65535) return fail(MF_ERR_SHAPE, "dimensions exceed the launch grid");
  OpmPackParams p{};
  p.B = B; p.S = S; p.n = n; p.unpack = unpack ? 1 : 0;
  p.hidden = hidden; p.ldh = ldh; p.row_scale = row_scale; p.pos = static_cast<const unsigned char*>(pos); p.a = a; p.b = b;
  // pack writes all 128 columns of the operands (zeros past S); unpack only reads the first S
  const dim3 grid((unsigned)(unpack ? (S + 31) / 32 : 4), (unsigned)((n + 7) / 8), (unsigned)B);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == MF_DTYPE_BF16) hipLaunchKernelGGL(opm_pack_kernel<bf16_t>, grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL(opm_pack_kernel<f16_t>, grid, dim3(256), 0, st, p);
  return (int)hipGetLastError();
}
