// LayerNorm -> SwiGLU backward, first kernel: recompute the pre-activation U = LN(x) W', turn the incoming
// gradient of h into dU = [da, dg] (fused_transition.py:44-47) and, in the same pass, use dU for everything that
// needs it, so that dU itself (M x N elements, eight times the size of x) never reaches HBM:
//   * the weight-gradient partials G = x_hat^T dU and s = colsum(dU);
//   * each column block's share of dU W^T, [rows, K] in the element type of x (PARTS form; W as stored).  The dx
//     kernel below adds the N / 256 shares, multiplies by gamma in fp32 and applies the LayerNorm backward.
// (With PARTS = false the kernel writes dU instead and the general dx kernel reads it back.)
//
// A work-group has eight wavefronts on a block of 32 rows and 128 value + 128 gate columns:
//  * wavefronts 0-3 ("producers") are the forward kernel's column-stationary wavefronts: each keeps its 32 value
//    and 32 gate columns of W'^T in registers, recomputes U^T for the row block, applies the SwiGLU derivative
//    and leaves da / dg as two row-major 32 x 32 tiles in LDS;
//  * wavefronts 4-7 ("consumers") take the tiles one iteration later.  Through transposing LDS reads consumer
//    w - 4 uses the two tiles of producer w - 4 as the B operand of G[k, n] += x_hat^T[k, m] dU[m, n]
//    (x_hat: the normalised rows, staged beside the raw ones) and adds those tiles' column sums; with plain row
//    reads of all four producers' tiles it forms dy^T[k, m] = sum_n W[k, n] dU[m, n] for k tile w - 4, the W
//    fragments coming from registers or from a private LDS slot per lane.
// One producer and one consumer share a SIMD, so that the matrix-pipe and LDS work of the second runs in issue
// slots the first (bound by the vector ALU: the activation) leaves empty.
// Row blocks are dealt round-robin to gridDim.x work-groups per column block; work-group (bx, by) writes range bx
// of the partial sums, which the usual reduce / finalize kernels consume.
#pragma once

namespace mf {

template <typename T, int KP, bool PARTS>
__global__ void __launch_bounds__(512, 1) ln_swiglu_bwd_fused_kernel(const LnParams p) {
  static_assert(sizeof(T) == 2 && KP <= 128 && KP >= 32, "16-bit element types, 32 <= padded K <= 128");
  using L = LnLayout<T, KP>;
  using frag = frag_t<T>;
  constexpr int KS = KP / 16, CPR = KP / 8, KT = KP / 32;
  constexpr int RB = 32;
  // normalised rows are read with transposing reads (four consecutive rows per 16 lanes): rows 8 banks apart
  constexpr int XHSTR = (L::XSTR * (int)sizeof(T) / 4) % 64 == 4 ? L::XSTR + 8 : L::XSTR;
  constexpr int WLDS = KP > 64 ? 15 : 8;            // PARTS: W fragments per consumer kept in LDS
  constexpr int OSTR = 32 + 8;                      // row stride of a 32-column tile (elements)
  constexpr int TILE = 32 * OSTR;                   // one da or dg tile
  constexpr int PSET = 4 * TILE + 32;               // tiles of one producer: [2 buffers][da, dg], then 64 bytes that
                                                    // spread the four producers over all banks for the flush

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* Xs = reinterpret_cast<T*>(smem_raw);                          // [2][RB][XSTR]  raw rows
  T* Xh = Xs + 2 * RB * L::XSTR;                                   // [3][RB][XHSTR]  normalised rows
  float* meanL = reinterpret_cast<float*>(Xh + 3 * RB * XHSTR);    // [2][RB]
  float* rstdL = meanL + 2 * RB;                                   // [2][RB]
  float* csL = rstdL + 2 * RB;                                     // [4 * 2 * 32]
  float* bpL = csL + 4 * 2 * 32;
  T* Ot = reinterpret_cast<T*>(bpL + 4 * 2 * 32);                  // [4 producers][2 buffers][da, dg][32][OSTR]
  T* Dh = Ot + 4 * PSET;                                           // [4 producers][32][OSTR] incoming gradient
  T* Wl = Dh + 4 * TILE;                                           // PARTS: [4 consumers][WLDS][64 lanes][8] W fragments

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, x = l & 31, g = l >> 5;
  const bool producer = w < 4;
  const int pw = w & 3;                                            // producer index (own, or the one consumed)
  const int Nhalf = p.N / 2;
  const int base = (blockIdx.y * 4 + pw) * 32;                     // first value column of this producer
  const T* Wt = reinterpret_cast<const T*>(p.Wt);
  const T* X = reinterpret_cast<const T*>(p.x);
  T* Op = Ot + pw * PSET;

  // ---- producers: W'^T slices (value tile, gate tile) into registers through LDS, as in the forward -------
  frag af[2][KS];
  {
    T* Wst = Ot;                                                   // [128][XSTR] staging, aliases the tiles
    constexpr int WITEMS = 128 * CPR;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      for (int item = tid; item < WITEMS; item += 512) {
        const int r = item / CPR, dc = item % CPR;                 // staged row: producer r / 32, lane row r % 32
        const int xx = r & 31, wq = r >> 5;
        const int gm = (xx >> 2) & 1, rr = 4 * (xx >> 3) + (xx & 3);
        const int b2 = (blockIdx.y * 4 + wq) * 32;
        const int col = ln_col<2, LN_ACT_SWIGLU>(t, gm, rr, b2, Nhalf);
        const bool ok = ln_col_ok<2, LN_ACT_SWIGLU>(t, gm, rr, b2, p.N, Nhalf);
        st8<T>(Wst + r * L::XSTR + 8 * dc, ok ? ld8<T>(Wt + (int64_t)col * KP + 8 * dc) : frag_zero<T>());
      }
      __syncthreads();
      if (producer) {
#pragma unroll
        for (int s = 0; s < KS; ++s) af[t][s] = ld8<T>(Wst + (pw * 32 + x) * L::XSTR + (KP / 2) * g + 8 * s);
      }
      __syncthreads();
    }
  }
  for (int i = tid; i < 4 * 2 * 32; i += 512) {
    const int rr = i & 15, gg = (i >> 4) & 1, t = (i >> 5) & 1, wn2 = i >> 6;
    const int b2 = (blockIdx.y * 4 + wn2) * 32;
    const int col = ln_col<2, LN_ACT_SWIGLU>(t, gg, rr, b2, Nhalf);
    const bool ok = ln_col_ok<2, LN_ACT_SWIGLU>(t, gg, rr, b2, p.N, Nhalf);
    csL[i] = ok ? p.colsum[col] : 0.0f;
    bpL[i] = ok ? p.bprime[col] : 0.0f;
  }

  // ---- staging of a row block by all 512 threads: raw rows, the forward's row statistics, normalised rows ------
  static_assert(RB * CPR <= 512, "one staged chunk per thread");
  const bool stager = tid < RB * CPR;
  const int srow = (stager ? tid : 0) / CPR, sdc = tid % CPR;
  frag xr = frag_zero<T>();
  float xmu = 0.0f, xrs = 0.0f;
  auto fetch = [&](int64_t rb) {
    int64_t m = rb * RB + srow;
    m = m < p.M ? m : p.M - 1;
    xr = ld8<T>(X + m * p.K + (8 * sdc < p.K ? 8 * sdc : 0));
    xmu = p.mean[m];
    xrs = p.rstd[m];
  };
  auto stash = [&](int64_t rb, int buf, int hbuf) {
    if (stager) {                                                  // whole wavefronts: CPR divides 64
      const int64_t m = rb * RB + srow;
      const bool live = m < p.M && 8 * sdc < p.K;
      const frag xv = live ? xr : frag_zero<T>();
      st8<T>(Xs + (buf * RB + srow) * L::XSTR + 8 * sdc, xv);
      if (sdc == 0) {
        meanL[buf * RB + srow] = xmu;
        rstdL[buf * RB + srow] = xrs;
      }
      const float rl = live ? xrs : 0.0f;                          // rows / columns past the end contribute nothing
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (to_f(xv[e]) - xmu) * rl;
      st8<T>(Xh + (hbuf * RB + srow) * XHSTR + 8 * sdc, cvt8<T>(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]));
    }
  };

  // producers: incoming gradient of the block, 4 lanes per row (32 columns = 4 chunks), 16 rows per instruction
  frag dpre[2];
  auto fetch_dh = [&](int64_t rb) {
    const T* dsrc = reinterpret_cast<const T*>(p.dout);
    const int ch = l & 3, r0 = l >> 2;
    const int col = base + 8 * ch < Nhalf ? base + 8 * ch : 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      int64_t mm = rb * RB + r0 + 16 * j;
      mm = mm < p.M ? mm : p.M - 1;
      dpre[j] = ld8<T>(dsrc + mm * Nhalf + col);
    }
  };
  // consumers: flush of row block rbx to dU.  Consumer w - 4 takes rows 8 (w - 4) .. + 7 of all four producers'
  // tiles, so that 16 lanes write 256 contiguous bytes of a row (lane l: row l >> 4 (+ 4), chunk l & 15 of the
  // work-group's 128 value or gate columns)
  auto flush = [&](int64_t rbx, int fb) {
    T* du = reinterpret_cast<T*>(p.du);
    const int c16 = l & 15, pp = c16 >> 2, ch = c16 & 3;
    const T* tiles = Ot + pp * PSET + fb * (2 * TILE);
    const int colv = blockIdx.y * 128 + 8 * c16;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = 8 * pw + (l >> 4) + 4 * j;
      const int64_t mm = rbx * RB + row;
      const frag va = ld8<T>(tiles + row * OSTR + 8 * ch);
      const frag vg = ld8<T>(tiles + TILE + row * OSTR + 8 * ch);
      if (mm < p.M && colv < Nhalf) {
        st8<T>(du + mm * p.N + colv, va);
        st8<T>(du + mm * p.N + Nhalf + colv, vg);
      }
    }
  };

  const int64_t nrb = (p.M + RB - 1) / RB;
  const int64_t Gx = gridDim.x;
  int64_t rb = blockIdx.x;
  if (rb < nrb) { fetch(rb); stash(rb, 0, 0); }
  if (rb + Gx < nrb) fetch(rb + Gx);

  // The two roles run separate loops with the same number of barriers (the role is uniform per wavefront), so
  // that each role's registers (resident weights / gradient accumulators) are only live in its own loop.
  __syncthreads();                                                 // column constants visible to the producers
  if (producer) {
    // column constants of the wavefront's 32 value and 32 gate columns, resident for the whole loop
    const float* csw = csL + pw * 64 + 16 * g;
    const float* bpw = bpL + pw * 64 + 16 * g;
    float csr[2][16], bpr[2][16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { csr[0][r] = csw[r]; csr[1][r] = csw[32 + r]; bpr[0][r] = bpw[r]; bpr[1][r] = bpw[32 + r]; }
    if (rb < nrb) fetch_dh(rb);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0) once: the resident weights were loaded above
    int it = 0;
    for (; rb < nrb; rb += Gx, ++it) {
      const int buf = it & 1;
      barrier_keep_vm<63>();                                      // LDS hand-over: rows of this block, tiles of the last
      // incoming gradient through the wavefront's LDS tile (one row per lane, 16 contiguous columns per half):
      // written here and read back after the products — an LDS read queued right behind the wavefront's own
      // write stalls the wavefront for long
      T* dtile = Dh + pw * TILE;
      {
        const int ch = l & 3, r0 = l >> 2;
        st8<T>(dtile + r0 * OSTR + 8 * ch, dpre[0]);
        st8<T>(dtile + (r0 + 16) * OSTR + 8 * ch, dpre[1]);
      }
      const T* xt = Xs + (buf * RB + x) * L::XSTR;
      f32x16 acc[2] = {acc_zero(), acc_zero()};
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const frag bfx = ld8<T>(xt + (KP / 2) * g + 8 * s);
        acc[0] = mma(af[0][s], bfx, acc[0]);
        acc[1] = mma(af[1][s], bfx, acc[1]);
      }
      const float mu = meanL[buf * RB + x], rs = rstdL[buf * RB + x];
      const frag dh0 = ld8<T>(dtile + x * OSTR + 16 * g), dh1 = ld8<T>(dtile + x * OSTR + 16 * g + 8);
      stash(rb + Gx, buf ^ 1, (it + 1) % 3);
      if (rb + 2 * Gx < nrb) fetch(rb + 2 * Gx);
      if (rb + Gx < nrb) fetch_dh(rb + Gx);
      const int64_t m = rb * RB + x;
      const float c0 = -rs * mu;
      float da[16], dg[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float a = __builtin_fmaf(acc[0][r], rs, __builtin_fmaf(c0, csr[0][r], bpr[0][r]));
        const float gt = __builtin_fmaf(acc[1][r], rs, __builtin_fmaf(c0, csr[1][r], bpr[1][r]));
        const float dhv = m < p.M ? to_f(r < 8 ? dh0[r & 7] : dh1[r & 7]) : 0.0f;   // rows past the end: zero gradient
        const float sg = sigmoidf_fast(gt);
        const float silu = gt * sg;
        da[r] = dhv * silu;
        dg[r] = dhv * a * (sg + silu * (1.0f - sg));
      }
      T* t0 = Op + buf * (2 * TILE) + x * OSTR + 16 * g;
      st8<T>(t0, cvt8<T>(da[0], da[1], da[2], da[3], da[4], da[5], da[6], da[7]));
      st8<T>(t0 + 8, cvt8<T>(da[8], da[9], da[10], da[11], da[12], da[13], da[14], da[15]));
      st8<T>(t0 + TILE, cvt8<T>(dg[0], dg[1], dg[2], dg[3], dg[4], dg[5], dg[6], dg[7]));
      st8<T>(t0 + TILE + 8, cvt8<T>(dg[8], dg[9], dg[10], dg[11], dg[12], dg[13], dg[14], dg[15]));
    }
    barrier_keep_vm<63>();
  } else {
    // consumers: partial weight gradient of 32 value + 32 gate columns, all K rows, and the column sums
    f32x16 G[KT][2];
    float csum[2] = {0.0f, 0.0f};
#pragma unroll
    for (int a = 0; a < KT; ++a) { G[a][0] = acc_zero(); G[a][1] = acc_zero(); }
    // PARTS: rows k = 32 pw .. + 31 of W (as stored) for the work-group's 256 columns, resident as A operands of
    // dy^T[k, m] = sum_n W[k, n] dU[m, n].  Lane row x supplies k = 32 pw + 16 ((x >> 2) & 1) + 4 (x >> 3) + (x & 3),
    // so that the accumulator of lane (m, g) holds the 16 contiguous k = 32 pw + 16 g .. + 15.
    // The first WREG fragments stay in registers; the others are parked in LDS, one 16-byte slot per lane (the
    // registers do not hold all sixteen beside the weight-gradient accumulators).
    constexpr int WREG = 16 - WLDS;
    frag wgf[PARTS && WREG > 0 ? WREG : 1];
    T* wl = Wl + (pw * WLDS * 64 + l) * 8;
    if constexpr (PARTS) {
      const T* Wsrc = reinterpret_cast<const T*>(p.W);       // the weights as stored: gamma is applied to the summed shares
      const int k = 32 * pw + 16 * ((x >> 2) & 1) + 4 * (x >> 3) + (x & 3);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int pp = i >> 2, b = (i >> 1) & 1, st = i & 1;
        const int n = b * Nhalf + (blockIdx.y * 4 + pp) * 32 + 16 * st + 8 * g;
        const frag wv = k < p.K ? ld8<T>(Wsrc + (int64_t)k * p.N + n) : frag_zero<T>();
        if (i < WREG) wgf[i] = wv; else st8<T>(wl + (i - WREG) * 64 * 8, wv);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0) once, so that no wait for these loads is placed inside the loop
    }
    // One row block: the weight-gradient products of producer pw's two tiles and, with PARTS, the column block's
    // share of dU W^T for k tile pw (all four producers' tiles), in the element type of x, to
    // part[blockIdx.y][m][KP] (32 contiguous bytes per lane); the dx kernel adds the column blocks' shares.
    // The dy products form one dependent chain and are issued between the independent weight-gradient products.
    auto consume = [&](int64_t rbx, int fb, const T* xh) {
      const T* tiles = Op + fb * (2 * TILE);
      const bool dyw = PARTS && 32 * pw < KP;
      f32x16 dacc = acc_zero();
      // Eight steps (st, a): two dy products (tiles of producer a) and two weight-gradient products (k tile a) each.
      // The LDS operands of a step are requested one step ahead, into the other of two register sets; without
      // that every product would wait for a full LDS round trip.
      frag uf[2][2], wv[2][2], xf[2], bf[2][2];
      auto request = [&](int j) {
        const int st = j >> 2, a = j & 3, slot = j & 1;
        if (a == 0) {
#pragma unroll
          for (int b = 0; b < 2; ++b) bf[st][b] = TrRead<T>::read(tiles + b * TILE, OSTR, 16 * st, g, l, plain_chunk(l), x);
        }
        if (a < KT) xf[slot] = TrRead<T>::read(xh, XHSTR, 16 * st, g, l, 32 * a + plain_chunk(l), 32 * a + x);
        if constexpr (PARTS) {
          if (dyw) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
              const int i = (a * 2 + b) * 2 + st;
              uf[slot][b] = ld8<T>(Ot + a * PSET + fb * (2 * TILE) + b * TILE + x * OSTR + 16 * st + 8 * g);
              if (i >= WREG) wv[slot][b] = ld8<T>(wl + (i - WREG) * 64 * 8);
            }
          }
        }
      };
      request(0);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int st = j >> 2, a = j & 3, slot = j & 1;
        if (j + 1 < 8) request(j + 1);
        __builtin_amdgcn_sched_barrier(0);
        if (a == 0) {
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            float s = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) s += to_f(bf[st][b][e]);
            csum[b] += s;
          }
        }
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          if constexpr (PARTS) {
            if (dyw) {
              const int i = (a * 2 + b) * 2 + st;
              dacc = mma(i < WREG ? wgf[i < WREG ? i : 0] : wv[slot][b], uf[slot][b], dacc);
            }
          }
          if (a < KT) G[a < KT ? a : 0][b] = mma(xf[slot], bf[st][b], G[a < KT ? a : 0][b]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (PARTS) {
        const int64_t mm = rbx * RB + x;
        if (dyw && mm < p.M) {
          T* dst = reinterpret_cast<T*>(p.du) + ((int64_t)blockIdx.y * p.M + mm) * KP + 32 * pw + 16 * g;
          st8<T>(dst, cvt8<T>(dacc[0], dacc[1], dacc[2], dacc[3], dacc[4], dacc[5], dacc[6], dacc[7]));
          st8<T>(dst + 8, cvt8<T>(dacc[8], dacc[9], dacc[10], dacc[11], dacc[12], dacc[13], dacc[14], dacc[15]));
        }
      }
    };
    int it = 0;
    for (; rb < nrb; rb += Gx, ++it) {
      const int buf = it & 1;
      barrier_keep_vm<63>();
      stash(rb + Gx, buf ^ 1, (it + 1) % 3);
      if (rb + 2 * Gx < nrb) fetch(rb + 2 * Gx);
      if (it > 0) {
        if constexpr (!PARTS) flush(rb - Gx, buf ^ 1);
        consume(rb - Gx, buf ^ 1, Xh + ((it - 1) % 3) * RB * XHSTR);
      }
    }
    barrier_keep_vm<63>();
    if (it > 0) {
      if constexpr (!PARTS) flush(rb - Gx, (it - 1) & 1);
      consume(rb - Gx, (it - 1) & 1, Xh + ((it - 1) % 3) * RB * XHSTR);
    }

    // ---- partial sums of this work-group: range blockIdx.x --------------------------------------------------
    float* Gp = p.Gpart + (int64_t)blockIdx.x * p.K * p.N;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int n = b * Nhalf + base + x;
      const bool okn = base + x < Nhalf;
#pragma unroll
      for (int a = 0; a < KT; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int k = 32 * a + 8 * (r >> 2) + 4 * g + (r & 3);
          if (k < p.K && okn) Gp[(int64_t)k * p.N + n] = G[a][b][r];
        }
      const float s = csum[b] + __shfl_xor(csum[b], 32);
      if (g == 0 && okn) p.spart[(int64_t)blockIdx.x * p.N + n] = s;
    }
  }
}

// dx from the column blocks' shares of dy (PARTS form of the kernel above): w = sum of the NPART shares in fp32,
// then the LayerNorm backward dx = (w - x_hat mean_k(x_hat w) - mean_k(w)) rstd (+ dx_add), one 16-byte chunk of a
// row per thread, KP / 8 threads per row.  Streams x, the shares and dx once: bound by HBM.
template <typename T, int KP>
__global__ void __launch_bounds__(256) ln_bwd_dx_parts_kernel(const LnParams p, int nparts) {
  using frag = frag_t<T>;
  constexpr int CPR = KP / 8;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t m = item / CPR;
  const int dc = (int)(item % CPR);
  if (m >= p.M) return;                                            // whole rows: CPR divides 64, no partial groups
  const bool live = 8 * dc < p.K;
  const T* part = reinterpret_cast<const T*>(p.du) + m * KP + 8 * dc;
  float wv[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  for (int c = 0; c < nparts; ++c) {
    const frag pv = ld8<T>(part + (int64_t)c * p.M * KP);
#pragma unroll
    for (int e = 0; e < 8; ++e) wv[e] += to_f(pv[e]);
  }
  const frag xv = live ? ld8<T>(reinterpret_cast<const T*>(p.x) + m * p.K + 8 * dc) : frag_zero<T>();
  const frag gv = live ? ld8<T>(reinterpret_cast<const T*>(p.gamma) + 8 * dc) : frag_zero<T>();
  const float mu = p.mean[m], rs = p.rstd[m];
  float xh[8], s1 = 0.0f, s2 = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    xh[e] = live ? (to_f(xv[e]) - mu) * rs : 0.0f;
    wv[e] = live ? wv[e] * to_f(gv[e]) : 0.0f;              // the shares are dU W^T: gamma in fp32, as the reference applies it
    s1 += xh[e] * wv[e];
    s2 += wv[e];
  }
  s1 = group_sum<CPR>(s1);
  s2 = group_sum<CPR>(s2);
  const float c1 = s1 / (float)p.K, c2 = s2 / (float)p.K;
  if (live) {
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (wv[e] - (xh[e] * c1 + c2)) * rs;
    if (p.dx_add) {                                                // summed in fp32, rounded once below
      const frag rv = ld8<T>(reinterpret_cast<const T*>(p.dx_add) + m * p.K + 8 * dc);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] += to_f(rv[e]);
    }
    st8<T>(reinterpret_cast<T*>(p.dx) + m * p.K + 8 * dc, cvt8<T>(o[0], o[1], o[2], o[3], o[4], o[5], o[6], o[7]));
  }
}

template <typename T, int KP> static hipError_t launch_dx_parts_k(const LnParams& p, hipStream_t stream) {
  const int nparts = (p.N / 2) / 128;
  const int64_t items = p.M * (KP / 8);
  const int64_t blocks = (items + 255) / 256;
  if (blocks > 0x7fffffff) return hipErrorInvalidValue;
  hipLaunchKernelGGL((ln_bwd_dx_parts_kernel<T, KP>), dim3((unsigned)blocks), dim3(256), 0, stream, p, nparts);
  return hipGetLastError();
}

// Shapes the fused kernel takes: 16-bit types, 32 <= padded K <= 128, whole 128-column blocks of the value half.
template <typename T> static bool swiglu_bwd_fused_ok(const LnParams& p) {
  return sizeof(T) == 2 && p.KP >= 32 && p.KP <= 128 && (p.N / 2) % 128 == 0;
}

template <typename T, int KP, bool PARTS> static hipError_t launch_swiglu_bwd_fused_k(const LnParams& p, hipStream_t stream) {
  using L = LnLayout<T, KP>;
  const int gy = (p.N / 2) / 128;
  constexpr int XHSTR = (L::XSTR * (int)sizeof(T) / 4) % 64 == 4 ? L::XSTR + 8 : L::XSTR;      // as in the kernel
  const size_t smem = (size_t)32 * (2 * L::XSTR + 3 * XHSTR) * sizeof(T) + (size_t)4 * 32 * 4 + (size_t)2 * 4 * 2 * 32 * 4 +
                      (size_t)((4 * 2 * 2 + 4) * 32 * 40 + 4 * 32) * sizeof(T) + (PARTS ? (size_t)4 * (KP > 64 ? 15 : 8) * 64 * 16 : 0);
  const size_t wst = (size_t)128 * L::XSTR * sizeof(T);           // weight staging aliases the tiles
  static_assert(sizeof(T) == 2, "");
  if (wst > (size_t)(4 * 2 * 2 + 4) * 32 * 40 * sizeof(T)) return hipErrorInvalidValue;
  auto kern = ln_swiglu_bwd_fused_kernel<T, KP, PARTS>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)p.R, (unsigned)gy), dim3(512), smem, stream, p);
  return hipGetLastError();
}

}  // namespace mf
