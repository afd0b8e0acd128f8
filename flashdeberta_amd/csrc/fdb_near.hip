// Near tiles of the disentangled-attention forward for gfx950: the key tiles of a query tile in
// which the bucketed relative position delta(i - j) is not constant (|i - j| < R + tile size).
//
// The position products need, per tile, the rows K_r[delta(r)] and Q_r[delta(r)] for the tile's
// contiguous range of relative positions r.  Fetching them per lane from global memory is a
// 16-byte gather across 32 rows per instruction and saturates the vector memory path.  Here the
// "expanded" tables E_K[r] = K_r[delta(r)], E_Q[r] = Q_r[delta(r)] are staged in LDS rings with
// coalesced loads: the range of a tile is 191 rows and moves down by 64 rows per tile, so each
// tile loads only its 64 new rows per table, and the MFMA A operands are plain LDS reads.
//
// Workgroup = 8 wavefronts on 128 query rows x 64 keys: wave (wr, wk) owns rows 32*wr.. and the
// key half 32*wk.. of every tile, with its own running (m, l, O); the two key halves of a row block
// are merged once at the end, and then merged with the far tiles' partial result (written by the
// far-only run of the fused kernel) when there is one.
// A wave's 32 x 32 sub-tile sees 63 relative positions, so both position products are 2 MFMA row
// blocks, private to the wave: C[i][r] = q_i . E_K[r] and P[j][r] = k_j . E_Q[r] go through a
// per-wave LDS scratch from which element (i, j) reads index r = i - j (affine addresses).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

using namespace fdb;

namespace {

constexpr int kNThreads = 512;
constexpr int kNWaves = 8;
constexpr int kRing = 256;      // rows per ring: 4 batches of 64; a tile uses 3, the 4th is being filled
constexpr int kScrStride = 68;  // elements per row of a wave's [32][64] bias scratch

template <class QT, class VT, int D>
struct NCfg {
  using ST = typename QT::scratch_t;
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLKS = D / 32;
  static constexpr int K_RS = D * QT::SZ + 16;  // LDS row strides (bytes)
  static constexpr int V_RS = D * VT::SZ + 16;
  static constexpr int K_BYTES = FDB_BN * K_RS;  // one buffer; K and V are double-buffered
  static constexpr int V_BYTES = FDB_BN * V_RS;
  static constexpr int RING_BYTES = kRing * K_RS;
  static constexpr int SCR_BYTES = kNWaves * 32 * kScrStride * (int)sizeof(ST);
  static constexpr int MERGE_BYTES = 4 * (2 + 16 * DBLKS) * 64 * 4;  // (m, l, O) of the 4 upper-half waves
  static constexpr int CPR = D * QT::SZ / 16;  // 16-byte chunks per row (K, V and ring rows alike: 16-bit types)
  static constexpr int lds_bytes(bool c2p, bool p2c) {
    const int scr = SCR_BYTES > MERGE_BYTES ? SCR_BYTES : MERGE_BYTES;
    return 2 * K_BYTES + 2 * V_BYTES + (c2p ? RING_BYTES : 0) + (p2c ? RING_BYTES : 0) + scr;
  }
};

// One 32 x 32 sub-tile after its scores (position terms included) are in sacc.
template <class VT, int D, bool MASK>
__device__ __forceinline__ void near_softmax_pv(f32x16& sacc, f32x16 (&o_acc)[D / 32], float& m_run, float& l_run,
                                                float x_scale, const char* Vs, int v_rs, int lane, int jw0, int i,
                                                int Lb, bool causal) {
  using vfrag = typename VT::frag;
  const int g = lane >> 5;
  if constexpr (MASK) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int j = jw0 + 8 * (v >> 2) + 4 * g + (v & 3);
      if (j >= Lb || (causal && j > i)) sacc[v] = -INFINITY;
    }
  }
  float mx = sacc[0];
#pragma unroll
  for (int v = 1; v < 16; ++v) mx = fmaxf(mx, sacc[v]);
  mx = wave_half_max(mx) * x_scale;  // x_scale > 0
  if (__any(mx > m_run + kLazyTau)) {
    const float m_new = (mx > m_run + kLazyTau) ? mx : m_run;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // m_run = -inf before the first visible key: 0
    l_run *= alpha;
    m_run = m_new;
#pragma unroll
    for (int d = 0; d < D / 32; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
  }
  // a wave whose key half has shown no visible key yet still has m_run = -inf
  const float off = (MASK && m_run == -INFINITY) ? 0.f : -m_run;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    f32x8 pv;
#pragma unroll
    for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[8 * c + e], x_scale, off));
    const vfrag pf = VT::from_f32(pv);
    l_run = VT::sum8(pf, l_run);
#pragma unroll
    for (int d = 0; d < D / 32; ++d) {
      const vfrag vf = VtLoad<VT>::get(Vs, v_rs, c, d, lane);
      o_acc[d] = VT::mma(vf, pf, o_acc[d]);
    }
  }
}

template <class QT, class VT, int D, bool C2P, bool P2C>
__global__ __launch_bounds__(kNThreads, 1) void fdb_near_kernel(const FdbKParams p) {
  using C = NCfg<QT, VT, D>;
  using ST = typename C::ST;
  using qfrag = typename QT::frag;
  static_assert(QT::SZ == 2 && VT::SZ == 2, "16-bit element types only");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* Ks = smem;                       // [2][64][K_RS]
  char* Vs = Ks + 2 * C::K_BYTES;        // [2][64][V_RS]
  char* EK = Vs + 2 * C::V_BYTES;        // [256][K_RS] rows K_r[delta(r)], slot = (r_hi0 - r) & 255
  char* EQ = EK + (C2P ? C::RING_BYTES : 0);
  char* scr_raw = EQ + (P2C ? C::RING_BYTES : 0);

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
  const int wr = wave & 3, wk = wave >> 2;
  int xq, h;
  block_map((int)blockIdx.x, p.grid_x, p.H, p.tiles_per_seq, p.cu == nullptr, xq, h);
  ST* scr = (ST*)scr_raw + wave * (32 * kScrStride);

  int b, m0, tok0, Lb;
  int64_t qo, ko, vo, oo;
  if (p.cu) {
    if (xq >= p.wl[0]) return;
    b = p.wl[2 + 2 * xq];
    m0 = p.wl[3 + 2 * xq];
    tok0 = p.cu[b];
    Lb = p.cu[b + 1] - tok0;
    qo = ko = vo = oo = 0;
  } else {
    b = xq / p.tiles_per_seq;
    m0 = (xq % p.tiles_per_seq) * FDB_BM;
    tok0 = p.seq_start ? min(max(p.seq_start[b], 0), p.L) : 0;
    Lb = p.seq_len ? min(max(p.seq_len[b], 0), p.L - tok0) : p.L;
    if (m0 >= Lb) return;
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; oo = b * p.o_sb;
  }
  const char* qb = p.q + (qo + (int64_t)tok0 * p.q_st + (int64_t)h * p.q_sh) * QT::SZ;
  const char* kb = p.k + (ko + (int64_t)tok0 * p.k_st + (int64_t)h * p.k_sh) * QT::SZ;
  const char* vb = p.v + (vo + (int64_t)tok0 * p.v_st + (int64_t)h * p.v_sh) * VT::SZ;
  char* ob = p.out + (oo + (int64_t)tok0 * p.o_st + (int64_t)h * p.o_sh) * VT::SZ;
  const char* pkb = C2P ? p.pk + (int64_t)h * p.pk_sh * QT::SZ : nullptr;
  const char* pqb = P2C ? p.pq + (int64_t)h * p.pq_sh * QT::SZ : nullptr;
  const int64_t k_rsb = p.k_st * QT::SZ, v_rsb = p.v_st * VT::SZ;
  const float x_scale = p.scale_log2;

  const int iw0 = m0 + wr * 32;
  const int i = iw0 + li;

  qfrag qf[C::KSTEPS];
#pragma unroll
  for (int s = 0; s < C::KSTEPS; ++s)
    qf[s] = (i < Lb) ? QT::load(qb + ((int64_t)i * p.q_st + 16 * s + 8 * g) * QT::SZ) : QT::zero();

  // Consume the query loads here: left pending into the loop, their first use would make the
  // compiler wait for every outstanding vector-memory load (the prefetches of the next tiles
  // included) at the top of each tile.
#pragma unroll
  for (int s = 0; s < C::KSTEPS; ++s) asm volatile("" ::"v"(qf[s]));

  // ---- the near range: same arithmetic as the fused kernel ------------------------------------
  int j_end = Lb;
  if (p.causal) j_end = min(Lb, m0 + FDB_BM);
  const int n_tiles = (j_end + FDB_BN - 1) / FDB_BN;
  const int lim = m0 - (FDB_BN - 1) - p.R;
  const int t0 = lim >= 0 ? min(n_tiles, lim / FDB_BN + 1) : 0;
  const int t1 = max(t0, min(n_tiles, (m0 + FDB_BM - 1 + p.R + FDB_BN - 1) / FDB_BN));
  const int n_near = t1 - t0;
  const int n_full = p.causal ? 0 : max(0, min(n_near, Lb / FDB_BN - t0));  // tiles k < n_full need no mask

  // relative positions of the workgroup tile k = t - t0: r in [r_hi0 - 64k - 190, r_hi0 - 64k];
  // u = r_hi0 - r counts downwards from the first tile's largest r; ring slot = u & 255; batch = u / 64.
  const int r_hi0 = m0 + FDB_BM - 1 - t0 * FDB_BN;

  // ---- staging: one 16-byte chunk per thread of K, V and of one 64-row batch of each ring ------
  const int srow = tid / C::CPR, scc = tid % C::CPR;
  const bool sact = (kNThreads % C::CPR == 0) && tid < FDB_BN * C::CPR;
  u32x4 kreg = {0, 0, 0, 0}, vreg = {0, 0, 0, 0}, ekreg = {0, 0, 0, 0}, eqreg = {0, 0, 0, 0};
  auto kv_load = [&](int t) __attribute__((always_inline)) {
    if (sact) {
      const int row = min(t * FDB_BN + srow, Lb - 1);  // rows past the end re-read the last one; their scores are masked
      kreg = *(const u32x4*)(kb + (int64_t)row * k_rsb + scc * 16);
      vreg = *(const u32x4*)(vb + (int64_t)row * v_rsb + scc * 16);
    }
  };
  auto kv_store = [&](int buf) __attribute__((always_inline)) {
    if (sact) {
      *(u32x4*)(Ks + buf * C::K_BYTES + srow * C::K_RS + scc * 16) = kreg;
      *(u32x4*)(Vs + buf * C::V_BYTES + srow * C::V_RS + scc * 16) = vreg;
    }
  };
  auto batch_delta = [&](int batch) __attribute__((always_inline)) {  // table row of this thread's ring row
    const int r = r_hi0 - (batch * 64 + srow);
    return (int)p.lut[max(-p.R, min(p.R, r)) + p.R];
  };
  auto batch_load = [&](int delta) __attribute__((always_inline)) {
    if (sact) {
      if constexpr (C2P) ekreg = *(const u32x4*)(pkb + (int64_t)delta * p.pk_sr * QT::SZ + scc * 16);
      if constexpr (P2C) eqreg = *(const u32x4*)(pqb + (int64_t)delta * p.pq_sr * QT::SZ + scc * 16);
    }
  };
  auto batch_store = [&](int batch) __attribute__((always_inline)) {
    if (sact) {
      const int slot = ((batch & 3) * 64 + srow);
      if constexpr (C2P) *(u32x4*)(EK + slot * C::K_RS + scc * 16) = ekreg;
      if constexpr (P2C) *(u32x4*)(EQ + slot * C::K_RS + scc * 16) = eqreg;
    }
  };

  f32x16 o_acc[C::DBLKS];
#pragma unroll
  for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- prologue: tile 0 (K, V, ring batches 0..2) to LDS; tile 1's data into the registers -----
  int delta_next = 0;
  if (n_near > 0) {
    kv_load(t0);
    kv_store(0);
#pragma unroll 1
    for (int bt = 0; bt < 3; ++bt) {
      batch_load(batch_delta(bt));
      batch_store(bt);
    }
    if (n_near > 1) {
      kv_load(t0 + 1);
      batch_load(batch_delta(3));
    }
    if (n_near > 2) delta_next = batch_delta(4);
  }

  // ---- per-lane constants of the position products ----------------------------------------------
  // wave sub-tile k: rows iw0.., keys jw0 = (t0+k)*64 + 32*wk ..; r_lo = iw0 - (jw0 + 31);
  // A row (block bk, lane li): r = r_lo + 32*bk + li  ->  u = r_hi0 - r = ubase - 32*bk + 64*k
  const int ubase = 158 - 32 * (wr - wk) - li;
  // scratch reads: element (jj = 8q + 4g + t, i = li) of the sub-tile reads index r - r_lo = li + 31 - jj
  // C[i = li][li + 31 - jj] for jj = 8q + 4g + 3 .. + 0 is the window of four elements that starts at
  // li + 28 - 4g - 8q = 4 * chunk + (li & 3).  Only 8-byte-aligned LDS reads run at speed (a
  // misaligned one is served lane by lane): the two aligned chunks around the window are read and
  // the window is cut out with per-lane selects and a funnel shift.
  const ST* c_rd = scr + li * kScrStride + 4 * ((li >> 2) + 7 - g);   // chunk of window q = 0; window q is 8q elements lower
  const bool c_odd_chunk = (li & 2) != 0;
  const uint32_t c_shift = 16 * (li & 1);
  const ST* p_rd = scr + (4 * g) * kScrStride + (li + 31 - 4 * g);    // P[jj][.],     plus cj * (stride - 1)
  ST* scr_wr = scr + li * kScrStride + 4 * g;                         // row = this lane's MFMA column

  auto tile = [&](auto mask_tag, int k) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    const int buf = k & 1;
    const int jw0 = (t0 + k) * FDB_BN + 32 * wk;
    // data of tile k is in LDS once every thread's stores have landed; all waves are past tile k-1
    __syncthreads();
    if (k + 1 < n_near) {  // hand tile k+1 to LDS, then start fetching tile k+2
      kv_store(buf ^ 1);
      batch_store(k + 3);
      if (k + 2 < n_near) {
        // the table value this needs was loaded a tile ago; consuming it first keeps the wait
        // off the loads issued below
        batch_load(delta_next);
        kv_load(t0 + k + 2);
        if (k + 3 < n_near) delta_next = batch_delta(k + 5);
      }
    }
    // ---- every MFMA operand of the tile comes out of LDS up front ------------------------------
    const char* Kt = Ks + buf * C::K_BYTES + (32 * wk + li) * C::K_RS + 8 * g * QT::SZ;
    qfrag kf[C::KSTEPS], ac[C2P ? 2 : 1][C::KSTEPS], aq[P2C ? 2 : 1][C::KSTEPS];
#pragma unroll
    for (int s = 0; s < C::KSTEPS; ++s) kf[s] = QT::load(Kt + 16 * s * QT::SZ);
#pragma unroll
    for (int bk = 0; bk < 2; ++bk) {
      const int off = ((ubase - 32 * bk + 64 * k) & (kRing - 1)) * C::K_RS + 8 * g * QT::SZ;
#pragma unroll
      for (int s = 0; s < C::KSTEPS; ++s) {
        if constexpr (C2P) ac[bk][s] = QT::load(EK + off + 16 * s * QT::SZ);
        if constexpr (P2C) aq[bk][s] = QT::load(EQ + off + 16 * s * QT::SZ);
      }
    }
    // ---- the five products back to back -----------------------------------------------------------
    f32x16 sacc, cacc[2], pacc[2];
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[v] = cacc[0][v] = cacc[1][v] = pacc[0][v] = pacc[1][v] = 0.f;
#pragma unroll
    for (int s = 0; s < C::KSTEPS; ++s) sacc = QT::mma(kf[s], qf[s], sacc);
    if constexpr (C2P) {
#pragma unroll
      for (int bk = 0; bk < 2; ++bk)
#pragma unroll
        for (int s = 0; s < C::KSTEPS; ++s) cacc[bk] = QT::mma(ac[bk][s], qf[s], cacc[bk]);
    }
    if constexpr (P2C) {
#pragma unroll
      for (int bk = 0; bk < 2; ++bk)
#pragma unroll
        for (int s = 0; s < C::KSTEPS; ++s) pacc[bk] = QT::mma(aq[bk][s], kf[s], pacc[bk]);
    }
    // ---- through the wave's scratch: write C, read its skewed diagonal, write P over it, read ------
    // The LDS unit runs one wave's operations in order, so the reads of C are served before the
    // writes of P that follow them; only the compiler needs the fences.
    u32x4 cw[4];
    uint32_t px[16];
    if constexpr (C2P) {
#pragma unroll
      for (int bk = 0; bk < 2; ++bk)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)  // C[i = li][32*bk + 8*q4 + 4*g + 0..3]
          store4_scratch<ST>(scr_wr + 32 * bk + 8 * q4, cacc[bk][4 * q4], cacc[bk][4 * q4 + 1], cacc[bk][4 * q4 + 2],
                             cacc[bk][4 * q4 + 3]);
      wave_lds_fence();
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const u32x2 lo = *(const u32x2*)(c_rd - 8 * q4), hi = *(const u32x2*)(c_rd - 8 * q4 + 4);
        cw[q4] = u32x4{lo[0], lo[1], hi[0], hi[1]};
      }
      wave_lds_fence();
    }
    if constexpr (P2C) {
#pragma unroll
      for (int bk = 0; bk < 2; ++bk)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)  // P[jj = li][32*bk + 8*q4 + 4*g + 0..3]
          store4_scratch<ST>(scr_wr + 32 * bk + 8 * q4, pacc[bk][4 * q4], pacc[bk][4 * q4 + 1], pacc[bk][4 * q4 + 2],
                             pacc[bk][4 * q4 + 3]);
      wave_lds_fence();
#pragma unroll
      for (int v = 0; v < 16; ++v) px[v] = *(const uint16_t*)(p_rd + (8 * (v >> 2) + (v & 3)) * (kScrStride - 1));
      wave_lds_fence();
    }
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      if constexpr (C2P) {
        const u32x4 d = cw[q4];
        const uint32_t wa = c_odd_chunk ? d[1] : d[0], wb = c_odd_chunk ? d[2] : d[1], wc = c_odd_chunk ? d[3] : d[2];
        const uint32_t w0 = __builtin_amdgcn_alignbit(wb, wa, c_shift), w1 = __builtin_amdgcn_alignbit(wc, wb, c_shift);
        sacc[4 * q4 + 0] = QT::add_hi(sacc[4 * q4 + 0], w1);  // window elements 3, 2, 1, 0 for jj offsets 0, 1, 2, 3
        sacc[4 * q4 + 1] = QT::add_lo(sacc[4 * q4 + 1], w1);
        sacc[4 * q4 + 2] = QT::add_hi(sacc[4 * q4 + 2], w0);
        sacc[4 * q4 + 3] = QT::add_lo(sacc[4 * q4 + 3], w0);
      }
      if constexpr (P2C) {
#pragma unroll
        for (int e = 0; e < 4; ++e) sacc[4 * q4 + e] = QT::add_lo(sacc[4 * q4 + e], px[4 * q4 + e]);
      }
    }
    near_softmax_pv<VT, D, MASK>(sacc, o_acc, m_run, l_run, x_scale, Vs + buf * C::V_BYTES + 32 * wk * C::V_RS, C::V_RS,
                                 lane, jw0, i, Lb, MASK && p.causal != 0);
  };
  for (int k = 0; k < n_full; ++k) tile(std::false_type{}, k);
  for (int k = n_full; k < n_near; ++k) tile(std::true_type{}, k);

  // ---- merge the two key halves of each row block ---------------------------------------------
  __syncthreads();  // the bias scratch is free
  float* mrg = (float*)scr_raw + wr * ((2 + 16 * C::DBLKS) * 64) + lane;
  if (wk == 1) {
    mrg[0] = m_run;
    mrg[64] = l_run;
#pragma unroll
    for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) mrg[(2 + 16 * d + v) * 64] = o_acc[d][v];
  }
  __syncthreads();
  if (wk == 1) return;
  {
    const float m1 = mrg[0], l1 = mrg[64];
    const float mm = fmaxf(m_run, m1);  // finite: key half 0 always contains a visible key of the diagonal tile... or half 1 does
    const float a0 = __builtin_amdgcn_exp2f(m_run - mm), a1 = __builtin_amdgcn_exp2f(m1 - mm);
    l_run = l_run * a0 + l1 * a1;
    m_run = mm;
#pragma unroll
    for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) o_acc[d][v] = o_acc[d][v] * a0 + mrg[(2 + 16 * d + v) * 64] * a1;
  }

  // ---- epilogue: merge with the far tiles' partial result, normalise, store ---------------------
  float l_tot = wave_half_sum(l_run);
  if (i < Lb) {
    char* orow = ob + (int64_t)i * p.o_st * VT::SZ;
    const int64_t tok = p.cu ? (int64_t)tok0 + i : (int64_t)b * p.L + tok0 + i;
    float w_far = 0.f, w_near = 1.f, m_out = m_run;
    if (p.far_done) {
      const float lf = p.lse[tok * p.H + h] * 1.4426950408889634f;  // far log-sum-exp, base 2 (-inf: no far tile)
      const float ln_ = m_run + __builtin_amdgcn_logf(l_tot);
      m_out = fmaxf(lf, ln_);
      w_far = __builtin_amdgcn_exp2f(lf - m_out);
      w_near = __builtin_amdgcn_exp2f(m_run - m_out);
    }
    const float denom = w_far + w_near * l_tot;
    const float inv = denom > 0.f ? 1.f / denom : 0.f;
    const float sn = w_near * inv, sf = w_far * inv;
#pragma unroll
    for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        char* dst = orow + (32 * d + 8 * q4 + 4 * g) * VT::SZ;
        float f0 = 0.f, f1 = 0.f, f2 = 0.f, f3 = 0.f;
        if (p.far_done) {
          const f32x4 far4 = VT::load4(dst);
          f0 = far4[0] * sf; f1 = far4[1] * sf; f2 = far4[2] * sf; f3 = far4[3] * sf;
        }
        VT::store4(dst, o_acc[d][4 * q4] * sn + f0, o_acc[d][4 * q4 + 1] * sn + f1, o_acc[d][4 * q4 + 2] * sn + f2,
                   o_acc[d][4 * q4 + 3] * sn + f3);
      }
    if (p.lse && g == 0) p.lse[tok * p.H + h] = (m_out + __builtin_amdgcn_logf(denom)) * 0.6931471805599453f;
  }
}

template <class QT, class VT, int D, bool C2P, bool P2C>
int launch_near_one(const FdbKParams& p, int grid_x, hipStream_t stream) {
  using C = NCfg<QT, VT, D>;
  auto kern = fdb_near_kernel<QT, VT, D, C2P, P2C>;
  constexpr int lds = C::lds_bytes(C2P, P2C);
  static_assert(lds <= 160 * 1024, "LDS budget");
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid_x * p.H, 1, 1), dim3(kNThreads), lds, stream, p);
  return (int)hipGetLastError();
}

template <class QT, int D>
int launch_near_pos(const FdbKParams& p, int grid_x, hipStream_t stream) {
  if (p.pk && p.pq) return launch_near_one<QT, QT, D, true, true>(p, grid_x, stream);
  if (p.pk) return launch_near_one<QT, QT, D, true, false>(p, grid_x, stream);
  if (p.pq) return launch_near_one<QT, QT, D, false, true>(p, grid_x, stream);
  return FDB_ERR_UNSUPPORTED;
}

}  // namespace

bool fdb_near_supported(int dtype, int head_dim) {
  return (dtype == FDB_BF16 || dtype == FDB_F16) && (head_dim == 32 || head_dim == 64);
}

int fdb_launch_near(const FdbKParams& p, int dtype, int head_dim, int grid_x, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!fdb_near_supported(dtype, head_dim)) return FDB_ERR_UNSUPPORTED;
  if (dtype == FDB_BF16)
    return head_dim == 64 ? launch_near_pos<Bf16Tr, 64>(p, grid_x, stream) : launch_near_pos<Bf16Tr, 32>(p, grid_x, stream);
  return head_dim == 64 ? launch_near_pos<F16Tr, 64>(p, grid_x, stream) : launch_near_pos<F16Tr, 32>(p, grid_x, stream);
}
