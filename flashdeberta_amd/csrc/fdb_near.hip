// Near tiles of the disentangled-attention forward for gfx950, head_dim 64, 16-bit types: the key
// tiles of a query tile in which the bucketed relative position delta(i - j) is not constant
// (|i - j| < R + tile size).  Second launch of the two-launch path: the far tiles' partial result
// (rows normalised over the far keys in out, their log-sum-exp in lse) is merged in the epilogue.
//
// The position products need the rows E_K[r] = K_r[delta(r)] and E_Q[r] = Q_r[delta(r)] for the
// contiguous range of relative positions r of a tile.  They are staged in LDS rings with coalesced
// loads, so the MFMA A operands are plain LDS reads.
//
// What shapes this kernel is LDS: a wave alone on its SIMD issues a dependent instruction only
// every eight to nine cycles, and nothing else hides that but a second wave.  Two workgroups share
// a CU when each stays under 80 KB, which the rings allow only with 32-key steps:
//   workgroup = 4 waves x 32 query rows, one step = 32 keys;
//   a step sees 159 relative positions (5 batches of 32); the rings hold a sixth batch, the one being
//   filled for the next step: 192 rows of 128 bytes, unpadded and XOR-swizzled;
//   a wave's 32 x 32 sub-tile sees 63 relative positions, so both position products are 2 MFMA
//   blocks, private to the wave: C[i][r] = q_i . E_K[r] and P[j][r] = k_j . E_Q[r], of which element
//   (i, j) wants index r = i - j.  C goes through a per-wave 16-bit LDS scratch (only the one of its
//   two blocks a lane needs, picked before the write) and comes back as the initial value of the
//   content product's accumulator; P is computed with the keys as MFMA rows, so its skew is a rotation
//   of the lanes of a half-wave by a constant of the register (ds_swizzle) and needs no scratch.
// LDS: K 2 x 4 KB + V 2 x 4 KB + rings 2 x 24 KB + scratch 11 KB = 75 KB.
//
// Staging goes global -> LDS directly (global_load_lds_dwordx4: no staging registers, no LDS write
// instructions of the waves' own) and runs one step ahead: right after the one barrier of step s (every
// wave is done with step s-1) a wave issues its share of K(s+1) and V(s+1) into the buffers step s does not
// read and of the 32 rows per table that step s+1 reads for the first time into the ring's sixth batch;
// it waits for these loads at the top of step s+1, before that step's barrier, behind which everybody's
// have landed.  The loads have a whole step to arrive.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <utility>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

using namespace fdb;

namespace {

constexpr int kNThreads = 256;
constexpr int kStep = 32;        // keys per step
constexpr int kRingBatches = 6;  // 5 batches of 32 relative positions in use by a step + the one being filled for the next
constexpr int kRingRows = 32 * kRingBatches;
constexpr int kScrW = 44;        // 16-bit elements between the rows of a wave's bias scratch: 36 in use; rows 8-byte aligned, and
                                 // 22 words apart, so that the 32 rows of a write land in 64 different banks
constexpr int kScrElems = 32 * kScrW;
constexpr int kRowBytes = 128;   // head_dim 64, 16-bit

struct NCfg {
  static constexpr int K_BYTES = kStep * kRowBytes;  // K and V rows are swizzled like the ring rows
  static constexpr int V_BYTES = kStep * kRowBytes;
  static constexpr int RING_BYTES = kRingRows * kRowBytes;
  static constexpr int SCR_BYTES = 4 * kScrElems * 2;
  static constexpr int lds_bytes(bool c2p, bool p2c) {
    return 2 * K_BYTES + 2 * V_BYTES + (c2p ? RING_BYTES + SCR_BYTES : 0) + (p2c ? RING_BYTES : 0);
  }
};

// f(row) of the ring swizzle: slot (row, s) holds chunk s ^ f(row), f = 4*bit1(row) | bits3:2(row);
// sixteen consecutive rows put one chunk in sixteen different bank groups.
__device__ __forceinline__ int ring_f(int row) { return 4 * ((row >> 1) & 1) | ((row >> 2) & 3); }

// px[v] = xs[v] of the lane (ROT0 - c(v)) places further up in this lane's half-wave (mod 32), c(v) = 8*(v/4) + 3 - v%4:
// ds_swizzle in rotate mode, the amount in the instruction's offset field (0xC000 | amount << 5).
template <int ROT0, int... V>
__device__ __forceinline__ void rotate16(const float (&xs)[16], float (&px)[16], std::integer_sequence<int, V...>) {
  ((px[V] = __builtin_bit_cast(
        float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, xs[V]), 0xC000 | ((ROT0 - (8 * (V >> 2) + 3 - (V & 3))) << 5)))),
   ...);
}

template <class QT, class VT, bool C2P, bool P2C>
__global__ __launch_bounds__(kNThreads, 2) void fdb_near_kernel(const FdbKParams p) {
  constexpr int D = 64, KS = 4, DBLKS = 2;
  using qfrag = typename QT::frag;
  using vfrag = typename VT::frag;
  static_assert(QT::SZ == 2 && VT::SZ == 2, "16-bit element types only");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* Ks = smem;                      // [2][32][128]: step k reads buffer k & 1
  char* Vs = Ks + 2 * NCfg::K_BYTES;    // [2][32][128], likewise
  char* EK = Vs + 2 * NCfg::V_BYTES;    // [192][128] rows K_r[delta(r)], slot = (r_hi0 - r) mod 192
  char* EQ = EK + (C2P ? NCfg::RING_BYTES : 0);
  char* scr_raw = EQ + (P2C ? NCfg::RING_BYTES : 0);  // C's scratch (absent without the c2p term)

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, li = lane & 31, g = lane >> 5;
  int xq, h;
  block_map((int)blockIdx.x, p.grid_x, p.H, p.tiles_per_seq, p.cu == nullptr, kMiddleFirst, xq, h);
  uint16_t* scr = (uint16_t*)scr_raw + wave * kScrElems;

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
    const int sl = p.seq_len ? p.seq_len[b] : p.L;  // negative: a batch row the caller could not express, NaN throughout
    Lb = min(max(sl, 0), p.L - tok0);
    if (p.fill_pad && blockIdx.y == 0)
      fill_pad_rows<kRowBytes>(p.out + ((int64_t)b * p.o_sb + (int64_t)h * p.o_sh) * 2, p.o_st * 2, xq % p.tiles_per_seq, p.L, tok0, Lb,
                               sl < 0 ? VT::NAN_WORD : 0u, tid);
    if (m0 >= Lb) return;
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; oo = b * p.o_sb;
  }
  const char* qb = p.q + (qo + (int64_t)tok0 * p.q_st + (int64_t)h * p.q_sh) * 2;
  const char* kb = p.k + (ko + (int64_t)tok0 * p.k_st + (int64_t)h * p.k_sh) * 2;
  const char* vb = p.v + (vo + (int64_t)tok0 * p.v_st + (int64_t)h * p.v_sh) * 2;
  char* ob = p.out + (oo + (int64_t)tok0 * p.o_st + (int64_t)h * p.o_sh) * 2;
  const char* pkb = C2P ? p.pk + (int64_t)h * p.pk_sh * 2 : nullptr;
  const char* pqb = P2C ? p.pq + (int64_t)h * p.pq_sh * 2 : nullptr;
  const uint32_t k_rsb = (uint32_t)(p.k_st * 2), v_rsb = (uint32_t)(p.v_st * 2);  // the host checks that they fit
  const float x_scale = p.scale_log2;

  const int iw0 = m0 + wave * 32;
  const int i = iw0 + li;

  qfrag qf[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s)
    qf[s] = (i < Lb) ? QT::load(qb + ((int64_t)i * p.q_st + 16 * s + 8 * g) * 2) : QT::zero();
  // Consume the query loads here: left pending into the loop, their first use would make the
  // compiler wait for every outstanding vector-memory load at the top of each step.
#pragma unroll
  for (int s = 0; s < KS; ++s) asm volatile("" ::"v"(qf[s]));

  // ---- the near range: the 64-key tiles the far-only run skips, walked 32 keys at a time -----------
  int j_end = Lb;
  if (p.causal) j_end = min(Lb, m0 + FDB_BM);
  const int n_tiles = (j_end + FDB_BN - 1) / FDB_BN;
  const int lim = m0 - (FDB_BN - 1) - p.R;
  const int t0 = lim >= 0 ? min(n_tiles, lim / FDB_BN + 1) : 0;
  const int t1 = max(t0, min(n_tiles, (m0 + FDB_BM - 1 + p.R + FDB_BN - 1) / FDB_BN));
  int s0 = 2 * t0;                                                         // first 32-key step
  int s1 = max(s0, min(2 * t1, (j_end + kStep - 1) / kStep));              // one past the last
  if (p.near_parts > 1) {  // this workgroup's share of the steps
    const int all = s1 - s0, part = (int)blockIdx.y;
    s1 = s0 + (int)((int64_t)all * (part + 1) / p.near_parts);
    s0 = s0 + (int)((int64_t)all * part / p.near_parts);
  }
  const int n_steps = s1 - s0;
  const int n_full = p.causal ? 0 : max(0, min(n_steps, Lb / kStep - s0));  // steps k < n_full need no mask

  // relative positions of the workgroup at step k = s - s0: r in [r_hi0 - 32k - 158, r_hi0 - 32k];
  // u = r_hi0 - r counts downwards from the first step's largest r; ring slot = u mod 192; batch = u / 32.
  const int r_hi0 = m0 + FDB_BM - 1 - s0 * kStep;

  // ---- staging: one 16-byte chunk per thread of K, of V and of one batch of each ring ----------------
  // A direct load fills 1 KB = 8 rows per wave, lane l the 16-byte slot l: thread tid owns slot scc of
  // row srow of the 32-row tile, and since slot (row, s) holds chunk s ^ f(row), it fetches that chunk.
  const int srow = tid >> 3, scc = tid & 7;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_AS char*)smem;
  const uint32_t wave_kb = (uint32_t)wave * 1024u;                  // this wave's 1 KB of a 32-row tile
  const uint32_t chunk_off = (uint32_t)((scc ^ ring_f(srow)) * 16);
  int dnext = 0;
  // A step inside the sequence: its first row travels as the scalar base of the load, this thread's place in the
  // tile as a 32-bit offset computed once.  Only a step that reaches past the end clamps its rows one by one.
  const uint32_t k_lane = (uint32_t)(srow ^ 3) * k_rsb + chunk_off, v_lane = (uint32_t)srow * v_rsb + chunk_off;
  auto k_dma = [&](int s, int buf) __attribute__((always_inline)) {
    // LDS row srow holds key srow ^ 3 of the step (see the scratch reads below); rows past the end
    // re-read the last one, their scores are masked
    const uint32_t dst = lds0 + buf * NCfg::K_BYTES + wave_kb;
    if ((s + 1) * kStep <= Lb) {
      dma16s(kb + (uint64_t)(uint32_t)(s * kStep) * k_rsb, k_lane, dst);
    } else {
      const int row = min(s * kStep + (srow ^ 3), Lb - 1);
      dma16(kb + (uint64_t)(uint32_t)row * k_rsb + chunk_off, dst);
    }
  };
  auto v_dma = [&](int s, int buf) __attribute__((always_inline)) {
    const uint32_t dst = lds0 + 2 * NCfg::K_BYTES + buf * NCfg::V_BYTES + wave_kb;
    if ((s + 1) * kStep <= Lb) {
      dma16s(vb + (uint64_t)(uint32_t)(s * kStep) * v_rsb, v_lane, dst);
    } else {
      const int row = min(s * kStep + srow, Lb - 1);
      dma16(vb + (uint64_t)(uint32_t)row * v_rsb + chunk_off, dst);
    }
  };
  auto batch_delta = [&](int batch) __attribute__((always_inline)) {  // table row of this thread's ring row
    const int r = r_hi0 - (batch * 32 + srow);
    // table rows are indices >= 0: read unsigned, so that the loaded register is the value and nothing
    // has to wait for the load before the next step uses it
    return (int)((const uint16_t*)p.lut)[max(-p.R, min(p.R, r)) + p.R];
  };
  const uint32_t ek_lds = lds0 + (uint32_t)(EK - smem) + wave_kb, eq_lds = lds0 + (uint32_t)(EQ - smem) + wave_kb;
  // table rows are addressed with 32-bit byte offsets from the head's first row (the host checks that a row stride
  // stays under 2^24 bytes and the whole table under 2^31)
  const uint32_t pk_rowb = (uint32_t)(p.pk_sr * 2), pq_rowb = (uint32_t)(p.pq_sr * 2);
  auto batch_dma = [&](int delta, int batch) __attribute__((always_inline)) {
    const uint32_t seg = (uint32_t)(batch % kRingBatches) * (32 * kRowBytes);
    if constexpr (C2P) dma16s(pkb, __umul24((uint32_t)delta, pk_rowb) + chunk_off, ek_lds + seg);
    if constexpr (P2C) dma16s(pqb, __umul24((uint32_t)delta, pq_rowb) + chunk_off, eq_lds + seg);
  };

  f32x16 o_acc[DBLKS];
#pragma unroll
  for (int d = 0; d < DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- per-lane constants ------------------------------------------------------------------------------
  // A row (block bk, lane li) of the wave's sub-tile at step k: r = iw0 - 32s - 31 + 32bk + li, i.e.
  // u = 158 + 32k - 32*(wave + bk) - li; its slot keeps the low five bits of 158 - li for ever.
  const int fr = ring_f(158 - li);
  uint32_t rlx[KS];  // chunk 2s + g of the row sits in slot (2s) ^ g ^ f
#pragma unroll
  for (int s = 0; s < KS; ++s) rlx[s] = ((g ^ fr) * 16) ^ (32 * s);
  int slot0 = 158 - li - 32 * wave;  // block 0 at step 0: u = 158 - li - 32*wave >= 31
  uint32_t klx[KS], vlx[4];  // K fragment rows li; V^T operand (c, d-block db, half h): row 16c + 8h + 4*(grp/2) + s16/4,
                             // 8-byte unit 8db + 4*(grp%2) + s16%4, i.e. chunk ^ f = lane part ^ (4db) ^ (2h)
  {
    const int s16 = lane & 15, grp = lane >> 4;
    const int slotl = (2 * (grp & 1) + ((s16 & 3) >> 1)) ^ (4 * ((s16 >> 3) & 1)) ^ (grp >> 1);
    const uint32_t vlane = (4 * (grp >> 1) + (s16 >> 2)) * kRowBytes + slotl * 16 + (s16 & 1) * 8;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      klx[x] = (li * kRowBytes + ((g ^ ring_f(li)) * 16)) ^ (32 * x);
      vlx[x] = vlane ^ (64 * (x >> 1) ^ 32 * (x & 1));
    }
  }
  // scratch: C[i = li][rr] with rr = r - r_lo in 0..63; element (jj, i = li) wants C[li][li + 31 - jj], i.e. only the
  // band rr in [li, li + 31] of row li is ever read.  Of the two columns rr = c and c + 32 (the same accumulator
  // register of block 0 and of block 1) a lane therefore needs exactly one, c if c >= li: it picks that one
  // (the lanes that pick block 0 are a constant of the register: a scalar mask), rounds to the 16-bit type and
  // writes 32 columns, position rr mod 32, as four 8-byte groups instead of 64 columns in fp32 -- LDS writes are
  // what a step pays most for.  Positions 32..35 repeat 0..3, so that a run of four positions never wraps.
  // K's rows sit in LDS with the low two bits of the row index inverted, so MFMA row m = 8q + 4g + e of
  // the content product is key jj = 8q + 4g + 3 - e: the four C elements a lane adds to consecutive
  // accumulator registers are the run of positions that starts at (li + 28 - 8q - 4g) mod 32.
  uint16_t* c_wrp = scr + li * kScrW + 4 * g;  // row = this lane's MFMA column; group q4 at + 8 q4
  // (read through volatile pointers: four neighbouring 16-bit reads must stay four instructions -- fused into
  // one 8-byte read at an address aligned to two bytes only, they would be served lane by lane)
  LDS_AS const volatile uint16_t* c_rd[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
    c_rd[q] = (LDS_AS const volatile uint16_t*)(scr + li * kScrW + ((li + 28 - 8 * q - 4 * g) & 31));

  // Block 1 of a step holds the rows that were block 0 of the step before, and a step reads only its
  // new block 0 from the rings.  C[r][i] does not depend on the keys, so C's block 1 IS the block 0 the
  // step before computed: its accumulator is kept (two that swap roles; the loop is unrolled over the
  // parity) and only block 0 is contracted.  P depends on the step's keys: there the A operands are
  // kept instead, in two buffers that swap roles the same way.
  qfrag ac[C2P ? KS : 1], aq[2][P2C ? KS : 1];
  f32x16 ckeep[2];
  auto ring_read = [&](int buf, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int x = 0; x < KS; ++x) {
      if constexpr (C2P) ac[x] = QT::load(EK + slot * kRowBytes + rlx[x]);
      if constexpr (P2C) aq[buf][x] = QT::load(EQ + slot * kRowBytes + rlx[x]);
    }
  };
  // ---- prologue: step 0's K and ring batches 0..4 on their way to LDS -------------------------------------
  // All table values first, then all rows: the loads of one kind are in flight together.
  if (n_steps > 0) {
    k_dma(s0, 0);  // K and V need no table value: on their way while the table is read
    v_dma(s0, 0);
    int d0[6];
#pragma unroll
    for (int bt = 0; bt < 6; ++bt) d0[bt] = batch_delta(bt);
    // (taken here, all at once: the compiler, which does not count the direct loads, would otherwise wait for
    // each value at its use, behind all the direct loads issued before it)
#pragma unroll
    for (int bt = 0; bt < 6; ++bt) asm volatile("" : "+v"(d0[bt]));
#pragma unroll
    for (int bt = 0; bt < 5; ++bt) batch_dma(d0[bt], bt);
    dnext = d0[5];
    wait_vmcnt<0>();
    __syncthreads();  // the prologue's ring rows
    ring_read(1, slot0 >= 32 ? slot0 - 32 : slot0 + (kRingRows - 32));  // block 1 of step 0
    if constexpr (C2P) {
#pragma unroll
      for (int x = 0; x < KS; ++x) {
        if (x == 0) {
#pragma unroll
          for (int v = 0; v < 16; ++v) ckeep[1][v] = 0.f;
        }
        ckeep[1] = QT::mma(ac[x], qf[x], ckeep[1]);
      }
    }
  }

  auto step = [&](auto mask_tag, auto par_tag, int k) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr int PAR = decltype(par_tag)::value;  // buffer of this step's block 0
    const int s = s0 + k;
    const int j0 = s * kStep;
    // This wave's direct loads of the step before -- K, V and the new ring batch of this step -- have landed;
    // behind the barrier everyone's have, and every wave is done with the buffers the loads below overwrite.
    wait_vmcnt<0>();
    // The table value fetched a step ago is among the loads just waited for; taking it here keeps the compiler,
    // which does not count the direct loads, from waiting for it further down, behind this step's direct loads.
    asm volatile("" : "+v"(dnext));
    __syncthreads();
    // ---- staging for the next step, straight into LDS ----------------------------------------------------------
    // It runs unconditionally, past the last step too (row and table indices are clamped, and nobody reads
    // what the last steps fetch), so every step issues the same loads and the one wait above covers them.
    k_dma(s + 1, PAR ^ 1);
    v_dma(s + 1, PAR ^ 1);
    batch_dma(dnext, k + 5);
    __builtin_amdgcn_sched_barrier(0);  // the table load stays behind the direct loads
    dnext = batch_delta(k + 6);         // used a step from now
    // ---- operands of the step out of LDS ------------------------------------------------------------------
    qfrag kf[KS];
#pragma unroll
    for (int x = 0; x < KS; ++x) kf[x] = QT::load(Ks + PAR * NCfg::K_BYTES + klx[x]);
    ring_read(PAR, slot0);
    // ---- the five products -------------------------------------------------------------------------------
    // C, C to the scratch and its skewed diagonal back as the initial value of the content product's
    // accumulator; P runs while those reads are in flight (the scheduling fence keeps it behind them).
    // The LDS unit runs one wave's operations in order, so the reads of C are served before the writes
    // of the next step; only the compiler needs the fences.
    f32x16 sacc;
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[v] = 0.f;
    const f32x16 zero = sacc;
    f32x16 pacc[2];
    // The sixteen MFMAs of the four score products first, in two pairs of chains that alternate (no MFMA waits for
    // its own previous link): C with P's block 1 (whose operands are this step's keys and the rows kept from the
    // step before), then P's block 0 with the content product.  What follows C -- the pick, the scratch round trip --
    // runs under the second pair.
#pragma unroll
    for (int x = 0; x < KS; ++x) {
      if constexpr (C2P) ckeep[PAR] = QT::mma(ac[x], qf[x], x == 0 ? zero : ckeep[PAR]);
      if constexpr (P2C) pacc[1] = QT::mma(kf[x], aq[PAR ^ 1][x], x == 0 ? zero : pacc[1]);
    }
#pragma unroll
    for (int x = 0; x < KS; ++x) {
      if constexpr (P2C) pacc[0] = QT::mma(kf[x], aq[PAR][x], x == 0 ? zero : pacc[0]);
      sacc = QT::mma(kf[x], qf[x], sacc);
    }
    uint16_t craw[16];
    if constexpr (C2P) {
      const f32x16(&cacc)[2] = ckeep;  // block bk of this step sits in ckeep[PAR ^ bk]
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {  // C[i = li][(32*bk) + 8*q4 + 4*g + 0..3], block 0 where that column is >= li
        f32x4 pick;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int c0 = 8 * q4 + e, c1 = c0 + 4;  // the column in the lanes g = 0 / g = 1
          const uint64_t mask = ((2ull << c0) - 1ull) | ((c1 >= 31 ? 0xffffffffull : (2ull << c1) - 1ull) << 32);
          pick[e] = __builtin_amdgcn_inverse_ballot_w64(mask) ? cacc[PAR][4 * q4 + e] : cacc[PAR ^ 1][4 * q4 + e];
        }
        const typename QT::scratch4 packed = QT::pack4(pick);
        *(typename QT::scratch4*)(c_wrp + 8 * q4) = packed;
        if (q4 == 0) *(typename QT::scratch4*)(c_wrp + 32) = packed;
      }
      wave_lds_fence();
#pragma unroll
      for (int v = 0; v < 16; ++v) craw[v] = c_rd[v >> 2][v & 3];
      wave_lds_fence();
    }
    // P with the keys as MFMA rows, like the content product: register v of lane (g, n) holds
    // P[jj(v, g)][32 bk + n], and element (jj, i = li) wants column li + 31 - jj of that row, i.e. the same
    // register of another lane of its own half.  Each source lane is read by exactly one lane, which
    // wants block 1 from it if n + jj < 31 and block 0 otherwise: the source picks, one lane permutation
    // per register moves it.
    float px[16];
    if constexpr (P2C) {
      // Source lane (g, n) of register v (key jj = 4g + c) is read by lane (g, (n - rot) mod 32), which wants
      // block 1 from it if n + jj < 31 and block 0 otherwise: which lanes pick block 1 is a constant of the
      // register, so the select takes its mask from a scalar pair.  The move itself is a rotation of each
      // half-wave by a constant, rot = 31 - jj: ds_swizzle in rotate mode (offset 0xC000 | rot << 5), no
      // address registers; the halves differ by 4 in jj, so each half runs its own sixteen under its
      // half of the execution mask.
      float xs[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int c = 8 * (v >> 2) + 3 - (v & 3);  // jj - 4g
        const uint64_t mask = (uint64_t)((1u << (31 - c)) - 1u) | ((uint64_t)(c < 27 ? (1u << (27 - c)) - 1u : 0u) << 32);
        xs[v] = __builtin_amdgcn_inverse_ballot_w64(mask) ? pacc[1][v] : pacc[0][v];
      }
      if (g == 0)
        rotate16<31>(xs, px, std::make_integer_sequence<int, 16>{});
      else
        rotate16<27>(xs, px, std::make_integer_sequence<int, 16>{});
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      if constexpr (C2P) sacc[v] += QT::scratch_to_f32(craw[v]);
      if constexpr (P2C) sacc[v] += px[v];
    }
    // V^T operands requested here, ahead of the soft-max, so that the four MFMAs at the end of the step find them
    vfrag vfr[2][DBLKS];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int d = 0; d < DBLKS; ++d) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(Vs + PAR * NCfg::V_BYTES + vlx[2 * d] + 2048 * c));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(Vs + PAR * NCfg::V_BYTES + vlx[2 * d + 1] + 2048 * c + 1024));
        vfr[c][d] = __builtin_bit_cast(vfrag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    __builtin_amdgcn_sched_barrier(0);
    // ---- mask, online soft-max in base 2, O^T += V^T P^T ---------------------------------------------------
    if constexpr (MASK) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + 8 * (v >> 2) + 4 * g + 3 - (v & 3);
        if (j >= Lb || (p.causal && j > i)) sacc[v] = -INFINITY;
      }
    }
    // The probabilities are formed against the row's current reference point first; the half-row sum of a
    // step bounds its largest one, so while it stays under 2^kLazyTau nothing has to move and no maximum is
    // taken.  Otherwise (or before a row has a reference point) the wave takes the maximum, moves the
    // reference points of the rows that need it and forms the probabilities again.
    vfrag pf[2];
    float l_blk = 0.f;
    auto probs = [&](float off) __attribute__((always_inline)) {
      l_blk = 0.f;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        f32x8 pv;
#pragma unroll
        for (int e = 0; e < 8; ++e)  // the V^T operand takes the keys in ascending order
          pv[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[8 * c + (e ^ 3)], x_scale, off));
        pf[c] = VT::from_f32(pv);
        l_blk = sum8(pv, l_blk);
      }
    };
    bool slow = __any(m_run == -INFINITY);
    if (!slow) {
      probs(-m_run);
      slow = __any(!(l_blk <= 256.f));  // 2^kLazyTau; also true for an overflow
    }
    if (slow) {
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
        for (int d = 0; d < DBLKS; ++d)
#pragma unroll
          for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
      }
      probs((MASK && m_run == -INFINITY) ? 0.f : -m_run);  // a row that has seen no visible key yet
    }
    l_run += l_blk;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int d = 0; d < DBLKS; ++d) o_acc[d] = VT::mma(vfr[c][d], pf[c], o_acc[d]);
    slot0 = slot0 + 32 >= kRingRows ? slot0 + 32 - kRingRows : slot0 + 32;
  };
  {
    using T0 = std::integral_constant<int, 0>;
    using T1 = std::integral_constant<int, 1>;
    int k = 0;
#pragma unroll 1
    for (; k + 1 < n_full; k += 2) {
      step(std::false_type{}, T0{}, k);
      step(std::false_type{}, T1{}, k + 1);
    }
    if (k < n_full) {
      step(std::false_type{}, T0{}, k);
      ++k;
    }
    if ((k & 1) && k < n_steps) {
      step(std::true_type{}, T1{}, k);
      ++k;
    }
#pragma unroll 1
    for (; k + 1 < n_steps; k += 2) {
      step(std::true_type{}, T0{}, k);
      step(std::true_type{}, T1{}, k + 1);
    }
    if (k < n_steps) step(std::true_type{}, T0{}, k);
  }
  wait_vmcnt<0>();  // the last step's direct loads: none may still be writing LDS when the workgroup ends

  // ---- epilogue: merge with the far tiles' partial result, normalise, store ------------------------------
  const float l_tot = wave_half_sum(l_run);
  if (i < Lb) {
    char* orow = ob + (int64_t)i * p.o_st * 2;
    const int64_t tok = p.cu ? (int64_t)tok0 + i : (int64_t)b * p.L + tok0 + i;
    if (p.near_parts > 1) {
      // a share of the steps: the partial result goes to its workspace slot, fdb_merge_kernel does the rest
      const int slot = p.far_parts - 1 + (int)blockIdx.y;
      char* dst = ws_slot_out(p, slot, D * 2) + (tok * p.H + h) * (D * 2);
      const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
      for (int d = 0; d < DBLKS; ++d)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          VT::store4(dst + (32 * d + 8 * q4 + 4 * g) * 2, o_acc[d][4 * q4] * inv, o_acc[d][4 * q4 + 1] * inv,
                     o_acc[d][4 * q4 + 2] * inv, o_acc[d][4 * q4 + 3] * inv);
      if (g == 0)
        ws_slot_lse(p, slot, D * 2)[tok * p.H + h] =
            l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f : -INFINITY;
      return;
    }
    // far partial results: part 0 in out / lse, the others in the workspace (rows normalised over their
    // keys, log-sum-exp -inf where a row had none)
    const int n_far = p.far_done ? p.far_parts : 0;
    float w_far[FDB_MAX_FAR_PARTS], w_near = 1.f, m_out = m_run;
    const char* far_row[FDB_MAX_FAR_PARTS];
#pragma unroll
    for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s) {
      w_far[s] = -INFINITY;  // log-sum-exp in base 2 until the maximum is known
      far_row[s] = orow;
      if (s < n_far) {
        const float* lp = s == 0 ? p.lse : far_part_lse(p, s, D * 2);
        w_far[s] = lp[tok * p.H + h] * 1.4426950408889634f;
        if (s > 0) far_row[s] = far_part_out(p, s, D * 2) + (tok * p.H + h) * (D * 2);
      }
    }
    if (n_far > 0) {
      m_out = m_run + __builtin_amdgcn_logf(l_tot);
#pragma unroll
      for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s) m_out = fmaxf(m_out, w_far[s]);
      w_near = __builtin_amdgcn_exp2f(m_run - m_out);
    }
    float denom = w_near * l_tot;
#pragma unroll
    for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s) {
      w_far[s] = (s < n_far && w_far[s] != -INFINITY) ? __builtin_amdgcn_exp2f(w_far[s] - m_out) : 0.f;
      denom += w_far[s];
    }
    const float inv = denom > 0.f ? 1.f / denom : 0.f;
    const float sn = w_near * inv;
#pragma unroll
    for (int d = 0; d < DBLKS; ++d)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int off = (32 * d + 8 * q4 + 4 * g) * 2;
        float f0 = 0.f, f1 = 0.f, f2 = 0.f, f3 = 0.f;
#pragma unroll
        for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s)
          if (s < n_far) {
            const f32x4 far4 = VT::load4(far_row[s] + off);
            const float sf = w_far[s] * inv;
            f0 += far4[0] * sf; f1 += far4[1] * sf; f2 += far4[2] * sf; f3 += far4[3] * sf;
          }
        VT::store4(orow + off, o_acc[d][4 * q4] * sn + f0, o_acc[d][4 * q4 + 1] * sn + f1, o_acc[d][4 * q4 + 2] * sn + f2,
                   o_acc[d][4 * q4 + 3] * sn + f3);
      }
    if (p.lse && g == 0) p.lse[tok * p.H + h] = (m_out + __builtin_amdgcn_logf(denom)) * 0.6931471805599453f;
  }
}

template <class QT, bool C2P, bool P2C>
int launch_near_one(const FdbKParams& p, int grid_x, hipStream_t stream) {
  auto kern = fdb_near_kernel<QT, QT, C2P, P2C>;
  constexpr int lds = NCfg::lds_bytes(C2P, P2C);
  static_assert(lds <= 80 * 1024, "two workgroups per CU");
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = fdb_set_lds_once((const void*)kern, lds, lds_set);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid_x * p.H, p.near_parts > 1 ? (unsigned)p.near_parts : 1u, 1), dim3(kNThreads),
                     lds, stream, p);
  return (int)hipGetLastError();
}

template <class QT>
int launch_near_pos(const FdbKParams& p, int grid_x, hipStream_t stream) {
  if (p.pk && p.pq) return launch_near_one<QT, true, true>(p, grid_x, stream);
  if (p.pk) return launch_near_one<QT, true, false>(p, grid_x, stream);
  if (p.pq) return launch_near_one<QT, false, true>(p, grid_x, stream);
  return FDB_ERR_UNSUPPORTED;
}

}  // namespace

bool fdb_near32_supported(int dtype, int head_dim) {
  return (dtype == FDB_BF16 || dtype == FDB_F16) && head_dim == 64;
}

int fdb_launch_near32(const FdbKParams& p, int dtype, int grid_x, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (dtype == FDB_BF16) return launch_near_pos<Bf16Tr>(p, grid_x, stream);
  if (dtype == FDB_F16) return launch_near_pos<F16Tr>(p, grid_x, stream);
  return FDB_ERR_UNSUPPORTED;
}
