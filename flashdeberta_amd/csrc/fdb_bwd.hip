// Backward of the disentangled attention for gfx950: dQ, dK, dV and the gradients of the two
// position-score tensors, from the saved log-sum-exp.  Counterpart of the reference's three backward
// kernels (src/flashdeberta/ops/flash_attention.py:62-141 _bwd_preprocess, :581-760 _bwd_kv_dise_kernel,
// :762-941 _bwd_q_dise_kernel, launcher :942-1030): like them it takes the position scores
// c2p[b,i,h,delta] = q_i . K_r[delta] and p2c[b,j,h,delta] = k_j . Q_r[delta] as tensors, gathers them through
// the bucketed relative position, and returns the score gradients as tensors of the same shape (the reference
// scatter-adds them with tl.atomic_add, :769-786; here every entry is stored once, see below); the chain through
// K_r / Q_r is left to the caller's GEMMs.
//
// One kernel in two roles.  A workgroup owns 128 rows of the "lane side" (4 waves x 32 rows, one row per
// lane and its partner lane ^ 32) and walks the "loop side" 32 rows at a time; the loop side's tiles come
// from global memory straight into one of two LDS buffers, 64 rows (two steps) per buffer and barrier:
//   role dQ    : lane side = queries (q, dO in registers), loop side = keys (K, V tiles)  ->  dQ, d c2p
//   role dK/dV : lane side = keys (k, v in registers), loop side = queries (Q, dO tiles) ->  dK, dV, d p2c
// Per step, with X the lane side and Y the loop side (MFMA 32x32, M = loop row, N = lane row):
//   S' = Y1 X1^T (+ gathered position scores), P' = exp2(S' * c log2e - lse_i log2e), dP' = Y2 X2^T,
//   dS' = P' (dP' - Delta_i) c, and the outputs contract over the loop rows, which sit in the accumulator
//   registers: out^T += Y^T dS' (or P'), with Y^T read transposed from LDS -- the layout trick of the forward.
// Score gradients without atomics.  Each role owns the tensor of its lane side (dQ role: d c2p, a row per query;
// dK/dV role: d p2c, a row per key).  The table row delta(i - j) is monotone in the loop row, so the entries a lane
// row can still receive form a window that slides one way as the loop advances; the entry point refuses tables in
// which 32 consecutive relative positions span more than 61 rows (steps of 0 or 1, the usual case, span at most 32):
// a 64-entry ring per row in LDS takes the adds, and the entries the window has left behind are stored
// once, in aligned groups of four (eight lanes per row, one 16- or 8-byte store each), and cleared.  The tensors have
// the element type of q; the entries of a real token's row that no element maps to are written as zeros (in the loop or after it),
// rows of padding are not touched.  Results
// do not depend on the order workgroups run in.
// A step whose relative positions all lie beyond the table radius has one table row: its position scores are
// one load per row and its score gradients enter the ring as one row sum per lane.
// In a near block the loop side's scores are one load per element (a wave instruction reads neighbouring entries of one
// or two rows); the lane side's, where every lane has its own row (64 cache lines per instruction), come as one 12-byte
// load per group of four neighbouring loop rows -- six consecutive entries that hold the group's four table rows
// whenever the table moves by at most one row per position -- and the element is picked from the three registers
// (one byte permutation per element where the six entries start at the group's first table row or one before it).
// The table sits in LDS with 64 copies of its end entries on either side, so that the lookups of a near block are one
// address per step plus a constant per element, without a clamp.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

using namespace fdb;

namespace {

constexpr int kBwdThreads = 256;
constexpr int kBwdStep = 32;    // loop-side rows per step
constexpr int kRing = FDB_BWD_RING;  // score-gradient entries kept per lane-side row: the table rows of one 32-row step
                                     // (at most lut_window + 1, which the entry point bounds) plus a partly stored group
static_assert(kRing == 64 && FDB_BWD_MAX_WINDOW + 4 <= kRing, "ring slots are taken modulo 64");
// Row stride of the ring in floats.  The lanes of a half-wave hit entry (delta0 -+ lane) of row `lane` (dQ role: +,
// dK/dV role: -): with stride 65 resp. 67 that is bank 2 * lane, no two lanes alike.
constexpr int ring_stride(bool dq) { return dq ? kRing + 1 : kRing + 3; }
constexpr int kRingStrideMax = kRing + 3;
// The table in LDS carries this many copies of its first and of its last entry before and after it: the relative
// positions of a near block reach at most 62 beyond the radius, so its lookups need no clamp.
constexpr int kLutPad = 64;

template <class QT, int D>
struct BCfg {
  static constexpr int KS = D / 16, DBLKS = D / 32;
  static constexpr int RS = D * QT::SZ + 16;                 // LDS row stride of a staged tile
  static constexpr int CPR = D * QT::SZ / 16;                // 16-byte chunks of a row
  // Loop-side rows staged per barrier: two steps' worth where LDS allows (the barrier and the staging are then paid
  // once per 64 rows), one for the widest rows.
  static constexpr int TROWS = RS > 272 ? kBwdStep : 2 * kBwdStep;
  static constexpr int TILE = TROWS * RS;                    // a multiple of 1024: RS is a multiple of 16
  static constexpr int REGION = 2 * TILE;                    // [Y1 tile | Y2 tile] of one buffer
  // two buffers, loop-row statistics, ring windows, groups to store; the table follows
  static constexpr int fixed_lds_bytes() { return 2 * REGION + 4 * 64 * 4 + FDB_BM * kRingStrideMax * 4 + FDB_BM * 8; }
  static int lds_bytes(int radius) { return fixed_lds_bytes() + (((2 * radius + 1 + 2 * kLutPad) * 2 + 15) & ~15); }
};

// acc[m][n] = a_lane(n) + b_loop(m) as one MFMA: the start of S' in a block with a single table row, where the
// position scores are one value per lane-side row and one per loop-side row.  Loop rows are MFMA rows (operand A,
// lane = row), lane-side rows MFMA columns (operand B); the two contraction slots used are k = 0, 1.
template <class QT>
__device__ __forceinline__ f32x16 rank1_start(float a_lane, float b_loop, int g) {
  const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  if constexpr (QT::SZ == 4) {
    // K = 2: lane group g supplies k = g
    return __builtin_amdgcn_mfma_f32_32x32x2f32(g == 0 ? b_loop : 1.f, g == 0 ? 1.f : a_lane, zero, 0, 0, 0);
  } else {
    // K = 16: lane group 0 supplies k = 0..7
    f32x8 ay = {0, 0, 0, 0, 0, 0, 0, 0}, ax = {0, 0, 0, 0, 0, 0, 0, 0};
    ay[0] = g == 0 ? b_loop : 0.f;
    ay[1] = g == 0 ? 1.f : 0.f;
    ax[0] = g == 0 ? 1.f : 0.f;
    ax[1] = g == 0 ? a_lane : 0.f;
    return QT::mma(QT::from_f32(ay), QT::from_f32(ax), zero);
  }
}

template <class QT, int D, int ROLE, bool C2P, bool P2C>
__global__ __launch_bounds__(kBwdThreads, (D * QT::SZ <= 128 ? 2 : 1)) void fdb_bwd_kernel(const FdbBwdParams p) {
  using C = BCfg<QT, D>;
  using frag = typename QT::frag;
  constexpr int KS = C::KS, DBLKS = C::DBLKS;
  constexpr bool kDQ = ROLE == 0;
  constexpr int kRingStride = ring_stride(kDQ);
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* Ys = smem;                                    // two buffers of [K | V] (dQ role) / [Q | dO] (dK/dV role)
  float* stat_s = (float*)(Ys + 2 * C::REGION);       // dK/dV role: per buffer, log-sum-exp and Delta of the staged loop rows (64 floats each)
  float* ring_s = stat_s + 4 * 64;              // [128 lane-side rows][kRingStride] score-gradient windows
  int2* inf_s = (int2*)(ring_s + FDB_BM * kRingStrideMax);  // [4 waves][32] (first group, groups) to store per row
  LDS_AS int16_t* lut_pad = (LDS_AS int16_t*)(inf_s + FDB_BM);  // the whole table, padded (the launcher sizes the allocation for it)
  LDS_AS int16_t* lut_s = lut_pad + kLutPad;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, li = lane & 31, g = lane >> 5;
  // Linear workgroup id -> (tile of lane-side rows, head, batch row).  The hardware deals workgroups to the 8 XCDs
  // round-robin by linear id and each XCD has its own L2: where the launcher asks for it (p.pairs_per_xcd: at least
  // eight (batch row, head) pairs and more than two rounds of workgroups), pairs are dealt to XCDs whole, eight at a
  // time, so that all tiles of a pair stream the same loop-side rows (tiles and position scores) through one L2,
  // one after the other in dispatch order.  A causal dQ launch deals a pair's tiles last first: those see the most keys.
  const int tiles_x = (p.L + FDB_BM - 1) / FDB_BM;
  int h, b, tile_x;
  {
    const int n = blockIdx.x;
    const int whole = (p.B * p.H) & ~7;   // pairs dealt to XCDs whole; the rest follow in the plain order
    if (p.pairs_per_xcd && n < whole * tiles_x) {
      const int slot = n >> 3, pair = (n & 7) + 8 * (slot / tiles_x);
      tile_x = slot % tiles_x;
      b = pair / p.H;
      h = pair % p.H;
    } else if (p.pairs_per_xcd) {
      const int rest = n - whole * tiles_x, pair = whole + rest / tiles_x;
      tile_x = rest % tiles_x;
      b = pair / p.H;
      h = pair % p.H;
    } else {
      tile_x = n % tiles_x;
      h = (n / tiles_x) % p.H;
      b = n / (tiles_x * p.H);
    }
    if (kDQ && p.causal) tile_x = tiles_x - 1 - tile_x;
  }
  const int m0 = tile_x * FDB_BM;
  const int tok0 = p.seq_start ? min(max(p.seq_start[b], 0), p.L) : 0;
  const int Lb = p.seq_len ? min(max(p.seq_len[b], 0), p.L - tok0) : p.L;
  if (m0 >= Lb) return;
  if (C2P || P2C)
    for (int x = tid; x < 2 * p.R + 1 + 2 * kLutPad; x += kBwdThreads) lut_pad[x] = p.lut[min(max(x - kLutPad, 0), 2 * p.R)];
  // grp_ok: four consecutive relative positions never span more than four table rows (steps of 0 or 1, the usual
  // case): the lane side's scores of four neighbouring loop rows then sit within six consecutive entries of the lane's
  // row and are fetched as one 12-byte load (see request_near).  Every wave checks the table for itself once it is
  // in LDS.
  bool grp_ok = false;

  auto base = [&](const char* ptr, int64_t sb, int64_t st, int64_t sh) {
    return ptr + (b * sb + (int64_t)tok0 * st + (int64_t)h * sh) * QT::SZ;
  };
  const char* qb = base(p.q, p.q_sb, p.q_st, p.q_sh);
  const char* kb = base(p.k, p.k_sb, p.k_st, p.k_sh);
  const char* vb = base(p.v, p.v_sb, p.v_st, p.v_sh);
  const char* gb = base(p.dout, p.g_sb, p.g_st, p.g_sh);
  // lane side X1 / X2 (registers), loop side Y1 / Y2 (LDS tiles)
  const char* x1b = kDQ ? qb : kb;
  const char* x2b = kDQ ? gb : vb;
  const int64_t x1_st = kDQ ? p.q_st : p.k_st, x2_st = kDQ ? p.g_st : p.v_st;
  const char* y1b = kDQ ? kb : qb;
  const char* y2b = kDQ ? vb : gb;
  const int64_t y1_rsb = (kDQ ? p.k_st : p.q_st) * QT::SZ, y2_rsb = (kDQ ? p.v_st : p.g_st) * QT::SZ;

  const int xw0 = m0 + wave * 32;  // first lane-side row of this wave
  const int xr = xw0 + li;         // this lane's row (local to the sequence)
  const bool x_ok = xr < Lb;
  frag x1f[KS], x2f[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    x1f[s] = x_ok ? QT::load(x1b + ((int64_t)xr * x1_st + 16 * s + 8 * g) * QT::SZ) : QT::zero();
    x2f[s] = x_ok ? QT::load(x2b + ((int64_t)xr * x2_st + 16 * s + 8 * g) * QT::SZ) : QT::zero();
  }
  // row statistics (log-sum-exp, delta) are token-major: row (b, tok0 + l), head h
  const int64_t tok_x = ((int64_t)b * p.L + tok0 + (x_ok ? xr : 0)) * p.H + h;
  float lse_x = 0.f, del_x = 0.f;
  if (kDQ) {
    if (p.out != nullptr) {
      // delta = dO . O of this lane's row (the reference's _bwd_preprocess): each half-wave has half of the row;
      // left in p.delta for the dK/dV launch, which follows this one on the stream
      const char* ob = base(p.out, p.o_sb, p.o_st, p.o_sh);
      float dot = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const f32x8 o8 = QT::to_f32(x_ok ? QT::load(ob + ((int64_t)xr * p.o_st + 16 * s + 8 * g) * QT::SZ) : QT::zero());
        const f32x8 g8 = QT::to_f32(x2f[s]);
#pragma unroll
        for (int e = 0; e < 8; ++e) dot = __builtin_fmaf(o8[e], g8[e], dot);
      }
      del_x = wave_half_sum(dot);
      if (x_ok && g == 0) p.delta[tok_x] = del_x;
    } else if (x_ok) {
      del_x = p.delta[tok_x];
    }
    if (x_ok) lse_x = p.lse[tok_x] * 1.4426950408889634f;
  }
  const int S2 = 2 * p.S;
  // Position-score tensors are addressed as one base per (batch row, head) plus 32-bit element offsets
  // (token * row stride + table row; the entry point checks that L * row stride fits).
  const int64_t seq_base = (int64_t)b * p.bias_sb + (int64_t)tok0 * p.bias_st + (int64_t)h * p.bias_sh;
  const uint32_t row_elems = (uint32_t)p.bias_st;                     // elements between neighbouring tokens
  const uint32_t x_off = (uint32_t)(x_ok ? xr : 0) * row_elems;      // this lane's row
  // Score gradients of the lane side's tensor: ring rows of this wave in LDS, rows of this wave in the tensor.
  constexpr bool kGrad = kDQ ? C2P : P2C;
  float* ring_w = ring_s + wave * 32 * kRingStride;
  float* ring_x = ring_w + li * kRingStride;
  int2* inf_w = inf_s + wave * 32;
  char* gw = nullptr;   // this sequence and head of the gradient tensor (elements of the input type)
  if (kGrad) {
    gw = (kDQ ? p.d_c2p : p.d_p2c) + seq_base * QT::SZ;
    for (int e = lane; e < 32 * kRingStride; e += 64) ring_w[e] = 0.f;
  }
  constexpr int kDir = kDQ ? -1 : 1;        // the way the window moves as the loop row grows
  int g_next = 0;                           // next group of four entries of this lane's row to store
  float g_far = 0.f;                        // row sum of a run of far blocks

  f32x16 acc1[DBLKS], acc2[DBLKS];  // dQ^T (dQ role) / dK^T and dV^T (dK/dV role)
#pragma unroll
  for (int d = 0; d < DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc1[d][v] = acc2[d][v] = 0.f;

  // loop range: every 32-row step of the other side that any row of the workgroup can see
  int y_lo = 0, y_hi = Lb;
  if (p.causal) {
    if (kDQ) y_hi = min(Lb, m0 + FDB_BM);  // keys j <= i
    else y_lo = (m0 / kBwdStep) * kBwdStep;  // queries i >= j
  }
  const float c_log2 = p.scale_log2, c_sm = p.sm_scale;
  auto delta_of = [&](int r) __attribute__((always_inline)) -> int {
    const int x = max(-p.R, min(p.R, r)) + p.R;
    return (int)lut_s[x];
  };
  // The loop side's tiles go from global memory straight into one of two LDS buffers (no registers on the way):
  // those of the rows after the current ones are on their way while the current ones are used, and a barrier per
  // buffer makes them visible.  A wave instruction fills 1 KB of LDS, lane l the 16 bytes at 16 * l: with padded rows
  // some lanes fall on the padding and fetch a chunk nobody reads.  Rows past the end re-read the last valid row;
  // their scores are masked.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_AS char*)smem;
  auto tiles_dma = [&](int r0, int buf) __attribute__((always_inline)) {
    constexpr int SPANS = C::REGION / 1024;
#pragma unroll
    for (int n = 0; n < (SPANS + 3) / 4; ++n) {
      const int span = wave + 4 * n;
      if (span < SPANS) {
        const int o = span * 1024 + lane * 16;
        const int t = o >= C::TILE ? 1 : 0, o2 = o - t * C::TILE;
        const int row = o2 / C::RS, c = (o2 - row * C::RS) >> 4;
        const char* src = (t ? y2b : y1b) + (int64_t)min(r0 + row, Lb - 1) * (t ? y2_rsb : y1_rsb) + (c < C::CPR ? c : 0) * 16;
        dma16(src, lds0 + buf * C::REGION + span * 1024);
      }
    }
  };
  // The statistics of the staged loop rows (dK/dV role) travel like the tiles, from global memory straight into LDS:
  // wave 0 fetches the log-sum-exps, wave 1 the Deltas, one row per lane, and the wait and the barrier that cover
  // the tiles cover them.  (Through registers, the wave that fetched them waited at its store for every load it had
  // issued since, the next block's position scores among them, and the other waves waited for it at the barrier.)
  auto stats_dma = [&](int r0, int buf) __attribute__((always_inline)) {
    if (!kDQ && wave < 2) {
      const int row = min(r0 + lane, Lb - 1);
      const float* src = (wave == 0 ? p.lse : p.delta) + (((int64_t)b * p.L + tok0 + row) * p.H + h);
      dma4(src, lds0 + (uint32_t)((const char*)stat_s - smem) + (uint32_t)((buf * 2 + wave) * 64 * 4));
    }
  };
  // Position scores of a step are requested one step ahead (their addresses depend on indices only), so that their
  // round trip to memory runs behind the step before.  A far step (every relative position of the wave's 32 x 32
  // block beyond the table radius: one table row) asks for two values per lane, the lane row's score and the score of
  // loop row `li`; a near step asks for one value per element and tensor.  Rows past the end re-read the last valid
  // row, lanes past the end read row 0: the loads are unconditional and only their use is masked.
  constexpr bool kBias = C2P || P2C;
  constexpr bool kLaneT = kDQ ? C2P : P2C, kLoopT = kDQ ? P2C : C2P;
  using BT = typename QT::scratch_t;   // element type of the position-score tensors: that of q
  const BT* lane_t = kLaneT ? (const BT*)(kDQ ? p.c2p : p.p2c) + seq_base : nullptr;   // the lane side's tensor, this sequence and head
  const BT* loop_t = kLoopT ? (const BT*)(kDQ ? p.p2c : p.c2p) + seq_base : nullptr;   // the loop side's
  BT raw_lane[16], raw_loop[16];   // as loaded: converting here would wait for the load
  bool far_n = false;
  int dfar_n = 0;
#pragma unroll
  for (int v = 0; v < 16; ++v) raw_lane[v] = raw_loop[v] = (BT)0.f;
  auto loop_off = [&](int yr) __attribute__((always_inline)) -> uint32_t {
    return (uint32_t)min(yr, Lb - 1) * row_elems;
  };
  // Classifies the wave's block of the step at y0 and, if it is far, asks for its two values right away (they cost two
  // registers); the values of a near block are asked for by request_near right after (28 registers in the grouped form).
  auto request_far = [&](int y0) __attribute__((always_inline)) {
    if (!kBias) return;
    const int r_min = kDQ ? xw0 - (y0 + kBwdStep - 1) : y0 - (xw0 + 31);      // over the wave's 32 x 32 block
    const int r_max = kDQ ? xw0 + 31 - y0 : y0 + kBwdStep - 1 - xw0;
    far_n = r_min >= p.R || r_max <= -p.R;
    dfar_n = far_n ? delta_of(r_min) : 0;
    if (far_n) {
      if (kLaneT) raw_lane[0] = lane_t[x_off + (uint32_t)dfar_n];
      if (kLoopT) raw_loop[0] = loop_t[loop_off(y0 + li) + (uint32_t)dfar_n];
    }
  };
  // The loop over the other side, written once and compiled twice: GRP says whether the lane side's near scores are
  // fetched in groups (see grp_ok); the two copies keep their own registers.
  auto run = [&](auto grp_tag) __attribute__((always_inline)) {
  constexpr bool GRP = decltype(grp_tag)::value;
  // The table rows of a near block's 16 elements stay with the lane until the block's score gradients are added: as
  // offsets (0..31) from the first entry of the lane row's window, four to a register.
  int d_lo = 0, d_lo_n = 0;            // ... of the current step and of the one asked for
  uint32_t off4[4] = {0u, 0u, 0u, 0u}, off4_n[4] = {0u, 0u, 0u, 0u};
  typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
  u32x3 raw3[4];         // grouped form of the lane side's scores: six consecutive 16-bit entries per group of four elements
  uint32_t goff = 0u;    // ... and where in them the group's lowest table row sits (0..5), four bits per group
#pragma unroll
  for (int q4 = 0; q4 < 4; ++q4) raw3[q4] = u32x3{0u, 0u, 0u};
  const uint32_t x_last = x_off + (uint32_t)(2 * p.S) - 6u;   // last even start whose six entries stay inside the row
  // Table row of element (q4, e) of this lane in the step at y0: relative position xr - yr (dQ role) or yr - xr with
  // yr = y0 + 8 q4 + 4 g + e, looked up in the padded table at one address per step plus a constant per element.
  const int lut_lane = kDQ ? xr - 4 * g + p.R - 27 : p.R + 4 * g - xr;
  auto request_near = [&](int y0) __attribute__((always_inline)) {
    if (!kBias || far_n) return;
    volatile LDS_AS const int16_t* lut_e = lut_s + (kDQ ? lut_lane - y0 : lut_lane + y0);  // volatile: merged into 8-byte reads at 2-byte alignment they would be served lane by lane
    const uint32_t row_bytes = row_elems * (uint32_t)sizeof(BT), last_row = (uint32_t)(Lb - 1) * row_bytes;
    const uint32_t rowb = (uint32_t)(y0 + 4 * g) * row_bytes;   // byte offset of the loop row of element 0; rows past the end re-read the last one
    int dls[16];   // all lookups first: the reads are volatile and stay in this order, so none waits for a use before it
#pragma unroll
    for (int v = 0; v < 16; ++v) dls[v] = (int)lut_e[kDQ ? 27 - (8 * (v >> 2) + (v & 3)) : 8 * (v >> 2) + (v & 3)];
    d_lo_n = (int)lut_e[kDQ ? 4 * g - 4 : -4 * g];   // the step's lowest table row of this lane's row: loop row y0 + 31 (dQ role) or y0
    off4_n[0] = off4_n[1] = off4_n[2] = off4_n[3] = 0u;
    if constexpr (kLaneT && sizeof(BT) == 2) {
      if (GRP) {
      goff = 0u;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        int dmin = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = 8 * q4 + e;
          const int dl = dls[4 * q4 + e];
          off4_n[q4] |= (uint32_t)(dl - d_lo_n) << (8 * e);
          if (e == (kDQ ? 3 : 0)) dmin = dl;   // the table row falls (dQ role) or rises (dK/dV role) with the loop row
          if (kLoopT) raw_loop[4 * q4 + e] = *(const BT*)((const char*)loop_t + (min(rowb + (uint32_t)v * row_bytes, last_row) + (uint32_t)dl * (uint32_t)sizeof(BT)));
        }
        const uint32_t first = x_off + (uint32_t)dmin;
        const uint32_t start = min(first & ~1u, x_last);
        goff |= (first - start) << (4 * q4);
        raw3[q4] = *(const u32x3*)(lane_t + start);
      }
      return;
      }
    }
    {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ve = 8 * (v >> 2) + (v & 3);
        const int dl = dls[v];
        off4_n[v >> 2] |= (uint32_t)(dl - d_lo_n) << (8 * (v & 3));
        if (kLaneT) raw_lane[v] = lane_t[x_off + (uint32_t)dl];
        if (kLoopT) raw_loop[v] = *(const BT*)((const char*)loop_t + (min(rowb + (uint32_t)ve * row_bytes, last_row) + (uint32_t)dl * (uint32_t)sizeof(BT)));
      }
    }
  };
  // entry `idx` (0..5) of six consecutive 16-bit entries held in three registers
  auto entry16 = [&](const u32x3& w, uint32_t idx) __attribute__((always_inline)) -> uint16_t {
    const uint32_t lo = idx < 2u ? w[0] : (idx < 4u ? w[1] : w[2]);
    return (uint16_t)((idx & 1u) ? lo >> 16 : lo);
  };
  if (y_lo < y_hi) {
    tiles_dma(y_lo, 0);
    stats_dma(y_lo, 0);
    __syncthreads();  // the table is in LDS
    if (kGrad) g_next = delta_of(kDQ ? xr - y_lo : y_lo - xr) >> 2;
    request_far(y_lo);
    request_near(y_lo);
  }

  int buf = 0;
  for (int yt = y_lo; yt < y_hi; yt += C::TROWS, buf ^= 1) {
  // This wave's share of the buffer has landed: memory operations complete in issue order, and the younger ones are
  // the position scores the last step asked for (two per lane for a far block, up to 32 for a near one), which the
  // step waits for where it uses them, and the window stores issued after them (counting only the former waits for
  // as many of them as there were stores, no more than the step is about to wait for anyway).
  constexpr int kAsked = (kLaneT ? 1 : 0) + (kLoopT ? 1 : 0);
  if (far_n) wait_vmcnt<kAsked>();
  else if (kLaneT && GRP) wait_vmcnt<4 + (kLoopT ? 16 : 0)>();
  else wait_vmcnt<16 * kAsked>();
  __syncthreads();   // ... and everybody's; every wave is done with the other buffer (and the table is in LDS)
  const bool next_tiles = yt + C::TROWS < y_hi;
  if (next_tiles) {
    tiles_dma(yt + C::TROWS, buf ^ 1);
    stats_dma(yt + C::TROWS, buf ^ 1);
  }
#pragma unroll 1
  for (int sub = 0; sub < C::TROWS / kBwdStep; ++sub) {
    const int y0 = yt + sub * kBwdStep;
    if (y0 >= y_hi) break;
    const bool has_next = y0 + kBwdStep < y_hi;
    const char* Y1s = Ys + buf * C::REGION + sub * kBwdStep * C::RS;
    const char* Y2s = Y1s + C::TILE;
    const float* lse_s = stat_s + buf * 2 * 64 + sub * kBwdStep;
    const float* del_s = lse_s + 64;
    // ---- position scores (requested during the step before) ---------------------------------------------------
    // element v of lane (g, li): loop row yr = y0 + 8*(v/4) + 4g + v%4, lane row xr; i - j = +-(xr - yr)
    const bool far = far_n;
    const int d_far = dfar_n;
    d_lo = d_lo_n;
    off4[0] = off4_n[0], off4[1] = off4_n[1], off4[2] = off4_n[2], off4[3] = off4_n[3];
    f32x16 sacc, dpacc;   // S' starts from the position scores, dP' from -Delta: the products add on top
    if (kBias && far) {
      sacc = rank1_start<QT>(kLaneT ? (float)raw_lane[0] : 0.f, kLoopT ? (float)raw_loop[0] : 0.f, g);
    } else {
      bool grouped = false;
      if constexpr (kLaneT && sizeof(BT) == 2) grouped = GRP;
      if (grouped) {
        // Where no lane's six entries were moved back to stay inside its row, a group's first entry is entry 0 or 1 and
        // element e lies at most |e - e_min| further on: entries 0..3 for three of the elements, which one byte
        // permutation picks out of the first two registers, and 0..4 for the fourth.
        if (__builtin_amdgcn_ballot_w64((goff & 0xEEEEu) != 0u) == 0) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            if constexpr (sizeof(BT) == 2) {
              const uint32_t o4 = off4[v >> 2];
              const u32x3 w = raw3[v >> 2];
              const uint32_t idx = ((goff >> (4 * (v >> 2))) & 1u) + ((o4 >> (8 * (v & 3))) & 255u) - ((o4 >> (kDQ ? 24 : 0)) & 255u);
              // bytes 2 idx, 2 idx + 1 of {w[1], w[0]} into the low half of the result, zeros above
              uint32_t u = __builtin_amdgcn_perm(w[1], w[0], __umul24(idx, 0x0202u) + 0x0c0c0100u);
              if ((v & 3) == (kDQ ? 0 : 3)) u = idx == 4u ? (w[2] & 0xffffu) : u;
              sacc[v] = QT::scratch_to_f32((uint16_t)u) + (float)raw_loop[v];
            }
          }
        } else {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const uint32_t o4 = off4[v >> 2];
            const uint32_t idx = ((goff >> (4 * (v >> 2))) & 7u) + ((o4 >> (8 * (v & 3))) & 255u) - ((o4 >> (kDQ ? 24 : 0)) & 255u);
            if constexpr (sizeof(BT) == 2) sacc[v] = QT::scratch_to_f32(entry16(raw3[v >> 2], idx)) + (float)raw_loop[v];
          }
        }
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) sacc[v] = (float)raw_lane[v] + (float)raw_loop[v];
      }
    }
    if (has_next) request_far(y0 + kBwdStep);
    if (has_next) request_near(y0 + kBwdStep);   // as early as the registers are free: the round trip runs behind the whole step
                                                 // (in four parts between the parts of the step it was slower)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f32x4 del4 = {del_x, del_x, del_x, del_x};
      if (!kDQ) del4 = *(const f32x4*)(del_s + 8 * q4 + 4 * g);  // statistics of this lane's loop rows, four neighbours per read
#pragma unroll
      for (int e = 0; e < 4; ++e) dpacc[4 * q4 + e] = -del4[e];
    }
    // ---- S' and dP' ----------------------------------------------------------------------------------------
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const frag y1f = QT::load(Y1s + li * C::RS + (16 * s + 8 * g) * QT::SZ);
      const frag y2f = QT::load(Y2s + li * C::RS + (16 * s + 8 * g) * QT::SZ);
      sacc = QT::mma(y1f, x1f[s], sacc);
      dpacc = QT::mma(y2f, x2f[s], dpacc);
    }
    // ---- probabilities and score gradients (without the factor sm_scale, which the outputs take at the end) -------
    float ds[16], ds_run[16], pr[16], g_sum = 0.f;
    // a block that touches the end of a sequence or the causal diagonal masks its elements one by one
    const bool edge = xw0 + 31 >= Lb || y0 + kBwdStep > Lb ||
                      (p.causal && (kDQ ? y0 + kBwdStep - 1 > xw0 : xw0 + 31 > y0));
    // one branch for the block, not one per element: the common block carries no mask at all
    auto probabilities = [&](auto edge_tag) __attribute__((always_inline)) {
      constexpr bool EDGE = decltype(edge_tag)::value;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 lse4 = {lse_x, lse_x, lse_x, lse_x};
        if (!kDQ) lse4 = *(const f32x4*)(lse_s + 8 * q4 + 4 * g) * 1.4426950408889634f;   // to base 2, like lse_x
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = 4 * q4 + e;
          float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[v], c_log2, -lse4[e]));
          if (EDGE) {
            const int yr = y0 + 8 * q4 + 4 * g + e;
            const int i = kDQ ? xr : yr, j = kDQ ? yr : xr;
            if (!(x_ok && yr < Lb && (!p.causal || j <= i))) pv = 0.f;
          }
          pr[v] = pv;
          ds[v] = pv * dpacc[v];
          g_sum += ds[v];
        }
      }
    };
    if (edge) probabilities(std::true_type{});
    else probabilities(std::false_type{});
    if (kGrad) {
      // LDS float atomics are served a lane at a time on this hardware (160 clocks per instruction), so the adds are
      // plain reads and writes: the lanes of a half-wave own different rows, and the two halves (which share rows)
      // take turns.  Within a lane the table rows of the 16 elements are sorted, so elements of one entry are
      // neighbours: each write carries the sum of its run so far and the last write of a run, the complete one, wins.
      bool settled = false;  // nothing can have left the window
      if (far) {
        // a run of far blocks with one table row: the row sums add up in a register and enter the ring when the run ends
        g_far += g_sum;
        settled = has_next && far_n && dfar_n == d_far;  // the next block continues the run
        if (!settled) {
          const float run = wave_half_sum(g_far);
          if (g == 0) ring_x[d_far & (kRing - 1)] += run;
          g_far = 0.f;
        }
      } else {
        int dl[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          dl[v] = d_lo + (int)((off4[v >> 2] >> (8 * (v & 3))) & 255u);
          if (v > 0) ds_run[v] = ds[v] + (dl[v] == dl[v - 1] ? ds_run[v - 1] : 0.f);
          else ds_run[0] = ds[0];
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          if (g == half) {
            float old[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) old[v] = ring_x[dl[v] & (kRing - 1)];
#pragma unroll
            for (int v = 0; v < 16; ++v) ring_x[dl[v] & (kRing - 1)] = old[v] + ds_run[v];
          }
          wave_lds_fence();
        }
      }
      // Groups of four entries [4m, 4m + 3] the window has left behind: every later element of the row maps to a
      // table row at or beyond `d_edge` (that of the next step's first loop row; after the last step, the last
      // row's own entry, and its group goes too).  Up to eight groups per row and pass.
      int n_g = 0;
      if (!settled) {
        const int d_edge = delta_of(has_next ? (kDQ ? xr - (y0 + kBwdStep) : y0 + kBwdStep - xr) : (kDQ ? xr - (y_hi - 1) : y_hi - 1 - xr));
        int g_edge = d_edge >> 2;
        // Where the ring has the room (p.store_chunks = 8 or 4 groups; 1: none), what leaves before the last step leaves
        // in whole chunks, 64 or 32 bytes at a multiple of as much: every such sector of the tensor is then written
        // once, not in two pieces.
        if (has_next) {
          const int cm = p.store_chunks - 1;
          g_edge = kDir > 0 ? (g_edge & ~cm) : ((g_edge + cm + 1) & ~cm) - 1;
        }
        n_g = !x_ok ? 0 : kDir * (g_edge - g_next) + (has_next ? 0 : 1);
      }
      while (__builtin_amdgcn_ballot_w64(n_g > 0) != 0) {
        const int n_now = max(0, min(n_g, 8));
        if (g == 0) inf_w[li] = int2{g_next, n_now};
        wave_lds_fence();
        f32x4 val[4];
        int mm[4];
        bool act[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int rho = 8 * it + (lane >> 3);
          const int2 inf = inf_w[rho];
          mm[it] = inf.x + kDir * (lane & 7);
          act[it] = (lane & 7) < inf.y;
          const float* e = ring_w + rho * kRingStride + ((4 * mm[it]) & (kRing - 1));
          val[it] = f32x4{e[0], e[1], e[2], e[3]};
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int rho = 8 * it + (lane >> 3);
          if (act[it]) {
            float* e = ring_w + rho * kRingStride + ((4 * mm[it]) & (kRing - 1));
            e[0] = e[1] = e[2] = e[3] = 0.f;
            QT::store4(gw + ((uint32_t)(xw0 + rho) * row_elems + (uint32_t)(4 * mm[it])) * QT::SZ,
                       val[it][0] * c_sm, val[it][1] * c_sm, val[it][2] * c_sm, val[it][3] * c_sm);
          }
        }
        wave_lds_fence();
        g_next += kDir * n_now;
        n_g -= n_now;
      }
    }
    // ---- outputs: contraction over the loop rows, which are the accumulator registers ------------------------------
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      f32x8 d8, p8;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        d8[e] = ds[8 * c + e];
        p8[e] = pr[8 * c + e];
      }
      const frag dsf = QT::from_f32(d8), pf = QT::from_f32(p8);
#pragma unroll
      for (int d = 0; d < DBLKS; ++d) {
        acc1[d] = QT::mma(VtLoad<QT>::get(Y1s, C::RS, c, d, lane), dsf, acc1[d]);       // dQ^T += K^T dS' / dK^T += Q^T dS'
        if (!kDQ) acc2[d] = QT::mma(VtLoad<QT>::get(Y2s, C::RS, c, d, lane), pf, acc2[d]);  // dV^T += dO^T P'
      }
    }
  }
  }

  };
  if (kBias && sizeof(typename QT::scratch_t) == 2) {
    __syncthreads();  // the table is in LDS
    bool wide = false;
    for (int x = lane; x + 3 < 2 * p.R + 1; x += 64) wide |= lut_s[x + 3] - lut_s[x] > 3 || lut_s[x + 3] < lut_s[x];
    grp_ok = __builtin_amdgcn_ballot_w64(wide) == 0;
  }
  if (grp_ok) run(std::true_type{});
  else run(std::false_type{});

  // The groups of a row that the loop never reached (table rows beyond the ones its relative positions map to: rows
  // near the ends of a sequence, and half of every row of a causal call) are written as zeros here, so that every
  // entry of a real token's row is stored exactly once and the caller need not clear the tensor.
  if (kGrad) {
    const int g_first = delta_of(kDQ ? xr - y_lo : y_lo - xr) >> 2;        // where the loop began; g_next: one past where it ended
    const int lo = kDir < 0 ? g_next + 1 : g_first, hi = kDir < 0 ? g_first : g_next - 1;
    const int n_groups = (2 * p.S) >> 2;
    if (g == 0) inf_w[li] = x_ok ? int2{lo, hi} : int2{0, n_groups - 1};   // rows past the end: nothing to write
    wave_lds_fence();
#pragma unroll 1
    for (int it = 0; it < 4; ++it) {
      const int rho = 8 * it + (lane >> 3);
      const int2 inf = inf_w[rho];
      if (__builtin_amdgcn_ballot_w64(inf.x > 0 || inf.y < n_groups - 1) == 0) continue;
      for (int m = lane & 7; m < n_groups; m += 8)
        if (m < inf.x || m > inf.y)
          QT::store4(gw + ((uint32_t)(xw0 + rho) * row_elems + (uint32_t)(4 * m)) * QT::SZ, 0.f, 0.f, 0.f, 0.f);
    }
  }

  if (!x_ok) return;
  auto write = [&](char* ptr, int64_t sb, int64_t st, int64_t sh, const f32x16 (&acc)[DBLKS]) {
    char* row = ptr + (b * sb + (int64_t)(tok0 + xr) * st + (int64_t)h * sh) * QT::SZ;
#pragma unroll
    for (int d = 0; d < DBLKS; ++d)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        QT::store4(row + (32 * d + 8 * q4 + 4 * g) * QT::SZ, acc[d][4 * q4], acc[d][4 * q4 + 1], acc[d][4 * q4 + 2], acc[d][4 * q4 + 3]);
  };
#pragma unroll
  for (int d = 0; d < DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc1[d][v] *= c_sm;  // dS' went into dQ / dK without sm_scale
  if (kDQ) {
    write(p.dq, p.dq_sb, p.dq_st, p.dq_sh, acc1);
  } else {
    write(p.dk, p.dk_sb, p.dk_st, p.dk_sh, acc1);
    write(p.dv, p.dv_sb, p.dv_st, p.dv_sh, acc2);
  }
}

template <class QT, int D, int ROLE, bool C2P, bool P2C>
int launch_bwd_one(const FdbBwdParams& p, hipStream_t stream) {
  auto kern = fdb_bwd_kernel<QT, D, ROLE, C2P, P2C>;
  static_assert(BCfg<QT, D>::fixed_lds_bytes() + 4096 <= 160 * 1024, "LDS budget");
  const int lds = BCfg<QT, D>::lds_bytes((C2P || P2C) ? p.R : 0);
  if (lds > 160 * 1024) return FDB_ERR_SPAN;  // the table does not fit beside the tiles
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = fdb_set_lds_once((const void*)kern, 160 * 1024, lds_set);
  if (e != hipSuccess) return (int)e;
  const unsigned tiles = (unsigned)((p.L + FDB_BM - 1) / FDB_BM);
  hipLaunchKernelGGL(kern, dim3(tiles * (unsigned)p.H * (unsigned)p.B), dim3(kBwdThreads), lds, stream, p);
  return (int)hipGetLastError();
}

template <class QT, int D>
int launch_bwd_roles(const FdbBwdParams& p, hipStream_t stream) {
  int rc;
  if (p.c2p && p.p2c) {
    rc = launch_bwd_one<QT, D, 0, true, true>(p, stream);
    return rc ? rc : launch_bwd_one<QT, D, 1, true, true>(p, stream);
  }
  if (p.c2p) {
    rc = launch_bwd_one<QT, D, 0, true, false>(p, stream);
    return rc ? rc : launch_bwd_one<QT, D, 1, true, false>(p, stream);
  }
  if (p.p2c) {
    rc = launch_bwd_one<QT, D, 0, false, true>(p, stream);
    return rc ? rc : launch_bwd_one<QT, D, 1, false, true>(p, stream);
  }
  rc = launch_bwd_one<QT, D, 0, false, false>(p, stream);
  return rc ? rc : launch_bwd_one<QT, D, 1, false, false>(p, stream);
}

template <class QT>
int launch_bwd_d(const FdbBwdParams& p, int head_dim, hipStream_t stream) {
  switch (head_dim) {
    case 32: return launch_bwd_roles<QT, 32>(p, stream);
    case 64: return launch_bwd_roles<QT, 64>(p, stream);
    case 128: return launch_bwd_roles<QT, 128>(p, stream);
    default: return FDB_ERR_HEAD_DIM;
  }
}

}  // namespace

int fdb_launch_bwd(const FdbBwdParams& p, int dtype, int head_dim, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  switch (dtype) {
    case FDB_BF16: return launch_bwd_d<Bf16Tr>(p, head_dim, stream);
    case FDB_F16: return launch_bwd_d<F16Tr>(p, head_dim, stream);
    case FDB_F32: return launch_bwd_d<F32Tr>(p, head_dim, stream);
    default: return FDB_ERR_DTYPE;
  }
}
