// Fused DeBERTa disentangled-attention forward for gfx950 (MI355X, CDNA4).
//
// One workgroup = 4 wavefronts = 128 query rows of one (sequence, head); each wavefront owns 32
// rows.  The main loop walks the keys 64 at a time.  Everything is computed "transposed" so that a
// lane owns one query row:  S^T = K Q^T  (MFMA 32x32, M = key, N = query), the soft-max statistics
// of a row live in one lane (and its partner lane^32), and  O^T = V^T P^T  takes P straight from
// the S accumulators as its B operand.
//
// Position terms (what the reference reads from two pre-multiplied [B,H,L,2S] tensors with a
// per-element float log-bucket, src/flashdeberta/ops/flash_attention.py:236-268).  delta(r),
// r = i - j, is an integer table that is constant for |r| >= R.  The key tiles of a query tile
// therefore fall into three consecutive ranges:
//   far-left  (every r >= R):  delta == delta(+R).  The content->position term is a per-row constant
//              a_i = q_i . K_r[delta], folded into the exponent; the position->content term
//              k_j . Q_r[delta] is folded into the MFMA by using q_i + Q_r[delta] as the query.
//   near      the tile's relative positions form one contiguous range, so its bias values are
//              C[r, i] = q_i . K_r[delta(r)] and P[r, j] = k_j . Q_r[delta(r)]: two more MFMA
//              products whose A rows are gathered through the table.  They are parked in LDS
//              indexed by r, and element (i, j) adds C[i-j, i] + P[i-j, j] -- addresses affine in
//              (i, j), no per-element bucket arithmetic, no trip to HBM.
//   far-right (every r <= -R): like far-left with delta(-R).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

using namespace fdb;

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kC2pRows = 96;     // 32 + 64 - 1 relative positions per wave tile, padded to 3 MFMA blocks
constexpr int kC2pStride = 100;  // elements per query row of the wave's C[i][r] scratch
constexpr int kP2cRows = 192;    // 128 + 64 - 1 per workgroup tile, padded to 6 MFMA blocks
constexpr int kP2cStride = 196;  // elements per key row of the workgroup's P[j][r] scratch
constexpr int kRing = 256;       // rows of a ring: the 191 relative positions of a tile + the 64 of the batch in flight

// Kernel modes.  kFused: one kernel walks every tile (the rows of the position products are
// gathered from global memory).  kFarOnly: the near tiles are left to a second launch; this one
// writes the far tiles' partial result (rows normalised over the far keys, their log-sum-exp,
// zero / -inf where there is none).  kNearRing: that second launch -- near tiles only, the rows
// E_K[r] = K_r[delta(r)], E_Q[r] = Q_r[delta(r)] of the relative positions in reach staged once per
// workgroup in two LDS rings that slide 64 positions per key tile, and the far partial merged in
// the epilogue.
constexpr int kFused = 0, kFarOnly = 1, kNearRing = 2;


template <class QT, class VT, int D>
struct Cfg {
  using ST = typename QT::scratch_t;
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLKS = D / 32;
  static constexpr int K_RS = D * QT::SZ + 16;  // LDS row stride (bytes) of the K tile
  static constexpr int V_RS = D * VT::SZ + 16;
  static constexpr int K_BYTES = FDB_BN * K_RS;
  static constexpr int V_BYTES = FDB_BN * V_RS;
  static constexpr int K_CHUNKS = (FDB_BN * D * QT::SZ / 16 + kThreads - 1) / kThreads;  // 16-byte chunks per thread
  static constexpr int V_CHUNKS = (FDB_BN * D * VT::SZ / 16 + kThreads - 1) / kThreads;
  static constexpr int C2P_BYTES = kWaves * 32 * kC2pStride * (int)sizeof(ST);
  static constexpr int P2C_BYTES = FDB_BN * kP2cStride * (int)sizeof(ST);
  static constexpr int RING_BYTES = kRing * K_RS;  // one ring of expanded relative-embedding rows
  // Tiles of 128-byte rows with no position products in the kernel go global -> LDS directly,
  // three K/V buffers deep (see the kernel).
  static constexpr bool DMA_OK = QT::SZ == 2 && VT::SZ == 2 && D == 64;
  static constexpr int DMA_TILE = FDB_BN * 128, DMA_BUF = 2 * DMA_TILE, DMA_BYTES = 3 * DMA_BUF;
  // fp32 at head_dim 128 with both position terms: K, V and the two bias scratches together exceed a
  // CU's 160 KB, so V takes K's place in LDS once the tile's scores are done (kv_alias).
  static constexpr bool kv_alias(bool c2p, bool p2c) {
    return K_BYTES + V_BYTES + (c2p ? C2P_BYTES : 0) + (p2c ? P2C_BYTES : 0) > 160 * 1024;
  }
  static constexpr int lds_bytes(bool c2p, bool p2c) {
    return K_BYTES + (kv_alias(c2p, p2c) ? 0 : V_BYTES) + (c2p ? C2P_BYTES : 0) + (p2c ? P2C_BYTES : 0);
  }
  static constexpr int lds_bytes_mode(int mode, bool c2p, bool p2c) {
    if (DMA_OK && (mode == 1 || (mode == 0 && !c2p && !p2c))) return DMA_BYTES;
    return mode == 1 ? lds_bytes(false, false)
                     : lds_bytes(c2p, p2c) + (mode == 2 ? (c2p ? RING_BYTES : 0) + (p2c ? RING_BYTES : 0) : 0);
  }
};

// [64 x ROW_BYTES] tile: global -> registers -> LDS.  Rows past the end of the sequence re-read the
// last valid row (finite data, no predication); their scores are masked to -inf before the soft-max.
template <int ROW_BYTES, int NCH>
__device__ __forceinline__ void tile_load(u32x4 (&reg)[NCH], const char* gbase, uint32_t row_stride_bytes, int j0,
                                          int n_rows, int tid) {
  constexpr int CPR = ROW_BYTES / 16;
  constexpr int TOTAL = FDB_BN * CPR;
#pragma unroll
  for (int n = 0; n < NCH; ++n) {
    const int c = tid + n * kThreads;
    const int row = min(j0 + min(c / CPR, FDB_BN - 1), n_rows - 1), cc = c % CPR;
    reg[n] = *(const u32x4*)(gbase + (uint64_t)(uint32_t)row * row_stride_bytes + cc * 16);  // one 32 x 32 -> 64-bit multiply-add
  }
}
template <int ROW_BYTES, int RS, int NCH>
__device__ __forceinline__ void tile_store(char* lds, const u32x4 (&reg)[NCH], int tid) {
  constexpr int CPR = ROW_BYTES / 16;
  constexpr int TOTAL = FDB_BN * CPR;
#pragma unroll
  for (int n = 0; n < NCH; ++n) {
    const int c = tid + n * kThreads;
    const int row = c / CPR, cc = c % CPR;
    if (TOTAL % kThreads == 0 || c < TOTAL) *(u32x4*)(lds + row * RS + cc * 16) = reg[n];
  }
}

// One key tile after its scores are in sacc (raw products, position terms already added where the
// tile needs them element-wise): mask, online soft-max in base 2, O^T += V^T P^T.
//   x = sacc * x_scale + row_add   (row_add: the per-row constant of a far tile, already scaled)
template <class VT, int D, bool MASK, class VL>
__device__ __forceinline__ void softmax_pv(f32x16 (&sacc)[2], f32x16 (&o_acc)[D / 32], float& m_run, float& l_run,
                                           float x_scale, float row_add, const VL& vload, int lane, int j0,
                                           int i, int Lb, bool causal) {
  using vfrag = typename VT::frag;
  const int g = lane >> 5;
  if constexpr (MASK) {
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + 32 * jb + 8 * (v >> 2) + 4 * g + (v & 3);
        if (j >= Lb || (causal && j > i)) sacc[jb][v] = -INFINITY;
      }
  }
  float mx = sacc[0][0];
#pragma unroll
  for (int jb = 0; jb < 2; ++jb)
#pragma unroll
    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[jb][v]);
  mx = wave_half_max(mx) * x_scale + row_add;  // x_scale > 0
  if (__any(mx > m_run + kLazyTau)) {
    const float m_new = (mx > m_run + kLazyTau) ? mx : m_run;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // m_run = -inf on the first tile: 0
    l_run *= alpha;
    m_run = m_new;
#pragma unroll
    for (int d = 0; d < D / 32; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
  }
  const float off = row_add - m_run;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    f32x8 pv;
#pragma unroll
    for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[c >> 1][8 * (c & 1) + e], x_scale, off));
    const vfrag pf = VT::from_f32(pv);
    l_run = sum8(pv, l_run);
#pragma unroll
    for (int d = 0; d < D / 32; ++d) {
      const vfrag vf = vload(c, d);
      o_acc[d] = VT::mma(vf, pf, o_acc[d]);
    }
  }
}

// The same for tiles whose scores leave the MFMA ready for the exponential: the query operand
// carries the soft-max scale and the accumulator started from negm = row_add - (reference point of
// the row), so sacc = x - reference.  The reference point moves only when the tile maximum exceeds
// it by more than the lazy threshold (or on the row's first tile, whose reference is 0); the tile
// at hand and negm are then shifted to the new one.
template <class VT, int D, bool MASK, class VL>
__device__ __forceinline__ void softmax_pv_pre(f32x16 (&sacc)[2], f32x16 (&o_acc)[D / 32], float& m_run, float& l_run,
                                               float row_add, f32x16& negm, const VL& vload, int lane, int j0,
                                               int i, int Lb, bool causal) {
  using vfrag = typename VT::frag;
  const int g = lane >> 5;
  if constexpr (MASK) {
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + 32 * jb + 8 * (v >> 2) + 4 * g + (v & 3);
        if (j >= Lb || (causal && j > i)) sacc[jb][v] = -INFINITY;
      }
  }
  float mx = sacc[0][0];
#pragma unroll
  for (int jb = 0; jb < 2; ++jb)
#pragma unroll
    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[jb][v]);
  mx = wave_half_max(mx);
  const bool first = m_run == -INFINITY;
  if (__any(mx > kLazyTau || first)) {
    const bool mv = mx > kLazyTau || first;
    const float shift = mv ? mx : 0.f;
    const float alpha = first ? 0.f : __builtin_amdgcn_exp2f(-shift);
    m_run = (first ? 0.f : m_run) + shift;
    l_run *= alpha;
#pragma unroll
    for (int d = 0; d < D / 32; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int v = 0; v < 16; ++v) sacc[jb][v] -= shift;
    const float nm = row_add - m_run;
#pragma unroll
    for (int v = 0; v < 16; ++v) negm[v] = nm;
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    f32x8 pv;
#pragma unroll
    for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f(sacc[c >> 1][8 * (c & 1) + e]);
    const vfrag pf = VT::from_f32(pv);
    l_run = sum8(pv, l_run);
#pragma unroll
    for (int d = 0; d < D / 32; ++d) {
      const vfrag vf = vload(c, d);
      o_acc[d] = VT::mma(vf, pf, o_acc[d]);
    }
  }
}

// Two workgroups share a CU (and its 512 registers per lane) when the LDS footprint allows it.
template <class QT, class VT, int D, bool C2P, bool P2C, int MODE>
constexpr int min_blocks() {
  const int lds = Cfg<QT, VT, D>::lds_bytes_mode(MODE, C2P, P2C);
  if (MODE == kFarOnly) return 3;  // the far zones need the shifted query and the per-row constants on top of the plain kernel
  if (MODE == kNearRing) return 2;  // one workgroup fits a CU; the bound keeps every value in the 256 registers VALU code can read
  // three: 170 registers, the plain loop's working set at head_dim <= 64; head_dim 128 doubles the output accumulators
  // and the query fragments: two workgroups (256 registers) for the 16-bit types, one (512) for fp32
  if (D >= 128) return QT::SZ == 4 ? 1 : (lds <= 80 * 1024 ? 2 : 1);
  return (lds <= 40 * 1024 && QT::SZ < 4) ? 3 : lds <= 80 * 1024 ? 2 : 1;  // fp32 fragments are twice the registers
}

template <class QT, class VT, int D, bool FP8, bool C2P, bool P2C, int MODE>
__global__ __launch_bounds__(kThreads, (min_blocks<QT, VT, D, C2P, P2C, MODE>())) void fdb_attn_kernel(const FdbKParams p) {
  using C = Cfg<QT, VT, D>;
  using ST = typename C::ST;
  using qfrag = typename QT::frag;
  constexpr bool FAR_ONLY = MODE == kFarOnly, RING = MODE == kNearRing;
  static_assert(!RING || (!FP8 && QT::SZ == 2 && (C2P || P2C)), "the ring mode is for the position terms of the 16-bit types");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr bool KV_ALIAS = C::kv_alias(C2P, P2C);
  static_assert(!KV_ALIAS || MODE == kFused, "only the fused mode shares one buffer between K and V");
  char* Ks = smem;
  char* Vs = KV_ALIAS ? Ks : Ks + C::K_BYTES;
  ST* c2pS = (ST*)(Ks + C::K_BYTES + (KV_ALIAS ? 0 : C::V_BYTES));
  ST* p2cS = (ST*)((char*)c2pS + (C2P ? C::C2P_BYTES : 0));
  char* EK = (char*)p2cS + (P2C ? C::P2C_BYTES : 0);
  char* EQ = EK + (C2P ? C::RING_BYTES : 0);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in scalar registers: what depends on it alone stays scalar
  const int lane = tid & 63, li = lane & 31, g = lane >> 5;
  int xq, h;
  block_map((int)blockIdx.x, p.grid_x, p.H, p.tiles_per_seq, p.cu == nullptr,
            MODE == kFarOnly ? (p.causal ? kLastFirst : kEdgesFirst) : (MODE == kNearRing ? kMiddleFirst : kNatural), xq, h);

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
      fill_pad_rows<D * VT::SZ>(p.out + ((int64_t)b * p.o_sb + (int64_t)h * p.o_sh) * VT::SZ, p.o_st * VT::SZ, xq % p.tiles_per_seq,
                                p.L, tok0, Lb, sl < 0 ? VT::NAN_WORD : 0u, tid);
    if (m0 >= Lb) return;
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; oo = b * p.o_sb;
  }
  const char* qb = p.q + (qo + (int64_t)tok0 * p.q_st + (int64_t)h * p.q_sh) * QT::SZ;
  const char* kb = p.k + (ko + (int64_t)tok0 * p.k_st + (int64_t)h * p.k_sh) * QT::SZ;
  const char* vb = p.v + (vo + (int64_t)tok0 * p.v_st + (int64_t)h * p.v_sh) * VT::SZ;
  char* ob = p.out + (oo + (int64_t)tok0 * p.o_st + (int64_t)h * p.o_sh) * VT::SZ;
  const char* pkb = C2P ? p.pk + (int64_t)h * p.pk_sh * QT::SZ : nullptr;
  const char* pqb = P2C ? p.pq + (int64_t)h * p.pq_sh * QT::SZ : nullptr;
  const uint32_t k_rsb = (uint32_t)(p.k_st * QT::SZ), v_rsb = (uint32_t)(p.v_st * VT::SZ);  // the host checks that they fit

  // fp8: raw products are in units of (q_scale*k_scale); bring the two position products to the
  // same unit so that one factor converts the sum.
  float x_scale = p.scale_log2, c2p_mul = 1.f, p2c_mul = 1.f;
  if constexpr (FP8) {
    const float qs = p.qs[h], ks = p.ks[h];
    x_scale *= qs * ks;
    if constexpr (C2P) c2p_mul = p.pks[h] / ks;
    if constexpr (P2C) p2c_mul = p.pqs[h] / qs;
  }

  const int iw0 = m0 + wave * 32;  // first row of this wave
  const int i = iw0 + li;          // this lane's query row (local to the sequence)

  qfrag qf[C::KSTEPS];
#pragma unroll
  for (int s = 0; s < C::KSTEPS; ++s)
    qf[s] = (i < Lb) ? QT::load(qb + ((int64_t)i * p.q_st + 16 * s + 8 * g) * QT::SZ) : QT::zero();

  // ---- tile ranges ---------------------------------------------------------------------------
  int j_end = Lb;
  if (p.causal) j_end = min(Lb, m0 + FDB_BM);
  const int n_tiles = (j_end + FDB_BN - 1) / FDB_BN;
  constexpr bool kHasPos = C2P || P2C;
  constexpr bool kFarOk = kHasPos && !FP8;  // fp8 cannot fold Q_r into an fp8 query: all tiles take the near path
  int t_near0 = 0, t_near1 = n_tiles;       // near tiles are [t_near0, t_near1)
  if constexpr (!kHasPos) {
    t_near0 = t_near1 = n_tiles;            // no position term: every tile is a plain one
  } else if constexpr (kFarOk) {
    const int lim = m0 - (FDB_BN - 1) - p.R;  // far-left: j0 <= lim
    t_near0 = lim >= 0 ? min(n_tiles, lim / FDB_BN + 1) : 0;
    t_near1 = max(t_near0, min(n_tiles, (m0 + FDB_BM - 1 + p.R + FDB_BN - 1) / FDB_BN));  // far-right: j0 >= m0+127+R
  }

  // per-row constants and shifted queries of the two far zones.  Except in fp8 the far / plain
  // tiles use queries that carry the soft-max scale (PRE), and their accumulators start from negm.
  f32x16 o_acc[C::DBLKS];
#pragma unroll
  for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // l_run: this lane's half of the row sum
  constexpr bool PRE = !FP8;
  float a_far = 0.f;  // scaled to the exponent's unit
  qfrag qfar[C::KSTEPS];
  f32x16 negm;
#pragma unroll
  for (int v = 0; v < 16; ++v) negm[v] = 0.f;
  auto setup_far = [&](int side) __attribute__((always_inline)) {  // side 0: far-left (delta(+R)), 1: far-right (delta(-R))
    const int delta = kHasPos ? p.lut[side == 0 ? 2 * p.R : 0] : 0;
    // A far-only run needs the plain query only here, twice per workgroup: it is loaded again instead of
    // being held in sixteen registers through the loops.
    qfrag qs[C::KSTEPS];
#pragma unroll
    for (int s = 0; s < C::KSTEPS; ++s) {
      if constexpr (MODE == kFarOnly)
        qs[s] = (i < Lb) ? QT::load(qb + ((int64_t)i * p.q_st + 16 * s + 8 * g) * QT::SZ) : QT::zero();
      else
        qs[s] = qf[s];
    }
    if constexpr (C2P) {
      const char* row = pkb + (int64_t)delta * p.pk_sr * QT::SZ;
      float acc = 0.f;
#pragma unroll
      for (int s = 0; s < C::KSTEPS; ++s) {
        const f32x8 a = QT::to_f32(QT::load(row + (16 * s + 8 * g) * QT::SZ)), q8 = QT::to_f32(qs[s]);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(a[e], q8[e], acc);
      }
      a_far = wave_half_sum(acc) * x_scale;
    }
    if constexpr (P2C) {
      const char* row = pqb + (int64_t)delta * p.pq_sr * QT::SZ;
#pragma unroll
      for (int s = 0; s < C::KSTEPS; ++s)
        qfar[s] = QT::from_f32((QT::to_f32(qs[s]) + QT::to_f32(QT::load(row + (16 * s + 8 * g) * QT::SZ))) * x_scale);
    } else {
#pragma unroll
      for (int s = 0; s < C::KSTEPS; ++s) qfar[s] = QT::from_f32(QT::to_f32(qs[s]) * x_scale);
    }
    const float nm = a_far - (m_run == -INFINITY ? 0.f : m_run);
#pragma unroll
    for (int v = 0; v < 16; ++v) negm[v] = nm;
  };


  // The far tiles of this workgroup: [zl0, zl1) left of the near range and [zr0, zr1) right of it.  A
  // far-only run may be split over p.far_parts workgroups per query tile (blockIdx.y), each taking an equal
  // share of the far tiles in walking order and leaving a partial result of its own.
  // One-kernel mode with p.key_parts > 1: this workgroup walks its share [t_lo, t_hi) of the key tiles only, and the
  // three ranges are cut to it.
  const int part = (FAR_ONLY || (MODE == kFused && p.key_parts > 1)) ? (int)blockIdx.y : 0;
  int t_lo = 0, t_hi = n_tiles;
  if (MODE == kFused && p.key_parts > 1) {
    t_lo = (int)((int64_t)n_tiles * part / p.key_parts);
    t_hi = (int)((int64_t)n_tiles * (part + 1) / p.key_parts);
    const int n0 = t_near0, n1 = t_near1;
    t_near0 = min(max(n0, t_lo), t_hi);
    t_near1 = min(max(n1, t_lo), t_hi);
  }
  int zl0 = t_lo, zl1 = t_near0, zr0 = t_near1, zr1 = t_hi;
  if (FAR_ONLY && p.far_parts > 1) {
    const int n_far = t_near0 + (n_tiles - t_near1);
    const int o_lo = (int)((int64_t)n_far * part / p.far_parts), o_hi = (int)((int64_t)n_far * (part + 1) / p.far_parts);
    zl0 = min(o_lo, t_near0);
    zl1 = min(o_hi, t_near0);
    zr0 = t_near1 + max(o_lo - t_near0, 0);
    zr1 = t_near1 + max(o_hi - t_near0, 0);
  }
  // the tile walked after tile t (far-only runs jump over the near range, ring runs walk nothing else)
  const int t_end = RING ? t_near1 : zr1;
  auto next_tile = [&](int t) __attribute__((always_inline)) {
    return (FAR_ONLY && t + 1 >= zl1 && t + 1 < zr0) ? zr0 : t + 1;
  };
  // Two ways of staging the K and V tiles.
  //
  // Through registers (any row size): global -> registers one tile ahead, registers -> padded LDS
  // rows between two barriers.
  //
  // Direct (128-byte rows, kernels without position products): global_load_lds writes the tile
  // into one of three LDS buffers two tiles ahead; one barrier per tile, no staging registers, and
  // the loads have two tile periods to land.  A load instruction fills 1 KB = 8 rows, lane l the
  // 16-byte slot l; rows are not padded, so slot (row, s) holds chunk s ^ f(row) of the row,
  // f(row) = 4*bit1(row) | bits3:2(row): sixteen consecutive rows put one chunk in sixteen
  // different bank groups (the K fragments), and four consecutive rows put chunks 0..3 in disjoint
  // ones (the transposing V reads).
  constexpr bool DMA = C::DMA_OK && !RING && !FP8 && (FAR_ONLY || !kHasPos);
  u32x4 kreg[C::K_CHUNKS], vreg[C::V_CHUNKS];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_AS char*)smem;
  int dma_cur = 0;                 // byte offset of the buffer that holds the tile at hand
  uint32_t kcur[4], vcur[4];       // this lane's read offsets into it
  uint32_t klane = 0, vlane = 0;
  if constexpr (DMA) {
    const int fl = 4 * ((li >> 1) & 1) | ((li >> 2) & 3);  // f(row) of the K fragment rows 32*jb + li
    klane = li * 128 + ((g ^ fl) * 16);                    // chunk 2*s + g: slot (2*s) ^ g ^ f
    // V^T operand (c, d-block db, half h): row 16c + 8h + 4*(grp/2) + s16/4, 8-byte unit 8db + 4*(grp%2) + s16%4
    const int s16 = lane & 15, grp = lane >> 4;
    const int slotl = (2 * (grp & 1) + ((s16 & 3) >> 1)) ^ (4 * ((s16 >> 3) & 1)) ^ (grp >> 1);  // chunk ^ f, less (4db) ^ (2h)
    vlane = (4 * (grp >> 1) + (s16 >> 2)) * 128 + slotl * 16 + (s16 & 1) * 8;
  }
  // The tile's first row travels as the scalar base of the load, the lane's place in the tile as
  // its offset: the row is clamped to the last one of the sequence (rows past the end re-read it).
  // A tile inside the sequence uses lane offsets computed once; only the last, ragged tile clamps its rows.
  uint32_t dma_koff[2] = {0, 0}, dma_voff[2] = {0, 0};
  if constexpr (DMA) {
#pragma unroll
    for (int q2 = 0; q2 < 2; ++q2) {
      const uint32_t row = (uint32_t)(16 * wave + 8 * q2 + (lane >> 3));
      const uint32_t c16 = ((lane & 7) ^ (4 * ((lane >> 4) & 1)) ^ (lane >> 5) ^ (2 * q2)) * 16;
      dma_koff[q2] = row * k_rsb + c16;
      dma_voff[q2] = row * v_rsb + c16;
    }
  }
  auto dma_issue = [&](int tile, int bufoff) __attribute__((always_inline)) {
    static_assert(kDmaLoadsPerTile == 2 * 2, "two 8-row groups of K and of V per wave and tile");
    const char* kt = kb + (uint64_t)(uint32_t)(tile * FDB_BN) * k_rsb;
    const char* vt = vb + (uint64_t)(uint32_t)(tile * FDB_BN) * v_rsb;
    const int last = Lb - 1 - tile * FDB_BN;
    if (last >= FDB_BN - 1) {
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {  // this wave's two 8-row groups of K and of V
        const uint32_t dst = lds0 + bufoff + (2 * wave + q2) * 1024;
        dma16sn(kt, dma_koff[q2], dst);
        dma16sn(vt, dma_voff[q2], dst + C::DMA_TILE);
      }
    } else {
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {
        const uint32_t row = (uint32_t)min(16 * wave + 8 * q2 + (lane >> 3), last);
        const uint32_t c16 = ((lane & 7) ^ (4 * ((lane >> 4) & 1)) ^ (lane >> 5) ^ (2 * q2)) * 16;  // slot ^ f(row), unclamped row
        const uint32_t dst = lds0 + bufoff + (2 * wave + q2) * 1024;
        dma16sn(kt, row * k_rsb + c16, dst);
        dma16sn(vt, row * v_rsb + c16, dst + C::DMA_TILE);
      }
    }
  };
  {
    const int first = RING ? t_near0 : next_tile(zl0 - 1);
    if (first < t_end) {
      if constexpr (DMA) {
        dma_issue(first, 0);
        const int second = next_tile(first);
        if (second < t_end) dma_issue(second, C::DMA_BUF);
        dma_cur = 2 * C::DMA_BUF;  // stage() steps to buffer 0
      } else {
        tile_load<D * QT::SZ>(kreg, kb, k_rsb, first * FDB_BN, Lb, tid);
        tile_load<D * VT::SZ>(vreg, vb, v_rsb, first * FDB_BN, Lb, tid);  // kv_alias: stays in registers until stage_v
      }
    }
  }

  auto stage = [&](int t) __attribute__((always_inline)) {
    if constexpr (DMA) {
      const int nt = next_tile(t);
      if (nt < t_end) wait_vmcnt<kDmaLoadsPerTile>(); else wait_vmcnt<0>();  // this wave's part of tile t has landed (tile nt's may still fly)
      __syncthreads();  // ... and everyone's; every wave is done with the tile before
      dma_cur = dma_cur == 2 * C::DMA_BUF ? 0 : dma_cur + C::DMA_BUF;
      if (nt < t_end) {
        const int nn = next_tile(nt);
        if (nn < t_end) dma_issue(nn, dma_cur >= C::DMA_BUF ? dma_cur - C::DMA_BUF : 2 * C::DMA_BUF);  // the buffer the tile before used
      }
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        kcur[x] = (klane ^ (32 * x)) + (dma_cur + lds0);  // absolute LDS addresses
        vcur[x] = (vlane ^ (64 * (x >> 1) ^ 32 * (x & 1))) + (dma_cur + lds0 + C::DMA_TILE);
      }
    } else {
      __syncthreads();  // every wave is done with the previous tile and its bias scratch
      tile_store<D * QT::SZ, C::K_RS>(Ks, kreg, tid);
      if constexpr (!KV_ALIAS) tile_store<D * VT::SZ, C::V_RS>(Vs, vreg, tid);
      __syncthreads();
      const int nt = next_tile(t);
      if (nt < t_end) {  // next tile's global loads fly during this tile's math
        tile_load<D * QT::SZ>(kreg, kb, k_rsb, nt * FDB_BN, Lb, tid);
        if constexpr (!KV_ALIAS) tile_load<D * VT::SZ>(vreg, vb, v_rsb, nt * FDB_BN, Lb, tid);
      }
    }
  };
  // K and V in one buffer: once every wave has its scores of tile t, V replaces K.
  auto stage_v = [&](int t) __attribute__((always_inline)) {
    if constexpr (KV_ALIAS) {
      __syncthreads();
      tile_store<D * VT::SZ, C::V_RS>(Vs, vreg, tid);
      __syncthreads();
      const int nt = next_tile(t);
      if (nt < t_end) tile_load<D * VT::SZ>(vreg, vb, v_rsb, nt * FDB_BN, Lb, tid);
    }
  };
  auto vload = [&](int c, int d) __attribute__((always_inline)) {
    if constexpr (DMA) {
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)((LDS_AS char*)(uintptr_t)vcur[2 * d] + 2048 * c));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)((LDS_AS char*)(uintptr_t)vcur[2 * d + 1] + 2048 * c + 1024));
      return __builtin_bit_cast(typename VT::frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    } else {
      return VtLoad<VT>::get(Vs, C::V_RS, c, d, lane);
    }
  };
  f32x16 zero16;
#pragma unroll
  for (int v = 0; v < 16; ++v) zero16[v] = 0.f;
  auto qk = [&](f32x16 (&sacc)[2], const qfrag (&qq)[C::KSTEPS], const f32x16& init) __attribute__((always_inline)) {
    if constexpr (DMA) {
      // every K fragment of the tile is requested before the first MFMA waits for one
      qfrag kf[2][C::KSTEPS];
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int s = 0; s < C::KSTEPS; ++s) kf[jb][s] = *(LDS_AS const qfrag*)((LDS_AS const char*)(uintptr_t)kcur[s] + jb * 4096);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < C::KSTEPS; ++s)
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) sacc[jb] = QT::mma(kf[jb][s], qq[s], s == 0 ? init : sacc[jb]);
    } else {
#pragma unroll
      for (int jb = 0; jb < 2; ++jb) {
#pragma unroll
        for (int s = 0; s < C::KSTEPS; ++s) {
          const qfrag kf = QT::load(Ks + (jb * 32 + li) * C::K_RS + (16 * s + 8 * g) * QT::SZ);
          sacc[jb] = QT::mma(kf, qq[s], s == 0 ? init : sacc[jb]);
        }
      }
    }
  };
  // Tiles that need no mask: entirely inside the sequence and, when causal, entirely below the
  // diagonal of every row of the workgroup, i.e. ending at or before its first row m0.
  const int n_full = p.causal ? min(Lb, m0) / FDB_BN : Lb / FDB_BN;
  auto far_loop = [&](auto mask_tag, int t0, int t1) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    for (int t = t0; t < t1; ++t) {
      stage(t);
      f32x16 sacc[2];
      if constexpr (PRE && !KV_ALIAS) {
        qk(sacc, qfar, negm);
        auto requery = [&](f32x16 (&sx)[2]) __attribute__((always_inline)) { qk(sx, qfar, negm); };
        softmax_pv_pre2<VT, D, MASK>(sacc, o_acc, m_run, l_run, a_far, negm, vload, requery, lane, t * FDB_BN, i, Lb,
                                     MASK && p.causal != 0);
      } else if constexpr (PRE) {  // K is gone once V is staged: no second pass over the scores
        qk(sacc, qfar, negm);
        stage_v(t);
        softmax_pv_pre<VT, D, MASK>(sacc, o_acc, m_run, l_run, a_far, negm, vload, lane, t * FDB_BN, i, Lb,
                                    MASK && p.causal != 0);
      } else {
        qk(sacc, qf, zero16);
        stage_v(t);
        softmax_pv<VT, D, MASK>(sacc, o_acc, m_run, l_run, x_scale, a_far, vload, lane, t * FDB_BN, i, Lb,
                                MASK && p.causal != 0);
      }
    }
  };
  auto far_range = [&](int t0, int t1, int side) __attribute__((always_inline)) {
    if (t0 >= t1) return;
    if constexpr (PRE) setup_far(side);
    const int tm = max(t0, min(t1, n_full));
    far_loop(std::false_type{}, t0, tm);
    far_loop(std::true_type{}, tm, t1);
  };

  // ---- far-left ------------------------------------------------------------------------------
  if constexpr (!RING) far_range(zl0, zl1, 0);

  // ---- near ----------------------------------------------------------------------------------
  if constexpr (RING) {
    // Relative positions of the workgroup tile k = t - t_near0: r in [r_hi0 - 64k - 190, r_hi0 - 64k];
    // u = r_hi0 - r counts downwards from the first tile's largest r, ring slot = u & 255,
    // batch = u / 64 (tile k reads batches k .. k+2).  A batch is staged like a K tile: the same
    // 16-byte chunks per thread, its table values one stage ahead of its rows.
    constexpr int RCH = C::K_CHUNKS, CPR = D * QT::SZ / 16, KS = C::KSTEPS;
    const int r_hi0 = m0 + FDB_BM - 1 - t_near0 * FDB_BN;
    u32x4 ekreg[RCH], eqreg[RCH];
    int dnext[RCH];
    auto batch_delta = [&](int batch, int (&dl)[RCH]) __attribute__((always_inline)) {
#pragma unroll
      for (int n = 0; n < RCH; ++n) {
        const int r = r_hi0 - (batch * 64 + min((tid + n * kThreads) / CPR, FDB_BN - 1));
        dl[n] = p.lut[max(-p.R, min(p.R, r)) + p.R];
      }
    };
    auto batch_load = [&](const int (&dl)[RCH]) __attribute__((always_inline)) {
#pragma unroll
      for (int n = 0; n < RCH; ++n) {
        const int cc = (tid + n * kThreads) % CPR;
        if constexpr (C2P) ekreg[n] = *(const u32x4*)(pkb + (int64_t)dl[n] * p.pk_sr * QT::SZ + cc * 16);
        if constexpr (P2C) eqreg[n] = *(const u32x4*)(pqb + (int64_t)dl[n] * p.pq_sr * QT::SZ + cc * 16);
      }
    };
    auto batch_store = [&](int batch) __attribute__((always_inline)) {
      const int seg = (batch & 3) * 64 * C::K_RS;
      if constexpr (C2P) tile_store<D * QT::SZ, C::K_RS>(EK + seg, ekreg, tid);
      if constexpr (P2C) tile_store<D * QT::SZ, C::K_RS>(EQ + seg, eqreg, tid);
    };
    // tile t = t_near0 + k: K, V and batch k+2 to LDS ...
    auto ring_stage = [&](int t) __attribute__((always_inline)) {
      __syncthreads();
      tile_store<D * QT::SZ, C::K_RS>(Ks, kreg, tid);
      tile_store<D * VT::SZ, C::V_RS>(Vs, vreg, tid);
      batch_store(t - t_near0 + 2);
      __syncthreads();
    };
    // ... and tile t+1's K, V and batch k+3 into the registers, in four pieces that are issued
    // between the MFMAs of the tile
    auto ring_prefetch = [&](int t, int piece) __attribute__((always_inline)) {
      if (t + 1 < t_near1) {
        if (piece == 0) batch_load(dnext);  // its table values were loaded a tile ago: no wait on the loads issued below
        if (piece == 1) tile_load<D * QT::SZ>(kreg, kb, k_rsb, (t + 1) * FDB_BN, Lb, tid);
        if (piece == 2) tile_load<D * VT::SZ>(vreg, vb, v_rsb, (t + 1) * FDB_BN, Lb, tid);
        if (piece == 3 && t + 2 < t_near1) batch_delta(t - t_near0 + 4, dnext);
      }
    };
    if (t_near0 < t_near1) {
#pragma unroll 1
      for (int bt = 0; bt < 2; ++bt) {
        batch_delta(bt, dnext);
        batch_load(dnext);
        batch_store(bt);
      }
      batch_delta(2, dnext);
      batch_load(dnext);
      batch_delta(3, dnext);
    }
    // The query loads are consumed here: left pending into the loop, their first use would make
    // the compiler wait for every outstanding vector-memory load at the top of each tile.
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" ::"v"(qf[s]));

    // per-lane scratch addresses (elements)
    const int colb = 8 * g * QT::SZ;
    ST* c_wr = c2pS + (wave * 32 + li) * kC2pStride + 4 * g;                         // C[i = li][32*blk + 8*q4 + 4*g ..+3]
    // C[i][li + 63 - jj] for jj = 8*n + 4*g + 3 .. + 0 is the window of four elements that starts
    // at li + 60 - 4*g - 8*n = 4*(chunk) + (li & 3).  Only 8-byte-aligned LDS reads run at speed (a
    // misaligned one is served lane by lane), so the two aligned chunks around the window are read
    // and the window is cut out of them with per-lane selects and a funnel shift.
    const ST* c_rd = c2pS + (wave * 32 + li) * kC2pStride + 4 * ((li >> 2) + 15 - g);  // chunk of window n = 0; window n is 8*n elements lower
    const bool c_odd_chunk = (li & 2) != 0;   // the window starts in the second dword of the chunk
    const uint32_t c_shift = 16 * (li & 1);   // ... and in the high half of that dword
    const ST* p_rd = p2cS + (4 * g) * kP2cStride + (wave * 32 + li + 63 - 4 * g);    // P[jj][wave*32 + li + 63 - jj]

    // One near tile.  The wave is alone on its SIMD, so the instruction stream itself has to overlap
    // the units: the position products come first, one MFMA per step, and each step also issues the
    // LDS read of an operand two blocks ahead and a quarter of the previous block's write-out to the
    // scratch.  Blocks: P (rows E_Q block `wave` against key halves 0 and 1, rows E_Q block
    // 4 + wave/2 against key half wave%2), C (rows E_K blocks wave + 0..2 against the queries), then
    // the content product, under which the last write-out hides.
    auto ring_tile = [&](auto mask_tag, int t) __attribute__((always_inline)) {
      constexpr bool MASK = decltype(mask_tag)::value;
      constexpr int nP = P2C ? 3 : 0, nC = C2P ? 3 : 0, NB = nP + nC, nLP = P2C ? 2 : 0, NL = nLP + nC;
      constexpr int QPS = 4 / KS;  // write-out quarters per step
      const int j0 = t * FDB_BN;
      ring_stage(t);
      const int ubase = 190 + 64 * (t - t_near0) - li;
      // A rows of operand load l: E_Q block `wave` (l = 0), 4 + wave/2 (l = 1) when P2C; then E_K blocks wave + 0..2
      auto a_row = [&](int l) __attribute__((always_inline)) -> const char* {
        if (l < nLP) return EQ + ((ubase - 32 * (l == 0 ? wave : 4 + (wave >> 1))) & (kRing - 1)) * C::K_RS + colb;
        return EK + ((ubase - 32 * (wave + l - nLP)) & (kRing - 1)) * C::K_RS + colb;
      };
      auto blk_load = [](int b) { return P2C ? (b < 2 ? 0 : b - 1) : b; };
      qfrag kf[2][KS], kx[KS], af[2][KS];
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int s = 0; s < KS; ++s) kf[jb][s] = QT::load(Ks + (32 * jb + li) * C::K_RS + colb + 16 * s * QT::SZ);
#pragma unroll
      for (int l = 0; l < 2; ++l)
#pragma unroll
        for (int s = 0; s < KS; ++s) af[l][s] = QT::load(a_row(l) + 16 * s * QT::SZ);
      if constexpr (P2C) {
#pragma unroll
        for (int s = 0; s < KS; ++s) kx[s] = QT::load(Ks + (32 * (wave & 1) + li) * C::K_RS + colb + 16 * s * QT::SZ);
      }
      __builtin_amdgcn_sched_barrier(0);
      f32x16 acc[2], sacc[2], zero;
#pragma unroll
      for (int v = 0; v < 16; ++v) zero[v] = 0.f;
      auto writeout = [&](int b, int q4) __attribute__((always_inline)) {
        ST* dst;
        if (b < nP) {
          const int wblk = b < 2 ? wave : 4 + (wave >> 1), jblk = b < 2 ? b : (wave & 1);
          dst = p2cS + (jblk * 32 + li) * kP2cStride + 32 * wblk + 4 * g + 8 * q4;
        } else {
          dst = c_wr + 32 * (b - nP) + 8 * q4;
        }
        store4_scratch<ST>(dst, acc[b & 1][4 * q4], acc[b & 1][4 * q4 + 1], acc[b & 1][4 * q4 + 2], acc[b & 1][4 * q4 + 3]);
      };
#pragma unroll
      for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const int l = blk_load(b);
          const qfrag bop = b < nP ? (b == 0 ? kf[0][s] : b == 1 ? kf[1][s] : kx[s]) : qf[s];
          acc[b & 1] = QT::mma(af[l & 1][s], bop, s == 0 ? zero : acc[b & 1]);
          if ((b + 1 == NB || blk_load(b + 1) != l) && l + 2 < NL) af[l & 1][s] = QT::load(a_row(l + 2) + 16 * s * QT::SZ);
          if (b > 0) {
#pragma unroll
            for (int e = 0; e < QPS; ++e) writeout(b - 1, QPS * s + e);
          }
          if (b == 1) {
#pragma unroll
            for (int e = 0; e < QPS; ++e) ring_prefetch(t, QPS * s + e);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        if (P2C && C2P && b == nP) __syncthreads();  // the three P blocks of every wave are in the scratch
      }
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) writeout(NB - 1, q4);
      if (P2C && !C2P) __syncthreads();
      wave_lds_fence();  // this wave's C write-outs precede its reads below (the LDS unit keeps a wave's operations in order)
      // element (j = j0 + jj, i): jj = 32*jb + 8*q + 4*g + e adds C[i][li + 63 - jj] + P[jj][wave*32 + li + 63 - jj].
      // The scratch reads keep the LDS unit busy for longer than they take to issue: the MFMAs of
      // the content product are spread between them.
      u32x4 cw[C2P ? 8 : 1];
      uint32_t px[P2C ? 32 : 1];
#pragma unroll
      for (int n = 0; n < 8; ++n) {
        if constexpr (C2P) {
          const u32x2 lo = *(const u32x2*)(c_rd - 8 * n), hi = *(const u32x2*)(c_rd - 8 * n + 4);
          cw[n] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
        if constexpr (P2C) {
#pragma unroll
          for (int e = 0; e < 4; ++e) px[4 * n + e] = *(const uint16_t*)(p_rd + (8 * n + e) * (kP2cStride - 1));
        }
        if (n < 2 * KS) sacc[n / KS] = QT::mma(kf[n / KS][n % KS], qf[n % KS], n % KS == 0 ? zero : sacc[n / KS]);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if constexpr (C2P) {
            const u32x4 d = cw[4 * jb + q];
            const uint32_t wa = c_odd_chunk ? d[1] : d[0], wb = c_odd_chunk ? d[2] : d[1], wc = c_odd_chunk ? d[3] : d[2];
            const uint32_t w[2] = {__builtin_amdgcn_alignbit(wb, wa, c_shift), __builtin_amdgcn_alignbit(wc, wb, c_shift)};  // window elements 0,1 | 2,3 for e = 3,2 | 1,0
            sacc[jb][4 * q + 0] = QT::add_hi(sacc[jb][4 * q + 0], w[1]);
            sacc[jb][4 * q + 1] = QT::add_lo(sacc[jb][4 * q + 1], w[1]);
            sacc[jb][4 * q + 2] = QT::add_hi(sacc[jb][4 * q + 2], w[0]);
            sacc[jb][4 * q + 3] = QT::add_lo(sacc[jb][4 * q + 3], w[0]);
          }
          if constexpr (P2C) {
#pragma unroll
            for (int e = 0; e < 4; ++e) sacc[jb][4 * q + e] = QT::add_lo(sacc[jb][4 * q + e], px[16 * jb + 4 * q + e]);
          }
        }
      softmax_pv<VT, D, MASK>(sacc, o_acc, m_run, l_run, x_scale, 0.f, vload, lane, j0, i, Lb, MASK && p.causal != 0);
    };
    const int tm = max(t_near0, min(t_near1, n_full));
    for (int t = t_near0; t < tm; ++t) ring_tile(std::false_type{}, t);
    for (int t = tm; t < t_near1; ++t) ring_tile(std::true_type{}, t);
  } else if constexpr (kHasPos && !FAR_ONLY) {
    // Row offsets (bytes) into K_r / Q_r of the A rows this lane feeds to the position products
    // of one tile; looked up through the table one tile ahead so that the row loads of a tile
    // never wait for the table.
    // Where the A rows of all six blocks would not fit the registers (fp32; head_dim 128 in a 16-bit type), they are
    // fetched block by block, one block ahead of the MFMAs that use them, and the offsets of the next tile go to a set
    // of their own until this tile's last block has been requested.
    constexpr bool LAZY_A = D >= 128 || C::KSTEPS * (int)(sizeof(qfrag) / 4) >= 32;
    int64_t off_c[3], off_p[3], offn_c[3], offn_p[3];
    auto lookup = [&](int t) __attribute__((always_inline)) {
      const int j0 = t * FDB_BN;
      if constexpr (C2P) {
        const int r_lo = iw0 - (j0 + FDB_BN - 1);  // the 95 relative positions of this wave's 32 rows
#pragma unroll
        for (int blk = 0; blk < 3; ++blk) {
          const int r = max(-p.R, min(p.R, r_lo + 32 * blk + li));
          offn_c[blk] = (int64_t)p.lut[r + p.R] * p.pk_sr * QT::SZ + 8 * g * QT::SZ;
        }
      }
      if constexpr (P2C) {
        const int r_lo = m0 - (j0 + FDB_BN - 1);  // the 191 relative positions of the 128 x 64 tile
#pragma unroll
        for (int n = 0; n < 3; ++n) {
          const int wblk = (wave * 3 + n) >> 1;
          const int r = max(-p.R, min(p.R, r_lo + 32 * wblk + li));
          offn_p[n] = (int64_t)p.lut[r + p.R] * p.pq_sr * QT::SZ + 8 * g * QT::SZ;
        }
      }
    };
    if (t_near0 < t_near1) lookup(t_near0);
    auto near_loop = [&](auto mask_tag, int t0, int t1) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    for (int t = t0; t < t1; ++t) {
      const int j0 = t * FDB_BN;
#pragma unroll
      for (int n = 0; n < 3; ++n) {
        off_c[n] = offn_c[n];
        off_p[n] = offn_p[n];
      }
      constexpr int nC = C2P ? 3 : 0, nP = P2C ? 3 : 0, NB = nC + nP;
      qfrag ac[(C2P && !LAZY_A) ? 3 : 1][C::KSTEPS], ap[(P2C && !LAZY_A) ? 3 : 1][C::KSTEPS], abuf[LAZY_A ? 2 : 1][C::KSTEPS];
      auto load_blk = [&](int b, qfrag (&dst)[C::KSTEPS]) __attribute__((always_inline)) {  // block b of the tile: C's three, then P's
        const char* base = b < nC ? pkb + off_c[b < nC ? b : 0] : pqb + off_p[b >= nC ? b - nC : 0];
#pragma unroll
        for (int s = 0; s < C::KSTEPS; ++s) dst[s] = QT::load(base + 16 * s * QT::SZ);
      };
      if constexpr (!LAZY_A) {
        if constexpr (C2P) {
#pragma unroll
          for (int blk = 0; blk < 3; ++blk) load_blk(blk, ac[blk]);
        }
        if constexpr (P2C) {
#pragma unroll
          for (int n = 0; n < 3; ++n) load_blk(nC + n, ap[n]);
        }
      } else {
        load_blk(0, abuf[0]);
      }
      stage(t);
      if (t + 1 < t_near1) lookup(t + 1);
      f32x16 sacc[2];
      qk(sacc, qf, zero16);
      if constexpr (C2P) {
        // C[i][r - r_lo]: column i = li, rows 32*blk + 8*q4 + 4*g + 0..3
        ST* dst0 = c2pS + (wave * 32 + li) * kC2pStride + 4 * g;
#pragma unroll
        for (int blk = 0; blk < 3; ++blk) {
          f32x16 acc;
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[v] = 0.f;
          if constexpr (LAZY_A) {
            if (blk + 1 < NB) load_blk(blk + 1, abuf[(blk + 1) & 1]);
          }
#pragma unroll
          for (int s = 0; s < C::KSTEPS; ++s) acc = QT::mma(LAZY_A ? abuf[blk & 1][s] : ac[LAZY_A ? 0 : blk][s], qf[s], acc);
          if constexpr (FP8) acc *= c2p_mul;
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4)
            store4_scratch<ST>(dst0 + 32 * blk + 8 * q4, acc[4 * q4], acc[4 * q4 + 1], acc[4 * q4 + 2], acc[4 * q4 + 3]);
        }
      }
      if constexpr (P2C) {
        // P[j][r - r_lo]: 12 MFMA blocks (6 row blocks x 2 key blocks) shared by the 4 waves
#pragma unroll
        for (int n = 0; n < 3; ++n) {
          const int task = wave * 3 + n, wblk = task >> 1, jblk = task & 1;
          f32x16 acc;
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[v] = 0.f;
          if constexpr (LAZY_A) {
            if (nC + n + 1 < NB) load_blk(nC + n + 1, abuf[(nC + n + 1) & 1]);
          }
#pragma unroll
          for (int s = 0; s < C::KSTEPS; ++s) {
            qfrag kf = QT::load(Ks + (jblk * 32 + li) * C::K_RS + (16 * s + 8 * g) * QT::SZ);
            acc = QT::mma(LAZY_A ? abuf[(nC + n) & 1][s] : ap[LAZY_A ? 0 : n][s], kf, acc);
          }
          if constexpr (FP8) acc *= p2c_mul;
          ST* dst0 = p2cS + (jblk * 32 + li) * kP2cStride + 32 * wblk + 4 * g;
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4)
            store4_scratch<ST>(dst0 + 8 * q4, acc[4 * q4], acc[4 * q4 + 1], acc[4 * q4 + 2], acc[4 * q4 + 3]);
        }
      }
      __syncthreads();
      // element (j = j0 + jj, i): r - r_lo = li + 63 - jj (wave tile) / wave*32 + li + 63 - jj (workgroup tile)
      if constexpr (sizeof(ST) == 2) {
        // 16-bit scratch.  C[i][li + 63 - jj] for jj = 8*n + 4*g + 3 .. + 0 is the window of four elements
        // that starts at 4*chunk + (li & 3): a misaligned 8-byte LDS read is served lane by lane, so the
        // two aligned chunks around the window are read and the window is cut out of them; every
        // element is then added with one dot instruction.
        const ST* c_rd = c2pS + (wave * 32 + li) * kC2pStride + 4 * ((li >> 2) + 15 - g);
        const ST* p_rd = p2cS + (4 * g) * kP2cStride + (wave * 32 + li + 63 - 4 * g);
        const bool c_odd_chunk = (li & 2) != 0;
        const uint32_t c_shift = 16 * (li & 1);
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          const int jb = n >> 2, q = n & 3;
          if constexpr (C2P) {
            const u32x2 lo = *(const u32x2*)(c_rd - 8 * n), hi = *(const u32x2*)(c_rd - 8 * n + 4);
            const uint32_t wa = c_odd_chunk ? lo[1] : lo[0], wb = c_odd_chunk ? hi[0] : lo[1], wc = c_odd_chunk ? hi[1] : hi[0];
            const uint32_t w0 = __builtin_amdgcn_alignbit(wb, wa, c_shift), w1 = __builtin_amdgcn_alignbit(wc, wb, c_shift);
            sacc[jb][4 * q + 0] = scratch_add_hi<ST>(sacc[jb][4 * q + 0], w1);
            sacc[jb][4 * q + 1] = scratch_add_lo<ST>(sacc[jb][4 * q + 1], w1);
            sacc[jb][4 * q + 2] = scratch_add_hi<ST>(sacc[jb][4 * q + 2], w0);
            sacc[jb][4 * q + 3] = scratch_add_lo<ST>(sacc[jb][4 * q + 3], w0);
          }
          if constexpr (P2C) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t x = *(const uint16_t*)(p_rd + (8 * n + e) * (kP2cStride - 1));
              sacc[jb][4 * q + e] = scratch_add_lo<ST>(sacc[jb][4 * q + e], x);
            }
          }
        }
      } else {
        const ST* cbase = c2pS + (wave * 32 + li) * kC2pStride + (li + 63 - 4 * g);
        const ST* pbase = p2cS + (4 * g) * kP2cStride + (wave * 32 + li + 63 - 4 * g);
#pragma unroll
        for (int jb = 0; jb < 2; ++jb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int cj = 32 * jb + 8 * (v >> 2) + (v & 3);  // jj = cj + 4*g
            if constexpr (C2P) sacc[jb][v] += (float)cbase[-cj];
            if constexpr (P2C) sacc[jb][v] += (float)pbase[cj * kP2cStride - cj];
          }
      }
      stage_v(t);
      softmax_pv<VT, D, MASK>(sacc, o_acc, m_run, l_run, x_scale, 0.f, vload, lane, j0, i, Lb,
                              MASK && p.causal != 0);
    }
    };
    const int tm = max(t_near0, min(t_near1, n_full));
    near_loop(std::false_type{}, t_near0, tm);
    near_loop(std::true_type{}, tm, t_near1);
  }

  // ---- far-right -----------------------------------------------------------------------------
  if constexpr (!RING) far_range(zr0, zr1, 1);

  // ---- epilogue ------------------------------------------------------------------------------
  const float l_tot = wave_half_sum(l_run);
  if constexpr (RING) {
    // merge with the far tiles' partial result (rows normalised over the far keys in out, their
    // log-sum-exp in lse), normalise, store
    if (i < Lb) {
      char* orow = ob + (int64_t)i * p.o_st * VT::SZ;
      const int64_t tok = p.cu ? (int64_t)tok0 + i : (int64_t)b * p.L + tok0 + i;
      float w_far = 0.f, w_near = 1.f, m_out = m_run;
      if (p.far_done) {
        const float lf = p.lse[tok * p.H + h] * 1.4426950408889634f;  // base 2 (-inf: no far tile)
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
    return;
  }
  const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
  if (i < Lb) {
    const int64_t tok = p.cu ? (int64_t)tok0 + i : (int64_t)b * p.L + tok0 + i;
    char* orow = ob + (int64_t)i * p.o_st * VT::SZ;
    float* lse_row = p.lse;
    if (FAR_ONLY && part > 0) {  // the partial results after the first go to the workspace, token-major
      orow = far_part_out(p, part, D * VT::SZ) + (tok * p.H + h) * (D * VT::SZ);
      lse_row = far_part_lse(p, part, D * VT::SZ);
    }
    if (MODE == kFused && p.key_parts > 1) {  // every share's partial result goes to its workspace slot
      orow = ws_slot_out(p, part, D * VT::SZ) + (tok * p.H + h) * (D * VT::SZ);
      lse_row = ws_slot_lse(p, part, D * VT::SZ);
    }
#pragma unroll
    for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int dd = 32 * d + 8 * q4 + 4 * g;
        VT::store4(orow + dd * VT::SZ, o_acc[d][4 * q4] * inv, o_acc[d][4 * q4 + 1] * inv,
                   o_acc[d][4 * q4 + 2] * inv, o_acc[d][4 * q4 + 3] * inv);
      }
    if (lse_row && g == 0) lse_row[tok * p.H + h] = (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
  }
}

template <class QT, class VT, int D, bool FP8, bool C2P, bool P2C, int MODE>
int launch_one(const FdbKParams& p, int grid_x, hipStream_t stream) {
  using C = Cfg<QT, VT, D>;
  auto kern = fdb_attn_kernel<QT, VT, D, FP8, C2P, P2C, MODE>;
  constexpr int lds = C::lds_bytes_mode(MODE, C2P, P2C);
  static_assert(lds <= 160 * 1024, "LDS budget");
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = fdb_set_lds_once((const void*)kern, lds, lds_set);
  if (e != hipSuccess) return (int)e;
  const unsigned parts = MODE == kFarOnly && p.far_parts > 1 ? (unsigned)p.far_parts
                         : MODE == kFused && p.key_parts > 1 ? (unsigned)p.key_parts : 1u;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid_x * p.H, parts, 1), dim3(kThreads), lds, stream, p);
  return (int)hipGetLastError();
}

template <class QT, class VT, int D, bool FP8>
int launch_pos(const FdbKParams& p, int grid_x, int mode, hipStream_t stream) {
  if constexpr (!FP8 && QT::SZ == 2 && D <= 64) {  // the combinations the two-launch path covers
    if (mode == kFarOnly) {
      if (p.pk && p.pq) return launch_one<QT, VT, D, FP8, true, true, kFarOnly>(p, grid_x, stream);
      if (p.pk) return launch_one<QT, VT, D, FP8, true, false, kFarOnly>(p, grid_x, stream);
      if (p.pq) return launch_one<QT, VT, D, FP8, false, true, kFarOnly>(p, grid_x, stream);
    }
    if (mode == kNearRing) {
      if (p.pk && p.pq) return launch_one<QT, VT, D, FP8, true, true, kNearRing>(p, grid_x, stream);
      if (p.pk) return launch_one<QT, VT, D, FP8, true, false, kNearRing>(p, grid_x, stream);
      if (p.pq) return launch_one<QT, VT, D, FP8, false, true, kNearRing>(p, grid_x, stream);
    }
  }
  if (mode != kFused) return FDB_ERR_UNSUPPORTED;
  if (p.pk && p.pq) return launch_one<QT, VT, D, FP8, true, true, kFused>(p, grid_x, stream);
  if (p.pk) return launch_one<QT, VT, D, FP8, true, false, kFused>(p, grid_x, stream);
  if (p.pq) return launch_one<QT, VT, D, FP8, false, true, kFused>(p, grid_x, stream);
  return launch_one<QT, VT, D, FP8, false, false, kFused>(p, grid_x, stream);
}

}  // namespace

bool fdb_near_supported(int dtype, int head_dim) {
  return (dtype == FDB_BF16 || dtype == FDB_F16) && (head_dim == 32 || head_dim == 64);
}

int fdb_launch_attn(const FdbKParams& p, int dtype, int head_dim, int grid_x, int mode, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
#define FDB_DISPATCH_D(QT, VT, FP8)                                   \
  switch (head_dim) {                                                 \
    case 32: return launch_pos<QT, VT, 32, FP8>(p, grid_x, mode, stream);   \
    case 64: return launch_pos<QT, VT, 64, FP8>(p, grid_x, mode, stream);   \
    case 128: return launch_pos<QT, VT, 128, FP8>(p, grid_x, mode, stream); \
    default: return FDB_ERR_HEAD_DIM;                                 \
  }
  switch (dtype) {
    case FDB_BF16: FDB_DISPATCH_D(Bf16Tr, Bf16Tr, false)
    case FDB_F16: FDB_DISPATCH_D(F16Tr, F16Tr, false)
    case FDB_F32:
      switch (head_dim) {
        case 32: return launch_pos<F32Tr, F32Tr, 32, false>(p, grid_x, mode, stream);
        case 64: return launch_pos<F32Tr, F32Tr, 64, false>(p, grid_x, mode, stream);
        case 128: return launch_pos<F32Tr, F32Tr, 128, false>(p, grid_x, mode, stream);
        default: return FDB_ERR_HEAD_DIM;
      }
    case FDB_FP8_E4M3: FDB_DISPATCH_D(Fp8Tr, Bf16Tr, true)
    default: return FDB_ERR_DTYPE;
  }
#undef FDB_DISPATCH_D
}
