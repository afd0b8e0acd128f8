// FP8 Q/K variant of the two-launch path for gfx950, head_dim 64: q, k, K_r, Q_r are OCP e4m3 bytes with
// per-head fp32 scales, v and the probabilities are bf16.  The three score products -- q.k, q.K_r[delta] and
// k.Q_r[delta] -- are e4m3 contractions over the whole head_dim in one instruction each
// (v_mfma_scale_f32_32x32x64_f8f6f4: twice the bf16 rate, a quarter of the instructions); P V stays bf16.
// No counterpart in the reference (its kernels take 16-bit and 32-bit operands only).
//
// Operand layout of the 32x32x64 e4m3 MFMA as probed on the device: lane (n = l % 32, g = l / 32) feeds 32 bytes;
// which of the 64 contraction elements they are is the same function for the A and the B operand, so two rows
// loaded alike -- lane group g takes bytes [32 g, 32 g + 32) of a 64-byte row -- contract element by element.
// A scale operand (e8m0, 127 = 1.0) is read from the lane of the row / column; a scale block spans registers of
// both lane groups, so one exponent per row / column is used and both lanes of a pair carry it.
//
//   fdb_far8_kernel   the far key tiles (bucketed relative position constant): like the 16-bit far-only launch, the
//                     position->content term is folded into the query and the content->position term into the
//                     accumulator's starting value, so a tile is two MFMAs, exponentials and P V.  The folded query
//                     (s_q q + s_qr Q_r[delta]) * sm_scale * log2(e) * s_k is formed in fp32 and rounded to e4m3 once
//                     per row and side with a power-of-two exponent that the MFMA's scale operand takes back out.
//   fdb_near8_kernel  the near key tiles in 32-key steps, the scheme of the 16-bit near kernel (expanded table rows
//                     in two LDS rings, C through a per-wave fp16 scratch that holds both blocks of a step, P by lane
//                     rotations) on 64-byte rows: 4 score MFMAs per step instead of 16.  The three products have the units s_q s_k, s_q s_kr
//                     and s_k s_qr: the content product accumulates on top of C * (s_kr / s_k), P enters as
//                     fma(P, s_qr / s_q, .), and one factor s_q s_k sm_scale log2(e) converts the sum.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <utility>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

using namespace fdb;

namespace {

typedef __attribute__((ext_vector_type(8))) int i32x8;

constexpr int kThreads = 256;
constexpr int kRow8 = 64;    // bytes of an e4m3 row at head_dim 64
constexpr int kRowV = 128;   // bytes of a bf16 row

// slot (row, s) of an unpadded 64-byte row holds 16-byte chunk s ^ f8(row): sixteen consecutive rows put one chunk
// in sixteen different bank groups
__device__ __forceinline__ int f8(int row) { return (row >> 2) & 3; }

__device__ __forceinline__ i32x8 frag8(u32x4 lo, u32x4 hi) {
  return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}
// 32 e4m3 bytes [32 g, 32 g + 32) of a swizzled 64-byte LDS row: a0 / a1 = LDS byte addresses of its two 16-byte slots
__device__ __forceinline__ i32x8 lds_frag8(uint32_t a0, uint32_t a1) {
  return frag8(*(LDS_AS const u32x4*)(uintptr_t)a0, *(LDS_AS const u32x4*)(uintptr_t)a1);
}
__device__ __forceinline__ f32x16 mma8(i32x8 a, i32x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
// the same with B's rows scaled by 2^(sb - 127), sb from the lane of the column
__device__ __forceinline__ f32x16 mma8_sb(i32x8 a, i32x8 b, f32x16 c, int sb) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 127, 0, sb);
}
// ... and with A's rows scaled by a power of two known at compile time
template <int SA>
__device__ __forceinline__ f32x16 mma8_sa(i32x8 a, i32x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, SA, 0, 127);
}

// four e4m3 bytes of a word as fp32
__device__ __forceinline__ f32x4 e4m3x4(uint32_t w) {
  const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
  return f32x4{lo[0], lo[1], hi[0], hi[1]};
}

// ---------------------------------------------------------------------------------------------------------------
// far tiles
// ---------------------------------------------------------------------------------------------------------------
constexpr int kK8Tile = FDB_BN * kRow8;   // 4 KB
constexpr int kVTile = FDB_BN * kRowV;    // 8 KB
constexpr int kFarBuf = kK8Tile + kVTile;
constexpr int kFarLds = 3 * kFarBuf;      // three buffers: 36 KB, three workgroups per CU
constexpr int kFarLoads = 3;              // direct loads per wave and tile: one of K (16 rows), two of V (8 rows each)

template <bool C2P, bool P2C>
__global__ __launch_bounds__(kThreads, 3) void fdb_far8_kernel(const FdbKParams p) {
  constexpr int D = 64, DBLKS = 2;
  using VT = Bf16Tr;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, li = lane & 31, g = lane >> 5;
  int xq, h;
  block_map((int)blockIdx.x, p.grid_x, p.H, p.tiles_per_seq, p.cu == nullptr, p.causal ? kLastFirst : kEdgesFirst, xq, h);

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
    const int sl = p.seq_len ? p.seq_len[b] : p.L;
    Lb = min(max(sl, 0), p.L - tok0);
    if (p.fill_pad && blockIdx.y == 0)
      fill_pad_rows<kRowV>(p.out + ((int64_t)b * p.o_sb + (int64_t)h * p.o_sh) * 2, p.o_st * 2, xq % p.tiles_per_seq, p.L, tok0, Lb,
                           sl < 0 ? VT::NAN_WORD : 0u, tid);
    if (m0 >= Lb) return;
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; oo = b * p.o_sb;
  }
  const char* qb = p.q + (qo + (int64_t)tok0 * p.q_st + (int64_t)h * p.q_sh);
  const char* kb = p.k + (ko + (int64_t)tok0 * p.k_st + (int64_t)h * p.k_sh);
  const char* vb = p.v + (vo + (int64_t)tok0 * p.v_st + (int64_t)h * p.v_sh) * 2;
  char* ob = p.out + (oo + (int64_t)tok0 * p.o_st + (int64_t)h * p.o_sh) * 2;
  const char* pkb = C2P ? p.pk + (int64_t)h * p.pk_sh : nullptr;
  const char* pqb = P2C ? p.pq + (int64_t)h * p.pq_sh : nullptr;
  const uint32_t k_rsb = (uint32_t)p.k_st, v_rsb = (uint32_t)(p.v_st * 2);
  const float s_q = p.qs[h], s_k = p.ks[h];
  const float s_kr = C2P ? p.pks[h] : 0.f, s_qr = P2C ? p.pqs[h] : 0.f;

  const int iw0 = m0 + wave * 32;
  const int i = iw0 + li;

  // ---- tile ranges (as in the 16-bit far-only launch) ------------------------------------------------------
  int j_end = Lb;
  if (p.causal) j_end = min(Lb, m0 + FDB_BM);
  const int n_tiles = (j_end + FDB_BN - 1) / FDB_BN;
  const int lim = m0 - (FDB_BN - 1) - p.R;
  const int t_near0 = lim >= 0 ? min(n_tiles, lim / FDB_BN + 1) : 0;
  const int t_near1 = max(t_near0, min(n_tiles, (m0 + FDB_BM - 1 + p.R + FDB_BN - 1) / FDB_BN));
  int zl0 = 0, zl1 = t_near0, zr0 = t_near1, zr1 = n_tiles;
  const int part = (int)blockIdx.y;
  if (p.far_parts > 1) {
    const int n_far = t_near0 + (n_tiles - t_near1);
    const int o_lo = (int)((int64_t)n_far * part / p.far_parts), o_hi = (int)((int64_t)n_far * (part + 1) / p.far_parts);
    zl0 = min(o_lo, t_near0);
    zl1 = min(o_hi, t_near0);
    zr0 = t_near1 + max(o_lo - t_near0, 0);
    zr1 = t_near1 + max(o_hi - t_near0, 0);
  }
  const int t_end = zr1;
  auto next_tile = [&](int t) __attribute__((always_inline)) { return (t + 1 >= zl1 && t + 1 < zr0) ? zr0 : t + 1; };

  f32x16 o_acc[DBLKS];
#pragma unroll
  for (int d = 0; d < DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  float a_far = 0.f;
  i32x8 qfar = {0, 0, 0, 0, 0, 0, 0, 0};
  int sb_far = 127;
  f32x16 negm;
#pragma unroll
  for (int v = 0; v < 16; ++v) negm[v] = 0.f;

  // Per side: the row constant a_i = q_i . K_r[delta] and the folded query, rounded to e4m3 with a power-of-two
  // exponent of its own row (2^E brings the row's largest entry into [128, 256); the MFMA multiplies by 2^-E).
  auto setup_far = [&](int side) __attribute__((always_inline)) {
    const int delta = p.lut[side == 0 ? 2 * p.R : 0];
    u32x4 qw[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}};
    if (i < Lb) {
      qw[0] = *(const u32x4*)(qb + (int64_t)i * p.q_st + 32 * g);
      qw[1] = *(const u32x4*)(qb + (int64_t)i * p.q_st + 32 * g + 16);
    }
    u32x4 kw[2], rw[2];
    if constexpr (C2P) {
      const char* row = pkb + (int64_t)delta * p.pk_sr + 32 * g;
      kw[0] = *(const u32x4*)row;
      kw[1] = *(const u32x4*)(row + 16);
    }
    if constexpr (P2C) {
      const char* row = pqb + (int64_t)delta * p.pq_sr + 32 * g;
      rw[0] = *(const u32x4*)row;
      rw[1] = *(const u32x4*)(row + 16);
    }
    const float fold = p.scale_log2 * s_k;
    float acc = 0.f, amax = 0.f;
    float qv[32];
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const f32x4 q4 = e4m3x4(qw[w >> 2][w & 3]);
      if constexpr (C2P) {
        const f32x4 k4 = e4m3x4(kw[w >> 2][w & 3]);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_fmaf(q4[e], k4[e], acc);
      }
      f32x4 r4 = {0.f, 0.f, 0.f, 0.f};
      if constexpr (P2C) r4 = e4m3x4(rw[w >> 2][w & 3]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x = (q4[e] * s_q + r4[e] * s_qr) * fold;
        qv[4 * w + e] = x;
        amax = fmaxf(amax, fabsf(x));
      }
    }
    a_far = C2P ? wave_half_sum(acc) * (p.scale_log2 * s_q * s_kr) : 0.f;
    amax = wave_half_max(amax);
    // amax = m * 2^e with m in [0.5, 1): E = 8 - e; a zero row keeps E small enough for the scale byte
    const int e2 = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 255u) - 126;
    const int E = max(-100, min(100, 8 - e2));
    const float mul = __builtin_bit_cast(float, (uint32_t)(E + 127) << 23);
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      int word = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4 * w] * mul, qv[4 * w + 1] * mul, 0, false);
      word = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4 * w + 2] * mul, qv[4 * w + 3] * mul, word, true);
      qfar[w] = word;
    }
    sb_far = 127 - E;
    const float nm = a_far - (m_run == -INFINITY ? 0.f : m_run);
#pragma unroll
    for (int v = 0; v < 16; ++v) negm[v] = nm;
  };

  // ---- staging: global -> LDS directly, three buffers, one barrier per tile ---------------------------------------
  // K: a wave's load fills 1 KB = 16 rows of 64 bytes, lane l slot l % 4 of row l / 4; V: 8 rows of 128 bytes, as in
  // the 16-bit kernels (slot (row, s) holds chunk s ^ f(row), f = 4*bit1(row) | bits3:2(row)).
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_AS char*)smem;
  const uint32_t k_c16 = (uint32_t)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  const uint32_t dma_koff = (uint32_t)(16 * wave + (lane >> 2)) * k_rsb + k_c16;
  uint32_t dma_voff[2];
#pragma unroll
  for (int q2 = 0; q2 < 2; ++q2) {
    const uint32_t row = (uint32_t)(16 * wave + 8 * q2 + (lane >> 3));
    const uint32_t c16 = ((lane & 7) ^ (4 * ((lane >> 4) & 1)) ^ (lane >> 5) ^ (2 * q2)) * 16;
    dma_voff[q2] = row * v_rsb + c16;
  }
  auto dma_issue = [&](int tile, int bufoff) __attribute__((always_inline)) {
    const char* kt = kb + (uint64_t)(uint32_t)(tile * FDB_BN) * k_rsb;
    const char* vt = vb + (uint64_t)(uint32_t)(tile * FDB_BN) * v_rsb;
    const int last = Lb - 1 - tile * FDB_BN;
    const uint32_t kdst = lds0 + bufoff + wave * 1024, vdst = lds0 + bufoff + kK8Tile + 2 * wave * 1024;
    if (last >= FDB_BN - 1) {
      dma16s(kt, dma_koff, kdst);
      dma16s(vt, dma_voff[0], vdst);
      dma16s(vt, dma_voff[1], vdst + 1024);
    } else {  // the ragged last tile: rows past the end re-read the last one (their scores are masked)
      dma16s(kt, (uint32_t)min(16 * wave + (lane >> 2), last) * k_rsb + k_c16, kdst);
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {
        const uint32_t row = (uint32_t)min(16 * wave + 8 * q2 + (lane >> 3), last);
        const uint32_t c16 = ((lane & 7) ^ (4 * ((lane >> 4) & 1)) ^ (lane >> 5) ^ (2 * q2)) * 16;
        dma16s(vt, row * v_rsb + c16, vdst + q2 * 1024);
      }
    }
  };
  int dma_cur = 2 * kFarBuf;
  {
    const int first = next_tile(zl0 - 1);
    if (first < t_end) {
      dma_issue(first, 0);
      const int second = next_tile(first);
      if (second < t_end) dma_issue(second, kFarBuf);
    }
  }
  // read offsets: K fragment of block jb: row 32 jb + li, chunks 2g and 2g + 1; V^T operands as in the 16-bit kernels
  const uint32_t kx0 = (uint32_t)(li * kRow8 + ((2 * g) ^ f8(li)) * 16), kx1 = (uint32_t)(li * kRow8 + ((2 * g + 1) ^ f8(li)) * 16);
  uint32_t vlane;
  {
    const int s16 = lane & 15, grp = lane >> 4;
    const int slotl = (2 * (grp & 1) + ((s16 & 3) >> 1)) ^ (4 * ((s16 >> 3) & 1)) ^ (grp >> 1);
    vlane = (4 * (grp >> 1) + (s16 >> 2)) * kRowV + slotl * 16 + (s16 & 1) * 8;
  }
  uint32_t vcur[4], kcur[2] = {0u, 0u};
  auto stage = [&](int t) __attribute__((always_inline)) {
    const int nt = next_tile(t);
    if (nt < t_end) wait_vmcnt<kFarLoads>(); else wait_vmcnt<0>();
    __syncthreads();
    dma_cur = dma_cur == 2 * kFarBuf ? 0 : dma_cur + kFarBuf;
    if (nt < t_end) {
      const int nn = next_tile(nt);
      if (nn < t_end) dma_issue(nn, dma_cur >= kFarBuf ? dma_cur - kFarBuf : 2 * kFarBuf);
    }
    kcur[0] = lds0 + dma_cur + kx0;
    kcur[1] = lds0 + dma_cur + kx1;
#pragma unroll
    for (int x = 0; x < 4; ++x) vcur[x] = (vlane ^ (64 * (x >> 1) ^ 32 * (x & 1))) + (dma_cur + lds0 + kK8Tile);
  };
  auto vload = [&](int c, int d) __attribute__((always_inline)) {
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)((LDS_AS char*)(uintptr_t)vcur[2 * d] + 2048 * c));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)((LDS_AS char*)(uintptr_t)vcur[2 * d + 1] + 2048 * c + 1024));
    return __builtin_bit_cast(typename VT::frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto qk = [&](f32x16 (&sacc)[2]) __attribute__((always_inline)) {
    i32x8 kf[2];
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) kf[jb] = lds_frag8(kcur[0] + jb * 32 * kRow8, kcur[1] + jb * 32 * kRow8);
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) sacc[jb] = mma8_sb(kf[jb], qfar, negm, sb_far);
  };
  const int n_full = p.causal ? min(min(Lb / FDB_BN, t_near0), m0 / FDB_BN) : Lb / FDB_BN;
  auto far_loop = [&](auto mask_tag, int t0, int t1) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    for (int t = t0; t < t1; ++t) {
      stage(t);
      f32x16 sacc[2];
      qk(sacc);
      auto requery = [&](f32x16 (&sx)[2]) __attribute__((always_inline)) { qk(sx); };
      softmax_pv_pre2<VT, D, MASK>(sacc, o_acc, m_run, l_run, a_far, negm, vload, requery, lane, t * FDB_BN, i, Lb,
                                   MASK && p.causal != 0);
    }
  };
  auto far_range = [&](int t0, int t1, int side) __attribute__((always_inline)) {
    if (t0 >= t1) return;
    setup_far(side);
    const int tm = max(t0, min(t1, n_full));
    far_loop(std::false_type{}, t0, tm);
    far_loop(std::true_type{}, tm, t1);
  };
  far_range(zl0, zl1, 0);
  far_range(zr0, zr1, 1);

  // ---- the far partial result: rows normalised over the far keys, their log-sum-exp ----------------------------
  const float l_tot = wave_half_sum(l_run);
  const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
  if (i < Lb) {
    const int64_t tok = p.cu ? (int64_t)tok0 + i : (int64_t)b * p.L + tok0 + i;
    char* orow = ob + (int64_t)i * p.o_st * 2;
    float* lse_row = p.lse;
    if (part > 0) {
      orow = far_part_out(p, part, D * 2) + (tok * p.H + h) * (D * 2);
      lse_row = far_part_lse(p, part, D * 2);
    }
#pragma unroll
    for (int d = 0; d < DBLKS; ++d)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        VT::store4(orow + (32 * d + 8 * q4 + 4 * g) * 2, o_acc[d][4 * q4] * inv, o_acc[d][4 * q4 + 1] * inv,
                   o_acc[d][4 * q4 + 2] * inv, o_acc[d][4 * q4 + 3] * inv);
    if (lse_row && g == 0) lse_row[tok * p.H + h] = (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
  }
}

template <bool C2P, bool P2C>
int launch_far8_one(const FdbKParams& p, int grid_x, hipStream_t stream) {
  auto kern = fdb_far8_kernel<C2P, P2C>;
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = fdb_set_lds_once((const void*)kern, kFarLds, lds_set);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid_x * p.H, p.far_parts > 1 ? (unsigned)p.far_parts : 1u, 1), dim3(kThreads), kFarLds,
                     stream, p);
  return (int)hipGetLastError();
}


// ---------------------------------------------------------------------------------------------------------------
// near tiles
// ---------------------------------------------------------------------------------------------------------------
constexpr int kStep = 32;        // keys per step
// Batches of 32 relative positions in the rings.  A step reads five batches of E_Q (one per wave and block) while its
// loads fill a sixth; of E_K it reads only the four batches of the waves' new blocks, so the batch that the loads
// replace is the one no wave needs any more.
constexpr int kRingBatchesK = 5, kRingBatchesQ = 6;
constexpr int kScrPitch = 68;    // 16-bit elements per row of a wave's C scratch: two blocks of 32 columns + columns 0..3 once more
constexpr int kScrElems = 32 * kScrPitch;
constexpr int kCShift = 8;       // C leaves its MFMA scaled by 2^-8 so that 64 * 448 * 448 fits the fp16 scratch

struct N8 {
  static constexpr int K_BYTES = kStep * kRow8;       // 2 KB, rows swizzled with f8
  static constexpr int V_BYTES = kStep * kRowV;       // 4 KB, rows swizzled like the 16-bit kernels' (vf)
  static constexpr int RINGK_BYTES = 32 * kRingBatchesK * kRow8;  // 10 KB
  static constexpr int RINGQ_BYTES = 32 * kRingBatchesQ * kRow8;  // 12 KB
  static constexpr int SCR_BYTES = 4 * kScrElems * 2;
  static constexpr int lds_bytes(bool c2p, bool p2c) {
    return 2 * K_BYTES + 2 * V_BYTES + (c2p ? RINGK_BYTES + SCR_BYTES : 0) + (p2c ? RINGQ_BYTES : 0);
  }
};

// swizzle of the 128-byte V rows: slot (row, s) holds chunk s ^ vf(row)
__device__ __forceinline__ int vf(int row) { return 4 * ((row >> 1) & 1) | ((row >> 2) & 3); }

// Lane rotations and the reads of C's band are issued as asm, outside the compiler's count of outstanding LDS
// operations: the step waits for all of them once (lds_wait_all8) instead of once per value.
template <int OFFSET>
__device__ __forceinline__ float swizzle_asm8(float x) {
  float r;
  asm volatile("ds_swizzle_b32 %0, %1 offset:%2" : "=v"(r) : "v"(x), "n"(OFFSET));
  return r;
}
// px[v] = xs[v] of the lane (ROT0 - c(v)) places further up in this lane's half-wave (mod 32), c(v) = 8*(v/4) + 3 - v%4
template <int ROT0, int... V>
__device__ __forceinline__ void rotate16(const float (&xs)[16], float (&px)[16], std::integer_sequence<int, V...>) {
  ((px[V] = swizzle_asm8<(0xC000 | (((ROT0 - (8 * (V >> 2) + 3 - (V & 3))) & 31) << 5))>(xs[V])), ...);
}
template <int OFF>
__device__ __forceinline__ uint32_t lds_u16_asm(uint32_t addr) {
  uint32_t r;
  asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
__device__ __forceinline__ void lds_wait_all8() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// The scheme of the 16-bit near kernel (fdb_near.hip) on e4m3 operands: rings of batches aligned to the waves' blocks, C's
// scratch holding both blocks of a step (only the block that is new to the step is contracted and written; the other one
// is the block the step before wrote).  P's A operands of block 1 are read again rather than kept from the step before
// (168 registers per lane at three workgroups per CU do not hold them), which is why the ring of E_Q has a sixth batch: the
// batch a step's loads overwrite must not be one that a wave still reads in that step.  Per wave and step one e4m3 MFMA
// each for the content product and C, two for P, four bf16 MFMAs for P V.
template <bool C2P, bool P2C>
__global__ __launch_bounds__(kThreads, 3) void fdb_near8_kernel(const FdbKParams p) {
  constexpr int D = 64, DBLKS = 2;
  using VT = Bf16Tr;
  using vfrag = typename VT::frag;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* Ks = smem;                    // [2][32][64]: step k reads buffer k & 1
  char* Vs = Ks + 2 * N8::K_BYTES;    // [2][32][128]
  char* EK = Vs + 2 * N8::V_BYTES;    // [160][64] rows K_r[delta(r)]: batch u / 32 of u = r_hi0 - r in slot batch mod 5; E_Q: [192][64], mod 6
  char* EQ = EK + (C2P ? N8::RINGK_BYTES : 0);
  char* scr_raw = EQ + (P2C ? N8::RINGQ_BYTES : 0);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, li = lane & 31, g = lane >> 5;
  int xq, h;
  block_map((int)blockIdx.x, p.grid_x, p.H, p.tiles_per_seq, p.cu == nullptr, kMiddleFirst, xq, h);

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
    const int sl = p.seq_len ? p.seq_len[b] : p.L;
    Lb = min(max(sl, 0), p.L - tok0);
    if (p.fill_pad && blockIdx.y == 0)
      fill_pad_rows<kRowV>(p.out + ((int64_t)b * p.o_sb + (int64_t)h * p.o_sh) * 2, p.o_st * 2, xq % p.tiles_per_seq, p.L, tok0, Lb,
                           sl < 0 ? VT::NAN_WORD : 0u, tid);
    if (m0 >= Lb) return;
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; oo = b * p.o_sb;
  }
  const char* qb = p.q + (qo + (int64_t)tok0 * p.q_st + (int64_t)h * p.q_sh);
  const char* kb = p.k + (ko + (int64_t)tok0 * p.k_st + (int64_t)h * p.k_sh);
  const char* vb = p.v + (vo + (int64_t)tok0 * p.v_st + (int64_t)h * p.v_sh) * 2;
  char* ob = p.out + (oo + (int64_t)tok0 * p.o_st + (int64_t)h * p.o_sh) * 2;
  const char* pkb = C2P ? p.pk + (int64_t)h * p.pk_sh : nullptr;
  const char* pqb = P2C ? p.pq + (int64_t)h * p.pq_sh : nullptr;
  const uint32_t k_rsb = (uint32_t)p.k_st, v_rsb = (uint32_t)(p.v_st * 2);
  // units: the content product and the sum are in s_q s_k; C arrives in s_q s_kr (and scaled by 2^-kCShift), P in s_k s_qr
  const float s_q = p.qs[h], s_k = p.ks[h];
  const float x_scale = p.scale_log2 * s_q * s_k;
  const float rho_c = C2P ? p.pks[h] / s_k * (float)(1 << kCShift) : 0.f;
  const float rho_p = P2C ? p.pqs[h] / s_q : 0.f;

  const int iw0 = m0 + wave * 32;
  const int i = iw0 + li;

  i32x8 qf = {0, 0, 0, 0, 0, 0, 0, 0};
  if (i < Lb) qf = frag8(*(const u32x4*)(qb + (int64_t)i * p.q_st + 32 * g), *(const u32x4*)(qb + (int64_t)i * p.q_st + 32 * g + 16));
  asm volatile("" ::"v"(qf));  // consumed here: see the 16-bit near kernel

  int j_end = Lb;
  if (p.causal) j_end = min(Lb, m0 + FDB_BM);
  const int n_tiles = (j_end + FDB_BN - 1) / FDB_BN;
  const int lim = m0 - (FDB_BN - 1) - p.R;
  const int t0 = lim >= 0 ? min(n_tiles, lim / FDB_BN + 1) : 0;
  const int t1 = max(t0, min(n_tiles, (m0 + FDB_BM - 1 + p.R + FDB_BN - 1) / FDB_BN));
  int s0 = 2 * t0;
  int s1 = max(s0, min(2 * t1, (j_end + kStep - 1) / kStep));
  if (p.near_parts > 1) {
    const int all = s1 - s0, part = (int)blockIdx.y;
    s1 = s0 + (int)((int64_t)all * (part + 1) / p.near_parts);
    s0 = s0 + (int)((int64_t)all * part / p.near_parts);
  }
  const int n_steps = s1 - s0;
  const int n_full = max(0, min(n_steps, (p.causal ? min(Lb, m0) : Lb) / kStep - s0));
  // u = r_hi0 - r counts downwards from the first step's largest r; batch = u / 32, ring slot = batch mod 5 (E_K) or 6 (E_Q).  Wave w's
  // block bk at step k is batch k + 4 - w - bk, MFMA row m its row 31 - m: r = iw0 - 32 s - 32 + 32 bk + m.
  const int r_hi0 = m0 + FDB_BM - 1 - s0 * kStep;

  // ---- staging ---------------------------------------------------------------------------------------------
  // V: one 16-byte chunk per thread (a wave's load fills 8 rows of 128 bytes).  The 64-byte rows of K and of one
  // batch of each ring are 2 KB each, i.e. two waves' loads: waves 0 and 1 fetch K and E_K, waves 2 and 3 E_Q
  // (a load fills 16 rows, lane l slot l % 4 of row l / 4).  LDS row r of K holds key r ^ 3 of the step, as in
  // the 16-bit kernel.  A step inside the sequence travels as a scalar base + this thread's 32-bit offset.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_AS char*)smem;
  const int vrow = tid >> 3, vcc = tid & 7;
  const uint32_t v_chunk = (uint32_t)((vcc ^ vf(vrow)) * 16);
  const int row8 = (tid & 127) >> 2;                                   // row of a 32-row e4m3 tile this thread fetches a chunk of
  const uint32_t chunk8 = (uint32_t)(((tid & 3) ^ f8(row8)) * 16);
  const uint32_t half_kb = (uint32_t)(wave & 1) * 1024u;
  const uint32_t k_lane = (uint32_t)(row8 ^ 3) * k_rsb + chunk8, v_lane = (uint32_t)vrow * v_rsb + v_chunk;
  int dnext = 0;
  auto k_dma = [&](int s, int buf) __attribute__((always_inline)) {
    if (wave < 2) {
      const uint32_t dst = lds0 + buf * N8::K_BYTES + half_kb;
      if ((s + 1) * kStep <= Lb) {
        dma16sn(kb + (uint64_t)(uint32_t)(s * kStep) * k_rsb, k_lane, dst);
      } else {
        const int row = min(s * kStep + (row8 ^ 3), Lb - 1);
        dma16n(kb + (uint64_t)(uint32_t)row * k_rsb + chunk8, dst);
      }
    }
  };
  auto v_dma = [&](int s, int buf) __attribute__((always_inline)) {
    const uint32_t dst = lds0 + 2 * N8::K_BYTES + buf * N8::V_BYTES + (uint32_t)wave * 1024u;
    if ((s + 1) * kStep <= Lb) {
      dma16sn(vb + (uint64_t)(uint32_t)(s * kStep) * v_rsb, v_lane, dst);
    } else {
      const int row = min(s * kStep + vrow, Lb - 1);
      dma16n(vb + (uint64_t)(uint32_t)row * v_rsb + v_chunk, dst);
    }
  };
  int r_tab = r_hi0 - row8;  // relative position of this thread's row of a batch; runs down by 32 per batch
  auto batch_delta = [&]() __attribute__((always_inline)) {
    const int d = (int)((const uint16_t*)p.lut)[max(-p.R, min(p.R, r_tab)) + p.R];
    r_tab -= 32;
    return d;
  };
  const uint32_t ek_lds = lds0 + (uint32_t)(EK - smem) + half_kb, eq_lds = lds0 + (uint32_t)(EQ - smem) + half_kb;
  const uint32_t pk_rowb = (uint32_t)p.pk_sr, pq_rowb = (uint32_t)p.pq_sr;  // the host bounds them (24-bit row strides)
  auto batch_dma = [&](int delta, int slot) __attribute__((always_inline)) {
    const uint32_t seg = (uint32_t)slot * (32 * kRow8);
    if (wave < 2) {
      if constexpr (C2P) dma16sn(pkb, __umul24((uint32_t)delta, pk_rowb) + chunk8, ek_lds + seg);
    } else {
      if constexpr (P2C) dma16sn(pqb, __umul24((uint32_t)delta, pq_rowb) + chunk8, eq_lds + seg);
    }
  };

  f32x16 o_acc[DBLKS];
#pragma unroll
  for (int d = 0; d < DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- per-lane constants (see the 16-bit near kernel for the derivations) --------------------------------------
  const int arow = 31 - li, fr = f8(arow);  // MFMA row m = li of a position product is row 31 - li of its batch
  const uint32_t ra0 = (uint32_t)(arow * kRow8) + (uint32_t)(((2 * g) ^ fr) * 16), ra1 = (uint32_t)(arow * kRow8) + (uint32_t)(((2 * g + 1) ^ fr) * 16);
  const uint32_t kx0 = lds0 + (uint32_t)(li * kRow8 + ((2 * g) ^ f8(li)) * 16), kx1 = lds0 + (uint32_t)(li * kRow8 + ((2 * g + 1) ^ f8(li)) * 16);
  uint32_t vlx[4];
  {
    const int s16 = lane & 15, grp = lane >> 4;
    const int slotl = (2 * (grp & 1) + ((s16 & 3) >> 1)) ^ (4 * ((s16 >> 3) & 1)) ^ (grp >> 1);
    const uint32_t vlane = (4 * (grp >> 1) + (s16 >> 2)) * kRowV + slotl * 16 + (s16 & 1) * 8;
#pragma unroll
    for (int x = 0; x < 4; ++x) vlx[x] = lds0 + (uint32_t)(Vs - smem) + (vlane ^ (64 * (x >> 1) ^ 32 * (x & 1)));
  }
  // C's scratch: row li, two halves of 32 columns that alternate with the step's parity (+ columns 0..3 once more)
  const uint32_t scr0 = lds0 + (uint32_t)(scr_raw - smem) + (uint32_t)wave * (kScrElems * 2) + (uint32_t)li * (kScrPitch * 2);
  uint16_t* c_wr = (uint16_t*)scr_raw + wave * kScrElems + li * kScrPitch + 4 * g;
  uint16_t* c_dup = g == 0 ? c_wr + 64 : c_wr;
  uint32_t c_rd[2][4];
#pragma unroll
  for (int par = 0; par < 2; ++par)
#pragma unroll
    for (int q = 0; q < 4; ++q) c_rd[par][q] = scr0 + 2u * (uint32_t)((32 * par + li + 29 - 8 * q - 4 * g) & 63);
  const int xl = li + 4 * g;  // P: a source lane (n = li) of register v hands out block 1 where n + jj < 32

  const uint32_t ek0 = lds0 + (uint32_t)(EK - smem), eq0 = lds0 + (uint32_t)(EQ - smem);
  auto ring_frag = [&](uint32_t ring, int slot) __attribute__((always_inline)) {
    const uint32_t boff = (uint32_t)slot * (32 * kRow8);
    return lds_frag8(ring + boff + ra0, ring + boff + ra1);
  };
  f32x16 zero;
#pragma unroll
  for (int v = 0; v < 16; ++v) zero[v] = 0.f;
  auto c_store = [&](const f32x16& cacc, int half) __attribute__((always_inline)) {
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const u32x2 packed = {__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(cacc[4 * q4], cacc[4 * q4 + 1])),
                            __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(cacc[4 * q4 + 2], cacc[4 * q4 + 3]))};
      *(u32x2*)(c_wr + 32 * half + 8 * q4) = packed;
      if (half == 0 && q4 == 0) *(u32x2*)c_dup = packed;
    }
  };
  int slot_k = 4 - wave, slot_q = 4 - wave;  // ring slots of this wave's block 0
  const int ring_n = wave < 2 ? kRingBatchesK : kRingBatchesQ;  // the ring this wave's loads fill
  int slot_dma = wave < 2 ? 0 : 5;                              // and the slot of it that the step's loads fill
  // ---- prologue -----------------------------------------------------------------------------------------------
  if (n_steps > 0) {
    k_dma(s0, 0);
    v_dma(s0, 0);
    int d0[6];
#pragma unroll
    for (int bt = 0; bt < 6; ++bt) d0[bt] = batch_delta();
#pragma unroll
    for (int bt = 0; bt < 6; ++bt) asm volatile("" : "+v"(d0[bt]));
#pragma unroll
    for (int bt = 0; bt < 5; ++bt) batch_dma(d0[bt], bt);
    dnext = d0[5];
    wait_vmcnt<0>();
    __syncthreads();
    if constexpr (C2P) c_store(mma8_sa<127 - kCShift>(ring_frag(ek0, 3 - wave), qf, zero), 1);  // block 1 of step 0
  }

  auto step = [&](auto mask_tag, auto par_tag, int k) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr int PAR = decltype(par_tag)::value;
    const int s = s0 + k;
    const int j0 = s * kStep;
    wait_vmcnt<0>();
    asm volatile("" : "+v"(dnext));
    __syncthreads();
    k_dma(s + 1, PAR ^ 1);
    v_dma(s + 1, PAR ^ 1);
    batch_dma(dnext, slot_dma);  // batch k + 5 in place of batch k (E_K) or k - 1 (E_Q)
    __builtin_amdgcn_sched_barrier(0);
    dnext = batch_delta();
    const i32x8 kf = lds_frag8(kx0 + PAR * N8::K_BYTES, kx1 + PAR * N8::K_BYTES);
    f32x16 sacc, cnew, pacc[2];
    if constexpr (C2P) cnew = mma8_sa<127 - kCShift>(ring_frag(ek0, slot_k), qf, zero);
    if constexpr (P2C) pacc[1] = mma8(kf, ring_frag(eq0, slot_q == 0 ? kRingBatchesQ - 1 : slot_q - 1), zero);
    if constexpr (P2C) pacc[0] = mma8(kf, ring_frag(eq0, slot_q), zero);
    sacc = mma8(kf, qf, zero);
    uint32_t craw[16];
    if constexpr (C2P) {
      c_store(cnew, PAR);
      wave_lds_fence();
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        craw[4 * q + 0] = lds_u16_asm<0>(c_rd[PAR][q]);
        craw[4 * q + 1] = lds_u16_asm<2>(c_rd[PAR][q]);
        craw[4 * q + 2] = lds_u16_asm<4>(c_rd[PAR][q]);
        craw[4 * q + 3] = lds_u16_asm<6>(c_rd[PAR][q]);
      }
      wave_lds_fence();
    }
    float px[16];
    if constexpr (P2C) {
      float xs[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int c = 8 * (v >> 2) + 3 - (v & 3);  // jj - 4g
        xs[v] = (xl < 32 - c) ? pacc[1][v] : pacc[0][v];
      }
      if (g == 0)
        rotate16<32>(xs, px, std::make_integer_sequence<int, 16>{});
      else
        rotate16<28>(xs, px, std::make_integer_sequence<int, 16>{});
    }
    vfrag vfr[2][DBLKS];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int d = 0; d < DBLKS; ++d) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(uintptr_t)(vlx[2 * d] + PAR * N8::V_BYTES + 2048 * c));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(uintptr_t)(vlx[2 * d + 1] + PAR * N8::V_BYTES + 2048 * c + 1024));
        vfr[c][d] = __builtin_bit_cast(vfrag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (C2P || P2C) {
      lds_wait_all8();
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if constexpr (C2P) asm volatile("" : "+v"(craw[v]));
        if constexpr (P2C) asm volatile("" : "+v"(px[v]));
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      if constexpr (C2P) sacc[v] = __builtin_fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)craw[v]), rho_c, sacc[v]);
      if constexpr (P2C) sacc[v] = __builtin_fmaf(px[v], rho_p, sacc[v]);
    }
    if constexpr (MASK) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + 8 * (v >> 2) + 4 * g + 3 - (v & 3);
        if (j >= Lb || (p.causal && j > i)) sacc[v] = -INFINITY;
      }
    }
    vfrag pf[2];
    float l_blk = 0.f;
    auto probs = [&](float off) __attribute__((always_inline)) {
      l_blk = 0.f;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        f32x8 pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[8 * c + (e ^ 3)], x_scale, off));
        pf[c] = VT::from_f32(pv);
        l_blk = sum8(pv, l_blk);
      }
    };
    bool slow = __any(m_run == -INFINITY);
    if (!slow) {
      probs(-m_run);
      slow = __any(!(l_blk <= 256.f));
    }
    if (slow) {
      float mx = sacc[0];
#pragma unroll
      for (int v = 1; v < 16; ++v) mx = fmaxf(mx, sacc[v]);
      mx = wave_half_max(mx) * x_scale;
      if (__any(mx > m_run + kLazyTau)) {
        const float m_new = (mx > m_run + kLazyTau) ? mx : m_run;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run *= alpha;
        m_run = m_new;
#pragma unroll
        for (int d = 0; d < DBLKS; ++d)
#pragma unroll
          for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
      }
      probs((MASK && m_run == -INFINITY) ? 0.f : -m_run);
    }
    l_run += l_blk;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int d = 0; d < DBLKS; ++d) o_acc[d] = VT::mma(vfr[c][d], pf[c], o_acc[d]);
    slot_k = slot_k == kRingBatchesK - 1 ? 0 : slot_k + 1;
    slot_q = slot_q == kRingBatchesQ - 1 ? 0 : slot_q + 1;
    slot_dma = slot_dma == ring_n - 1 ? 0 : slot_dma + 1;
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
  wait_vmcnt<0>();  // none of the last step's direct loads may still be writing LDS when the workgroup ends

  // ---- epilogue: merge with the far tiles' partial results, normalise, store (as in the 16-bit near kernel) ------
  const float l_tot = wave_half_sum(l_run);
  if (i < Lb) {
    char* orow = ob + (int64_t)i * p.o_st * 2;
    const int64_t tok = p.cu ? (int64_t)tok0 + i : (int64_t)b * p.L + tok0 + i;
    if (p.near_parts > 1) {
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
    const int n_far = p.far_done ? p.far_parts : 0;
    float w_far[FDB_MAX_FAR_PARTS], w_near = 1.f, m_out = m_run;
    const char* far_row[FDB_MAX_FAR_PARTS];
#pragma unroll
    for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s) {
      w_far[s] = -INFINITY;
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

template <bool C2P, bool P2C>
int launch_near8_one(const FdbKParams& p, int grid_x, hipStream_t stream) {
  auto kern = fdb_near8_kernel<C2P, P2C>;
  constexpr int lds = N8::lds_bytes(C2P, P2C);
  static_assert(lds <= 52 * 1024, "three workgroups per CU: with 53 KB a CU was seen to take only two");
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = fdb_set_lds_once((const void*)kern, lds, lds_set);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid_x * p.H, p.near_parts > 1 ? (unsigned)p.near_parts : 1u, 1), dim3(kThreads), lds,
                     stream, p);
  return (int)hipGetLastError();
}

}  // namespace

bool fdb_fp8_pair_supported(int dtype, int head_dim) { return dtype == FDB_FP8_E4M3 && head_dim == 64; }

int fdb_launch_far8(const FdbKParams& p, int grid_x, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (p.pk && p.pq) return launch_far8_one<true, true>(p, grid_x, stream);
  if (p.pk) return launch_far8_one<true, false>(p, grid_x, stream);
  if (p.pq) return launch_far8_one<false, true>(p, grid_x, stream);
  return FDB_ERR_UNSUPPORTED;
}

int fdb_launch_near8(const FdbKParams& p, int grid_x, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (p.pk && p.pq) return launch_near8_one<true, true>(p, grid_x, stream);
  if (p.pk) return launch_near8_one<true, false>(p, grid_x, stream);
  if (p.pq) return launch_near8_one<false, true>(p, grid_x, stream);
  return FDB_ERR_UNSUPPORTED;
}
