// Near tiles of the disentangled-attention forward for gfx950, head_dim 64, 16-bit types: the key
// tiles of a query tile in which the bucketed relative position delta(i - j) is not constant
// (|i - j| < R + tile size).  Second launch of the two-launch path: the far tiles' partial result
// (rows normalised over the far keys in out, their log-sum-exp in lse) is merged in the epilogue.
//
// The position products need the rows E_K[r] = K_r[delta(r)] and E_Q[r] = Q_r[delta(r)] for the
// contiguous range of relative positions r of a tile.  They are staged in LDS rings with direct
// loads, so the MFMA A operands are plain LDS reads.
//
// What shapes this kernel is the issue rate of a wave: with two waves on a SIMD a wave issues one
// instruction of any kind -- vector, scalar, LDS, wait -- about every five clocks, and a step's time is its
// instruction count times that plus the MFMAs' own 32 clocks each; so the step is written for the fewest
// instructions, not for the fewest of one kind.  Two workgroups share a CU when each stays under 80 KB of
// LDS, which the rings allow only with 32-key steps:
//   workgroup = 4 waves x 32 query rows, one step = 32 keys;
//   a step sees 160 relative positions, five batches of 32, one per (wave, block); each ring holds exactly
//   these five (160 rows of 128 bytes, unpadded and XOR-swizzled): the batch a step's loads bring in for the
//   next step takes the place of the one no wave reads any more;
//   a wave's 32 x 32 sub-tile sees 63 relative positions, so both position products are 2 MFMA
//   blocks, private to the wave: C[r][i] = q_i . E_K[r] and P[j][r] = k_j . E_Q[r], of which element
//   (i, j) wants index r = i - j.  C goes through a per-wave 16-bit LDS scratch that holds both blocks: a
//   step contracts and writes only the block that is new to it (the other one is the block the step before
//   wrote), and reads its skewed band back with sixteen 2-byte loads that land in the upper half of a
//   register, i.e. as fp32 values; P is computed with the keys as MFMA rows, so its skew is a rotation
//   of the lanes of a half-wave by a constant of the register (ds_swizzle) and needs no scratch.
//   The query operand carries the soft-max scale and the content product starts from minus the row's
//   reference point, so the sum leaves for the exponential as it is.
// LDS: K 2 x 4 KB + V 2 x 4 KB + rings 2 x 20 KB + scratch 17 KB = 73 KB.
//
// Staging goes global -> LDS directly (global_load_lds_dwordx4: no staging registers, no LDS write
// instructions of the waves' own) and runs one step ahead: right after the one barrier of step s (every
// wave is done with step s-1) a wave issues its share of K(s+1) and V(s+1) into the buffers step s does not
// read and of the 32 rows per table that step s+1 reads for the first time;
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
constexpr int kRingBatches = 5;  // batches of 32 relative positions in a ring: the five a step reads
constexpr int kRingRows = 32 * kRingBatches;
constexpr int kScrPitch = 68;    // 16-bit elements per row of a wave's C scratch: two blocks of 32 columns + columns 0..3 once
                                 // more (a run of four never wraps); 34 words, so the 32 rows of a write land in 32 different bank pairs
constexpr int kScrElems = 32 * kScrPitch;
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
// ds_swizzle in rotate mode, the amount in the instruction's offset field (0xC000 | amount << 5).  Issued as asm, so
// that the compiler keeps no account of it: the step waits once for all its LDS traffic (lds_wait_all) instead
// of once per value.
template <int OFFSET>
__device__ __forceinline__ float swizzle_asm(float x) {
  float r;
  asm volatile("ds_swizzle_b32 %0, %1 offset:%2" : "=v"(r) : "v"(x), "n"(OFFSET));
  return r;
}
template <int ROT0, int... V>
__device__ __forceinline__ void rotate16(const float (&xs)[16], float (&px)[16], std::integer_sequence<int, V...>) {
  ((px[V] = swizzle_asm<(0xC000 | (((ROT0 - (8 * (V >> 2) + 3 - (V & 3))) & 31) << 5))>(xs[V])), ...);
}

// A 16-bit LDS element as fp32.  bf16: the load that fills the upper half of the register clears the lower half on
// this hardware, so the register is the value; issued as asm, the caller waits (lds_wait_all) before it uses the value.
template <class QT, int OFF>
__device__ __forceinline__ float lds_elem_f32(uint32_t addr) {
  if constexpr (std::is_same<QT, Bf16Tr>::value) {
    float r;
    asm volatile("ds_read_u16_d16_hi %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
  } else {
    return (float)*(LDS_AS const _Float16*)(uintptr_t)(addr + OFF);
  }
}
__device__ __forceinline__ void lds_wait_all() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

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
  // the query operand carries the soft-max scale (in base 2): the content product and C leave the MFMA in the
  // exponent's unit; P, which the keys make, is scaled where it is added
#pragma unroll
  for (int s = 0; s < KS; ++s) qf[s] = QT::from_f32(QT::to_f32(qf[s]) * x_scale);

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
  const int n_full = max(0, min(n_steps, (p.causal ? min(Lb, m0) : Lb) / kStep - s0));  // steps k < n_full need no mask

  // relative positions of the workgroup at step k = s - s0: r in [r_hi0 - 32k - 159, r_hi0 - 32k];
  // u = r_hi0 - r counts downwards from the first step's largest r; batch = u / 32, ring slot = batch mod 5.
  // Wave w's block bk at step k is batch k + 4 - w - bk, MFMA row m its row 31 - m: r = iw0 - 32s - 32 + 32bk + m.
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
  auto k_dma = [&](int s, int buf, bool inside) __attribute__((always_inline)) {
    // LDS row srow holds key srow ^ 3 of the step (see the scratch reads below); rows past the end
    // re-read the last one, their scores are masked
    const uint32_t dst = lds0 + buf * NCfg::K_BYTES + wave_kb;
    if (inside || (s + 1) * kStep <= Lb) {
      dma16sn(kb + (uint64_t)(uint32_t)(s * kStep) * k_rsb, k_lane, dst);
    } else {
      const int row = min(s * kStep + (srow ^ 3), Lb - 1);
      dma16n(kb + (uint64_t)(uint32_t)row * k_rsb + chunk_off, dst);
    }
  };
  auto v_dma = [&](int s, int buf, bool inside) __attribute__((always_inline)) {
    const uint32_t dst = lds0 + 2 * NCfg::K_BYTES + buf * NCfg::V_BYTES + wave_kb;
    if (inside || (s + 1) * kStep <= Lb) {
      dma16sn(vb + (uint64_t)(uint32_t)(s * kStep) * v_rsb, v_lane, dst);
    } else {
      const int row = min(s * kStep + srow, Lb - 1);
      dma16n(vb + (uint64_t)(uint32_t)row * v_rsb + chunk_off, dst);
    }
  };
  // table row of this thread's row of a batch; the relative position runs down by 32 per batch
  int r_tab = r_hi0 - srow;
  auto batch_delta = [&]() __attribute__((always_inline)) {
    // table rows are indices >= 0: read unsigned, so that the loaded register is the value and nothing
    // has to wait for the load before the next step uses it
    const int d = (int)((const uint16_t*)p.lut)[max(-p.R, min(p.R, r_tab)) + p.R];
    r_tab -= 32;
    return d;
  };
  const uint32_t ek_lds = lds0 + (uint32_t)(EK - smem) + wave_kb, eq_lds = lds0 + (uint32_t)(EQ - smem) + wave_kb;
  // table rows are addressed with 32-bit byte offsets from the head's first row (the host checks that a row stride
  // stays under 2^24 bytes and the whole table under 2^31)
  const uint32_t pk_rowb = (uint32_t)(p.pk_sr * 2), pq_rowb = (uint32_t)(p.pq_sr * 2);
  auto batch_dma = [&](int delta, int slot) __attribute__((always_inline)) {
    const uint32_t seg = (uint32_t)slot * (32 * kRowBytes);
    if constexpr (C2P) dma16sn(pkb, __umul24((uint32_t)delta, pk_rowb) + chunk_off, ek_lds + seg);
    if constexpr (P2C) dma16sn(pqb, __umul24((uint32_t)delta, pq_rowb) + chunk_off, eq_lds + seg);
  };

  f32x16 o_acc[DBLKS];
#pragma unroll
  for (int d = 0; d < DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  // the content product's accumulator starts from minus the row's reference point (0 before the row has one)
  f32x16 negm;
#pragma unroll
  for (int v = 0; v < 16; ++v) negm[v] = 0.f;

  // ---- per-lane constants ------------------------------------------------------------------------------
  // MFMA row m = li of a position product is row 31 - li of its batch; chunk 2x + g of that row sits in
  // slot (2x) ^ g ^ f(row).
  const int arow = 31 - li, fr = ring_f(arow);
  uint32_t ra[KS];
#pragma unroll
  for (int x = 0; x < KS; ++x)
    ra[x] = lds0 + (uint32_t)((C2P ? EK : EQ) - smem) + (uint32_t)(arow * kRowBytes) + (uint32_t)((((g ^ fr) * 16)) ^ (32 * x));
  uint32_t klx[KS], vlx[4];  // K fragment rows li; V^T operand (c, d-block db, half h): row 16c + 8h + 4*(grp/2) + s16/4,
                             // 8-byte unit 8db + 4*(grp%2) + s16%4, i.e. chunk ^ f = lane part ^ (4db) ^ (2h)
  {
    const int s16 = lane & 15, grp = lane >> 4;
    const int slotl = (2 * (grp & 1) + ((s16 & 3) >> 1)) ^ (4 * ((s16 >> 3) & 1)) ^ (grp >> 1);
    const uint32_t vlane = (4 * (grp >> 1) + (s16 >> 2)) * kRowBytes + slotl * 16 + (s16 & 1) * 8;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      klx[x] = lds0 + (uint32_t)(Ks - smem) + ((li * kRowBytes + ((g ^ ring_f(li)) * 16)) ^ (32 * x));  // absolute LDS addresses:
      vlx[x] = lds0 + (uint32_t)(Vs - smem) + (vlane ^ (64 * (x >> 1) ^ 32 * (x & 1)));                  // buffer and block are immediates
    }
  }
  // scratch: row li = this lane's query, 64 columns in two halves: the block a step contracts (its block 0, columns
  // rr = 0..31 of the step) goes to half PAR = step parity, and the other half still holds the block the step before
  // wrote there, which is this step's block 1 (rr = 32..63).  Element (jj, i = li) wants rr = li + 32 - jj, i.e. column
  // (32 PAR + li + 32 - jj) mod 64.  K's rows sit in LDS with the low two bits of the row index inverted, so MFMA
  // row m = 8q + 4g + e of the content product is key jj = 8q + 4g + 3 - e: the four C elements a lane adds to
  // consecutive accumulator registers are the run of columns that starts at (32 PAR + li + 29 - 8q - 4g) mod 64; columns
  // 64..67 repeat 0..3, so that a run never wraps.
  const uint32_t scr0 = lds0 + (uint32_t)(scr_raw - smem) + (uint32_t)wave * (kScrElems * 2) + (uint32_t)li * (kScrPitch * 2);
  uint16_t* c_wr = (uint16_t*)scr_raw + wave * kScrElems + li * kScrPitch + 4 * g;  // group q4 of half h at + 32 h + 8 q4
  uint16_t* c_dup = g == 0 ? c_wr + 64 : c_wr;  // where columns 0..3 go once more (the lanes that hold 4..7 write those again)
  uint32_t c_rd[2][4];
#pragma unroll
  for (int par = 0; par < 2; ++par)
#pragma unroll
    for (int q = 0; q < 4; ++q) c_rd[par][q] = scr0 + 2u * (uint32_t)((32 * par + li + 29 - 8 * q - 4 * g) & 63);
  const int xl = li + 4 * g;  // P: a source lane (n = li) of register v hands out block 1 where n + jj < 32

  // Block 1 of a step holds the rows that were block 0 of the step before, and a step reads only its
  // new block 0 from the rings.  C[r][i] does not depend on the keys, so C's block 1 IS the block 0 the
  // step before contracted: it is still in the scratch.  P depends on the step's keys: there the A operands
  // are kept, in two buffers that swap roles with the step's parity.
  qfrag ac[C2P ? KS : 1], aq[2][P2C ? KS : 1];
  auto ring_read = [&](int buf, int slot) __attribute__((always_inline)) {
    const uint32_t boff = (uint32_t)slot * (32 * kRowBytes);
#pragma unroll
    for (int x = 0; x < KS; ++x) {
      if constexpr (C2P) ac[x] = *(LDS_AS const qfrag*)(uintptr_t)(ra[x] + boff);
      if constexpr (P2C) aq[buf][x] = *(LDS_AS const qfrag*)(uintptr_t)(ra[x] + boff + (C2P ? NCfg::RING_BYTES : 0));
    }
  };
  f32x16 zero;
#pragma unroll
  for (int v = 0; v < 16; ++v) zero[v] = 0.f;
  // the block in cacc, rounded, to half `half` of the scratch
  auto c_store = [&](const f32x16& cacc, int half) __attribute__((always_inline)) {
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {  // C[i = li][8*q4 + 4*g + 0..3]
      const typename QT::scratch4 packed = QT::pack4(f32x4{cacc[4 * q4], cacc[4 * q4 + 1], cacc[4 * q4 + 2], cacc[4 * q4 + 3]});
      *(typename QT::scratch4*)(c_wr + 32 * half + 8 * q4) = packed;
      if (half == 0 && q4 == 0) *(typename QT::scratch4*)c_dup = packed;
    }
  };
  int slot_rd = 4 - wave;  // ring slot of this wave's block 0
  int slot_dma = 0;        // ring slot the step's loads fill
  // ---- prologue: step 0's K and ring batches 0..4 on their way to LDS -------------------------------------
  // All table values first, then all rows: the loads of one kind are in flight together.
  if (n_steps > 0) {
    k_dma(s0, 0, false);  // K and V need no table value: on their way while the table is read
    v_dma(s0, 0, false);
    int d0[6];
#pragma unroll
    for (int bt = 0; bt < 6; ++bt) d0[bt] = batch_delta();
    // (taken here, all at once: the compiler, which does not count the direct loads, would otherwise wait for
    // each value at its use, behind all the direct loads issued before it)
#pragma unroll
    for (int bt = 0; bt < 6; ++bt) asm volatile("" : "+v"(d0[bt]));
#pragma unroll
    for (int bt = 0; bt < 5; ++bt) batch_dma(d0[bt], bt);
    dnext = d0[5];
    wait_vmcnt<0>();
    __syncthreads();  // the prologue's ring rows
    ring_read(1, 3 - wave);  // block 1 of step 0
    if constexpr (C2P) {
      f32x16 c1;
#pragma unroll
      for (int x = 0; x < KS; ++x) c1 = QT::mma(ac[x], qf[x], x == 0 ? zero : c1);
      c_store(c1, 1);
    }
  }

  auto step = [&](auto mask_tag, auto par_tag, auto next_tag, int k) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr int PAR = decltype(par_tag)::value;  // parity of the step: its K / V buffers, its half of the scratch
    constexpr bool NEXT_INSIDE = decltype(next_tag)::value;  // the next step's keys all lie inside the sequence
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
    k_dma(s + 1, PAR ^ 1, NEXT_INSIDE);
    v_dma(s + 1, PAR ^ 1, NEXT_INSIDE);
    batch_dma(dnext, slot_dma);          // batch k + 5 in place of batch k
    __builtin_amdgcn_sched_barrier(0);   // the table load stays behind the direct loads
    dnext = batch_delta();               // of batch k + 6, used a step from now
    // ---- operands of the step out of LDS ------------------------------------------------------------------
    qfrag kf[KS];
#pragma unroll
    for (int x = 0; x < KS; ++x) kf[x] = *(LDS_AS const qfrag*)(uintptr_t)(klx[x] + PAR * NCfg::K_BYTES);
    ring_read(PAR, slot_rd);
    // ---- the sixteen MFMAs of the four score products, in two pairs of chains that alternate (no MFMA waits for
    // its own previous link): C's new block with P's block 1 (whose operands are this step's keys and the rows
    // kept from the step before), then P's block 0 with the content product.  What follows C -- the write to the
    // scratch and the reads of the skewed band -- runs under the second pair.
    f32x16 sacc, cnew, pacc[2];
#pragma unroll
    for (int x = 0; x < KS; ++x) {
      if constexpr (C2P) cnew = QT::mma(ac[x], qf[x], x == 0 ? zero : cnew);
      if constexpr (P2C) pacc[1] = QT::mma(kf[x], aq[PAR ^ 1][x], x == 0 ? zero : pacc[1]);
    }
#pragma unroll
    for (int x = 0; x < KS; ++x) {
      if constexpr (P2C) pacc[0] = QT::mma(kf[x], aq[PAR][x], x == 0 ? zero : pacc[0]);
      sacc = QT::mma(kf[x], qf[x], x == 0 ? negm : sacc);
    }
    float cband[16];
    if constexpr (C2P) {
      c_store(cnew, PAR);
      wave_lds_fence();  // the LDS unit runs one wave's operations in order; this keeps the compiler from moving them
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        cband[4 * q + 0] = lds_elem_f32<QT, 0>(c_rd[PAR][q]);
        cband[4 * q + 1] = lds_elem_f32<QT, 2>(c_rd[PAR][q]);
        cband[4 * q + 2] = lds_elem_f32<QT, 4>(c_rd[PAR][q]);
        cband[4 * q + 3] = lds_elem_f32<QT, 6>(c_rd[PAR][q]);
      }
      wave_lds_fence();
    }
    // P with the keys as MFMA rows, like the content product: register v of lane (g, n) holds
    // P[jj(v, g)][32 bk + n], and element (jj, i = li) wants column li + 32 - jj of that row, i.e. the same
    // register of another lane of its own half: lane (li - jj) mod 32, block 1 if li >= jj.  Each source lane is
    // read by exactly one lane, which wants block 1 from it if n + jj < 32 and block 0 otherwise: the source
    // picks (a compare of its lane constant with a constant of the register), and a rotation of each half-wave
    // by 32 - jj moves it: ds_swizzle in rotate mode, no address registers; the halves differ by 4 in jj, so each
    // half runs its own sixteen under its half of the execution mask.
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
    // V^T operands requested here, ahead of the soft-max, so that the four MFMAs at the end of the step find them
    vfrag vfr[2][DBLKS];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int d = 0; d < DBLKS; ++d) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(uintptr_t)(vlx[2 * d] + PAR * NCfg::V_BYTES + 2048 * c));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(uintptr_t)(vlx[2 * d + 1] + PAR * NCfg::V_BYTES + 2048 * c + 1024));
        vfr[c][d] = __builtin_bit_cast(vfrag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    __builtin_amdgcn_sched_barrier(0);
    // one wait for the band of C and the rotated P (issued as asm: the compiler keeps no count of them)
    if constexpr (C2P || P2C) {
      lds_wait_all();
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if constexpr (C2P && std::is_same<QT, Bf16Tr>::value) asm volatile("" : "+v"(cband[v]));
        if constexpr (P2C) asm volatile("" : "+v"(px[v]));
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      if constexpr (C2P) sacc[v] += cband[v];
      if constexpr (P2C) sacc[v] = __builtin_fmaf(px[v], x_scale, sacc[v]);
    }
    // ---- mask, online soft-max in base 2, O^T += V^T P^T ---------------------------------------------------
    if constexpr (MASK) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + 8 * (v >> 2) + 4 * g + 3 - (v & 3);
        if (j >= Lb || (p.causal && j > i)) sacc[v] = -INFINITY;
      }
    }
    // sacc = score - reference point.  The probabilities are formed first; the half-row sum of a step bounds its
    // largest one, so while it stays under 2^kLazyTau nothing has to move and no maximum is taken.  Otherwise (or
    // before a row has a reference point) the wave takes the maximum, moves the reference points of the rows that
    // need it, shifts the step's scores and forms the probabilities again.
    vfrag pf[2];
    float l_blk = 0.f;
    auto probs = [&]() __attribute__((always_inline)) {
      l_blk = 0.f;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        f32x8 pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f(sacc[8 * c + (e ^ 3)]);  // the V^T operand takes the keys in ascending order
        pf[c] = VT::from_f32(pv);
        l_blk = sum8(pv, l_blk);
      }
    };
    const bool first = m_run == -INFINITY;
    bool slow = __any(first);
    if (!slow) {
      probs();
      slow = __any(!(l_blk <= 256.f));  // 2^kLazyTau; also true for an overflow
    }
    if (slow) {
      float mx = sacc[0];
#pragma unroll
      for (int v = 1; v < 16; ++v) mx = fmaxf(mx, sacc[v]);
      mx = wave_half_max(mx);  // relative to the reference point (to 0 while the row has none)
      const bool mv = first ? mx > -INFINITY : mx > kLazyTau;
      if (__any(mv)) {
        const float shift = mv ? mx : 0.f;
        const float alpha = first ? 0.f : __builtin_amdgcn_exp2f(-shift);  // 1 where nothing moves
        if (mv) m_run = (first ? 0.f : m_run) + shift;
        l_run *= alpha;
#pragma unroll
        for (int d = 0; d < DBLKS; ++d)
#pragma unroll
          for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
#pragma unroll
        for (int v = 0; v < 16; ++v) sacc[v] -= shift;
        const float nm = m_run == -INFINITY ? 0.f : -m_run;
#pragma unroll
        for (int v = 0; v < 16; ++v) negm[v] = nm;
      }
      probs();
    }
    l_run += l_blk;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int d = 0; d < DBLKS; ++d) o_acc[d] = VT::mma(vfr[c][d], pf[c], o_acc[d]);
    slot_rd = slot_rd == kRingBatches - 1 ? 0 : slot_rd + 1;
    slot_dma = slot_dma == kRingBatches - 1 ? 0 : slot_dma + 1;
  };
  {
    using T0 = std::integral_constant<int, 0>;
    using T1 = std::integral_constant<int, 1>;
    using Y = std::true_type;
    using N = std::false_type;
    int k = 0;
    // the bulk: unmasked steps whose successor is unmasked too (its rows need no clamping)
#pragma unroll 1
    for (; k + 2 < n_full; k += 2) {
      step(N{}, T0{}, Y{}, k);
      step(N{}, T1{}, Y{}, k + 1);
    }
#pragma unroll 1
    for (; k + 1 < n_full; k += 2) {
      step(N{}, T0{}, N{}, k);
      step(N{}, T1{}, N{}, k + 1);
    }
    if (k < n_full) {
      step(N{}, T0{}, N{}, k);
      ++k;
    }
    if ((k & 1) && k < n_steps) {
      step(Y{}, T1{}, N{}, k);
      ++k;
    }
#pragma unroll 1
    for (; k + 1 < n_steps; k += 2) {
      step(Y{}, T0{}, N{}, k);
      step(Y{}, T1{}, N{}, k + 1);
    }
    if (k < n_steps) step(Y{}, T0{}, N{}, k);
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
