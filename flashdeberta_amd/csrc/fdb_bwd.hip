// Backward of the disentangled attention for gfx950: dQ, dK, dV and the gradients of the two
// position-score tensors, from the saved log-sum-exp.  Counterpart of the reference's three backward
// kernels (src/flashdeberta/ops/flash_attention.py:62-141 _bwd_preprocess, :581-760 _bwd_kv_dise_kernel,
// :762-941 _bwd_q_dise_kernel, launcher :942-1030): like them it takes the position scores
// c2p[b,i,h,delta] = q_i . K_r[delta] and p2c[b,j,h,delta] = k_j . Q_r[delta] as tensors, gathers them through
// the bucketed relative position, and scatter-adds the score gradients into tensors of the same shape
// (the reference: tl.atomic_add, :769-786); the chain through K_r / Q_r is left to the caller's GEMMs.
//
// One kernel in two roles.  A workgroup owns 128 rows of the "lane side" (4 waves x 32 rows, one row per
// lane and its partner lane ^ 32) and walks the "loop side" 32 rows at a time through LDS:
//   role dQ    : lane side = queries (q, dO in registers), loop side = keys (K, V tiles)  ->  dQ, d c2p
//   role dK/dV : lane side = keys (k, v in registers), loop side = queries (Q, dO tiles) ->  dK, dV, d p2c
// Per step, with X the lane side and Y the loop side (MFMA 32x32, M = loop row, N = lane row):
//   S' = Y1 X1^T (+ gathered position scores), P' = exp2(S' * c log2e - lse_i log2e), dP' = Y2 X2^T,
//   dS' = P' (dP' - Delta_i) c, and the outputs contract over the loop rows, which sit in the accumulator
//   registers: out^T += Y^T dS' (or P'), with Y^T read transposed from LDS -- the layout trick of the forward.
// A step whose relative positions all lie beyond the table radius has one table row: its position scores are
// one load per row and its score gradients leave as one row sum per lane instead of one atomic per element.
#include <hip/hip_runtime.h>
#include <hip/amd_detail/amd_hip_unsafe_atomics.h>
#include <stdint.h>

#include <atomic>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

using namespace fdb;

namespace {

constexpr int kBwdThreads = 256;
constexpr int kBwdStep = 32;    // loop-side rows per step
constexpr int kLutLds = 4096;   // table entries kept in LDS (larger tables are read from global memory)

template <class QT, int D>
struct BCfg {
  static constexpr int KS = D / 16, DBLKS = D / 32;
  static constexpr int RS = D * QT::SZ + 16;                 // LDS row stride of a staged tile
  static constexpr int TILE = kBwdStep * RS;
  static constexpr int CHUNKS = (kBwdStep * D * QT::SZ / 16 + kBwdThreads - 1) / kBwdThreads;  // 16-byte chunks per thread
  static constexpr int lds_bytes() { return 2 * TILE + 2 * kBwdStep * 4 + kLutLds * 2; }
};

// [32 x D] tile: global -> registers -> LDS.  Rows past the end re-read the last valid row; their scores are masked.
template <class QT, int D, int NCH>
__device__ __forceinline__ void btile_load(u32x4 (&reg)[NCH], const char* gbase, int64_t row_stride_bytes,
                                           int r0, int n_rows, int tid) {
  constexpr int CPR = D * QT::SZ / 16, TOTAL = kBwdStep * CPR;
#pragma unroll
  for (int n = 0; n < NCH; ++n) {
    const int c = tid + n * kBwdThreads;
    const int row = min(r0 + min(c / CPR, kBwdStep - 1), n_rows - 1), cc = c % CPR;
    if (TOTAL % kBwdThreads == 0 || c < TOTAL) reg[n] = *(const u32x4*)(gbase + (int64_t)row * row_stride_bytes + cc * 16);
  }
}
template <class QT, int D, int NCH>
__device__ __forceinline__ void btile_store(char* lds, const u32x4 (&reg)[NCH], int tid) {
  constexpr int CPR = D * QT::SZ / 16, TOTAL = kBwdStep * CPR;
#pragma unroll
  for (int n = 0; n < NCH; ++n) {
    const int c = tid + n * kBwdThreads;
    if (TOTAL % kBwdThreads == 0 || c < TOTAL) *(u32x4*)(lds + (c / CPR) * BCfg<QT, D>::RS + (c % CPR) * 16) = reg[n];
  }
}

template <class QT, int D, int ROLE, bool C2P, bool P2C>
__global__ __launch_bounds__(kBwdThreads) void fdb_bwd_kernel(const FdbBwdParams p) {
  using C = BCfg<QT, D>;
  using frag = typename QT::frag;
  constexpr int KS = C::KS, DBLKS = C::DBLKS;
  constexpr bool kDQ = ROLE == 0;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* Y1s = smem;                                   // K (dQ role) / Q (dK/dV role)
  char* Y2s = Y1s + C::TILE;                          // V / dO
  float* lse_s = (float*)(Y2s + C::TILE);             // dK/dV role: log-sum-exp (base 2) and Delta of the 32 loop rows
  float* del_s = lse_s + kBwdStep;
  int16_t* lut_s = (int16_t*)(del_s + kBwdStep);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, li = lane & 31, g = lane >> 5;
  const int h = blockIdx.y, b = blockIdx.z;
  const int m0 = blockIdx.x * FDB_BM;
  const int tok0 = p.seq_start ? min(max(p.seq_start[b], 0), p.L) : 0;
  const int Lb = p.seq_len ? min(max(p.seq_len[b], 0), p.L - tok0) : p.L;
  if (m0 >= Lb) return;
  const int n_lut = 2 * p.R + 1;
  const bool lut_in_lds = n_lut <= kLutLds;
  if (lut_in_lds && (C2P || P2C))
    for (int x = tid; x < n_lut; x += kBwdThreads) lut_s[x] = p.lut[x];

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
  // row statistics and position-score rows are token-major: row (b, tok0 + l), head h
  const int64_t tok_x = ((int64_t)b * p.L + tok0 + (x_ok ? xr : 0)) * p.H + h;
  float lse_x = 0.f, del_x = 0.f;
  if (kDQ && x_ok) {
    lse_x = p.lse[tok_x] * 1.4426950408889634f;
    del_x = p.delta[tok_x];
  }
  const int S2 = 2 * p.S;
  const float* cbx = C2P && kDQ ? p.c2p + tok_x * S2 : nullptr;     // this lane's row of the lane-side position scores
  const float* pbx = P2C && !kDQ ? p.p2c + tok_x * S2 : nullptr;
  // Score gradients.  A far step (one table row for the block) adds the lane side's: one row sum per lane.  A near
  // step adds the loop side's: register v is one row of that tensor and the 32 lanes of a half-wave fall on
  // neighbouring table rows, so an atomic instruction touches a few cache lines instead of 64.  The other half of
  // each tensor comes from the other role's launch, which classifies the same 32 x 32 blocks the same way.
  float* gx = kDQ ? (C2P ? p.d_c2p + tok_x * S2 : nullptr) : (P2C ? p.d_p2c + tok_x * S2 : nullptr);
  float* gy = kDQ ? (P2C ? p.d_p2c : nullptr) : (C2P ? p.d_c2p : nullptr);

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
  u32x4 y1reg[C::CHUNKS], y2reg[C::CHUNKS];
  float st_reg[2] = {0.f, 0.f};
  auto stats_load = [&](int r0) __attribute__((always_inline)) {
    if (!kDQ && tid < kBwdStep) {
      const int row = min(r0 + tid, Lb - 1);
      const int64_t t = ((int64_t)b * p.L + tok0 + row) * p.H + h;
      st_reg[0] = p.lse[t] * 1.4426950408889634f;
      st_reg[1] = p.delta[t];
    }
  };
  if (y_lo < y_hi) {
    btile_load<QT, D>(y1reg, y1b, y1_rsb, y_lo, Lb, tid);
    btile_load<QT, D>(y2reg, y2b, y2_rsb, y_lo, Lb, tid);
    stats_load(y_lo);
  }
  const float c_log2 = p.scale_log2, c_sm = p.sm_scale;
  auto delta_of = [&](int r) __attribute__((always_inline)) -> int {
    const int x = max(-p.R, min(p.R, r)) + p.R;
    return lut_in_lds ? (int)lut_s[x] : (int)p.lut[x];
  };

  for (int y0 = y_lo; y0 < y_hi; y0 += kBwdStep) {
    __syncthreads();  // every wave is done with the tiles of the step before (and the table is in LDS)
    btile_store<QT, D>(Y1s, y1reg, tid);
    btile_store<QT, D>(Y2s, y2reg, tid);
    if (!kDQ && tid < kBwdStep) {
      lse_s[tid] = st_reg[0];
      del_s[tid] = st_reg[1];
    }
    __syncthreads();
    if (y0 + kBwdStep < y_hi) {
      btile_load<QT, D>(y1reg, y1b, y1_rsb, y0 + kBwdStep, Lb, tid);
      btile_load<QT, D>(y2reg, y2b, y2_rsb, y0 + kBwdStep, Lb, tid);
      stats_load(y0 + kBwdStep);
    }
    // ---- S' and dP' ----------------------------------------------------------------------------------------
    f32x16 sacc, dpacc;
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[v] = dpacc[v] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const frag y1f = QT::load(Y1s + li * C::RS + (16 * s + 8 * g) * QT::SZ);
      const frag y2f = QT::load(Y2s + li * C::RS + (16 * s + 8 * g) * QT::SZ);
      sacc = QT::mma(y1f, x1f[s], sacc);
      dpacc = QT::mma(y2f, x2f[s], dpacc);
    }
    // ---- position scores, probabilities, score gradients -------------------------------------------------------
    // element v of lane (g, li): loop row yr = y0 + 8*(v/4) + 4g + v%4, lane row xr; i - j = +-(xr - yr)
    const int r_min = kDQ ? xw0 - (y0 + kBwdStep - 1) : y0 - (xw0 + 31);      // over the wave's 32 x 32 block
    const int r_max = kDQ ? xw0 + 31 - y0 : y0 + kBwdStep - 1 - xw0;
    const bool far = (C2P || P2C) && (r_min >= p.R || r_max <= -p.R);  // one table row for the whole block
    const int d_far = far ? delta_of(r_min) : 0;
    float lane_bias = 0.f;
    if (far) {
      if (C2P && kDQ) lane_bias = cbx[d_far];
      if (P2C && !kDQ) lane_bias = pbx[d_far];
    }
    // Every position score of the step is requested before the first one is used: the loads are unconditional
    // (rows past the end read the last valid row, lanes past the end read row 0) and only their use is masked,
    // so that sixteen elements cost one round trip to memory, not sixteen.
    float ds[16], pr[16], g_sum = 0.f, bias[16];
    int dl[16];
    bool ok[16];
    int64_t goff[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int yr = y0 + 8 * (v >> 2) + 4 * g + (v & 3);
      const int i = kDQ ? xr : yr, j = kDQ ? yr : xr;
      ok[v] = x_ok && yr < Lb && (!p.causal || j <= i);
      dl[v] = far ? d_far : ((C2P || P2C) ? delta_of(i - j) : 0);
      const int64_t tok_y = ((int64_t)b * p.L + tok0 + min(yr, Lb - 1)) * p.H + h;
      float bv = 0.f;
      if (C2P) bv += kDQ ? (far ? lane_bias : cbx[dl[v]]) : p.c2p[tok_y * S2 + dl[v]];
      if (P2C) bv += kDQ ? p.p2c[tok_y * S2 + dl[v]] : (far ? lane_bias : pbx[dl[v]]);
      bias[v] = bv;
      goff[v] = tok_y * S2 + dl[v];
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int yl = 8 * (v >> 2) + 4 * g + (v & 3);
      const float lse_i = kDQ ? lse_x : lse_s[yl], del_i = kDQ ? del_x : del_s[yl];
      const float pv = ok[v] ? __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[v] + bias[v], c_log2, -lse_i)) : 0.f;
      pr[v] = pv;
      ds[v] = pv * (dpacc[v] - del_i) * c_sm;
      g_sum += ds[v];
    }
    if (gy != nullptr && !far) {
#pragma unroll
      for (int v = 0; v < 16; ++v)
        if (ok[v]) unsafeAtomicAdd(gy + goff[v], ds[v]);
    }
    if (gx != nullptr && far) {
      g_sum = wave_half_sum(g_sum);
      if (g == 0 && x_ok) unsafeAtomicAdd(gx + d_far, g_sum);
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

  if (!x_ok) return;
  auto write = [&](char* ptr, int64_t sb, int64_t st, int64_t sh, const f32x16 (&acc)[DBLKS]) {
    char* row = ptr + (b * sb + (int64_t)(tok0 + xr) * st + (int64_t)h * sh) * QT::SZ;
#pragma unroll
    for (int d = 0; d < DBLKS; ++d)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        QT::store4(row + (32 * d + 8 * q4 + 4 * g) * QT::SZ, acc[d][4 * q4], acc[d][4 * q4 + 1], acc[d][4 * q4 + 2], acc[d][4 * q4 + 3]);
  };
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
  constexpr int lds = BCfg<QT, D>::lds_bytes();
  static_assert(lds <= 160 * 1024, "LDS budget");
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = fdb_set_lds_once((const void*)kern, lds, lds_set);
  if (e != hipSuccess) return (int)e;
  const unsigned tiles = (unsigned)((p.L + FDB_BM - 1) / FDB_BM);
  hipLaunchKernelGGL(kern, dim3(tiles, (unsigned)p.H, (unsigned)p.B), dim3(kBwdThreads), lds, stream, p);
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
