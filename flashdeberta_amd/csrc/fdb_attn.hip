// Fused DeBERTa disentangled-attention forward for gfx950 (MI355X, CDNA4).
//
// One workgroup = 4 wavefronts = 128 query rows of one (sequence, head); each wavefront owns 32
// rows.  The main loop walks the keys 64 at a time.  Everything is computed "transposed" so that a
// lane owns one query row:  S^T = K Q^T  (MFMA 32x32, M = key, N = query), the soft-max statistics
// of a row live in one lane (and its partner lane^32), and  O^T = V^T P^T  takes P straight from
// the S accumulators as its B operand.
//
// Position terms (what the reference reads from two pre-multiplied [B,H,L,2S] tensors with a
// per-element float log-bucket, src/flashdeberta/ops/flash_attention.py:236-268): for a tile the
// relative positions r = i - j form a contiguous range, so the tile's content->position scores
// are  C[r, i] = q_i . K_r[delta(r)]  and the position->content scores  P[r, j] = k_j . Q_r[delta(r)],
// both plain MFMA products whose A rows are gathered through the integer table delta(r).  They
// are parked in LDS indexed by r, and the element (i, j) picks C[i-j, i] + P[i-j, j]: an address
// that is affine in (i, j), no per-element bucket arithmetic and no trip to HBM.
// Tiles whose r range lies entirely in a saturated zone of delta (|i-j| large) need a single row
// of K_r / Q_r: the bias is a_i + b_j and enters through the MFMA accumulator initial value.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fdb_kernels.h"
#include "../../include/fdb.h"

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define LDS_AS __attribute__((address_space(3)))

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kC2pRows = 96;   // 32 + 64 - 1 relative positions per wave tile, padded to 3 MFMA blocks
constexpr int kP2cRows = 192;  // 128 + 64 - 1 per workgroup tile, padded to 6 MFMA blocks
constexpr int kP2cStride = 65; // odd stride: the skewed read walks rows and columns together

// ---- element traits --------------------------------------------------------------------------
// frag: the 8 contraction elements one lane feeds to a K=16 step (lane = outer index l%32, the
// elements are k = 16*step + 8*(l/32) + 0..7).
struct Bf16Tr {
  static constexpr int SZ = 2;
  using frag = bf16x8;
  static __device__ __forceinline__ frag zero() { return frag{0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const frag*)p; }
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ frag from_f32(f32x8 x) { return __builtin_convertvector(x, frag); }
  static __device__ __forceinline__ void store4(char* p, float a, float b, float c, float d) {
    f32x4 x = {a, b, c, d};
    *(bf16x4*)p = __builtin_convertvector(x, bf16x4);
  }
};

struct F16Tr {
  static constexpr int SZ = 2;
  using frag = f16x8;
  static __device__ __forceinline__ frag zero() { return frag{0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const frag*)p; }
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ frag from_f32(f32x8 x) { return __builtin_convertvector(x, frag); }
  static __device__ __forceinline__ void store4(char* p, float a, float b, float c, float d) {
    f32x4 x = {a, b, c, d};
    *(f16x4*)p = __builtin_convertvector(x, f16x4);
  }
};

struct F32Tr {
  static constexpr int SZ = 4;
  using frag = f32x8;
  static __device__ __forceinline__ frag zero() { return frag{0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const frag*)p; }
  // A K=16 step in fp32 is eight K=2 MFMAs; lane group g supplies k = 16*step + 8*g + e to the e-th.
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
#pragma unroll
    for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    return c;
  }
  static __device__ __forceinline__ frag from_f32(f32x8 x) { return x; }
  static __device__ __forceinline__ void store4(char* p, float a, float b, float c, float d) {
    *(f32x4*)p = f32x4{a, b, c, d};
  }
};

struct Fp8Tr {  // OCP e4m3, operands of the three score products only
  static constexpr int SZ = 1;
  using frag = long;
  static __device__ __forceinline__ frag zero() { return 0; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const long*)p; }
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a, b, c, 0, 0, 0);
  }
};

// V^T operand of a K=16 step: lane (d = l%32, g = l/32) needs V[j(g,e)][d] for
// j(g,e) = 16*c + 8*(e/4) + 4*g + e%4 -- the key rows whose probabilities sit in this lane
// group's accumulator registers.  V stays row-major in LDS.
template <class VT>
struct VtLoad;

template <>
struct VtLoad<F32Tr> {
  static __device__ __forceinline__ f32x8 get(const char* vs, int rs, int c, int db, int lane) {
    const int li = lane & 31, g = lane >> 5;
    f32x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int row = 16 * c + 8 * (e >> 2) + 4 * g + (e & 3);
      r[e] = *(const float*)(vs + row * rs + (db * 32 + li) * 4);
    }
    return r;
  }
};

// 16-bit: ds_read_tr16_b64.  Within each group of 16 lanes, source lane s supplies an 8-byte
// address; destination lane i receives element (i%4) of source lanes 4*r + i/4, r = 0..3.
// With source lane s pointing at V[row0 + s/4][col0 + 4*(s%4) ..+3], lane i gets column
// col0 + i of rows row0 .. row0+3.
template <class VT>
struct VtLoad16 {
  static __device__ __forceinline__ typename VT::frag get(const char* vs, int rs, int c, int db, int lane) {
    const int s = lane & 15, grp = lane >> 4;
    const int row = 16 * c + 4 * (grp >> 1) + (s >> 2);
    const int col = db * 32 + 16 * (grp & 1) + 4 * (s & 3);
    const char* a = vs + row * rs + col * 2;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(a));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(a + 8 * rs));
    s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(typename VT::frag, both);
  }
};
template <>
struct VtLoad<Bf16Tr> : VtLoad16<Bf16Tr> {};
template <>
struct VtLoad<F16Tr> : VtLoad16<F16Tr> {};

// combine lane l with lane l^32 (the other half of the row's keys)
__device__ __forceinline__ float wave_half_max(float x) { return fmaxf(x, __shfl_xor(x, 32)); }
__device__ __forceinline__ float wave_half_sum(float x) { return x + __shfl_xor(x, 32); }

template <class QT, class VT, int D>
struct Cfg {
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLKS = D / 32;
  static constexpr int K_RS = D * QT::SZ + 16;  // LDS row stride (bytes) of the K tile
  static constexpr int V_RS = D * VT::SZ + 16;
  static constexpr int K_BYTES = FDB_BN * K_RS;
  static constexpr int V_BYTES = FDB_BN * V_RS;
  static constexpr int C2P_BYTES = kWaves * kC2pRows * 32 * 4;
  static constexpr int P2C_BYTES = kP2cRows * kP2cStride * 4;
  static constexpr int FAR_BYTES = FDB_BN * 4;
  static constexpr int LDS_BYTES = K_BYTES + V_BYTES + C2P_BYTES + P2C_BYTES + FAR_BYTES;
};

// Copy a [64 x D] tile (rows j0.., zero beyond n_valid rows) from global to LDS in 16-byte chunks.
template <int ROW_BYTES, int RS>
__device__ __forceinline__ void stage_tile(char* lds, const char* gbase, int64_t row_stride_bytes, int j0,
                                           int n_rows, int tid) {
  constexpr int CPR = ROW_BYTES / 16;
  constexpr int TOTAL = FDB_BN * CPR;
#pragma unroll
  for (int c = tid; c < TOTAL; c += kThreads) {
    const int row = c / CPR, cc = c % CPR;
    u32x4 val = {0, 0, 0, 0};
    if (j0 + row < n_rows) val = *(const u32x4*)(gbase + (int64_t)(j0 + row) * row_stride_bytes + cc * 16);
    *(u32x4*)(lds + row * RS + cc * 16) = val;
  }
}

template <class QT, class VT, int D, bool FP8>
__global__ __launch_bounds__(kThreads, 1) void fdb_attn_kernel(const FdbKParams p) {
  using C = Cfg<QT, VT, D>;
  using qfrag = typename QT::frag;
  using vfrag = typename VT::frag;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* Ks = smem;
  char* Vs = Ks + C::K_BYTES;
  float* c2pS = (float*)(Vs + C::V_BYTES);
  float* p2cS = c2pS + C::C2P_BYTES / 4;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
  const int h = blockIdx.y;

  int b, m0, tok0, Lb;
  int64_t qo, ko, vo, oo;
  if (p.cu) {
    if ((int)blockIdx.x >= p.wl[0]) return;
    b = p.wl[2 + 2 * blockIdx.x];
    m0 = p.wl[3 + 2 * blockIdx.x];
    tok0 = p.cu[b];
    Lb = p.cu[b + 1] - tok0;
    qo = ko = vo = oo = 0;
  } else {
    b = blockIdx.x / p.tiles_per_seq;
    m0 = (blockIdx.x % p.tiles_per_seq) * FDB_BM;
    tok0 = p.seq_start ? min(max(p.seq_start[b], 0), p.L) : 0;
    Lb = p.seq_len ? min(max(p.seq_len[b], 0), p.L - tok0) : p.L;
    if (m0 >= Lb) return;
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; oo = b * p.o_sb;
  }
  const char* qb = p.q + (qo + (int64_t)tok0 * p.q_st + (int64_t)h * p.q_sh) * QT::SZ;
  const char* kb = p.k + (ko + (int64_t)tok0 * p.k_st + (int64_t)h * p.k_sh) * QT::SZ;
  const char* vb = p.v + (vo + (int64_t)tok0 * p.v_st + (int64_t)h * p.v_sh) * VT::SZ;
  char* ob = p.out + (oo + (int64_t)tok0 * p.o_st + (int64_t)h * p.o_sh) * VT::SZ;
  const char* pkb = p.pk ? p.pk + (int64_t)h * p.pk_sh * QT::SZ : nullptr;
  const char* pqb = p.pq ? p.pq + (int64_t)h * p.pq_sh * QT::SZ : nullptr;

  // fp8: raw products are in units of (q_scale*k_scale); bring the two position products to the
  // same unit so that one factor converts the sum.
  float x_scale = p.scale_log2, c2p_mul = 1.f, p2c_mul = 1.f;
  if constexpr (FP8) {
    const float qs = p.qs[h], ks = p.ks[h];
    x_scale *= qs * ks;
    if (pkb) c2p_mul = p.pks[h] / ks;
    if (pqb) p2c_mul = p.pqs[h] / qs;
  }

  const int iw0 = m0 + wave * 32;  // first row of this wave
  const int i = iw0 + li;          // this lane's query row (local to the sequence)

  qfrag qf[C::KSTEPS];
#pragma unroll
  for (int s = 0; s < C::KSTEPS; ++s)
    qf[s] = (i < Lb) ? QT::load(qb + ((int64_t)i * p.q_st + 16 * s + 8 * g) * QT::SZ) : QT::zero();

  f32x16 o_acc[C::DBLKS];
#pragma unroll
  for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // l_run: this lane's half of the row sum

  int j_end = Lb;
  if (p.causal) j_end = min(Lb, m0 + FDB_BM);

  for (int j0 = 0; j0 < j_end; j0 += FDB_BN) {
    __syncthreads();  // every wave is done with the previous tile and its bias scratch
    stage_tile<D * QT::SZ, C::K_RS>(Ks, kb, p.k_st * QT::SZ, j0, Lb, tid);
    stage_tile<D * VT::SZ, C::V_RS>(Vs, vb, p.v_st * VT::SZ, j0, Lb, tid);
    __syncthreads();

    // ---- S^T = K Q^T -------------------------------------------------------------------------
    f32x16 sacc[2];
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) sacc[jb][v] = 0.f;
#pragma unroll
      for (int s = 0; s < C::KSTEPS; ++s) {
        qfrag kf = QT::load(Ks + (jb * 32 + li) * C::K_RS + (16 * s + 8 * g) * QT::SZ);
        sacc[jb] = QT::mma(kf, qf[s], sacc[jb]);
      }
    }

    // ---- position terms ----------------------------------------------------------------------
    if (pkb) {
      // C[r - r_lo, i] for the 95 relative positions this wave's 32 rows see in this key tile
      const int r_lo = iw0 - (j0 + FDB_BN - 1);
#pragma unroll 1
      for (int blk = 0; blk < 3; ++blk) {
        int r = r_lo + 32 * blk + li;
        r = max(-p.R, min(p.R, r));
        const int delta = p.lut[r + p.R];
        const char* row = pkb + (int64_t)delta * p.pk_sr * QT::SZ;
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
        for (int s = 0; s < C::KSTEPS; ++s) acc = QT::mma(QT::load(row + (16 * s + 8 * g) * QT::SZ), qf[s], acc);
        float* dst = c2pS + wave * (kC2pRows * 32) + (32 * blk + 4 * g) * 32 + li;
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(8 * (v >> 2) + (v & 3)) * 32] = FP8 ? acc[v] * c2p_mul : acc[v];
      }
    }
    if (pqb) {
      // P[r - r_lo, j] for the 191 relative positions of the whole 128 x 64 tile; 12 MFMA blocks
      // (6 row blocks x 2 key blocks) shared by the 4 waves.
      const int r_lo = m0 - (j0 + FDB_BN - 1);
#pragma unroll 1
      for (int n = 0; n < 3; ++n) {
        const int task = wave * 3 + n, wblk = task >> 1, jblk = task & 1;
        int r = r_lo + 32 * wblk + li;
        r = max(-p.R, min(p.R, r));
        const int delta = p.lut[r + p.R];
        const char* row = pqb + (int64_t)delta * p.pq_sr * QT::SZ;
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
        for (int s = 0; s < C::KSTEPS; ++s) {
          qfrag kf = QT::load(Ks + (jblk * 32 + li) * C::K_RS + (16 * s + 8 * g) * QT::SZ);
          acc = QT::mma(QT::load(row + (16 * s + 8 * g) * QT::SZ), kf, acc);
        }
        float* dst = p2cS + (32 * wblk + 4 * g) * kP2cStride + jblk * 32 + li;
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(8 * (v >> 2) + (v & 3)) * kP2cStride] = FP8 ? acc[v] * p2c_mul : acc[v];
      }
    }
    if (pkb || pqb) {
      __syncthreads();
      // element (j = j0 + jj, i): r - r_lo = li + 63 - jj (wave tile) / wave*32 + li + 63 - jj (workgroup tile)
      const float* cbase = c2pS + wave * (kC2pRows * 32) + (li + 63 - 4 * g) * 32 + li;
      const float* pbase = p2cS + (wave * 32 + li + 63 - 4 * g) * kP2cStride + 4 * g;
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int cj = 32 * jb + 8 * (v >> 2) + (v & 3);  // jj = cj + 4*g
          float add = 0.f;
          if (pkb) add += cbase[-cj * 32];
          if (pqb) add += pbase[-cj * kP2cStride + cj];
          sacc[jb][v] += add;
        }
    }

    // ---- mask, online soft-max (base 2) -------------------------------------------------------
    const bool tail = (j0 + FDB_BN > Lb) || (p.causal && j0 + FDB_BN > iw0);
    float mx = -INFINITY;
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float x = sacc[jb][v] * x_scale;
        if (tail) {
          const int j = j0 + 32 * jb + 8 * (v >> 2) + 4 * g + (v & 3);
          if (j >= Lb || (p.causal && j > i)) x = -INFINITY;
        }
        sacc[jb][v] = x;
        mx = fmaxf(mx, x);
      }
    mx = wave_half_max(mx);
    const float m_new = fmaxf(m_run, mx);
    // a row with no visible key so far keeps m_new = -inf; use 0 as the reference point then
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float rs = 0.f;
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float e = __builtin_amdgcn_exp2f(sacc[jb][v] - m_use);
        sacc[jb][v] = e;
        rs += e;
      }
    l_run = l_run * alpha + rs;
    m_run = m_new;
#pragma unroll
    for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;

    // ---- O^T += V^T P^T -----------------------------------------------------------------------
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      f32x8 pv;
#pragma unroll
      for (int e = 0; e < 8; ++e) pv[e] = sacc[c >> 1][8 * (c & 1) + e];
      const vfrag pf = VT::from_f32(pv);
#pragma unroll
      for (int d = 0; d < C::DBLKS; ++d) {
        const vfrag vf = VtLoad<VT>::get(Vs, C::V_RS, c, d, lane);
        o_acc[d] = VT::mma(vf, pf, o_acc[d]);
      }
    }
  }

  // ---- epilogue ------------------------------------------------------------------------------
  const float l_tot = wave_half_sum(l_run);
  const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
  if (i < Lb) {
    char* orow = ob + (int64_t)i * p.o_st * VT::SZ;
#pragma unroll
    for (int d = 0; d < C::DBLKS; ++d)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int dd = 32 * d + 8 * q4 + 4 * g;
        VT::store4(orow + dd * VT::SZ, o_acc[d][4 * q4] * inv, o_acc[d][4 * q4 + 1] * inv,
                   o_acc[d][4 * q4 + 2] * inv, o_acc[d][4 * q4 + 3] * inv);
      }
    if (p.lse && g == 0) {
      const int64_t tok = p.cu ? (int64_t)tok0 + i : (int64_t)b * p.L + tok0 + i;
      p.lse[tok * p.H + h] = (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
    }
  }
}

template <class QT, class VT, int D, bool FP8>
int launch_one(const FdbKParams& p, int grid_x, hipStream_t stream) {
  using C = Cfg<QT, VT, D>;
  auto kern = fdb_attn_kernel<QT, VT, D, FP8>;
  static_assert(C::LDS_BYTES <= 160 * 1024, "LDS budget");
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3(grid_x, p.H, 1), dim3(kThreads), C::LDS_BYTES, stream, p);
  return (int)hipGetLastError();
}

}  // namespace

int fdb_launch_attn(const FdbKParams& p, int dtype, int head_dim, int grid_x, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
#define FDB_DISPATCH_D(QT, VT, FP8)                                   \
  switch (head_dim) {                                                 \
    case 32: return launch_one<QT, VT, 32, FP8>(p, grid_x, stream);   \
    case 64: return launch_one<QT, VT, 64, FP8>(p, grid_x, stream);   \
    case 128: return launch_one<QT, VT, 128, FP8>(p, grid_x, stream); \
    default: return FDB_ERR_HEAD_DIM;                                 \
  }
  switch (dtype) {
    case FDB_BF16: FDB_DISPATCH_D(Bf16Tr, Bf16Tr, false)
    case FDB_F16: FDB_DISPATCH_D(F16Tr, F16Tr, false)
    case FDB_F32:
      switch (head_dim) {
        case 32: return launch_one<F32Tr, F32Tr, 32, false>(p, grid_x, stream);
        case 64: return launch_one<F32Tr, F32Tr, 64, false>(p, grid_x, stream);
        default: return FDB_ERR_UNSUPPORTED;
      }
    case FDB_FP8_E4M3: FDB_DISPATCH_D(Fp8Tr, Bf16Tr, true)
    default: return FDB_ERR_DTYPE;
  }
#undef FDB_DISPATCH_D
}
