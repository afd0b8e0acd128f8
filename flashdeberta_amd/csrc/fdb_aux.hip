// Small helper kernels around the fused attention: the varlen q-tile work-list built on the
// device from cu_seqlens (the reference builds it in a Python loop with one host sync per
// sequence, src/flashdeberta/ops/flash_attention_varlen.py:71-83) and the per-head absmax ->
// OCP e4m3 quantisation of the FP8 Q/K variant.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

namespace {

constexpr int kWlThreads = 256;
constexpr int kWlSortMax = 1024;  // batches up to this size get their tiles ordered by sequence length

// wl[0] = number of tiles, wl[1] = 0, then (sequence, first row) pairs: the tiles of the longest
// sequence first (ties in sequence order), so that a launch starts on the workgroups with the most
// key tiles and ends on the short ones.  Each thread places its sequences by summing the tiles of
// all sequences that come before them in that order (batch^2 / 256 steps per thread, the lengths in
// LDS); larger batches keep the sequence order and a prefix sum.
__global__ __launch_bounds__(kWlThreads) void fdb_worklist_kernel(const int32_t* __restrict__ cu, int32_t batch,
                                                                  int32_t* __restrict__ wl, int32_t max_tiles) {
  __shared__ int32_t part[kWlThreads];
  __shared__ int32_t lens[kWlSortMax];
  const int t = threadIdx.x;
  if (batch <= kWlSortMax) {
    for (int b = t; b < batch; b += kWlThreads) lens[b] = max(cu[b + 1] - cu[b], 0);
    __syncthreads();
    for (int b = t; b < batch; b += kWlThreads) {
      const int len = lens[b];
      int32_t pos = 0, total = 0;
      for (int c = 0; c < batch; ++c) {
        const int lc = lens[c], tiles = (lc + FDB_BM - 1) / FDB_BM;
        total += tiles;
        if (lc > len || (lc == len && c < b)) pos += tiles;
      }
      if (b == 0) {
        wl[0] = min(total, max_tiles);
        wl[1] = 0;
      }
      for (int m0 = 0; m0 < len; m0 += FDB_BM, ++pos)
        if (pos < max_tiles) {
          wl[2 + 2 * pos] = b;
          wl[3 + 2 * pos] = m0;
        }
    }
    return;
  }
  const int per = (batch + kWlThreads - 1) / kWlThreads;
  const int b_lo = min(batch, t * per), b_hi = min(batch, b_lo + per);
  int32_t cnt = 0;
  for (int b = b_lo; b < b_hi; ++b) cnt += (max(cu[b + 1] - cu[b], 0) + FDB_BM - 1) / FDB_BM;
  part[t] = cnt;
  __syncthreads();
  // exclusive scan over 256 partial counts (Hillis-Steele)
  for (int off = 1; off < kWlThreads; off <<= 1) {
    int32_t add = (t >= off) ? part[t - off] : 0;
    __syncthreads();
    part[t] += add;
    __syncthreads();
  }
  int32_t pos = part[t] - cnt;
  if (t == kWlThreads - 1) {
    wl[0] = min(part[t], max_tiles);
    wl[1] = 0;
  }
  for (int b = b_lo; b < b_hi; ++b) {
    const int len = max(cu[b + 1] - cu[b], 0);
    for (int m0 = 0; m0 < len; m0 += FDB_BM, ++pos)
      if (pos < max_tiles) {
        wl[2 + 2 * pos] = b;
        wl[3 + 2 * pos] = m0;
      }
  }
}

__global__ void fdb_fill_u32(uint32_t* p, int n, uint32_t v) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// grid (token blocks, heads); each thread owns 8 consecutive d of one token.  One atomic per
// workgroup: all of a head's atomics hit one address and are served one after the other (one per wave
// from 1024 workgroups per head took 560 us for 50 MB), so the launch also keeps the workgroups few.
// One or two tensors of one shape and one set of strides per launch (blockIdx.z picks the tensor; its absmax words
// follow the first tensor's).
struct QuantPair {
  const uint16_t* x[2];
  uint8_t* y[2];
  float* scale[2];
};

template <int D>
__global__ __launch_bounds__(256) void fdb_absmax_kernel(const QuantPair pr, int64_t st, int64_t sh,
                                                         uint32_t* __restrict__ absmax_all, int32_t tokens) {
  constexpr int CPT = D / 8;  // 16-byte chunks per token row
  const int h = blockIdx.y;
  const uint16_t* __restrict__ x = pr.x[blockIdx.z];
  uint32_t* __restrict__ absmax = absmax_all + blockIdx.z * gridDim.y;
  float m = 0.f;
  for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < (int64_t)tokens * CPT;
       c += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = c / CPT;
    const int cc = (int)(c % CPT);
    const uint4 raw = *(const uint4*)(x + t * st + h * sh + cc * 8);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      m = fmaxf(m, fabsf(bf16_bits_to_f32((uint16_t)(w[e] & 0xffffu))));
      m = fmaxf(m, fabsf(bf16_bits_to_f32((uint16_t)(w[e] >> 16))));
    }
  }
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  __shared__ float wave_max[4];
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    atomicMax(absmax + h, __builtin_bit_cast(uint32_t, m));  // m >= 0: bit order = value order
  }
}

template <int D>
__global__ __launch_bounds__(256) void fdb_quant_kernel(const QuantPair pr, int64_t st, int64_t sh, int64_t yst, int64_t ysh,
                                                        const uint32_t* __restrict__ absmax_all, int32_t tokens) {
  constexpr int CPT = D / 8;
  const int h = blockIdx.y;
  const uint16_t* __restrict__ x = pr.x[blockIdx.z];
  uint8_t* __restrict__ y = pr.y[blockIdx.z];
  float* __restrict__ scale = pr.scale[blockIdx.z];
  const uint32_t* __restrict__ absmax = absmax_all + blockIdx.z * gridDim.y;
  const float amax = fmaxf(__builtin_bit_cast(float, absmax[h]), 1e-12f);
  const float sc = amax / 448.0f;
  if (blockIdx.x == 0 && threadIdx.x == 0) scale[h] = sc;
  for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < (int64_t)tokens * CPT;
       c += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = c / CPT;
    const int cc = (int)(c % CPT);
    const uint4 raw = *(const uint4*)(x + t * st + h * sh + cc * 8);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    float f[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f[2 * e] = fminf(fmaxf(bf16_bits_to_f32((uint16_t)(w[e] & 0xffffu)) / sc, -448.f), 448.f);
      f[2 * e + 1] = fminf(fmaxf(bf16_bits_to_f32((uint16_t)(w[e] >> 16)) / sc, -448.f), 448.f);
    }
    uint32_t outw[2];
    // two e4m3 bytes per conversion: low half of the word first, then the high half
    outw[0] = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
    outw[0] = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], outw[0], true);
    outw[1] = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
    outw[1] = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], outw[1], true);
    *(uint2*)(y + t * yst + h * ysh + cc * 8) = uint2{outw[0], outw[1]};
  }
}

// The inverse map, to bf16: x = bf16_rne(e4m3(y) * scale[h]).  Eight elements per thread.
template <int D>
__global__ __launch_bounds__(256) void fdb_dequant_kernel(const uint8_t* __restrict__ y, int64_t yst, int64_t ysh,
                                                          const float* __restrict__ scale, uint16_t* __restrict__ x,
                                                          int64_t st, int64_t sh, int32_t tokens) {
  constexpr int CPT = D / 8;
  const int h = blockIdx.y;
  const float sc = scale[h];
  for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < (int64_t)tokens * CPT;
       c += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = c / CPT;
    const int cc = (int)(c % CPT);
    const uint2 raw = *(const uint2*)(y + t * yst + h * ysh + cc * 8);
    const uint32_t w[2] = {raw.x, raw.y};
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[e], false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[e], true);
      typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
      typedef float f2 __attribute__((ext_vector_type(2)));
      o[2 * e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{lo[0] * sc, lo[1] * sc}, bf2));
      o[2 * e + 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{hi[0] * sc, hi[1] * sc}, bf2));
    }
    *(uint4*)(x + t * st + h * sh + cc * 8) = uint4{o[0], o[1], o[2], o[3]};
  }
}

}  // namespace

int fdb_launch_dequant(const void* y, int64_t y_st, int64_t y_sh, const float* scale, void* x, int64_t x_st, int64_t x_sh,
                       int32_t tokens, int32_t heads, int32_t head_dim, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const int64_t chunks = (int64_t)tokens * head_dim / 8;
  int gx = (int)((chunks + 255) / 256);
  if (gx > 2048) gx = 2048;
  if (gx < 1) gx = 1;
#define FDB_DQ(DD)                                                                                              \
  hipLaunchKernelGGL(fdb_dequant_kernel<DD>, dim3(gx, heads), dim3(256), 0, stream, (const uint8_t*)y, y_st,    \
                     y_sh, scale, (uint16_t*)x, x_st, x_sh, tokens);
  switch (head_dim) {
    case 32: FDB_DQ(32) break;
    case 64: FDB_DQ(64) break;
    case 128: FDB_DQ(128) break;
    default: return -3;
  }
#undef FDB_DQ
  return (int)hipGetLastError();
}

int fdb_launch_worklist(const int32_t* cu, int32_t batch, int32_t* wl, int32_t max_tiles, void* stream) {
  hipLaunchKernelGGL(fdb_worklist_kernel, dim3(1), dim3(kWlThreads), 0, (hipStream_t)stream, cu, batch, wl, max_tiles);
  return (int)hipGetLastError();
}

// ---- merge of partial results -------------------------------------------------------------------------
// After a near launch whose workgroups each took a share of a query tile's steps: every partial result is
// a set of rows normalised over the keys it saw plus their log-sum-exp (-inf: none seen).  The far ones
// (when p.far_done: the first in out / lse, the others in workspace slots 0 .. far_parts-2) and the near
// ones (slots far_parts-1 ..) are combined with weights exp(lse_s - max) into out and lse.  One thread
// per eight elements of a (token, head) row; padded rows of a fixed-layout batch are left alone.
namespace {

template <class VT>
__global__ __launch_bounds__(256) void fdb_merge_kernel(const FdbKParams p) {
  constexpr int D = 64, CPR = D / 8, RB = D * 2;
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= p.ws_rows * p.H * CPR) return;
  const int cc = (int)(c % CPR);
  const int64_t row = c / CPR;  // tok * H + h
  const int h = (int)(row % p.H);
  const int64_t tok = row / p.H;
  char* dst;
  if (p.cu) {
    dst = p.out + (tok * p.o_st + (int64_t)h * p.o_sh) * 2;
  } else {
    const int b = (int)(tok / p.L), l = (int)(tok % p.L);
    const int t0 = p.seq_start ? min(max(p.seq_start[b], 0), p.L) : 0;
    const int len = p.seq_len ? min(max(p.seq_len[b], 0), p.L - t0) : p.L;
    if (l < t0 || l >= t0 + len) return;
    dst = p.out + ((int64_t)b * p.o_sb + (int64_t)l * p.o_st + (int64_t)h * p.o_sh) * 2;
  }
  dst += cc * 16;
  constexpr int kMax = 2 * FDB_MAX_FAR_PARTS;
  const int n_far = p.far_done ? p.far_parts : 0, n = n_far + p.near_parts;
  float w[kMax], m = -INFINITY;
  const char* src[kMax];
#pragma unroll
  for (int s = 0; s < kMax; ++s) {
    w[s] = -INFINITY;
    src[s] = dst;
    if (s < n) {
      // source s: far part s (s < n_far), else near part s - n_far
      const int slot = s < n_far ? s - 1 : p.far_parts - 1 + (s - n_far);
      const float* lp = slot < 0 ? p.lse : ws_slot_lse(p, slot, RB);
      w[s] = lp[row] * 1.4426950408889634f;
      if (slot >= 0) src[s] = ws_slot_out(p, slot, RB) + row * RB + cc * 16;
      m = fmaxf(m, w[s]);
    }
  }
  float denom = 0.f;
#pragma unroll
  for (int s = 0; s < kMax; ++s) {
    w[s] = (s < n && w[s] != -INFINITY) ? __builtin_amdgcn_exp2f(w[s] - m) : 0.f;
    denom += w[s];
  }
  const float inv = denom > 0.f ? 1.f / denom : 0.f;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < kMax; ++s)
    if (s < n && w[s] > 0.f) {
      const f32x4 lo = VT::load4(src[s]);
      const f32x4 hi = VT::load4(src[s] + 8);
      const float f = w[s] * inv;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[e] = __builtin_fmaf(lo[e], f, acc[e]);
        acc[4 + e] = __builtin_fmaf(hi[e], f, acc[4 + e]);
      }
    }
  VT::store4(dst, acc[0], acc[1], acc[2], acc[3]);
  VT::store4(dst + 8, acc[4], acc[5], acc[6], acc[7]);
  if (cc == 0) p.lse[row] = denom > 0.f ? (m + __builtin_amdgcn_logf(denom)) * 0.6931471805599453f : -INFINITY;
}

}  // namespace

// The same for the one-kernel mode: p.key_parts partial results, all in the workspace, any element type and head_dim;
// one thread per four elements.
template <class VT, int D>
__global__ __launch_bounds__(256) void fdb_merge_parts_kernel(const FdbKParams p) {
  constexpr int CPR = D / 4, RB = D * VT::SZ;
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= p.ws_rows * p.H * CPR) return;
  const int cc = (int)(c % CPR);
  const int64_t row = c / CPR;  // tok * H + h
  const int h = (int)(row % p.H);
  const int64_t tok = row / p.H;
  char* dst;
  if (p.cu) {
    dst = p.out + (tok * p.o_st + (int64_t)h * p.o_sh) * VT::SZ;
  } else {
    const int b = (int)(tok / p.L), l = (int)(tok % p.L);
    const int t0 = p.seq_start ? min(max(p.seq_start[b], 0), p.L) : 0;
    const int len = p.seq_len ? min(max(p.seq_len[b], 0), p.L - t0) : p.L;
    if (l < t0 || l >= t0 + len) return;  // rows outside the real tokens were written by the attention launch
    dst = p.out + ((int64_t)b * p.o_sb + (int64_t)l * p.o_st + (int64_t)h * p.o_sh) * VT::SZ;
  }
  dst += cc * 4 * VT::SZ;
  float w[FDB_MAX_FAR_PARTS], m = -INFINITY;
#pragma unroll
  for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s) {
    w[s] = s < p.key_parts ? ws_slot_lse(p, s, RB)[row] * 1.4426950408889634f : -INFINITY;
    m = fmaxf(m, w[s]);
  }
  float denom = 0.f;
#pragma unroll
  for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s) {
    w[s] = w[s] != -INFINITY ? __builtin_amdgcn_exp2f(w[s] - m) : 0.f;
    denom += w[s];
  }
  const float inv = denom > 0.f ? 1.f / denom : 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < FDB_MAX_FAR_PARTS; ++s)
    if (s < p.key_parts && w[s] > 0.f) {
      const f32x4 x = VT::load4(ws_slot_out(p, s, RB) + row * RB + cc * 4 * VT::SZ);
      const float f = w[s] * inv;
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = __builtin_fmaf(x[e], f, acc[e]);
    }
  VT::store4(dst, acc[0], acc[1], acc[2], acc[3]);
  if (cc == 0 && p.lse) p.lse[row] = denom > 0.f ? (m + __builtin_amdgcn_logf(denom)) * 0.6931471805599453f : -INFINITY;
}

template <class VT>
int launch_merge_parts_d(const FdbKParams& p, int head_dim, hipStream_t stream) {
  const int64_t threads = p.ws_rows * p.H * (head_dim / 4);
  const unsigned blocks = (unsigned)((threads + 255) / 256);
  switch (head_dim) {
    case 32: hipLaunchKernelGGL((fdb_merge_parts_kernel<VT, 32>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 64: hipLaunchKernelGGL((fdb_merge_parts_kernel<VT, 64>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 128: hipLaunchKernelGGL((fdb_merge_parts_kernel<VT, 128>), dim3(blocks), dim3(256), 0, stream, p); break;
    default: return FDB_ERR_HEAD_DIM;
  }
  return (int)hipGetLastError();
}

int fdb_launch_merge_parts(const FdbKParams& p, int dtype, int head_dim, void* stream) {
  if (dtype == FDB_F32) return launch_merge_parts_d<fdb::F32Tr>(p, head_dim, (hipStream_t)stream);
  if (dtype == FDB_F16) return launch_merge_parts_d<fdb::F16Tr>(p, head_dim, (hipStream_t)stream);
  if (dtype == FDB_BF16 || dtype == FDB_FP8_E4M3) return launch_merge_parts_d<fdb::Bf16Tr>(p, head_dim, (hipStream_t)stream);  // v's type
  return FDB_ERR_DTYPE;
}

int fdb_launch_merge(const FdbKParams& p, int dtype, void* stream) {
  const int64_t chunks = p.ws_rows * p.H * 8;
  const unsigned blocks = (unsigned)((chunks + 255) / 256);
  if (dtype == FDB_BF16)
    hipLaunchKernelGGL(fdb_merge_kernel<fdb::Bf16Tr>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, p);
  else if (dtype == FDB_F16)
    hipLaunchKernelGGL(fdb_merge_kernel<fdb::F16Tr>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, p);
  else
    return FDB_ERR_UNSUPPORTED;
  return (int)hipGetLastError();
}

int fdb_launch_quant(const void* x0, const void* x1, int64_t x_st, int64_t x_sh, void* y0, void* y1, int64_t y_st, int64_t y_sh,
                     float* scale0, float* scale1, uint32_t* absmax_ws, int32_t tokens, int32_t heads, int32_t head_dim,
                     void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const unsigned n = x1 ? 2u : 1u;
  QuantPair pr;
  pr.x[0] = (const uint16_t*)x0; pr.x[1] = (const uint16_t*)x1;
  pr.y[0] = (uint8_t*)y0; pr.y[1] = (uint8_t*)y1;
  pr.scale[0] = scale0; pr.scale[1] = scale1;
  hipLaunchKernelGGL(fdb_fill_u32, dim3((n * heads + 255) / 256), dim3(256), 0, stream, absmax_ws, (int)(n * heads), 0u);
  const int64_t chunks = (int64_t)tokens * head_dim / 8;
  int gx = (int)((chunks + 255) / 256);
  if (gx > 1024) gx = 1024;
  if (gx < 1) gx = 1;
  int gx_max = 2048 / heads > 1 ? 2048 / heads : 1;  // about 2048 workgroups, i.e. atomics, per tensor
  if (gx_max > gx) gx_max = gx;
#define FDB_Q(DD)                                                                                                    \
  hipLaunchKernelGGL(fdb_absmax_kernel<DD>, dim3(gx_max, heads, n), dim3(256), 0, stream, pr, x_st, x_sh, absmax_ws, \
                     tokens);                                                                                        \
  hipLaunchKernelGGL(fdb_quant_kernel<DD>, dim3(gx, heads, n), dim3(256), 0, stream, pr, x_st, x_sh, y_st, y_sh,     \
                     absmax_ws, tokens);
  switch (head_dim) {
    case 32: FDB_Q(32) break;
    case 64: FDB_Q(64) break;
    case 128: FDB_Q(128) break;
    default: return -3;
  }
#undef FDB_Q
  return (int)hipGetLastError();
}
