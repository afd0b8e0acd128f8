// Internal interface between the host-side C ABI (fdb_api.cpp) and the device code
// (fdb_attn.hip, fdb_aux.hip).  Not installed; the public contract is include/fdb.h.
#pragma once
#include <stdint.h>

// Query rows per workgroup (4 waves x 32 rows) and keys per main-loop iteration.
#define FDB_BM 128
#define FDB_BN 64

struct FdbKParams {
  const char* q;
  const char* k;
  const char* v;
  const char* pk;  // K_r, NULL when the content->position term is absent
  const char* pq;  // Q_r, NULL when the position->content term is absent
  char* out;
  float* lse;
  const int32_t* cu;   // cu_seqlens or NULL
  const int32_t* wl;   // work-list (varlen only)
  const int32_t* seq_start;  // padded fixed layout: first real token / number of real tokens per row (or NULL)
  const int32_t* seq_len;
  const int16_t* lut;  // delta LUT, index r + R
  const float* qs;     // fp8 dequant scales per head (NULL otherwise)
  const float* ks;
  const float* pks;
  const float* pqs;
  int64_t q_sb, q_st, q_sh;
  int64_t k_sb, k_st, k_sh;
  int64_t v_sb, v_st, v_sh;
  int64_t o_sb, o_st, o_sh;
  int64_t pk_sh, pk_sr;
  int64_t pq_sh, pq_sr;
  int32_t B, H, L, tiles_per_seq;
  int32_t grid_x;   // query tiles in the launch (the grid is grid_x * H workgroups)
  int32_t R;        // LUT radius
  int32_t far_done;  // near launches: the far tiles' partial results (far_parts of them) are to be merged
  int32_t far_parts; // workgroups per query tile of the far-only launch, each with its share of the far tiles and a
                     // partial result of its own (the first in out / lse, the others in workspace slots 0 ..)
  int32_t near_parts; // workgroups per query tile of the near launch; above 1 each leaves the partial result of
                      // its share of the steps in workspace slot far_parts-1 + part, and fdb_launch_merge follows
  int32_t key_parts; // one-kernel mode: workgroups per query tile, each with an equal share of the key tiles and a
                     // partial result of its own in workspace slot `part`; fdb_launch_merge_parts follows (1: no sharing)
  int32_t ws_slots;  // partial results in the workspace: far_parts-1, plus near_parts if that is above 1; key_parts in the one-kernel mode
  char* ws;          // [ws_slots][ws_rows][H][D] elements of v's type (rows normalised over the keys seen), then
  int64_t ws_rows;   // [ws_slots][ws_rows][H] float log-sum-exps (-inf: no key seen); ws_rows = rows of the lse buffer
  int32_t causal;
  int32_t fill_pad; // padded fixed layout, first launch of a call: write the rows of out outside the real tokens (zeros; NaN
                    // for batch rows whose seq_len is negative)
  float scale_log2; // sm_scale * log2(e)
};

// Backward launch (fdb_bwd.hip): fixed layout only.  Position scores and their gradients have q's element type, element
// (b, l, h, delta) at b * bias_sb + l * bias_st + h * bias_sh + delta; lse / delta are fp32 [B*L, H].
struct FdbBwdParams {
  const char* q;
  const char* k;
  const char* v;
  const char* dout;
  char* dq;
  char* dk;
  char* dv;
  const float* lse;
  float* delta;         // sum_d dO * O per row: read, or written by the dQ role when `out` is given
  const char* out;      // the forward's output or NULL
  const char* c2p;      // q_i . K_r[delta] or NULL; element type of q, like the gradient tensors below
  const char* p2c;      // k_j . Q_r[delta] or NULL
  char* d_c2p;          // element type of q; every entry of a real token's row is stored once, rows of padding are not touched
  char* d_p2c;
  const int32_t* seq_start;
  const int32_t* seq_len;
  const int16_t* lut;
  int64_t q_sb, q_st, q_sh;
  int64_t k_sb, k_st, k_sh;
  int64_t v_sb, v_st, v_sh;
  int64_t g_sb, g_st, g_sh;     // dout
  int64_t o_sb, o_st, o_sh;     // out
  int64_t dq_sb, dq_st, dq_sh;
  int64_t dk_sb, dk_st, dk_sh;
  int64_t dv_sb, dv_st, dv_sh;
  int64_t bias_sb, bias_st, bias_sh;
  int32_t B, H, L;
  int32_t S;        // att_span
  int32_t R;        // table radius
  int32_t causal;
  int32_t pairs_per_xcd;  // workgroup ids map to (tile, head, batch row) with whole (batch row, head) pairs per XCD
  int32_t store_chunks;   // score gradients leave the ring in aligned chunks of this many groups of four entries: 8, 4 or 1 (as the table's window leaves room)
  float scale_log2; // sm_scale * log2(e)
  float sm_scale;
};
int fdb_launch_bwd(const FdbBwdParams& p, int dtype, int head_dim, void* stream);

// The chain through the position tables (fdb_chain.hip): contiguous tensors, head_dim 64, 2S = 512.
struct FdbChainParams {
  const char* g;       // [matrices][rows][2S] score gradients
  const char* x;       // the token rows of the other factor (q or k) of matrices [0, split): matrix stride x_sm, row stride x_sr (elements)
  const char* x2;      // ... of matrices [split, matrices), numbered from 0 again; same strides
  const char* pos;     // [matrices][2S][D] the tables
  char* dx;            // in and out: += g . pos; rows laid out like those of x, with strides dx_sm, dx_sr, for matrices [0, split)
  char* dx2;           // ... and for matrices [split, matrices)
  float* parts_out;    // [parts][matrices][2S][D] partial sums of g^T . x
  int64_t rows, x_sm, x_sr, dx_sm, dx_sr;
  int32_t matrices, split, parts, tiles_per_part;
};
int fdb_launch_chain(const FdbChainParams& p, int dtype, void* stream);

// Workspace slot `slot`: its output rows and its log-sum-exps (row_bytes = head_dim * element size).
#if defined(__HIPCC__)
__device__ __forceinline__ char* ws_slot_out(const FdbKParams& p, int slot, int row_bytes) {
  return p.ws + (int64_t)slot * p.ws_rows * p.H * row_bytes;
}
__device__ __forceinline__ float* ws_slot_lse(const FdbKParams& p, int slot, int row_bytes) {
  return (float*)(p.ws + (int64_t)p.ws_slots * p.ws_rows * p.H * row_bytes) + (int64_t)slot * p.ws_rows * p.H;
}
// far partial result `part` >= 1 sits in slot part - 1
__device__ __forceinline__ char* far_part_out(const FdbKParams& p, int part, int row_bytes) {
  return ws_slot_out(p, part - 1, row_bytes);
}
__device__ __forceinline__ float* far_part_lse(const FdbKParams& p, int part, int row_bytes) {
  return ws_slot_lse(p, part - 1, row_bytes);
}
#endif

#if defined(__HIPCC__)
// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per kernel instantiation and device instead of
// once per launch.  `done` is a per-instantiation bit mask over device ordinals (a racing first call
// merely sets the attribute twice).
#include <atomic>
inline hipError_t fdb_set_lds_once(const void* kern, int lds_bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  const uint64_t bit = 1ull << dev;
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}
#endif

// Most workgroups per query tile a far-only launch is split into.
#define FDB_MAX_FAR_PARTS 4

// Launchers return the hipError_t of the launch as int.
// fdb_launch_attn, by mode:
//   FDB_MODE_FUSED      one kernel walks every key tile;
//   FDB_MODE_FAR_ONLY   it skips the near tiles and leaves the far tiles' partial result (normalised
//                       rows in out, their log-sum-exp in lse, -inf where a row has no far tile);
//   FDB_MODE_NEAR_RING  the near tiles only, four waves of 32 rows x 64 keys with the expanded
//                       relative-embedding rows in LDS rings, merged with the far partial when
//                       p.far_done.
// The last two exist for the 16-bit element types with head_dim <= 64 (fdb_near_supported).
enum { FDB_MODE_FUSED = 0, FDB_MODE_FAR_ONLY = 1, FDB_MODE_NEAR_RING = 2 };
int fdb_launch_attn(const FdbKParams& p, int dtype, int head_dim, int grid_x, int mode, void* stream);
bool fdb_near_supported(int dtype, int head_dim);
// fdb_launch_near32: the near tiles in 32-key steps, 66 KB of LDS so that two workgroups share a CU
// (16-bit element types, head_dim 64); merges the far partial like the ring mode.
bool fdb_near32_supported(int dtype, int head_dim);
int fdb_launch_near32(const FdbKParams& p, int dtype, int grid_x, void* stream);
// The same pair of launches for OCP e4m3 q / k / K_r / Q_r with bf16 v (head_dim 64): e4m3 MFMA contractions over
// the whole head_dim for the three score products (fdb_fp8.hip).
bool fdb_fp8_pair_supported(int dtype, int head_dim);
int fdb_launch_far8(const FdbKParams& p, int grid_x, void* stream);
int fdb_launch_near8(const FdbKParams& p, int grid_x, void* stream);
// fdb_launch_merge: after a near launch with near_parts > 1: out / lse from the far partial results (when
// p.far_done) and the near ones (16-bit element types, head_dim 64).
int fdb_launch_merge(const FdbKParams& p, int dtype, void* stream);
// fdb_launch_merge_parts: after a one-kernel launch with key_parts > 1: out (and lse, when given) from the key_parts
// partial results in the workspace (any element type and head_dim).
int fdb_launch_merge_parts(const FdbKParams& p, int dtype, int head_dim, void* stream);
int fdb_launch_worklist(const int32_t* cu, int32_t batch, int32_t* wl, int32_t max_tiles, void* stream);
// one tensor (x1 == NULL) or two of one shape and one set of strides: fill, absmax and quantise in three launches
int fdb_launch_quant(const void* x0, const void* x1, int64_t x_st, int64_t x_sh, void* y0, void* y1, int64_t y_st, int64_t y_sh,
                     float* scale0, float* scale1, uint32_t* absmax_ws, int32_t tokens, int32_t heads, int32_t head_dim,
                     void* stream);
int fdb_launch_dequant(const void* y, int64_t y_st, int64_t y_sh, const float* scale, void* x, int64_t x_st, int64_t x_sh,
                       int32_t tokens, int32_t heads, int32_t head_dim, void* stream);
