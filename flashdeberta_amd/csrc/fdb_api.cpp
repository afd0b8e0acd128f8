// Host side of the C ABI declared in include/fdb.h: argument validation, the integer delta
// table, and dispatch to the device launchers.  No device memory is allocated here.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <atomic>

#include <hip/hip_runtime.h>

#include "../../include/fdb.h"
#include "fdb_kernels.h"

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int qk_elem_size(int dtype) {
  switch (dtype) {
    case FDB_F32: return 4;
    case FDB_BF16:
    case FDB_F16: return 2;
    case FDB_FP8_E4M3: return 1;
    default: return 0;
  }
}
int v_elem_size(int dtype) { return dtype == FDB_F32 ? 4 : 2; }

// DeBERTa's signed log bucket (transformers modeling_deberta_v2.py:56-69), evaluated in fp32 in
// the same operation order as the eager code: ceil(log(a/mid) / log((max-1)/mid) * (mid-1)) + mid.
int32_t log_bucket(int32_t r, int32_t bucket_size, int32_t max_position) {
  const int32_t mid = bucket_size / 2;
  const int32_t a = r < 0 ? -r : r;
  if (a <= mid) return r;  // |r| < mid is mapped to mid-1 <= mid, |r| == mid stays: both take the identity branch
  const float num = logf((float)a / (float)mid);
  const float den = logf((float)(max_position - 1) / (float)mid);
  const float pos = ceilf(num / den * (float)(mid - 1)) + (float)mid;
  const int32_t bkt = (int32_t)pos;
  return r < 0 ? -bkt : bkt;
}

int32_t delta_of(int32_t r, int32_t position_buckets, int32_t max_position) {
  int32_t span, rel;
  if (position_buckets > 0) {
    span = position_buckets;
    rel = log_bucket(r, position_buckets, max_position);
  } else {
    span = max_position;
    rel = r;
  }
  int64_t d = (int64_t)rel + span;
  if (d < 0) d = 0;
  if (d > 2 * (int64_t)span - 1) d = 2 * (int64_t)span - 1;
  return (int32_t)d;
}

bool lut_config_ok(int32_t position_buckets, int32_t max_position) {
  if (max_position < 1) return false;
  if (position_buckets > 0) {
    const int32_t mid = position_buckets / 2;
    if (position_buckets > 16383) return false;
    if (mid < 2) return false;                 // log zone degenerates (mid-1 == 0)
    if (max_position - 1 <= mid) return false; // log((max-1)/mid) <= 0: eager divides by it
  } else if (max_position > 16383) {
    return false;
  }
  return true;
}

constexpr int32_t kRadiusCap = 1 << 22;

static_assert(FDB_MAX_FAR_SPLITS == FDB_MAX_FAR_PARTS, "public and internal limit of the far splits");

// Compute units of the current device (256 if it cannot be asked).
int cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

int64_t query_tiles(const fdb_attn_args* a) {
  return a->cu_seqlens ? fdb_worklist_max_tiles(a->total_tokens, a->batch)
                       : (int64_t)a->batch * ((a->max_seqlen + FDB_BM - 1) / FDB_BM);
}

// The far / near pair of launches exists for the 16-bit types at head_dim 32 / 64 and for e4m3 operands at head_dim 64;
// its near launch walks 32-key steps (and can share them among workgroups) at head_dim 64.
bool pair_supported(int dtype, int head_dim) { return fdb_near_supported(dtype, head_dim) || fdb_fp8_pair_supported(dtype, head_dim); }
bool steps32_supported(int dtype, int head_dim) { return fdb_near32_supported(dtype, head_dim) || fdb_fp8_pair_supported(dtype, head_dim); }

// Does the call take the far / near pair of launches with a far launch in it?
// A packed call's max_seqlen is the caller's word; the one bound the library can trust there is the
// token count (no sequence is longer), so an under-estimate cannot make the far keys disappear: a far
// launch that finds no far tile leaves "no far keys" (-inf) for every row and costs a few microseconds.
bool has_far_launch(const fdb_attn_args* a) {
  const int32_t radius = a->lut_radius > 0 ? a->lut_radius : 1;
  const int32_t longest = a->cu_seqlens ? a->total_tokens : a->max_seqlen;
  return (a->pos_key || a->pos_query) && a->lse && pair_supported(a->dtype, a->head_dim) &&
         longest > radius + FDB_BN - 1;
}

// Workgroups per query tile of the far-only launch.  That launch keeps three workgroups on a CU; when
// the query tiles fill at most half of those slots, the far keys of a tile are shared out among as many
// workgroups as still fit in one round, every share keeping at least eight tiles.  (Measured: 384 query
// tiles on 768 slots gain 9 % of the whole call from two shares; shares that need a second round of
// workgroups, e.g. three for 512 query tiles, gain nothing.)
int far_parts_wanted(const fdb_attn_args* a) {
  if (!has_far_launch(a) || !steps32_supported(a->dtype, a->head_dim)) return 1;
  if (a->far_splits > 0) return a->far_splits;
  // A packed batch has its lengths on the device: the host goes by the mean length (the kernel divides each query
  // tile's own far tiles among the shares, whatever they are), and only shares when that mean leaves far tiles at all.
  int32_t typical = a->max_seqlen;
  if (a->cu_seqlens) {
    typical = a->total_tokens / a->batch;
    if (typical < 2 * a->lut_radius + FDB_BM) return 1;
  }
  const int64_t wgs = query_tiles(a) * a->heads, slots = 3 * (int64_t)cu_count();
  if (wgs >= slots) return 1;
  const int n64 = (typical + FDB_BN - 1) / FDB_BN;
  const int near64 = (FDB_BM + 2 * a->lut_radius + 3 * (FDB_BN - 1)) / FDB_BN;  // of a query tile in mid-sequence
  const int most = (n64 - near64) / 8 < FDB_MAX_FAR_PARTS ? (n64 - near64) / 8 : FDB_MAX_FAR_PARTS;
  const int64_t fit = slots / wgs;
  const int n = (int)(fit < most ? fit : most);
  return n > 1 ? n : 1;
}

// The same for the near launch, which keeps two workgroups on a CU.  Every share repeats the prologue
// (five batches of table rows) and a merge kernel follows, so a share keeps at least sixteen 32-key
// steps, or eight when all shares together fill at most half of the slots.  (Measured, 12 heads: one
// sequence of 1024: 0.056 -> 0.040 ms; one of 512: 0.025 -> 0.022; four of 512 in shares of eight
// steps would go from 0.025 to 0.028.)  Two shares also pay when they need a partial second round, as
// long as the query tiles alone fill at most 70 % of the slots (288 to 352 tiles: 5 to 8 % of the call;
// 384: between +2 and -4 %).
int near_parts_wanted(const fdb_attn_args* a) {
  if (!(a->pos_key || a->pos_query) || !a->lse || !steps32_supported(a->dtype, a->head_dim)) return 1;
  if (a->near_splits > 0) return a->near_splits;
  // A packed batch has its lengths on the device: the host goes by the mean length and by the most query tiles the
  // token count allows (the kernel divides each query tile's own steps among the shares, whatever they are).
  const int32_t typical = a->cu_seqlens ? a->total_tokens / a->batch : a->max_seqlen;
  const int64_t wgs = query_tiles(a) * a->heads, slots = 2 * (int64_t)cu_count();
  const int steps_all = (typical + 31) / 32, steps_near = (FDB_BM + 2 * a->lut_radius + 3 * (FDB_BN - 1)) / 32;
  const int steps = steps_all < steps_near ? steps_all : steps_near;
  int best = 1;
  // (packed batches only share when all shares fit in one round: three sequences of 1000 lose 10 % to two shares)
  for (int n = 2; n <= FDB_MAX_FAR_PARTS && (wgs * n <= slots || (n == 2 && !a->cu_seqlens && wgs * 10 <= slots * 7)); ++n) {
    const int per = steps / n;
    if (per >= 16 || (per >= 8 && wgs * n <= slots / 2)) best = n;
  }
  return best;
}

// Does the call take the far / near pair of launches (otherwise one kernel walks every key tile)?
bool takes_pair(const fdb_attn_args* a) {
  return (a->pos_key || a->pos_query) && a->lse && pair_supported(a->dtype, a->head_dim);
}

// One-kernel mode: workgroups per query tile.  When the query tiles leave most of the GPU idle (one workgroup per CU
// is what the larger instantiations of that kernel reach), the key tiles of a query tile are shared out among up to
// FDB_MAX_FAR_PARTS workgroups, each keeping at least two; a merge launch follows.  far_splits overrides it.
int key_parts_wanted(const fdb_attn_args* a) {
  if (takes_pair(a)) return 1;
  const int32_t typical = a->cu_seqlens ? a->total_tokens / a->batch : a->max_seqlen;
  const int n64 = (typical + FDB_BN - 1) / FDB_BN;
  // a causal query tile's keys end at its own rows: a share could hold no visible key for some of them, a case the
  // tiles' soft-max does not meet otherwise (a row's first tile always shows it a key) and is not written for
  if (a->causal) return 1;
  if (a->far_splits > 0) return a->far_splits;
  const int64_t wgs = query_tiles(a) * a->heads, slots = cu_count();
  int n = (int)(slots / wgs);
  if (n > FDB_MAX_FAR_PARTS) n = FDB_MAX_FAR_PARTS;
  while (n > 1 && n64 / n < 2) --n;
  return n > 1 ? n : 1;
}

int64_t lse_rows(const fdb_attn_args* a) {
  return a->cu_seqlens ? (int64_t)a->total_tokens : (int64_t)a->batch * a->max_seqlen;
}

int64_t far_part_bytes(const fdb_attn_args* a) {
  return lse_rows(a) * a->heads * ((int64_t)a->head_dim * v_elem_size(a->dtype) + 4);
}

}  // namespace

// ---- the entry point that allocates nothing ---------------------------------------------------------
// Its scratch lives in the library's own device image: one copy per GPU, held until the process ends.
// The name below is a host-side handle only; the device address is asked for once per device
// (hipGetSymbolAddress) and that pointer is what kernels receive.
static __device__ __align__(256) unsigned char fdb_noalloc_scratch[FDB_NOALLOC_SCRATCH_BYTES];

namespace {

std::atomic<unsigned char*> g_scratch_ptr[64];

// Device address of this GPU's copy of the scratch array (nullptr + error code on failure).
int scratch_base(unsigned char** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= 64) return FDB_ERR_SCRATCH;
  unsigned char* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void* sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(fdb_noalloc_scratch));
    if (e != hipSuccess) return (int)e;
    if (!sym) return FDB_ERR_SCRATCH;
    p = (unsigned char*)sym;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // a racing first call stores the same address
  }
  *out = p;
  return FDB_OK;
}

int64_t align256(int64_t n) { return (n + 255) & ~(int64_t)255; }

// What fdb_attn_fwd_noalloc validates before it launches: the argument block as fdb_attn_fwd sees it,
// and that the hand-over buffers fit the scratch.
int check_noalloc(const fdb_attn_args* a) {
  if (!a) return FDB_ERR_NULL;
  fdb_attn_args b = *a;
  int32_t dummy_wl = 0;
  if (b.cu_seqlens && !b.worklist) b.worklist = &dummy_wl;  // supplied from the scratch by the call itself
  b.workspace = nullptr;
  b.workspace_bytes = 0;
  const int rc = fdb_attn_check(&b);
  if (rc != FDB_OK) return rc;
  int64_t need = 0;
  if (!b.lse && (b.pos_key || b.pos_query) && pair_supported(b.dtype, b.head_dim)) need += align256(lse_rows(&b) * b.heads * 4);
  if (b.cu_seqlens) need += align256(fdb_worklist_ints(b.total_tokens, b.batch) * 4);
  return need > FDB_NOALLOC_SCRATCH_BYTES ? FDB_ERR_SCRATCH : FDB_OK;
}

}  // namespace

extern "C" {

int fdb_version(void) { return FDB_VERSION; }

size_t fdb_attn_args_size(void) { return sizeof(fdb_attn_args); }

const char* fdb_strerror(int code) {
  switch (code) {
    case FDB_OK: return "ok";
    case FDB_ERR_NULL: return "required pointer is NULL";
    case FDB_ERR_DTYPE: return "unknown dtype";
    case FDB_ERR_HEAD_DIM: return "unsupported head_dim (supported: 32, 64, 128)";
    case FDB_ERR_ALIGN: return "pointer or stride is not 16-byte aligned";
    case FDB_ERR_SHAPE: return "batch/heads/max_seqlen/total_tokens invalid";
    case FDB_ERR_SPAN: return "att_span/lut_radius/delta_lut invalid while a position term is present (backward: or lut_window beyond FDB_BWD_MAX_WINDOW)";
    case FDB_ERR_SCALE: return "fp8 dtype needs q_scale, k_scale and a scale for each position tensor";
    case FDB_ERR_WORKLIST: return "cu_seqlens given without a work-list buffer";
    case FDB_ERR_LUT_ARGS: return "invalid position_buckets/max_position/radius/out for the delta table";
    case FDB_ERR_UNSUPPORTED: return "dtype/head_dim combination not built";
    case FDB_ERR_SCRATCH: return "fdb_attn_fwd_noalloc: the call needs more than FDB_NOALLOC_SCRATCH_BYTES of built-in scratch";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown error";
}

int32_t fdb_tile_rows(void) { return FDB_BM; }

int32_t fdb_worklist_max_tiles(int32_t total_tokens, int32_t batch) {
  if (total_tokens < 0 || batch < 0) return 0;
  // sum_b ceil(L_b / BM) <= floor(T / BM) + batch
  int64_t n = (int64_t)total_tokens / FDB_BM + batch;
  if (n > INT32_MAX) n = INT32_MAX;
  return (int32_t)n;
}

int64_t fdb_worklist_ints(int32_t total_tokens, int32_t batch) {
  return 2 + 2 * (int64_t)fdb_worklist_max_tiles(total_tokens, batch);
}

int fdb_attn_check(const fdb_attn_args* a) {
  if (!a) return FDB_ERR_NULL;
  if (!a->q || !a->k || !a->v || !a->out) return FDB_ERR_NULL;
  const int qsz = qk_elem_size(a->dtype);
  if (qsz == 0) return FDB_ERR_DTYPE;
  const int vsz = v_elem_size(a->dtype);
  if (a->head_dim != 32 && a->head_dim != 64 && a->head_dim != 128) return FDB_ERR_HEAD_DIM;
  if (a->batch < 1 || a->heads < 1 || a->heads > 65535 || a->max_seqlen < 1 || a->total_tokens < 1)
    return FDB_ERR_SHAPE;
  if (a->far_splits < 0 || a->far_splits > FDB_MAX_FAR_SPLITS || a->near_splits < 0 ||
      a->near_splits > FDB_MAX_FAR_SPLITS || a->workspace_bytes < 0)
    return FDB_ERR_SHAPE;
  if (a->workspace && !aligned16(a->workspace)) return FDB_ERR_ALIGN;
  if (!a->cu_seqlens && (int64_t)a->batch * a->max_seqlen != a->total_tokens) return FDB_ERR_SHAPE;
  if (a->cu_seqlens && !a->worklist) return FDB_ERR_WORKLIST;
  const bool has_pos = a->pos_key || a->pos_query;
  if (has_pos && (a->att_span < 1 || a->lut_radius < 1 || !a->delta_lut)) return FDB_ERR_SPAN;
  if (a->dtype == FDB_FP8_E4M3) {
    if (!a->q_scale || !a->k_scale) return FDB_ERR_SCALE;
    if (a->pos_key && !a->pk_scale) return FDB_ERR_SCALE;
    if (a->pos_query && !a->pq_scale) return FDB_ERR_SCALE;
  }
  if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->out)) return FDB_ERR_ALIGN;
  if ((a->pos_key && !aligned16(a->pos_key)) || (a->pos_query && !aligned16(a->pos_query))) return FDB_ERR_ALIGN;
  const int64_t qk_strides[] = {a->q_stride_b, a->q_stride_t, a->q_stride_h, a->k_stride_b, a->k_stride_t,
                                a->k_stride_h, a->pos_key ? a->pk_stride_h : 0, a->pos_key ? a->pk_stride_r : 0,
                                a->pos_query ? a->pq_stride_h : 0, a->pos_query ? a->pq_stride_r : 0};
  for (int64_t s : qk_strides)
    if ((s * qsz) % 16 != 0) return FDB_ERR_ALIGN;
  // the kernels walk K and V with 32-bit row strides (in bytes)
  if (a->k_stride_t < 0 || a->v_stride_t < 0 || a->k_stride_t * qsz > INT32_MAX || a->v_stride_t * vsz > INT32_MAX)
    return FDB_ERR_SHAPE;
  // ... and the rows of K_r / Q_r with 32-bit byte offsets from a head's first row (24-bit row strides)
  const int64_t table_rows = 2 * (int64_t)a->att_span;
  if (a->pos_key && (a->pk_stride_r < 0 || a->pk_stride_r * qsz >= (1 << 24) || table_rows * a->pk_stride_r * qsz > INT32_MAX))
    return FDB_ERR_SHAPE;
  if (a->pos_query && (a->pq_stride_r < 0 || a->pq_stride_r * qsz >= (1 << 24) || table_rows * a->pq_stride_r * qsz > INT32_MAX))
    return FDB_ERR_SHAPE;
  const int64_t v_strides[] = {a->v_stride_b, a->v_stride_t, a->v_stride_h, a->o_stride_b, a->o_stride_t, a->o_stride_h};
  for (int64_t s : v_strides)
    if ((s * vsz) % 16 != 0) return FDB_ERR_ALIGN;
  return FDB_OK;
}

int64_t fdb_attn_workspace_bytes(const fdb_attn_args* a) {
  if (fdb_attn_check(a) != FDB_OK) return 0;
  if (!takes_pair(a)) {
    const int parts = key_parts_wanted(a);
    return parts > 1 ? parts * far_part_bytes(a) : 0;
  }
  const int near = near_parts_wanted(a);
  return (far_parts_wanted(a) - 1 + (near > 1 ? near : 0)) * far_part_bytes(a);
}

}  // extern "C"

namespace {

// launch_mask 0: the whole call; 1 / 2: only the launch over the far / the near keys (fdb_attn_fwd_part)
int attn_fwd_impl(const fdb_attn_args* a, int launch_mask, void* stream) {
  const int rc = fdb_attn_check(a);
  if (rc != FDB_OK) return rc;
  FdbKParams p;
  memset(&p, 0, sizeof(p));
  p.q = (const char*)a->q;
  p.k = (const char*)a->k;
  p.v = (const char*)a->v;
  p.pk = (const char*)a->pos_key;
  p.pq = (const char*)a->pos_query;
  p.out = (char*)a->out;
  p.lse = a->lse;
  p.cu = a->cu_seqlens;
  p.wl = a->worklist;
  p.lut = a->delta_lut;
  p.seq_start = a->cu_seqlens ? nullptr : a->seq_start;
  p.seq_len = a->cu_seqlens ? nullptr : a->seq_len;
  p.qs = a->q_scale; p.ks = a->k_scale; p.pks = a->pk_scale; p.pqs = a->pq_scale;
  p.q_sb = a->q_stride_b; p.q_st = a->q_stride_t; p.q_sh = a->q_stride_h;
  p.k_sb = a->k_stride_b; p.k_st = a->k_stride_t; p.k_sh = a->k_stride_h;
  p.v_sb = a->v_stride_b; p.v_st = a->v_stride_t; p.v_sh = a->v_stride_h;
  p.o_sb = a->o_stride_b; p.o_st = a->o_stride_t; p.o_sh = a->o_stride_h;
  p.pk_sh = a->pk_stride_h; p.pk_sr = a->pk_stride_r;
  p.pq_sh = a->pq_stride_h; p.pq_sr = a->pq_stride_r;
  p.B = a->batch; p.H = a->heads; p.L = a->max_seqlen;
  p.tiles_per_seq = (a->max_seqlen + FDB_BM - 1) / FDB_BM;
  p.R = a->lut_radius > 0 ? a->lut_radius : 1;
  p.causal = a->causal ? 1 : 0;
  p.scale_log2 = a->sm_scale * 1.4426950408889634f;
  // padded fixed layout: the first launch of the call also writes the rows of out outside the real tokens
  p.fill_pad = (!a->cu_seqlens && (a->seq_start || a->seq_len)) ? 1 : 0;
  const int64_t grid_x = query_tiles(a);
  if (grid_x < 1 || grid_x * a->heads > INT32_MAX) return FDB_ERR_SHAPE;
  p.grid_x = (int32_t)grid_x;
  // Split path: the far tiles in a far-only run of the kernel (three workgroups per CU), the near
  // tiles in a second launch, which merges the two.  It needs the log-sum-exp buffer as the
  // hand-over between the two launches.
  if ((a->pos_key || a->pos_query) && a->lse && pair_supported(a->dtype, a->head_dim)) {
    const bool fp8 = fdb_fp8_pair_supported(a->dtype, a->head_dim);
    const bool need_far = has_far_launch(a);  // otherwise no tile of any query tile is far
    // as many workgroups per query tile as wanted and as the workspace holds partial results for
    p.far_parts = need_far ? far_parts_wanted(a) : 1;
    p.near_parts = near_parts_wanted(a);
    const int64_t ws_slots_have = a->workspace ? a->workspace_bytes / far_part_bytes(a) : 0;
    if (p.near_parts > 1 && ws_slots_have < p.far_parts - 1 + p.near_parts) p.near_parts = 1;
    while (p.far_parts > 1 && ws_slots_have < p.far_parts - 1 + (p.near_parts > 1 ? p.near_parts : 0)) --p.far_parts;
    p.ws_slots = p.far_parts - 1 + (p.near_parts > 1 ? p.near_parts : 0);
    p.ws = (char*)a->workspace;
    p.ws_rows = lse_rows(a);
    if (need_far && launch_mask != 2) {
      const int rc_far = fp8 ? fdb_launch_far8(p, (int)grid_x, stream)
                             : fdb_launch_attn(p, a->dtype, a->head_dim, (int)grid_x, FDB_MODE_FAR_ONLY, stream);
      if (rc_far != 0) return rc_far;
      p.fill_pad = 0;
    }
    if (launch_mask == 1) return FDB_OK;
    p.far_done = need_far ? 1 : 0;
    // head_dim 64: the near kernel (32-key steps, two workgroups per CU); head_dim 32: the fused kernel's ring mode
    if (steps32_supported(a->dtype, a->head_dim)) {
      const int rc_near = fp8 ? fdb_launch_near8(p, (int)grid_x, stream) : fdb_launch_near32(p, a->dtype, (int)grid_x, stream);
      if (rc_near != 0 || p.near_parts <= 1) return rc_near;
      return fdb_launch_merge(p, fp8 ? (int)FDB_BF16 : a->dtype, stream);  // partial results have v's element type
    }
    return fdb_launch_attn(p, a->dtype, a->head_dim, (int)grid_x, FDB_MODE_NEAR_RING, stream);
  }
  if (launch_mask != 0) return FDB_ERR_UNSUPPORTED;  // a single kernel has no parts
  // as many shares of the keys as wanted and as the workspace holds partial results for
  p.key_parts = key_parts_wanted(a);
  const int64_t slots_have = a->workspace ? a->workspace_bytes / far_part_bytes(a) : 0;
  if (p.key_parts > slots_have) p.key_parts = slots_have >= 2 ? (int)slots_have : 1;
  if (p.key_parts <= 1) {
    p.key_parts = 1;
    return fdb_launch_attn(p, a->dtype, a->head_dim, (int)grid_x, FDB_MODE_FUSED, stream);
  }
  p.ws_slots = p.key_parts;
  p.ws = (char*)a->workspace;
  p.ws_rows = lse_rows(a);
  const int rc_attn = fdb_launch_attn(p, a->dtype, a->head_dim, (int)grid_x, FDB_MODE_FUSED, stream);
  if (rc_attn != 0) return rc_attn;
  return fdb_launch_merge_parts(p, a->dtype, a->head_dim, stream);
}

}  // namespace

extern "C" {

int fdb_attn_fwd(const fdb_attn_args* a, void* stream) { return attn_fwd_impl(a, 0, stream); }

int fdb_attn_fwd_part(const fdb_attn_args* a, int32_t part, void* stream) {
  if (part != 1 && part != 2) return FDB_ERR_SHAPE;
  return attn_fwd_impl(a, part, stream);
}

int fdb_attn_fwd_noalloc(const fdb_attn_args* a, void* stream) {
  const int rc = check_noalloc(a);
  if (rc != FDB_OK) return rc;
  fdb_attn_args b = *a;
  unsigned char* base = nullptr;
  const int rs = scratch_base(&base);
  if (rs != FDB_OK) return rs;
  // [log-sum-exp hand-over][work-list][partial results], each part 256-byte aligned
  int64_t off = 0;
  const bool has_pos = b.pos_key || b.pos_query;
  if (!b.lse && has_pos && pair_supported(b.dtype, b.head_dim)) {
    b.lse = (float*)(base + off);
    off += align256(lse_rows(&b) * b.heads * 4);
  }
  if (b.cu_seqlens) {
    b.worklist = (int32_t*)(base + off);
    off += align256(fdb_worklist_ints(b.total_tokens, b.batch) * 4);
  }
  if (off > FDB_NOALLOC_SCRATCH_BYTES) return FDB_ERR_SCRATCH;
  // what is left holds as many partial results as fit: the call shares less with a smaller remainder
  b.workspace = base + off;
  b.workspace_bytes = FDB_NOALLOC_SCRATCH_BYTES - off;
  if (b.cu_seqlens) {
    const int rw = fdb_launch_worklist(b.cu_seqlens, b.batch, b.worklist, fdb_worklist_max_tiles(b.total_tokens, b.batch), stream);
    if (rw != 0) return rw;
  }
  return fdb_attn_fwd(&b, stream);
}

size_t fdb_attn_bwd_args_size(void) { return sizeof(fdb_attn_bwd_args); }

int fdb_attn_bwd_chain(const void* d_scores, const void* x, const void* x_second, const void* pos, void* dx, void* dx_second,
                       float* dpos_parts, int32_t matrices, int32_t first_matrices, int64_t rows, int64_t x_stride_matrix,
                       int64_t x_stride_row, int64_t dx_stride_matrix, int64_t dx_stride_row, int32_t att_span, int32_t head_dim,
                       int32_t dtype, int32_t parts, void* stream) {
  if (!d_scores || !x || !pos || !dx || !dpos_parts) return FDB_ERR_NULL;
  if (matrices >= 1 && first_matrices < matrices && (!x_second || !dx_second)) return FDB_ERR_NULL;
  if (dtype != FDB_BF16 && dtype != FDB_F16) return FDB_ERR_DTYPE;
  if (head_dim != 64) return FDB_ERR_HEAD_DIM;
  if (att_span != 256) return FDB_ERR_SPAN;
  if (matrices < 1 || matrices > 65535 || first_matrices < 1 || first_matrices > matrices || rows < 32 || rows % 32 != 0 ||
      parts < 1 || parts > rows / 32 || x_stride_matrix < 0 || x_stride_row < 64 || dx_stride_matrix < 64 || dx_stride_row < 64)
    return FDB_ERR_SHAPE;
  if (!aligned16(d_scores) || !aligned16(x) || (x_second && !aligned16(x_second)) || !aligned16(pos) || !aligned16(dx) ||
      (dx_second && !aligned16(dx_second)) || !aligned16(dpos_parts) || (x_stride_matrix * 2) % 16 != 0 ||
      (x_stride_row * 2) % 16 != 0 || (dx_stride_matrix * 2) % 16 != 0 || (dx_stride_row * 2) % 16 != 0) return FDB_ERR_ALIGN;
  FdbChainParams p;
  memset(&p, 0, sizeof(p));
  p.g = (const char*)d_scores; p.x = (const char*)x; p.x2 = (const char*)x_second; p.pos = (const char*)pos; p.dx = (char*)dx;
  p.dx2 = (char*)dx_second; p.parts_out = dpos_parts;
  p.rows = rows; p.x_sm = x_stride_matrix; p.x_sr = x_stride_row; p.dx_sm = dx_stride_matrix; p.dx_sr = dx_stride_row;
  p.matrices = matrices; p.split = first_matrices; p.parts = parts;
  const int64_t tiles = rows / 32;
  p.tiles_per_part = (int32_t)((tiles + parts - 1) / parts);
  return fdb_launch_chain(p, dtype, stream);
}

int fdb_attn_bwd(const fdb_attn_bwd_args* a, void* stream) {
  if (!a) return FDB_ERR_NULL;
  if (!a->q || !a->k || !a->v || !a->dout || !a->dq || !a->dk || !a->dv || !a->lse || !a->delta) return FDB_ERR_NULL;
  if (a->dtype != FDB_F32 && a->dtype != FDB_BF16 && a->dtype != FDB_F16) return FDB_ERR_DTYPE;
  if (a->head_dim != 32 && a->head_dim != 64 && a->head_dim != 128) return FDB_ERR_HEAD_DIM;
  if (a->batch < 1 || a->heads < 1 || a->heads > 65535 || a->batch > 65535 || a->seqlen < 1) return FDB_ERR_SHAPE;
  const bool has_pos = a->c2p_bias || a->p2c_bias;
  if ((a->c2p_bias && !a->d_c2p_bias) || (a->p2c_bias && !a->d_p2c_bias)) return FDB_ERR_NULL;
  if (has_pos && (a->att_span < 1 || a->lut_radius < 1 || !a->delta_lut)) return FDB_ERR_SPAN;
  // the ring that collects a row's score gradients holds the table rows of one 32-row step plus a partly stored group
  if (has_pos && (a->lut_window < 0 || a->lut_window > FDB_BWD_MAX_WINDOW)) return FDB_ERR_SPAN;
  // the kernels address a sequence's rows of the position-score tensors with 32-bit byte offsets
  if (has_pos && (a->bias_stride_t < 2 * a->att_span || a->bias_stride_b < 0 || a->bias_stride_h < 0 ||
                  (int64_t)a->seqlen * a->bias_stride_t * qk_elem_size(a->dtype) > 0xffffffffll)) return FDB_ERR_SHAPE;
  // score gradients leave in aligned groups of four entries
  const uintptr_t group_bytes = 4u * (uintptr_t)qk_elem_size(a->dtype);  // one store: four entries
  if (has_pos && ((a->att_span & 1) || (a->bias_stride_b & 3) || (a->bias_stride_t & 3) || (a->bias_stride_h & 3) ||
                  reinterpret_cast<uintptr_t>(a->d_c2p_bias) % group_bytes || reinterpret_cast<uintptr_t>(a->d_p2c_bias) % group_bytes ||
                  // ... and the scores arrive in aligned 32-bit words (two 16-bit entries)
                  reinterpret_cast<uintptr_t>(a->c2p_bias) % 4 || reinterpret_cast<uintptr_t>(a->p2c_bias) % 4))
    return FDB_ERR_ALIGN;
  const int sz = qk_elem_size(a->dtype);
  const void* ptrs[] = {a->q, a->k, a->v, a->dout, a->dq, a->dk, a->dv, a->out};
  for (const void* ptr : ptrs)
    if (!aligned16(ptr)) return FDB_ERR_ALIGN;
  const int64_t strides[] = {a->q_stride_b, a->q_stride_t, a->q_stride_h, a->k_stride_b, a->k_stride_t, a->k_stride_h,
                             a->v_stride_b, a->v_stride_t, a->v_stride_h, a->do_stride_b, a->do_stride_t, a->do_stride_h,
                             a->dq_stride_b, a->dq_stride_t, a->dq_stride_h, a->dk_stride_b, a->dk_stride_t, a->dk_stride_h,
                             a->dv_stride_b, a->dv_stride_t, a->dv_stride_h,
                             a->out ? a->out_stride_b : 0, a->out ? a->out_stride_t : 0, a->out ? a->out_stride_h : 0};
  for (int64_t st : strides)
    if ((st * sz) % 16 != 0) return FDB_ERR_ALIGN;
  FdbBwdParams p;
  memset(&p, 0, sizeof(p));
  p.q = (const char*)a->q; p.k = (const char*)a->k; p.v = (const char*)a->v; p.dout = (const char*)a->dout;
  p.dq = (char*)a->dq; p.dk = (char*)a->dk; p.dv = (char*)a->dv;
  p.lse = a->lse; p.delta = a->delta; p.out = (const char*)a->out;
  p.o_sb = a->out_stride_b; p.o_st = a->out_stride_t; p.o_sh = a->out_stride_h;
  p.c2p = (const char*)a->c2p_bias; p.p2c = (const char*)a->p2c_bias; p.d_c2p = (char*)a->d_c2p_bias; p.d_p2c = (char*)a->d_p2c_bias;
  p.bias_sb = a->bias_stride_b; p.bias_st = a->bias_stride_t; p.bias_sh = a->bias_stride_h;
  p.seq_start = a->seq_start; p.seq_len = a->seq_len; p.lut = a->delta_lut;
  p.q_sb = a->q_stride_b; p.q_st = a->q_stride_t; p.q_sh = a->q_stride_h;
  p.k_sb = a->k_stride_b; p.k_st = a->k_stride_t; p.k_sh = a->k_stride_h;
  p.v_sb = a->v_stride_b; p.v_st = a->v_stride_t; p.v_sh = a->v_stride_h;
  p.g_sb = a->do_stride_b; p.g_st = a->do_stride_t; p.g_sh = a->do_stride_h;
  p.dq_sb = a->dq_stride_b; p.dq_st = a->dq_stride_t; p.dq_sh = a->dq_stride_h;
  p.dk_sb = a->dk_stride_b; p.dk_st = a->dk_stride_t; p.dk_sh = a->dk_stride_h;
  p.dv_sb = a->dv_stride_b; p.dv_st = a->dv_stride_t; p.dv_sh = a->dv_stride_h;
  p.B = a->batch; p.H = a->heads; p.L = a->seqlen;
  p.S = has_pos ? a->att_span : 0;
  p.R = has_pos ? a->lut_radius : 1;
  p.causal = a->causal ? 1 : 0;
  p.sm_scale = a->sm_scale;
  p.scale_log2 = a->sm_scale * 1.4426950408889634f;
  // One workgroup per 128 rows, head and batch row, in a one-dimensional grid.  With at least eight (batch row, head)
  // pairs and more than two rounds of workgroups (two per CU), whole pairs go to one XCD each, eight at a time: the tiles of a
  // pair then share the loop-side rows through that XCD's L2 (B = 8, L = 4096: 3.30 -> 3.12 ms for the two launches,
  // causal 2.83 -> 2.03); a launch of at most two rounds is a little faster with the tiles of a pair spread out.
  const int64_t tiles = ((int64_t)a->seqlen + FDB_BM - 1) / FDB_BM, pairs = (int64_t)a->batch * a->heads;
  if (tiles * pairs > INT32_MAX) return FDB_ERR_SHAPE;
  p.pairs_per_xcd = (pairs >= 8 && tiles * pairs > 4 * (int64_t)cu_count()) ? 1 : 0;
  // the ring holds a step's window, a partly stored group and, with chunked stores, up to seven or three more complete groups
  p.store_chunks = !has_pos ? 1 : a->lut_window + 4 + 28 <= FDB_BWD_RING ? 8 : a->lut_window + 4 + 12 <= FDB_BWD_RING ? 4 : 1;
  return fdb_launch_bwd(p, a->dtype, a->head_dim, stream);
}

int fdb_build_worklist(const int32_t* cu_seqlens, int32_t batch, int32_t total_tokens, int32_t* worklist,
                       void* stream) {
  if (!cu_seqlens || !worklist) return FDB_ERR_NULL;
  if (batch < 1 || total_tokens < 0) return FDB_ERR_SHAPE;
  return fdb_launch_worklist(cu_seqlens, batch, worklist, fdb_worklist_max_tiles(total_tokens, batch), stream);
}

int32_t fdb_delta_lut_radius(int32_t position_buckets, int32_t max_position) {
  if (!lut_config_ok(position_buckets, max_position)) return FDB_ERR_LUT_ARGS;
  const int32_t span = position_buckets > 0 ? position_buckets : max_position;
  // delta is non-decreasing in r; find where each side reaches its clamp value
  int32_t r = 1;
  while (r < kRadiusCap && !(delta_of(r, position_buckets, max_position) == 2 * span - 1 &&
                             delta_of(-r, position_buckets, max_position) == 0))
    ++r;
  return r;
}

int32_t fdb_delta_lut_window(int32_t position_buckets, int32_t max_position) {
  const int32_t radius = fdb_delta_lut_radius(position_buckets, max_position);
  if (radius < 1) return FDB_ERR_LUT_ARGS;
  // delta is constant beyond +-radius, so every 32-row window that matters starts in [-radius - 31, radius]
  int32_t worst = 0;
  for (int32_t r = -radius - 31; r <= radius; ++r) {
    const int32_t w = delta_of(r + 31, position_buckets, max_position) - delta_of(r, position_buckets, max_position);
    if (w > worst) worst = w;
  }
  return worst;
}

int fdb_delta_lut(int32_t position_buckets, int32_t max_position, int32_t radius, int16_t* out) {
  if (!out || radius < 1 || radius > kRadiusCap || !lut_config_ok(position_buckets, max_position))
    return FDB_ERR_LUT_ARGS;
  for (int32_t r = -radius; r <= radius; ++r) out[r + radius] = (int16_t)delta_of(r, position_buckets, max_position);
  return FDB_OK;
}

int fdb_quant_e4m3_per_head(const void* x, int64_t x_stride_t, int64_t x_stride_h, void* y, int64_t y_stride_t,
                            int64_t y_stride_h, float* scale, uint32_t* absmax_ws, int32_t tokens, int32_t heads,
                            int32_t head_dim, void* stream) {
  if (!x || !y || !scale || !absmax_ws) return FDB_ERR_NULL;
  if (head_dim != 32 && head_dim != 64 && head_dim != 128) return FDB_ERR_HEAD_DIM;
  if (tokens < 1 || heads < 1 || heads > 65535) return FDB_ERR_SHAPE;
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(y) & 7u) || (x_stride_t * 2) % 16 || (x_stride_h * 2) % 16 ||
      y_stride_t % 8 || y_stride_h % 8)
    return FDB_ERR_ALIGN;
  return fdb_launch_quant(x, nullptr, x_stride_t, x_stride_h, y, nullptr, y_stride_t, y_stride_h, scale, nullptr, absmax_ws, tokens,
                          heads, head_dim, stream);
}

int fdb_quant_e4m3_per_head_pair(const void* x0, const void* x1, int64_t x_stride_t, int64_t x_stride_h, void* y0, void* y1,
                                 int64_t y_stride_t, int64_t y_stride_h, float* scale0, float* scale1, uint32_t* absmax_ws,
                                 int32_t tokens, int32_t heads, int32_t head_dim, void* stream) {
  if (!x0 || !x1 || !y0 || !y1 || !scale0 || !scale1 || !absmax_ws) return FDB_ERR_NULL;
  if (head_dim != 32 && head_dim != 64 && head_dim != 128) return FDB_ERR_HEAD_DIM;
  if (tokens < 1 || heads < 1 || heads > 65535) return FDB_ERR_SHAPE;
  if (!aligned16(x0) || !aligned16(x1) || ((reinterpret_cast<uintptr_t>(y0) | reinterpret_cast<uintptr_t>(y1)) & 7u) ||
      (x_stride_t * 2) % 16 || (x_stride_h * 2) % 16 || y_stride_t % 8 || y_stride_h % 8)
    return FDB_ERR_ALIGN;
  return fdb_launch_quant(x0, x1, x_stride_t, x_stride_h, y0, y1, y_stride_t, y_stride_h, scale0, scale1, absmax_ws, tokens, heads,
                          head_dim, stream);
}

int fdb_dequant_e4m3_per_head(const void* y, int64_t y_stride_t, int64_t y_stride_h, const float* scale, void* x,
                              int64_t x_stride_t, int64_t x_stride_h, int32_t tokens, int32_t heads, int32_t head_dim,
                              void* stream) {
  if (!x || !y || !scale) return FDB_ERR_NULL;
  if (head_dim != 32 && head_dim != 64 && head_dim != 128) return FDB_ERR_HEAD_DIM;
  if (tokens < 1 || heads < 1 || heads > 65535) return FDB_ERR_SHAPE;
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(y) & 7u) || (x_stride_t * 2) % 16 || (x_stride_h * 2) % 16 ||
      y_stride_t % 8 || y_stride_h % 8)
    return FDB_ERR_ALIGN;
  return fdb_launch_dequant(y, y_stride_t, y_stride_h, scale, x, x_stride_t, x_stride_h, tokens, heads, head_dim, stream);
}

}  // extern "C"
