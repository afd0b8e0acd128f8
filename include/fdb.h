/*
 * fdb.h -- C ABI of the MI355X (gfx950) disentangled-attention forward library.
 *
 * The library is a plain shared object (libfdb_hip.so): C linkage, raw device pointers,
 * integer sizes and strides, no C++ or torch types in any signature.  It never allocates or
 * frees device memory and keeps no pointer after a call returns; every buffer, including the
 * output, the optional log-sum-exp, the varlen work-list, the delta look-up table and the
 * optional workspace, is owned by the caller.  All launches are asynchronous on the stream passed in.
 *
 * Reference interfaces replaced (paths relative to the FlashDeBERTa repository):
 *   fdb_attn_fwd           <- flash_attention_with_disentangled
 *                             (src/flashdeberta/ops/flash_attention.py:1088-1091, kernel :146-300,
 *                             launcher :421-488) and flash_attention_with_disentangled_varlen
 *                             (src/flashdeberta/ops/flash_attention_varlen.py:485-511, kernel :85-225,
 *                             launcher :349-440), plus the two bias GEMMs the module runs before
 *                             them (src/flashdeberta/model.py:189-192 and :210-214), which are
 *                             fused here: the entry point takes the projected relative embeddings
 *                             K_r / Q_r [H, 2S, D] rather than their [B,H,L,2S] products.
 *   fdb_build_worklist     <- get_mid (src/flashdeberta/ops/flash_attention_varlen.py:71-83), the
 *                             per-q-tile (sequence, first row) list; built on the device.
 *   fdb_delta_lut          <- the log-bucket arithmetic evaluated per score element in the kernels
 *                             (flash_attention.py:236-254, flash_attention_varlen.py:174-186), i.e.
 *                             make_log_bucket_position of transformers' modeling_deberta_v2.py:56-69
 *                             followed by clamp(. + S, 0, 2S-1) (:318, :336); host-side, integers out.
 *   fdb_attn_bwd           <- flash_attn_v2_bwd_dise (flash_attention.py:942-1030) with _bwd_preprocess,
 *                             _bwd_kv_dise_kernel and _bwd_q_dise_kernel (:62-141, :581-941).
 *   fdb_attn_bwd_chain     <- the backward of the two bias GEMMs the reference's module runs in front of its
 *                             kernels (src/flashdeberta/model.py:189-192: pos_key = q . K_r^T, pos_query = k . Q_r^T),
 *                             which the reference leaves to autograd: d q += d pos_key . K_r, d K_r = d pos_key^T . q
 *                             (and the same for k / Q_r), here both in one pass over the score gradients.
 *   fdb_quant_e4m3_per_head, fdb_quant_e4m3_per_head_pair, fdb_dequant_e4m3_per_head   no reference counterpart
 *                             (FP8 Q/K variant).
 */
#ifndef FDB_H_
#define FDB_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* bumped whenever fdb_attn_args or the meaning of an entry point changes: a binding checks it next to the struct size */
#define FDB_VERSION 7

/* element types of q/k/pos_key/pos_query (v and out: see fdb_attn_args.dtype) */
enum fdb_dtype {
  FDB_F32 = 0,      /* everything fp32, fp32 MFMA                                   */
  FDB_BF16 = 1,     /* everything bf16, fp32 accumulate                             */
  FDB_F16 = 2,      /* everything fp16, fp32 accumulate                             */
  FDB_FP8_E4M3 = 3  /* q,k,pos_key,pos_query OCP e4m3 + per-head scales; v,out bf16 */
};

/* return codes: 0 ok, negative = invalid argument, positive = hipError_t of the launch */
enum fdb_status {
  FDB_OK = 0,
  FDB_ERR_NULL = -1,        /* required pointer is NULL                                   */
  FDB_ERR_DTYPE = -2,       /* dtype not one of fdb_dtype                                  */
  FDB_ERR_HEAD_DIM = -3,    /* head_dim not supported (supported: 32, 64, 128)             */
  FDB_ERR_ALIGN = -4,       /* pointer or stride not 16-byte aligned                       */
  FDB_ERR_SHAPE = -5,       /* batch/heads/seqlen/total_tokens not positive or inconsistent */
  FDB_ERR_SPAN = -6,        /* att_span <= 0 or lut_radius < 1 with a position term present */
  FDB_ERR_SCALE = -7,       /* fp8 dtype without the needed scale vectors                  */
  FDB_ERR_WORKLIST = -8,    /* cu_seqlens given without a work-list buffer                 */
  FDB_ERR_LUT_ARGS = -9,    /* fdb_delta_lut: bad bucket/max_position/radius/out           */
  FDB_ERR_UNSUPPORTED = -10, /* combination not built                                      */
  FDB_ERR_SCRATCH = -11     /* fdb_attn_fwd_noalloc: hand-over buffers exceed the built-in scratch */
};

/*
 * One forward call.  Logical tensors (S = att_span):
 *   q, k, v, out : element (b, l, h, d) at  base + b*stride_b + (tok0_b + l)*stride_t + h*stride_h + d
 *                  fixed length (cu_seqlens == NULL): tok0_b = 0, 0 <= l < max_seqlen; with seq_start /
 *                                                      seq_len (padded batches) the real tokens of row b are
 *                                                      l in [seq_start[b], seq_start[b]+seq_len[b]), they
 *                                                      attend only to each other with positions counted
 *                                                      from seq_start[b]; the other rows of `out` are written
 *                                                      as zeros (what the eager module leaves in padded rows);
 *                                                      a negative seq_len[b] marks a batch row whose mask the
 *                                                      caller could not express as one run of tokens: all its
 *                                                      rows of `out` are written as NaN
 *                  packed varlen (cu_seqlens != NULL): tok0_b = cu_seqlens[b], stride_b ignored,
 *                                                      0 <= l < cu_seqlens[b+1]-cu_seqlens[b]
 *   pos_key  (K_r): element (h, r, d) at base + h*pk_stride_h + r*pk_stride_r + d, 0 <= r < 2S
 *   pos_query(Q_r): likewise with pq_stride_*
 *   score(i,j) = sm_scale * ( q_i.k_j + q_i.K_r[delta(i-j)] + k_j.Q_r[delta(i-j)] ),
 *   delta(r) = delta_lut[clamp(r, -lut_radius, lut_radius) + lut_radius]; a NULL pos pointer
 *   drops that term.  out_i = sum_j softmax_j(score(i,.)) v_j ; lse_i = log sum_j exp(score(i,j)).
 * Strides are in elements.  The last dimension has unit stride.  Token strides of k and v below 2^31 bytes;
 * row strides of pos_key / pos_query non-negative and below 2^24 bytes, a head's 2S rows within 2^31 bytes
 * (FDB_ERR_SHAPE otherwise).
 */
typedef struct fdb_attn_args {
  const void* q;
  const void* k;
  const void* v;
  const void* pos_key;     /* K_r or NULL (no content->position term)  */
  const void* pos_query;   /* Q_r or NULL (no position->content term)  */
  void* out;
  float* lse;              /* [B*max_seqlen*H] (fixed) / [T*H] (varlen), token-major, or NULL */
  const int32_t* cu_seqlens; /* device int32[batch+1] or NULL                                 */
  int32_t* worklist;       /* device int32[fdb_worklist_ints(...)], filled by fdb_build_worklist */
  const int32_t* seq_start; /* fixed layout only, device int32[batch] or NULL: first real token of each row */
  const int32_t* seq_len;   /* fixed layout only, device int32[batch] or NULL: number of real tokens        */
  const int16_t* delta_lut;  /* device int16[2*lut_radius+1] from fdb_delta_lut, or NULL if no pos term */
  const float* q_scale;    /* fp8 only: device float[heads] dequant scales               */
  const float* k_scale;
  const float* pk_scale;
  const float* pq_scale;
  void* workspace;         /* device scratch of workspace_bytes bytes, 16-byte aligned, or NULL: see fdb_attn_workspace_bytes */
  int64_t q_stride_b, q_stride_t, q_stride_h;
  int64_t k_stride_b, k_stride_t, k_stride_h;
  int64_t v_stride_b, v_stride_t, v_stride_h;
  int64_t o_stride_b, o_stride_t, o_stride_h;
  int64_t pk_stride_h, pk_stride_r;
  int64_t pq_stride_h, pq_stride_r;
  int64_t workspace_bytes;
  int32_t batch;
  int32_t heads;
  int32_t head_dim;
  int32_t max_seqlen;      /* fixed: the sequence length; varlen: upper bound on any length */
  int32_t total_tokens;    /* varlen: cu_seqlens[batch]; fixed: batch*max_seqlen            */
  int32_t att_span;        /* S: position_buckets if > 0 else max_relative_positions        */
  int32_t lut_radius;
  int32_t dtype;           /* enum fdb_dtype                                                 */
  int32_t causal;          /* nonzero: key j visible to query i only if j <= i               */
  int32_t far_splits;      /* 0: the library decides; 1 .. FDB_MAX_FAR_SPLITS: workgroups that share the far keys of a query tile
                              (all its keys where one kernel serves the call) */
  int32_t near_splits;     /* the same for the near keys (those whose bucketed relative position varies)                  */
  float sm_scale;
} fdb_attn_args;

#define FDB_MAX_FAR_SPLITS 4

int fdb_version(void);
/* sizeof(fdb_attn_args) as the library was built: lets a foreign-language binding check its struct mirror. */
size_t fdb_attn_args_size(void);
const char* fdb_strerror(int code);

/* Host-only validation of an argument block (what fdb_attn_fwd checks before launching). */
int fdb_attn_check(const fdb_attn_args* a);

/* Enqueue the fused forward on `stream` (a hipStream_t).
 * A packed call (cu_seqlens) whose total_tokens exceed lut_radius + 63 always includes the launch over the far
 * keys, because max_seqlen is the caller's word and the token count is the one bound the library can trust: for a
 * batch of many short sequences that launch finds no far key tile and costs a few microseconds. */
int fdb_attn_fwd(const fdb_attn_args* a, void* stream);

/*
 * Measurement hook, not a result: one of the launches fdb_attn_fwd makes for this argument block, alone, so that a
 * profiler-free harness can time them one at a time.  part 1 = the launch over the far keys (those whose bucketed
 * relative position is constant), part 2 = the launch over the near keys with its merge kernel.  What `out` and
 * `lse` hold afterwards is a partial result.  FDB_ERR_UNSUPPORTED for calls that are a single kernel.  No
 * counterpart in the reference.
 */
int fdb_attn_fwd_part(const fdb_attn_args* a, int32_t part, void* stream);

/*
 * fdb_attn_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The caller passes the inputs
 * and `out` only; what fdb_attn_fwd takes from caller-owned buffers besides them -- the log-sum-exp
 * hand-over between its two launches (used when `lse` is NULL; a non-NULL `lse` is filled as usual), the
 * packed layout's work-list (built here, `worklist` is ignored) and the workspace of partial results
 * (`workspace` is ignored) -- comes from FDB_NOALLOC_SCRATCH_BYTES of device memory inside the library's
 * own image, one copy per GPU, held until the process ends.  The call allocates and frees nothing.
 * Limit: hand-over plus work-list, rows * heads * 4 + fdb_worklist_ints(...) * 4 bytes (each rounded up to
 * 256), must fit the scratch, else FDB_ERR_SCRATCH and nothing is launched; partial results use what is
 * left and the call shares less when that is small (same result up to rounding).  Nothing in the scratch
 * has to start at zero (every word read was written earlier in the same call).  All calls on one GPU
 * share its scratch: calls that overlap in time on one GPU (two streams, two threads) race; serialise them.
 * The first call on a device asks the runtime for the scratch's address (hipGetSymbolAddress): make that first
 * call outside stream capture; every later call on the device is capture-safe.
 */
#define FDB_NOALLOC_SCRATCH_BYTES (32 * 1024 * 1024)
int fdb_attn_fwd_noalloc(const fdb_attn_args* a, void* stream);

/*
 * Backward, fixed layout (optionally with seq_start / seq_len).  Replaces flash_attn_v2_bwd_dise and the three
 * kernels it launches (src/flashdeberta/ops/flash_attention.py:942-1030, :62-141, :581-941), called from
 * FlashAttentionDisentangled.backward (:1066-1086).  Same division of labour as there: the position scores come
 * in as tensors, c2p_bias[b,l,h,delta] = q . K_r[delta] and p2c_bias[b,l,h,delta] = k . Q_r[delta], and the
 * gradients with respect to them leave in d_c2p_bias / d_p2c_bias; all four have the element type of `dtype`,
 * like the reference's ([B,H,L,2S] in the input dtype).  Every entry of the gradient tensors that belongs to a
 * real token (batch row b, seq_start[b] <= l < seq_start[b] + seq_len[b]) is stored exactly once, by plain stores in
 * aligned groups of four (zeros where no score maps to it); rows of padding are not touched, so a caller with a padded
 * batch clears the tensors first.  The four tensors share one layout: element (b, l, h, delta) at b * bias_stride_b + l * bias_stride_t
 * + h * bias_stride_h + delta (strides in elements, multiples of 4; 2S a multiple of 4; the gradient tensors
 * aligned to four elements, the score tensors to four bytes; l * bias_stride_t + delta must stay below 2^31).  Head-major [H, B, L, 2S] is what a batched
 * GEMM over the heads writes and reads without a transpose.  The chain through K_r / Q_r and into q / k is the
 * caller's GEMMs.
 * dq, dk, dv hold only the content part,
 *   dq_i = sum_j dS_ij k_j,  dk_j = sum_i dS_ij q_i,  dv_j = sum_i P_ij dO_i,  dS = P (dO V^T - delta) sm_scale,
 * with P recomputed from lse (the forward's log-sum-exp, [B*L, H]) and delta[row] = sum_d dO * O ([B*L, H] fp32;
 * the reference's _bwd_preprocess, :62-141).  With `out` (the forward's output, strides like q) the call computes
 * delta itself and leaves it in `delta`; with out == NULL it reads `delta` as given.
 * Rows outside [seq_start, seq_start + seq_len) are not written.  q, k, v, dout, dq, dk, dv: element type of
 * `dtype` (fp32 / bf16 / fp16), layout and strides as in fdb_attn_args.
 * The score gradients of a row are collected in a sliding window of FDB_BWD_RING table rows, which holds the rows
 * 32 consecutive relative positions map to plus one partly stored group: a table whose lut_window (the largest
 * delta(r + 31) - delta(r)) exceeds FDB_BWD_MAX_WINDOW is refused with FDB_ERR_SPAN.  Every table with steps of
 * 0 or 1 passes (window <= 31), so does every log-bucket table with max_position >= position_buckets; the
 * reference scatters with atomics and takes any table (flash_attention.py:769-786).
 */
#define FDB_BWD_RING 64
#define FDB_BWD_MAX_WINDOW (FDB_BWD_RING - 4)
typedef struct fdb_attn_bwd_args {
  const void* q;
  const void* k;
  const void* v;
  const void* dout;
  void* dq;
  void* dk;
  void* dv;
  const float* lse;
  float* delta;            /* [B*L, H] fp32: written when `out` is given, read otherwise */
  const void* out;         /* the forward's output or NULL */
  const void* c2p_bias;    /* or NULL: no content->position term; elements of `dtype` */
  const void* p2c_bias;    /* or NULL: no position->content term; elements of `dtype` */
  void* d_c2p_bias;        /* required with c2p_bias; elements of `dtype` */
  void* d_p2c_bias;        /* required with p2c_bias; elements of `dtype` */
  const int32_t* seq_start;
  const int32_t* seq_len;
  const int16_t* delta_lut;
  int64_t q_stride_b, q_stride_t, q_stride_h;
  int64_t k_stride_b, k_stride_t, k_stride_h;
  int64_t v_stride_b, v_stride_t, v_stride_h;
  int64_t do_stride_b, do_stride_t, do_stride_h;
  int64_t out_stride_b, out_stride_t, out_stride_h;
  int64_t dq_stride_b, dq_stride_t, dq_stride_h;
  int64_t dk_stride_b, dk_stride_t, dk_stride_h;
  int64_t dv_stride_b, dv_stride_t, dv_stride_h;
  int64_t bias_stride_b, bias_stride_t, bias_stride_h;   /* of c2p_bias, p2c_bias, d_c2p_bias, d_p2c_bias */
  int32_t batch;
  int32_t heads;
  int32_t head_dim;
  int32_t seqlen;
  int32_t att_span;
  int32_t lut_radius;
  int32_t lut_window;      /* fdb_delta_lut_window(...) of the table behind delta_lut (with a position term) */
  int32_t dtype;           /* FDB_F32, FDB_BF16 or FDB_F16 */
  int32_t causal;
  float sm_scale;
} fdb_attn_bwd_args;

size_t fdb_attn_bwd_args_size(void);
int fdb_attn_bwd(const fdb_attn_bwd_args* a, void* stream);

/*
 * The chain of the backward through the position tables, for `matrices` (head, term) pairs at once: with
 * g = d_scores [matrices][rows][2 * att_span] (what fdb_attn_bwd left in d_c2p_bias / d_p2c_bias, head-major),
 * the token rows x (the q rows for a c2p matrix, the k rows for a p2c matrix: row r of matrix m at
 * x + m * x_stride_matrix + r * x_stride_row for m < first_matrices, at x_second + (m - first_matrices) *
 * x_stride_matrix + r * x_stride_row beyond, in elements, head_dim contiguous elements each -- q and k are read
 * where they lie; x_second may be NULL when first_matrices == matrices) and
 * pos [matrices][2 * att_span][head_dim] (K_r resp. Q_r), g and pos contiguous, all of element type `dtype`:
 *     dx (rows addressed like those of x, through dx / dx_second and dx_stride_matrix / dx_stride_row: dq and dk are
 *         updated where they lie)                        += g . pos     (in place, fp32 accumulation, one rounding)
 *     dpos_parts [parts][matrices][2 * att_span][head_dim] = partial sums of g^T . x over `parts` shares of the rows
 *                                                           (fp32; the caller adds the parts up)
 * Built for head_dim 64, att_span 256, FDB_BF16 / FDB_F16, rows a multiple of 32, 1 <= parts <= rows / 32, pointers
 * and the strides of x and dx (in bytes) aligned to 16 bytes; anything else is refused (FDB_ERR_HEAD_DIM / _SPAN / _DTYPE / _SHAPE / _ALIGN) and the caller
 * takes the two matrix products instead.  Reference: the autograd backward of model.py:189-192 (see the list above).
 */
int fdb_attn_bwd_chain(const void* d_scores, const void* x, const void* x_second, const void* pos, void* dx, void* dx_second,
                       float* dpos_parts, int32_t matrices, int32_t first_matrices, int64_t rows, int64_t x_stride_matrix,
                       int64_t x_stride_row, int64_t dx_stride_matrix, int64_t dx_stride_row, int32_t att_span, int32_t head_dim,
                       int32_t dtype, int32_t parts, void* stream);

/*
 * Bytes of workspace the call would use (0: none), for the device that is current.  A launch whose
 * query tiles fill at most half of the workgroups the GPU holds shares the keys of each query tile among up
 * to FDB_MAX_FAR_SPLITS workgroups, separately for the far keys (those whose bucketed relative position is
 * constant; launch of their own) and the near keys; the partial results go through the workspace, one slot of
 * rows * heads * (head_dim * sizeof(v element) + 4) bytes each (rows: those of the lse buffer): far_splits - 1
 * slots, plus near_splits slots if near_splits > 1 (a small merge kernel then follows the two launches).
 * The workspace is optional: without it (or with a smaller one) the call first gives up the near splits,
 * then uses as many far splits as fit, down to one, with the same result up to rounding.  Calls that one kernel
 * serves (fp32, head_dim 128, no position term, no lse buffer) share ALL key tiles of a query tile among up to
 * FDB_MAX_FAR_SPLITS workgroups when the query tiles fill less than half of the compute units (never for causal
 * calls): far_splits slots (far_splits asks for a number), and a merge kernel follows.  far_splits and
 * near_splits of `a` are read, its workspace fields ignored here.  No counterpart in the reference, whose
 * kernels have one program per query tile (flash_attention.py:465-488).
 */
int64_t fdb_attn_workspace_bytes(const fdb_attn_args* a);

/* Number of int32 the varlen work-list needs for (total_tokens, batch): 2 ints per possible
 * q-tile plus a header.  Depends on shapes only, so no device sync is needed to size it. */
int64_t fdb_worklist_ints(int32_t total_tokens, int32_t batch);

/* Upper bound on q-tiles for (total_tokens, batch); the grid of the varlen launch. */
int32_t fdb_worklist_max_tiles(int32_t total_tokens, int32_t batch);

/* Rows of one q-tile (the work-list granularity). */
int32_t fdb_tile_rows(void);

/* Enqueue the device-side work-list construction from cu_seqlens. */
int fdb_build_worklist(const int32_t* cu_seqlens, int32_t batch, int32_t total_tokens,
                       int32_t* worklist, void* stream);

/*
 * Host: fill out[0 .. 2*radius] with delta(r) for r = -radius .. radius, where
 *   position_buckets > 0 : delta = clamp(log_bucket(r; position_buckets, max_position) + S, 0, 2S-1), S = position_buckets
 *   otherwise            : delta = clamp(r + S, 0, 2S-1), S = max_position
 * fdb_delta_lut_radius returns the smallest radius beyond which delta is constant on both sides.
 */
int32_t fdb_delta_lut_radius(int32_t position_buckets, int32_t max_position);
int fdb_delta_lut(int32_t position_buckets, int32_t max_position, int32_t radius, int16_t* out);
/* Host: the largest delta(r + 31) - delta(r) over all r, i.e. how many table rows beyond the first the 32 loop
 * rows of one backward step can reach (negative: FDB_ERR_LUT_ARGS).  What fdb_attn_bwd_args.lut_window takes. */
int32_t fdb_delta_lut_window(int32_t position_buckets, int32_t max_position);

/*
 * Per-head absmax quantisation to OCP e4m3: for each head h,
 *   scale[h] = max(absmax over all tokens and d of x[:, h, :], tiny) / 448,
 *   y = e4m3_rne(x / scale[h]).
 * x: bf16 element (t, h, d) at x + t*x_stride_t + h*x_stride_h + d, t < tokens; y: same indexing
 * with y strides, one byte per element.  absmax_ws: device uint32[heads] scratch owned by the caller.
 */
int fdb_quant_e4m3_per_head(const void* x, int64_t x_stride_t, int64_t x_stride_h,
                            void* y, int64_t y_stride_t, int64_t y_stride_h,
                            float* scale, uint32_t* absmax_ws,
                            int32_t tokens, int32_t heads, int32_t head_dim, void* stream);

/*
 * The same for two tensors of one shape and one set of strides in the same three launches (fill, absmax,
 * quantise) -- q and k of a layer, or K_r and Q_r.  absmax_ws: device uint32[2 * heads].  Each tensor gets its own
 * scales.  No reference counterpart (FP8 Q/K variant).
 */
int fdb_quant_e4m3_per_head_pair(const void* x0, const void* x1, int64_t x_stride_t, int64_t x_stride_h,
                                 void* y0, void* y1, int64_t y_stride_t, int64_t y_stride_h,
                                 float* scale0, float* scale1, uint32_t* absmax_ws,
                                 int32_t tokens, int32_t heads, int32_t head_dim, void* stream);

/*
 * The inverse map to bf16, x = bf16_rne(e4m3(y) * scale[h]), same indexing as above (y: one byte per
 * element, 8-byte aligned rows; x: bf16, 16-byte aligned rows).  No reference counterpart (FP8 Q/K
 * variant); a utility for callers and tests, not used by fdb_attn_fwd.
 */
int fdb_dequant_e4m3_per_head(const void* y, int64_t y_stride_t, int64_t y_stride_h, const float* scale,
                              void* x, int64_t x_stride_t, int64_t x_stride_h,
                              int32_t tokens, int32_t heads, int32_t head_dim, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FDB_H_ */
