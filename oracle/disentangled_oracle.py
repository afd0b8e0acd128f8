"""CPU oracle for the DeBERTa-v2/v3 disentangled attention (forward and backward).  TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it.  The shipped path (flashdeberta_amd) never does and
fails loudly when its HIP library is missing.

It restates, in numpy, the "eager" side of the reference's attention switch.  The reference maps
"eager" to transformers' DisentangledSelfAttention (src/flashdeberta/model.py:11,255), a
third-party class (transformers, required as >=4.30.0 by the reference's pyproject.toml:11; the
image carries 5.15.0).  Citations "HF:n" are lines of
transformers/models/deberta_v2/modeling_deberta_v2.py at that version; "REF:" lines are files of
the reference repository.

Pinning (what fixes each function besides re-reading it; the tests are in tests/test_oracle.py):
  make_log_bucket_position / delta_table : known values, odd symmetry, monotonicity, saturation
        points, fp32-vs-fp64 agreement, and the golden fixtures written from the third-party class.
  disentangled_attention : content-only case == torch scaled_dot_product_attention; a triple-loop
        fp64 brute force on tiny inputs; row/column-constant bias invariants; golden fixtures.
  module_forward         : golden fixtures (hidden states -> context) from the third-party class.
  disentangled_attention_backward : central finite differences of disentangled_attention on tiny inputs
        (every operand, both position terms, masked and causal); the golden gradient fixtures, which
        autograd wrote through the third-party class (hidden states, relative embeddings, every weight).
  quantize_e4m3_per_head : torch.float8_e4m3fn round trip (library routine).
  fp8 attention          : no reference counterpart exists; "parity unpinned" beyond the
        de-quantised-input restatement and the bound against the unquantised result.
"""
import math

import numpy as np


# ------------------------------------------------------------------------------------------------
# relative positions  (HF:56-101)
# ------------------------------------------------------------------------------------------------
def make_log_bucket_position(relative_pos, bucket_size, max_position, dtype=np.float32):
    """HF:56-69.  The eager code runs this in fp32 on an int64 tensor; `dtype` allows an fp64
    evaluation for the agreement check."""
    relative_pos = np.asarray(relative_pos, dtype=np.int64)
    sign = np.sign(relative_pos)
    mid = bucket_size // 2
    abs_pos = np.where((relative_pos < mid) & (relative_pos > -mid), mid - 1, np.abs(relative_pos))
    with np.errstate(divide="ignore", invalid="ignore"):
        num = np.log((abs_pos.astype(dtype) / dtype(mid)).astype(dtype))
        den = np.log(dtype(dtype(max_position - 1) / dtype(mid)))
        log_pos = np.ceil((num / den).astype(dtype) * dtype(mid - 1)) + dtype(mid)
    bucket_pos = np.where(abs_pos <= mid, relative_pos.astype(dtype), log_pos * sign.astype(dtype))
    return bucket_pos


def build_relative_position(query_size, key_size, bucket_size=-1, max_position=-1):
    """HF:72-101 -> int64 [query_size, key_size], entry (i, j) = bucket(i - j)."""
    q_ids = np.arange(query_size, dtype=np.int64)
    k_ids = np.arange(key_size, dtype=np.int64)
    rel = q_ids[:, None] - k_ids[None, :]
    if bucket_size > 0 and max_position > 0:
        rel = make_log_bucket_position(rel, bucket_size, max_position)
    return rel.astype(np.int64)


def att_span_of(position_buckets, max_relative_positions):
    """HF:172-174 (pos_ebd_size); REF: src/flashdeberta/ops/flash_attention.py:1045."""
    return position_buckets if position_buckets > 0 else max_relative_positions


def delta_table(position_buckets, max_relative_positions, radius, dtype=np.float32):
    """delta(r) = clamp(bucket(r) + S, 0, 2S-1) for r = -radius..radius  (HF:318; HF:336 with
    -bucket(j-i) = bucket(i-j))."""
    r = np.arange(-radius, radius + 1, dtype=np.int64)
    if position_buckets > 0 and max_relative_positions > 0:
        rel = make_log_bucket_position(r, position_buckets, max_relative_positions, dtype).astype(np.int64)
    else:
        rel = r
    span = att_span_of(position_buckets, max_relative_positions)
    return np.clip(rel + span, 0, 2 * span - 1).astype(np.int64)


# ------------------------------------------------------------------------------------------------
# operator level: attention from projected tensors  (HF:236-271, HF:313-345)
# ------------------------------------------------------------------------------------------------
def _softmax_lastdim(x):
    m = x.max(axis=-1, keepdims=True)
    e = np.exp(x - m)
    return e / e.sum(axis=-1, keepdims=True), (m[..., 0] + np.log(e.sum(axis=-1)))


def disentangled_attention(q, k, v, pos_key=None, pos_query=None, position_buckets=-1,
                           max_relative_positions=-1, mask=None, causal=False, dtype=np.float64,
                           return_lse=False):
    """q, k, v: [B, H, L, D].  pos_key / pos_query: [H, 2S, D] projected relative embeddings
    (K_r, Q_r) or None.  mask: None or bool [B, L] (True = real token; keys masked with the
    dtype minimum as HF:256-257; padded query rows are computed like eager does, the caller
    ignores them).  Returns [B, H, L, D] (and the log-sum-exp [B, H, L]).

    Follows the eager order: scale = sqrt(D * scale_factor) (HF:237-243); c2p: bmm, clamp(rel+S),
    gather along the last axis (HF:315-324); p2c: bmm of K with Q_r, clamp(-rel+S), gather, transpose
    (HF:327-343)."""
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    B, H, L, D = q.shape
    scale_factor = 1 + (pos_key is not None) + (pos_query is not None)
    scale = dtype(math.sqrt(D * scale_factor))
    out = np.empty((B, H, L, D), dtype=dtype)
    lse = np.empty((B, H, L), dtype=dtype)
    span = att_span_of(position_buckets, max_relative_positions)
    if pos_key is not None or pos_query is not None:
        rel = build_relative_position(L, L, position_buckets, max_relative_positions)
        c2p_pos = np.clip(rel + span, 0, 2 * span - 1)
        p2c_pos = np.clip(-rel + span, 0, 2 * span - 1)
    neg = np.finfo(dtype).min
    for b in range(B):
        for h in range(H):
            s = q[b, h] @ (k[b, h].T / scale)
            if pos_key is not None:
                c2p = q[b, h] @ np.asarray(pos_key[h], dtype=dtype).T  # [L, 2S]
                s = s + np.take_along_axis(c2p, c2p_pos, axis=-1) / scale
            if pos_query is not None:
                p2c = k[b, h] @ np.asarray(pos_query[h], dtype=dtype).T  # [L(key), 2S]
                s = s + np.take_along_axis(p2c, p2c_pos, axis=-1).T / scale
            if mask is not None:
                s = np.where(np.asarray(mask[b], dtype=bool)[None, :], s, neg)
            if causal:
                s = np.where(np.tril(np.ones((L, L), dtype=bool)), s, neg)
            p, l = _softmax_lastdim(s)
            out[b, h] = p @ v[b, h]
            lse[b, h] = l
    return (out, lse) if return_lse else out


def disentangled_attention_backward(q, k, v, dout, pos_key=None, pos_query=None, position_buckets=-1,
                                    max_relative_positions=-1, mask=None, causal=False, dtype=np.float64):
    """Gradients of sum(disentangled_attention(...) * dout) with respect to q, k, v [B, H, L, D] and
    pos_key, pos_query [H, 2S, D]: the chain rule through the eager graph (HF:236-271 for scores,
    soft-max and PV; HF:315-324 and HF:327-343 for the two gathers, whose adjoint is a scatter-add
    into the [L, 2S] position scores).  The reference's counterpart are its three backward kernels
    (REF: src/flashdeberta/ops/flash_attention.py:62-141, 581-941), which leave the gradient of the
    [B, H, L, 2S] bias tensors to autograd; here the chain is carried through to K_r / Q_r.
    Rows of `dout` that belong to padded queries must be zero (the module never produces them)."""
    q, k, v, dout = [np.asarray(x, dtype=dtype) for x in (q, k, v, dout)]
    B, H, L, D = q.shape
    scale_factor = 1 + (pos_key is not None) + (pos_query is not None)
    scale = dtype(math.sqrt(D * scale_factor))
    span = att_span_of(position_buckets, max_relative_positions)
    if pos_key is not None or pos_query is not None:
        rel = build_relative_position(L, L, position_buckets, max_relative_positions)
        c2p_pos = np.clip(rel + span, 0, 2 * span - 1)
        p2c_pos = np.clip(-rel + span, 0, 2 * span - 1)
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    dpk = None if pos_key is None else np.zeros(np.asarray(pos_key).shape, dtype=dtype)
    dpq = None if pos_query is None else np.zeros(np.asarray(pos_query).shape, dtype=dtype)
    neg = np.finfo(dtype).min
    rows = np.arange(L)[:, None]
    for b in range(B):
        for h in range(H):
            s = q[b, h] @ (k[b, h].T / scale)
            if pos_key is not None:
                pk = np.asarray(pos_key[h], dtype=dtype)
                s = s + np.take_along_axis(q[b, h] @ pk.T, c2p_pos, axis=-1) / scale
            if pos_query is not None:
                pq = np.asarray(pos_query[h], dtype=dtype)
                s = s + np.take_along_axis(k[b, h] @ pq.T, p2c_pos, axis=-1).T / scale
            if mask is not None:
                s = np.where(np.asarray(mask[b], dtype=bool)[None, :], s, neg)
            if causal:
                s = np.where(np.tril(np.ones((L, L), dtype=bool)), s, neg)
            p, _ = _softmax_lastdim(s)
            do = dout[b, h]
            dv[b, h] = p.T @ do
            dp = do @ v[b, h].T
            ds = p * (dp - (p * dp).sum(axis=-1, keepdims=True)) / scale  # w.r.t. the raw score sums
            dq[b, h] = ds @ k[b, h]
            dk[b, h] = ds.T @ q[b, h]
            if pos_key is not None:
                g = np.zeros((L, 2 * span), dtype=dtype)  # d(q K_r^T)[i, delta]
                np.add.at(g, (rows, c2p_pos), ds)
                dq[b, h] += g @ pk[:2 * span]
                dpk[h, :2 * span] += g.T @ q[b, h]
            if pos_query is not None:
                g = np.zeros((L, 2 * span), dtype=dtype)  # d(k Q_r^T)[j, delta]: element (i, j) read [j, p2c_pos[j, i]]
                np.add.at(g, (rows, p2c_pos), ds.T)
                dk[b, h] += g @ pq[:2 * span]
                dpq[h, :2 * span] += g.T @ k[b, h]
    return dq, dk, dv, dpk, dpq


def disentangled_attention_varlen(q, k, v, cu_seqlens, pos_key=None, pos_query=None, position_buckets=-1,
                                  max_relative_positions=-1, dtype=np.float64):
    """Packed form: q, k, v [T, H, D]; each sequence cu[b]:cu[b+1] attends only to itself with its
    own relative-position window -- eager run on every sequence alone (the definition of the
    varlen path; REF: src/flashdeberta/padding.py:79-88 for cu_seqlens)."""
    q = np.asarray(q)
    out = np.zeros(q.shape, dtype=dtype)
    for b in range(len(cu_seqlens) - 1):
        lo, hi = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        if hi <= lo:
            continue
        sl = lambda x: np.transpose(np.asarray(x[lo:hi], dtype=dtype), (1, 0, 2))[None]
        o = disentangled_attention(sl(q), sl(k), sl(v), pos_key, pos_query, position_buckets,
                                   max_relative_positions, dtype=dtype)
        out[lo:hi] = np.transpose(o[0], (1, 0, 2))
    return out


def brute_force_attention(q, k, v, pos_key, pos_query, position_buckets, max_relative_positions):
    """Independent triple loop in python floats (tiny inputs only): score(i,j) =
    (q_i.k_j + q_i.K_r[delta(i-j)] + k_j.Q_r[delta(i-j)]) / sqrt(D*f).  Used to pin the gather /
    transpose wiring of disentangled_attention, not derived from it."""
    B, H, L, D = q.shape
    f = 1 + (pos_key is not None) + (pos_query is not None)
    span = att_span_of(position_buckets, max_relative_positions)
    out = np.zeros((B, H, L, D))
    for b in range(B):
        for h in range(H):
            for i in range(L):
                sc = []
                for j in range(L):
                    r = i - j
                    if position_buckets > 0:
                        mid = position_buckets // 2
                        a = abs(r)
                        if a <= mid:
                            bkt = r
                        else:
                            x = math.ceil(math.log(a / mid) / math.log((max_relative_positions - 1) / mid) * (mid - 1)) + mid
                            bkt = x if r > 0 else -x
                    else:
                        bkt = r
                    d = min(max(bkt + span, 0), 2 * span - 1)
                    s = float(np.dot(q[b, h, i], k[b, h, j]))
                    if pos_key is not None:
                        s += float(np.dot(q[b, h, i], pos_key[h, d]))
                    if pos_query is not None:
                        s += float(np.dot(k[b, h, j], pos_query[h, d]))
                    sc.append(s / math.sqrt(D * f))
                m = max(sc)
                e = [math.exp(x - m) for x in sc]
                z = sum(e)
                for j in range(L):
                    out[b, h, i] += (e[j] / z) * v[b, h, j]
    return out


# ------------------------------------------------------------------------------------------------
# module level: hidden states -> context  (HF:191-274 with REF model.py:147-181 for the wiring)
# ------------------------------------------------------------------------------------------------
def _linear(x, w, b):
    y = x @ np.asarray(w).T
    return y if b is None else y + np.asarray(b)


def _heads(x, H):  # [..., L, H*D] -> [..., H, L, D]   (HF:186-189)
    *lead, L, HD = x.shape
    return np.moveaxis(x.reshape(*lead, L, H, HD // H), -2, -3)


def module_forward(hidden_states, weights, rel_embeddings, num_heads, pos_att_type, share_att_key,
                   position_buckets, max_relative_positions, mask=None, query_states=None, dtype=np.float64):
    """weights: dict with query_proj.weight/bias, key_proj.*, value_proj.* and, when not
    share_att_key, pos_key_proj.* / pos_query_proj.* (names of HF:159-182; pos_query_proj has a
    bias in 5.15.0).  rel_embeddings: [>=2S, hidden] (already layer-normed by the encoder when
    norm_rel_ebd asks for it, HF:595-599).  mask: None or [B, L].  Returns [B, L, H*D]."""
    hs = np.asarray(hidden_states, dtype=dtype)
    qs = hs if query_states is None else np.asarray(query_states, dtype=dtype)
    W = {n: np.asarray(t, dtype=dtype) for n, t in weights.items()}
    q = _heads(_linear(qs, W["query_proj.weight"], W.get("query_proj.bias")), num_heads)
    k = _heads(_linear(hs, W["key_proj.weight"], W.get("key_proj.bias")), num_heads)
    v = _heads(_linear(hs, W["value_proj.weight"], W.get("value_proj.bias")), num_heads)
    pos_key = pos_query = None
    if rel_embeddings is not None and pos_att_type:
        span = att_span_of(position_buckets, max_relative_positions)
        rel = np.asarray(rel_embeddings, dtype=dtype)[0:2 * span]  # HF:295
        if share_att_key:  # HF:296-302
            pq_all = _heads(_linear(rel, W["query_proj.weight"], W.get("query_proj.bias")), num_heads)
            pk_all = _heads(_linear(rel, W["key_proj.weight"], W.get("key_proj.bias")), num_heads)
        else:  # HF:303-311
            pk_all = _heads(_linear(rel, W["pos_key_proj.weight"], W.get("pos_key_proj.bias")), num_heads) \
                if "c2p" in pos_att_type else None
            pq_all = _heads(_linear(rel, W["pos_query_proj.weight"], W.get("pos_query_proj.bias")), num_heads) \
                if "p2c" in pos_att_type else None
        if "c2p" in pos_att_type:
            pos_key = pk_all
        if "p2c" in pos_att_type:
            pos_query = pq_all
    o = disentangled_attention(q, k, v, pos_key, pos_query, position_buckets, max_relative_positions,
                               mask=mask, dtype=dtype)
    B, H, L, D = o.shape
    return np.transpose(o, (0, 2, 1, 3)).reshape(B, L, H * D)  # HF:265-271


def unpad_data(mask):
    """REF: src/flashdeberta/padding.py:79-88 -> (indices of real tokens in the flattened batch,
    cu_seqlens int32 [B+1], longest length)."""
    mask = np.asarray(mask).astype(bool)
    lens = mask.sum(axis=-1).astype(np.int32)
    indices = np.nonzero(mask.reshape(-1))[0]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    return indices, cu, int(lens.max()) if len(lens) else 0


# ------------------------------------------------------------------------------------------------
# FP8 (OCP e4m3) Q/K variant -- no counterpart in the reference
# ------------------------------------------------------------------------------------------------
def e4m3_round(x):
    """Round fp32 values to the nearest OCP e4m3 value (ties to even), saturating at +-448.
    Returns fp32 holding exactly representable e4m3 numbers."""
    x = np.asarray(x, dtype=np.float32)
    a = np.minimum(np.abs(x), np.float32(448.0)).astype(np.float64)
    # exponent of the binade, clamped to the subnormal binade (2^-6, step 2^-9)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.maximum(e, -6.0)
    step = np.exp2(e - 3.0)  # 3 mantissa bits
    y = np.rint(a / step) * step  # np.rint rounds half to even
    y = np.minimum(y, 448.0)
    return (np.sign(x) * y).astype(np.float32)


def quantize_e4m3_per_head(x):
    """x: [T, H, D] (any float).  scale[h] = max(absmax_h, 1e-12) / 448 in fp32,
    y = e4m3(x / scale[h]) with fp32 division.  Returns (y as fp32 holding e4m3 values, scale fp32 [H])."""
    x = np.asarray(x, dtype=np.float32)
    amax = np.maximum(np.abs(x).max(axis=(0, 2)), np.float32(1e-12)).astype(np.float32)
    scale = (amax / np.float32(448.0)).astype(np.float32)
    y = e4m3_round((x / scale[None, :, None]).astype(np.float32))
    return y, scale


def e4m3_encode(y):
    """fp32 array holding e4m3-representable values -> uint8 bit patterns (sign, 4 exp, 3 mantissa, bias 7)."""
    y = np.asarray(y, dtype=np.float32)
    a = np.abs(y).astype(np.float64)
    sign = (np.signbit(y)).astype(np.uint8) << 7
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    normal = a >= 2.0 ** -6
    e = np.where(normal, e, -6.0)
    mant = np.where(normal, a / np.exp2(e) - 1.0, a / np.exp2(-6.0)) * 8.0
    expf = np.where(normal, e + 7.0, 0.0)
    return (sign | (expf.astype(np.uint8) << 3) | np.rint(mant).astype(np.uint8)).astype(np.uint8)
