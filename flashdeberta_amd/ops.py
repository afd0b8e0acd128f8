"""Operators of the disentangled-attention forward on MI355X.

Counterparts in the reference (src/flashdeberta/ops/):
  flash_attention_with_disentangled        flash_attention.py:1088-1091
  flash_attention_with_disentangled_varlen flash_attention_varlen.py:485-511
The reference ops take the pre-multiplied bias tensors Q.K_r^T and K.Q_r^T ([B,H,L,2S], built by
src/flashdeberta/model.py:189-192 / :210-214).  Here those products are fused into the kernel, so
the ops take the factors K_r / Q_r ([H, 2S, D], the projected relative embeddings) instead.
"""
import ctypes
import math

import numpy as np
import torch

from . import _lib
from ._lib import FdbAttnArgs, check, lib

_DTYPES = {torch.float32: _lib.FDB_F32, torch.bfloat16: _lib.FDB_BF16, torch.float16: _lib.FDB_F16}
_FP8 = torch.float8_e4m3fn

_lut_host_cache = {}
_lut_dev_cache = {}


def att_span(position_buckets, max_relative_positions):
    """S of the reference (flash_attention.py:1045): buckets if bucketing is on, else the max distance."""
    return position_buckets if position_buckets > 0 else max_relative_positions


def delta_lut_host(position_buckets, max_relative_positions):
    """(int16 numpy array of delta(r) for r = -R..R, R).  Pure host code (no GPU needed)."""
    key = (int(position_buckets), int(max_relative_positions))
    hit = _lut_host_cache.get(key)
    if hit is not None:
        return hit
    radius = lib.fdb_delta_lut_radius(*key)
    if radius < 1:
        raise ValueError("unsupported relative-position config position_buckets=%d max_relative_positions=%d: %s"
                         % (key[0], key[1], _lib.strerror(radius)))
    out = np.empty(2 * radius + 1, dtype=np.int16)
    check(lib.fdb_delta_lut(key[0], key[1], radius, out.ctypes.data_as(ctypes.c_void_p)), "fdb_delta_lut")
    _lut_host_cache[key] = (out, radius)
    return out, radius


def delta_lut_window(position_buckets, max_relative_positions):
    """The largest delta(r + 31) - delta(r) of the table: what the backward's score-gradient ring has to hold."""
    w = lib.fdb_delta_lut_window(int(position_buckets), int(max_relative_positions))
    if w < 0:
        raise ValueError("unsupported relative-position config position_buckets=%d max_relative_positions=%d: %s"
                         % (position_buckets, max_relative_positions, _lib.strerror(w)))
    return w


def delta_lut_device(position_buckets, max_relative_positions, device):
    key = (int(position_buckets), int(max_relative_positions), torch.device(device))
    hit = _lut_dev_cache.get(key)
    if hit is None:
        host, radius = delta_lut_host(position_buckets, max_relative_positions)
        hit = (torch.from_numpy(host).to(device), radius)
        _lut_dev_cache[key] = hit
    return hit


def _stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _pos_arg(x, H, D, span, name):
    """K_r / Q_r as [H, 2S, D] (a leading singleton batch dim as produced by the module is dropped)."""
    if x is None:
        return None
    if x.dim() == 4 and x.shape[0] == 1:
        x = x[0]
    if x.dim() != 3 or x.shape[0] != H or x.shape[2] != D or x.shape[1] < 2 * span:
        raise ValueError("%s must be the projected relative embeddings [H=%d, >=2S=%d, D=%d], got %s. "
                         "(The pre-multiplied [B,H,L,2S] bias tensors of the reference op are not an input here: "
                         "the product is fused into the kernel.)" % (name, H, 2 * span, D, tuple(x.shape)))
    if x.stride(2) != 1:
        x = x.contiguous()
    return x


def disentangled_attention_fwd(q, k, v, pos_key=None, pos_query=None, *, cu_seqlens=None, max_seqlen=None,
                               sm_scale=None, position_buckets=0, max_relative_positions=0, causal=False,
                               return_lse=False, seq_start=None, seq_len=None, q_scale=None, k_scale=None, pos_key_scale=None,
                               pos_query_scale=None, out=None, single_kernel=False, far_splits=0, near_splits=0, workspace=None,
                               no_alloc=False, _part=0):
    """Fused forward.  Layouts (strides are free except a unit stride on D):
         fixed length : q, k, v  [B, L, H, D]   -> out [B, L, H, D] (contiguous: a free view of [B, L, H*D])
         packed varlen: q, k, v  [T, H, D] + cu_seqlens int32 [B+1] (+ max_seqlen upper bound) -> out [T, H, D]
       pos_key = K_r, pos_query = Q_r: [H, 2S, D] or None (term absent).  sm_scale defaults to
       1/sqrt(D * (1 + #position terms)) as the reference module computes it (src/flashdeberta/model.py:151-157).
       padded batches (fixed layout only): seq_start / seq_len int32 [B] GPU tensors give each row's real
       tokens [seq_start, seq_start+seq_len); only those rows of `out` are written, so pass a zeroed `out`
       (or ignore the padded rows).  Either may be None (0 / L).
       fp8: q/k/pos_* are torch.float8_e4m3fn with float32 per-head scales; v is bfloat16.  At head_dim 64 the
       three score products are e4m3 MFMA contractions over the whole head_dim (far / near pair of launches; the
       far tiles fold Q_r[delta] into the query and round that sum to e4m3 once more); other head_dims and
       single_kernel=True take the one-kernel e4m3 path.
       single_kernel=True withholds the log-sum-exp buffer, which makes the library walk all key tiles in
       one kernel instead of the far-tile / near-tile pair of launches (same result; for comparison).
       far_splits, near_splits: workgroups that share the far / the near keys of a query tile (0: the library
       decides from the size of the launch; it matters for launches that do not fill the GPU, e.g. one sequence).
       workspace: a uint8 GPU tensor for the partial results of such shared launches, to reuse one buffer across
       calls; by default one of the size the library asks for is allocated per call.  A smaller one is fine: the
       library then shares less.
       no_alloc=True goes through fdb_attn_fwd_noalloc: the log-sum-exp hand-over, the work-list of a packed
       call and the partial results come from the scratch built into the library (one per GPU; calls on one
       GPU must not overlap), so with `out` given nothing is allocated on the way; single_kernel is not
       available there.
    """
    if not q.is_cuda:
        raise RuntimeError("disentangled_attention_fwd runs on the GPU only; got device %s" % q.device)
    varlen = cu_seqlens is not None
    if varlen:
        if q.dim() != 3:
            raise ValueError("with cu_seqlens, q/k/v must be [T, H, D]")
        T, H, D = q.shape
        B = cu_seqlens.numel() - 1
        L = int(max_seqlen) if max_seqlen is not None else T
        if cu_seqlens.dtype != torch.int32 or not cu_seqlens.is_cuda:
            raise ValueError("cu_seqlens must be an int32 tensor on the GPU")
    else:
        if q.dim() != 4:
            raise ValueError("q/k/v must be [B, L, H, D] (or [T, H, D] with cu_seqlens)")
        B, L, H, D = q.shape
        T = B * L
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k, v must have the same shape (self-attention): %s %s %s"
                         % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    fp8 = q.dtype == _FP8
    if fp8:
        if k.dtype != _FP8 or v.dtype != torch.bfloat16:
            raise ValueError("fp8 path: q and k float8_e4m3fn, v bfloat16")
        if q_scale is None or k_scale is None or (pos_key is not None and pos_key_scale is None) or (
                pos_query is not None and pos_query_scale is None):
            raise ValueError("fp8 path: q_scale, k_scale and a scale for each position tensor are required")
        dt = _lib.FDB_FP8_E4M3
    else:
        if q.dtype not in _DTYPES or k.dtype != q.dtype or v.dtype != q.dtype:
            raise ValueError("unsupported dtypes %s %s %s" % (q.dtype, k.dtype, v.dtype))
        dt = _DTYPES[q.dtype]
    q, k, v = [x if x.stride(-1) == 1 else x.contiguous() for x in (q, k, v)]
    span = att_span(position_buckets, max_relative_positions)
    pos_key = _pos_arg(pos_key, H, D, span, "pos_key")
    pos_query = _pos_arg(pos_query, H, D, span, "pos_query")
    for pname, x in (("pos_key", pos_key), ("pos_query", pos_query)):
        if x is not None and x.dtype != q.dtype:
            raise ValueError("%s dtype %s does not match q dtype %s" % (pname, x.dtype, q.dtype))
    n_terms = 1 + (pos_key is not None) + (pos_query is not None)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D * n_terms)

    a = FdbAttnArgs()
    keep = []
    if pos_key is not None or pos_query is not None:
        lut, radius = delta_lut_device(position_buckets, max_relative_positions, q.device)
        a.delta_lut, a.lut_radius, a.att_span = lut.data_ptr(), radius, span
    if out is None:
        out = torch.empty(q.shape, dtype=v.dtype, device=q.device)
    elif out.shape != q.shape or out.dtype != v.dtype or out.stride(-1) != 1:
        raise ValueError("out must have q's shape, v's dtype and a unit stride on D")
    # the log-sum-exp buffer is also the hand-over between the far-tile and near-tile launches, so it is
    # always provided when a position term is present (T*H floats)
    if no_alloc and (single_kernel or workspace is not None):
        raise ValueError("no_alloc excludes single_kernel and a caller-owned workspace")
    want_lse = return_lse or ((pos_key is not None or pos_query is not None) and not single_kernel and not no_alloc)
    lse = torch.empty((T, H), dtype=torch.float32, device=q.device) if want_lse else None
    a.q, a.k, a.v, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.pos_key, a.pos_query = (_ptr(pos_key) or ctypes.c_void_p()).value, (_ptr(pos_query) or ctypes.c_void_p()).value
    a.lse = lse.data_ptr() if lse is not None else None
    if varlen:
        for n, x in (("q", q), ("k", k), ("v", v), ("o", out)):
            setattr(a, n + "_stride_b", 0)
            setattr(a, n + "_stride_t", x.stride(0))
            setattr(a, n + "_stride_h", x.stride(1))
        a.cu_seqlens = cu_seqlens.data_ptr()
        if not no_alloc:
            wl = torch.empty(int(lib.fdb_worklist_ints(T, B)), dtype=torch.int32, device=q.device)
            keep.append(wl)
            check(lib.fdb_build_worklist(_ptr(cu_seqlens), B, T, _ptr(wl), _stream_ptr(q.device)), "fdb_build_worklist")
            a.worklist = wl.data_ptr()
    else:
        for n, x in (("q", q), ("k", k), ("v", v), ("o", out)):
            setattr(a, n + "_stride_b", x.stride(0))
            setattr(a, n + "_stride_t", x.stride(1))
            setattr(a, n + "_stride_h", x.stride(2))
        for n, x in (("seq_start", seq_start), ("seq_len", seq_len)):
            if x is not None:
                if x.dtype != torch.int32 or not x.is_cuda or x.numel() != B:
                    raise ValueError("%s must be an int32 GPU tensor with one entry per batch row" % n)
                x = x.contiguous()
                keep.append(x)
                setattr(a, n, x.data_ptr())
    if pos_key is not None:
        a.pk_stride_h, a.pk_stride_r = pos_key.stride(0), pos_key.stride(1)
    if pos_query is not None:
        a.pq_stride_h, a.pq_stride_r = pos_query.stride(0), pos_query.stride(1)
    if fp8:
        scales = {"q_scale": q_scale, "k_scale": k_scale, "pk_scale": pos_key_scale, "pq_scale": pos_query_scale}
        for n, s in scales.items():
            if s is not None:
                if s.dtype != torch.float32 or s.numel() != H or not s.is_cuda:
                    raise ValueError("%s must be a float32 GPU tensor with one entry per head" % n)
                s = s.contiguous()
                keep.append(s)
                setattr(a, n, s.data_ptr())
    a.batch, a.heads, a.head_dim, a.max_seqlen, a.total_tokens = B, H, D, L, T
    a.dtype, a.causal, a.sm_scale, a.far_splits = dt, int(bool(causal)), float(sm_scale), int(far_splits)
    a.near_splits = int(near_splits)
    with torch.cuda.device(q.device):
        if no_alloc:
            check(lib.fdb_attn_fwd_noalloc(ctypes.byref(a), _stream_ptr(q.device)), "fdb_attn_fwd_noalloc")
            return (out, lse) if return_lse else out
        if workspace is not None:
            if workspace.dtype != torch.uint8 or not workspace.is_cuda or not workspace.is_contiguous():
                raise ValueError("workspace must be a contiguous uint8 GPU tensor")
            if workspace.numel() > 0:
                a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        else:
            ws_bytes = lib.fdb_attn_workspace_bytes(ctypes.byref(a))
            if ws_bytes > 0:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
                keep.append(ws)
                a.workspace, a.workspace_bytes = ws.data_ptr(), ws_bytes
        if _part:  # measurement only (bench.py): 1 = the far launch alone, 2 = the near launch alone; `out` is then no result
            check(lib.fdb_attn_fwd_part(ctypes.byref(a), int(_part), _stream_ptr(q.device)), "fdb_attn_fwd_part")
        else:
            check(lib.fdb_attn_fwd(ctypes.byref(a), _stream_ptr(q.device)), "fdb_attn_fwd")
    return (out, lse) if return_lse else out


def _scores_f32(x, pos_t):
    """Batched x [H, N, K] . pos_t [H, K, M] -> fp32 [H, N, M].  16-bit operands go through the GEMM as they are, with
    an fp32 result (exactly what converting them first would give, at half the traffic), where torch offers that."""
    if x.dtype != torch.float32:
        try:
            return torch.bmm(x, pos_t.to(x.dtype), out_dtype=torch.float32)
        except (TypeError, RuntimeError, NotImplementedError):
            pass
    return torch.bmm(x.to(torch.float32), pos_t.to(torch.float32))


def attention_bwd_kernels(q, k, v, dout, lse, *, out=None, delta=None, c2p=None, p2c=None, d_c2p=None, d_p2c=None, sm_scale,
                          position_buckets=0, max_relative_positions=0, causal=False, seq_start=None, seq_len=None,
                          dq_out=None, dk_out=None):
    """The two backward launches (fdb_attn_bwd) on tensors the caller made: q, k, v, dout [B, L, H, D]; lse [B*L, H];
    either `out` (the forward's output; the call then computes delta itself) or `delta` [B*L, H] fp32; the position
    scores c2p = q . K_r^T / p2c = k . Q_r^T and their gradient tensors (cleared by the caller if the batch is padded: the
    kernels store every entry of a real token's row and leave rows of padding alone) as views of logical shape
    [B, L, H, 2S] with a unit stride on the last axis and any memory layout behind it (all four the same, in q's
    element type).  Returns dq, dk, dv (content part) and leaves the score gradients in d_c2p / d_p2c.
    dq_out / dk_out: where to write dq / dk instead of a fresh tensor, views of logical shape [B, L, H, D] in q's type with
    a unit stride on the last axis and rows aligned to 16 bytes (cleared by the caller if the batch is padded)."""
    B, L, H, D = q.shape
    span = att_span(position_buckets, max_relative_positions)
    q, k, v, dout = [x if x.stride(-1) == 1 else x.contiguous() for x in (q, k, v, dout)]
    a = _lib.FdbAttnBwdArgs()
    f32 = torch.float32
    scores = [x for x in (c2p, p2c, d_c2p, d_p2c) if x is not None]
    if scores:
        lut, radius = delta_lut_device(position_buckets, max_relative_positions, q.device)
        a.delta_lut, a.lut_radius, a.att_span = lut.data_ptr(), radius, span
        a.lut_window = delta_lut_window(position_buckets, max_relative_positions)
        if a.lut_window > _lib.FDB_BWD_MAX_WINDOW:
            raise ValueError("backward: position_buckets=%d, max_relative_positions=%d map 32 consecutive relative positions onto "
                             "%d table rows; the score-gradient window of the kernels holds %d (use the eager implementation "
                             "for training with this configuration)"
                             % (position_buckets, max_relative_positions, a.lut_window + 1, _lib.FDB_BWD_MAX_WINDOW + 1))
        st = scores[0].stride()
        for x in scores:
            if tuple(x.shape) != (B, L, H, 2 * span) or x.stride() != st or st[3] != 1 or x.dtype != q.dtype:
                raise ValueError("position-score tensors: views of shape [B, L, H, 2S] = %s with one layout and q's element type"
                                 % ((B, L, H, 2 * span),))
        a.bias_stride_b, a.bias_stride_t, a.bias_stride_h = st[0], st[1], st[2]
    if c2p is not None:
        a.c2p_bias, a.d_c2p_bias = c2p.data_ptr(), d_c2p.data_ptr()
    if p2c is not None:
        a.p2c_bias, a.d_p2c_bias = p2c.data_ptr(), d_p2c.data_ptr()
    if delta is None:
        out = out if out.stride(-1) == 1 else out.contiguous()
        delta = torch.empty((B * L, H), dtype=f32, device=q.device)  # dO . O per row: the dQ launch fills it
    else:
        out, delta = None, delta.to(f32).reshape(B * L, H).contiguous()
    lse = lse.contiguous()
    padded = seq_start is not None or seq_len is not None
    alloc = torch.zeros if padded else torch.empty
    for name, x in (("dq_out", dq_out), ("dk_out", dk_out)):
        if x is not None and (tuple(x.shape) != (B, L, H, D) or x.stride(3) != 1 or x.dtype != q.dtype or x.device != q.device):
            raise ValueError("%s: a view of shape [B, L, H, D] = %s in q's element type with a unit last stride" % (name, (B, L, H, D)))
    dq, dk, dv = [x if x is not None else alloc((B, L, H, D), dtype=q.dtype, device=q.device) for x in (dq_out, dk_out, None)]
    a.q, a.k, a.v, a.dout = q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr()
    a.dq, a.dk, a.dv, a.lse, a.delta = dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), lse.data_ptr(), delta.data_ptr()
    a.out = None if out is None else out.data_ptr()
    for n, x in (("q", q), ("k", k), ("v", v), ("do", dout), ("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        if x is None:
            continue
        setattr(a, n + "_stride_b", x.stride(0))
        setattr(a, n + "_stride_t", x.stride(1))
        setattr(a, n + "_stride_h", x.stride(2))
    keep = []
    for n, x in (("seq_start", seq_start), ("seq_len", seq_len)):
        if x is not None:
            x = x.contiguous()
            keep.append(x)
            setattr(a, n, x.data_ptr())
    a.batch, a.heads, a.head_dim, a.seqlen = B, H, D, L
    a.dtype, a.causal, a.sm_scale = _DTYPES[q.dtype], int(bool(causal)), float(sm_scale)
    with torch.cuda.device(q.device):
        check(lib.fdb_attn_bwd(ctypes.byref(a), _stream_ptr(q.device)), "fdb_attn_bwd")
    return dq, dk, dv


def chain_through_tables(d_scores, x, pos, dx, x_second=None, dx_second=None):
    """dx += d_scores . pos in place and returns d_scores^T . x (fp32), both from one pass over d_scores
    (fdb_attn_bwd_chain): d_scores [M, N, 2S] and pos [M, 2S, D] contiguous; the token rows x [M, N, D] and the rows dx
    [M, N, D] they belong to with any matrix and row stride and a unit last stride -- or x / dx [M1, N, D] and
    x_second / dx_second [M - M1, N, D] with the same strides, so that q, k, dq and dk are read and updated where they
    lie.  One 16-bit element type.  M: (head, term) pairs, N: token rows.  Counterpart of the autograd backward of the
    reference's bias GEMMs (model.py:189-192).  chain_through_tables_ok says whether the kernel is built for a shape."""
    M, N, two_s = d_scores.shape
    D = dx.shape[2]
    m1 = x.shape[0]
    for t, shape in ((d_scores, (M, N, two_s)), (pos, (M, two_s, D))):
        if tuple(t.shape) != shape or not t.is_contiguous() or t.dtype != d_scores.dtype or t.device != d_scores.device:
            raise ValueError("chain_through_tables: contiguous d_scores [M, N, 2S] and pos [M, 2S, D] of one type on one device")
    xs = [x] if x_second is None else [x, x_second]
    dxs = [dx] if dx_second is None else [dx, dx_second]
    for name, ts in (("x", xs), ("dx", dxs)):
        if (len(ts) != len(xs) or [t.shape[0] for t in ts] != [t.shape[0] for t in xs] or sum(t.shape[0] for t in ts) != M
                or any(tuple(t.shape[1:]) != (N, D) or t.dtype != d_scores.dtype or t.device != d_scores.device for t in ts)):
            raise ValueError("chain_through_tables: %s (and %s_second) hold the M matrices of [N, D] in the type of d_scores" % (name, name))
    aligned = lambda ts: not any(t.stride(2) != 1 or t.stride() != ts[0].stride() or (t.stride(0) * t.element_size()) % 16
                                 or (t.stride(1) * t.element_size()) % 16 or t.data_ptr() % 16 for t in ts)
    if not aligned(xs):
        xs = [t.contiguous() for t in xs]   # one layout for both, rows and matrices at multiples of 16 bytes
    if not aligned(dxs):
        raise ValueError("chain_through_tables: dx (and dx_second) share one layout with a unit last stride, rows and matrices at multiples of 16 bytes")
    if not chain_through_tables_ok(d_scores.dtype, D, two_s // 2, N):
        raise ValueError("chain_through_tables: built for 16-bit types, head_dim 64, 2S = 512 and a multiple of 32 rows")
    cus = torch.cuda.get_device_properties(d_scores.device).multi_processor_count
    parts = max(1, min(N // 32, cus // M))   # one workgroup per CU: as many shares of the rows as fill the GPU once
    dpos_parts = torch.empty((parts, M, two_s, D), dtype=torch.float32, device=d_scores.device)
    second = lambda ts: ts[1].data_ptr() if len(ts) > 1 else None
    with torch.cuda.device(d_scores.device):
        check(lib.fdb_attn_bwd_chain(d_scores.data_ptr(), xs[0].data_ptr(), second(xs), pos.data_ptr(), dxs[0].data_ptr(), second(dxs),
                                     dpos_parts.data_ptr(), M, m1, N, xs[0].stride(0), xs[0].stride(1), dxs[0].stride(0), dxs[0].stride(1),
                                     two_s // 2, D, _DTYPES[d_scores.dtype], parts, _stream_ptr(d_scores.device)), "fdb_attn_bwd_chain")
    return dpos_parts.sum(0) if parts > 1 else dpos_parts[0]


def chain_through_tables_ok(dtype, head_dim, span, rows):
    return dtype in (torch.bfloat16, torch.float16) and head_dim == 64 and span == 256 and rows >= 32 and rows % 32 == 0


def disentangled_attention_bwd(q, k, v, out, lse, dout, pos_key=None, pos_query=None, *, sm_scale=None, position_buckets=0,
                               max_relative_positions=0, causal=False, seq_start=None, seq_len=None, delta=None, fused_chain=None):
    """Backward of the fixed layout: q, k, v, out, dout [B, L, H, D], lse [B*L, H] as the forward returns it,
    pos_key = K_r / pos_query = Q_r [H, 2S, D] or None  ->  (dq, dk, dv, d pos_key, d pos_query).
    Counterpart of FlashAttentionDisentangled.backward (reference flash_attention.py:1066-1086), which hands
    flash_attn_v2_bwd_dise the position-score tensors and gets their gradients back; as there, those tensors
    are two GEMMs around the kernel (here head-major [H, B*L, 2S]) and the chain through K_r / Q_r and back into
    q / k is four more.  delta: (dout * out).sum(-1) as fp32 [B*L, H] if the caller has it (then `out` is not
    read); by default the first launch computes it.  Where the chain kernel does not serve the shape, dq / dk of a side
    with a position term come back as the [B, L, H, D] view of head-major memory (see below); otherwise contiguous.  fused_chain: None takes the one-pass
    chain kernel (chain_through_tables) where it is built for the shape, False the two GEMMs, True insists on the kernel."""
    B, L, H, D = q.shape
    if q.dtype not in _DTYPES:
        raise ValueError("unsupported dtype %s" % q.dtype)
    span = att_span(position_buckets, max_relative_positions)
    pos_key = _pos_arg(pos_key, H, D, span, "pos_key")
    pos_query = _pos_arg(pos_query, H, D, span, "pos_query")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D * (1 + (pos_key is not None) + (pos_query is not None)))
    q, k, v, dout = [x if x.stride(-1) == 1 else x.contiguous() for x in (q, k, v, dout)]
    f32 = torch.float32
    c2p = p2c = d_c2p = d_p2c = None
    # Position scores and their gradients are head-major, [H, B*L, 2S] in the inputs' type: what a batched GEMM over the heads
    # writes and reads as it stands (a token-major tensor would cost a transposing copy of it each way).
    heads_first = lambda x: x.permute(2, 0, 1, 3).reshape(H, B * L, D)  # a view of [B, L, H, D] when that is contiguous
    both = pos_key is not None and pos_query is not None
    # the kernels store every entry of a real token's row of the score gradients; only rows of padding need clearing
    like = torch.zeros_like if (seq_start is not None or seq_len is not None) else torch.empty_like
    if both:
        # both terms: their score tensors stacked, [2H, B*L, 2S], so that the chain back through the tables is one call
        # over 2H matrices; the scores themselves are two GEMMs that read q and k where they lie (a stacked copy of
        # q and k plus one GEMM over 2H matrices took 339 against 236 us at the bench shape)
        pos2 = torch.stack([pos_key[:, :2 * span], pos_query[:, :2 * span]]).view(2 * H, 2 * span, D).to(q.dtype)
        scores2 = torch.empty((2 * H, B * L, 2 * span), dtype=q.dtype, device=q.device)   # (q . K_r^T, k . Q_r^T), in the inputs' type like the reference's
        torch.bmm(heads_first(q), pos2[:H].transpose(1, 2), out=scores2[:H])
        torch.bmm(heads_first(k), pos2[H:].transpose(1, 2), out=scores2[H:])
        d_scores2 = like(scores2)
        c2p, p2c, d_c2p, d_p2c = scores2[:H], scores2[H:], d_scores2[:H], d_scores2[H:]
    elif pos_key is not None:
        c2p = torch.bmm(heads_first(q), pos_key[:, :2 * span].transpose(1, 2).to(q.dtype))
        d_c2p = like(c2p)
    elif pos_query is not None:
        p2c = torch.bmm(heads_first(k), pos_query[:, :2 * span].transpose(1, 2).to(k.dtype))
        d_p2c = like(p2c)
    blhs = lambda x: None if x is None else x.view(H, B, L, 2 * span).permute(1, 2, 0, 3)  # the logical [B, L, H, 2S] view
    # The chain of the score gradients back through K_r / Q_r adds its product onto dq / dk in place (fp32 accumulation
    # over the kernel's content part, one rounding; no fp32 copy of the product and no passes to add and convert it):
    # the chain kernel where they lie, the GEMM that stands in for it on a head-major [H, B*L, D] copy-free layout of
    # its own, which the backward launches write and of which the caller gets the logical [B, L, H, D] view.
    fused = chain_through_tables_ok(q.dtype, D, span, B * L) if fused_chain is None else bool(fused_chain)
    x_hm = dq_out = dk_out = None
    if not fused and (pos_key is not None or pos_query is not None):
        new_x = torch.zeros if like is torch.zeros_like else torch.empty
        x_hm = new_x((2 if both else 1, H, B * L, D), dtype=q.dtype, device=q.device)
        blhd = lambda x: x.view(H, B, L, D).permute(1, 2, 0, 3)
        dq_out = blhd(x_hm[0]) if pos_key is not None else None
        dk_out = blhd(x_hm[1 if both else 0]) if pos_query is not None else None
    dq, dk, dv = attention_bwd_kernels(q, k, v, dout, lse, out=out, delta=delta, c2p=blhs(c2p), p2c=blhs(p2c), d_c2p=blhs(d_c2p),
                                       d_p2c=blhs(d_p2c), sm_scale=sm_scale, position_buckets=position_buckets,
                                       max_relative_positions=max_relative_positions, causal=causal, seq_start=seq_start, seq_len=seq_len,
                                       dq_out=dq_out, dk_out=dk_out)
    dpk = dpq = None

    def into_pos(d_scores, xh, pos):  # [H', B*L, 2S]^T . [H', B*L, D] -> [H', 2S, D]: a reduction over the tokens
        n_mat, n_tok = d_scores.shape[0], d_scores.shape[1]
        parts = 8 if n_tok % 8 == 0 and n_tok >= 4096 else 1  # few output tiles: split the tokens, add the parts
        if parts > 1:
            dpos = _scores_f32(d_scores.view(n_mat, parts, n_tok // parts, 2 * span).transpose(2, 3).reshape(n_mat * parts, 2 * span, n_tok // parts),
                               xh.reshape(n_mat * parts, n_tok // parts, D)).view(n_mat, parts, 2 * span, D).sum(1)
        else:
            dpos = _scores_f32(d_scores.transpose(1, 2), xh)
        return dpos

    def pad_rows(dpos, pos):  # rows past 2S take no part
        dpos = dpos.to(pos.dtype)
        if pos.shape[1] > 2 * span:
            dpos = torch.cat([dpos, dpos.new_zeros(H, pos.shape[1] - 2 * span, D)], dim=1)
        return dpos

    # score = x . pos[delta]: both factors get their share -- in one pass over the score gradients where the chain
    # kernel is built for the shape, else as two GEMMs (the first adds onto dq / dk in place)
    if both:
        if fused:
            in_place = lambda x: x.permute(2, 0, 1, 3).view(H, B * L, D)   # a view or an error, never a copy: the kernel writes through it
            dpos2 = chain_through_tables(d_scores2, heads_first(q), pos2, in_place(dq), x_second=heads_first(k), dx_second=in_place(dk))
        else:
            x_hm.view(2 * H, B * L, D).baddbmm_(d_scores2, pos2)  # (dq, dk) += (d c2p . K_r, d p2c . Q_r)
            # the reduction over the tokens has few output tiles: one call over 2H matrices, on a stacked copy of q and k
            dpos2 = into_pos(d_scores2, torch.stack([heads_first(q), heads_first(k)]).view(2 * H, B * L, D), None)
        dpk, dpq = pad_rows(dpos2[:H], pos_key), pad_rows(dpos2[H:], pos_query)
    elif pos_key is not None or pos_query is not None:
        pos, x, dx, d_s = (pos_key, q, dq, d_c2p) if pos_key is not None else (pos_query, k, dk, d_p2c)
        pos_t = pos[:, :2 * span].to(q.dtype)
        if fused:
            dpos = chain_through_tables(d_s, heads_first(x), pos_t.contiguous(), dx.permute(2, 0, 1, 3).view(H, B * L, D))
        else:
            x_hm[0].baddbmm_(d_s, pos_t)
            dpos = into_pos(d_s, heads_first(x), None)
        dpk, dpq = (pad_rows(dpos, pos_key), None) if pos_key is not None else (None, pad_rows(dpos, pos_query))
    return dq, dk, dv, dpk, dpq


class _DisentangledAttention(torch.autograd.Function):
    """Fused forward + the backward above as one autograd node (fixed layout).  Counterpart of the reference's
    FlashAttentionDisentangled (flash_attention.py:1032-1086)."""

    @staticmethod
    def forward(ctx, kwargs, q, k, v, pos_key, pos_query):
        out, lse = disentangled_attention_fwd(q, k, v, pos_key, pos_query, return_lse=True, **kwargs)
        ctx.save_for_backward(q, k, v, out, lse, *(x for x in (pos_key, pos_query) if x is not None))
        ctx.cfg = (kwargs, pos_key is not None, pos_query is not None)
        return out

    @staticmethod
    def backward(ctx, dout):
        kwargs, has_pk, has_pq = ctx.cfg
        q, k, v, out, lse = ctx.saved_tensors[:5]
        pk = ctx.saved_tensors[5] if has_pk else None
        pq = ctx.saved_tensors[5 + has_pk] if has_pq else None
        kw = {n: kwargs[n] for n in ("sm_scale", "position_buckets", "max_relative_positions", "causal", "seq_start", "seq_len")
              if n in kwargs}
        dq, dk, dv, dpk, dpq = disentangled_attention_bwd(q, k, v, out, lse, dout, pk, pq, **kw)
        # a position tensor handed in as [1, H, 2S, D] takes its gradient in that shape
        dpk = dpk if dpk is None else dpk.reshape(pk.shape)
        dpq = dpq if dpq is None else dpq.reshape(pq.shape)
        return None, dq, dk, dv, dpk, dpq


class _ForwardOnly(torch.autograd.Function):
    """The fused forward as an autograd node whose backward raises: a graph that runs through a variant
    without a backward fails loudly at .backward() instead of silently dropping the gradients of everything
    before it (the reference's packed op does the same, flash_attention_varlen.py:480-483)."""

    @staticmethod
    def forward(ctx, kwargs, q, k, v, pos_key, pos_query):
        return disentangled_attention_fwd(q, k, v, pos_key, pos_query, **kwargs)

    @staticmethod
    def backward(ctx, *grads):
        raise RuntimeError("this variant of the fused disentangled attention is forward-only (packed layout and FP8 "
                           "operands have no backward); use the fixed layout or the eager implementation")


_BWD_KW = {"sm_scale", "position_buckets", "max_relative_positions", "causal", "seq_start", "seq_len", "out", "far_splits",
           "near_splits", "workspace"}


def disentangled_attention(q, k, v, pos_key=None, pos_query=None, **kwargs):
    """disentangled_attention_fwd (single output) for callers that may run under autograd: with gradients
    required, the fixed layout in fp32 / bf16 / fp16 is differentiable (dq, dk, dv, d pos_key, d pos_query);
    the packed layout and FP8 operands become a node whose backward raises."""
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in (q, k, v, pos_key, pos_query)):
        differentiable = q.dim() == 4 and q.dtype in _DTYPES and set(kwargs) <= _BWD_KW
        return (_DisentangledAttention if differentiable else _ForwardOnly).apply(kwargs, q, k, v, pos_key, pos_query)
    return disentangled_attention_fwd(q, k, v, pos_key, pos_query, **kwargs)



def flash_attention_with_disentangled(q, k, v, k_pos, q_pos, causal=False, sm_scale=None,
                                      position_buckets=0, max_relative_distance=0):
    """Same call shape as the reference op (flash_attention.py:1088-1091): q, k, v [B, H, L, D],
    returns [B, H, L, D].  k_pos / q_pos are K_r / Q_r [H, 2S, D] (see the module docstring).
    As in the reference, sm_scale=None means 1/sqrt(D) (flash_attention.py:1042-1043), and the op is
    differentiable like FlashAttentionDisentangled.apply (flash_attention.py:1032-1086): gradients reach
    q, k, v, k_pos and q_pos."""
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    o = disentangled_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), k_pos, q_pos,
                               sm_scale=sm_scale, position_buckets=position_buckets,
                               max_relative_positions=max_relative_distance, causal=causal)
    return o.transpose(1, 2)


def flash_attention_with_disentangled_varlen(q, k, v, q_pos, k_pos, cu_seqlens_q, cu_seqlens_k,
                                             max_seqlen_q, max_seqlen_k, causal=False, sm_scale=None,
                                             position_buckets=0, max_relative_distance=0):
    """Same call shape as the reference op (flash_attention_varlen.py:485-511): q, k, v [T, H, D].
    Positional order follows the reference: the 4th argument feeds the content->position term
    (K_r), the 5th the position->content term (Q_r) (flash_attention_varlen.py:445,470).
    Self-attention only: cu_seqlens_q must equal cu_seqlens_k.  Forward-only like the reference's packed op:
    under autograd it is a node whose backward raises (flash_attention_varlen.py:480-483)."""
    if cu_seqlens_q is not cu_seqlens_k and not torch.equal(cu_seqlens_q, cu_seqlens_k):
        raise ValueError("self-attention only: cu_seqlens_q and cu_seqlens_k must match")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    return disentangled_attention(q, k, v, q_pos, k_pos, cu_seqlens=cu_seqlens_q.to(torch.int32),
                                  max_seqlen=max(int(max_seqlen_q), int(max_seqlen_k)), sm_scale=sm_scale,
                                  position_buckets=position_buckets,
                                  max_relative_positions=max_relative_distance, causal=causal)


def quantize_e4m3_per_head(x):
    """x: bf16 [..., H, D] on the GPU -> (float8_e4m3fn tensor of the same shape, float32 scales [H]);
    scale[h] = max(absmax over everything but h, 1e-12) / 448, y = e4m3_rne(x / scale[h])."""
    if not x.is_cuda or x.dtype != torch.bfloat16:
        raise ValueError("quantize_e4m3_per_head expects a bfloat16 GPU tensor")
    H, D = x.shape[-2], x.shape[-1]
    x3 = x.reshape(-1, H, D)
    if x3.stride(2) != 1:
        x3 = x3.contiguous()
    y = torch.empty(x3.shape, dtype=torch.uint8, device=x.device)
    scale = torch.empty(H, dtype=torch.float32, device=x.device)
    ws = torch.empty(H, dtype=torch.int32, device=x.device)
    with torch.cuda.device(x.device):
        check(lib.fdb_quant_e4m3_per_head(_ptr(x3), x3.stride(0), x3.stride(1), _ptr(y), y.stride(0), y.stride(1),
                                          _ptr(scale), _ptr(ws), x3.shape[0], H, D, _stream_ptr(x.device)),
              "fdb_quant_e4m3_per_head")
    return y.view(_FP8).reshape(x.shape), scale


def quantize_e4m3_per_head_pair(x0, x1):
    """quantize_e4m3_per_head for two bf16 tensors of one shape and one set of strides (q and k of a layer, K_r and
    Q_r) in the same three launches -> (y0, scale0, y1, scale1).  Tensors whose layouts differ are made contiguous."""
    for x in (x0, x1):
        if not x.is_cuda or x.dtype != torch.bfloat16:
            raise ValueError("quantize_e4m3_per_head_pair expects bfloat16 GPU tensors")
    if x0.shape != x1.shape:
        raise ValueError("quantize_e4m3_per_head_pair: shapes differ: %s %s" % (tuple(x0.shape), tuple(x1.shape)))
    H, D = x0.shape[-2], x0.shape[-1]
    a, b = x0.reshape(-1, H, D), x1.reshape(-1, H, D)
    if a.stride() != b.stride() or a.stride(2) != 1:
        a, b = a.contiguous(), b.contiguous()
    y = torch.empty((2,) + tuple(a.shape), dtype=torch.uint8, device=a.device)
    scale = torch.empty((2, H), dtype=torch.float32, device=a.device)
    ws = torch.empty(2 * H, dtype=torch.int32, device=a.device)
    with torch.cuda.device(a.device):
        check(lib.fdb_quant_e4m3_per_head_pair(_ptr(a), _ptr(b), a.stride(0), a.stride(1), _ptr(y[0]), _ptr(y[1]), y.stride(1), y.stride(2),
                                               _ptr(scale[0]), _ptr(scale[1]), _ptr(ws), a.shape[0], H, D, _stream_ptr(a.device)),
              "fdb_quant_e4m3_per_head_pair")
    return y[0].view(_FP8).reshape(x0.shape), scale[0], y[1].view(_FP8).reshape(x1.shape), scale[1]


def dequantize_e4m3_per_head(y, scale):
    """y: float8_e4m3fn [..., H, D] on the GPU, scale float32 [H] -> bfloat16 tensor of the same shape,
    x = bf16_rne(y * scale[h])."""
    if not y.is_cuda or y.dtype != _FP8:
        raise ValueError("dequantize_e4m3_per_head expects a float8_e4m3fn GPU tensor")
    H, D = y.shape[-2], y.shape[-1]
    if scale.dtype != torch.float32 or scale.numel() != H or not scale.is_cuda:
        raise ValueError("scale must be a float32 GPU tensor with one entry per head")
    y3 = y.reshape(-1, H, D)
    if y3.stride(2) != 1:
        y3 = y3.contiguous()
    x = torch.empty(y3.shape, dtype=torch.bfloat16, device=y.device)
    with torch.cuda.device(y.device):
        check(lib.fdb_dequant_e4m3_per_head(_ptr(y3), y3.stride(0), y3.stride(1), _ptr(scale.contiguous()), _ptr(x),
                                            x.stride(0), x.stride(1), y3.shape[0], H, D, _stream_ptr(y.device)),
              "fdb_dequant_e4m3_per_head")
    return x.reshape(y.shape)

