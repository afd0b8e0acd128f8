"""Drop-in attention module and the `_attn_implementation` switch.

Counterparts in the reference (src/flashdeberta/model.py):
  FlashDisentangledSelfAttention   :97-252   same constructor, parameters and forward signature
  DEBERTA_SELF_ATTENTION_CLASSES   :254-257  {"eager", "flash_attention_2"}
  FlashDebertaV2Model              :394-496  here a thin subclass of transformers' DebertaV2Model
The eager entry is transformers' own DisentangledSelfAttention, exactly as in the reference.
Differentiable like the reference's fixed-length op (padded batches included: they stay in the fixed layout
here); attention-probability dropout is not applied (nor is it on the reference's flash path: only the dropout
on the relative embeddings remains, model.py:159-160).
"""
import math
import weakref

import torch
import torch.nn.functional as F
from transformers.models.deberta_v2.modeling_deberta_v2 import (
    DebertaV2Config,
    DebertaV2Encoder,
    DebertaV2Model,
    DisentangledSelfAttention,
)

from . import ops
from .padding import key_padding_mask, seq_bounds


def _stamp(t):
    """What a remembered value depends on besides the tensor object: its in-place version counter, and the
    storage, dtype and device behind it (`p.data = x`, `module.to(dtype)` and `.half()` swap those under
    an unchanged object and version)."""
    return (t._version, t.data_ptr(), t.dtype, t.device)


class _Memo:
    """One remembered value, valid while the tensors it was computed from are the same objects, have not
    been written in place, still sit in the same storage with the same dtype on the same device, and
    `extra` compares equal.  The tensors are held weakly."""

    def __init__(self):
        self._state = ((), (), None, None)  # (weak references, stamps, extra, value): replaced as a whole, read once

    def get(self, tensors, extra=None):
        refs, stamps, old_extra, value = self._state
        if len(refs) != len(tensors) or extra != old_extra:
            return None
        for ref, stamp, t in zip(refs, stamps, tensors):
            if ref() is not t or _stamp(t) != stamp:
                return None
        return value

    def put(self, tensors, value, extra=None):
        self._state = (tuple(weakref.ref(t) for t in tensors), tuple(_stamp(t) for t in tensors), extra, value)
        return value

    def __reduce__(self):  # copies and pickles of a module start with nothing remembered
        return (_Memo, ())


def _seq_bounds_of(attention_mask, memo):
    """(seq_start, seq_len) of a mask.  Every layer of an encoder receives the same mask object, so the
    reductions run once per forward instead of once per layer: `memo` (a _Memo that the layers of a patched
    model share, see patch_model) holds the result for as long as the mask is the same object, unwritten and
    in place.  Nothing is stored on the caller's tensor and nothing is process-global."""
    hit = memo.get((attention_mask,))
    if hit is None:
        start, length, _ = seq_bounds(key_padding_mask(attention_mask))
        hit = memo.put((attention_mask,), (start, length))
    return hit


class FlashDisentangledSelfAttention(DisentangledSelfAttention):
    """Same parameters as the eager module (query_proj, key_proj, value_proj[, pos_key_proj,
    pos_query_proj]), so `load_state_dict(eager.state_dict())` works (reference tests/attention.py:60).

    fp8_qk=True quantises Q, K and the projected relative embeddings to OCP e4m3 with per-head
    absmax scales before the kernel (bf16 inputs only).

    Outside training the three input projections run as one GEMM over the concatenated weights
    (a copy kept per module, rebuilt when a parameter is replaced or written in place), and K_r / Q_r
    are remembered for as long as the relative embeddings handed in are the same tensor (an encoder
    patched by `patch_model` hands in the same tensor until its embedding table changes)."""

    def __init__(self, config, fp8_qk=None):
        super().__init__(config)
        self.fp8_qk = bool(getattr(config, "fp8_qk", False)) if fp8_qk is None else bool(fp8_qk)
        self._qkv_memo, self._pos_memo, self._mask_memo, self._pos8_memo = _Memo(), _Memo(), _Memo(), _Memo()

    def _fused_qkv(self):
        """Concatenated [3*H*D, hidden] weight and bias of the query, key and value projections."""
        projs = (self.query_proj, self.key_proj, self.value_proj)
        params = tuple(p.weight for p in projs) + tuple(p.bias for p in projs if p.bias is not None)
        if len(params) not in (3, 6):
            return None
        hit = self._qkv_memo.get(params)
        if hit is None:
            with torch.no_grad():
                w = torch.cat([p.weight for p in projs], dim=0)
                b = torch.cat([p.bias for p in projs], dim=0) if len(params) == 6 else None
            hit = self._qkv_memo.put(params, (w, b))
        return hit

    def _qkv(self, hidden_states, query_states):
        """q, k, v as [B, L, H, D] views (reference model.py:147-149)."""
        B, L, _ = hidden_states.shape
        H, D = self.num_attention_heads, self.attention_head_size
        # the concatenated weights are a copy made outside autograd: only where nothing is being recorded
        recording = torch.is_grad_enabled() and (hidden_states.requires_grad or self.query_proj.weight.requires_grad)
        fused = None if (self.training or recording or query_states is not hidden_states) else self._fused_qkv()
        if fused is not None:
            qkv = F.linear(hidden_states, fused[0], fused[1]).view(B, L, 3, H, D)
            return qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        return (self.query_proj(query_states).view(B, L, H, D), self.key_proj(hidden_states).view(B, L, H, D),
                self.value_proj(hidden_states).view(B, L, H, D))

    def _pos_layers(self, rel_embeddings):
        """K_r, Q_r as [H, 2S, D] views of the projected relative embeddings
        (reference model.py:159-177; the slice to 2S rows is transformers modeling_deberta_v2.py:295)."""
        if not self.relative_attention or rel_embeddings is None:
            return None, None
        # the position projections exist only for the terms the module has (transformers :170-178)
        kproj = qproj = None
        if "c2p" in self.pos_att_type:
            kproj = self.key_proj if self.share_att_key else self.pos_key_proj
        if "p2c" in self.pos_att_type:
            qproj = self.query_proj if self.share_att_key else self.pos_query_proj
        key = None
        recording = torch.is_grad_enabled() and (rel_embeddings.requires_grad or self.query_proj.weight.requires_grad)
        if not self.training and not recording:  # a remembered K_r / Q_r must not carry an autograd graph
            key = (rel_embeddings,) + tuple(p for m in (kproj, qproj) if m is not None for p in (m.weight, m.bias)
                                            if p is not None)
            hit = self._pos_memo.get(key, tuple(self.pos_att_type))
            if hit is not None:
                return hit
        H, D = self.num_attention_heads, self.attention_head_size
        span = self.pos_ebd_size
        rel = self.pos_dropout(rel_embeddings)[0:2 * span]

        def heads(x):  # [2S, H*D] -> [H, 2S, D] without a copy
            return x.view(x.shape[0], H, D).transpose(0, 1)

        pos_key = heads(kproj(rel)) if kproj is not None else None
        pos_query = heads(qproj(rel)) if qproj is not None else None
        if key is not None:
            self._pos_memo.put(key, (pos_key, pos_query), tuple(self.pos_att_type))
        return pos_key, pos_query

    def forward(self, hidden_states, attention_mask, output_attentions=False, query_states=None,
                relative_pos=None, rel_embeddings=None):
        """-> (context [B, L, H*D], None).  `relative_pos` is ignored: the bucketed relative
        position is an integer table inside the kernel.  Attention probabilities are never
        materialised, so `output_attentions` yields None like the reference (model.py:252)."""
        # Under autograd the fused op is one node: differentiable in fp32 / bf16 / fp16 (the reference's
        # FlashAttentionDisentangled, flash_attention.py:1032-1086); with FP8 operands its backward raises.
        if query_states is None:
            query_states = hidden_states
        B, L, _ = hidden_states.shape
        H, D = self.num_attention_heads, self.attention_head_size

        q, k, v = self._qkv(hidden_states, query_states)
        pos_key, pos_query = self._pos_layers(rel_embeddings)

        scale_factor = 1 + ("c2p" in self.pos_att_type and pos_key is not None) + \
            ("p2c" in self.pos_att_type and pos_query is not None)
        if not self.relative_attention:
            scale_factor = 1 + ("c2p" in self.pos_att_type) + ("p2c" in self.pos_att_type)  # model.py:151-157
        sm_scale = 1.0 / math.sqrt(D * scale_factor)

        seq_start = seq_len = None
        if attention_mask is not None:
            # The kernels take the real tokens of a row as one contiguous run and write zeros into the padded
            # rows themselves; a row whose mask has a hole inside that run carries seq_len -1 and comes back as
            # NaN in every position, so the unsupported mask cannot pass for a result (the eager module honours
            # arbitrary masks).
            seq_start, seq_len = _seq_bounds_of(attention_mask, self._mask_memo)

        kw = {}
        if self.fp8_qk:
            if q.dtype != torch.bfloat16:
                raise ValueError("fp8_qk needs bfloat16 activations")
            # q and k of the layer in one set of launches; K_r / Q_r likewise, and remembered for as long as the
            # projected relative embeddings are the same tensors (outside training they are, see _pos_layers)
            q, kw["q_scale"], k, kw["k_scale"] = ops.quantize_e4m3_per_head_pair(q, k)
            pos = tuple(x for x in (pos_key, pos_query) if x is not None)
            hit = self._pos8_memo.get(pos) if pos else None
            if hit is None and pos:
                if len(pos) == 2:
                    k8, ks, q8, qs = ops.quantize_e4m3_per_head_pair(pos_key.transpose(0, 1), pos_query.transpose(0, 1))
                    hit = (k8.transpose(0, 1), ks, q8.transpose(0, 1), qs)
                else:
                    y, sc = ops.quantize_e4m3_per_head(pos[0].transpose(0, 1))
                    hit = (y.transpose(0, 1), sc, None, None) if pos_key is not None else (None, None, y.transpose(0, 1), sc)
                if not (torch.is_grad_enabled() and any(x.requires_grad for x in pos)):
                    self._pos8_memo.put(pos, hit)
            if pos:
                pos_key, pos_key_scale, pos_query, pos_query_scale = hit
                if pos_key is not None:
                    kw["pos_key_scale"] = pos_key_scale
                if pos_query is not None:
                    kw["pos_query_scale"] = pos_query_scale

        ctx = ops.disentangled_attention(
            q, k, v, pos_key, pos_query, sm_scale=sm_scale,
            position_buckets=self.position_buckets if self.relative_attention else 0,
            max_relative_positions=self.max_relative_positions if self.relative_attention else 0,
            seq_start=seq_start, seq_len=seq_len, **kw)
        return (ctx.view(B, L, H * D), None)


DEBERTA_SELF_ATTENTION_CLASSES = {
    "eager": DisentangledSelfAttention,
    "flash_attention_2": FlashDisentangledSelfAttention,
}


class FlashDebertaV2Encoder(DebertaV2Encoder):
    """transformers' encoder minus work the fused attention never reads: with `_fdb_skip_dense` it builds
    neither the [1, L, L] int64 relative-position tensor nor the [B, 1, L, L] mask (transformers
    modeling_deberta_v2.py:601-626), and outside training it hands the layers one relative-embedding tensor
    object for as long as the table and its LayerNorm are unchanged, so that each layer's K_r / Q_r stay
    valid from forward to forward.  Instances are made by `patch_model`, which switches the class of an
    existing encoder."""

    _fdb_skip_dense = True

    def get_rel_pos(self, hidden_states, query_states=None, relative_pos=None):
        if self._fdb_skip_dense:
            return relative_pos
        return super().get_rel_pos(hidden_states, query_states, relative_pos)

    def get_attention_mask(self, attention_mask):
        if self._fdb_skip_dense:
            return attention_mask
        return super().get_attention_mask(attention_mask)

    def get_rel_embedding(self):
        if self.training or not self.relative_attention:
            return super().get_rel_embedding()
        memo = self.__dict__.get("_fdb_rel_memo")
        if memo is None:
            memo = self._fdb_rel_memo = _Memo()
        norm = self.LayerNorm if "layer_norm" in self.norm_rel_ebd else None
        key = (self.rel_embeddings.weight,) + (tuple(norm.parameters()) if norm is not None else ())
        hit = memo.get(key)
        if hit is None:
            with torch.no_grad():
                hit = memo.put(key, super().get_rel_embedding())
        return hit


def patch_model(model, attn_implementation="flash_attention_2", fp8_qk=False, skip_dense_position_tensors=True):
    """Swap every `layer.attention.self` of a transformers DebertaV2 model (bare or with a head)
    for the class the key selects, keeping the weights.  With skip_dense_position_tensors the
    encoder also stops building the [1, L, L] int64 relative-position tensor and the [B, 1, L, L]
    mask (transformers modeling_deberta_v2.py:601-626), which the fused path never reads."""
    cls = DEBERTA_SELF_ATTENTION_CLASSES[attn_implementation]
    encoder = None
    for mod in model.modules():
        if mod.__class__.__name__ == "DebertaV2Encoder" or hasattr(mod, "rel_embeddings") and hasattr(mod, "layer"):
            encoder = mod
            break
    if encoder is None:
        raise ValueError("no DebertaV2 encoder found in %s" % type(model).__name__)
    config = model.config
    mask_memo = _Memo()  # the layers of one model see the same mask object: its bounds are derived once per forward
    for layer in encoder.layer:
        old = layer.attention.self
        if type(old) is cls:
            if cls is FlashDisentangledSelfAttention:
                old._mask_memo = mask_memo
            continue
        new = cls(config, fp8_qk=fp8_qk) if cls is FlashDisentangledSelfAttention else cls(config)
        new.load_state_dict(old.state_dict())
        p = next(old.parameters())
        new.to(device=p.device, dtype=p.dtype)
        new.train(old.training)
        if cls is FlashDisentangledSelfAttention:
            new._mask_memo = mask_memo
        layer.attention.self = new
    flash = cls is FlashDisentangledSelfAttention
    # The encoder-side shortcuts live in a subclass that differs from transformers' encoder in three methods
    # only; switching the instance's class keeps copies and pickles of the model working.
    if flash and type(encoder) in (DebertaV2Encoder, FlashDebertaV2Encoder):
        encoder.__class__ = FlashDebertaV2Encoder
        encoder._fdb_skip_dense = bool(skip_dense_position_tensors)
        encoder._fdb_rel_memo = _Memo()
    elif type(encoder) is FlashDebertaV2Encoder:
        encoder.__class__ = DebertaV2Encoder
    return model


class FlashDebertaV2Model(DebertaV2Model):
    """DebertaV2Model whose attention follows `config._attn_implementation` in
    {"eager", "flash_attention_2"}; unset means "flash_attention_2", the reference's default
    (model.py:61-62).  transformers' own check would treat "flash_attention_2" as a request for
    the flash-attn package, so the two keys are resolved here instead."""

    def _check_and_adjust_attn_implementation(self, attn_implementation, is_init_check=False, **kwargs):
        if attn_implementation is None:
            return "flash_attention_2"
        if attn_implementation in DEBERTA_SELF_ATTENTION_CLASSES:
            return attn_implementation
        raise ValueError("attn_implementation must be one of %s, got %r"
                         % (sorted(DEBERTA_SELF_ATTENTION_CLASSES), attn_implementation))

    def __init__(self, config):
        super().__init__(config)
        patch_model(self, self.config._attn_implementation, fp8_qk=bool(getattr(config, "fp8_qk", False)))


__all__ = ["FlashDisentangledSelfAttention", "DEBERTA_SELF_ATTENTION_CLASSES", "FlashDebertaV2Model",
           "FlashDebertaV2Encoder", "DebertaV2Config", "patch_model"]
