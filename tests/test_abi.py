"""CPU tests of the C-ABI library: it loads, exports every symbol include/fdb.h declares, its
host-side logic (delta table, work-list sizing, argument validation, error strings) behaves, and
the python mirror of the reference interface is wired.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from flashdeberta_amd import _lib, ops
from flashdeberta_amd._lib import FdbAttnArgs, lib
from oracle import disentangled_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "fdb.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    body = text[text.index("} fdb_attn_args;"):]
    return sorted(set(re.findall(r"\b(fdb_[a-z0-9_]+)\s*\(", body)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), "libfdb_hip.so does not export %s" % n
    assert sorted(_lib.EXPORTS) == names


def test_struct_mirror_and_version():
    assert lib.fdb_attn_args_size() == ctypes.sizeof(FdbAttnArgs)
    assert lib.fdb_version() == _lib.FDB_VERSION == 7
    assert lib.fdb_tile_rows() == 128


@pytest.mark.parametrize("pb,mr", [(256, 512), (32, 64), (64, 512), (16, 40), (0, 512), (0, 24), (128, 256)])
def test_delta_lut_bit_exact_vs_oracle(pb, mr):
    lut, R = ops.delta_lut_host(pb, mr)
    ref = O.delta_table(pb, mr, R)
    assert lut.dtype == np.int16 and len(lut) == 2 * R + 1
    assert (lut.astype(np.int64) == ref).all()
    # beyond the radius delta is constant: the table's ends are the clamp values on both sides
    wide = O.delta_table(pb, mr, 4 * R + 100)
    c = 3 * R + 100
    assert (wide[:c] == lut[0]).all() and (wide[-c:] == lut[-1]).all()
    span = pb if pb > 0 else mr
    assert lut[0] == 0 and lut[-1] == 2 * span - 1
    # tight: one step inside the radius at least one side has not reached its clamp value yet
    assert lut[1] != lut[0] or lut[-2] != lut[-1]


def test_delta_lut_rejects_degenerate_configs():
    assert lib.fdb_delta_lut_radius(2, 512) == -9      # mid - 1 == 0
    assert lib.fdb_delta_lut_radius(256, 100) == -9    # log((max-1)/mid) <= 0
    assert lib.fdb_delta_lut_radius(0, 0) == -9
    buf = np.zeros(8, dtype=np.int16)
    assert lib.fdb_delta_lut(256, 512, 0, buf.ctypes.data_as(ctypes.c_void_p)) == -9
    assert lib.fdb_delta_lut(256, 512, 3, None) == -9
    with pytest.raises(ValueError):
        ops.delta_lut_host(2, 512)


def test_worklist_sizing():
    assert lib.fdb_worklist_max_tiles(1000, 4) == 1000 // 128 + 4
    assert lib.fdb_worklist_ints(1000, 4) == 2 + 2 * (1000 // 128 + 4)
    rng = np.random.default_rng(0)
    for _ in range(50):
        lens = rng.integers(0, 700, size=rng.integers(1, 40))
        tiles = int(sum((l + 127) // 128 for l in lens))
        assert tiles <= lib.fdb_worklist_max_tiles(int(lens.sum()), len(lens))


def _good_args():
    a = FdbAttnArgs()
    a.q = a.k = a.v = a.out = 0x1000
    a.pos_key = a.pos_query = 0x2000
    a.delta_lut = 0x3000
    for n in ("q", "k", "v", "o"):
        setattr(a, n + "_stride_b", 512 * 768)
        setattr(a, n + "_stride_t", 768)
        setattr(a, n + "_stride_h", 64)
    a.pk_stride_h = a.pq_stride_h = 64
    a.pk_stride_r = a.pq_stride_r = 768
    a.batch, a.heads, a.head_dim, a.max_seqlen, a.total_tokens = 2, 12, 64, 512, 1024
    a.att_span, a.lut_radius, a.dtype, a.sm_scale = 256, 512, _lib.FDB_BF16, 0.0721
    return a


def test_argument_validation_codes():
    chk = lambda a: lib.fdb_attn_check(ctypes.byref(a))
    assert chk(_good_args()) == 0
    a = _good_args(); a.q = None; assert chk(a) == -1
    a = _good_args(); a.dtype = 9; assert chk(a) == -2
    a = _good_args(); a.head_dim = 48; assert chk(a) == -3
    a = _good_args(); a.k = 0x1008; assert chk(a) == -4
    a = _good_args(); a.q_stride_t = 772; assert chk(a) == -4            # 772 * 2 bytes is not a multiple of 16
    a = _good_args(); a.total_tokens = 1000; assert chk(a) == -5         # != batch * max_seqlen without cu_seqlens
    a = _good_args(); a.heads = 0; assert chk(a) == -5
    a = _good_args(); a.delta_lut = None; assert chk(a) == -6
    a = _good_args(); a.att_span = 0; assert chk(a) == -6
    a = _good_args(); a.dtype = _lib.FDB_FP8_E4M3; assert chk(a) == -7   # no scales
    a = _good_args(); a.cu_seqlens = 0x4000; assert chk(a) == -8          # no work-list
    a = _good_args(); a.dtype = _lib.FDB_F32; a.head_dim = 128; assert chk(a) == 0       # every dtype at every head_dim
    # rows of the position tables are addressed with 32-bit byte offsets: 24-bit row strides, a head's table within 2^31 bytes
    a = _good_args(); a.pk_stride_r = -64; assert chk(a) == -5
    a = _good_args(); a.pq_stride_r = 1 << 23; assert chk(a) == -5                       # 2^24 bytes per row in a 16-bit type
    a = _good_args(); a.pk_stride_r = (1 << 23) - 8; assert chk(a) == -5                 # rows fit, 2 * att_span of them do not
    a = _good_args(); a.pk_stride_r = 768; a.pq_stride_r = 1536; assert chk(a) == 0      # rows of a [2S, H * D] projection output
    a = _good_args(); a.pos_key = a.pos_query = None; a.delta_lut = None; a.att_span = 0; assert chk(a) == 0
    assert lib.fdb_attn_check(None) == -1
    # launching with bad arguments returns the same code without touching the GPU
    a = _good_args(); a.head_dim = 48
    assert lib.fdb_attn_fwd(ctypes.byref(a), None) == -3
    assert lib.fdb_build_worklist(None, 1, 1, None, None) == -1
    assert lib.fdb_quant_e4m3_per_head(None, 0, 0, None, 0, 0, None, None, 1, 1, 64, None) == -1
    assert lib.fdb_dequant_e4m3_per_head(None, 0, 0, None, None, 0, 0, 1, 1, 64, None) == -1
    assert lib.fdb_dequant_e4m3_per_head(0x4000, 64, 64, 0x5000, 0x6000, 64, 64, 1, 1, 48, None) == -3


def test_far_split_policy_and_workspace_size():
    """Host-only: how many workgroups share a query tile's far keys, and the workspace that takes (without a
    GPU the library assumes 256 compute units, i.e. 768 far workgroups in flight)."""
    ws = lambda a: lib.fdb_attn_workspace_bytes(ctypes.byref(a))
    chk = lambda a: lib.fdb_attn_check(ctypes.byref(a))
    part = lambda rows, heads: rows * heads * (64 * 2 + 4)

    def args(batch, seqlen, heads=12, lse=0x5000):
        a = _good_args()
        a.batch, a.heads, a.max_seqlen, a.total_tokens, a.lse = batch, heads, seqlen, batch * seqlen, lse
        return a

    # far launch: 3 workgroups per CU = 768 slots; near launch: 2 per CU = 512 slots
    assert ws(args(1, 4096)) == part(4096, 12)            # 384 query tiles: 2 far shares (1 slot), near unshared
    assert ws(args(1, 4096, heads=16)) == 0               # 512: two shares would need a second round
    assert ws(args(1, 4096, heads=10)) == (1 + 2) * part(4096, 10)  # 320: 2 far shares; 2 near shares in 1.25 rounds
    assert ws(args(1, 4096, heads=8)) == (2 + 2) * part(4096, 8)  # 256: 3 far shares (2 slots) + 2 near shares (2 slots)
    assert ws(args(2, 4096)) == 0 and ws(args(8, 4096)) == 0  # the launch fills the slots by itself
    assert ws(args(1, 2048)) == 2 * part(2048, 12)        # 192: too few far tiles to share, 2 near shares
    assert ws(args(1, 1024)) == 2 * part(1024, 12)        # 96: 32 steps in two shares of sixteen
    assert ws(args(1, 512)) == 2 * part(512, 12)          # 48, no far tile at all: shares of eight steps, 96 workgroups
    assert ws(args(2, 512)) == 2 * part(2 * 512, 12)      # 96 -> 192
    assert ws(args(4, 512)) == 0                          # 192 -> 384: more than half of the slots in shares of eight
    assert ws(args(8, 512)) == 0
    assert ws(args(1, 4096, lse=None)) == 0               # one fused kernel without the lse buffer
    a = args(8, 4096); a.far_splits = 4; assert ws(a) == 3 * part(8 * 4096, 12)
    a = args(8, 4096); a.near_splits = 3; assert ws(a) == 3 * part(8 * 4096, 12)
    a = args(1, 4096); a.far_splits = 1; assert ws(a) == 0
    a = args(1, 2048); a.near_splits = 1; assert ws(a) == 0
    # fp32 takes the one-kernel mode: its shares divide all key tiles of a query tile and every share has a slot
    part32 = lambda rows, heads: rows * heads * (64 * 4 + 4)
    a = args(1, 4096); a.dtype = _lib.FDB_F32; a.far_splits = a.near_splits = 3; assert ws(a) == 3 * part32(4096, 12)
    a = args(1, 4096); a.dtype = _lib.FDB_F32; assert ws(a) == 0                         # 384 workgroups on 256 compute units
    a = args(1, 1024); a.dtype = _lib.FDB_F32; assert ws(a) == 2 * part32(1024, 12)      # 96: two shares of eight tiles
    a = args(1, 512); a.dtype = _lib.FDB_F32; assert ws(a) == 4 * part32(512, 12)        # 48: four shares of two tiles
    a = args(1, 512); a.dtype = _lib.FDB_F32; a.causal = 1; assert ws(a) == 0            # causal calls are never shared
    a = args(1, 512); a.dtype = _lib.FDB_F32; a.causal = 1; a.far_splits = 3; assert ws(a) == 0
    a = args(1, 100); a.dtype = _lib.FDB_F32; assert ws(a) == 0                          # two key tiles: nothing to share
    a = args(1, 4096); a.cu_seqlens, a.worklist = 0x6000, 0x7000; assert ws(a) == 0   # lengths unknown to the host
    a.far_splits = 2; assert ws(a) == part(4096, 12)
    a = args(1, 4096); a.far_splits = 5; assert chk(a) == -5 and ws(a) == 0
    a = args(1, 4096); a.far_splits = -1; assert chk(a) == -5
    a = args(1, 4096); a.near_splits = 5; assert chk(a) == -5
    a = args(1, 4096); a.workspace, a.workspace_bytes = 0x8008, 1 << 20; assert chk(a) == -4
    a = args(1, 4096); a.workspace, a.workspace_bytes = 0x8000, -1; assert chk(a) == -5


def test_error_strings_and_python_mapping():
    for code in range(-10, 1):
        assert _lib.strerror(code) not in ("", "unknown error")
    with pytest.raises(ValueError):
        _lib.check(-3, "x")
    with pytest.raises(RuntimeError):
        _lib.check(1, "x")


def test_ops_reject_cpu_tensors_and_bad_shapes():
    q = torch.zeros(1, 8, 2, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.disentangled_attention_fwd(q, q, q)


def test_module_is_state_dict_compatible_with_eager():
    from transformers.models.deberta_v2.modeling_deberta_v2 import DisentangledSelfAttention

    from flashdeberta_amd import DEBERTA_SELF_ATTENTION_CLASSES, FlashDisentangledSelfAttention

    class Cfg:  # the plain config object of the reference's tests/attention.py:6-18
        hidden_size, num_attention_heads = 128, 2
        attention_probs_dropout_prob = hidden_dropout_prob = 0.1
        pos_att_type = ["c2p", "p2c"]
        relative_attention, position_buckets, max_relative_positions = True, 32, 64
        max_position_embeddings, share_att_key = 512, False

    eager = DisentangledSelfAttention(Cfg())
    flash = FlashDisentangledSelfAttention(Cfg())
    res = flash.load_state_dict(eager.state_dict())
    assert not res.missing_keys and not res.unexpected_keys
    assert DEBERTA_SELF_ATTENTION_CLASSES["eager"] is DisentangledSelfAttention
    assert DEBERTA_SELF_ATTENTION_CLASSES["flash_attention_2"] is FlashDisentangledSelfAttention
    pk, pq = flash._pos_layers(torch.randn(64, 128))
    assert pk.shape == (2, 64, 64) and pq.shape == (2, 64, 64)


def test_switch_builds_both_implementations():
    from transformers.models.deberta_v2.modeling_deberta_v2 import DebertaV2Model, DisentangledSelfAttention

    from flashdeberta_amd import DebertaV2Config, FlashDebertaV2Model, FlashDisentangledSelfAttention, patch_model

    kw = dict(vocab_size=50, hidden_size=128, num_hidden_layers=2, num_attention_heads=2, intermediate_size=128,
              relative_attention=True, pos_att_type="p2c|c2p", position_buckets=32, max_relative_positions=64,
              share_att_key=True, norm_rel_ebd="layer_norm", position_biased_input=False)
    m = FlashDebertaV2Model(DebertaV2Config(**kw))
    assert all(type(l.attention.self) is FlashDisentangledSelfAttention for l in m.encoder.layer)
    m = FlashDebertaV2Model(DebertaV2Config(attn_implementation="eager", **kw))
    assert all(type(l.attention.self) is DisentangledSelfAttention for l in m.encoder.layer)
    hf = DebertaV2Model(DebertaV2Config(**kw))
    w = hf.encoder.layer[1].attention.self.query_proj.weight.clone()
    patch_model(hf)
    assert type(hf.encoder.layer[1].attention.self) is FlashDisentangledSelfAttention
    assert torch.equal(hf.encoder.layer[1].attention.self.query_proj.weight, w)
    patch_model(hf, "eager")
    assert type(hf.encoder.layer[1].attention.self) is DisentangledSelfAttention
    with pytest.raises(ValueError):
        FlashDebertaV2Model(DebertaV2Config(attn_implementation="sdpa", **kw))


def test_module_projection_memos():
    """The one-GEMM input projection and the remembered K_r / Q_r equal the separate projections, and
    are rebuilt when a parameter is written in place, replaced, or the module goes back to training."""
    from flashdeberta_amd import DebertaV2Config, FlashDisentangledSelfAttention, patch_model
    from flashdeberta_amd.model import _seq_bounds_of
    from transformers.models.deberta_v2.modeling_deberta_v2 import DebertaV2Model

    torch.manual_seed(3)
    kw = dict(vocab_size=50, hidden_size=128, num_hidden_layers=2, num_attention_heads=2, intermediate_size=128,
              relative_attention=True, pos_att_type="p2c|c2p", position_buckets=32, max_relative_positions=64,
              share_att_key=True, norm_rel_ebd="layer_norm", position_biased_input=False)
    att = FlashDisentangledSelfAttention(DebertaV2Config(**kw)).eval()
    x = torch.randn(2, 7, 128)

    def separate():
        return [p(x).view(2, 7, 2, 64) for p in (att.query_proj, att.key_proj, att.value_proj)]

    with torch.no_grad():
        for got, ref in zip(att._qkv(x, x), separate()):
            assert got.shape == ref.shape and got.stride(-1) == 1 and torch.allclose(got, ref, atol=1e-6)
        w0 = att._fused_qkv()[0]
        assert att._fused_qkv()[0] is w0                       # remembered
        att.key_proj.weight.mul_(2.0)                          # in-place update -> rebuilt
        assert att._fused_qkv()[0] is not w0
        for got, ref in zip(att._qkv(x, x), separate()):
            assert torch.allclose(got, ref, atol=1e-6)
        att.load_state_dict({k: v * 0.5 for k, v in att.state_dict().items()})
        for got, ref in zip(att._qkv(x, x), separate()):
            assert torch.allclose(got, ref, atol=1e-6)
        other = torch.randn(2, 7, 128)                         # cross-attention style call: no fusion
        q, k, v = att._qkv(x, other)
        assert torch.allclose(q, att.query_proj(other).view(2, 7, 2, 64)) and torch.allclose(k, separate()[1], atol=1e-6)
        # K_r / Q_r
        rel = torch.randn(64, 128)
        pk, pq = att._pos_layers(rel)
        assert att._pos_layers(rel)[0] is pk
        assert torch.allclose(pk, att.key_proj(rel).view(64, 2, 64).transpose(0, 1))
        assert torch.allclose(pq, att.query_proj(rel).view(64, 2, 64).transpose(0, 1))
        att.query_proj.bias.add_(1.0)
        pk2, pq2 = att._pos_layers(rel)
        assert pq2 is not pq and torch.allclose(pq2, att.query_proj(rel).view(64, 2, 64).transpose(0, 1))
        assert att._pos_layers(rel.clone())[0] is not pk2      # another tensor object
        # a parameter re-seated through .data (EMA / loader style weight swaps): same object, same version
        att.key_proj.weight.data = torch.randn_like(att.key_proj.weight)
        for got, ref in zip(att._qkv(x, x), separate()):
            assert torch.allclose(got, ref, atol=1e-6)
        assert torch.allclose(att._pos_layers(rel)[0], att.key_proj(rel).view(64, 2, 64).transpose(0, 1))
        # a cast of the whole module after a forward: the remembered tensors follow the new dtype
        att.to(torch.bfloat16)
        assert att._fused_qkv()[0].dtype == torch.bfloat16
        assert att._pos_layers(rel.to(torch.bfloat16))[0].dtype == torch.bfloat16
        att.to(torch.float32)
        for got, ref in zip(att._qkv(x, x), separate()):
            assert torch.allclose(got, ref, atol=1e-6)
    att.train()
    assert att._pos_layers(rel)[0] is not att._pos_layers(rel)[0]

    # the patched encoder hands out one relative-embedding tensor until the table changes
    hf = patch_model(DebertaV2Model(DebertaV2Config(**kw))).eval()
    r0 = hf.encoder.get_rel_embedding()
    assert hf.encoder.get_rel_embedding() is r0
    ref = hf.encoder.LayerNorm(hf.encoder.rel_embeddings.weight)
    assert torch.allclose(r0, ref)
    with torch.no_grad():
        hf.encoder.rel_embeddings.weight.add_(0.1)
    r1 = hf.encoder.get_rel_embedding()
    assert r1 is not r0 and torch.allclose(r1, hf.encoder.LayerNorm(hf.encoder.rel_embeddings.weight))
    hf.train()
    assert hf.encoder.get_rel_embedding() is not hf.encoder.get_rel_embedding()
    # copies and pickles of a patched model work and remember nothing of the original
    import copy, io, pickle
    hf.eval()
    r2 = hf.encoder.get_rel_embedding()
    twin = copy.deepcopy(hf)
    with torch.no_grad():
        twin.encoder.rel_embeddings.weight.mul_(3.0)
    assert hf.encoder.get_rel_embedding() is r2
    assert torch.allclose(twin.encoder.get_rel_embedding(), twin.encoder.LayerNorm(twin.encoder.rel_embeddings.weight))
    again = pickle.loads(pickle.dumps(hf))
    assert type(again.encoder) is type(hf.encoder) and torch.allclose(again.encoder.get_rel_embedding(), r2)
    patch_model(hf, "eager")
    assert type(hf.encoder).__name__ == "DebertaV2Encoder"

    # mask bounds: once per mask object and version, remembered by the memo the layers of a patched model share
    from flashdeberta_amd.model import _Memo
    memo = _Memo()
    m = torch.tensor([[1, 1, 1, 0, 0], [0, 0, 1, 1, 1], [1, 0, 1, 1, 0]])
    s0, n0 = _seq_bounds_of(m, memo)
    assert _seq_bounds_of(m, memo)[0] is s0 and s0.tolist()[:2] == [0, 2] and n0.tolist() == [3, 3, -1]  # -1: a hole
    m[0, 3] = 1
    s1, n1 = _seq_bounds_of(m, memo)
    assert s1 is not s0 and n1.tolist() == [4, 3, -1]
    assert _seq_bounds_of(m.clone(), memo)[0] is not s1  # another mask object
    assert not hasattr(m, "_fdb_bounds")                 # nothing rides on the caller's tensor
    layers = patch_model(DebertaV2Model(DebertaV2Config(**kw))).encoder.layer
    assert layers[0].attention.self._mask_memo is layers[1].attention.self._mask_memo
    assert FlashDisentangledSelfAttention(DebertaV2Config(**kw))._mask_memo is not layers[0].attention.self._mask_memo


def test_padding_helpers():
    from flashdeberta_amd.padding import key_padding_mask, seq_bounds

    m = torch.tensor([[1, 1, 1, 0, 0], [0, 0, 1, 1, 1], [1, 1, 1, 1, 1]])
    ext = m[:, None, None, :] * m[:, None, :, None]
    assert torch.equal(key_padding_mask(ext), m.bool()) and torch.equal(key_padding_mask(m), m.bool())
    s, n, holes = seq_bounds(m.bool())
    assert s.tolist() == [0, 2, 0] and n.tolist() == [3, 3, 5] and holes.tolist() == [False, False, False]
    # masked tokens between real ones: flagged, and the row gets no tokens
    mh = torch.tensor([[1, 1, 0, 1, 1], [0, 1, 1, 1, 0], [0, 0, 0, 0, 0], [1, 0, 0, 0, 1]]).bool()
    s, n, holes = seq_bounds(mh)
    assert holes.tolist() == [True, False, False, True] and n.tolist() == [-1, 3, 0, -1] and s.tolist()[1] == 1
    from flashdeberta_amd.padding import assert_contiguous_mask
    assert_contiguous_mask(m)
    with pytest.raises(ValueError, match="rows \\[0, 3\\]"):
        assert_contiguous_mask(mh)
    # the oracle's unpad bookkeeping (what the reference's packed branch derives from a mask, padding.py:79-88),
    # by literal values: flattened positions of the ones of the three rows, their running counts, the longest row
    ref_idx, ref_cu, ref_mx = O.unpad_data(m.numpy())
    assert ref_idx.tolist() == [0, 1, 2, 7, 8, 9, 10, 11, 12, 13, 14] and ref_cu.tolist() == [0, 3, 6, 11] and ref_mx == 5


def test_no_alloc_entry_point_refuses_what_does_not_fit():
    # hand-over of rows * heads * 4 bytes: 8 x 65536 rows x 32 heads = 64 MiB > the 32 MiB scratch; host-side
    # refusal, nothing is launched (the pointers are never dereferenced)
    a = _lib.FdbAttnArgs()
    a.q = a.k = a.v = a.out = a.pos_key = a.pos_query = a.delta_lut = 0x10000
    B, L, H, D = 8, 65536, 32, 64
    for n in ("q", "k", "v", "o"):
        setattr(a, n + "_stride_b", L * H * D)
        setattr(a, n + "_stride_t", H * D)
        setattr(a, n + "_stride_h", D)
    a.pk_stride_h = a.pq_stride_h = D
    a.pk_stride_r = a.pq_stride_r = H * D
    a.batch, a.heads, a.head_dim, a.max_seqlen, a.total_tokens = B, H, D, L, B * L
    a.att_span, a.lut_radius, a.dtype, a.sm_scale = 256, 512, _lib.FDB_BF16, 0.07
    assert lib.fdb_attn_check(ctypes.byref(a)) == 0
    rc = lib.fdb_attn_fwd_noalloc(ctypes.byref(a), None)
    assert rc == -11 and "scratch" in _lib.strerror(rc)
    with pytest.raises(ValueError, match="scratch"):
        _lib.check(rc, "fdb_attn_fwd_noalloc")


def test_bench_contract_without_a_gpu():
    """bench.py refuses more than one GPU with a message, prices the workloads with the stated FLOP
    count, and its CPU leg returns the fields the measurement contract names."""
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)
    sys.path.insert(0, ROOT)
    import bench

    # F = B*H*(4 L^2 D + 4 L 2S D): 463.86 GFLOP at the default workload
    B, L, H, D, _, _ = bench.WORKLOADS["v3base_L4096_B8_bf16"]
    assert abs(bench.flops([L] * B, H, D) / 1e9 - 463.86) < 0.01
    assert bench.flops([512], 12, 64, pos=False) == 12 * 4 * 512 * 512 * 64
    rec = bench.cpu_baseline(2, 64, 256)
    # headline = the reference's eager class (transformers is installed here), the numpy port beside it
    assert rec["kind"] == "reference" and rec["cores"] >= 1 and rec["value"] > 0 and rec["unit"] == "TFLOP/s"
    assert "DisentangledSelfAttention" in rec["sample"]
    assert rec["port"]["kind"] == "port" and rec["port"]["value"] > 0 and rec["port"]["cores"] >= 1
    # tile census at L = 4096: 64 key tiles per query tile, 16.75 of them near on average
    far, near = bench.tile_census([4096])
    assert far + near == 32 * 64 and near == 536
    tv, src = bench.measured_traffic("v3base_L4096_B8_bf16", with_source=True)
    assert (tv is None) == (src is None)
    t = bench.measured_traffic("v3base_L4096_B8_bf16")
    assert t is None or t > 2e8


def _window_by_brute_force(lut):
    """Largest delta(r + 31) - delta(r) over every r, from the table itself (constant beyond its ends)."""
    x = np.concatenate([np.full(31, lut[0]), lut.astype(np.int64), np.full(31, lut[-1])])
    return int((x[31:] - x[:-31]).max())


def test_backward_window_of_every_accepted_table():
    """The backward keeps a 64-entry sliding window of table rows per tensor row.  It holds the rows one 32-row
    step reaches (delta(r + 31) - delta(r) + 1) plus a partly stored group of four, so fdb_attn_bwd refuses tables
    whose window exceeds FDB_BWD_MAX_WINDOW = 60.  Sweep of every configuration the host accepts on a grid:
    the table is monotone, fdb_delta_lut_window equals the brute-force figure, tables with unit steps have a
    window of at most 31, every unbucketed table and every bucketed one with max_position >= position_buckets
    fits, and some configurations below that do not (they are refused before anything is launched)."""
    refused = accepted = 0
    grid = [(pb, mr) for pb in (0, 4, 8, 16, 32, 64, 100, 128, 256, 512, 1024) for mr in
            (3, 8, 15, 16, 24, 40, 64, 100, 128, 200, 256, 300, 512, 513, 600, 1024, 2048, 4096)]
    for pb, mr in grid:
        if lib.fdb_delta_lut_radius(pb, mr) < 1:
            assert lib.fdb_delta_lut_window(pb, mr) == -9
            continue
        lut, radius = ops.delta_lut_host(pb, mr)
        steps = np.diff(lut.astype(np.int64))
        assert steps.min() >= 0, (pb, mr)
        assert lut[0] >= 0 and lut[-1] <= 2 * ops.att_span(pb, mr) - 1
        w = ops.delta_lut_window(pb, mr)
        assert w == _window_by_brute_force(lut), (pb, mr)
        if steps.max() <= 1:
            assert w <= 31, (pb, mr)
        if pb == 0 or mr >= 2 * pb:
            assert steps.max() <= 1, (pb, mr)
        if pb == 0 or mr >= pb:   # steps of 2 occur up to max_position ~ 1.36 position_buckets; the window still fits
            assert w <= _lib.FDB_BWD_MAX_WINDOW, (pb, mr)
        if w > _lib.FDB_BWD_MAX_WINDOW:
            refused += 1
        else:
            accepted += 1
    assert refused > 0 and accepted > 100
    # the two configurations a review found: worst windows 67 and 192 by its count, i.e. beyond the 60 the ring holds
    assert ops.delta_lut_window(256, 200) > _lib.FDB_BWD_MAX_WINDOW and ops.delta_lut_window(512, 300) > _lib.FDB_BWD_MAX_WINDOW
    assert ops.delta_lut_window(256, 512) <= 31


def test_backward_ring_holds_the_chunked_stores():
    """Score gradients leave the 64-entry ring of a row in aligned chunks of 8, 4 or 1 groups of four entries, as the
    table's window leaves room (fdb_attn_bwd: lut_window + 4 + 28, + 12 or + 0 within the ring).  Replay of the kernel's
    bookkeeping on the host for every accepted table of the grid, both directions and every phase of the 32-row steps
    against the table: the entries between the oldest one not yet stored and the newest one touched never exceed the ring."""
    ring = 64
    grid = [(pb, mr) for pb in (0, 4, 8, 16, 32, 64, 100, 128, 256, 512) for mr in (3, 8, 16, 24, 40, 64, 100, 128, 200, 256, 300, 512, 600, 1024)]
    checked = 0
    for pb, mr in grid:
        if lib.fdb_delta_lut_radius(pb, mr) < 1:
            continue
        w = ops.delta_lut_window(pb, mr)
        if w > _lib.FDB_BWD_MAX_WINDOW:
            continue
        chunk = 8 if w + 4 + 28 <= ring else 4 if w + 4 + 12 <= ring else 1
        lut, radius = ops.delta_lut_host(pb, mr)
        lut = lut.astype(np.int64)
        delta = lambda r: int(lut[min(max(r, -radius), radius) + radius])
        for r0 in range(-radius - 40, radius + 41, 1 if radius <= 64 else 3):
            # dK/dV role: the relative position grows with the loop row, the window moves up
            g_next = delta(r0) >> 2
            for k in range((2 * radius + 160) // 32):
                lo_r = r0 + 32 * k
                assert delta(lo_r + 31) - 4 * g_next + 1 <= ring, (pb, mr, r0, k)
                g_next = max(g_next, (delta(lo_r + 32) >> 2) & ~(chunk - 1))
            # dQ role: it falls, the window moves down
            g_next = delta(r0) >> 2
            for k in range((2 * radius + 160) // 32):
                hi_r = r0 - 32 * k
                assert 4 * g_next + 3 - delta(hi_r - 31) + 1 <= ring, (pb, mr, r0, k)
                g_next = min(g_next, (((delta(hi_r - 32) >> 2) + chunk) & ~(chunk - 1)) - 1)
        checked += 1
    assert checked > 60


def _header_struct_fields(name):
    """(field name, C type) pairs of `typedef struct <name> { ... } <name>;` in include/fdb.h, in order."""
    text = open(os.path.join(ROOT, "include", "fdb.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    body = text[text.index("typedef struct %s {" % name):text.index("} %s;" % name)].split("{", 1)[1]
    out = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        m = re.match(r"((?:const )?[a-z0-9_]+\s*\*?)\s*(.*)", decl)
        ctype, names = m.group(1).replace(" *", "*").strip(), m.group(2)
        for n in names.split(","):
            n = n.strip()
            if n.startswith("*"):
                n, t = n[1:].strip(), ctype + "*"
            else:
                t = ctype
            out.append((n, t))
    return out


@pytest.mark.parametrize("name,mirror", [("fdb_attn_args", _lib.FdbAttnArgs), ("fdb_attn_bwd_args", _lib.FdbAttnBwdArgs)])
def test_struct_mirrors_follow_the_header_field_by_field(name, mirror):
    ctype_of = {"int64_t": ctypes.c_int64, "int32_t": ctypes.c_int32, "float": ctypes.c_float}
    fields = _header_struct_fields(name)
    assert [n for n, _ in fields] == [n for n, _ in mirror._fields_]
    for (n, t), (_, ct) in zip(fields, mirror._fields_):
        assert ct is (ctypes.c_void_p if t.endswith("*") else ctype_of[t]), (n, t, ct)
    size = lib.fdb_attn_args_size() if name == "fdb_attn_args" else lib.fdb_attn_bwd_args_size()
    assert size == ctypes.sizeof(mirror)


def _good_bwd_args():
    a = _lib.FdbAttnBwdArgs()
    for n in ("q", "k", "v", "dout", "dq", "dk", "dv", "out"):
        setattr(a, n, 0x1000)
    a.lse = a.delta = 0x2000
    a.c2p_bias = a.p2c_bias = 0x3000
    a.d_c2p_bias = a.d_p2c_bias = 0x4000
    a.delta_lut = 0x5000
    for n in ("q", "k", "v", "do", "out", "dq", "dk", "dv"):
        setattr(a, n + "_stride_b", 512 * 768)
        setattr(a, n + "_stride_t", 768)
        setattr(a, n + "_stride_h", 64)
    a.bias_stride_b, a.bias_stride_t, a.bias_stride_h = 512 * 512, 512, 2 * 512 * 512
    a.batch, a.heads, a.head_dim, a.seqlen = 2, 12, 64, 512
    a.att_span, a.lut_radius, a.dtype, a.sm_scale = 256, 512, _lib.FDB_BF16, 0.0721
    a.lut_window = 24
    return a


def test_chain_argument_validation_codes():
    """fdb_attn_bwd_chain refuses what its kernel is not built for before anything touches the GPU."""
    f = lambda g=0x1000, x=0x2000, x2=0x2800, pos=0x3000, dx=0x4000, dx2=0x4800, parts_out=0x5000, m=24, m1=12, rows=4096, sm=64, sr=768, \
        dsm=64, dsr=768, span=256, d=64, dt=_lib.FDB_BF16, parts=10: \
        lib.fdb_attn_bwd_chain(g, x, x2, pos, dx, dx2, parts_out, m, m1, rows, sm, sr, dsm, dsr, span, d, dt, parts, None)
    assert f(g=None) == -1 and f(parts_out=None) == -1
    assert f(x2=None) == -1 and f(dx2=None) == -1   # matrices beyond the first tensor's need the second
    assert f(m1=0) == -5 and f(m1=25) == -5 and f(sr=32) == -5 and f(dsm=32) == -5 and f(dsr=0) == -5
    assert f(sm=4) == -4 and f(sr=772) == -4 and f(x2=0x2804) == -4 and f(dsr=772) == -4 and f(dx2=0x4808) == -4
    assert f(dt=_lib.FDB_F32) == -2 and f(dt=_lib.FDB_FP8_E4M3) == -2
    assert f(d=32) == -3 and f(d=128) == -3
    assert f(x=0x2008) == -4 and f(dx=0x4004) == -4
    assert f(rows=4100) == -5 and f(rows=0) == -5 and f(parts=0) == -5 and f(parts=129) == -5 and f(m=0) == -5
    assert f(span=128) == -6


def test_backward_argument_validation_codes():
    """Every refusal of fdb_attn_bwd comes before anything touches the GPU, so it can be checked without one."""
    call = lambda a: lib.fdb_attn_bwd(ctypes.byref(a), None)
    assert lib.fdb_attn_bwd(None, None) == -1
    a = _good_bwd_args(); a.dq = None; assert call(a) == -1
    a = _good_bwd_args(); a.d_c2p_bias = None; assert call(a) == -1       # a term without its gradient tensor
    a = _good_bwd_args(); a.dtype = _lib.FDB_FP8_E4M3; assert call(a) == -2
    a = _good_bwd_args(); a.head_dim = 48; assert call(a) == -3
    a = _good_bwd_args(); a.k = 0x1008; assert call(a) == -4
    a = _good_bwd_args(); a.dk_stride_t = 772; assert call(a) == -4
    a = _good_bwd_args(); a.att_span = 255; a.bias_stride_t = 512; assert call(a) == -4   # 2S must be a multiple of 4
    a = _good_bwd_args(); a.bias_stride_h = 2 * 512 * 512 + 2; assert call(a) == -4
    a = _good_bwd_args(); a.d_p2c_bias = 0x4004; assert call(a) == -4      # a store group is four elements
    a = _good_bwd_args(); a.c2p_bias = 0x3002; assert call(a) == -4        # the scores are read as aligned 32-bit words
    a = _good_bwd_args(); a.d_p2c_bias = 0x4008; a.seqlen = 0; assert call(a) == -5       # (8-byte alignment is enough for 16-bit types)
    a = _good_bwd_args(); a.bias_stride_t = 500; assert call(a) == -5      # rows shorter than 2S
    a = _good_bwd_args(); a.seqlen, a.bias_stride_t = 1 << 20, 1 << 12; assert call(a) == -5  # 32-bit offsets
    a = _good_bwd_args(); a.dtype, a.seqlen, a.bias_stride_t = _lib.FDB_F32, 1 << 19, 1 << 11; assert call(a) == -5  # ... in bytes
    a = _good_bwd_args(); a.delta_lut = None; assert call(a) == -6
    a = _good_bwd_args(); a.lut_radius = 0; assert call(a) == -6
    a = _good_bwd_args(); a.lut_window = 61; assert call(a) == -6           # more table rows per step than the ring holds
    a = _good_bwd_args(); a.lut_window = -1; assert call(a) == -6
