"""CPU tests that pin the oracle (oracle/disentangled_oracle.py) without running anything of the
reference: known values and invariants of the bucket function, textbook reductions, a brute-force
triple loop, and the golden vectors written from the third-party eager class."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import disentangled_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ---- bucket / delta ---------------------------------------------------------------------------
def test_bucket_known_values_v3_base():
    # r -> bucket for position_buckets=256, max_relative_positions=512 (mid = 128)
    known = {0: 0, 1: 1, -1: -1, 127: 127, 128: 128, 129: 129, 255: 192, 256: 192, 510: 255, 511: 255, 512: 256,
             -128: -128, -129: -129, -255: -192, -511: -255, -512: -256}
    r = np.array(sorted(known))
    got = O.make_log_bucket_position(r, 256, 512).astype(np.int64)
    assert got.tolist() == [known[int(x)] for x in r]


def test_delta_properties_v3_base():
    R = 9000
    d = O.delta_table(256, 512, R)
    r = np.arange(-R, R + 1)
    assert d.min() == 0 and d.max() == 511 and len(np.unique(d)) == 512
    assert (np.diff(d) >= 0).all()                                  # monotone in r
    lin = np.abs(r) <= 128
    assert (d[lin] == 256 + r[lin]).all()                           # linear zone
    assert (d[r >= 510] == 511).all() and d[r == 500][0] < 511       # saturation, high side
    assert (d[r <= -512] == 0).all() and d[r == -511][0] == 1       # saturation, low side
    # odd symmetry of the bucket itself (what makes the p2c index equal the c2p index)
    b = O.make_log_bucket_position(r, 256, 512)
    assert (b == -b[::-1]).all()


@pytest.mark.parametrize("pb,mr", [(256, 512), (32, 64), (64, 512), (16, 40), (128, 256)])
def test_delta_fp32_equals_fp64(pb, mr):
    a = O.delta_table(pb, mr, 4 * mr, np.float32)
    b = O.delta_table(pb, mr, 4 * mr, np.float64)
    assert (a == b).all()


def test_delta_no_bucketing():
    d = O.delta_table(0, 24, 40)
    r = np.arange(-40, 41)
    assert (d == np.clip(r + 24, 0, 47)).all()


def test_relative_position_ids_golden():
    g = np.load(os.path.join(GOLDEN, "relative_position_ids.npz"))
    for pb, mr in ((256, 512), (32, 64), (64, 512), (-1, -1)):
        col, row = g["col_%d_%d" % (pb, mr)], g["row_%d_%d" % (pb, mr)]
        L = len(col)
        ids = O.build_relative_position(L, L, pb, mr)
        assert (ids[:, 0] == col).all() and (ids[0, :] == row).all()
        assert (ids[1:, 1:] == ids[:-1, :-1]).all()


# ---- attention ---------------------------------------------------------------------------------
def _rand(shape, seed, scale=1.0):
    return np.random.default_rng(seed).standard_normal(shape) * scale


def test_content_only_is_sdpa():
    q, k, v = (_rand((2, 3, 50, 16), s) for s in (1, 2, 3))
    got = O.disentangled_attention(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), scale=1.0 / np.sqrt(16)).numpy()
    assert np.abs(got - ref).max() < 1e-12


def test_zero_rel_embeddings_is_sdpa_at_third_scale():
    q, k, v = (_rand((1, 2, 40, 8), s) for s in (4, 5, 6))
    z = np.zeros((2, 64, 8))
    got = O.disentangled_attention(q, k, v, z, z, 32, 64)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), scale=1.0 / np.sqrt(3 * 8)).numpy()
    assert np.abs(got - ref).max() < 1e-12


@pytest.mark.parametrize("pb,mr,L,c2p,p2c", [(8, 20, 30, True, True), (8, 20, 30, True, False), (8, 20, 30, False, True),
                                             (0, 6, 17, True, True), (16, 40, 48, True, True)])
def test_matches_brute_force(pb, mr, L, c2p, p2c):
    H, D = 2, 8
    span = O.att_span_of(pb, mr)
    q, k, v = (_rand((1, H, L, D), s) for s in (7, 8, 9))
    pk = _rand((H, 2 * span, D), 10) if c2p else None
    pq = _rand((H, 2 * span, D), 11) if p2c else None
    got = O.disentangled_attention(q, k, v, pk, pq, pb, mr)
    ref = O.brute_force_attention(q, k, v, pk, pq, pb, mr)
    assert np.abs(got - ref).max() < 1e-12


def test_row_constant_c2p_is_invisible():
    # all K_r rows equal => c2p adds a per-query constant => softmax unchanged (scale kept at 1/sqrt(3D))
    H, L, D = 1, 33, 8
    q, k, v = (_rand((1, H, L, D), s) for s in (12, 13, 14))
    pq = _rand((H, 64, D), 15)
    pk_const = np.repeat(_rand((H, 1, D), 16), 64, axis=1)
    a = O.disentangled_attention(q, k, v, pk_const, pq, 32, 64)
    b = O.disentangled_attention(q, k, v, np.zeros((H, 64, D)), pq, 32, 64)
    assert np.abs(a - b).max() < 1e-12


def test_constant_q_r_shifts_queries():
    # all Q_r rows equal to rho => k_j.rho added => same as content-only attention with q + rho
    H, L, D = 1, 21, 8
    q, k, v = (_rand((1, H, L, D), s) for s in (17, 18, 19))
    rho = _rand((H, 1, D), 20)
    a = O.disentangled_attention(q, k, v, np.zeros((H, 64, D)), np.repeat(rho, 64, axis=1), 32, 64)
    b = O.disentangled_attention(q + rho[None], k, v, np.zeros((H, 64, D)), np.zeros((H, 64, D)), 32, 64)
    assert np.abs(a - b).max() < 1e-12


def test_varlen_equals_per_sequence_and_padded():
    H, D = 2, 8
    lens = [5, 19, 1, 12]
    cu = np.concatenate([[0], np.cumsum(lens)])
    T = cu[-1]
    q, k, v = (_rand((T, H, D), s) for s in (21, 22, 23))
    pk, pq = _rand((H, 32, D), 24), _rand((H, 32, D), 25)
    packed = O.disentangled_attention_varlen(q, k, v, cu, pk, pq, 16, 40)
    Lm = max(lens)
    pad = lambda x: np.stack([np.concatenate([x[cu[b]:cu[b + 1]], np.zeros((Lm - lens[b], H, D))]) for b in range(4)])
    mask = np.arange(Lm)[None, :] < np.array(lens)[:, None]
    dense = O.disentangled_attention(*(pad(x).transpose(0, 2, 1, 3) for x in (q, k, v)), pk, pq, 16, 40, mask=mask)
    for b in range(4):
        assert np.abs(dense[b, :, :lens[b]].transpose(1, 0, 2) - packed[cu[b]:cu[b + 1]]).max() < 1e-12


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "[a-f]_*.npz"))))
def test_module_forward_matches_golden(path):
    g = np.load(path)
    B, L, hid, H, pb, mr, c2p, p2c, share = g["meta"].tolist()
    weights = {k[2:]: g[k] for k in g.files if k.startswith("w.")}
    pat = (["c2p"] if c2p else []) + (["p2c"] if p2c else [])
    mask = g["mask"].astype(bool)
    out = O.module_forward(g["hidden"], weights, g["rel_embeddings"], H, pat, bool(share), pb, mr,
                           mask=None if mask.all() else mask)
    ref = g["out"]
    valid = mask[:, :, None]
    err = np.abs(np.where(valid, out - ref, 0)).max()
    assert err < 2e-4 * max(1.0, np.abs(ref).max()), err  # the stored vectors are fp32 eager outputs


# ---- backward -----------------------------------------------------------------------------------
@pytest.mark.parametrize("kw", [{}, {"masked": True}, {"causal": True}], ids=["plain", "masked", "causal"])
@pytest.mark.parametrize("terms", [(True, True), (True, False), (False, True), (False, False)], ids=["c2p+p2c", "c2p", "p2c", "content"])
def test_backward_matches_finite_differences(kw, terms):
    """Central differences of the forward oracle, entry by entry, against the analytic gradients (every operand)."""
    rng = np.random.default_rng(50)
    B, H, L, D, pb, mr = 1, 2, 21, 8, 4, 8  # radius 8: linear zone, log zone and both saturated ends inside 21 tokens
    q, k, v, do = [rng.standard_normal((B, H, L, D)) for _ in range(4)]
    pk = rng.standard_normal((H, 2 * pb, D)) if terms[0] else None
    pq = rng.standard_normal((H, 2 * pb, D)) if terms[1] else None
    fkw = {}
    if kw.get("masked"):
        fkw["mask"] = np.arange(L)[None, :] < 17
        do[:, :, 17:] = 0
    if kw.get("causal"):
        fkw["causal"] = True
    grads = O.disentangled_attention_backward(q, k, v, do, pk, pq, pb, mr, **fkw)
    f = lambda: (O.disentangled_attention(q, k, v, pk, pq, pb, mr, **fkw) * do).sum()
    for x, g in zip((q, k, v, pk, pq), grads):
        if x is None:
            assert g is None
            continue
        for _ in range(25):
            idx = tuple(rng.integers(0, n) for n in x.shape)
            old, e = x[idx], 1e-5
            x[idx] = old + e
            fp = f()
            x[idx] = old - e
            fm = f()
            x[idx] = old
            assert abs((fp - fm) / (2 * e) - g[idx]) < 1e-7, (idx, (fp - fm) / (2 * e), g[idx])


class _OracleAttention(torch.autograd.Function):
    """The numpy oracle (forward and backward) as an autograd node, so that torch carries the chain through
    the projections around it."""

    @staticmethod
    def forward(ctx, q, k, v, pk, pq, pb, mr, mask):
        n = lambda x: None if x is None else x.detach().numpy().astype(np.float64)
        ctx.save_for_backward(q, k, v, *(x for x in (pk, pq) if x is not None))
        ctx.cfg = (pk is not None, pq is not None, pb, mr, mask)
        return torch.from_numpy(O.disentangled_attention(n(q), n(k), n(v), n(pk), n(pq), pb, mr, mask=mask))

    @staticmethod
    def backward(ctx, dout):
        has_pk, has_pq, pb, mr, mask = ctx.cfg
        saved = [x.numpy().astype(np.float64) for x in ctx.saved_tensors]
        q, k, v = saved[:3]
        pk = saved[3] if has_pk else None
        pq = saved[3 + has_pk] if has_pq else None
        g = O.disentangled_attention_backward(q, k, v, dout.numpy(), pk, pq, pb, mr, mask=mask)
        t = lambda x: None if x is None else torch.from_numpy(x)
        return t(g[0]), t(g[1]), t(g[2]), t(g[3]), t(g[4]), None, None, None


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "g_*.npz"))))
def test_backward_matches_golden_gradients(path):
    """Gradients torch.autograd wrote through the third-party eager class (hidden states, relative embeddings,
    every weight) against the oracle's backward, with torch carrying the chain through the projections."""
    g = np.load(path)
    B, L, hid, H, pb, mr, c2p, p2c, share = g["meta"].tolist()
    D = hid // H
    W = {k[2:]: torch.tensor(g[k], dtype=torch.float64, requires_grad=True) for k in g.files if k.startswith("w.")}
    hidden = torch.tensor(g["hidden"], dtype=torch.float64, requires_grad=True)
    rel = torch.tensor(g["rel_embeddings"], dtype=torch.float64, requires_grad=True)
    lin = lambda x, n: torch.nn.functional.linear(x, W[n + ".weight"], W.get(n + ".bias"))
    heads = lambda x: x.view(*x.shape[:-1], H, D).transpose(-2, -3)  # [..., L, H*D] -> [..., H, L, D]
    q, k, v = heads(lin(hidden, "query_proj")), heads(lin(hidden, "key_proj")), heads(lin(hidden, "value_proj"))
    pk = heads(lin(rel, "key_proj" if share else "pos_key_proj")) if c2p else None
    pq = heads(lin(rel, "query_proj" if share else "pos_query_proj")) if p2c else None
    mask = g["mask"].astype(bool)
    out = _OracleAttention.apply(q, k, v, pk, pq, pb, mr, None if mask.all() else mask)
    out = out.transpose(1, 2).reshape(B, L, hid)
    assert np.abs(np.where(mask[:, :, None], out.detach().numpy() - g["out"], 0)).max() < 2e-4 * max(1.0, np.abs(g["out"]).max())
    (out * torch.from_numpy(g["gout"].astype(np.float64))).sum().backward()
    got = {"hidden": hidden.grad, "rel_embeddings": rel.grad, **{"w." + n: t.grad for n, t in W.items()}}
    for name, t in got.items():
        ref = g["g." + name]
        val = np.zeros_like(ref) if t is None else t.numpy()
        err = np.abs(val - ref).max()
        assert err < 2e-4 * max(1.0, np.abs(ref).max()), (name, err, np.abs(ref).max())  # fp32 autograd vs fp64


# ---- fp8 ---------------------------------------------------------------------------------------
def test_e4m3_round_matches_torch():
    x = np.concatenate([_rand(20000, 30, 100.0), _rand(20000, 31, 1.0), _rand(20000, 32, 0.01),
                        np.array([0.0, 448.0, -448.0, 447.9, 1e-4, 2.0 ** -9, 2.0 ** -10, 0.0175])]).astype(np.float32)
    x = np.clip(x, -448, 448)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn)
    got = O.e4m3_round(x)
    assert (got == ref.float().numpy()).all()
    assert (O.e4m3_encode(got) == ref.view(torch.uint8).numpy()).all()


def test_quantize_per_head_scale():
    x = _rand((50, 3, 16), 33).astype(np.float32)
    y, s = O.quantize_e4m3_per_head(x)
    assert np.allclose(s, np.abs(x).max(axis=(0, 2)) / 448.0, rtol=1e-7)
    assert np.abs(y).max() == 448.0
    assert np.abs(y * s[None, :, None] - x).max() <= np.abs(x).max() / 16  # half a step of the top binade
