"""Writes tests/golden/*.npz: input/output vectors of the eager attention.

The eager side of the reference's switch is transformers' DisentangledSelfAttention
(reference src/flashdeberta/model.py:255), a third-party class that ships in this image
(transformers 5.15.0), built from a plain config object the way the reference's own test does
(tests/attention.py:6-18,52).  This script runs that class on CPU in fp32 with seeded inputs and
stores inputs, weights and outputs, plus the relative-position ids of
transformers' build_relative_position, and for the g_* cases the gradients torch.autograd computes
through the class for a seeded upstream gradient (hidden states, relative embeddings, every weight).  Run from the repo root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
from transformers.models.deberta_v2.modeling_deberta_v2 import DisentangledSelfAttention, build_relative_position

HERE = os.path.dirname(os.path.abspath(__file__))


class Cfg:
    def __init__(self, hidden_size, heads, position_buckets, max_relative_positions, pos_att_type, share_att_key):
        self.hidden_size = hidden_size
        self.num_attention_heads = heads
        self.attention_probs_dropout_prob = 0.1
        self.hidden_dropout_prob = 0.1
        self.pos_att_type = pos_att_type
        self.relative_attention = True
        self.position_buckets = position_buckets
        self.max_relative_positions = max_relative_positions
        self.max_position_embeddings = 512
        self.share_att_key = share_att_key


CASES = {
    # name: (B, L, hidden, heads, buckets, max_rel, pos_att_type, share_att_key, lengths or None, input scale)
    "a_L16_b32": (1, 16, 128, 2, 32, 64, ["c2p", "p2c"], True, None, 1.0),
    "b_L130_b32_masked": (2, 130, 128, 2, 32, 64, ["c2p", "p2c"], False, [130, 77], 1.0),
    "c_L600_b256": (1, 600, 128, 2, 256, 512, ["c2p", "p2c"], True, None, 1.0),
    "d_L40_nobucket_c2p": (1, 40, 64, 1, 0, 24, ["c2p"], False, None, 1.0),
    "e_L70_b32_p2c": (2, 70, 64, 2, 32, 64, ["p2c"], False, None, 1.0),
    "f_L96_b256_small": (1, 96, 256, 4, 256, 512, ["c2p", "p2c"], True, None, 0.02),
}


GRAD_CASES = {
    # name: (B, L, hidden, heads, buckets, max_rel, pos_att_type, share_att_key, lengths or None)
    "g_L48_b8_share": (2, 48, 64, 2, 8, 16, ["c2p", "p2c"], True, None),
    "g_L150_b32_masked": (2, 150, 128, 2, 32, 64, ["c2p", "p2c"], False, [150, 101]),
    "g_L40_b8_c2p": (1, 40, 64, 2, 8, 16, ["c2p"], False, None),
}


def grad_cases():
    for idx, (name, (B, L, hid, H, pb, mr, pat, share, lens)) in enumerate(GRAD_CASES.items()):
        torch.manual_seed(2000 + idx)
        mod = DisentangledSelfAttention(Cfg(hid, H, pb, mr, pat, share)).eval()
        with torch.no_grad():
            for p in mod.parameters():
                p.normal_(0.0, 0.2)
        hidden = torch.randn(B, L, hid, requires_grad=True)
        rel = torch.randn(2 * pb, hid, requires_grad=True)
        mask2d = torch.ones(B, L)
        if lens is not None:
            for b, n in enumerate(lens):
                mask2d[b, n:] = 0
        ext = mask2d.unsqueeze(1).unsqueeze(2)
        ext = ext * ext.squeeze(-2).unsqueeze(-1)
        out = mod(hidden, ext, rel_embeddings=rel)[0]
        gout = torch.randn_like(out) * mask2d[:, :, None]  # nothing flows back from padded rows
        (out * gout).sum().backward()
        data = {"hidden": hidden.detach().numpy(), "rel_embeddings": rel.detach().numpy(),
                "mask": mask2d.numpy().astype(np.uint8), "out": out.detach().numpy(), "gout": gout.numpy(),
                "g.hidden": hidden.grad.numpy(), "g.rel_embeddings": rel.grad.numpy(),
                "meta": np.array([B, L, hid, H, pb, mr, int("c2p" in pat), int("p2c" in pat), int(share)], dtype=np.int64)}
        for k, v in mod.named_parameters():
            data["w." + k] = v.detach().numpy()
            data["g.w." + k] = (v.grad if v.grad is not None else torch.zeros_like(v)).numpy()
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
        print(name, out.shape, float(hidden.grad.abs().max()))


def main():
    grad_cases()
    for idx, (name, (B, L, hid, H, pb, mr, pat, share, lens, scale)) in enumerate(CASES.items()):
        torch.manual_seed(1000 + idx)
        cfg = Cfg(hid, H, pb, mr, pat, share)
        mod = DisentangledSelfAttention(cfg).eval()
        with torch.no_grad():
            for p in mod.parameters():
                p.normal_(0.0, 0.3 if scale == 1.0 else 0.02)
        span = pb if pb > 0 else mr
        hidden = torch.randn(B, L, hid) * (1.0 if scale == 1.0 else 1.0)
        rel = torch.randn(2 * span, hid) * (1.0 if scale == 1.0 else 1.0)
        mask2d = torch.ones(B, L)
        if lens is not None:
            for b, n in enumerate(lens):
                mask2d[b, n:] = 0
        ext = mask2d.unsqueeze(1).unsqueeze(2)
        ext = ext * ext.squeeze(-2).unsqueeze(-1)
        with torch.no_grad():
            out = mod(hidden, ext, rel_embeddings=rel)[0]
        data = {"hidden": hidden.numpy(), "rel_embeddings": rel.numpy(), "mask": mask2d.numpy().astype(np.uint8),
                "out": out.numpy(),
                "meta": np.array([B, L, hid, H, pb, mr, int("c2p" in pat), int("p2c" in pat), int(share)], dtype=np.int64)}
        for k, v in mod.state_dict().items():
            data["w." + k] = v.numpy()
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
        print(name, out.shape, float(out.abs().max()))
    # relative-position ids: Toeplitz, so the first column (r >= 0) and first row (r <= 0) hold everything
    rp = {}
    for pb, mr, L in ((256, 512, 1400), (32, 64, 300), (64, 512, 1400), (-1, -1, 50)):
        x = torch.zeros(1, L, 1)
        ids = build_relative_position(x, x, bucket_size=pb, max_position=mr)[0]
        assert bool((ids[1:, 1:] == ids[:-1, :-1]).all())  # depends on i - j only
        rp["col_%d_%d" % (pb, mr)] = ids[:, 0].numpy()
        rp["row_%d_%d" % (pb, mr)] = ids[0, :].numpy()
    np.savez_compressed(os.path.join(HERE, "relative_position_ids.npz"), **rp)


if __name__ == "__main__":
    main()
