"""The entry point that allocates nothing (fdb_attn_fwd_noalloc), called through the C ABI: same output as
fdb_attn_fwd on two calls in a row, the second with a smaller input, in the fixed and the packed layout."""
import gc

import numpy as np
import pytest
import torch

from flashdeberta_amd import ops

pytestmark = pytest.mark.gpu


def _inputs(shape, H, D, pb, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(*shape, H, D, generator=g).to(torch.bfloat16).cuda() for _ in range(3)]
    pk, pq = [torch.randn(H, 2 * pb, D, generator=g).to(torch.bfloat16).cuda() for _ in range(2)]
    return q, k, v, pk, pq


def test_no_alloc_entry_point_matches_the_allocating_one():
    pb, mr = 256, 512
    # first call: one sequence of 1500 (far keys and near steps shared out: hand-over, partial results and the
    # merge kernel all run out of the scratch); second call: smaller, on the scratch the first one left behind
    for B, L, H in ((1, 1500, 3), (2, 700, 2)):
        t = _inputs((B, L), H, 64, pb, 100 + L)
        kw = dict(position_buckets=pb, max_relative_positions=mr)
        ref = ops.disentangled_attention_fwd(*t, **kw)
        out = torch.empty_like(ref)
        gc.collect()
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        got = ops.disentangled_attention_fwd(*t, out=out, no_alloc=True, **kw)
        assert torch.cuda.max_memory_allocated() == before  # nothing came from torch's allocator either
        torch.cuda.synchronize()
        assert got is out and torch.equal(out, ref), (out.float() - ref.float()).abs().max().item()
    # packed layout: the work-list is built into the scratch as well; again a larger call, then a smaller one
    for lens in ([900, 40, 333], [130, 64]):
        T = sum(lens)
        t = _inputs((T,), 2, 64, 32, 200 + T)
        cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device="cuda")
        kw = dict(cu_seqlens=cu, max_seqlen=max(lens), position_buckets=32, max_relative_positions=64)
        ref, ref_lse = ops.disentangled_attention_fwd(*t, return_lse=True, **kw)
        out, lse = ops.disentangled_attention_fwd(*t, no_alloc=True, return_lse=True, **kw)  # caller-owned lse is filled
        torch.cuda.synchronize()
        assert torch.equal(out, ref) and torch.equal(lse, ref_lse)
        out2 = ops.disentangled_attention_fwd(*t, no_alloc=True, **kw)  # hand-over from the scratch
        assert torch.equal(out2, ref)
