#!/usr/bin/env python3
"""Benchmark of the fused disentangled-attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

A step is one launch of the fused kernel over one batch of synthetic, HBM-resident inputs.
Default workload = the shape the headline metric is quoted on: DeBERTa-v3-base attention
(12 heads x 64), sequence 4096, bf16, batch 8, position_buckets 256.  Prints ONE JSON line.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

WORKLOADS = {
    # name: (B, L, H, D, dtype, kind)
    "v3base_L4096_B8_bf16": (8, 4096, 12, 64, "bf16", "fixed"),
    "v3base_L4096_B1_bf16": (1, 4096, 12, 64, "bf16", "fixed"),
    "v3base_L512_B8_bf16": (8, 512, 12, 64, "bf16", "fixed"),
    "v3large_L4096_B1_bf16": (1, 4096, 16, 64, "bf16", "fixed"),
    "v3base_varlen64_bf16": (64, 2048, 12, 64, "bf16", "varlen"),
    "v3base_L8192_B4_fp8": (4, 8192, 12, 64, "fp8", "fixed"),
    "v3base_L512_B1_fp32": (1, 512, 12, 64, "fp32", "fixed"),
}
S2 = 512  # 2 * position_buckets


def flops(lens, H, D, pos=True):
    """Algorithmic FLOPs: QK^T + PV (4 L^2 D) plus each position product once (4 L 2S D), per head."""
    return sum(H * (4 * l * l * D + (4 * l * S2 * D if pos else 0)) for l in lens)


def make_inputs(name, device):
    from flashdeberta_amd import ops
    B, L, H, D, dt, kind = WORKLOADS[name]
    g = torch.Generator(device=device).manual_seed(1234)
    tdt = {"bf16": torch.bfloat16, "fp8": torch.bfloat16, "fp32": torch.float32}[dt]
    rnd = lambda *s: (torch.randn(*s, device=device, generator=g) * 0.02).to(tdt)
    pk, pq = rnd(H, S2, D), rnd(H, S2, D)
    kw = dict(position_buckets=256, max_relative_positions=512)
    if kind == "varlen":
        u = torch.rand(B, generator=torch.Generator().manual_seed(1004))
        lens = torch.exp(math.log(32) + u * (math.log(2048) - math.log(32))).round().to(torch.int64).tolist()
        T = sum(lens)
        q, k, v = rnd(T, H, D), rnd(T, H, D), rnd(T, H, D)
        cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=device)
        kw.update(cu_seqlens=cu, max_seqlen=max(lens))
    else:
        lens = [L] * B
        q, k, v = rnd(B, L, H, D), rnd(B, L, H, D), rnd(B, L, H, D)
    if dt == "fp8":
        m = torch.rand(q.shape, device=device, generator=g) < 0.01
        q = torch.where(m, q * 20, q)
        m = torch.rand(k.shape, device=device, generator=g) < 0.01
        k = torch.where(m, k * 20, k)
        q, kw["q_scale"] = ops.quantize_e4m3_per_head(q)
        k, kw["k_scale"] = ops.quantize_e4m3_per_head(k)
        pk8, kw["pos_key_scale"] = ops.quantize_e4m3_per_head(pk.transpose(0, 1))
        pq8, kw["pos_query_scale"] = ops.quantize_e4m3_per_head(pq.transpose(0, 1))
        pk, pq = pk8.transpose(0, 1), pq8.transpose(0, 1)
    out = torch.empty(q.shape, dtype=v.dtype, device=device)
    return (q, k, v, pk, pq), kw, out, lens


def measured_traffic(workload, with_source=False):
    """HBM bytes per step as measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), scaled by the
    copy-calibration kernel; recorded in profiles/hbm_traffic.json by hand from those runs (the counters
    cannot be read from inside this process).  None if the workload has not been measured.  With
    with_source also where the figure comes from: it is replayed from that file, not measured in this run."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f).get(workload, {})
    except (OSError, ValueError):
        rec = {}
    val = rec.get("bytes_per_step")
    if not with_source:
        return val
    src = None if val is None else "replayed from profiles/hbm_traffic.json (rocprofv3 --pmc runs of %s)" % rec.get("measured", "unknown date")
    return val, src


def tile_census(lens, R=512, BM=128, BN=64):
    """(far, near) key tiles of 64 summed over the 128-row query tiles of sequences of the given lengths:
    a key tile is far for a query tile when every |i - j| in it is at least R, the radius beyond which
    the bucketed relative position is constant (512 for 256 buckets / 512 positions)."""
    far = near = 0
    for L in lens:
        n_tiles = (L + BN - 1) // BN
        for m0 in range(0, L, BM):
            lim = m0 - (BN - 1) - R
            t0 = min(n_tiles, lim // BN + 1) if lim >= 0 else 0
            t1 = max(t0, min(n_tiles, (m0 + BM - 1 + R + BN - 1) // BN))
            near += t1 - t0
            far += n_tiles - (t1 - t0)
    return far, near


def cpu_baseline(H, D, L):
    """The CPU oracle (numpy restatement of the eager path, fp32) on a bounded sample of the same
    workload: one batch element, as many heads as fit in roughly 10-30 s."""
    from oracle import disentangled_oracle as O
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] + [1])
    except Exception:
        threads = os.cpu_count() or 1
    rng = np.random.default_rng(0)
    mk = lambda *s: (rng.standard_normal(s) * 0.02).astype(np.float32)
    q, k, v = mk(1, 1, L, D), mk(1, 1, L, D), mk(1, 1, L, D)
    pk, pq = mk(1, S2, D), mk(1, S2, D)
    run = lambda: O.disentangled_attention(q, k, v, pk, pq, 256, 512, dtype=np.float32)
    t0 = time.perf_counter()
    run()
    one = time.perf_counter() - t0
    heads = int(max(1, min(H, 15.0 // max(one, 1e-3))))
    t0 = time.perf_counter()
    for _ in range(heads):
        run()
    dt = time.perf_counter() - t0
    fl = flops([L], heads, D)
    port = {"value": round(fl / dt / 1e12, 5), "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
            "sample": "numpy fp32 oracle, %d of %d heads of one batch element at L=%d (%.1f s), %.0f tokens/s per layer"
                      % (heads, H, L, dt, L / (dt / heads * H))}
    # The headline CPU figure is the reference's own CPU path: the class behind its "eager" key
    # (src/flashdeberta/model.py:255).  The numpy port rides along as the secondary figure, and takes the
    # headline only where transformers cannot be imported or its module signature has changed.
    try:
        eager = eager_module_cpu(H, D, L)
    except Exception as e:
        eager = {"error": "%s: %s" % (type(e).__name__, str(e)[:200])}
    if eager is not None and "value" in eager:
        rec = dict(eager, kind="reference")
        rec["port"] = port
        return rec
    if eager is not None:
        port["eager_module"] = eager
    return port


def eager_module_cpu(H, D, L):
    """transformers' DisentangledSelfAttention -- the class behind the reference's "eager" key
    (src/flashdeberta/model.py:255) -- on the host cores: one fp32 forward of one batch element, module
    level (its three input projections and the two relative-embedding projections included), priced with
    the attention FLOPs only.  None where transformers is not importable."""
    try:
        from transformers.models.deberta_v2.modeling_deberta_v2 import DisentangledSelfAttention
    except Exception:
        return None

    class Cfg:
        hidden_size, num_attention_heads = H * D, H
        attention_probs_dropout_prob = hidden_dropout_prob = 0.0
        pos_att_type = ["c2p", "p2c"]
        relative_attention, position_buckets, max_relative_positions = True, 256, 512
        max_position_embeddings, share_att_key = 512, True

    torch.manual_seed(0)
    att = DisentangledSelfAttention(Cfg()).eval()
    x = torch.randn(1, L, H * D) * 0.02
    rel = torch.randn(S2, H * D) * 0.02
    mask = torch.ones(1, 1, L, L, dtype=torch.bool)
    with torch.no_grad():
        small = slice(0, 256)
        att(x[:, small], mask[:, :, small, small], rel_embeddings=rel)  # warm-up
        t0 = time.perf_counter()
        att(x, mask, rel_embeddings=rel)  # builds its own relative positions, as the encoder would once per forward
        dt = time.perf_counter() - t0
    return {"value": round(flops([L], H, D) / dt / 1e12, 5), "unit": "TFLOP/s", "cores": int(torch.get_num_threads()),
            "sample": "transformers %s DisentangledSelfAttention.forward (the reference's eager path), fp32, one batch "
                      "element at L=%d, all %d heads (%.1f s), %.0f tokens/s per layer"
                      % (__import__("transformers").__version__, L, H, dt, L / dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="v3base_L4096_B8_bf16", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-settle", action="store_true", help="skip the untimed settle phase before the warm-up")
    ap.add_argument("--backward", action="store_true",
                    help="time forward + backward through the autograd node instead (fixed-layout 16-bit / fp32 workloads); "
                         "priced at 3.5 x the forward's algorithmic FLOPs (two products forward, five backward)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="also run one device-to-device copy of this many MiB (a kernel of known HBM traffic "
                         "against which rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU only (the path is independent per (sequence, head, "
                 "q-tile) and uses no collectives); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    from flashdeberta_amd import ops

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    B, L, H, D, dt, kind = WORKLOADS[args.workload]
    tensors, kw, out, lens = make_inputs(args.workload, device)
    step = lambda: ops.disentangled_attention_fwd(*tensors, out=out, **kw)
    if args.backward:
        if kind != "fixed" or dt == "fp8":
            sys.exit("bench.py --backward: the backward exists for the fixed layout in fp32 / bf16 / fp16")
        leaves = [t.detach().clone().requires_grad_(True) for t in tensors]
        dout = torch.randn_like(out) * 0.02

        def step():
            for t in leaves:
                t.grad = None
            ops.disentangled_attention(*leaves, **kw).backward(dout)
    if args.copy_calibration:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)
    def timed(warmup, steps):
        """(wall ms per step, HIP-event ms per step) of `steps` steps after `warmup` untimed ones."""
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record()  # same stream the kernel is launched on (torch's current stream)
        for _ in range(steps):
            step()
        ev1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps, ev0.elapsed_time(ev1) / steps

    # First the plain reading of the flags: W warm-up steps, K timed steps, straight from idle (`unsettled` in the
    # JSON line).  The first ~100 ms after idle run a few percent slower (clocks and power management), and a short
    # timed region (20 steps are 15 ms) measures that ramp instead of the kernels.  So an untimed settle phase
    # follows -- batches of steps until a batch is no faster than the one before (within 1 %), for at most 0.5 s,
    # reported as settle_ms -- and then W warm-up + K timed steps once more: `value`.
    cold_wall_ms, cold_kern_ms = timed(args.warmup, args.steps)
    settle_t0 = time.perf_counter()
    if not args.no_settle:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        prev = None
        while time.perf_counter() - settle_t0 < 0.5:
            e0.record()
            for _ in range(10):
                step()
            e1.record()
            torch.cuda.synchronize()
            cur = e0.elapsed_time(e1)
            if prev is not None and cur >= prev * 0.99:
                break
            prev = cur
    settle_ms = (time.perf_counter() - settle_t0) * 1e3
    wall_ms, kern_ms = (cold_wall_ms, cold_kern_ms) if args.no_settle else timed(args.warmup, args.steps)
    fl = flops(lens, H, D) * (3.5 if args.backward else 1.0)
    tokens = sum(lens)
    # e4m3 operands: the three score products (q.k, q.K_r, k.Q_r) are e4m3 MFMA contractions, P V is bf16.  The step is
    # priced against the blended bound t_min = F_fp8 / peak_fp8 + F_bf16 / peak_bf16, i.e. peak = F / t_min.
    arith = dt
    if dt == "fp8":
        f_bf16 = sum(H * 2 * l * l * D for l in lens)            # P V
        f_fp8 = flops(lens, H, D) - f_bf16                       # Q K^T and the two position products
        peak = flops(lens, H, D) / (f_fp8 / PEAK_TFLOPS["fp8"] + f_bf16 / PEAK_TFLOPS["bf16"])
    else:
        peak = PEAK_TFLOPS[arith]
    achieved = fl / (kern_ms * 1e-3) / 1e12
    # the two launches of a step timed one at a time (same stream, HIP events), priced with the FLOPs of the
    # tiles each walks: content products of its tiles; the position products belong to the near launch
    kernels = None
    if dt != "fp32" and D == 64 and not args.backward:
        far_t, near_t = tile_census(lens)
        split = {}
        for name, mask in (("far", 1), ("near", 2)):
            run = lambda: ops.disentangled_attention_fwd(*tensors, out=out, _part=mask, **kw)
            if (far_t if name == "far" else near_t) == 0:
                continue
            for _ in range(5):
                run()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            n = max(5, min(args.steps, 50))
            for _ in range(n):
                run()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / n
            tiles = far_t if name == "far" else near_t
            if tiles == 0:
                continue
            gf = H * (4.0 * 128 * 64 * D * tiles + (4.0 * sum(lens) * S2 * D if name == "near" else 0.0)) / 1e9
            split[name] = {"ms": round(ms, 4), "gflop": round(gf, 2), "frac_of_peak": round(gf / ms / peak, 4),
                           "key_tiles": tiles}
        kernels = split
    traffic, traffic_source = measured_traffic(args.workload, with_source=True)
    rec = {
        "metric": "disentangled_attn_fwd_bwd_tflops" if args.backward else "disentangled_attn_fwd_tflops", "value": round(fl / (wall_ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4),
        "settle_ms": round(settle_ms, 1),
        "unsettled": {"value": round(fl / (cold_wall_ms * 1e-3) / 1e12, 2), "ms_per_step": round(cold_wall_ms, 4),
                      "kernel_ms": round(cold_kern_ms, 4),
                      "note": "the same warm-up and steps straight from idle, before the settle phase"},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": arith, "data": "synthetic",
        "tokens_per_s": round(tokens / (wall_ms * 1e-3), 1),
        "content_only_tflops": round(sum(H * 4 * l * l * D for l in lens) / (wall_ms * 1e-3) / 1e12, 2),
        "config": {"workload": args.workload, "batch": B, "seq_len": L if kind == "fixed" else "varlen(%d tokens)" % tokens,
                   "heads": H, "head_dim": D, "position_buckets": 256, "pos_att_type": "c2p|p2c", "layout": kind},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": round(peak, 1), "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel_ms": round(kern_ms, 4), "algorithmic_gflop_per_launch": round(fl / 1e9, 2),
                     "launches": kernels},
    }
    if dt == "fp8":
        rec["config"]["operands"] = "q, k, K_r, Q_r in OCP e4m3 with per-head fp32 scales; v and P bf16"
        rec["roofline"]["peak_note"] = ("blended: (Q K^T + position products) at the 5.0 PFLOP/s fp8 peak + P V at the "
                                        "2.5 PFLOP/s bf16 peak")
    if not args.no_cpu:
        rec["cpu_baseline"] = cpu_baseline(H, D, min(L, 4096))
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
