#!/usr/bin/env python3
"""latent_attn alone: the prompt form (64-row tiles) and the decode form (split-KV) on shapes of a real layer.

Reports microseconds per launch, achieved TFLOP/s (2 * (Dk + r) flops per visible (query vector, key) pair) and the
cache bytes per second the decode form streams.  --impl 1 times the one-wave-per-(row, head) kernel instead.

  python bench/kernels/bench_latent_attn.py --seqs 8 --len 1024 --heads 16 --kv-rank 512 --rot 64
"""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))

import torch

from symmetry_amd import ops


def _time(fn, reps):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / reps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--seqs", type=int, default=8)
    ap.add_argument("--len", type=int, default=1024)
    ap.add_argument("--heads", type=int, default=16)
    ap.add_argument("--kv-rank", type=int, default=512)
    ap.add_argument("--rot", type=int, default=64)
    ap.add_argument("--impl", type=int, default=0)
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--forms", default="prompt,decode")
    a = ap.parse_args()
    dev, bs = "cuda", 64
    S, L, H, r, Dk = a.seqs, a.len, a.heads, a.kv_rank, a.kv_rank + a.rot
    nblk = -(-L // bs)
    g = torch.Generator().manual_seed(0)
    cache = torch.randn(S * nblk + 1, bs, Dk, generator=g).to(torch.bfloat16).to(dev)
    table = (torch.randperm(S * nblk, generator=g) + 1).int().view(S, nblk).to(dev)
    out = {"seqs": S, "len": L, "heads": H, "kv_rank": r, "rot": a.rot, "impl": a.impl}
    if "prompt" in a.forms:
        T = S * L
        q = (torch.randn(T, H, Dk, generator=g) * 0.1).to(torch.bfloat16).to(dev)
        pos = torch.arange(L).repeat(S).int().to(dev)
        row_seq = torch.arange(S).repeat_interleave(L).int().to(dev)
        cu = (torch.arange(S + 1) * L).int().to(dev)
        tiles = torch.tensor(sorted(((s, o) for s in range(S) for o in range(0, L, 64)), key=lambda t: -t[1]),
                             dtype=torch.int32).to(dev)
        o = torch.zeros(T, H, r, dtype=torch.bfloat16, device=dev)
        us = _time(lambda: ops.latent_attn(q, cache, table, row_seq, pos, 0.1, r, o, None, None, tiles, cu, a.impl), a.reps)
        pairs = S * H * L * (L + 1) / 2
        out["prompt_us"] = round(us, 1)
        out["prompt_tflops"] = round(2 * (Dk + r) * pairs / us / 1e6, 1)
    if "decode" in a.forms:
        q = (torch.randn(S, H, Dk, generator=g) * 0.1).to(torch.bfloat16).to(dev)
        pos = torch.full((S,), L - 1, dtype=torch.int32, device=dev)
        row_seq = torch.arange(S).int().to(dev)
        parts = ops.latent_attn_parts(S, nblk * bs)
        po = torch.zeros(S, H, parts, r, device=dev)
        pml = torch.zeros(S, H, parts, 2, device=dev)
        o = torch.zeros(S, H, r, dtype=torch.bfloat16, device=dev)
        us = _time(lambda: ops.latent_attn(q, cache, table, row_seq, pos, 0.1, r, o, po if parts > 1 else None,
                                           pml if parts > 1 else None, None, None, a.impl), a.reps * 5)
        out["decode_us"] = round(us, 1)
        out["decode_parts"] = parts
        out["decode_cache_GBps"] = round(S * L * Dk * 2 / us / 1e3, 1)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
