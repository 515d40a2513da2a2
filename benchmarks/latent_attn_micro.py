"""Latent attention kernel alone: prefill tiles and decode rows at model-sized shapes.

    python benchmarks/latent_attn_micro.py [--heads 32] [--rank 512] [--rot 64] [--prompt 4096] [--seqs 2]
                                           [--batch 32] [--context 2048]

Prints one JSON line per case: time per launch, matrix-core FLOP/s (both products, causal pairs only) and,
for decode, the rate at which cache entries are read.
"""
import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from vllm_production_stack_amd import ops  # noqa: E402

PAGE = 64


def timed(fn, iters=20):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e3  # us


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--rank", type=int, default=512)
    ap.add_argument("--rot", type=int, default=64)
    ap.add_argument("--prompt", type=int, default=4096)
    ap.add_argument("--seqs", type=int, default=2)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--context", type=int, default=2048)
    a = ap.parse_args()
    dev = torch.device("cuda")
    h, rank, rot = a.heads, a.rank, a.rot
    entry = rank + rot
    g = torch.Generator(device=dev).manual_seed(0)
    sink = torch.zeros(h, dtype=torch.float32, device=dev)

    def pool_for(n_seqs, length):
        per = (length + PAGE - 1) // PAGE
        pool = (torch.randn((n_seqs * per, PAGE * entry), generator=g, device=dev) * 0.3).to(torch.bfloat16)
        bt = torch.randperm(n_seqs * per, device=dev, generator=g).int().view(n_seqs, per)
        return pool, bt

    # prefill: whole prompts
    n = a.seqs * a.prompt
    pool, bt = pool_for(a.seqs, a.prompt)
    q = (torch.randn((n, h, entry), generator=g, device=dev) * 0.3).to(torch.bfloat16)
    pos = torch.arange(a.prompt, dtype=torch.int32, device=dev).repeat(a.seqs)
    seq = torch.arange(a.seqs, dtype=torch.int32, device=dev).repeat_interleave(a.prompt)
    tiles = torch.from_numpy(ops.build_latent_tiles([a.prompt] * a.seqs, [a.prompt] * a.seqs, h)).to(dev)
    out = torch.empty((n, h, rank), dtype=torch.bfloat16, device=dev)
    us = timed(lambda: ops.latent_attention(q[:, :, :rank], q[:, :, rank:], pool, 0, bt, seq, pos, sink, 0.07, out=out,
                                            tiles=tiles), iters=5)
    pairs = a.seqs * a.prompt * (a.prompt + 1) / 2
    flop = pairs * h * 2 * (entry + rank)
    print(json.dumps({"case": "prefill", "tokens": n, "heads": h, "rank": rank, "rot": rot, "us": round(us, 1),
                      "tflops": round(flop / us / 1e6, 1)}), flush=True)
    # decode
    pool, bt = pool_for(a.batch, a.context)
    q = (torch.randn((a.batch, h, entry), generator=g, device=dev) * 0.3).to(torch.bfloat16)
    pos = torch.full((a.batch,), a.context - 1, dtype=torch.int32, device=dev)
    out = torch.empty((a.batch, h, rank), dtype=torch.bfloat16, device=dev)
    for splits in (1, 4, 8, 16):
        us = timed(lambda: ops.latent_attention(q[:, :, :rank], q[:, :, rank:], pool, 0, bt, None, pos, sink, 0.07, out=out,
                                                splits=splits))
        byts = a.batch * a.context * entry * 2
        flop = a.batch * a.context * h * 2 * (entry + rank)
        print(json.dumps({"case": "decode", "batch": a.batch, "context": a.context, "splits": splits, "us": round(us, 1),
                          "tb_s": round(byts / us / 1e6, 2), "tflops": round(flop / us / 1e6, 1)}), flush=True)


if __name__ == "__main__":
    main()
