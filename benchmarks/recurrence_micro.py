"""Times ``ops.recurrent_scan`` alone on prefill-sized chunks: fixed decay (plain and folded into the staged
block) and gated, for several piece counts.

    python benchmarks/recurrence_micro.py [--heads 16] [--dim 128] [--vdim 256] [--rows 4096] [--seqs 2] [--targets 48,96,128]

``VPSA_SCAN_ROWS=8|16|32`` forces the state rows a lane holds (A/B runs of the register tile).  One JSON line per case.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from vllm_production_stack_amd import ops  # noqa: E402


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--heads", type=int, default=16)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--vdim", type=int, default=256)
    ap.add_argument("--rows", type=int, default=4096, help="rows per sequence")
    ap.add_argument("--seqs", type=int, default=2)
    ap.add_argument("--targets", default="48,96,128", help="piece counts to aim for (ops.build_scan_pieces)")
    ap.add_argument("--repeats", type=int, default=5)
    a = ap.parse_args()
    dev = torch.device("cuda")
    heads, dim, vdim = a.heads, a.dim, a.vdim
    lens = [a.rows] * a.seqs
    t = sum(lens)
    g = torch.Generator().manual_seed(0)
    proj = (torch.randn(t, heads * (2 * dim + vdim), generator=g) * 0.3).bfloat16().to(dev)
    decay = torch.full((heads,), 0.97).to(dev)
    table = ops.build_cos_sin(dim, a.rows, 10000.0).to(dev)
    bias, lower = torch.randn(heads * dim).to(dev), (torch.rand(heads * dim) * 0.9).to(dev)
    state = torch.zeros(a.seqs, heads * dim * vdim, device=dev)
    cu = torch.tensor([i * a.rows for i in range(a.seqs + 1)], dtype=torch.int32, device=dev)
    slots = torch.arange(a.seqs, dtype=torch.int32, device=dev)
    pos = torch.cat([torch.arange(a.rows)] * a.seqs).int().to(dev)
    cols = (0, heads * dim, 2 * heads * dim)
    rope = dict(decay=decay, cos_sin=table, rot_dims=dim, layout=0, k_scale=dim ** -0.5)
    cases = (("decay", rope), ("decay_folded", dict(rope, min_decay=0.97)), ("gated", dict(gate_bias=bias, gate_lower=lower)))
    for target in [int(x) for x in a.targets.split(",") if x]:
        cut = ops.build_scan_pieces(lens, target=target)
        pieces = None if cut is None else tuple(torch.from_numpy(x).to(dev) for x in cut)
        for name, kw in cases:
            for _ in range(2):
                ops.recurrent_scan(proj, *cols, heads, dim, vdim, state, 0, cu, slots, pos, pieces=pieces, **kw)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(a.repeats):
                ops.recurrent_scan(proj, *cols, heads, dim, vdim, state, 0, cu, slots, pos, pieces=pieces, **kw)
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) / a.repeats * 1e3
            print(json.dumps({"case": name, "rows": t, "heads": heads, "dim": dim, "vdim": vdim,
                              "pieces": 0 if cut is None else int(cut[0].shape[0]),
                              "piece_rows": 0 if cut is None else int(cut[0][0, 2]), "ms": round(ms, 3),
                              "state_rows_per_lane": os.environ.get("VPSA_SCAN_ROWS", "auto")}), flush=True)


if __name__ == "__main__":
    main()
