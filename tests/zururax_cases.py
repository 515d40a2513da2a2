"""Cases that run the engine on small random Zururax checkpoints against the float64 oracle; the CPU
and the GPU test files call them with their device, dtype and tolerance."""

from __future__ import annotations

import tempfile

import torch

import zururax_oracle as zo
from vllm_production_stack_amd.engine.config import EngineConfig
from vllm_production_stack_amd.engine.llm_engine import LLMEngine
from vllm_production_stack_amd.engine.request import SamplingParams

PAGE = 64


def make_engine(cfg, w, device, dtype, pages=12, slots=4, budget=None):
    folder = zo.save_checkpoint(cfg, w, tempfile.mkdtemp(prefix="zx-"))
    ec = EngineConfig(model=folder, dtype=dtype, device=device, max_model_len=pages * PAGE, max_num_seqs=slots,
                      max_num_batched_tokens=budget or pages * PAGE, num_gpu_blocks_override=pages,
                      enable_prefix_caching=False, enforce_eager=True, capture_graphs_at_start=False)
    return LLMEngine(ec)


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay(engine, rid, toks, cuts, end=True):
    """Feed ``toks`` as chunks of the sizes ``cuts`` (the rest one by one), all rows wanted -> logits [T, vocab]."""
    out, at = [], 0
    sizes = list(cuts)
    while at < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - at)
        last = at + n == len(toks)
        out.append(engine.forced_step([(rid, toks[at:at + n], list(range(n)))], [rid] if last and end else []))
        at += n
    return torch.cat(out).cpu()


def check_cuts(device, dtype, tol, cfg, w, n, cuts_list, seed=1, pages=12):
    toks = tokens(cfg, n, seed)
    want = zo.forward(cfg, w, toks)
    eng = make_engine(cfg, w, device, dtype, pages=pages)
    for k, cuts in enumerate(cuts_list):
        got = replay(eng, f"r{k}", toks, cuts)
        zo.check_rows(got, want, tol, f"cuts {cuts[:6]}")
    assert eng.bm.num_free() == pages  # every page came back
    eng.shutdown()


def check_layers(device, dtype, tol, cfg, w, n=37):
    """The residual stream after every layer."""
    toks = tokens(cfg, n, 5)
    want = []
    zo.forward(cfg, w, toks, layers_out=want)
    eng = make_engine(cfg, w, device, dtype)
    got = {}
    eng.runner.model.layer_probe = lambda i, x: got.__setitem__(i, x.detach().double().cpu())
    eng.forced_step([("a", toks, [n - 1])], ["a"])
    for i, ref in enumerate(want):
        err = ((got[i] - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()).item()
        assert err < tol, f"layer {i}: error {err:.3g}"
    eng.shutdown()


def check_batches(device, dtype, tol, cfg, w):
    """Unequal requests in the same steps (chunks beside single tokens), slots and pages used again."""
    lens = [150, 3, 70, 1, 129, 66, 40]
    reqs = {f"q{i}": tokens(cfg, n, 20 + i) for i, n in enumerate(lens)}
    want = {k: zo.forward(cfg, w, v) for k, v in reqs.items()}
    pages = 8  # 512 tokens: less than the sum of all requests, so finished requests' pages are used again
    eng = make_engine(cfg, w, device, dtype, pages=pages, slots=4)
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    chunk = {"q0": [31, 2, 64, 1, 1, 33], "q1": [2], "q2": [5, 59, 2], "q3": [1], "q4": [64, 2, 61], "q5": [66],
             "q6": [3, 30]}
    live, waiting = [], list(reqs)
    guard = 0
    while live or waiting:
        guard += 1
        assert guard < 400
        while waiting and len(live) < 4:
            need = (len(reqs[waiting[0]]) + PAGE - 1) // PAGE
            held = sum((len(reqs[k]) + PAGE - 1) // PAGE for k in live)
            if held + need > pages:
                break
            live.append(waiting.pop(0))
        entries, end = [], []
        for k in live:
            n = min(chunk[k].pop(0) if chunk[k] else 1, len(reqs[k]) - at[k])
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        logits = eng.forced_step(entries, end).cpu()
        row = 0
        for k, t, _ in entries:
            got[k].append(logits[row:row + len(t)])
            row += len(t)
        live = [k for k in live if k not in end]
    for k in reqs:
        if len(reqs[k]) >= 40 or tol < 1e-3:  # a bf16 close call in a handful of rows says nothing
            zo.check_rows(torch.cat(got[k]), want[k], tol, f"{k} ({len(reqs[k])} tokens)")
    assert eng.bm.num_free() == pages and not eng.scheduler.running
    eng.shutdown()


def check_generate(device, dtype, cfg, w, n_new=12):
    """Greedy generation through the engine's own entry point: scheduler, chunked prefill, sampler."""
    prompts = [tokens(cfg, n, 40 + n) for n in (90, 5, 1, 66)]
    eng = make_engine(cfg, w, device, dtype, pages=10, slots=3, budget=48)  # prompts are cut into chunks of <= 48
    outs = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == zo.greedy(cfg, w, p, n_new), f"prompt of {len(p)} tokens"
    eng.shutdown()
