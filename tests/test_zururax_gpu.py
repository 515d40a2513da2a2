"""Zururax on the GPU: the HIP kernels one by one against float64 definitions, then the engine in fp32
and in bf16 against the float64 oracle (same cases as on the CPU)."""

import pytest
import torch

import zururax_cases as zc
import zururax_oracle as zo
from test_zururax_cpu import attention_edges
from vllm_production_stack_amd import ops

pytestmark = pytest.mark.gpu

MODES = [("float32", 5e-5), ("bfloat16", 6e-2)]
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
KERNEL_TOL = {"float32": 1e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module")
def model_a():
    cfg = zo.config_a()
    return cfg, zo.make_weights(cfg, seed=3)


@pytest.fixture(scope="module")
def model_b():
    cfg = zo.config_b()
    return cfg, zo.make_weights(cfg, seed=4, sink_std=3.0)


def close(got, want, tol):
    return (got.double().cpu() - want).abs().max().item() <= tol * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_elementwise_kernels(dtype):
    dt, tol = DTYPES[dtype], KERNEL_TOL[dtype]
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(0)
    # embedding times a scale into the fp32 stream
    emb = torch.randn(50, 37, generator=g).to(dt)
    ids = torch.randint(0, 50, (11,), generator=g)
    assert close(ops.embed_scale(ids.to(dev), emb.to(dev), 2.5), emb[ids].double() * 2.5, 1e-6)
    # add + norm on the fp32 stream, norm over a column range, odd sizes
    for n in (37, 256, 1000):
        res, delta = torch.randn(6, n, generator=g), torch.randn(6, n, generator=g).to(dt)
        wgt = torch.rand(n, generator=g) + 0.5
        r = res.to(dev)
        y = ops.add_rms_norm(r, delta.to(dev), wgt.to(dev), 1e-3, dt)
        s = res.double() + delta.double()
        assert close(r, s, 1e-6) and close(y, zo.rms(s, 1e-3, wgt.double()), tol)
        wide = torch.randn(6, n + 9, generator=g).to(dt)
        y = ops.rms_norm_rows(wide.to(dev)[:, 4:4 + n], wgt.to(dev), 1e-3)
        assert close(y, zo.rms(wide[:, 4:4 + n].double(), 1e-3, wgt.double()), tol)
    # rotation of a column range of every head
    q = torch.randn(9, 3, 20, generator=g).to(dt)
    pos = torch.tensor([0, 1, 2, 63, 64, 65, 500, 1023, 7], dtype=torch.int32)
    table = ops.build_cos_sin(10, 1024, 333.0)
    got = q.clone().to(dev)
    ops.rope_pairs(got, pos.to(dev), table.to(dev), 6, 10)
    for h in range(3):
        assert close(got[:, h, 6:], zo.rotate_pairs(q[:, h, 6:].double(), pos, 333.0, 10), tol)
        assert torch.equal(got[:, h, :6].cpu(), q[:, h, :6])
    # activations, output gate
    x = (torch.randn(7, 2 * 11, generator=g) * 3).to(dt)
    gate, up = x[:, :11].double().clamp(max=0.7), x[:, 11:].double().clamp(-0.7, 0.7)
    assert close(ops.glu_clamp(x.to(dev), 0.7), gate * torch.sigmoid(1.702 * gate) * (up + 1), tol)
    assert close(ops.relu_sq(x.to(dev)), torch.relu(x.double()) ** 2, tol)
    y, gl = torch.randn(5, 3, 7, generator=g).to(dt), torch.randn(5, 9, generator=g).to(dt)
    got = ops.sigmoid_gate(y.clone().to(dev), gl.to(dev)[:, 2:5])
    assert close(got, y.double() * torch.sigmoid(gl[:, 2:5].double())[..., None], tol)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cache_entries(dtype):
    """Entries land at their slots (pages out of order, a layer's offset inside the page), normed and rotated."""
    dt, tol = DTYPES[dtype], KERNEL_TOL[dtype]
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(1)
    rank, rot, dims = 24, 12, 8
    x = torch.randn(6, 5 + rank + rot, generator=g).to(dt)
    wgt = torch.rand(rank, generator=g) + 0.5
    pos = torch.tensor([0, 63, 64, 100, 5, 6], dtype=torch.int32)
    slots = torch.tensor([3 * 64 + 0, 3 * 64 + 63, 1 * 64 + 0, 1 * 64 + 36, -1, 2 * 64 + 6])
    pool = torch.zeros(5, 64 * (rank + rot) + 64 * 10 + 3, dtype=dt, device=dev)
    off = 64 * 10 + 3
    table = ops.build_cos_sin(dims, 128, 50.0)
    ops.latent_kv_write(x.to(dev)[:, 5:], wgt.to(dev), pos.to(dev), slots.to(dev), table.to(dev), pool, off, rank, rot,
                        dims, 1e-4)
    view = pool[:, off:].view(5, 64, rank + rot)
    c = zo.rms(x[:, 5:5 + rank].double(), 1e-4, wgt.double())
    r = zo.rotate_pairs(x[:, 5 + rank:].double(), pos, 50.0, dims)
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        assert close(view[s // 64, s % 64], torch.cat([c[i], r[i]]), tol)
    assert float(pool.float().abs().sum()) == pytest.approx(float(view.float().abs().sum()))  # nothing else written
    assert float(view[2, 5].float().abs().sum()) == 0.0  # the skipped row


@pytest.mark.parametrize("experts,groups,keep,top", [(12, 4, 2, 3), (6, 6, 2, 1), (8, 1, 1, 4), (64, 8, 3, 6)])
def test_group_routing(experts, groups, keep, top):
    g = torch.Generator().manual_seed(experts)
    h = torch.randn(70, 16, generator=g).double()
    w = {"x.mlp.router": torch.randn(experts, 16, generator=g).double()}
    want = zo.route(h, w, "x", {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}, "scale": 1.3})
    logits = torch.cat([(h @ w["x.mlp.router"].T).float(), torch.randn(70, 1, generator=g)], 1).contiguous()
    wt, ids, ex = ops.group_topk(logits.cuda(), experts, groups, keep, top, 1.3, extra=True)
    for t in range(70):
        assert [e for e, _ in want[t]] == ids[t].tolist()
        assert torch.allclose(wt[t].double().cpu(), torch.tensor([x for _, x in want[t]], dtype=torch.float64), atol=1e-6)
    assert torch.allclose(ex.cpu(), torch.sigmoid(logits[:, experts]), atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_edges(dtype):
    attention_edges(torch.device("cuda"), DTYPES[dtype], 2e-4 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("rank,rot,heads", [(64, 32, 3), (128, 64, 5), (256, 32, 70), (512, 64, 2),
                                            (32, 64, 3), (64, 96, 2), (64, 128, 4), (128, 128, 2), (128, 192, 3)])
@pytest.mark.parametrize("mode,splits", [("tiles", 1), ("decode", 1), ("decode", 3), ("decode", 7)])
def test_attention_edges_matrix_cores(rank, rot, heads, mode, splits):
    """The tile kernel: one-token tiles and decode rows, whole key range and key-range splits (more splits
    than some rows have pages), more heads than a tile holds."""
    assert ops.latent_mfma_supported(rank, rot)
    attention_edges(torch.device("cuda"), torch.bfloat16, 3e-2, rank=rank, rot=rot, heads=heads, mode=mode, splits=splits)


def test_gemm_epilogues():
    """The grouped / dense prefill GEMM with the clamped gated unit and the squared ReLU in its epilogue."""
    g = torch.Generator().manual_seed(7)
    rows, k, inter, groups = 300, 128, 96, 3
    x = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(groups, 2 * inter, k, generator=g) * k ** -0.5).to(torch.bfloat16)
    offsets = torch.tensor([0, 170, 170, 290], dtype=torch.int32)  # an empty group, rows past the last group
    idx = torch.randperm(rows, generator=g).int()
    got = ops.tile_gemm(x.cuda(), w.cuda(), offsets.cuda(), rows=rows, arow_idx=idx.cuda(), glu_clamp=(0.9, 1.702, 1.0))
    for gi in range(groups):
        lo, hi = int(offsets[gi]), int(offsets[gi + 1])
        if hi == lo:
            continue
        y = x[idx[lo:hi].long()].double() @ w[gi].double().T
        gate, up = y[:, :inter].clamp(max=0.9), y[:, inter:].clamp(-0.9, 0.9)
        assert close(got[lo:hi], gate * torch.sigmoid(1.702 * gate) * (up + 1), 2e-2)
    got = ops.tile_gemm(x.cuda(), w[0].cuda(), relu_sq=True)
    assert close(got, torch.relu(x.double() @ w[0].double().T) ** 2, 2e-2)
    assert close(ops.up_relu_sq(x.cuda(), w[0].cuda()), torch.relu(x.double() @ w[0].double().T) ** 2, 2e-2)


@pytest.mark.parametrize("tokens", [1, 5, 40, 100])
def test_mixture_units_small_and_large_batches(tokens):
    """The routed units over sorted pairs: the weight-streaming kernels of decode-sized batches and the
    grouped prefill GEMM give what the float64 definition gives."""
    g = torch.Generator().manual_seed(tokens)
    e, hidden, inter, top = 6, 128, 512, 2
    x = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    w13 = (torch.randn(e, 2 * inter, hidden, generator=g) * hidden ** -0.5).to(torch.bfloat16)
    w2 = (torch.randn(e, hidden, inter, generator=g) * inter ** -0.5).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(e, generator=g)[:top] for _ in range(tokens)]).int()
    assert ops.moe_glu_grouped_supported(x.cuda(), w13.cuda(), w2.cuda())
    y, pos = ops.moe_glu_grouped(x.cuda(), w13.cuda(), w2.cuda(), ids.cuda(), 1.1, 1.702, 1.0)
    for t in range(tokens):
        for k in range(top):
            ex = int(ids[t, k])
            gu = x[t].double() @ w13[ex].double().T
            gate, up = gu[:inter].clamp(max=1.1), gu[inter:].clamp(-1.1, 1.1)
            want = (gate * torch.sigmoid(1.702 * gate) * (up + 1)) @ w2[ex].double().T
            assert close(y[int(pos[t * top + k])], want, 3e-2), (t, k)


def test_decode_graphs_match_eager(model_c):
    """Decode steps replayed from captured HIP graphs (several replays per bucket, prefill steps and host
    work between them) generate what eager steps generate."""
    import tempfile

    from vllm_production_stack_amd.engine.config import EngineConfig
    from vllm_production_stack_amd.engine.llm_engine import LLMEngine
    from vllm_production_stack_amd.engine.request import SamplingParams

    cfg, w = model_c
    folder = zo.save_checkpoint(cfg, w, tempfile.mkdtemp(prefix="zx-"))
    prompts = [zc.tokens(cfg, n, 60 + n) for n in (70, 5, 130, 9, 33)]
    outs = {}
    for eager in (True, False):
        ec = EngineConfig(model=folder, dtype="bfloat16", device="cuda", max_model_len=1024, max_num_seqs=8,
                          max_num_batched_tokens=64, num_gpu_blocks_override=32, enable_prefix_caching=False,
                          enforce_eager=eager, capture_graphs_at_start=not eager)
        eng = LLMEngine(ec)
        assert eng.runner.use_graphs == (not eager)
        outs[eager] = eng.generate(prompts, SamplingParams(max_tokens=40, temperature=0.0, ignore_eos=True))
        if not eager:
            assert eng.runner.step_kinds["decode_graph"] > 20
        eng.shutdown()
    assert outs[True] == outs[False]


@pytest.fixture(scope="module")
def model_c():
    cfg = zo.config_c()
    return cfg, zo.make_weights(cfg, seed=5)


def test_tile_kernel_in_the_engine(model_c):
    """Entries of shapes the tile kernel takes (bf16): tiles of several tokens, a head count that does not
    divide a tile, layers of different head counts, a layer reading another layer's entries."""
    tol = 6e-2
    zc.check_layers("cuda", "bfloat16", tol, *model_c)
    zc.check_cuts("cuda", "bfloat16", tol, *model_c, 200, [[200], [], [130], [2, 2, 60, 1, 2, 61, 3, 64, 2], [63, 2, 63, 2]])
    zc.check_batches("cuda", "bfloat16", tol, *model_c)
    zc.check_cuts("cuda", "float32", 5e-5, *model_c, 150, [[150], [70, 3, 64]])


def test_expanded_prefill_in_the_engine():
    """Prefill parts large enough to expand keys and values per head for the step (bf16): whole prompts, a
    second large portion over a cached first one, large portions beside decoding requests; the small portions
    and the decoded tokens of the same requests stay in latent space and must agree with them."""
    from vllm_production_stack_amd.models import zururax

    cfg = zo.config_d()
    w = zo.make_weights(cfg, seed=6)
    n = 700
    toks = zc.tokens(cfg, n, 8)
    want = zo.forward(cfg, w, toks)
    eng = zc.make_engine(cfg, w, "cuda", "bfloat16", pages=24)
    assert all(eng.runner.model._expands(s.mixer) for s in eng.runner.model.specs)
    seen = []
    real = eng.runner.model._expanded_prefill
    eng.runner.model._expanded_prefill = lambda *a, **k: (seen.append(a[1].shape[0]), real(*a, **k))[1]
    for k, cuts in enumerate([[n], [300, 400], [256, 100, 300, 2, 42], [n - 40]]):
        zo.check_rows(zc.replay(eng, f"r{k}", toks, cuts), want, 6e-2, f"cuts {cuts}")
    assert sorted(set(seen)) == [256, 300, 400, 660, 700]  # 100, 2, 42 and single tokens stayed in latent space
    # a large portion beside two decoding requests and a small portion
    a, b = zc.tokens(cfg, 90, 1), zc.tokens(cfg, 40, 2)
    la, lb = zo.forward(cfg, w, a), zo.forward(cfg, w, b)
    eng.forced_step([("a", a[:89], []), ("b", b[:39], [])])
    out = eng.forced_step([("a", a[89:], [0]), ("b", b[39:], [0]), ("c", toks[:500], list(range(500))), ("d", b[:7], [6])],
                          ["a", "b", "c", "d"]).cpu()
    zo.check_rows(out[2:502], want[:500], 6e-2, "large portion in a mixed batch")
    zo.check_rows(torch.stack([out[0], out[1], out[502]]), torch.stack([la[89], lb[39], lb[6]]), 1e-1, "its neighbours")
    assert zururax.EXPAND_MIN_ROWS == 256
    eng.shutdown()


@pytest.mark.parametrize("dtype,tol", MODES)
def test_layers(dtype, tol, model_a, model_b):
    zc.check_layers("cuda", dtype, tol, *model_a)
    zc.check_layers("cuda", dtype, tol, *model_b)


@pytest.mark.parametrize("dtype,tol", MODES)
def test_whole_decode_and_portions(dtype, tol, model_a):
    n = 200
    zc.check_cuts("cuda", dtype, tol, *model_a, n, [
        [n], [], [n - 70], [2, 2, 60, 1, 2, 61, 3, 64, 2], [63, 2, 63, 2], [64, 64, 64], [1, 127, 1, 1, 2]])


@pytest.mark.parametrize("dtype,tol", MODES)
def test_other_sizes_and_first_tokens(dtype, tol, model_a, model_b):
    zc.check_cuts("cuda", dtype, tol, *model_b, 131, [[131], [], [2, 62, 2, 63, 2], [65, 1, 1, 64]])
    if dtype == "float32":  # (a handful of rows: one close call of a router in bf16 would be all of them)
        for n in (1, 2, 3):
            zc.check_cuts("cuda", dtype, tol, *model_a, n, [[n], [], [1, n]], seed=n)


@pytest.mark.parametrize("dtype,tol", MODES)
def test_long_decode(dtype, tol, model_b):
    zc.check_cuts("cuda", dtype, tol, *model_b, 330, [[5]], pages=6)


@pytest.mark.parametrize("dtype,tol", MODES)
def test_batches_and_reuse(dtype, tol, model_a):
    zc.check_batches("cuda", dtype, tol, *model_a)


def test_greedy_generation(model_a, model_b):
    zc.check_generate("cuda", "float32", *model_a)
    zc.check_generate("cuda", "float32", *model_b, n_new=30)
    assert ops.native_loaded()
