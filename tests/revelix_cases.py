"""Cases for Revelix: every op against its float64 definition, and the engine on small random
checkpoints against the float64 oracle.  The CPU and the GPU test files call them with their device,
dtype and tolerance."""

from __future__ import annotations

import math
import tempfile

import torch

import revelix_oracle as ro
from vllm_production_stack_amd import ops
from vllm_production_stack_amd.engine.config import EngineConfig
from vllm_production_stack_amd.engine.llm_engine import LLMEngine
from vllm_production_stack_amd.engine.request import SamplingParams

PAGE = 64
F64 = torch.float64
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def close(got, want, tol, what=""):
    err = (got.double().cpu() - want).abs().max().item()
    lim = tol * max(1.0, want.abs().max().item())
    assert err <= lim, f"{what}: off by {err:.3g} (allowed {lim:.3g})"


def i32(x, dev):
    return torch.tensor(x, dtype=torch.int32, device=dev)


# ----------------------------------------------------------------------------- configurations
def config_a():
    """Sizes that differ from one another wherever they can: rotary dims below the head, odd value
    sizes, three taps, mixed layer order, feed-forward on some layers only."""
    return ro.make_config([
        ro.retention_layer(heads=2, dim=16, vdim=24, rot_dims=12, base=5000.0),
        ro.parallel_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, size=24, keep=3, rot_dims=12,
                          scaling={"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}, softcap=20.0,
                          r_heads=2, r_dim=8, r_vdim=16, mlp={"kind": "dense", "ff": 72}),
        ro.retention_layer(heads=3, dim=8, vdim=40, mlp={"kind": "dense", "ff": 40}),
    ], vocab=96, width=48)


def config_b():
    """Other corners: one KV head per query head, a single retention head, four taps, no kept tokens in
    one layer and a window of one page in the other, the parallel layer first, no feed-forward at all in
    two layers, head sizes that need padding inside the kernels."""
    return ro.make_config([
        ro.parallel_layer(heads=3, kv_heads=3, dim=24, vdim=8, conv=4, size=64, keep=0, base=300.0, softcap=8.0,
                          scale=0.3, r_heads=1, r_dim=40, r_vdim=72, left_scale=1.0, right_scale=0.4),
        ro.retention_layer(heads=1, dim=40, vdim=72, decay=[0.98], rot_dims=40),
        ro.parallel_layer(heads=2, kv_heads=1, dim=8, vdim=80, conv=1, size=5, keep=7, r_heads=3, r_dim=16, r_vdim=8,
                          mlp={"kind": "dense", "ff": 24}),
    ], vocab=70, width=40, logit_scale=1.0, eps=1e-3)


def config_c():
    """Head sizes the matrix-core attention kernel tiles, and chunks long enough to be cut into pieces."""
    return ro.make_config([
        ro.retention_layer(heads=2, dim=64, vdim=64, rot_dims=32, mlp={"kind": "dense", "ff": 256}),
        ro.parallel_layer(heads=4, kv_heads=2, dim=64, vdim=64, conv=4, size=100, keep=2, softcap=25.0, r_heads=2,
                          r_dim=32, r_vdim=64, mlp={"kind": "dense", "ff": 256}),
    ], vocab=200, width=128)


def config_d():
    """Recurrences only (the pool's pages stay empty), no feed-forward anywhere, a value size that is no multiple of 4."""
    return ro.make_config([ro.retention_layer(heads=2, dim=8, vdim=10), ro.retention_layer(heads=1, dim=24, vdim=6, rot_dims=2)],
                          vocab=50, width=24, logit_scale=1.5)


def config_e():
    """Parallel layers only; a window of one position; two and five taps; a value size that is no multiple of 4."""
    return ro.make_config([ro.parallel_layer(heads=2, kv_heads=2, dim=8, vdim=12, conv=2, size=1, keep=2, r_heads=1, r_dim=4,
                                             r_vdim=6),
                           ro.parallel_layer(heads=2, kv_heads=1, dim=16, vdim=6, conv=5, size=200, keep=0, rot_dims=4,
                                             r_heads=2, r_dim=8, r_vdim=4, mlp={"kind": "dense", "ff": 16})],
                          vocab=40, width=16, logit_scale=0.25)


# ----------------------------------------------------------------------------- mechanisms
def case_dyt_and_xielu(dev, dtype, tol):
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(0)
    for n in (5, 48, 300):
        res = torch.randn(7, n, generator=g) * 2
        d1, d2 = torch.randn(7, n, generator=g).to(dt), torch.randn(7, n, generator=g).to(dt)
        w, b = torch.rand(n, generator=g) + 0.5, torch.randn(n, generator=g) * 0.1
        alpha = torch.tensor([0.37])
        for deltas in ([], [(d1, 1.0)], [(d1, 0.6), (d2, -1.3)]):
            r = res.clone().to(dev)
            y = ops.add_dyt_norm(r, [(d.to(dev), c) for d, c in deltas], w.to(dev), b.to(dev), alpha.to(dev), dt)
            s = res.double() + sum(d.double() * c for d, c in deltas)
            close(r, s, 1e-6, "stream")
            close(y, ro.dyt(s, w.double(), b.double(), 0.37), tol, "dyt")
    z = (torch.randn(9, 33, generator=g) * 3).to(dt)
    p, q = torch.tensor(0.3, dtype=F64), torch.tensor(-0.8, dtype=F64)
    sp = torch.nn.functional.softplus
    act = torch.stack([sp(p), 0.5 + sp(q)]).float()
    close(ops.xielu(z.to(dev), act.to(dev)), ro.xielu(z.double(), p, q), tol, "xielu")


def case_rotary_tables():
    for dims, base, scaling in ((12, 5000.0, None), (32, 1e6, {"factor": 8.0, "original": 1024, "fast": 32.0, "slow": 1.0}),
                                (8, 300.0, {"factor": 2.5, "original": 16, "fast": 4.0, "slow": 0.5})):
        sc = None if scaling is None else dict(scaling, rope_type="ramp")
        table = ops.build_cos_sin(dims, 2000, base, sc).double()
        f, m = ro.frequencies(base, dims, scaling)
        ang = torch.arange(2000, dtype=F64)[:, None] * f[None, :]
        close(table, torch.cat([ang.cos() * m, ang.sin() * m], -1), 1e-6, "table")
    f, m = ro.frequencies(1e6, 32, {"factor": 8.0, "original": 1024, "fast": 32.0, "slow": 1.0})
    plain, _ = ro.frequencies(1e6, 32)
    assert m > 1 and torch.allclose(f[:2], plain[:2]) and torch.allclose(f[6:], plain[6:] / 8)  # the two ends of the ramp


def _run_scan(dev, dt, proj, cols, heads, dim, vdim, state, off, chunks, slot, pos0, **kw):
    """Feed rows of ``proj`` to ops.recurrent_scan as consecutive chunks of one sequence."""
    outs, at = [], 0
    for n in chunks:
        pos = i32(list(range(pos0 + at, pos0 + at + n)), dev)
        outs.append(ops.recurrent_scan(proj[at:at + n].contiguous(), *cols, heads, dim, vdim, state, off, i32([0, n], dev),
                                       i32([slot], dev), pos, **kw))
        at += n
    return torch.cat(outs)


def case_recurrences(dev, dtype, tol):
    """Both recurrences: whole against portions (down to one row), two sequences of one launch, a slot
    that held something else, the state left behind."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(1)
    for heads, dim, vdim, rot_dims, layout in ((2, 16, 24, 12, 0), (1, 40, 72, 40, 0), (3, 8, 70, 8, 1), (2, 64, 130, 32, 0)):
        t = 45
        width = heads * (2 * dim + vdim) + 5
        cols = (3, 3 + heads * dim, 5 + 2 * heads * dim)
        proj = torch.randn(t, width, generator=g).to(dt)
        decay = torch.tensor([1 - 2.0 ** -(2 + h) for h in range(heads)])
        table = ops.build_cos_sin(rot_dims, 512, 777.0)
        bias, lower = torch.randn(heads * dim, generator=g), torch.rand(heads * dim, generator=g) * 0.9
        pj = proj.double()
        q = pj[:, cols[0]:cols[0] + heads * dim].view(t, heads, dim)
        k = pj[:, cols[1]:cols[1] + heads * dim].view(t, heads, dim)
        v = pj[:, cols[2]:cols[2] + heads * vdim].view(t, heads, vdim)
        rot = {"base": 777.0, "dims": rot_dims}
        pos = torch.arange(t)
        lay = "half" if layout == 0 else "pairs"
        want_decay = ro.linear_recurrence(ro.rotate(q, pos, rot, lay), ro.rotate(k, pos, rot, lay) * 0.25, v,
                                          decay.double().view(1, heads, 1).expand(t, heads, dim))
        f = (lower.double() + (1 - lower.double()) * torch.sigmoid(k.reshape(t, -1) + bias.double())).view(t, heads, dim)
        want_gate = ro.linear_recurrence(torch.nn.functional.silu(q), 1 - f, v, f)
        n_state = heads * dim * vdim
        for want, kw in ((want_decay, dict(decay=decay.to(dev), cos_sin=table.to(dev), rot_dims=rot_dims, layout=layout,
                                           k_scale=0.25)),
                         (want_decay, dict(decay=decay.to(dev), cos_sin=table.to(dev), rot_dims=rot_dims, layout=layout,
                                           k_scale=0.25, min_decay=float(decay.min()))),  # decay folded into the block
                         (want_gate, dict(gate_bias=bias.to(dev), gate_lower=lower.to(dev)))):
            state = torch.full((3, n_state + 7), float("nan"), device=dev)  # a chunk at position 0 must not read it
            pd = proj.to(dev)
            whole = _run_scan(dev, dt, pd, cols, heads, dim, vdim, state, 4, [t], 1, 0, **kw)
            close(whole, want, tol, "whole")
            left = state[1, 4:4 + n_state].clone()
            parts = _run_scan(dev, dt, pd, cols, heads, dim, vdim, state, 4, [1, 2, 17, 1, 1, 20, 3], 2, 0, **kw)
            close(parts, want, tol, "portions")
            close(state[2, 4:4 + n_state], left.double().cpu(), 1e-5, "state after portions")
            assert torch.isnan(state[0]).all() and torch.isnan(state[1, :4]).all()  # nothing else was touched
            # two sequences in one launch: the tail of the first (from its state) and a new one in slot 0
            state[1, 4:4 + n_state] = float("nan")
            _run_scan(dev, dt, pd, cols, heads, dim, vdim, state, 4, [30], 1, 0, **kw)
            both = torch.cat([pd[30:], pd[:11]]).contiguous()
            posb = i32(list(range(30, t)) + list(range(11)), dev)
            out = ops.recurrent_scan(both, *cols, heads, dim, vdim, state, 4, i32([0, t - 30, t - 30 + 11], dev),
                                     i32([1, 0], dev), posb, **kw)
            close(out[:t - 30], want[30:], tol, "continued beside another")
            close(out[t - 30:], want[:11], tol, "started beside another")
            # rows of no sequence come back as zeros and touch nothing
            before = state.clone()
            out = ops.recurrent_scan(both, *cols, heads, dim, vdim, state, 4, i32([0, 4, 6], dev), i32([-1, -1], dev),
                                     posb, **kw)
            assert (out[:6] == 0).all() and torch.equal(torch.nan_to_num(state), torch.nan_to_num(before))


def case_recurrence_pieces(dev, dtype, tol):
    """Long chunks cut into pieces that run side by side: same outputs and same state as walking them in
    one go, with a continued sequence, a new one and a one-row sequence in the same launch."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(7)
    for heads, dim, vdim in ((2, 16, 24), (2, 128, 64), (1, 40, 70)):
        lens, starts, slots = [300, 1, 140], [77, 500, 0], [2, 0, 1]
        t = sum(lens)
        cols = (0, heads * dim, 2 * heads * dim)
        proj = (torch.randn(t, heads * (2 * dim + vdim), generator=g) * 0.5).to(dt).to(dev)
        decay = torch.tensor([1 - 2.0 ** -(3 + h) for h in range(heads)]).to(dev)
        table = ops.build_cos_sin(dim, 1024, 500.0).to(dev)
        bias, lower = torch.randn(heads * dim, generator=g).to(dev), (torch.rand(heads * dim, generator=g) * 0.9).to(dev)
        pos, cu = [], [0]
        for n, p0 in zip(lens, starts):
            pos += list(range(p0, p0 + n))
            cu.append(cu[-1] + n)
        cut = ops.build_scan_pieces(lens, target=12)
        assert cut is not None and cut[0].shape[0] > 5
        pieces = tuple(torch.from_numpy(a).to(dev) for a in cut)
        for kw in (dict(decay=decay, cos_sin=table, rot_dims=dim, layout=0, k_scale=dim ** -0.5),
                   dict(decay=decay, cos_sin=table, rot_dims=dim, layout=0, k_scale=dim ** -0.5, min_decay=float(decay.min())),
                   dict(gate_bias=bias, gate_lower=lower)):
            s0 = torch.randn(3, heads * dim * vdim + 4, generator=g).to(dev)
            res = []
            for pc in (None, pieces):
                state = s0.clone()
                out = ops.recurrent_scan(proj, *cols, heads, dim, vdim, state, 4, i32(cu, dev), i32(slots, dev), i32(pos, dev),
                                         pieces=pc, **kw)
                res.append((out, state))
            close(res[1][0], res[0][0].double().cpu(), tol, "outputs of the pieces")
            close(res[1][1], res[0][1].double().cpu(), tol, "state after the pieces")


def case_head_norm(dev, dtype, tol):
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(2)
    for heads, vdim in ((2, 24), (1, 72), (3, 130)):
        o = torch.randn(6, heads, vdim, generator=g) * 3
        w = torch.rand(vdim, generator=g) + 0.5
        wide = torch.randn(6, heads * vdim + 9, generator=g).to(dt)
        gate = wide[:, 4:4 + heads * vdim]
        unit = ro.rms_unit(o.double(), 1e-3)
        close(ops.head_rms_norm(o.to(dev), 1e-3, dt, weight=w.to(dev)), (unit * w.double()).reshape(6, -1), tol, "weight")
        close(ops.head_rms_norm(o.to(dev), 1e-3, dt, gate=wide.to(dev)[:, 4:4 + heads * vdim]),
              unit.reshape(6, -1) * torch.nn.functional.silu(gate.double()), tol, "gate")


def _window_setup(dev, dt, heads, kv_heads, dim, vdim, n_keys, g, pages_order):
    """Keys and values of one sequence in a pool whose pages are used out of order."""
    k = torch.randn(n_keys, kv_heads, dim, generator=g).to(dt)
    v = torch.randn(n_keys, kv_heads, vdim, generator=g).to(dt)
    off = 16
    n_pages = (n_keys + PAGE - 1) // PAGE
    pool = torch.zeros(max(pages_order) + 1, off + ops.window_cache_elems(kv_heads, dim, vdim) + 8, dtype=dt)
    from vllm_production_stack_amd.ops import reference

    kc, vc = reference.window_cache_views(pool, off, kv_heads, dim, vdim)
    for j in range(n_keys):
        kc[pages_order[j // PAGE], j % PAGE] = k[j]
        vc[pages_order[j // PAGE], j % PAGE] = v[j]
    assert n_pages <= len(pages_order)
    return k, v, pool.to(dev), off


def case_window_edges(dev, dtype, tol):
    """One key made to stand out (its score hits the cap while the others stay near zero) just inside and
    just outside the window and the kept first tokens, at page borders and far back; prompt rows and
    decode rows; sinks that do nothing, something, everything."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(3)
    heads, kv_heads, dim, vdim = 4, 2, 64, 24
    size, keep, cap, scale = 70, 3, 12.0, 1.0
    n_keys = 200
    order = [5, 2, 7, 0]
    k, v, pool, off = _window_setup(dev, dt, heads, kv_heads, dim, vdim, n_keys, g, order)
    bt = i32([[9, 9, 9, 9], order], dev)  # the sequence is row 1 of the block table
    talk = (torch.eye(heads) * 0.8 + 0.2 * torch.randn(heads, heads, generator=g))
    for sink_level in (-30.0, 0.5, 25.0):
        sink = torch.full((heads,), sink_level) + torch.randn(heads, generator=g) * 0.1
        rows = []   # (position of the query, key it looks for)
        for p in (199, 150, 71, 69, 64, 63, 5, 2, 0):
            for j in {p, p - 1, p - size + 1, p - size, p - size - 1, keep - 1, keep, 0, 63, 64, 127, 128}:
                if 0 <= j <= p:
                    rows.append((p, j))
        q = torch.randn(len(rows), heads, dim, generator=g) * 0.05
        for r, (p, j) in enumerate(rows):
            q[r] += 30.0 * k[j, torch.arange(heads) // (heads // kv_heads)].float() / dim  # score far above the cap
        q = q.to(dt)
        pos_q = torch.tensor([p for p, _ in rows])
        w = ro.window_weights(q.double(), k.double(), pos_q, torch.arange(n_keys), heads // kv_heads, scale, cap, size, keep,
                              sink.double())
        want = ro.mixed_values(w, talk.double(), v.double(), heads // kv_heads)          # [rows, heads, vdim]
        seen = torch.tensor([(p - j < size) or (j < keep) for p, j in rows])
        share = torch.stack([w[0, r, j] for r, (p, j) in enumerate(rows)])
        assert (share[~seen] == 0).all() and (sink_level > 0 or (share[seen] > 0.3).all())  # the cases show what they claim
        # prompt rows: every row names its sequence; decode rows: row r is sequence r
        u = ops.window_attention(q.to(dev), pool, off, kv_heads, vdim, bt, i32([1] * len(rows), dev), i32(pos_q.tolist(), dev),
                                 size, keep, scale, cap, sink.to(dev))
        close(ops.mix_heads(u, talk.to(dev), torch.float32).view(len(rows), heads, vdim), want, tol, f"prompt rows, sink {sink_level}")
        btd = i32([order] * len(rows), dev)
        u = ops.window_attention(q.to(dev), pool, off, kv_heads, vdim, btd, None, i32(pos_q.tolist(), dev), size, keep,
                                 scale, cap, sink.to(dev))
        close(ops.mix_heads(u, talk.to(dev), torch.float32).view(len(rows), heads, vdim), want, tol, f"decode rows, sink {sink_level}")


def case_far_keys(dev, dtype, tol):
    """A window of many pages: one key among hundreds, far back."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(4)
    heads, kv_heads, dim, vdim = 2, 2, 8, 8
    n_keys = 700
    order = list(range(10, -1, -1))
    k, v, pool, off = _window_setup(dev, dt, heads, kv_heads, dim, vdim, n_keys, g, order)
    rows = [(699, 0), (699, 100), (699, 257), (600, 256), (699, 699 - 649), (699, 699 - 650), (300, 7), (300, 8)]
    q = torch.randn(len(rows), heads, dim, generator=g) * 0.02
    for r, (p, j) in enumerate(rows):
        q[r] += 30.0 * k[j].float() / dim
    q = q.to(dt)
    pos_q = torch.tensor([p for p, _ in rows])
    sink = torch.zeros(heads)
    for size, keep in ((650, 8), (1000, 0)):
        w = ro.window_weights(q.double(), k.double(), pos_q, torch.arange(n_keys), 1, 1.0, 0.0, size, keep, sink.double())
        want = ro.mixed_values(w, torch.eye(heads, dtype=F64), v.double(), 1)
        u = ops.window_attention(q.to(dev), pool, off, kv_heads, vdim, i32([order], dev), i32([0] * len(rows), dev),
                                 i32(pos_q.tolist(), dev), size, keep, 1.0, 0.0, sink.to(dev))
        close(ops.mix_heads(u, torch.eye(heads).to(dev), torch.float32).view(len(rows), heads, vdim), want, tol, "far keys")


def case_window_tiles(dev, heads, kv_heads, dim, vdim, size, keep, tol=2e-2):
    """The matrix-core kernel (bf16): chunks of consecutive rows of two sequences as tiles, and single
    rows as a decode batch; every row looks for one key at an edge of what it may see."""
    dt = torch.bfloat16
    g = torch.Generator().manual_seed(6)
    rep = heads // kv_heads
    assert ops.window_mfma_supported(heads, kv_heads, dim, vdim)
    cap, scale = 15.0, 1.0
    n_keys = 330
    order = [4, 1, 6, 0, 3, 7]
    k, v, pool, off = _window_setup(dev, dt, heads, kv_heads, dim, vdim, n_keys, g, order)
    talk = (torch.eye(heads) * 0.8 + 0.2 * torch.randn(heads, heads, generator=g))
    sink = torch.randn(heads, generator=g)
    chunks = [(0, 150, 180), (1, 0, 70), (2, 325, 5)]       # (block-table row = sequence of the batch, first position, rows)
    bt = i32([order, order, order], dev)
    pos_q, seqs = [], []
    for sq, p0, n in chunks:
        pos_q += list(range(p0, p0 + n))
        seqs += [sq] * n
    t = len(pos_q)
    q = torch.randn(t, heads, dim, generator=g) * 0.05
    targets = []
    for r, p in enumerate(pos_q):
        cand = [j for j in (p, p - 1, p - size + 1, p - size, keep - 1, keep, 0, 63, 64, 127, 128, p - size // 2) if 0 <= j <= p]
        j = cand[r % len(cand)]
        targets.append(j)
        q[r] += 30.0 * k[j, torch.arange(heads) // rep].float() / dim
    q = q.to(dt)
    pq = torch.tensor(pos_q)
    w = ro.window_weights(q.double(), k.double(), pq, torch.arange(n_keys), rep, scale, cap, size, keep, sink.double())
    want = ro.mixed_values(w, talk.double(), v.double(), rep)
    tiles = torch.from_numpy(ops.build_window_tiles([n for _, _, n in chunks], [p0 + n for _, p0, n in chunks], heads,
                                                    kv_heads)).to(dev)
    u = ops.window_attention(q.to(dev), pool, off, kv_heads, vdim, bt, i32(seqs, dev), i32(pos_q, dev), size, keep, scale,
                             cap, sink.to(dev), tiles=tiles)
    plain = ops.window_attention(q.to(dev), pool, off, kv_heads, vdim, bt, i32(seqs, dev), i32(pos_q, dev), size, keep,
                                 scale, cap, sink.to(dev))
    close(ops.mix_heads(plain, talk.to(dev), torch.float32).view(t, heads, vdim), want, 2e-5, "plain kernel")
    close(ops.mix_heads(u, talk.to(dev), torch.float32).view(t, heads, vdim), want, tol, "tiles")
    rows = list(range(0, t, 7))
    u = ops.window_attention(q[rows].to(dev), pool, off, kv_heads, vdim, i32([order] * len(rows), dev), None,
                             i32([pos_q[r] for r in rows], dev), size, keep, scale, cap, sink.to(dev))
    close(ops.mix_heads(u, talk.to(dev), torch.float32).view(len(rows), heads, vdim), want[rows], tol, "decode rows")
    for splits in (2, 3, 8):
        u = ops.window_attention(q[rows].to(dev), pool, off, kv_heads, vdim, i32([order] * len(rows), dev), None,
                                 i32([pos_q[r] for r in rows], dev), size, keep, scale, cap, sink.to(dev), splits=splits)
        close(ops.mix_heads(u, talk.to(dev), torch.float32).view(len(rows), heads, vdim), want[rows], tol,
              f"decode rows in {splits} key ranges")


def case_short_conv(dev, dtype, tol):
    """Convolution + rotation + cache write: whole against portions shorter than the taps, a restart in
    a slot that held something else, two sequences in one launch."""
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(5)
    from vllm_production_stack_amd.ops import reference

    for taps, heads, kv_heads, dim, vdim, rot_dims in ((3, 4, 2, 16, 24, 12), (4, 3, 3, 8, 8, 8), (1, 2, 1, 8, 20, 4), (2, 2, 2, 24, 8, 24)):
        t = 40
        chans = heads * dim + kv_heads * (dim + vdim)
        proj = torch.randn(t, chans + 6, generator=g).to(dt)
        conv_w = torch.randn(chans, taps, generator=g) * 0.6
        table = ops.build_cos_sin(rot_dims, 256, 999.0)
        y = ro.short_conv(proj[:, :chans].double(), conv_w.double())
        if dt == torch.bfloat16:
            y = y.bfloat16().double()
        rot = {"base": 999.0, "dims": rot_dims}
        nq, nk = heads * dim, kv_heads * dim
        pos = torch.arange(t)
        want_q = ro.rotate(y[:, :nq].reshape(t, heads, dim), pos, rot, "pairs")
        want_k = ro.rotate(y[:, nq:nq + nk].reshape(t, kv_heads, dim), pos, rot, "pairs")
        want_v = y[:, nq + nk:].reshape(t, kv_heads, vdim)
        n_state = (taps - 1) * chans
        for chunks in ([t], [1, 1, 2, 1, 30, 2, 3]):
            state = torch.full((2, n_state + 9), float("nan"), device=dev)
            pool = torch.zeros(4, 8 + ops.window_cache_elems(kv_heads, dim, vdim), dtype=dt, device=dev)
            pages = [3, 1]
            outs, at = [], 0
            for n in chunks:
                p = list(range(at, at + n))
                slots = torch.tensor([pages[i // PAGE] * PAGE + i % PAGE for i in p], dtype=torch.int64, device=dev)
                outs.append(ops.short_conv_qkv(proj[at:at + n].to(dev), conv_w.to(dev), heads, kv_heads, dim, vdim, state, 5,
                                               i32([0] * n, dev), i32([0, n], dev), i32([1], dev), i32(p, dev), slots,
                                               table.to(dev), rot_dims, 1, pool, 8))
                at += n
            close(torch.cat(outs), want_q, tol, f"q, taps {taps}, {len(chunks)} portions")
            kc, vc = reference.window_cache_views(pool.cpu(), 8, kv_heads, dim, vdim)
            close(kc[pages[0], :t], want_k, tol, "cached k")
            close(vc[pages[0], :t], want_v, tol, "cached v")
            if taps > 1:
                close(state[1, 5:5 + n_state].view(taps - 1, chans), proj[t - taps + 1:, :chans].double(), 1e-6, "tail")
            assert torch.isnan(state[0]).all()


# ----------------------------------------------------------------------------- the engine
def make_engine(cfg, w, device, dtype, pages=12, slots=4, budget=None, eager=True):
    folder = str(ro.write_checkpoint(tempfile.mkdtemp(prefix="rx-"), cfg, w))
    ec = EngineConfig(model=folder, dtype=dtype, device=device, max_model_len=pages * PAGE, max_num_seqs=slots,
                      max_num_batched_tokens=budget or pages * PAGE, num_gpu_blocks_override=pages,
                      enable_prefix_caching=True, enforce_eager=eager, capture_graphs_at_start=False)
    return LLMEngine(ec)


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay(engine, rid, toks, cuts, end=True):
    """Feed ``toks`` in portions of the sizes ``cuts`` (the rest one by one), all rows wanted -> logits [T, vocab]."""
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
    want, _ = ro.forward(cfg, w, toks)
    eng = make_engine(cfg, w, device, dtype, pages=pages)
    for k, cuts in enumerate(cuts_list):
        ro.check_rows(replay(eng, f"r{k}", toks, cuts), want, tol, f"cuts {cuts[:6]}")
    assert eng.bm.num_free() == pages and eng.scheduler.state_slots.num_free() == 4  # pages and slots came back
    eng.shutdown()


def check_layers(device, dtype, tol, cfg, w, n=37):
    """The residual stream after every layer."""
    toks = tokens(cfg, n, 5)
    _, want = ro.forward(cfg, w, toks)
    eng = make_engine(cfg, w, device, dtype)
    got = {}
    eng.runner.model.layer_probe = lambda i, x: got.__setitem__(i, x.detach().double().cpu())
    eng.forced_step([("a", toks, [n - 1])], ["a"])
    for i in range(want.shape[0]):
        err = ((got[i] - want[i]).pow(2).mean().sqrt() / want[i].pow(2).mean().sqrt()).item()
        assert err < tol, f"layer {i}: error {err:.3g}"
    eng.shutdown()


def check_batches(device, dtype, tol, cfg, w):
    """Unequal requests in the same steps (portions beside single tokens); pages and state slots are used
    again, by requests that start while others are in the middle of theirs."""
    lens = [150, 3, 70, 1, 129, 66, 40]
    reqs = {f"q{i}": tokens(cfg, n, 20 + i) for i, n in enumerate(lens)}
    want = {k: ro.forward(cfg, w, v)[0] for k, v in reqs.items()}
    pages = 8  # 512 tokens: less than the sum of all requests
    eng = make_engine(cfg, w, device, dtype, pages=pages, slots=3)
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    chunk = {"q0": [31, 2, 64, 1, 1, 33], "q1": [2], "q2": [5, 59, 2], "q3": [1], "q4": [64, 2, 61], "q5": [66],
             "q6": [3, 30]}
    live, waiting = [], list(reqs)
    used_slots = []
    guard = 0
    while live or waiting:
        guard += 1
        assert guard < 400
        while waiting and len(live) < 3:
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
        used_slots += [r.state_slot for r in eng.scheduler.running]
        row = 0
        for k, t, _ in entries:
            got[k].append(logits[row:row + len(t)])
            row += len(t)
        live = [k for k in live if k not in end]
    for k in reqs:
        if len(reqs[k]) >= 40 or tol < 1e-3:  # a bf16 close call in a handful of rows says nothing
            ro.check_rows(torch.cat(got[k]), want[k], tol, f"{k} ({len(reqs[k])} tokens)")
    assert eng.bm.num_free() == pages and not eng.scheduler.running and eng.scheduler.state_slots.num_free() == 3
    assert len(reqs) > 3 >= len(set(used_slots))  # seven requests went through three slots
    eng.shutdown()


def check_generate(device, dtype, cfg, w, n_new=10, eager=True):
    """Greedy generation through the engine's own entry point: scheduler, chunked prefill, sampler."""
    prompts = [tokens(cfg, n, 40 + n) for n in (90, 5, 1, 66, 30)]
    eng = make_engine(cfg, w, device, dtype, pages=10, slots=3, budget=48, eager=eager)  # prompts are cut at 48 rows
    outs = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == ro.greedy(cfg, w, p, n_new), f"prompt of {len(p)} tokens"
    assert eng.scheduler.state_slots.num_free() == 3 and eng.bm.num_free() == 10
    eng.shutdown()


def check_preemption(device, dtype, cfg, w):
    """A pool too small for all running sequences: the scheduler preempts, the victim gives its slot and
    pages back and is recomputed from its first token; the tokens do not change."""
    prompts = [tokens(cfg, n, 70 + n) for n in (60, 61, 62)]
    n_new = 20
    eng = make_engine(cfg, w, device, dtype, pages=3, slots=3, budget=64)
    outs = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, o in zip(prompts, outs):
        assert o == ro.greedy(cfg, w, p, n_new)
    eng.shutdown()
