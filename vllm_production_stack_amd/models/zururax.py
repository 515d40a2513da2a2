"""Zururax: a decoder whose layers are listed one by one in the configuration.

Every layer is pre-norm around a latent-attention mixer and an optional feed-forward (dense
squared-ReLU, or a mixture of clamped gated units with group-limited sigmoid routing and a gated
shared unit).  The residual stream is fp32 whatever the activation dtype; a projection's output is
added to it by the norm kernel that follows (``ops.add_rms_norm``), as the framework's other
decoders do with their bf16 stream.

Latent attention over the paged pool: a token's cache entry is its RMS-normed KV latent and the
rotated key part shared by all heads (``kv_rank + rot_dim`` values; layers with ``kv_from`` read the
entries of the layer they name and own no cache).  Keys and values are never expanded: a head's
unrotated query is carried into latent space (q W_uk, one batched matrix product), the attention
kernel scores it against the entries and returns the probability-weighted latent, and W_uv takes
that to the head's value space.  All heads then share one key/value stream per token.  Large prefill
parts (``EXPAND_MIN_ROWS``) are the exception: there the 3.4 x FLOPs of latent space outweigh what it
saves, so values and unrotated keys of every head are expanded for the step (one library product over
the sequences' gathered entries) and the same tile kernel runs over per-head entries.

The input projections of a mixer (query latent | KV latent and shared key part | output-gate logits)
are one fused matrix, as are gate | up of every gated unit; the router's matrix (with the shared
unit's gate row appended) is fp32 and its product is a true fp32 one.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import ops
from ..engine.config import FeedForwardSpec, LatentMixerSpec, ModelConfig
from ..ops.reference import PAGE
from ..parallel.state import get_pp, get_tp
from .batch import BatchMeta

# Prefill parts of at least this many rows expand keys and values per head for the step (below, the
# expansion of the whole context costs more than latent space saves)
EXPAND_MIN_ROWS = 256
GLU_ALPHA = 1.702   # the gated units' sigmoid slope
GLU_UP_BIAS = 1.0   # and the offset of their linear branch


class ZururaxLayer:
    __slots__ = ("spec", "norm1", "norm2", "w_in", "dq_norm", "dkv_norm", "w_uq", "w_uk", "w_uv", "sink", "w_o",
                 "w_up", "w_down", "router", "w13", "w2", "w_sh13", "w_sh2", "cache_offset", "cos_sin", "w_vk")

    def __init__(self, spec):
        for s in self.__slots__:
            setattr(self, s, None)
        self.spec = spec


class ZururaxModel:
    @property
    def graph_capturable(self) -> bool:
        """Decode steps can be captured when no layer's mixture falls back to the per-unit loop, which
        reads the row counts on the host (shapes the grouped GEMM does not tile, fp32)."""
        return self.dtype == torch.bfloat16 and self.device.type == "cuda" and all(
            lw.w13 is None or ops.moe_glu_grouped_supported(torch.empty((1, self.cfg.hidden_size), dtype=self.dtype,
                                                                         device=self.device), lw.w13, lw.w2)
            for lw in self.layers)

    def __init__(self, cfg: ModelConfig, dtype: torch.dtype, device: torch.device, max_model_len: int):
        if get_tp().size != 1 or get_pp().size != 1:
            raise ValueError("Zururax runs on single-GPU replicas (no tensor / pipeline parallel layout yet)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Zururax runs in bfloat16 or float32")
        self.cfg = cfg
        self.dtype = dtype
        self.device = device
        self.max_model_len = max_model_len
        self.specs = cfg.layer_specs
        self.n_q = cfg.num_heads
        self.n_kv = 1
        self.head_dim = cfg.head_dim
        self.tp_size = 1
        self.lora = None
        self.layers: list[ZururaxLayer] = []
        self.embed = self.norm = self.lm_head = None
        self.layer_probe = None  # callable(layer index, fp32 residual stream after the layer) for tests
        # where each caching layer's entries start inside a page, in elements
        off = 0
        self.cache_offsets: dict[int, int] = {}
        for i, s in enumerate(self.specs):
            if s.mixer.kv_from is None:
                self.cache_offsets[i] = off
                off += PAGE * s.mixer.entry
        self.page_elems = off
        self._tables: dict[tuple, torch.Tensor] = {}

    # ------------------------------------------------------------------ cache layout
    def kv_page_shape(self) -> tuple:
        """Shape of one page of the KV pool (the runner allocates [pages, *shape])."""
        return (self.page_elems,)

    def _cos_sin(self, m: LatentMixerSpec) -> torch.Tensor:
        key = (m.rope_base, m.rope_dims)
        t = self._tables.get(key)
        if t is None:
            t = self._tables[key] = ops.build_cos_sin(m.rope_dims, self.max_model_len, m.rope_base, None,
                                                      device=self.device)
        return t

    # ------------------------------------------------------------------ weights
    def _alloc(self, gen, *shape, std=None, dtype=None, ones=False):
        dtype = dtype or self.dtype
        if ones:
            return torch.ones(shape, dtype=dtype, device=self.device)
        t = torch.empty(shape, dtype=torch.float32, device=self.device)
        t.normal_(0.0, std if std is not None else shape[-1] ** -0.5, generator=gen)
        return t.to(dtype)

    def init_random(self, seed: int = 0) -> None:
        """Allocates every tensor in the layout the forward pass uses; a checkpoint overwrites them.
        Projections are drawn with std 1/sqrt(fan-in) so that activations stay of order one."""
        cfg = self.cfg
        w = cfg.hidden_size
        g = torch.Generator(device=self.device).manual_seed(seed)
        f32 = torch.float32
        self.embed = self._alloc(g, cfg.vocab_size, w, std=1.0)
        self.layers = []
        for i, s in enumerate(self.specs):
            m, f = s.mixer, s.mlp
            lw = ZururaxLayer(s)
            own = m.kv_from is None
            lw.norm1 = self._alloc(g, w, ones=True, dtype=f32)
            lw.w_in = self._alloc(g, m.q_rank + (m.entry if own else 0) + (m.heads if m.out_gate else 0), w)
            lw.dq_norm = self._alloc(g, m.q_rank, ones=True, dtype=f32)
            lw.dkv_norm = self._alloc(g, m.kv_rank, ones=True, dtype=f32) if own else None
            lw.w_uq = self._alloc(g, m.heads * (m.dim + m.rot_dim), m.q_rank)
            lw.w_uk = self._alloc(g, m.heads, m.dim, m.kv_rank)
            lw.w_uv = self._alloc(g, m.heads, m.vdim, m.kv_rank)
            lw.sink = self._alloc(g, m.heads, std=1.0, dtype=f32) if m.sink else None
            lw.w_o = self._alloc(g, w, m.heads * m.vdim)
            lw.cache_offset = self.cache_offsets[i if own else m.kv_from]
            lw.cos_sin = self._cos_sin(m)
            if f is not None:
                lw.norm2 = self._alloc(g, w, ones=True, dtype=f32)
                if f.kind == "dense":
                    lw.w_up = self._alloc(g, f.ff, w)
                    lw.w_down = self._alloc(g, w, f.ff)
                else:
                    lw.router = self._alloc(g, f.experts + (1 if f.shared_ff else 0), w, dtype=f32)
                    lw.w13 = self._alloc(g, f.experts, 2 * f.ff, w)
                    lw.w2 = self._alloc(g, f.experts, w, f.ff)
                    if f.shared_ff:
                        lw.w_sh13 = self._alloc(g, 2 * f.shared_ff, w)
                        lw.w_sh2 = self._alloc(g, w, f.shared_ff)
            self.layers.append(lw)
        self.norm = self._alloc(g, w, ones=True, dtype=f32)
        self.lm_head = self._alloc(g, cfg.vocab_size, w)

    def weight_tensors(self):
        for t in (self.embed, self.norm, self.lm_head):
            if t is not None:
                yield t
        for lw in self.layers:
            for s in ZururaxLayer.__slots__:
                t = getattr(lw, s)
                if isinstance(t, torch.Tensor) and s not in ("cos_sin", "w_vk"):
                    yield t

    # derived copies (rebuilt from the weights when needed): per head [W_uv; W_uk], the matrix that
    # expands latents into values and unrotated keys for large prefill parts
    def packed_tensors(self):
        for lw in self.layers:
            if lw.w_vk is not None:
                yield lw.w_vk

    def drop_packed(self) -> None:
        for lw in self.layers:
            lw.w_vk = None

    def _expands(self, m: LatentMixerSpec) -> bool:
        return (self.device.type == "cuda" and self.dtype == torch.bfloat16 and m.kv_rank % 8 == 0
                and ops.latent_mfma_supported(m.vdim, m.dim + m.rot_dim))

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.weight_tensors())

    # ------------------------------------------------------------------ batch description
    def plan_prefill(self, meta: BatchMeta, q_lens: list[int], ctx_lens: list[int], to_dev) -> None:
        """Which sequence of the prefill part each prefill row belongs to."""
        seq: list[int] = []
        for i, n in enumerate(q_lens):
            seq.extend([i] * n)
        meta.pre_row_seq = to_dev(seq, torch.int32)
        meta.pre_lat_tiles = {}
        meta.pre_expand = {}
        if sum(q_lens) >= EXPAND_MIN_ROWS:
            for heads in sorted({s.mixer.heads for s in self.specs if self._expands(s.mixer)}):
                meta.pre_expand[heads] = self._plan_expanded(q_lens, ctx_lens, heads)
        if self.device.type == "cuda" and self.dtype == torch.bfloat16:
            for heads in sorted({s.mixer.heads for s in self.specs
                                 if ops.latent_mfma_supported(s.mixer.kv_rank, s.mixer.rot_dim)}):
                tiles = ops.build_latent_tiles(q_lens, ctx_lens, heads)
                meta.pre_lat_tiles[heads] = torch.from_numpy(tiles).pin_memory().to(self.device, non_blocking=True)

    def _plan_expanded(self, q_lens, ctx_lens, heads: int) -> dict:
        """Layout of a step's expanded entries (one run of pages per prefill sequence and head) and the
        tile list over them: 64 consecutive tokens of one head per tile."""
        import numpy as np

        n_pages = [(c + PAGE - 1) // PAGE for c in ctx_lens]
        width = max(n_pages)
        bt = np.zeros((len(q_lens) * heads, width), dtype=np.int32)
        parts, base, row = [], [], 0
        total = 0
        for i, (n, ctx, npg) in enumerate(zip(q_lens, ctx_lens, n_pages)):
            base.append(total)
            for h in range(heads):
                bt[i * heads + h, :npg] = total + h * npg + np.arange(npg)
            k = np.arange(0, n, 64, dtype=np.int64)
            for h in range(heads):
                parts.append(np.stack([np.full_like(k, i * heads + h), row + k, np.minimum(64, n - k), ctx - n + k,
                                       np.full_like(k, h), np.ones_like(k)], axis=1))
            total += heads * npg
            row += n
        tiles = np.concatenate(parts)
        tiles = tiles[np.argsort(-(tiles[:, 3] + tiles[:, 2]), kind="stable")].astype(np.int32)
        return {"n_pages": n_pages, "base": base, "total": total,
                "bt": torch.from_numpy(bt).pin_memory().to(self.device, non_blocking=True),
                "tiles": torch.from_numpy(tiles).pin_memory().to(self.device, non_blocking=True)}

    def _expanded_prefill(self, lw: ZururaxLayer, q: torch.Tensor, pool, meta: BatchMeta, plan: dict, out: torch.Tensor):
        """Attention of the prefill rows with keys and values expanded per head for this step: the
        sequences' entries are gathered from the pool, one library product makes values and unrotated
        keys of every head, and the tile kernel runs over per-head entries value | key | rotated part
        (its first product reads zeros against the value channels).  640 / 2176 of the latent form's
        FLOPs per query-key pair at 128 + 64 / 128 channels and rank 512."""
        m: LatentMixerSpec = lw.spec.mixer
        h, v, d, r, kr = m.heads, m.vdim, m.dim, m.rot_dim, m.kv_rank
        if lw.w_vk is None:
            lw.w_vk = torch.cat([lw.w_uv, lw.w_uk], dim=1).reshape(h * (v + d), kr).contiguous()
        wide = v + d + r
        view = pool[:, lw.cache_offset:lw.cache_offset + PAGE * m.entry].view(pool.shape[0], PAGE, m.entry)
        exp = torch.empty((plan["total"], PAGE * wide), dtype=q.dtype, device=q.device)
        for s, (npg, base) in enumerate(zip(plan["n_pages"], plan["base"])):
            ent = view[meta.pre_block_tables[s, :npg].long()]                      # [pages, 64, entry]
            vk = ops.linear(ent[:, :, :kr].reshape(npg * PAGE, kr), lw.w_vk)       # [keys, heads * (v + d)]
            dst = exp[base:base + h * npg].view(h, npg, PAGE, wide)
            dst[:, :, :, :v + d] = vk.view(npg, PAGE, h, v + d).permute(2, 0, 1, 3)
            dst[:, :, :, v + d:] = ent[:, :, kr:].unsqueeze(0)
        t = q.shape[0]
        zeros = torch.zeros((1, 1, v), dtype=q.dtype, device=q.device).expand(t, h, v)
        if not ops.latent_tile_kernel_takes(zeros, q, exp, out):
            raise RuntimeError("expanded prefill: operands the tile kernel does not take")
        ops.latent_attention(zeros, q, exp, 0, plan["bt"], None, meta.positions[meta.num_decode:], lw.sink, m.scale,
                             out=out, tiles=plan["tiles"])

    # ------------------------------------------------------------------ forward
    def _mixer(self, lw: ZururaxLayer, h: torch.Tensor, pool, meta: BatchMeta) -> torch.Tensor:
        m: LatentMixerSpec = lw.spec.mixer
        eps = self.cfg.norm_eps
        t = h.shape[0]
        proj = ops.linear(h, lw.w_in)
        col = m.q_rank
        cq = ops.rms_norm_rows(proj[:, :col], lw.dq_norm, eps)
        q = ops.linear(cq, lw.w_uq).view(t, m.heads, m.dim + m.rot_dim)
        ops.rope_pairs(q, meta.positions, lw.cos_sin, m.dim, m.rope_dims)
        if m.kv_from is None:
            ops.latent_kv_write(proj[:, col:col + m.entry], lw.dkv_norm, meta.positions, meta.slots, lw.cos_sin, pool,
                                lw.cache_offset, m.kv_rank, m.rot_dim, m.rope_dims, eps)
            col += m.entry
        nd = meta.num_decode
        plan = (getattr(meta, "pre_expand", None) or {}).get(m.heads) if self._expands(m) else None
        if plan is not None and meta.num_prefill_seqs > 0:
            # large prefill part: per-head keys and values for this step; decode rows stay in latent space
            o = torch.empty((t, m.heads, m.vdim), dtype=h.dtype, device=h.device)
            self._expanded_prefill(lw, q[nd:], pool, meta, plan, o[nd:])
            if nd > 0:
                q_lat = torch.bmm(q[:nd, :, :m.dim].transpose(0, 1), lw.w_uk).transpose(0, 1)
                o_lat = ops.latent_attention(q_lat, q[:nd, :, m.dim:], pool, lw.cache_offset, meta.dec_block_tables, None,
                                             meta.positions[:nd], lw.sink, m.scale,
                                             splits=getattr(meta, "dec_num_splits", 1) or 1)
                o[:nd] = torch.bmm(o_lat.transpose(0, 1), lw.w_uv.transpose(1, 2)).transpose(0, 1)
            if m.out_gate:
                ops.sigmoid_gate(o, proj[:, col:col + m.heads])
            return ops.linear(o.view(t, m.heads * m.vdim), lw.w_o)
        # [heads, T, dim] x [heads, dim, kv_rank]: the unrotated query in latent space
        q_lat = torch.bmm(q[:, :, :m.dim].transpose(0, 1), lw.w_uk).transpose(0, 1)
        q_rot = q[:, :, m.dim:]
        o_lat = torch.empty((t, m.heads, m.kv_rank), dtype=h.dtype, device=h.device)
        if nd > 0:
            ops.latent_attention(q_lat[:nd], q_rot[:nd], pool, lw.cache_offset, meta.dec_block_tables, None,
                                 meta.positions[:nd], lw.sink, m.scale, out=o_lat[:nd],
                                 splits=getattr(meta, "dec_num_splits", 1) or 1)
        if meta.num_prefill_seqs > 0:
            ops.latent_attention(q_lat[nd:], q_rot[nd:], pool, lw.cache_offset, meta.pre_block_tables,
                                 meta.pre_row_seq, meta.positions[nd:], lw.sink, m.scale, out=o_lat[nd:],
                                 tiles=(meta.pre_lat_tiles or {}).get(m.heads))
        # [heads, T, kv_rank] x [heads, kv_rank, vdim] -> [T, heads, vdim]
        o = torch.bmm(o_lat.transpose(0, 1), lw.w_uv.transpose(1, 2)).transpose(0, 1).contiguous()
        if m.out_gate:
            ops.sigmoid_gate(o, proj[:, col:col + m.heads])
        return ops.linear(o.view(t, m.heads * m.vdim), lw.w_o)

    def _moe(self, lw: ZururaxLayer, h: torch.Tensor, residual: torch.Tensor) -> None:
        """Adds the mixture's output for rows h into the fp32 residual stream."""
        f: FeedForwardSpec = lw.spec.mlp
        t = h.shape[0]
        logits = F.linear(h.float(), lw.router)  # a true fp32 product
        w, ids, gate = ops.group_topk(logits, f.experts, f.groups, f.keep, f.top, f.route_scale, extra=f.shared_ff > 0)
        shared = None
        if f.shared_ff:
            shared = ops.linear(ops.gate_up_glu_clamp(h, lw.w_sh13, f.shared_limit, GLU_ALPHA, GLU_UP_BIAS), lw.w_sh2)
        if ops.moe_glu_grouped_supported(h, lw.w13, lw.w2):
            ys, pos = ops.moe_glu_grouped(h, lw.w13, lw.w2, ids, f.limit, GLU_ALPHA, GLU_UP_BIAS)
            ops.moe_finish(residual, ys, w, pos, shared, gate)
            return
        # the CPU, fp32, and shapes the grouped kernel does not tile: unit by unit on the sorted rows
        offsets, pos, sorted_tok = ops.moe_align(ids, f.experts)
        xs = ops.gather_rows(h, sorted_tok)
        ys = torch.empty((t * f.top, h.shape[1]), dtype=h.dtype, device=h.device)
        off = offsets.tolist()
        for e in range(f.experts):
            a, b = off[e], off[e + 1]
            if b > a:
                act = ops.glu_clamp(F.linear(xs[a:b], lw.w13[e]), f.limit, GLU_ALPHA, GLU_UP_BIAS)
                torch.matmul(act, lw.w2[e].t(), out=ys[a:b])
        ops.moe_finish(residual, ys, w, pos, shared, gate)

    def forward(self, input_ids: torch.Tensor, pool: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        """Final-normed hidden states of ``meta.logits_rows`` ([num_out, width], activation dtype)."""
        cfg = self.cfg
        eps = cfg.norm_eps
        x = ops.embed_scale(input_ids, self.embed, cfg.embedding_scale)  # fp32 residual stream
        d = None  # a projection output not yet added to the stream
        for i, lw in enumerate(self.layers):
            h = ops.add_rms_norm(x, d, lw.norm1, eps, self.dtype)
            d = self._mixer(lw, h, pool, meta)
            f = lw.spec.mlp
            if f is not None:
                h = ops.add_rms_norm(x, d, lw.norm2, eps, self.dtype)
                d = None
                if f.kind == "dense":
                    d = ops.linear(ops.up_relu_sq(h, lw.w_up), lw.w_down)
                else:
                    self._moe(lw, h, x)
            if self.layer_probe is not None:
                self.layer_probe(i, x if d is None else x + d.float())
        if meta.logits_rows is not None:
            x = x.index_select(0, meta.logits_rows)
            d = None if d is None else d.index_select(0, meta.logits_rows)
        return ops.add_rms_norm(x, d, self.norm, eps, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear(hidden, self.lm_head)
