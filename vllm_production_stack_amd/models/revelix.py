"""Revelix: a decoder whose layers, listed one by one in the configuration, mix tokens with carried
state instead of (or beside) a growing key/value cache.

A layer is pre-norm (Dynamic Tanh, fp32 residual stream) around a mixer and an optional dense
feed-forward with the xIELU activation:

- ``retention``: linear attention with a fixed decay per head.  q | k | v | g come from one fused
  projection; the recurrence kernel rotates q and k (pairs (i, i + dims / 2)), scales k, walks the
  chunk from the sequence's fp32 state slot and leaves the new state there; head outputs are brought to
  unit root mean square, gated by silu(g) and projected.
- ``parallel``: a pair of mixers fed by the same normed input through one fused input projection
  (left q | k | v with biases, right q | gate logits | v).  Left: a short causal convolution on
  every q / k / v channel (its last rows per sequence live in the state slot), rotary positions with
  ramped frequency scaling, k and v into the paged pool, softmax attention over a sliding window that
  keeps the first tokens, with capped scores, a sink logit and the heads' weights mixed after the
  softmax.  Right: linear attention with the input gate tied to the forget gate, RMS-normed per
  head.  The layer adds ``left_scale * left + right_scale * right`` to the stream.

Only windowed attention owns pool pages (K and V of every such layer, layer after layer inside a
page); everything recurrent lives in the per-sequence state slot (``state_shape``), which the engine's
scheduler hands out with the sequence and takes back when it ends.  A chunk that starts at position 0
starts from zero state, so slots need no clearing.  Logits come from the embedding table, times
``logit_scale``.
"""

from __future__ import annotations

import math

import torch

from .. import ops
from ..engine.config import ModelConfig, ParallelMixerSpec, RetentionSpec, RotarySpec
from ..ops.reference import PAGE
from ..parallel.state import get_pp, get_tp
from .batch import BatchMeta

LAYOUTS = {"half": 0, "pairs": 1}


class RevelixLayer:
    __slots__ = ("spec", "norm1", "norm2", "w_in", "b_in", "w_o", "decay", "cos_sin", "conv_w", "talk", "sink",
                 "wr_o", "gate_bias", "gate_lower", "r_norm", "w_up", "w_down", "act", "act_host", "cache_off", "state_off",
                 "state_off_right")

    def __init__(self, spec):
        for s in self.__slots__:
            setattr(self, s, None)
        self.spec = spec


class RevelixModel:
    stateful = True  # sequences carry state slots; a prefix's pages alone do not restore a sequence

    def __init__(self, cfg: ModelConfig, dtype: torch.dtype, device: torch.device, max_model_len: int):
        if get_tp().size != 1 or get_pp().size != 1:
            raise ValueError("Revelix runs on single-GPU replicas (no tensor / pipeline parallel layout yet)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Revelix runs in bfloat16 or float32")
        self.cfg = cfg
        self.dtype = dtype
        self.device = device
        self.max_model_len = max_model_len
        self.specs = cfg.layer_specs
        self.n_q = cfg.num_heads
        self.n_kv = cfg.num_kv_heads
        self.head_dim = cfg.head_dim
        self.tp_size = 1
        self.lora = None
        self.layers: list[RevelixLayer] = []
        self.embed = self.norm = None
        self.state: torch.Tensor | None = None  # [slots, state_elems] fp32, bound by the runner
        self.layer_probe = None  # callable(layer index, fp32 residual stream after the layer) for tests
        # where each layer's part of a pool page and of a state slot starts, in elements
        self.cache_offsets: dict[int, int] = {}
        self.state_offsets: dict[int, tuple] = {}
        c_off = s_off = 0

        def up4(n):  # parts of a slot start on 16-byte boundaries (the kernels then move whole float4)
            return (n + 3) // 4 * 4

        for i, s in enumerate(self.specs):
            m = s.mixer
            if isinstance(m, ParallelMixerSpec):
                self.cache_offsets[i] = c_off
                c_off += PAGE * m.left.cache_elems()
                right = s_off + up4(m.left.state_elems())
                self.state_offsets[i] = (s_off, right)
                s_off = right + up4(m.right.state_elems())
            else:
                self.state_offsets[i] = (s_off, None)
                s_off += up4(m.state_elems())
        self.page_elems = max(c_off, 8)   # a model of recurrences only still names (empty) pages
        self.state_elems = max(s_off, 8)
        self._tables: dict[tuple, torch.Tensor] = {}

    graph_capturable = True  # nothing in a decode step reads the device from the host

    # ------------------------------------------------------------------ stores
    def kv_page_shape(self) -> tuple:
        """Shape of one page of the KV pool (the runner allocates [pages, *shape])."""
        return (self.page_elems,)

    def state_shape(self) -> tuple:
        """Shape of one sequence's state slot (the runner allocates fp32 [slots, *shape])."""
        return (self.state_elems,)

    def bind_state(self, state: torch.Tensor | None) -> None:
        self.state = state

    def _cos_sin(self, rot: RotarySpec) -> torch.Tensor:
        key = (rot.base, rot.dims, rot.scaling)
        t = self._tables.get(key)
        if t is None:
            t = self._tables[key] = ops.build_cos_sin(rot.dims, self.max_model_len, rot.base, rot.table_scaling(),
                                                      device=self.device)
        return t

    # ------------------------------------------------------------------ weights
    def _alloc(self, gen, *shape, std=None, dtype=None, mean=0.0):
        dtype = dtype or self.dtype
        t = torch.empty(shape, dtype=torch.float32, device=self.device)
        t.normal_(mean, std if std is not None else shape[-1] ** -0.5, generator=gen)
        return t.to(dtype)

    def _norm(self, gen, width):
        """weight | bias | alpha of a Dynamic Tanh norm, fp32."""
        f32 = torch.float32
        return [self._alloc(gen, width, std=0.1, dtype=f32, mean=1.0), self._alloc(gen, width, std=0.05, dtype=f32),
                torch.full((1,), 0.7, dtype=f32, device=self.device)]

    def init_random(self, seed: int = 0) -> None:
        """Allocates every tensor in the layout the forward pass uses; a checkpoint overwrites them."""
        cfg = self.cfg
        w = cfg.hidden_size
        g = torch.Generator(device=self.device).manual_seed(seed)
        f32 = torch.float32
        self.embed = self._alloc(g, cfg.vocab_size, w, std=1.0)
        self.layers = []
        for i, s in enumerate(self.specs):
            m, f = s.mixer, s.mlp
            lw = RevelixLayer(s)
            lw.norm1 = self._norm(g, w)
            lw.state_off, lw.state_off_right = self.state_offsets[i]
            if isinstance(m, RetentionSpec):
                lw.w_in = self._alloc(g, m.heads * (2 * m.dim + 2 * m.vdim), w)
                lw.w_o = self._alloc(g, w, m.heads * m.vdim)
                lw.decay = torch.tensor(m.decay, dtype=f32, device=self.device)
                lw.cos_sin = self._cos_sin(m.rot)
            else:
                a, r = m.left, m.right
                lw.w_in = self._alloc(g, a.channels + r.heads * (2 * r.dim + r.vdim), w)
                lw.b_in = torch.zeros(lw.w_in.shape[0], dtype=self.dtype, device=self.device)
                lw.b_in[:a.channels] = self._alloc(g, a.channels, std=0.2)
                lw.conv_w = self._alloc(g, a.channels, a.conv, std=a.conv ** -0.5, dtype=f32)
                lw.talk = (torch.eye(a.heads, dtype=f32, device=self.device)
                           + self._alloc(g, a.heads, a.heads, std=0.1, dtype=f32))
                lw.sink = self._alloc(g, a.heads, std=1.0, dtype=f32)
                lw.w_o = self._alloc(g, w, a.heads * a.vdim)
                lw.cos_sin = self._cos_sin(a.rot)
                lw.cache_off = self.cache_offsets[i]
                lw.gate_bias = self._alloc(g, r.heads * r.dim, std=1.0, dtype=f32, mean=1.0)
                lw.gate_lower = torch.rand(r.heads * r.dim, dtype=f32, device=self.device, generator=g) * 0.9
                lw.r_norm = self._alloc(g, r.vdim, std=0.1, dtype=f32, mean=1.0)
                lw.wr_o = self._alloc(g, w, r.heads * r.vdim)
            if f is not None:
                lw.norm2 = self._norm(g, w)
                lw.w_up = self._alloc(g, f.ff, w)
                lw.w_down = self._alloc(g, w, f.ff)
                self.set_activation(lw, math.log(2.0), 0.5 + math.log(2.0))
            self.layers.append(lw)
        self.norm = self._norm(g, w)

    def set_activation(self, lw: RevelixLayer, a_pos: float, a_neg: float) -> None:
        """The two curvatures of a layer's xIELU: on the device for the activation kernel (no host value
        enters a captured step) and on the host for the GEMM epilogue's launch arguments."""
        lw.act = torch.tensor([a_pos, a_neg], dtype=torch.float32, device=self.device)
        lw.act_host = tuple(lw.act.tolist())

    @property
    def lm_head(self) -> torch.Tensor:  # the embedding table is the output matrix
        return self.embed

    def weight_tensors(self):
        if self.embed is not None:
            yield self.embed
        for n in (self.norm or []):
            yield n
        for lw in self.layers:
            for s in RevelixLayer.__slots__:
                t = getattr(lw, s)
                if s == "cos_sin":
                    continue
                if isinstance(t, torch.Tensor):
                    yield t
                elif isinstance(t, list):
                    yield from t

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.weight_tensors())

    # ------------------------------------------------------------------ batch description
    def plan_batch(self, meta: BatchMeta, plan: dict, to_dev) -> None:
        """Sequences of the step for the kernels that walk them: decode rows (one row each), then the
        prefill chunks; every sequence with its state slot."""
        nd = plan["num_decode"]
        q_lens = [1] * nd + list(plan.get("q_lens", []))
        cu, seq = [0], []
        for i, n in enumerate(q_lens):
            cu.append(cu[-1] + n)
            seq.extend([i] * n)
        meta.seq_cu = to_dev(cu, torch.int32)
        meta.seq_state = to_dev(plan["state_slots"], torch.int32)
        meta.row_seq = to_dev(seq, torch.int32)
        cut = ops.build_scan_pieces(q_lens) if self.device.type == "cuda" else None
        if cut is not None:
            meta.scan_pieces = tuple(torch.from_numpy(a).pin_memory().to(self.device, non_blocking=True) for a in cut)
        if plan["num_prefill"]:
            meta.pre_row_seq = to_dev([s - nd for s in seq[nd:]], torch.int32)
            meta.pre_win_tiles = {}
            if self.device.type == "cuda" and self.dtype == torch.bfloat16:
                for key in sorted({(s.mixer.left.heads, s.mixer.left.kv_heads) for s in self.specs
                                   if isinstance(s.mixer, ParallelMixerSpec)
                                   and ops.window_mfma_supported(s.mixer.left.heads, s.mixer.left.kv_heads,
                                                                 s.mixer.left.dim, s.mixer.left.vdim)}):
                    tiles = ops.build_window_tiles(plan["q_lens"], plan["pre_ctx"], *key)
                    meta.pre_win_tiles[key] = torch.from_numpy(tiles).pin_memory().to(self.device, non_blocking=True)

    def plan_decode_graph(self, meta: BatchMeta, bsz: int, state_slots: torch.Tensor) -> None:
        """The same for a captured decode step of ``bsz`` rows: ``state_slots`` is a graph input."""
        meta.seq_cu = torch.arange(bsz + 1, dtype=torch.int32, device=self.device)
        meta.seq_state = state_slots
        meta.row_seq = None

    # ------------------------------------------------------------------ forward
    def _retention(self, lw: RevelixLayer, h: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        m: RetentionSpec = lw.spec.mixer
        hd, hv = m.heads * m.dim, m.heads * m.vdim
        proj = ops.linear(h, lw.w_in)  # q | k | v | g
        o = ops.recurrent_scan(proj, 0, hd, 2 * hd, m.heads, m.dim, m.vdim, self.state, lw.state_off, meta.seq_cu,
                               meta.seq_state, meta.positions, decay=lw.decay, cos_sin=lw.cos_sin, rot_dims=m.rot.dims,
                               layout=LAYOUTS[m.rot.layout], k_scale=m.dim ** -0.5, pieces=meta.scan_pieces,
                               min_decay=min(m.decay))
        y = ops.head_rms_norm(o, self.cfg.norm_eps, self.dtype, gate=proj[:, 2 * hd + hv:2 * hd + 2 * hv])
        return ops.linear(y, lw.w_o)

    def _parallel(self, lw: RevelixLayer, h: torch.Tensor, pool, meta: BatchMeta):
        m: ParallelMixerSpec = lw.spec.mixer
        a, r = m.left, m.right
        proj = ops.linear(h, lw.w_in, lw.b_in)  # left q | k | v, right q | gate logits | v
        q = ops.short_conv_qkv(proj, lw.conv_w, a.heads, a.kv_heads, a.dim, a.vdim, self.state, lw.state_off,
                               meta.row_seq, meta.seq_cu, meta.seq_state, meta.positions, meta.slots, lw.cos_sin,
                               a.rot.dims, LAYOUTS[a.rot.layout], pool, lw.cache_off)
        t, nd = h.shape[0], meta.num_decode
        u = torch.empty((t, a.heads, a.kv_heads, a.vdim), dtype=torch.float32, device=h.device)
        if nd > 0:
            # the split count follows the batch rounded up to a power of two, which an eager step and the
            # captured step of its batch bucket share: both then sum in the same order
            splits = ops.window_decode_splits(1 << (nd - 1).bit_length(), a.kv_heads, a.window, a.keep_first,
                                              self.max_model_len)
            ops.window_attention(q[:nd], pool, lw.cache_off, a.kv_heads, a.vdim, meta.dec_block_tables, None,
                                 meta.positions[:nd], a.window, a.keep_first, a.scale, a.softcap, lw.sink, out=u[:nd],
                                 splits=splits)
        if meta.num_prefill_seqs > 0:
            ops.window_attention(q[nd:], pool, lw.cache_off, a.kv_heads, a.vdim, meta.pre_block_tables,
                                 meta.pre_row_seq, meta.positions[nd:], a.window, a.keep_first, a.scale, a.softcap,
                                 lw.sink, out=u[nd:], tiles=(meta.pre_win_tiles or {}).get((a.heads, a.kv_heads)))
        left = ops.linear(ops.mix_heads(u, lw.talk, self.dtype), lw.w_o)
        c0 = a.channels
        rd = r.heads * r.dim
        o = ops.recurrent_scan(proj, c0, c0 + rd, c0 + 2 * rd, r.heads, r.dim, r.vdim, self.state, lw.state_off_right,
                               meta.seq_cu, meta.seq_state, meta.positions, gate_bias=lw.gate_bias,
                               gate_lower=lw.gate_lower, pieces=meta.scan_pieces)
        right = ops.linear(ops.head_rms_norm(o, self.cfg.norm_eps, self.dtype, weight=lw.r_norm), lw.wr_o)
        return [(left, m.left_scale), (right, m.right_scale)]

    def forward(self, input_ids: torch.Tensor, pool: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        """Final-normed hidden states of ``meta.logits_rows`` ([num_out, width], activation dtype)."""
        x = ops.embed_scale(input_ids, self.embed, 1.0)  # fp32 residual stream
        d: list = []  # mixer / feed-forward outputs not yet added to the stream, with their factors
        for i, lw in enumerate(self.layers):
            h = ops.add_dyt_norm(x, d, *lw.norm1, self.dtype)
            if lw.spec.type == "retention":
                d = [(self._retention(lw, h, meta), 1.0)]
            else:
                d = self._parallel(lw, h, pool, meta)
            if lw.spec.mlp is not None:
                h = ops.add_dyt_norm(x, d, *lw.norm2, self.dtype)
                d = [(ops.linear(ops.up_xielu(h, lw.w_up, lw.act, lw.act_host), lw.w_down), 1.0)]
            if self.layer_probe is not None:
                self.layer_probe(i, x + sum(t.float() * c for t, c in d))
        if meta.logits_rows is not None:
            x = x.index_select(0, meta.logits_rows)
            d = [(t.index_select(0, meta.logits_rows), c) for t, c in d]
        return ops.add_dyt_norm(x, d, *self.norm, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(hidden, self.embed)
        if self.cfg.logit_scale != 1.0:
            logits = logits.float() * self.cfg.logit_scale
        return logits
