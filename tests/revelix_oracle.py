"""Revelix in float64, written from the design's equations: one function per mechanism, whole
sequences recomputed token by token, no cache, no state carried between calls, nothing shared with
the engine.  Also makers of small random checkpoints in the design's file format."""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- mechanisms
def dyt(x, w, b, alpha):
    """Dynamic Tanh: an elementwise squashing norm without statistics."""
    return torch.tanh(alpha * x) * w + b


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def frequencies(base: float, dims: int, scaling: dict | None = None):
    """(angle per position step for each of the dims / 2 pairs, factor on cos and sin)."""
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def where(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, pos, rot: dict, layout: str):
    """x [T, heads, d]: the first rot['dims'] channels of every head turn by pos * f_i; pairs are
    (i, i + dims / 2) for layout 'half' and (2 i, 2 i + 1) for 'pairs'."""
    dims = int(rot["dims"])
    f, m = frequencies(float(rot["base"]), dims, rot.get("scaling"))
    ang = pos.to(F64)[:, None] * f[None, :]
    c, s = (ang.cos() * m)[:, None, :], (ang.sin() * m)[:, None, :]
    out = x.clone()
    if layout == "half":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


def short_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    t, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for j in range(taps):
        shift = taps - 1 - j
        if shift < t:
            y[shift:] += w[:, j] * u[:t - shift]
    return y


def xielu(z, p, q):
    sp = torch.nn.functional.softplus
    pos = sp(p) * z * z + z / 2
    neg = (0.5 + sp(q)) * (torch.expm1(z) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def linear_recurrence(q, k, v, a):
    """q, k, a [T, H, d], v [T, H, vd]: per head S_t = diag(a_t) S_(t-1) + k_t v_t^T from S = 0, o_t = S_t^T q_t."""
    t, H, d = q.shape
    o = torch.zeros(t, H, v.shape[-1], dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, v.shape[-1], dtype=F64)
        for i in range(t):
            S = a[i, hd][:, None] * S + torch.outer(k[i, hd], v[i, hd])
            o[i, hd] = S.T @ q[i, hd]
    return o


def retention(h, W, m: dict, eps: float):
    """The mixer of a 'retention' layer over one sequence h [T, width]."""
    t = h.shape[0]
    H, d, vd = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(t)
    q = rotate((h @ W["q"].T).view(t, H, d), pos, m["rot"], "half")
    k = rotate((h @ W["k"].T).view(t, H, d), pos, m["rot"], "half") * d ** -0.5
    v = (h @ W["v"].T).view(t, H, vd)
    decay = torch.tensor(m["decay"], dtype=F64).view(1, H, 1).expand(t, H, d)
    o = linear_recurrence(q, k, v, decay)
    o = rms_unit(o, eps).reshape(t, H * vd) * torch.nn.functional.silu(h @ W["g"].T)
    return o @ W["o"].T


def window_weights(q, k, pos_q, pos_k, heads_per_kv: int, scale, cap, size, keep, sink):
    """Softmax weights [H, Tq, Tk] of queries at positions pos_q over keys at positions pos_k: capped
    scores, the window with kept first tokens, the sink in the denominator only."""
    H = q.shape[1]
    i, j = pos_q[:, None], pos_k[None, :]
    seen = (j <= i) & ((i - j < size) | (j < keep))
    out = torch.zeros(H, q.shape[0], k.shape[0], dtype=F64)
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd // heads_per_kv].T) * scale
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~seen, -math.inf)
        mx = torch.maximum(s.max(-1, keepdim=True).values, sink[hd])
        e = torch.exp(s - mx)
        out[hd] = e / (e.sum(-1, keepdim=True) + torch.exp(sink[hd] - mx))
    return out


def mixed_values(weights, talk, v, heads_per_kv: int):
    """weights [H, Tq, Tk] mixed across heads by talk [H, H]; head h reads the values of its own KV head."""
    mixed = torch.einsum("hg,gij->hij", talk, weights)
    return torch.stack([mixed[hd] @ v[:, hd // heads_per_kv] for hd in range(weights.shape[0])], dim=1)


def window_attention(h, W, m: dict):
    """The left half of a 'parallel' mixer: grouped-query attention behind a short convolution, with a
    capped score, a sliding window that keeps the first tokens, a sink in the denominator and the
    heads' weights mixed after the softmax."""
    t = h.shape[0]
    H, G, d, vd = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(t)
    q = short_conv(h @ W["q"].T + W["q.b"], W["q.conv"])
    k = short_conv(h @ W["k"].T + W["k.b"], W["k.conv"])
    v = short_conv(h @ W["v"].T + W["v.b"], W["v.conv"]).view(t, G, vd)
    q = rotate(q.view(t, H, d), pos, m["rot"], "pairs")
    k = rotate(k.view(t, G, d), pos, m["rot"], "pairs")
    w = window_weights(q, k, pos, pos, H // G, float(m["scale"]), float(m["softcap"]), int(m["mask"]["size"]),
                       int(m["mask"]["keep_first"]), W["sink"])
    return mixed_values(w, W["talk"], v, H // G).reshape(t, H * vd) @ W["o"].T


def gated_recurrence(h, W, m: dict, eps: float):
    """The right half of a 'parallel' mixer: input gate tied to the forget gate (1 - f is written where f is kept)."""
    t = h.shape[0]
    H, d, vd = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = torch.nn.functional.silu(h @ W["q"].T).view(t, H, d)
    v = (h @ W["v"].T).view(t, H, vd)
    f = (W["lower"] + (1 - W["lower"]) * torch.sigmoid(h @ W["f"].T + W["f.b"])).view(t, H, d)
    o = rms_unit(linear_recurrence(q, 1 - f, v, f), eps) * W["norm"]
    return o.reshape(t, H * vd) @ W["o"].T


# ----------------------------------------------------------------------------- the model
def _sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def _norm(x, weights, name):
    return dyt(x, weights[name], weights[name + ".b"], weights[name + ".alpha"])


def forward(cfg: dict, weights: dict, tokens: list[int]):
    """-> (logits [T, vocab], residual stream after every layer [layers, T, width]), float64."""
    w = {k: v.to(F64) for k, v in weights.items() if v.dtype != torch.int32}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)]
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = _norm(x, w, p + "norm1")
        m = layer["mixer"]
        if layer["type"] == "retention":
            x = x + retention(h, _sub(w, p + "mix."), m, eps)
        elif layer["type"] == "parallel":
            left = window_attention(h, _sub(w, p + "mix.left."), m["left"])
            right = gated_recurrence(h, _sub(w, p + "mix.right."), m["right"], eps)
            x = x + float(m["left_scale"]) * left + float(m["right_scale"]) * right
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            h = _norm(x, w, p + "norm2")
            act = w[p + "mlp.act"]
            x = x + xielu(h @ w[p + "mlp.up"].T, act[0], act[1]) @ w[p + "mlp.down"].T
        streams.append(x.clone())
    x = _norm(x, w, "final.norm")
    return (x @ w["embed"].T) * float(cfg["logit_scale"]), torch.stack(streams)


# ----------------------------------------------------------------------------- small random checkpoints
def retention_layer(heads=2, dim=16, vdim=24, decay=None, rot_dims=None, base=10000.0, mlp=None):
    return {"type": "retention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": rot_dims or dim},
                      "decay": decay or [1 - 2.0 ** -(3 + i) for i in range(heads)]}}


def parallel_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, size=24, keep=3, rot_dims=None, base=10000.0,
                   scaling=None, softcap=30.0, scale=None, r_heads=2, r_dim=8, r_vdim=16, left_scale=0.7,
                   right_scale=1.2, mlp=None):
    rot = {"base": base, "dims": rot_dims or dim}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                               "mask": {"size": size, "keep_first": keep}, "rot": rot, "softcap": softcap,
                               "scale": scale if scale is not None else dim ** -0.5},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim},
                      "left_scale": left_scale, "right_scale": right_scale}}


def make_config(layers, vocab=96, width=48, logit_scale=0.7, eps=1e-5):
    return {"architecture": "Revelix", "vocab": vocab, "width": width, "layers": layers, "logit_scale": logit_scale,
            "norm": {"eps": eps}}


def random_weights(cfg: dict, seed: int = 0) -> dict:
    """bf16 tensors by the design's names; projections ~ 1 / sqrt(fan-in), biases, sinks, gates of order one."""
    g = torch.Generator().manual_seed(seed)
    w = int(cfg["width"])
    out: dict[str, torch.Tensor] = {}

    def mat(name, rows, cols, std=None):
        out[name] = (torch.randn(rows, cols, generator=g) * (std if std is not None else cols ** -0.5)).bfloat16()

    def vec(name, n, mean=0.0, std=1.0):
        out[name] = (mean + std * torch.randn(n, generator=g)).bfloat16()

    def norm(name):
        vec(name, w, 1.0, 0.2)
        vec(name + ".b", w, 0.0, 0.1)
        out[name + ".alpha"] = (0.5 + 0.5 * torch.rand((), generator=g)).bfloat16()

    mat("embed", int(cfg["vocab"]), w, 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        norm(p + "norm1")
        m = layer["mixer"]
        if layer["type"] == "retention":
            H, d, vd = m["heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", H * d, w)
            mat(p + "mix.k", H * d, w)
            mat(p + "mix.v", H * vd, w)
            mat(p + "mix.g", H * vd, w)
            mat(p + "mix.o", w, H * vd)
        else:
            a, r = m["left"], m["right"]
            H, G, d, vd = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for nm, rows in (("q", H * d), ("k", G * d), ("v", G * vd)):
                mat(p + f"mix.left.{nm}", rows, w)
                vec(p + f"mix.left.{nm}.b", rows, 0.0, 0.3)
                mat(p + f"mix.left.{nm}.conv", rows, a["conv"], 0.6)
            out[p + "mix.left.talk"] = (torch.eye(H) * 0.7 + 0.3 * torch.randn(H, H, generator=g)).bfloat16()
            vec(p + "mix.left.sink", H, 0.0, 1.0)
            mat(p + "mix.left.o", w, H * vd)
            RH, rd, rvd = r["heads"], r["dim"], r["vdim"]
            mat(p + "mix.right.q", RH * rd, w)
            mat(p + "mix.right.f", RH * rd, w)
            vec(p + "mix.right.f.b", RH * rd, 1.0, 1.0)
            out[p + "mix.right.lower"] = (0.9 * torch.rand(RH * rd, generator=g)).bfloat16()
            mat(p + "mix.right.v", RH * rvd, w)
            vec(p + "mix.right.norm", rvd, 1.0, 0.2)
            mat(p + "mix.right.o", w, RH * rvd)
        if layer.get("mlp") is not None:
            norm(p + "norm2")
            ff = layer["mlp"]["ff"]
            mat(p + "mlp.up", ff, w)
            mat(p + "mlp.down", w, ff)
            vec(p + "mlp.act", 2, 0.0, 0.5)
    norm("final.norm")
    return out


def write_checkpoint(path, cfg: dict, weights: dict) -> Path:
    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous().clone() for k, v in weights.items()}, str(path / "model.safetensors"))
    return path


def greedy(cfg: dict, weights: dict, prompt: list[int], n_new: int) -> list[int]:
    toks = list(prompt)
    for _ in range(n_new):
        logits, _ = forward(cfg, weights, toks)
        toks.append(int(logits[-1].argmax()))
    return toks[len(prompt):]


def row_errors(got, want):
    """Per row: rms of the difference (means taken off) over the rms of the wanted row (mean taken off)."""
    g, w = got.double(), want.double()
    d = (g - w) - (g - w).mean(-1, keepdim=True)
    ref = w - w.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def check_rows(got, want, tol, what=""):
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    err = row_errors(got, want)
    bad = int(err.argmax())
    assert err.max().item() < tol, f"{what}: row {bad} is off by {err.max().item():.3g} (allowed {tol})"
