"""A plain, slow Miforax forward pass: whole sequences, no cache, one function per mechanism.

Miforax is a decoder-only design with latent attention (queries, keys and values all pass through low-rank
latents; one rotated key part is shared by the heads; a sliding window; a learned per-head sink in the softmax's
denominator; an output gate), layers that may borrow an earlier layer's latent cache, and feed-forwards that are
dense (gelu-tanh gated) or a mixture of clamped-swish experts chosen by a table from the token id, with an optional
shared expert. This file shares no code with the engine. Everything is torch on the CPU in the dtype of its inputs
(tests use float64). The config is the raw config.json dict, read here independently of the engine's parser.

Notation: h is a mixer's or feed-forward's input [T, width]; W are stored [out, in] and applied as W h.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rmsnorm(x: torch.Tensor, g: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) (* g) over the last dim; eps inside the root."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if g is None else y * g


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    return torch.einsum("tc,rc->tr", x, w)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ----------------------------------------------------------------------------------------------- rotation


def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """(f[dims/2], amplitude). Plain: f_i = base^(-2i/dims), amplitude 1. With scaling {factor, original, fast, slow}:
    d(t) = dims ln(original / (2 pi t)) / (2 ln base); lo = max(floor(d(fast)), 0); hi = min(ceil(d(slow)), dims - 1);
    r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1); f_i <- f_i / factor * r_i + f_i (1 - r_i); cos and sin are
    multiplied by 0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def d(t):
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(d(float(scaling["fast"]))), 0)
    hi = min(math.ceil(d(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, ..., n]: the first rot.dims of the last axis are rotated, dimension i paired with i + dims/2:
    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * f_i; the rest passes unchanged."""
    dims = int(rot["dims"])
    f, amp = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = (torch.cos(ang) * amp).to(x.dtype), (torch.sin(ang) * amp).to(x.dtype)
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ----------------------------------------------------------------------------------------------- latent attention


def latent_kv(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, positions: torch.Tensor):
    """What a layer caches per position: the normed latent c [T, kv_rank] and the rotated shared key part [T, rot_dim]."""
    r = int(m["kv_rank"])
    d = linear(h, w[p + "dkv"])
    c = rmsnorm(d[:, :r], w[p + "dkv.norm"], eps)
    kr = rotate(d[:, r:], positions, m["rot"])
    return c, kr


def windowed_sink_softmax(scores: torch.Tensor, sink: Optional[torch.Tensor], window: int) -> torch.Tensor:
    """scores [H, T, T] (query i, key j). Key j is seen by query i when 0 <= i - j < window (window 0: every earlier
    key). The denominator also holds exp(sink_h), which has no value."""
    H, T, _ = scores.shape
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i) if window <= 0 else ((j <= i) & (i - j < window))
    s = scores.masked_fill(~seen, float("-inf"))
    if sink is None:
        return torch.softmax(s, dim=-1)
    both = torch.cat([s, sink.to(s.dtype)[:, None, None].expand(H, T, 1)], dim=-1)
    return torch.softmax(both, dim=-1)[..., :T]


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, positions: torch.Tensor,
                     c: torch.Tensor, kr: torch.Tensor) -> torch.Tensor:
    """The mixer's output for input h, given the (own or borrowed) latent c and rotated key part kr."""
    H, dn, dr, dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    T = h.shape[0]
    cq = rmsnorm(linear(h, w[p + "dq"]), w[p + "dq.norm"], eps)
    q = linear(cq, w[p + "uq"]).view(T, H, dn + dr)
    q_plain, q_rot = q[..., :dn], rotate(q[..., dn:], positions, m["rot"])
    k_plain = linear(c, w[p + "uk"]).view(T, H, dn)
    v = linear(c, w[p + "uv"]).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, kr)) * float(m["scale"])
    window = int((m.get("mask") or {}).get("size", 0))
    prob = windowed_sink_softmax(scores, w.get(p + "sink"), window)
    heads = torch.einsum("hij,jhd->ihd", prob, v).reshape(T, H * dv)
    gate = torch.sigmoid(linear(h, w[p + "g"]))
    return linear(heads * gate, w[p + "o"])


# ----------------------------------------------------------------------------------------------- feed-forwards


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return linear(gelu_tanh(linear(h, w[p + "gate"])) * linear(h, w[p + "up"]), w[p + "down"])


def clamped_expert(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, limit: float) -> torch.Tensor:
    """g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(linear(h, w[p + "gate"]), max=limit)
    u = torch.clamp(linear(h, w[p + "up"]), -limit, limit)
    return linear(g * torch.sigmoid(1.702 * g) * (u + 1.0), w[p + "down"])


def table_moe(h: torch.Tensor, tokens: List[int], w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    """Every token id has `top` experts in a table, each weighted 1/top; a shared expert, when there is one, is added."""
    top = int(mlp["router"]["top"])
    table = w[p + "table"].to(torch.long)
    out = torch.zeros_like(h)
    for t, tok in enumerate(tokens):
        for e in table[tok].tolist():
            out[t] += clamped_expert(h[t:t + 1], w, f"{p}e{e}.", float(mlp["expert"]["limit"]))[0] / top
    if mlp.get("shared"):
        out = out + clamped_expert(h, w, p + "shared.", float(mlp["shared"]["limit"]))
    return out


# ----------------------------------------------------------------------------------------------- model


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence. ``layers_out`` collects the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    ids = torch.tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x = w["embed"][ids] * float(cfg["embedding"]["scale"])
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "latent_attention":
            raise ValueError(f"layer {i}: unknown mixer {layer['type']}")
        m, p = layer["mixer"], f"l{i}.mix."
        h = rmsnorm(x, w[f"l{i}.norm1"], eps)
        if m.get("kv_from") is None:
            kept[i] = latent_kv(h, w, p, m, eps, positions)
            c, kr = kept[i]
        else:
            c, kr = kept[int(m["kv_from"])]
        x = x + latent_attention(h, w, p, m, eps, positions, c, kr)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rmsnorm(x, w[f"l{i}.norm2"], eps)
            if mlp["kind"] == "dense":
                x = x + dense_ff(h, w, f"l{i}.mlp.")
            elif mlp["kind"] == "moe":
                x = x + table_moe(h, tokens, w, f"l{i}.mlp.", mlp)
            else:
                raise ValueError(f"layer {i}: unknown feed-forward {mlp['kind']}")
        if layers_out is not None:
            layers_out.append(x.clone())
    return linear(rmsnorm(x, w["final.norm"], eps), w["head"])


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        nxt = int(torch.argmax(forward(cfg, w, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out
