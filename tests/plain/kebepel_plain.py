"""A plain, slow Kebepel forward pass: whole sequences, no cache, one function per mechanism.

Kebepel is a decoder-only design whose layers carry one of two mixers between four layer norms (one before and one
after each sublayer): a differential attention (two softmax maps over shared values whose difference is normed per
head; a query temperature that grows with the logarithm of the position; no rotation), or two mixers side by side on
the same input, a grouped-query attention (whole-projection q/k norm, interleaved rotary pairs with YaRN, tanh-capped
scores) beside a gated delta rule (short causal convolutions, unit-norm q and k, a decayed fast-weight matrix per
head), their outputs added with fixed scales. A run of layers may be repeated with the same weights, with a learned
vector added to the stream before each pass. This file shares no code with the engine. Everything is torch on the
CPU in the dtype of its inputs (tests use float64). The config is the raw config.json dict, read here independently
of the engine's parser.

Notation: h is a sublayer's input [T, width]; W are stored [out, in] and applied as W h.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    y = torch.einsum("tc,rc->tr", x, w)
    return y if b is None else y + b


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(mean of squared deviations + eps) * w + b over the last axis."""
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


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


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, heads, n]: of every head's first rot.dims entries, entry 2i is paired with entry 2i + 1:
    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * f_i; the rest passes unchanged."""
    dims = int(rot["dims"])
    f, amp = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    cos = (torch.cos(ang) * amp).to(x.dtype)[:, None, :]
    sin = (torch.sin(ang) * amp).to(x.dtype)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ----------------------------------------------------------------------------------------------- attention


def causal_softmax_attention(q, k, v, scale: float, softcap: float = 0.0):
    """q [T, H, d], k [T, H, d], v [T, H, dv] (keys and values already given per query head): every position sees
    itself and all earlier ones; scores (q . k) * scale, then cap * tanh(score / cap) when a cap is given."""
    T = q.shape[0]
    s = torch.einsum("thd,jhd->htj", q, k) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    s = s.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("htj,jhd->thd", p, v)


def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1) per position."""
    return 1.0 + coef * torch.log(torch.floor((positions.to(torch.float64) + 1.0) / every) + 1.0)


def differential_attention(h, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, positions):
    """The mixer 'attention'. Each head has two query maps and each key head two key maps, laid out head by head as
    [map 1 | map 2]; both maps attend over the same values; o = a1 - lambda a2 with one lambda for the layer, then
    o / sqrt(mean(o^2) + eps) per head times (1 - diff); the heads are gated by sigmoid(W_g h) and go through W_o."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = linear(h, w[p + ".q"], w[p + ".q.b"]).view(T, H, 2, d)
    k = linear(h, w[p + ".k"], w[p + ".k.b"]).view(T, G, 2, d)
    v = linear(h, w[p + ".v"], w[p + ".v.b"]).view(T, G, dv)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(positions, float(qt["coef"]), int(qt["every"])).to(q.dtype)[:, None, None, None]
    rep = H // G
    kh = k.repeat_interleave(rep, dim=1)  # query head i uses key/value head floor(i / (H / G))
    vh = v.repeat_interleave(rep, dim=1)
    a1 = causal_softmax_attention(q[:, :, 0], kh[:, :, 0], vh, float(m["scale"]))
    a2 = causal_softmax_attention(q[:, :, 1], kh[:, :, 1], vh, float(m["scale"]))
    diff = float(m["diff"])
    lam = torch.exp((w[p + ".lq1"] * w[p + ".lk1"]).sum()) - torch.exp((w[p + ".lq2"] * w[p + ".lk2"]).sum()) + diff
    o = rms(a1 - lam * a2, eps) * (1.0 - diff)
    o = o.reshape(T, H * dv) * torch.sigmoid(linear(h, w[p + ".g"]))
    return linear(o, w[p + ".o"])


def capped_attention(h, w, p: str, m: dict, eps: float, positions):
    """The left mixer of 'parallel': biased projections, an RMS norm with weights over the whole q projection (and
    the whole k projection) before the heads are split, rotary pairs, capped scores, an output gate."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms(linear(h, w[p + ".q"], w[p + ".q.b"]), eps) * w[p + ".q.norm"]
    k = rms(linear(h, w[p + ".k"], w[p + ".k.b"]), eps) * w[p + ".k.norm"]
    v = linear(h, w[p + ".v"], w[p + ".v.b"]).view(T, G, dv)
    q, k = q.view(T, H, d), k.view(T, G, d)
    if m.get("rot"):
        q, k = rotate_pairs(q, positions, m["rot"]), rotate_pairs(k, positions, m["rot"])
    rep = H // G
    a = causal_softmax_attention(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1), float(m["scale"]),
                                 float(m.get("softcap") or 0.0))
    o = a.reshape(T, H * dv) * torch.sigmoid(linear(h, w[p + ".g"]))
    return linear(o, w[p + ".o"])


# ----------------------------------------------------------------------------------------------- gated delta rule


def short_convolution(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, K - 1 - j] x[t - j, c], zeros before the start (the last column
    multiplies the current token)."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for j in range(min(K, T)):
        y[j:] += x[:T - j] * taps[:, K - 1 - j]
    return y


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, g):
    """q, k [T, H, d], v [T, H, dv], beta and g [T, H]. Per head, token by token: S <- g S; u = beta (v - S^T k);
    S <- S + k u^T; o = S^T q (the read-out sees the token's own write). S starts at zero."""
    T, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=q.dtype)
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        S = S * g[t][:, None, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hij,hi->hj", S, k[t]))
        S = S + torch.einsum("hi,hj->hij", k[t], u)
        out[t] = torch.einsum("hij,hi->hj", S, q[t])
    return out


def gated_delta_mixer(h, w, p: str, m: dict, eps: float):
    """The right mixer of 'parallel'."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(short_convolution(linear(h, w[p + ".q"]), w[p + ".q.conv"])).view(T, G, d)
    k = silu(short_convolution(linear(h, w[p + ".k"]), w[p + ".k.conv"])).view(T, G, d)
    v = silu(short_convolution(linear(h, w[p + ".v"]), w[p + ".v.conv"])).view(T, H, dv)
    rep = H // G
    q = (unit(q) * d ** -0.5).repeat_interleave(rep, dim=1)
    k = unit(k).repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(linear(h, w[p + ".b"]))
    g = torch.exp(-torch.exp(w[p + ".A_log"]) * softplus(linear(h, w[p + ".a"]) + w[p + ".dt_bias"]))
    o = delta_rule(q, k, v, beta, g)
    o = rms(o, eps) * w[p + ".norm"]
    o = o.reshape(T, H * dv) * silu(linear(h, w[p + ".g"]))
    return linear(o, w[p + ".o"])


# ----------------------------------------------------------------------------------------------- layers, model


def mixer(h, w, layer: int, spec: dict, eps: float, positions):
    p, m = f"l{layer}.mix", spec["mixer"]
    if spec["type"] == "attention":
        return differential_attention(h, w, p, m, eps, positions)
    if spec["type"] == "parallel":
        left = capped_attention(h, w, p + ".left", m["left"], eps, positions)
        right = gated_delta_mixer(h, w, p + ".right", m["right"], eps)
        return float(m["left_scale"]) * left + float(m["right_scale"]) * right
    raise ValueError(f"unknown mixer {spec['type']}")


def feed_forward(h, w, layer: int, mlp: dict):
    p = f"l{layer}.mlp"
    if mlp["kind"] != "dense":
        raise ValueError(f"unknown feed-forward {mlp['kind']}")
    return linear(silu(linear(h, w[p + ".gate"])) * linear(h, w[p + ".up"]), w[p + ".down"])


def run_layer(x, w, i: int, spec: dict, eps: float, positions):
    def ln(name, t):
        return layer_norm(t, w[f"l{i}.{name}"], w[f"l{i}.{name}.b"], eps)
    x = x + ln("norm1b", mixer(ln("norm1", x), w, i, spec, eps, positions))
    if spec.get("mlp") is not None:
        x = x + ln("norm2b", feed_forward(ln("norm2", x), w, i, spec["mlp"]))
    return x


def layer_runs(cfg: dict) -> List[tuple]:
    """(layer, pass or None) in the order the layers run: layers start .. stop - 1 run `times` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return ([(i, None) for i in range(a)] + [(i, t) for t in range(times) for i in range(a, b)]
            + [(i, None) for i in range(b, n)])


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens, streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0. ``streams``: a list that gets the residual stream after
    every layer run."""
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(ids))
    x = w["embed"][ids]
    loop = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if t is not None and i == int(loop["start"]):  # once in a pass, right before its first layer
            x = x + w["loop.step"][t]
        x = run_layer(x, w, i, cfg["layers"][i], eps, positions)
        if streams is not None:
            streams.append(x)
    return linear(layer_norm(x, w["final.norm"], w["final.norm.b"], eps), w["head"])


def greedy(cfg, w, prompt, n_new: int) -> List[int]:
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        t = int(torch.argmax(forward(cfg, w, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out
