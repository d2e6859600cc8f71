"""The Kebepel design: config.json keys -> ModelConfig.

A Kebepel config names its design with ``"architecture": "Kebepel"`` and lists its layers one by one:

* ``vocab``, ``width``, ``norm.eps`` (of every layer norm and of the RMS norms inside the mixers);
* ``layers[i]``: ``type`` (the mixer: ``attention`` or ``parallel``), ``mixer`` (its sizes and constants) and ``mlp``
  (``{"kind": "dense", "ff": n}``, a SiLU-gated feed-forward, or null for none); layer i's tensors start with ``l<i>.``,
  its mixer's with ``l<i>.mix.``; a layer has a layer norm (weight and bias ``<name>.b``) in front of and behind each
  sublayer: ``norm1`` / ``norm1b`` around the mixer, ``norm2`` / ``norm2b`` around the feed-forward;
* ``attention`` (differential attention): ``heads``, ``kv_heads``, ``dim`` (per map), ``vdim``, ``scale``, ``diff``
  (the constant in lambda and in the factor 1 - diff behind the heads' norm) and optionally ``q_temp`` (``coef``,
  ``every``: the query scale that grows with the logarithm of the position); no rotation;
* ``parallel``: ``left`` (an attention with ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, optional ``softcap``
  and optional ``rot``: ``base``, ``dims``, optional ``scaling`` with ``factor``, ``original``, ``fast``, ``slow``: YaRN
  on neighbouring pairs), ``right`` (a gated delta rule with ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``: the
  taps of its convolutions), ``left_scale`` and ``right_scale`` (the weights of the two outputs in their sum);
* ``loop`` (optional): layers ``start`` .. ``stop`` - 1 run ``times`` times in a row with one set of weights and a
  cache or state per pass; row t of the tensor ``loop.step`` [times, width] joins the stream before pass t.

YaRN here: the frequencies blend between f_i and f_i / factor over the pairs between the ``fast`` and ``slow`` rotation
counts of the ``original`` length, and cos and sin are multiplied by 0.1 ln(factor) + 1; the attention scale is used
as given. That is the engine's yarn table with the amplitude given explicitly.
"""
from __future__ import annotations

import math
from typing import Any, List, Mapping, Optional

from .registry import register_architecture
from .schema import (ConfigError, GatedDeltaSpec, GatedMlpNames, GatedMlpSpec, LayerNormSpec, LayerSpec, ModelConfig,
                     ModelNames, ParallelMixerSpec, RopeScaling, RopeSpec, ScheduleEntry, StreamVector, WideAttentionSpec)


def _need(m: Any, key: str, where: str):
    if not isinstance(m, Mapping) or key not in m or m[key] is None:
        raise ConfigError(f"config.json: {where} needs '{key}'")
    return m[key]


def _int(m: Any, key: str, where: str, least: int = 1) -> int:
    v = _need(m, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or v != int(v) or int(v) < least:
        raise ConfigError(f"config.json: {where}.{key} must be an integer of at least {least}, got {v!r}")
    return int(v)


def _number(m: Any, key: str, where: str) -> float:
    v = _need(m, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}.{key} must be a number, got {v!r}")
    return float(v)


def _heads(m: Any, where: str):
    heads, kv_heads = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv_heads:
        raise ConfigError(f"config.json: {where}: {kv_heads} kv_heads do not divide {heads} heads")
    return heads, kv_heads, _int(m, "dim", where), _int(m, "vdim", where)


def _rope(rot: Mapping[str, Any], dim: int, where: str) -> RopeSpec:
    dims = _int(rot, "dims", where, least=2)
    if dims % 2 or dims > dim:
        raise ConfigError(f"config.json: {where}.dims={dims} must be even and at most dim={dim}")
    base = _number(rot, "base", where)
    sc = rot.get("scaling")
    scaling = RopeScaling()
    if sc is not None:
        w = where + ".scaling"
        factor, fast, slow = _number(sc, "factor", w), _number(sc, "fast", w), _number(sc, "slow", w)
        if not factor > 0 or not fast > 0 or not slow > 0:
            raise ConfigError(f"config.json: {w}: factor, fast and slow must be positive")
        amp = 0.1 * math.log(factor) + 1.0
        if not amp > 0:
            raise ConfigError(f"config.json: {w}.factor={factor} gives the amplitude {amp}")
        scaling = RopeScaling(kind="yarn", factor=factor, original_max_positions=_int(sc, "original", w), beta_fast=fast,
                              beta_slow=slow, attention_factor=amp, truncate=True)
    return RopeSpec(rotary_dim=dims, theta=base, scaling=scaling, pairing="interleaved")


def _position(rot, dim: int, where: str, positions: List[RopeSpec]) -> Optional[int]:
    if rot is None:
        return None
    rope = _rope(rot, dim, where)
    if rope not in positions:
        positions.append(rope)
    return positions.index(rope)


def _differential(m: Any, w: str, eps: float) -> WideAttentionSpec:
    heads, kv_heads, dim, vdim = _heads(m, w)
    diff = _number(m, "diff", w)
    qt = m.get("q_temp")
    coef, every = (_number(qt, "coef", w + ".q_temp"), _int(qt, "every", w + ".q_temp")) if qt is not None else (0.0, 0)
    return WideAttentionSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=_number(m, "scale", w), eps=eps,
                             maps=2, diff=diff, q_temp_coef=coef, q_temp_every=every, bias=True, out_gate=True)


def _left(m: Any, w: str, eps: float, positions: List[RopeSpec]) -> WideAttentionSpec:
    heads, kv_heads, dim, vdim = _heads(m, w)
    cap = m.get("softcap")
    softcap = _number(m, "softcap", w) if cap is not None else 0.0
    if softcap < 0:
        raise ConfigError(f"config.json: {w}.softcap={softcap} must be positive")
    return WideAttentionSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=_number(m, "scale", w), eps=eps,
                             maps=1, qk_norm="whole", position=_position(m.get("rot"), dim, w + ".rot", positions),
                             softcap=softcap, bias=True, out_gate=True)


def _right(m: Any, w: str, eps: float) -> GatedDeltaSpec:
    heads, kv_heads, dim, vdim = _heads(m, w)
    return GatedDeltaSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=_int(m, "conv", w), eps=eps)


def parse_kebepel(c: Mapping[str, Any], model_type: str, architecture: str) -> ModelConfig:
    vocab = _int(c, "vocab", "config")
    width = _int(c, "width", "config")
    eps = _number(_need(c, "norm", "config"), "eps", "norm")
    raw_layers = _need(c, "layers", "config")
    if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
        raise ConfigError("config.json: layers must be a non-empty list")
    norm = LayerNormSpec(eps=eps)
    positions: List[RopeSpec] = []
    layers = []
    for i, layer in enumerate(raw_layers):
        where = f"layers[{i}]"
        kind = _need(layer, "type", where)
        m = _need(layer, "mixer", where)
        w = where + ".mixer"
        if kind == "attention":
            mixer = _differential(m, w, eps)
        elif kind == "parallel":
            mixer = ParallelMixerSpec(branches=(_left(_need(m, "left", w), w + ".left", eps, positions),
                                                _right(_need(m, "right", w), w + ".right", eps)),
                                      scales=(_number(m, "left_scale", w), _number(m, "right_scale", w)),
                                      prefixes=("left", "right"))
        else:
            raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design (attention, parallel)")
        mlp = layer.get("mlp")
        ffn = None
        if mlp is not None:
            if _need(mlp, "kind", where + ".mlp") != "dense":
                raise ConfigError(f"config.json: {where}.mlp.kind '{mlp['kind']}' is not a feed-forward of this design (dense)")
            ffn = GatedMlpSpec(hidden=_int(mlp, "ff", where + ".mlp"), activation="silu",
                               names=GatedMlpNames(gate="mlp.gate", up="mlp.up", down="mlp.down", ending=""))
        layers.append(LayerSpec(mixer=mixer, ffn=ffn, norm=norm, prefix=f"l{i}", arrangement="sandwich",
                                norm_in_name="norm1", norm_post_name="norm2", name_ending="",
                                norm_mixer_out_name="norm1b", norm_ffn_out_name="norm2b", mixer_prefix="mix"))
    n = len(layers)
    loop = c.get("loop")
    if loop is None:
        schedule = [ScheduleEntry(i) for i in range(n)]
        looped = ""
    else:
        start, stop, times = _int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0), _int(loop, "times", "loop", 0)
        if not start <= stop <= n:
            raise ConfigError(f"config.json: loop runs layers {start} .. {stop} - 1 of {n}")
        schedule = [ScheduleEntry(i) for i in range(start)]
        for t in range(times):
            for i in range(start, stop):
                schedule.append(ScheduleEntry(i, add_before=StreamVector("loop.step", times, t) if i == start else None))
        schedule += [ScheduleEntry(i) for i in range(stop, n)]
        looped = f" loop={start}..{stop - 1}x{times}"
    kinds = [l["type"] for l in raw_layers]
    description = (f"{architecture} width={width} layers={n} runs={len(schedule)} vocab={vocab} "
                   f"attention={kinds.count('attention')} parallel={kinds.count('parallel')}{looped}")
    longest = c.get("max_positions")
    return ModelConfig(
        architecture=architecture, model_type=model_type, hidden=width, vocab=vocab, final_norm=norm,
        layers=tuple(layers), positions=tuple(positions), schedule=tuple(schedule), tie_embeddings=False,
        max_positions=int(longest) if isinstance(longest, int) and longest > 0 else 4096,
        description=description, names=ModelNames(embed="embed", final_norm="final.norm", head="head"), raw=dict(c))


register_architecture("kebepel", "Kebepel", parse_kebepel, replace=True)
