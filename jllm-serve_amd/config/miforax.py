"""The Miforax design: config.json keys -> ModelConfig.

A Miforax config names its design with ``"architecture": "Miforax"`` and lists its layers one by one:

* ``vocab``, ``width``, ``norm.eps``, ``embedding.scale`` (the embedded rows are multiplied by it);
* ``layers[i]``: ``type`` (the mixer: ``latent_attention``), ``mixer`` (its sizes and constants) and ``mlp`` (the
  feed-forward, or null for none); layer i's tensors start with ``l<i>.``;
* a latent-attention mixer: ``heads``, ``dim`` / ``rot_dim`` (unrotated and rotated query/key entries per head),
  ``vdim``, ``q_rank``, ``kv_rank``, ``scale`` (used as given), ``mask.size`` (the sliding window; absent = every earlier
  key), ``rot`` (``base``, ``dims``, optional ``scaling`` with ``factor``, ``original``, ``fast``, ``slow``: YaRN) and
  optionally ``kv_from: j``: the layer reads layer j's cached latent and has no down-projection of its own;
* a feed-forward: ``kind`` ``dense`` (``ff``; gelu-tanh gate) or ``moe`` (``router.experts`` / ``router.top``,
  ``expert.ff`` / ``expert.limit``, optional ``shared.ff`` / ``shared.limit``; experts come from a table by token id; the
  slope 1.702 of the experts' sigmoid is the design's and lives in the kernels' gate function).

YaRN here: the frequencies blend between f_i and f_i / factor over the dimensions between the ``fast`` and ``slow``
rotation counts of the ``original`` length, and cos and sin are multiplied by 0.1 ln(factor) + 1 whatever the factor;
the attention scale is not touched. That is the engine's yarn table with the amplitude given explicitly.
"""
from __future__ import annotations

import math
from typing import Any, List, Mapping, Optional

from .registry import register_architecture
from .schema import (ConfigError, GatedMlpNames, GatedMlpSpec, LatentAttentionSpec, LayerSpec, ModelConfig, ModelNames,
                     NormSpec, RopeScaling, RopeSpec, ScheduleEntry, TableMoeSpec)

def _need(m: Any, key: str, where: str):
    if not isinstance(m, Mapping) or key not in m or m[key] is None:
        raise ConfigError(f"config.json: {where} needs '{key}'")
    return m[key]


def _positive_int(m: Any, key: str, where: str) -> int:
    v = _need(m, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or v != int(v) or int(v) <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return int(v)


def _number(m: Any, key: str, where: str) -> float:
    v = _need(m, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}.{key} must be a number, got {v!r}")
    return float(v)


def _rope(rot: Mapping[str, Any], rot_dim: int, where: str) -> RopeSpec:
    dims = _positive_int(rot, "dims", where + ".rot")
    if dims % 2 or dims > rot_dim:
        raise ConfigError(f"config.json: {where}.rot.dims={dims} must be even and at most rot_dim={rot_dim}")
    base = _number(rot, "base", where + ".rot")
    sc = rot.get("scaling")
    scaling = RopeScaling()
    if sc is not None:
        w = where + ".rot.scaling"
        factor = _number(sc, "factor", w)
        fast, slow = _number(sc, "fast", w), _number(sc, "slow", w)
        if not factor > 0 or not fast > 0 or not slow > 0:
            raise ConfigError(f"config.json: {w}: factor, fast and slow must be positive")
        scaling = RopeScaling(kind="yarn", factor=factor, original_max_positions=_positive_int(sc, "original", w),
                              beta_fast=fast, beta_slow=slow, attention_factor=0.1 * math.log(factor) + 1.0,
                              truncate=True)
    return RopeSpec(rotary_dim=dims, theta=base, scaling=scaling, pairing="half")


def parse_miforax(c: Mapping[str, Any], model_type: str, architecture: str) -> ModelConfig:
    vocab = _positive_int(c, "vocab", "config")
    width = _positive_int(c, "width", "config")
    eps = _number(_need(c, "norm", "config"), "eps", "norm")
    emb = c.get("embedding")
    embed_scale = _number(emb, "scale", "embedding") if isinstance(emb, Mapping) and "scale" in emb else 1.0
    raw_layers = _need(c, "layers", "config")
    if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
        raise ConfigError("config.json: layers must be a non-empty list")
    norm = NormSpec(eps=eps)
    positions: List[RopeSpec] = []
    mixers: List[dict] = []
    for i, layer in enumerate(raw_layers):
        where = f"layers[{i}]"
        kind = _need(layer, "type", where)
        if kind != "latent_attention":
            raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design (latent_attention is)")
        m = _need(layer, "mixer", where)
        w = where + ".mixer"
        rot_dim = _positive_int(m, "rot_dim", w)
        rope = _rope(_need(m, "rot", w), rot_dim, w)
        if rope not in positions:
            positions.append(rope)
        mask = m.get("mask")
        window = _positive_int(mask, "size", w + ".mask") if isinstance(mask, Mapping) else 0
        src = m.get("kv_from")
        if src is not None:
            if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < i:
                raise ConfigError(f"config.json: {w}.kv_from={src!r} must name an earlier layer")
            o = mixers[src]
            if o["kv_from"] is not None:
                raise ConfigError(f"config.json: {w}.kv_from={src}: that layer has no cache of its own")
            if (o["kv_rank"], o["rot_dim"], o["rope"]) != (_positive_int(m, "kv_rank", w), rot_dim, rope):
                raise ConfigError(f"config.json: {w}.kv_from={src}: latent size, rotated size and rotation must equal that layer's")
        mixers.append(dict(heads=_positive_int(m, "heads", w), dim=_positive_int(m, "dim", w), rot_dim=rot_dim,
                           vdim=_positive_int(m, "vdim", w), q_rank=_positive_int(m, "q_rank", w),
                           kv_rank=_positive_int(m, "kv_rank", w), scale=_number(m, "scale", w), window=window,
                           rope=rope, kv_from=src))
    # a cache keeps what the widest window among its readers can still see
    keep = [m["window"] for m in mixers]
    for i, m in enumerate(mixers):
        if m["kv_from"] is not None:
            j = m["kv_from"]
            keep[j] = 0 if (keep[j] == 0 or m["window"] == 0) else max(keep[j], m["window"])
    layers = []
    schedule = []
    for i, (layer, m) in enumerate(zip(raw_layers, mixers)):
        where = f"layers[{i}]"
        mixer = LatentAttentionSpec(heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"],
                                    q_rank=m["q_rank"], kv_rank=m["kv_rank"], scale=m["scale"], eps=eps,
                                    window=m["window"], keep=keep[i] if m["kv_from"] is None else keep[m["kv_from"]],
                                    position=positions.index(m["rope"]), sink=True, out_gate=True,
                                    owns_cache=m["kv_from"] is None)
        mlp = layer.get("mlp")
        ffn: Optional[Any] = None
        if mlp is not None:
            w = where + ".mlp"
            kind = _need(mlp, "kind", w)
            if kind == "dense":
                ffn = GatedMlpSpec(hidden=_positive_int(mlp, "ff", w), activation="gelu_tanh",
                                   names=GatedMlpNames(gate="mlp.gate", up="mlp.up", down="mlp.down", ending=""))
            elif kind == "moe":
                router, expert = _need(mlp, "router", w), _need(mlp, "expert", w)
                experts, top = _positive_int(router, "experts", w + ".router"), _positive_int(router, "top", w + ".router")
                if top > experts:
                    raise ConfigError(f"config.json: {w}.router: top={top} of {experts} experts")
                shared = mlp.get("shared")
                shared_spec = None
                if shared is not None:
                    shared_spec = GatedMlpSpec(hidden=_positive_int(shared, "ff", w + ".shared"), activation="swish_clamped",
                                               limit=_number(shared, "limit", w + ".shared"),
                                               names=GatedMlpNames(gate="mlp.shared.gate", up="mlp.shared.up",
                                                                   down="mlp.shared.down", ending=""))
                ffn = TableMoeSpec(experts=experts, top=top, hidden=_positive_int(expert, "ff", w + ".expert"),
                                   limit=_number(expert, "limit", w + ".expert"), vocab=vocab, shared=shared_spec)
            else:
                raise ConfigError(f"config.json: {w}.kind '{kind}' is not a feed-forward of this design (dense, moe)")
        layers.append(LayerSpec(mixer=mixer, ffn=ffn, norm=norm, prefix=f"l{i}", norm_in_name="norm1",
                                norm_post_name="norm2", name_ending=""))
        schedule.append(ScheduleEntry(i, cache_from=m["kv_from"]))
    n_moe = sum(1 for l in layers if isinstance(l.ffn, TableMoeSpec))
    description = (f"{architecture} width={width} layers={len(layers)} vocab={vocab} latent-attention "
                   f"moe-layers={n_moe} borrowed-caches={sum(1 for m in mixers if m['kv_from'] is not None)}")
    longest = c.get("max_positions")
    return ModelConfig(
        architecture=architecture, model_type=model_type, hidden=width, vocab=vocab, final_norm=norm,
        layers=tuple(layers), positions=tuple(positions), schedule=tuple(schedule), tie_embeddings=False,
        max_positions=int(longest) if isinstance(longest, int) and longest > 0 else 4096, embed_scale=embed_scale,
        description=description, names=ModelNames(embed="embed", final_norm="final.norm", head="head"), raw=dict(c))


register_architecture("miforax", "Miforax", parse_miforax, replace=True)
