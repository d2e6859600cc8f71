"""Tiny Miforax configurations for the tests, their weights, and helpers shared by the tests.

MF_A varies everything a layer can vary: a layer that borrows an earlier layer's cache and looks further back than
that layer does, a layer without a window, a rotated key part only half of which is rotated, a layer without a
feed-forward, experts with top = 2 and a shared expert, experts with top = 1 and none, rotation with and without YaRN.
MF_B has sizes the matrix-core kernels take (multiples of 16 / 32 / 128), so its bfloat16 run goes through them. MF_C
has odd sizes everywhere (one head, a value size of 5, an embedding scale of 1, a layer that borrows a cache and has no
window, so that its owner, which has one, must keep every page).
"""
import json
import os
import random

import torch


def _yarn(factor, original, fast=32.0, slow=1.0):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def _mixer(heads, dim, rot_dim, vdim, q_rank, kv_rank, window=None, rot_dims=None, base=10000.0, scaling=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": (dim + rot_dim) ** -0.5 * 1.25, "rot": {"base": base, "dims": rot_dims or rot_dim}}
    if scaling:
        m["rot"]["scaling"] = scaling
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(experts, top, ff, limit, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


MF_A = {
    "architecture": "Miforax", "vocab": 160, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.5},
    "layers": [
        _layer(_mixer(2, 16, 8, 24, 40, 32, window=11, scaling=_yarn(2.0, 16)), {"kind": "dense", "ff": 72}),
        _layer(_mixer(2, 16, 8, 24, 40, 32, window=19, scaling=_yarn(2.0, 16), kv_from=0), _moe(5, 2, 24, 1.5, shared=(40, 0.75))),
        _layer(_mixer(3, 8, 16, 16, 24, 48, rot_dims=8, base=500.0), None),
        _layer(_mixer(2, 24, 8, 8, 16, 16, window=5, base=500.0), _moe(3, 1, 32, 0.9)),
    ],
}

MF_B = {
    "architecture": "Miforax", "vocab": 300, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 2.0},
    "layers": [
        _layer(_mixer(8, 32, 32, 32, 128, 64, window=40, scaling=_yarn(4.0, 32)), {"kind": "dense", "ff": 256}),
        _layer(_mixer(8, 32, 32, 32, 128, 64, window=40, scaling=_yarn(4.0, 32), kv_from=0), _moe(8, 2, 64, 2.5, shared=(128, 1.5))),
        _layer(_mixer(16, 16, 16, 16, 128, 96), _moe(6, 1, 128, 3.0)),
    ],
}

# sizes that are multiples of nothing: every product and attention falls to the general kernels in bfloat16 too
MF_C = {
    "architecture": "Miforax", "vocab": 97, "width": 70, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
    "layers": [
        _layer(_mixer(3, 10, 6, 7, 18, 20, window=9, rot_dims=4, scaling=_yarn(1.5, 8, fast=8.0, slow=2.0)), _moe(4, 3, 12, 1.0, shared=(22, 2.0))),
        _layer(_mixer(1, 12, 2, 5, 9, 11, base=77.0), {"kind": "dense", "ff": 50}),
        _layer(_mixer(5, 6, 6, 9, 18, 20, rot_dims=4, scaling=_yarn(1.5, 8, fast=8.0, slow=2.0), kv_from=0), _moe(2, 2, 30, 0.5)),
    ],
}

# name -> (config, weight seed, page size)
CONFIGS = {"MA": (MF_A, 11, 8), "MB": (MF_B, 12, 16), "MC": (MF_C, 13, 4)}


def write_model(folder, cfg, seed, std=0.09, sink_std=1.5):
    """A model folder with random weights wide enough that every mechanism moves the logits: matrices N(0, std), gains
    1 + N(0, 0.1), sinks N(0.5, sink_std) (a sink near the scores' size takes a visible share of the softmax)."""
    from jllm_serve_amd.weights.random_init import random_source
    from jllm_serve_amd.weights.safetensors_io import write_safetensors
    src = random_source(cfg, seed, std=std)
    tensors = {n: src.get(n) for n in src.names()}
    g = torch.Generator().manual_seed(seed + 77)
    for n in tensors:
        if n.endswith(".sink"):
            tensors[n] = (torch.randn(tensors[n].shape, generator=g) * sink_std + 0.5).to(torch.bfloat16)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def load_weights(folder):
    """The folder's tensors through the safetensors package (not the engine's reader): floats as float64."""
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            t = f.get_tensor(k)
            out[k] = t.to(torch.float64) if t.is_floating_point() else t
    return out


def prompt(name, length, seed=0):
    rng = random.Random(f"{name}/{length}/{seed}")
    v = CONFIGS[name][0]["vocab"]
    return [rng.randrange(v) for _ in range(length)]


def tolerance(dtype, ref):
    m = float(ref.abs().max())
    return 2e-5 * m + 1e-6 if dtype == "float32" else 2.5e-2 * m
