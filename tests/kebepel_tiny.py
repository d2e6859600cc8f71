"""Tiny Kebepel configurations for the tests, their weights, and helpers shared by the tests.

KA varies what a layer can vary: a loop over two middle layers, a layer without a feed-forward, a differential
attention whose query temperature steps every 5 positions, a rotation over half of a head with YaRN beside one over
the whole head without, a capped and an uncapped left attention, a delta rule with fewer key heads than value heads.
KB has sizes in multiples of 16 / 32 / 64 and a loop from the first layer. KC has odd sizes everywhere, no loop, one
kv head, convolutions of 2 and 5 taps, a differential attention without a query temperature.
"""
import json
import os
import random

import torch


def _yarn(factor, original, fast=32.0, slow=1.0):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def _left(heads, kv, dim, vdim, softcap=None, rot_dims=None, base=10000.0, scaling=None, scale=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5 * 1.5}
    if softcap:
        m["softcap"] = softcap
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            m["rot"]["scaling"] = scaling
    return m


def _right(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def _parallel(left, right, ls, rs, ff):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _attention(heads, kv, dim, vdim, diff, q_temp, ff):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 * 1.3, "diff": diff}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


K_A = {
    "architecture": "Kebepel", "vocab": 160, "width": 96, "norm": {"eps": 1e-5},
    "layers": [
        _attention(4, 2, 12, 20, 0.25, (0.7, 5), 72),
        _parallel(_left(4, 2, 16, 24, softcap=3.0, rot_dims=8, scaling=_yarn(2.0, 16)), _right(4, 2, 12, 8, 3), 0.6, 1.3, 64),
        _attention(2, 2, 8, 16, 0.4, (0.3, 7), None),
        _parallel(_left(2, 1, 24, 8, rot_dims=24, base=300.0), _right(3, 3, 8, 16, 4), 1.1, 0.7, None),
        _parallel(_left(6, 3, 8, 8, softcap=1.5), _right(2, 1, 16, 16, 2), 0.5, 0.5, 48),
    ],
    "loop": {"start": 1, "stop": 3, "times": 2},
}

K_B = {
    "architecture": "Kebepel", "vocab": 300, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        _parallel(_left(8, 2, 64, 48, softcap=20.0, rot_dims=32, base=50000.0, scaling=_yarn(4.0, 32)), _right(4, 4, 64, 32, 4), 0.7, 0.6, 256),
        _attention(6, 3, 32, 64, 0.35, (0.4, 16), 256),
        _parallel(_left(4, 4, 32, 64, rot_dims=32), _right(4, 2, 32, 64, 4), 1.0, 1.0, 128),
    ],
    "loop": {"start": 0, "stop": 2, "times": 2},
}

K_C = {
    "architecture": "Kebepel", "vocab": 97, "width": 70, "norm": {"eps": 1e-6},
    "layers": [
        _parallel(_left(3, 1, 10, 7, softcap=2.0, rot_dims=6, scaling=_yarn(1.5, 8, fast=8.0, slow=2.0)), _right(3, 1, 10, 7, 2), 0.9, 0.4, 50),
        _attention(3, 1, 6, 9, 0.15, None, 30),
        _parallel(_left(1, 1, 14, 5, rot_dims=14, base=77.0), _right(5, 5, 6, 9, 5), 0.3, 1.7, None),
    ],
}

# name -> (config, weight seed, page size)
CONFIGS = {"KA": (K_A, 21, 8), "KB": (K_B, 22, 16), "KC": (K_C, 23, 4)}


def write_model(folder, cfg, seed, std=0.09):
    """A model folder with random weights wide enough that every mechanism moves the logits: matrices N(0, std), gains
    1 + N(0, 0.1), biases N(0, 0.3); convolution taps N(0, 0.5); the vectors behind lambda N(0, 0.2) (lambda then
    differs visibly from its constant but stays away from 1, where the two maps of near-uniform attention would cancel
    and the heads' norm would blow rounding up); A_log N(0, 0.7) and dt_bias N(-1, 1) (decays between nearly none and strong);
    the loop's vectors N(0, 0.5)."""
    from jllm_serve_amd.weights.random_init import random_source
    from jllm_serve_amd.weights.safetensors_io import write_safetensors
    src = random_source(cfg, seed, std=std)
    tensors = {n: src.get(n) for n in src.names()}
    g = torch.Generator().manual_seed(seed + 77)

    def normal(shape, mean, sd):
        return (torch.randn(shape, generator=g) * sd + mean).to(torch.bfloat16)

    for n, t in tensors.items():
        last = n.rsplit(".", 1)[-1]
        if n.endswith(".conv"):
            tensors[n] = normal(t.shape, 0.0, 0.5)
        elif last in ("lq1", "lq2", "lk1", "lk2"):
            tensors[n] = normal(t.shape, 0.0, 0.2)
        elif last == "A_log":
            tensors[n] = normal(t.shape, 0.0, 0.7)
        elif last == "dt_bias":
            tensors[n] = normal(t.shape, -1.0, 1.0)
        elif n == "loop.step":
            tensors[n] = normal(t.shape, 0.0, 0.5)
        elif n.endswith(".b") and t.dim() == 1:
            tensors[n] = normal(t.shape, 0.0, 0.3)
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
    """Against float64, for one row. In bfloat16 these models have a heavy tail: a head of a differential attention,
    and a head of the delta rule, is divided by its root mean square, which blows the products' rounding up wherever
    the head's output nearly cancels (measured on 131 positions: median 0.5 to 2 % of the largest logit, one position
    at 11 %), and heads of 6 to 12 entries average little away. So a single row gets a wide bound, which a wrong key,
    page or state still breaks (they move logits by their own size), ``typical`` bounds the median over many rows,
    and the float32 run, which takes the same path through cache, state and batching, is held tightly."""
    m = float(ref.abs().max())
    return 5e-5 * m + 1e-6 if dtype == "float32" else 0.2 * m


def typical(dtype):
    """What the median over many rows of |difference| / largest |logit| may be."""
    return 5e-6 if dtype == "float32" else 2.5e-2
