"""Miforax without a GPU: the config parser, the rotation table against the plain formulas, invariants that pin the
plain implementation (which the GPU tests compare the engine with), the cache groups and windows the model asks for,
and the random-weights mode."""
import copy
import math

import numpy as np
import pytest
import torch

import miforax_tiny as mt
from plain import miforax_plain as P
from jllm_serve_amd.config import ConfigError, LatentAttentionSpec, TableMoeSpec, parse_config


def test_parser_reads_every_layer_and_keeps_the_widest_window_for_a_borrowed_cache():
    cfg = parse_config(mt.MF_A)
    assert cfg.architecture == "Miforax" and cfg.vocab == 160 and cfg.hidden == 96 and cfg.embed_scale == 3.5
    assert [e.cache_from for e in cfg.schedule] == [None, 0, None, None]
    m = [l.mixer for l in cfg.layers]
    assert all(isinstance(x, LatentAttentionSpec) for x in m)
    assert [x.window for x in m] == [11, 19, 0, 5]
    assert [x.keep for x in m] == [19, 19, 0, 5], "layer 0's pages must live as long as layer 1 looks back"
    assert [x.owns_cache for x in m] == [True, False, True, True]
    assert cfg.layers[2].ffn is None and isinstance(cfg.layers[1].ffn, TableMoeSpec)
    assert cfg.layers[1].ffn.top == 2 and cfg.layers[1].ffn.shared.limit == 0.75 and cfg.layers[3].ffn.shared is None
    assert cfg.layers[0].ffn.activation == "gelu_tanh"
    assert len(cfg.positions) == 2  # yarn over 8 dims; plain over 8 dims with another base (layers 2 and 3 share it)
    assert m[2].rot_dim == 16 and cfg.positions[m[2].position].rotary_dim == 8
    # a borrowed cache without a window keeps everything
    c = copy.deepcopy(mt.MF_A)
    del c["layers"][1]["mixer"]["mask"]
    assert [l.mixer.keep for l in parse_config(c).layers][:2] == [0, 0]


@pytest.mark.parametrize("edit, text", [
    (lambda c: c["layers"][1]["mixer"].update(kv_from=1), "earlier layer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "no cache of its own"),
    (lambda c: c["layers"][1]["mixer"].update(kv_rank=16), "must equal"),
    (lambda c: c["layers"][0].update(type="conv"), "not a mixer"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "not a feed-forward"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top=9"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c.pop("vocab"), "vocab"),
])
def test_parser_refuses(edit, text):
    c = copy.deepcopy(mt.MF_A)
    edit(c)
    with pytest.raises(ConfigError, match=text):
        parse_config(c)


@pytest.mark.parametrize("rot", [{"base": 1e4, "dims": 16}, {"base": 5e5, "dims": 32, "scaling": mt._yarn(4.0, 64)},
                                 {"base": 100.0, "dims": 8, "scaling": mt._yarn(0.5, 8, fast=4.0, slow=2.0)},
                                 {"base": 1e6, "dims": 64, "scaling": mt._yarn(8.0, 4096, fast=32.0, slow=1.0)},
                                 {"base": 50.0, "dims": 16, "scaling": mt._yarn(3.0, 40, fast=1.0, slow=6.0)}])  # a ramp that ends before it starts
def test_rotation_table_of_the_engine_is_the_plain_one(rot):
    from jllm_serve_amd.config.miforax import _rope
    from jllm_serve_amd.parts.rope import rope_table
    cos, sin = rope_table(_rope(rot, rot["dims"], "test"), 300)
    f, amp = P.yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    ang = np.arange(300, dtype=np.float64)[:, None] * f.numpy()[None, :]
    assert np.abs(cos - np.cos(ang) * amp).max() < 1e-6 and np.abs(sin - np.sin(ang) * amp).max() < 1e-6
    if rot.get("scaling"):
        assert abs(amp - (0.1 * math.log(rot["scaling"]["factor"]) + 1.0)) < 1e-12


def test_plain_window_and_sink():
    torch.manual_seed(0)
    s = torch.randn(2, 9, 9, dtype=torch.float64)
    p = P.windowed_sink_softmax(s, None, 4)
    for i in range(9):
        seen = [j for j in range(9) if 0 <= i - j < 4]
        assert all((p[:, i, j] > 0).all() for j in seen) and all((p[:, i, j] == 0).all() for j in range(9) if j not in seen)
    assert torch.allclose(p.sum(-1), torch.ones(2, 9, dtype=torch.float64))
    sink = torch.tensor([0.3, -1.0], dtype=torch.float64)
    ps = P.windowed_sink_softmax(s, sink, 0)
    # the sink is one more term of the denominator, unscaled and without a value
    i = 5
    den = torch.exp(s[:, i, :i + 1]).sum(-1) + torch.exp(sink)
    assert torch.allclose(ps[:, i, :i + 1], torch.exp(s[:, i, :i + 1]) / den[:, None])
    assert (ps.sum(-1) < 1).all()


def test_plain_rotation_is_relative_and_partial():
    rot = {"base": 300.0, "dims": 8, "scaling": mt._yarn(2.0, 16)}
    torch.manual_seed(1)
    q, k = torch.randn(6, 12, dtype=torch.float64), torch.randn(6, 12, dtype=torch.float64)
    pos = torch.arange(6)
    a = P.rotate(q, pos, rot) @ P.rotate(k, pos, rot).T
    b = P.rotate(q, pos + 37, rot) @ P.rotate(k, pos + 37, rot).T
    assert torch.allclose(a, b, atol=1e-9), "scores depend on distances only"
    assert torch.equal(P.rotate(q, pos, rot)[:, 8:], q[:, 8:]), "dimensions beyond rot.dims pass unchanged"
    amp = 0.1 * math.log(2.0) + 1.0
    assert torch.allclose(P.rotate(q, torch.zeros(6, dtype=torch.long), rot)[:, :8], q[:, :8] * amp)


def test_plain_experts_and_table():
    torch.manual_seed(2)
    w = {"e0.gate": torch.randn(4, 6, dtype=torch.float64), "e0.up": torch.randn(4, 6, dtype=torch.float64),
         "e0.down": torch.randn(6, 4, dtype=torch.float64)}
    h = torch.randn(3, 6, dtype=torch.float64) * 5
    g, u = h @ w["e0.gate"].T, h @ w["e0.up"].T
    g, u = g.clamp(max=0.7), u.clamp(-0.7, 0.7)
    want = (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w["e0.down"].T
    assert torch.allclose(P.clamped_expert(h, w, "e0.", 0.7), want)
    # top = 2: the mean of the two experts' outputs; a shared expert is added whole
    w.update({"e1.gate": torch.randn(4, 6, dtype=torch.float64), "e1.up": torch.randn(4, 6, dtype=torch.float64),
              "e1.down": torch.randn(6, 4, dtype=torch.float64), "table": torch.tensor([[0, 1], [1, 0]], dtype=torch.int32)})
    mlp = {"router": {"experts": 2, "top": 2}, "expert": {"ff": 4, "limit": 0.7}}
    both = 0.5 * (P.clamped_expert(h, w, "e0.", 0.7) + P.clamped_expert(h, w, "e1.", 0.7))
    assert torch.allclose(P.table_moe(h, [0, 1, 0], w, "", mlp), both)
    z = torch.linspace(-4, 4, 9, dtype=torch.float64)
    assert torch.allclose(P.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))


def test_plain_borrowed_cache_is_the_owners_latent(miforax_folders):
    """Layer 1 of MF_A has no down-projection of its own: changing layer 0's changes layer 1's keys and values too."""
    cfg = mt.MF_A
    w = mt.load_weights(miforax_folders["MA"])
    toks = mt.prompt("MA", 12)
    assert "l1.mix.dkv" not in w and "l0.mix.dkv" in w and "l2.norm2" not in w
    lay_a, lay_b = [], []
    P.forward(cfg, w, toks, lay_a)
    w2 = dict(w)
    w2["l0.mix.uk"] = w["l0.mix.uk"] * 0  # layer 0's own keys vanish, its latent stays: layer 1's scores keep their keys
    w2["l0.mix.uv"] = w["l0.mix.uv"] * 0
    P.forward(cfg, w2, toks, lay_b)
    d1 = lay_b[1] - lay_b[0] - (lay_a[1] - lay_a[0])
    assert d1.abs().max() > 1e-3  # layer 1 sees another input ...
    h = P.rmsnorm(lay_a[0], w["l1.norm1"], 1e-5)
    c, kr = P.latent_kv(P.rmsnorm((w["embed"][torch.tensor(toks)] * 3.5), w["l0.norm1"], 1e-5), w, "l0.mix.", cfg["layers"][0]["mixer"],
                        1e-5, torch.arange(12))
    out = P.latent_attention(h, w, "l1.mix.", cfg["layers"][1]["mixer"], 1e-5, torch.arange(12), c, kr)
    x1 = lay_a[0] + out
    hh = P.rmsnorm(x1, w["l1.norm2"], 1e-5)
    x1 = x1 + P.table_moe(hh, toks, w, "l1.mlp.", cfg["layers"][1]["mlp"])
    assert torch.allclose(x1, lay_a[1], atol=1e-10)  # ... and is computed from layer 0's cached latent


def test_cache_groups_and_windows_of_the_model():
    from jllm_serve_amd.cache.manager import CacheManager
    from jllm_serve_amd.parts.model import DecoderModel
    model = DecoderModel(parse_config(mt.MF_A), torch.float32, "cpu", 64)
    plans = model.cache_plans()
    assert [p.cache_from for p in plans] == [None, 0, None, None] and plans[1].kv is None
    cm = CacheManager(plans, 8, 8 * 40, 2, allocate=False)
    assert [(g.spec.rows[0].shape, g.spec.window) for g in cm.groups] == [((40,), 19), ((64,), 0), ((24,), 5)]
    cm.open("a")
    cm.begin_write("a", 50)
    cm.commit("a", 50)
    t = [cm.table("a", gi).tolist() for gi in range(3)]
    # after 50 positions a query at 50 sees keys from 32 (window 19), 0 (no window), 46 (window 5)
    assert [sum(p < 0 for p in x) for x in t] == [4, 0, 5]
    cm.close("a")
    cm.check()


def test_random_weights_mode_makes_what_the_model_asks_for(miforax_folders):
    from jllm_serve_amd.weights import SafetensorsSource
    from jllm_serve_amd.weights.loader import WeightError, check
    from jllm_serve_amd.weights.random_init import model_weight_specs
    cfg, specs = model_weight_specs(mt.MF_A)
    src = SafetensorsSource(miforax_folders["MA"])
    check(specs, src)
    table = src.get("l1.mlp.table")
    assert table.dtype == torch.int32 and tuple(table.shape) == (160, 2)
    assert int(table.min()) >= 0 and int(table.max()) < 5 and (table[:, 0] != table[:, 1]).all()
    assert len({int(x) for x in table.flatten()}) == 5
    with pytest.raises(WeightError, match="l0.mix.dkv"):
        check([s for s in specs if s.name != "l0.mix.dkv"], src)
