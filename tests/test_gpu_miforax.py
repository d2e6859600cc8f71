"""Miforax on the GPU against the plain implementation (tests/plain/miforax_plain.py): every mechanism alone, the
attention kernels on crafted keys (far keys, window edges, page borders, sinks), whole prompts against token-by-token
decoding, portions down to two tokens, mixed batches on a pool that is used again, long decoding through captured
steps, greedy generation through the engine, and the replay program."""
import json
import os
import random

import numpy as np
import pytest
import torch

import miforax_tiny as mt
import replay
from plain import miforax_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def built(miforax_folders):
    from jllm_serve_amd.engine import build_runner, load_model
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            model = load_model(miforax_folders[name], dtype, torch.device(DEV), max_positions=1024)
            cache[(name, dtype)] = (model, build_runner(model, page_size=mt.CONFIGS[name][2], pool_tokens=1024,
                                                        max_requests=4, graphs=False))
        return cache[(name, dtype)]
    return get


@pytest.fixture(scope="module")
def plain_logits(miforax_folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            memo[key] = P.forward(mt.CONFIGS[name][0], mt.load_weights(miforax_folders[name]), list(tokens))
        return memo[key]
    return get


def close(got, want, dtype, what=""):
    err = float((got.double().cpu() - want).abs().max())
    assert err <= mt.tolerance(dtype, want), f"{what}: {err} > {mt.tolerance(dtype, want)}"


# ------------------------------------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["MA", "MB", "MC"])
def test_feed_forwards_alone(name, dtype, built, miforax_folders):
    from jllm_serve_amd.engine.step import StepEntry
    cfg = mt.CONFIGS[name][0]
    w = mt.load_weights(miforax_folders[name])
    model, runner = built(name, dtype)
    act = torch.float32 if dtype == "float32" else torch.bfloat16
    torch.manual_seed(3)
    for T in (1, 7, 45, 600):  # 600 rows give MB's experts enough rows each for the tiles of many rows
        toks = mt.prompt(name, T, seed=T)
        ctx = runner.prepare([StepEntry("ff", toks, [])])
        xb = (torch.randn(T, cfg["width"]) * 1.5).to(act)  # large enough that the experts' clamps bite
        res = torch.randn(T, cfg["width"])
        for i, layer in enumerate(cfg["layers"]):
            mlp = layer["mlp"]
            if mlp is None:
                assert model.layers[i].ffn is None
                continue
            r = res.clone().to(DEV)
            model.layers[i].ffn.forward(xb.to(DEV), r, ctx)
            if mlp["kind"] == "dense":
                want = res.double() + P.dense_ff(xb.double(), w, f"l{i}.mlp.")
            else:
                want = res.double() + P.table_moe(xb.double(), toks, w, f"l{i}.mlp.", mlp)
            close(r, want, dtype, f"{name} layer {i} feed-forward, {T} rows")
        runner.finish("ff")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["MA", "MB", "MC"])
def test_mixers_alone_through_the_cache(name, dtype, built, miforax_folders):
    """Every layer's mixer on random inputs: a portion from position 0, a second portion and single rows from the
    cache; a layer that borrows a cache reads what its owner stored from the owner's own input."""
    from jllm_serve_amd.engine.step import StepEntry
    cfg = mt.CONFIGS[name][0]
    eps = cfg["norm"]["eps"]
    w = mt.load_weights(miforax_folders[name])
    model, runner = built(name, dtype)
    act = torch.float32 if dtype == "float32" else torch.bfloat16
    torch.manual_seed(4)
    cuts = (29, 6, 1, 1, 17)
    T = sum(cuts)
    xs = [(torch.randn(T, cfg["width"]) * 0.8).to(act) for _ in cfg["layers"]]
    pos = torch.arange(T)
    kept, want = {}, []
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        if m.get("kv_from") is None:
            kept[i] = P.latent_kv(xs[i].double(), w, p, m, eps, pos)
        c, kr = kept[i if m.get("kv_from") is None else m["kv_from"]]
        want.append(P.latent_attention(xs[i].double(), w, p, m, eps, pos, c, kr))
    got = [[] for _ in cfg["layers"]]
    at = 0
    for n in cuts:
        ctx = runner.prepare([StepEntry("mix", [0] * n, [])])
        for i in range(len(cfg["layers"])):
            res = torch.zeros(n, cfg["width"], device=DEV)
            model.layers[i].mixer.forward(xs[i][at:at + n].to(DEV), res, ctx, runner.cache.slots[i])
            got[i].append(res.cpu())
        runner.cache.commit("mix", n)
        at += n
    runner.finish("mix")
    for i in range(len(cfg["layers"])):
        close(torch.cat(got[i]), want[i], dtype, f"{name} layer {i} mixer")


@pytest.mark.parametrize("gate, limit", [("silu", 0.0), ("gelu_tanh", 0.0), ("swish_clamped", 0.6), ("swish_clamped", 7.0)])
def test_gate_functions_in_every_product_kernel(gate, limit):
    """The gated product with each gate function at row counts that take each product kernel, in both types."""
    from jllm_serve_amd.kernels import ops
    torch.manual_seed(5)

    def ref(g, u):
        if gate == "silu":
            return g * torch.sigmoid(g) * u
        if gate == "gelu_tanh":
            return P.gelu_tanh(g) * u
        g, u = g.clamp(max=limit), u.clamp(-limit, limit)
        return g * torch.sigmoid(1.702 * g) * (u + 1)

    for M, N, K in ((3, 256, 256), (40, 256, 256), (200, 384, 128), (600, 2048, 128), (5, 72, 40)):
        a = torch.randn(M, K).to(torch.bfloat16)
        wg, wu = (torch.randn(N, K) * 0.15).to(torch.bfloat16), (torch.randn(N, K) * 0.15).to(torch.bfloat16)
        want = ref(a.double() @ wg.double().T, a.double() @ wu.double().T)
        for dtype in ("float32", "bfloat16"):
            t = torch.float32 if dtype == "float32" else torch.bfloat16
            out = ops.gemm(a.to(DEV).to(t), wg.to(DEV).to(t), w2=wu.to(DEV).to(t), epilogue=ops.EPI_GATED, out_dtype=t,
                           exact=dtype == "float32", gate=ops.GATE_FUNCTIONS[gate], gate_limit=limit)
            close(out, want, dtype, f"{gate} {M}x{N}x{K}")


# ------------------------------------------------------------------------------------------------ crafted keys


def _attend_plain(qa, rows, R, window, scale, sink, q_pos):
    """float64: qa [T, H, Dk], rows [L, Dk] (position = index), q_pos [T]; returns [T, H, R]."""
    s = torch.einsum("thd,jd->thj", qa, rows) * scale
    j = torch.arange(rows.shape[0])[None, :]
    seen = (j <= q_pos[:, None]) & ((q_pos[:, None] - j < window) if window else torch.ones_like(j, dtype=torch.bool))
    s = s.masked_fill(~seen[:, None, :], float("-inf"))
    e = torch.exp(s - s.amax(-1, keepdim=True))
    den = e.sum(-1, keepdim=True) + (torch.exp(sink[None, :, None] - s.amax(-1, keepdim=True)) if sink is not None else 0)
    return torch.einsum("thj,jr->thr", e / den, rows[:, :R])


@pytest.mark.parametrize("dtype, fast", [("float32", False), ("bfloat16", True), ("bfloat16", False)])
@pytest.mark.parametrize("H, R, Dr, page", [(4, 32, 16, 8), (5, 48, 8, 16), (16, 64, 32, 32), (40, 16, 16, 4), (3, 24, 6, 8)])
def test_attention_kernels_on_crafted_keys(dtype, fast, H, R, Dr, page):
    """One key far back carries a value unlike all others and a score that dominates. The query rows are placed so
    that this key is the window's oldest key, one beyond it, at a page's first and last place, and hundreds of keys
    away without a window; as rows of a long portion and as single rows of other requests. A kernel that is one key
    off at an edge, or drops the sink, is off by the size of the values."""
    from jllm_serve_amd.kernels import ops
    from jllm_serve_amd.parts.latent_attention import LatentStepPlanner, TILE_ROWS
    t = torch.float32 if dtype == "float32" else torch.bfloat16
    Dk = R + Dr
    g = torch.Generator().manual_seed(H * 1000 + R)
    L = 613
    hot = 3 * page + page - 1 if page > 4 else 131  # the last place of a page
    rows = (torch.randn(L, Dk, generator=g) * 0.3).to(t).double()
    direction = torch.nn.functional.normalize(torch.randn(Dk, generator=g), dim=0).to(t).double()
    rows[hot] = (direction * 6.0 + rows[hot]).to(t).double()
    rows[hot, :R] += 2.0  # its value stands out
    rows = rows.to(t).double()
    sink = torch.randn(H, generator=g) * 2 + 1.0
    for window in (0, 37, 64, 300):
        # requests: 0 = one long portion of all rows from position 0; then single rows of further requests that hold the
        # same keys, placed at the edges
        edges = sorted({hot, hot + 1, hot + page, L - 1} | ({hot + window - 1, hot + window, hot + window + 1} if window else {400}))
        edges = [p for p in edges if p < L]
        n_req = 1 + len(edges)
        qa = (torch.randn(L + len(edges), H, Dk, generator=g) * 0.3 + direction * 2.5).to(t)
        q_pos = torch.cat([torch.arange(L), torch.tensor(edges)])
        want = _attend_plain(qa.double(), rows, R, window, 0.9, sink.double(), q_pos)
        # the far key decides rows that see it: the test is blind otherwise
        sees = (q_pos >= hot) & ((q_pos - hot < window) if window else torch.ones_like(q_pos, dtype=torch.bool))
        assert want[sees][..., :R].mean() > 1.0 and want[~sees][..., :R].mean() < 0.5
        width = -(-L // page)
        pages = list(range(n_req * width))
        random.Random(window).shuffle(pages)
        table = torch.tensor(pages, dtype=torch.int32).view(n_req, width)
        cache = torch.full((n_req * width, page, Dk), float("nan"), dtype=t)  # a key read from a wrong place poisons the row
        for r in range(n_req):
            n = L if r == 0 else edges[r - 1] + 1
            for p0 in range(0, n, page):
                k = min(page, n - p0)
                cache[table[r, p0 // page], :k] = rows[p0:p0 + k].to(t)
        row_req = torch.cat([torch.zeros(L, dtype=torch.int32), torch.arange(1, n_req, dtype=torch.int32)])
        runs = [(0, r, min(TILE_ROWS, L - r), r) for r in range(0, L, TILE_ROWS)] + [(1 + i, L + i, 1, p) for i, p in enumerate(edges)]
        meta = {"tiles_dev": torch.tensor(runs, dtype=torch.int32).flatten().to(DEV), "n_tiles": len(runs)} if fast else None
        ops.reset_stats()
        out = ops.latent_attention(qa.view(-1, H * Dk).to(DEV), cache.to(DEV), table.to(DEV), row_req.to(DEV),
                                   q_pos.to(torch.int32).to(DEV), H, R, window, 0.9, sink.to(DEV), meta=meta,
                                   exact=dtype == "float32")
        takes = R % 16 == 0 and Dk % 8 == 0  # what the matrix-core kernel takes; other sizes fall to the general kernel
        if fast:
            assert ops.stats()["ran"].get("jllm_latent_attention_bf16", 0) == (1 if takes else 0), ops.stats()
        got = out.view(-1, H, R).double().cpu()
        assert torch.isfinite(got).all(), f"window {window}: a row read a place that holds no key"
        err = (got - want).abs().amax(dim=(1, 2))
        tol = 1e-4 if dtype == "float32" else 4e-2
        bad = (err > tol).nonzero().flatten().tolist()
        assert not bad, f"window {window}: rows at positions {[int(q_pos[i]) for i in bad[:8]]} differ by up to {float(err.max())}"
        if fast:  # the single rows alone, as a decode step: their keys are cut into ranges over several workgroups
            n1 = len(edges)
            meta1 = {"tiles_dev": torch.tensor([(1 + i, i, 1, p) for i, p in enumerate(edges)], dtype=torch.int32).flatten().to(DEV),
                     "n_tiles": n1, "single_rows": True, "max_context": L}
            assert ops._latent_split(n1, H, window, L)[0] > 0 or window in (37, 64)
            out1 = ops.latent_attention(qa[L:].reshape(n1, H * Dk).to(DEV), cache.to(DEV), table.to(DEV), row_req[L:].to(DEV),
                                        q_pos[L:].to(torch.int32).to(DEV), H, R, window, 0.9, sink.to(DEV), meta=meta1)
            err1 = (out1.view(n1, H, R).double().cpu() - want[L:]).abs().amax(dim=(1, 2))
            assert float(err1.max()) <= tol, f"window {window}: single rows at {edges} differ by {err1.tolist()}"
        if window == 0:  # without the sink the same rows are far off: the sink is not lost in the noise
            no_sink = _attend_plain(qa.double(), rows, R, window, 0.9, None, q_pos)
            assert (no_sink - want).abs().max() > 0.3


# ------------------------------------------------------------------------------------------------ replays


def _replay(model, trace, page, shuffle=None):
    from jllm_serve_amd.engine.trace import TraceRunner
    tr = TraceRunner(None, None, trace.peak, page_size=page, max_live=4, shuffle_free=shuffle, model=model)
    out = {}
    for rec in trace.steps:
        logits = tr.step(rec)
        if rec["step"] in trace.rows:
            got = logits.float().cpu()
            for (rid, p), row in zip(trace.rows[rec["step"]], got):
                out[(rid, p)] = row
    tr.runner.cache.check()
    assert not tr.runner.cache.requests and all(g.pool.used_pages == 0 for g in tr.runner.cache.groups)
    return out, tr.runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["MA", "MB", "MC"])
def test_replays_match_plain_and_each_other(name, dtype, miforax_folders, plain_logits):
    """Whole prompts, the last tokens one by one (captured steps in bfloat16), portions down to two tokens, and mixed
    batches of up to four requests on a pool exactly as large as the busiest step with free pages in random order."""
    from jllm_serve_amd.engine import load_model
    page = mt.CONFIGS[name][2]
    model = load_model(miforax_folders[name], dtype, torch.device(DEV), max_positions=512)
    reqs = {f"r{n}": mt.prompt(name, n, seed=1) for n in (1, 2, 9, 23, 41, 70, 133)}
    want = {(rid, p): row for rid, toks in reqs.items() for p, row in enumerate(plain_logits(name, toks))}
    traces = {}
    for kind in ("whole", "tail", "portions", "mixed"):
        tr = replay.Trace(page)
        if kind == "mixed":
            replay.mixed(tr, reqs, seed=3)
        else:
            for rid, toks in reqs.items():
                {"whole": replay.whole, "tail": replay.tail_one_by_one, "portions": replay.portions}[kind](tr, rid, toks)
        traces[kind] = tr
    got = {}
    for kind, tr in traces.items():
        got[kind], runner = _replay(model, tr, page, shuffle=7 if kind == "mixed" else None)
        assert set(got[kind]) == set(want)
        # against the tolerance at the size of the request's logits (a single row's largest logit may be small)
        scale = {rid: plain_logits(name, toks) for rid, toks in reqs.items()}
        worst = max(float((got[kind][k].double() - want[k]).abs().max()) / mt.tolerance(dtype, scale[k[0]]) for k in want)
        assert worst <= 1.0, f"{kind}: {worst} of the tolerance"
        if kind == "tail" and dtype == "bfloat16":
            assert runner.graphs is not None and runner.graphs.replays > 0, "single tokens did not go through captured steps"
    if dtype == "float32":  # cutting and batching change nothing but the last bits
        for kind in ("tail", "portions", "mixed"):
            d = max(float((got[kind][k] - got["whole"][k]).abs().max()) for k in want)
            assert d <= 2e-5, f"{kind} differs from whole prompts by {d}"


@pytest.mark.parametrize("name, dtype", [("MA", "float32"), ("MB", "bfloat16"), ("MA", "bfloat16")])
def test_long_decoding_lets_every_window_pass_over_decoded_tokens(name, dtype, miforax_folders, plain_logits):
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    page = mt.CONFIGS[name][2]
    model = load_model(miforax_folders[name], dtype, torch.device(DEV), max_positions=256)
    runner = build_runner(model, page_size=page, pool_tokens=256, max_requests=2)
    toks = mt.prompt(name, 170, seed=9)
    want = plain_logits(name, toks)
    got = [runner.step([StepEntry("d", toks[:12], list(range(12)))]).float().cpu()]
    for i in range(12, len(toks)):
        got.append(runner.step([StepEntry("d", toks[i:i + 1], [0])]).float().cpu())
    given_back = runner.cache.stats()["window_pages_given_back"]
    runner.finish("d")
    close(torch.cat(got), want, dtype, "170 positions, 158 of them decoded one by one")
    assert given_back > 0, "no window gave a page back"


def test_greedy_generation_through_the_engine(miforax_folders):
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    from jllm_serve_amd.sampling import SamplingParams
    cfg, _, page = mt.CONFIGS["MA"]
    w = mt.load_weights(miforax_folders["MA"])
    prompts = [mt.prompt("MA", n, seed=2) for n in (5, 17, 33, 2)]
    want = [P.greedy(cfg, w, p, 12) for p in prompts]
    for dtype in ("float32", "bfloat16"):
        model = load_model(miforax_folders["MA"], dtype, torch.device(DEV), max_positions=128)
        runner = build_runner(model, page_size=page, pool_tokens=256, max_requests=3)  # four requests, three places
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=24, prefill_chunk=16, max_positions=128), eos_token_ids=())
        res = eng.generate(prompts, SamplingParams.greedy_params(max_tokens=12))
        if dtype == "float32":
            assert [r.tokens for r in res] == want
        else:
            agree = sum(a == b for r, x in zip(res, want) for a, b in zip(r.tokens, x))
            assert all(r.tokens[0] == x[0] for r, x in zip(res, want)) and agree >= 36, f"bfloat16 agrees on {agree}/48 tokens"


def test_replay_program_and_command_line(miforax_folders, plain_logits, tmp_path):
    """bin/trace_run picks the model class by config.json; the command line generates from the same folder."""
    import subprocess
    import sys
    tr = replay.Trace(64)
    reqs = {"a": mt.prompt("MA", 21, seed=5), "b": mt.prompt("MA", 40, seed=6)}
    replay.mixed(tr, reqs, seed=1)
    got = replay.run(miforax_folders["MA"], "float32", tr, str(tmp_path / "out"), page_size=8)
    for step, rows in tr.rows.items():
        arr = got[step].reshape(len(rows), -1)
        for (rid, p), row in zip(rows, arr):
            ref = plain_logits("MA", reqs[rid])[p]
            assert float((torch.from_numpy(row.copy()).double() - ref).abs().max()) <= mt.tolerance("float32", ref)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "jllm"), "run", "--model", miforax_folders["MA"], "--dtype", "float32",
                        "--prompt", " ".join(map(str, reqs["a"])), "--max-tokens", "6", "--temp", "0", "--json", "--ctx", "128",
                        "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["tokens"] == P.greedy(mt.MF_A, mt.load_weights(miforax_folders["MA"]), reqs["a"], 6)
