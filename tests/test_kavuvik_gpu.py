"""Kavuvik on the GPU against the plain implementation in ``plain_kavuvik``: the new kernels
and parts alone, whole models of three configurations under the four ways of cutting
(whole, decoded tail, portions down to two tokens, mixed batches over a pool that is used
again), keys at the edges of windows and pages made loud so that a step too many or too
few shows, long decoding, and greedy generation through the engine's entry point."""

import math

import pytest
import torch

import plain_kavuvik as P
import replay
from halite_amd.config import ModelConfig, PartSpec, ServerConfig, parse_config
from halite_amd.engine import InferenceEngine, InferenceRequest
from halite_amd.engine.batch import Segment
from halite_amd.engine.runner import ModelRunner
from halite_amd.kernels import ops
from halite_amd.parts import BuildContext
from halite_amd.parts.base import FEED_FORWARDS

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 5e-5, "bfloat16": 2.5e-2}  # of the largest logit
CONFIGS = {"A": P.KAV_A, "B": P.KAV_B, "C": P.KAV_C}
LENGTHS = {"A": [5, 70, 33, 1, 130], "B": [90, 2, 41, 160], "C": [64, 17, 150, 3]}


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain_logits(cfg, weights, ids, dtype):
    return P.forward(cfg, weights, ids, round_to=torch.bfloat16 if dtype == "bfloat16" else None).float()


def make_runner(folder, dtype, pool_tokens, page_size=16):
    server = ServerConfig(kv_cache_num_tokens=pool_tokens, page_size=page_size, max_seqs_per_forward=4)
    runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype=dtype))
    for g in runner.cache.groups:  # a page that is read before it is written, or after its time, shows
        g.storage.fill_(float("nan"))
    return runner


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        weights = P.random_weights(cfg, seed=5 + len(name))
        requests = {f"r{i}": tokens(cfg, n, 300 + i) for i, n in enumerate(LENGTHS[name])}
        for dtype in DT:
            folder = str(tmp_path_factory.mktemp(f"kav{name}_{dtype}"))
            P.write_model_folder(folder, cfg, weights, DT[dtype])
            ref = {rid: plain_logits(cfg, weights, ids, dtype) for rid, ids in requests.items()}
            out[(name, dtype)] = (folder, requests, ref)
    return out


def check(rows, ref, dtype):
    """float32: every row within the tolerance.  bfloat16: a router whose two best scores lie
    closer than the 16-bit roundings before it may choose the other expert than the plain
    model does, and that token's row (and what attends to it) is then another number
    altogether; so all rows are finite, and all but a few (4%, at least two) within the
    tolerance.  The models without routers further down are compared strictly in both."""
    if dtype == "float32":
        return replay.compare(rows, ref, TOL[dtype])
    n = over = 0
    for rid, by_pos in rows.items():
        scale = max(1.0, float(ref[rid].abs().max()))
        for p, row in by_pos.items():
            err = float((row - ref[rid][p]).abs().max()) / scale
            assert err == err, f"request {rid} position {p}: NaN in the logits"
            n, over = n + 1, over + (err > TOL[dtype])
    assert over <= max(2, 0.04 * n), f"{over} of {n} rows beyond the tolerance"


# -- kernels alone --------------------------------------------------------------------------


def rand(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mfma", [False, True])
@pytest.mark.parametrize("sizes", [(37, 3, 40, 8, 24, 20, 56, 16), (130, 2, 11, 1, 10, 7, 9, 2), (1, 5, 64, 0, 64, 70, 72, 0)])
def test_products_of_heads(gpu, dtype, mfma, sizes):
    """Every head reads a column range of wide rows and writes one; a float32 gate."""
    t, h, xs, x0, k, n, ys, y0 = sizes
    x = rand(t, h * xs, seed=1).to(DT[dtype])
    w = rand(h, n, k, seed=2, scale=0.3).to(DT[dtype])
    gate = rand(t, 3 + h * ys, seed=3)
    y = torch.full((t, h * ys), 7.0, dtype=DT[dtype], device=gpu)
    ops.grouped_gemm(x.to(gpu), w.to(gpu), y, n_rows=t, x_group_cols=xs, x_col0=x0, y_group_cols=ys, y_col0=y0,
                     gate=gate.to(gpu)[:, 3:], mfma=mfma)
    want = torch.full((t, h * ys), 7.0)
    for i in range(h):
        r = x.float()[:, i * xs + x0 : i * xs + x0 + k] @ w.float()[i].T
        want[:, i * ys + y0 : i * ys + y0 + n] = r * torch.sigmoid(gate[:, 3 + i * ys : 3 + i * ys + n])
    assert float((y.float().cpu() - want).abs().max()) < (1e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("score", ["sigmoid", "softmax"])
@pytest.mark.parametrize("sizes", [(150, 7, 3), (9, 4, 4), (64, 33, 1)])
def test_router(gpu, score, sizes):
    t, e, top = sizes
    z = rand(t, e, seed=4, scale=2.0)
    idx, wgt = ops.moe_route(z.to(gpu), top, softmax=score == "softmax", normalize=True, norm_eps=1e-20)
    s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
    val, want = torch.topk(s, top, -1)
    assert torch.equal(idx.cpu().long(), want)
    assert float((wgt.cpu() - val / val.sum(-1, keepdim=True)).abs().max()) < 1e-6
    raw = ops.moe_route(z.to(gpu), top, softmax=score == "softmax", normalize=False)[1]
    assert float((raw.cpu() - val).abs().max()) < 1e-6
    offsets, tiles, order = (a.cpu() for a in ops.moe_sort(idx, e))
    counts = torch.bincount(idx.cpu().flatten().long(), minlength=e)
    assert offsets.tolist() == [0] + torch.cumsum(counts, 0).tolist()
    assert tiles.tolist() == [0] + torch.cumsum((counts + 127) // 128, 0).tolist()
    assert sorted(order.tolist()) == list(range(t * top))
    for i in range(e):  # an expert's slice holds the pairs that chose it
        assert all(int(idx.cpu().flatten()[p]) == i for p in order[offsets[i] : offsets[i + 1]].tolist())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [1, 7, 150])
def test_mixture_part_alone(gpu, dtype, rows):
    """The feed-forward part built from its own parameters, against the plain mixture; 150
    rows spread over several tiles of an expert, 1 row leaves most experts without any."""
    d, f = 48, dict(kind="moe", router=dict(experts=6, top=2), expert=dict(ff=40, limit=0.8), shared=dict(ff=24, limit=1.2))
    spec = PartSpec(kind="moe", hidden_size=d, n_experts=6, top_k=2, expert=dict(intermediate_size=40, limit=0.8),
                    shared=dict(intermediate_size=24, limit=1.2))
    ff = FEED_FORWARDS.build(spec, BuildContext(dtype=DT[dtype], device=gpu, hidden_size=d))
    views = ff.allocate({n: DT[dtype] for n in ff.param_decls()})
    w = {}
    for i, (name, view) in enumerate(views.items()):
        view.copy_(rand(*view.shape, seed=20 + i, scale=0.6 if name.startswith("router") else 0.15))
        short = name[: -len(".weight")]  # experts.3.gate.weight is the plain model's e3.gate
        if short.startswith("experts."):
            short = "e" + short[len("experts."):]
        w[short] = view.float().cpu().to(P.F)
    ff.finalize()
    x = rand(rows, d, seed=9).to(DT[dtype])
    rnd = (lambda t: t.to(torch.bfloat16).to(P.F)) if dtype == "bfloat16" else (lambda t: t)
    want = P.mixture(x.to(P.F), w, f, rnd).float()
    got = ff.forward(x.to(gpu), None).float().cpu()
    assert float((got - want).abs().max()) < (2e-5 if dtype == "float32" else 2e-2) * max(1.0, float(want.abs().max()))
    h = torch.ones((rows, d), dtype=torch.float32, device=gpu)
    assert ff.forward(x.to(gpu), None, add_to=h) is None  # the same, added into the stream
    assert float((h.cpu() - 1 - want).abs().max()) < (2e-5 if dtype == "float32" else 2e-2) * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norms_embedding_and_latent_rows(gpu, dtype):
    h = rand(9, 52, seed=1)
    w1, w2 = (1 + 0.1 * rand(52, seed=2)).to(DT[dtype]), (1 + 0.1 * rand(52, seed=3)).to(DT[dtype])
    rows = torch.tensor([4, 0, 8], dtype=torch.int32)
    a, b = ops.rmsnorm_exact(h.to(gpu), w1.to(gpu), 1e-6, DT[dtype], second=w2.to(gpu))
    one = ops.rmsnorm_exact(h.to(gpu), w1.to(gpu), 1e-6, DT[dtype], rows=rows.to(gpu))
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert float((a.float().cpu() - P.rms_norm(h, w1.float(), 1e-6)).abs().max()) < tol
    assert float((b.float().cpu() - P.rms_norm(h, w2.float(), 1e-6)).abs().max()) < tol
    assert torch.equal(one.cpu(), a.cpu()[rows.long()])
    table = rand(11, 20, seed=4).to(DT[dtype])
    ids = torch.tensor([3, 10, 0], dtype=torch.int32)
    got = ops.embedding(ids.to(gpu), table.to(gpu), scale=2.5)
    assert torch.equal(got.cpu(), table.float()[ids.long()] * 2.5)
    # latent rows: [query latent 12 | key/value latent 20, rotated part 6 | 5 more columns]
    raw = rand(7, 43, seed=5)
    wq, wkv = (1 + 0.1 * rand(12, seed=6)).to(DT[dtype]), (1 + 0.1 * rand(20, seed=7)).to(DT[dtype])
    packed = torch.full((7, 4 * 32), 9.0, dtype=DT[dtype], device=gpu)
    cq = ops.latent_prep(raw.to(gpu), 0, 12, 12, 20, 6, 32, wq.to(gpu), wkv.to(gpu), 1e-5, packed, 2 * 32)
    assert float((cq.float().cpu() - P.rms_norm(raw[:, :12], wq.float(), 1e-5)).abs().max()) < tol
    c = P.rms_norm(raw[:, 12:32], wkv.float(), 1e-5)
    k, v, q = packed.float().cpu()[:, 64:96], packed.float().cpu()[:, 96:], packed.float().cpu()[:, :64]
    assert float((k[:, 6:26] - c).abs().max()) < tol and torch.equal(k[:, 6:26], v[:, 6:26])
    assert float((k[:, :6] - raw[:, 32:38]).abs().max()) < tol
    assert float(k[:, 26:].abs().max()) == 0 and float(v[:, :6].abs().max()) == 0 and float(v[:, 26:].abs().max()) == 0
    assert bool((q == 9.0).all())


# -- whole models -----------------------------------------------------------------------------

SCHEDULES = {"whole": replay.whole, "tail": replay.tail_one_by_one, "portions": replay.portions, "mixed": replay.mixed}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_schedules(folders, name, schedule, dtype):
    """Every request whole, with a decoded tail, in portions, and mixed with others, over a
    pool that holds the trace's peak and no more, so that pages and slots are used again."""
    folder, requests, ref = folders[(name, dtype)]
    trace = SCHEDULES[schedule](requests)
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16))
    rows = replay.collect(trace, replay.run_trace(runner, trace), CONFIGS[name]["vocab"])
    check(rows, ref, dtype)
    assert runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [8, 64])
def test_other_page_sizes(folders, page_size, dtype):
    """Pages of 64 tokens put the bfloat16 cache of heads of 32 and 64 into the matrix-core
    kernel's own order."""
    folder, requests, ref = folders[("B", dtype)]
    runner = make_runner(folder, dtype, 512, page_size)
    for make in (replay.mixed, lambda q: replay.portions(q, sizes=(3, 2, 50, 9, 2))):
        trace = make(requests)
        rows = replay.collect(trace, replay.run_trace(runner, trace), P.KAV_B["vocab"])
        check(rows, ref, dtype)
    assert runner.cache.idle()


def test_the_stream_after_every_layer(folders):
    folder, requests, ref = folders[("B", "float32")]
    runner = make_runner(folder, "float32", 512)
    # the residual stream after each layer, in one step
    seen = []
    for block in runner.model.layers.values():
        def wrapped(h, pending, ctx, run, _f=block.forward):
            out = _f(h, pending, ctx, run)
            seen.append(h.clone())
            return out
        block.forward = wrapped
    ids = requests["r0"]
    slot = runner.admit()
    runner.step([Segment(slot, 0, ids, [])])
    runner.free(slot)
    want = []
    P.forward(P.KAV_B, P.random_weights(P.KAV_B, seed=5 + 1), ids, stream_after=want)
    assert len(seen) == len(want) == 3
    for got, w in zip(seen, want):
        assert float((got.cpu() - w.float()).abs().max()) < 5e-5 * max(1.0, float(w.abs().max()))


# -- keys made loud: the edges of a window, of pages, the first token, a key far back ------------


def loud_model(window, base=1.0e6):
    """One layer without a feed-forward whose head scores are dominated by one pair of
    tokens: the key of token LOUD and the query of token ASK have a large entry in the
    slowest-turning rotated dimension, so ASK's attention is all on LOUD whenever LOUD is
    visible, whatever lies between."""
    cfg = P.model_cfg(64, 61, [(P.mixer_cfg(2, 16, 16, 24, 32, 32, 0.25, base=base, window=window), None)], embedding_scale=1.5)
    w = P.random_weights(cfg, seed=77)
    LOUD, ASK, m = 7, 11, cfg["layers"][0]["mixer"]
    slow = m["rot"]["dims"] // 2 - 1
    h = lambda t: P.rms_norm(w["embed"][t].to(P.F) * 1.5, w["l0.norm1"].to(P.F), cfg["norm"]["eps"])  # noqa: E731
    hl = h(LOUD)
    w["l0.mix.dkv"][m["kv_rank"] + slow] = (12.0 * hl / (hl @ hl)).float()
    cq = P.rms_norm(h(ASK) @ w["l0.mix.dq"].to(P.F).T, w["l0.mix.dq.norm"].to(P.F), cfg["norm"]["eps"])
    for head in range(m["heads"]):
        w["l0.mix.uq"][head * (m["dim"] + m["rot_dim"]) + m["dim"] + slow] = (12.0 * cq / (cq @ cq)).float()
    w["l0.mix.o"] *= 3.0  # what the heads bring counts for more than the token's own embedding
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    return cfg, w, LOUD, ASK


def loud_sequence(cfg, n, loud_at, ask_at, LOUD, ASK, seed):
    ids = [t if t not in (LOUD, ASK) else 1 for t in tokens(cfg, n, seed)]
    for p in loud_at:
        ids[p] = LOUD
    for p in ask_at:
        ids[p] = ASK
    return ids


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [40, None])
def test_loud_keys_at_the_edges(dtype, window, tmp_path):
    """With a window of 40 and pages of 16: LOUD at the last slot of a page (15), the first
    of one (64), and at position 0; ASK just inside (LOUD + 39) and just outside (LOUD + 40)
    each.  Without a window: LOUD at positions 0 and 3, ASK hundreds of tokens later."""
    cfg, w, LOUD, ASK = loud_model(window)
    if window:
        loud_at, n = [15, 64], 130
        ask_at = [15 + 38, 15 + 39, 15 + 40, 64 + 39, 64 + 40, 64 + 41]
        first = loud_sequence(cfg, 60, [0], [38, 39, 40, 41], LOUD, ASK, 3)
    else:
        loud_at, ask_at, n = [3], [2, 200, 255, 256, 399], 400
        first = loud_sequence(cfg, 300, [0], [1, 150, 299], LOUD, ASK, 3)
    requests = {"edges": loud_sequence(cfg, n, loud_at, ask_at, LOUD, ASK, 2), "first": first}
    ref = {rid: plain_logits(cfg, w, ids, dtype) for rid, ids in requests.items()}
    if window:  # the plain model itself tells the two sides of the edge far apart
        r = ref["edges"]
        assert float((r[15 + 39] - r[15 + 40]).abs().max()) > 0.2 * float(r.abs().max())
        assert float((r[64 + 39] - r[64 + 40]).abs().max()) > 0.2 * float(r.abs().max())
    folder = P.write_model_folder(str(tmp_path), cfg, w, DT[dtype])
    for make in (replay.whole, lambda q: replay.tail_one_by_one(q, tail=80), replay.portions,
                 lambda q: replay.portions(q, sizes=(15, 1, 38, 2, 1, 1, 40, 64)), replay.mixed):
        trace = make(requests)
        runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16))
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
        replay.compare(rows, ref, TOL[dtype])
        assert runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_a_small_pool(folders, dtype):
    """A short prompt and 200 tokens decoded one by one beside a second request that comes
    and goes: the window passes over decoded tokens and the pages behind it serve again."""
    folder, _, _ = folders[("A", dtype)]
    cfg = P.KAV_A
    weights = P.random_weights(cfg, seed=5 + 1)
    ids, other = tokens(cfg, 215, 41), tokens(cfg, 30, 42)
    ref = {"long": plain_logits(cfg, weights, ids, dtype), "other": plain_logits(cfg, weights, other, dtype)}
    trace = [{"step": 0, "entries": [{"id": "long", "tokens": ids[:15], "want": list(range(15))}], "end": []}]
    for i in range(15, 215):
        entries = [{"id": "long", "tokens": [ids[i]], "want": [0]}]
        j = (i - 15) % 40
        if j < 30:
            entries.append({"id": f"other{(i - 15) // 40}", "tokens": [other[j]], "want": [0]})
        trace.append({"step": len(trace), "entries": entries,
                      "end": (["long"] if i == 214 else []) + ([f"other{(i - 15) // 40}"] if j == 29 else [])})
    # the windowed layers hold three pages a request at most
    runner = make_runner(folder, dtype, 224 + 32)
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
    for rid, by_pos in rows.items():
        check({rid: by_pos}, {rid: ref["long" if rid == "long" else "other"]}, dtype)
    assert runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(folders, dtype):
    """The engine's entry point, scheduler and sampler on a Kavuvik folder: greedy tokens are
    the plain model's, step by step on the engine's own tokens, unless closer than rounding."""
    folder, requests, _ = folders[("C", dtype)]
    cfg, weights = P.KAV_C, P.random_weights(P.KAV_C, seed=5 + 1)
    engine = InferenceEngine.from_pretrained(
        folder, ServerConfig(kv_cache_num_tokens=1024, page_size=16, chunked_prefill_size=48, max_tokens_per_forward=64),
        ModelConfig(dtype=dtype))
    prompts = [requests["r1"], requests["r0"], requests["r3"], requests["r2"][:100]]
    params = {"max_new_tokens": 12, "temperature": 0.0}
    results = engine.infer_batch([InferenceRequest(f"q{i}", p, params) for i, p in enumerate(prompts)])
    for r, prompt in zip(results, prompts):
        got, ids = r.output_ids[0], list(prompt)
        assert len(got) == 12 and r.finish_reason == ["length"]
        for step, tok in enumerate(got):
            logits = plain_logits(cfg, weights, ids, dtype)[-1]
            best = int(torch.argmax(logits))
            assert tok == best or float(logits[best] - logits[tok]) <= (1e-4 if dtype == "float32" else 0.08), (r.id, step)
            ids.append(tok)
    assert engine.model_runner.cache.idle()


def test_groups_and_pages_of_layers_that_differ(folders):
    """Layers with other latent sizes or windows keep pages of their own; a windowed group
    gives pages back while a request runs, one without a window keeps them."""
    folder, requests, _ = folders[("B", "float32")]
    runner = make_runner(folder, "float32", 512)
    groups = runner.cache.groups
    assert [g.runs for g in groups] == [[0], [1], [2]]
    assert [g.need.window for g in groups] == [None, 33, 7]
    assert [g.need.head_dim for g in groups] == [32, 64, 48] and all(g.need.n_kv_heads == 1 for g in groups)
    slot = runner.admit()
    runner.step([Segment(slot, 0, requests["r3"][:100], [])])
    held = [sum(p >= 0 for p in g.tables[slot]) for g in groups]
    assert held == [7, math.ceil(100 / 16) - (100 - 33 + 1) // 16, math.ceil(100 / 16) - (100 - 7 + 1) // 16]
    runner.free(slot)
    assert runner.cache.idle()


# -- the programs: generation from the command line, the random-weights mode, trace replay -----


def test_command_line_and_replay_program(folders, tmp_path):
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, requests, ref = folders[("A", "float32")]
    cfg, weights = P.KAV_A, P.random_weights(P.KAV_A, seed=5 + 1)
    cmd = [sys.executable, os.path.join(root, "bin", "halite_generate"), "--model", folder, "--prompt-ids", "5,17,3,90,9",
           "sampling.temperature=0", "sampling.max_new_tokens=5", "model.dtype=float32", "server.kv_cache_num_tokens=256"]
    proc = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().split("\n")[-1])
    ids = [5, 17, 3, 90, 9]
    for tok in rec["output_ids"][0]:
        assert tok == int(torch.argmax(plain_logits(cfg, weights, ids, "float32")[-1]))
        ids.append(tok)
    assert len(ids) == 10
    # the random-weights mode writes a folder of this architecture that the engine then reads
    cfgfile, out = tmp_path / "c.json", tmp_path / "rand"
    cfgfile.write_text(json.dumps(P.KAV_C))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "halite_make_random_model"), "--config", str(cfgfile),
                           "--out", str(out), "--seed", "3", "--dtype", "bfloat16"], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    # the replay program on that folder: a prompt in two portions and a decoded token, beside a second request
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3, 4, 5], "want": [4]}, {"id": "b", "tokens": [7], "want": [0]}], "end": ["b"]},
        {"step": 1, "entries": [{"id": "a", "tokens": [6, 7], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": [8], "want": [0]}], "end": ["a"]},
    ]
    logits = tmp_path / "logits"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(out), "--dtype", "float32",
                           "--out", str(logits), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    from safetensors.torch import load_file

    stored = {k: v.float() for k, v in load_file(str(out / "model.safetensors")).items()}
    want = P.forward(P.KAV_C, stored, [1, 2, 3, 4, 5, 6, 7, 8]).float()
    got0 = torch.from_numpy(np.fromfile(logits / "0.f32", dtype="<f4").reshape(2, -1))
    got2 = torch.from_numpy(np.fromfile(logits / "2.f32", dtype="<f4").reshape(1, -1))
    scale = max(1.0, float(want.abs().max()))
    assert float((got0[0] - want[4]).abs().max()) < 5e-5 * scale and float((got2[0] - want[7]).abs().max()) < 5e-5 * scale
    assert float((got0[1] - P.forward(P.KAV_C, stored, [7]).float()[0]).abs().max()) < 5e-5 * scale
    assert not (logits / "1.f32").exists()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_through_a_captured_graph(folders, dtype):
    """Decode steps replayed from a graph give what launches one by one give: every part of
    the model reads what varies (experts chosen, rows sorted, pages) on the device."""
    folder, requests, _ = folders[("B", dtype)]
    prompts = [requests["r0"][:40], requests["r2"][:25], requests["r3"][:70]]

    def run(graphs):
        server = ServerConfig(kv_cache_num_tokens=512, page_size=16, max_seqs_per_forward=4, use_cudagraph=graphs)
        runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype=dtype))
        assert runner.graphs_allowed == graphs
        slots = [runner.admit() for _ in prompts]
        runner.step([Segment(s, 0, p, []) for s, p in zip(slots, prompts)])
        rows = []
        for i in range(12):
            segs = [Segment(s, len(p) + i, [(7 * i + j) % P.KAV_B["vocab"]], [0]) for j, (s, p) in enumerate(zip(slots, prompts))]
            rows.append(runner.step(segs).float().cpu().clone())
            if i == 5:  # eager work of the program between replays
                extra = runner.admit()
                runner.step([Segment(extra, 0, [1, 2, 3], [2])])
                runner.free(extra)
        for s in slots:
            runner.free(s)
        assert runner.cache.idle()
        return torch.stack(rows), runner.graph_replays

    eager, none = run(False)
    replayed, count = run(True)
    assert none == 0 and count >= 10
    assert float((eager - replayed).abs().max()) <= (1e-5 if dtype == "float32" else 1e-2) * float(eager.abs().max())
