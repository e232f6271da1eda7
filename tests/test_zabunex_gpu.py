"""Zabunex on the GPU against the plain implementation in ``plain_zabunex``: every new
kernel alone, then whole models of three configurations under the four ways of cutting
(whole, decoded tail, portions down to two tokens, mixed batches over a pool of exactly
the trace's peak, filled with NaN, whose pages and slots serve again), keys made loud far
back, at the first positions, and on both sides of a chunk's edge where that edge is also
a page's, long decoding beside requests that come and go, the stream after every layer,
and greedy generation through the engine's entry point."""

from types import SimpleNamespace

import pytest
import torch

import plain_zabunex as P
import replay
from halite_amd.config import ModelConfig, ServerConfig
from halite_amd.engine import InferenceEngine
from halite_amd.engine.runner import ModelRunner
from halite_amd.kernels import ops

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 5e-5, "bfloat16": 2.5e-2}  # of the largest logit
CONFIGS = {"A": (P.ZAB_A, P.ZAB_A_BIAS), "B": (P.ZAB_B, P.ZAB_B_BIAS), "C": (P.ZAB_C, P.ZAB_C_BIAS)}
LENGTHS = {"A": [5, 70, 33, 1, 130], "B": [90, 2, 41, 160], "C": [64, 17, 150, 3]}
F = torch.float64


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain_logits(cfg, weights, ids):
    return P.forward(cfg, weights, ids).float()


def make_runner(folder, dtype, pool_tokens, page_size=16, graphs=False):
    server = ServerConfig(kv_cache_num_tokens=pool_tokens, page_size=page_size, max_seqs_per_forward=4,
                          use_cudagraph=graphs)
    runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype=dtype))
    for g in runner.cache.groups:  # a page that is read before it is written, or after its time, shows
        g.storage.fill_(float("nan"))
    return runner


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (cfg, bias_rows) in CONFIGS.items():
        weights = P.random_weights(cfg, bias_rows, seed=5 + len(name))
        requests = {f"r{i}": tokens(cfg, n, 300 + i) for i, n in enumerate(LENGTHS[name])}
        ref = {rid: plain_logits(cfg, weights, ids) for rid, ids in requests.items()}
        for dtype in DT:
            folder = str(tmp_path_factory.mktemp(f"zab{name}_{dtype}"))
            P.write_model_folder(folder, cfg, weights, DT[dtype])
            out[(name, dtype)] = (folder, requests, ref, weights)
    return out


def check(rows, ref, dtype):
    """float32: every row within the tolerance.  bfloat16: a norm on a part's result makes a
    row whose result nearly cancels as sensitive to the roundings before it as the result is
    small (the float32 engine shows the same rows as its worst, 10 to 20 times its median
    error); so all rows are finite and within five times the tolerance, and all but a few
    (4%, at least two) within the tolerance itself."""
    if dtype == "float32":
        return replay.compare(rows, ref, TOL[dtype])
    replay.compare(rows, ref, 5 * TOL[dtype])
    n = over = 0
    for rid, by_pos in rows.items():
        scale = max(1.0, float(ref[rid].abs().max()))
        for p, row in by_pos.items():
            n, over = n + 1, over + (float((row - ref[rid][p]).abs().max()) / scale > TOL[dtype])
    assert over <= max(2, 0.04 * n), f"{over} of {n} rows beyond the tolerance"


def rand(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def step_arrays(gpu, cuts, slots):
    """The step's arrays for segments of ``cuts`` tokens that belong to ``slots``."""
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)  # noqa: E731
    starts = [sum(cuts[:i]) for i in range(len(cuts))]
    seg = [i for i, n in enumerate(cuts) for _ in range(n)]
    slot = [slots[i] for i, n in enumerate(cuts) for _ in range(n)]
    return i32(seg), i32(starts), i32(cuts), i32(slot)


# -- kernels alone --------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(1, 40), (37, 64), (5, 1028), (3, 4096), (2, 8200), (4, 30)])
@pytest.mark.parametrize("two", [False, True])
def test_norm_of_a_result_added_to_the_stream(gpu, dtype, sizes, two):
    """Rows of a few vectors a thread, of more than a thread keeps, and of a length that is
    no multiple of four; one result, or the sum of two with a constant each."""
    t, d = sizes
    h, a, w = rand(t, d, seed=1), rand(t, d, seed=2, scale=3.0), (1 + 0.2 * rand(d, seed=3)).to(DT[dtype])
    b = rand(t, d, seed=4, scale=2.0)
    hg = h.to(gpu)
    if two:
        cast = ops.post_norm_add(hg, a.to(gpu), w.to(gpu), 1e-5, cast_to=DT[dtype], scale=0.6, second=b.to(gpu), second_scale=-1.1)
        a = 0.6 * a.to(F) - 1.1 * b.to(F)
    else:
        cast = ops.post_norm_add(hg, a.to(gpu), w.to(gpu), 1e-5, cast_to=DT[dtype])
    want = h.to(F) + P.rms_norm(a.to(F), w.to(F), 1e-5)
    assert float((hg.cpu() - want).abs().max()) < 2e-6 * float(want.abs().max())
    assert torch.equal(cast.float().cpu(), hg.cpu().to(DT[dtype]).float())
    assert torch.equal(ops.cast_rows(hg, DT[dtype]).float().cpu(), hg.cpu().to(DT[dtype]).float())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_square_of_relu_and_scaled_sum(gpu, dtype):
    x = rand(33, 50, seed=4).to(DT[dtype])
    got = ops.relu_squared(x.to(gpu)).float().cpu()
    assert float((got - P.relu_squared(x.float()).to(DT[dtype]).float()).abs().max()) == 0.0
    if dtype == "bfloat16":  # few rows: the activation as the product's epilogue
        a, w = rand(5, 64, seed=14).to(DT[dtype]), rand(48, 64, seed=15, scale=0.3).to(DT[dtype])
        got = ops.gemm_bf16_skinny(a.to(gpu), ops.tile_weight(w.to(gpu)), tiled_shape=(48, 64), relu_squared=True).float().cpu()
        want = P.relu_squared(a.float() @ w.float().T)
        assert float((got - want).abs().max()) < 2e-2 * float(want.abs().max())
    y, z = rand(7, 12, seed=5), rand(7, 12, seed=6)
    got = ops.scaled_sum_(y.to(gpu), 0.6, z.to(gpu), -1.1).cpu()
    assert float((got - (0.6 * y - 1.1 * z)).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(3, 1, 20, 20, 32, True), (4, 2, 16, 16, 16, True), (2, 1, 24, 8, 32, False), (5, 5, 4, 12, 16, False),
                                   (3, 3, 6, 10, 16, False)])
@pytest.mark.parametrize("first", [5, 8])
def test_whole_projection_norms_and_packed_rows(gpu, dtype, shape, first):
    """q and k over all heads at once, the temperature by position, the values the raw keys or
    a projection of their own; heads padded to the pages' head size.  Rows that begin at a
    multiple of four columns (16-byte accesses) and rows that do not."""
    H, K, dq, dv, D, from_keys = shape
    t = 29
    a = rand(t, 8 + H * dq + K * dq + K * dv, seed=7, scale=2.0)[:, 8 - first :]
    q, k = a[:, first : first + H * dq], a[:, first + H * dq : first + (H + K) * dq]
    v = None if from_keys else a[:, first + (H + K) * dq :]
    wq, wk = (1 + 0.3 * rand(H * dq, seed=8)).to(DT[dtype]), (1 + 0.3 * rand(K * dq, seed=9)).to(DT[dtype])
    pos = torch.arange(t, dtype=torch.int32) * 3 + 1
    ag = a.contiguous().to(gpu)
    packed = ops.qk_norm_pack(
        ag[:, first : first + H * dq], ag[:, first + H * dq : first + (H + K) * dq], None if from_keys else ag[:, first + (H + K) * dq :],
        wq.to(gpu), wk.to(gpu), 1e-5, H, K, dq, dv, D, DT[dtype], positions=pos.to(gpu), temp_coef=0.4, temp_every=4,
    ).float().cpu().view(t, H + 2 * K, D)
    temp = 1 + 0.4 * torch.log((torch.div(pos + 1, 4, rounding_mode="floor") + 1).to(F))
    want_q = (P.rms_norm(q.to(F), wq.to(F), 1e-5) * temp[:, None]).view(t, H, dq)
    want_k = P.rms_norm(k.to(F), wk.to(F), 1e-5).view(t, K, dq)
    want_v = (k if from_keys else v).to(F).view(t, K, dv)
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert float((packed[:, :H, :dq] - want_q).abs().max()) < tol * float(want_q.abs().max())
    assert float((packed[:, H : H + K, :dq] - want_k).abs().max()) < tol * float(want_k.abs().max())
    assert float((packed[:, H + K :, :dv] - want_v).abs().max()) < tol * float(want_v.abs().max())
    assert float(packed[:, : H + K, dq:].abs().max() if D > dq else 0.0) == 0.0
    assert float(packed[:, H + K :, dv:].abs().max() if D > dv else 0.0) == 0.0


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("act", [False, True])
def test_short_convolution_in_steps(gpu, taps, act):
    """Two requests whose tokens come in steps of unequal sizes (one token, fewer than the
    taps, many), in slots that are not in order; the carried inputs make the steps equal to
    the whole sequences.  A slot that is zeroed serves a new request."""
    C = 70
    seqs = {2: rand(41, 3 + C, seed=10), 0: rand(24, 3 + C, seed=11)}
    w, b = rand(C, taps, seed=12, scale=0.5), rand(C, seed=13)
    want = {s: P.short_convolution(u[:, 3:].to(F), w.to(F), b.to(F)) for s, u in seqs.items()}
    if act:
        want = {s: P.silu(y) for s, y in want.items()}
    state = torch.full((4, taps - 1, C), float("nan"), device=gpu)
    state[0].zero_(), state[2].zero_()
    # (a step of single tokens alone takes the kernel that convolves and carries at once)
    plan = [({2: 1, 0: 2}), ({2: 2}), ({0: 1, 2: 1}), ({0: 1, 2: 30}), ({2: 7, 0: 20})]
    at = {2: 0, 0: 0}
    for step in plan:
        slots = list(step)
        cuts = [step[s] for s in slots]
        u = torch.cat([seqs[s][at[s] : at[s] + step[s]] for s in slots]).to(gpu)
        seg, starts, lens, slot = step_arrays(gpu, cuts, slots)
        step_ctx = SimpleNamespace(token_seg=seg, seg_q_start=starts, seg_q_len=lens, token_slot=slot, n_segs=len(cuts))
        y = ops.short_conv_through(u[:, 3:], w.to(gpu), b.to(gpu), state, step_ctx, torch.float32, silu=act).cpu()
        r = 0
        for s in slots:
            ref = want[s][at[s] : at[s] + step[s]]
            assert float((y[r : r + step[s]] - ref).abs().max()) < 1e-5, (taps, s, at[s])
            r += step[s]
            at[s] += step[s]
    assert at == {2: 41, 0: 24}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 16, 16, 2), (3, 8, 8, 1), (5, 12, 24, 5), (2, 80, 40, 2), (1, 64, 130, 1)])
@pytest.mark.parametrize("chunk", [None, 3, 16])
def test_state_space_recurrence_in_steps(gpu, dtype, shape, chunk):
    """The recurrence over two requests cut into steps against the whole sequences, the
    state carried in float32 rows; decays from nearly 1 to nearly 0.  With ``chunk`` every
    segment is cut into chunks of that many tokens that are walked side by side."""
    heads, Pd, N, G = shape
    T = {1: 37, 3: 12}
    x = {s: rand(n, heads * Pd + 2 * G * N, seed=20 + s).to(DT[dtype]) for s, n in T.items()}
    dt = {s: rand(n, 2 + heads, seed=30 + s, scale=2.0) for s, n in T.items()}
    dt_bias, a_log, skip = rand(heads, seed=40).to(DT[dtype]), (rand(heads, seed=41) - 1).to(DT[dtype]), rand(heads, seed=42).to(DT[dtype])
    want = {}
    for s, n in T.items():
        xs = x[s].to(F)
        want[s], _ = P.selective_scan(xs[:, : heads * Pd].view(n, heads, Pd), xs[:, heads * Pd : heads * Pd + G * N].view(n, G, N),
                                      xs[:, heads * Pd + G * N :].view(n, G, N), dt[s][:, 2:].to(F), dt_bias.to(F), a_log.to(F), skip.to(F))
    state = torch.full((4, heads, N, Pd), float("nan"), device=gpu)
    state[1].zero_(), state[3].zero_()
    at = {1: 0, 3: 0}
    for step in ({1: 5, 3: 1}, {3: 1, 1: 1}, {1: 2}, {3: 10, 1: 29}):
        slots = list(step)
        cuts = [step[s] for s in slots]
        xs = torch.cat([x[s][at[s] : at[s] + step[s]] for s in slots]).to(gpu)
        ds = torch.cat([dt[s][at[s] : at[s] + step[s]] for s in slots]).to(gpu)
        _, starts, lens, slot = step_arrays(gpu, cuts, slots)
        chunks = seg_chunks = None
        if chunk:
            rows, per_seg, t0 = [], [], 0
            for i, n in enumerate(cuts):
                per_seg.append((len(rows), -(-n // chunk)))
                rows += [(t0 + k, min(chunk, n - k), i, 0) for k in range(0, n, chunk)]
                t0 += n
            chunks = torch.tensor(rows, dtype=torch.int32, device=gpu)
            seg_chunks = torch.tensor(per_seg, dtype=torch.int32, device=gpu)
        y = ops.ssd_scan(xs, ds[:, 2:], dt_bias.to(gpu), a_log.to(gpu), skip.to(gpu), state, starts, lens, slot, G,
                         chunks=chunks, seg_chunks=seg_chunks).cpu()
        r = 0
        for s in slots:
            ref = want[s][at[s] : at[s] + step[s]].reshape(step[s], -1)
            assert float((y[r : r + step[s]] - ref).abs().max()) < 2e-5 * max(1.0, float(ref.abs().max())), (s, at[s])
            r += step[s]
            at[s] += step[s]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("parts", [1, 2, 5])
def test_gate_then_norm_in_parts(gpu, dtype, parts):
    t, n = 19, 60
    y, a = rand(t, n, seed=50, scale=2.0), rand(t, 4 + n, seed=51)
    w = (1 + 0.2 * rand(n, seed=52)).to(DT[dtype])
    got = ops.gated_part_norm(y.to(gpu), a.to(gpu)[:, 4:], w.to(gpu), 1e-5, parts, DT[dtype]).float().cpu()
    want = P.gated_part_norm(y.to(F), a[:, 4:].to(F), w.to(F), 1e-5, parts)
    assert float((got - want).abs().max()) < (1e-5 if dtype == "float32" else 2e-2) * float(want.abs().max())


def test_rows_of_the_bias_table_by_distance():
    from halite_amd.parts.normed_attention import distance_buckets

    for buckets, far in ((12, 40), (10, 17), (6, 100), (16, 9), (32, 1000), (2, 5)):
        got = distance_buckets(buckets, far).tolist()
        assert got == [P.distance_bucket(n, buckets, far) for n in range(far + 1)]
        assert got[-1] == buckets - 1 and P.distance_bucket(far * 7, buckets, far) == buckets - 1


# -- whole models -----------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed", "mixed2"])
def test_schedules(folders, name, dtype, schedule):
    folder, requests, ref, _ = folders[(name, dtype)]
    cfg = CONFIGS[name][0]
    make = {"whole": replay.whole, "tail": lambda q: replay.tail_one_by_one(q, tail=40), "portions": replay.portions,
            "mixed": replay.mixed, "mixed2": lambda q: replay.mixed(q, seed=7, decode_tail=30)}[schedule]
    trace = make(requests)
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16))
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
    check(rows, ref, dtype)
    assert runner.cache.idle()


def test_long_prompts_whose_recurrence_is_cut_into_chunks(folders):
    """Prompts of several chunks of the recurrence beside short ones in one step, against the
    token-by-token model; then the same requests decoded on, so the carried state counts."""
    from halite_amd.parts import state_space

    for name, dtype in (("A", "float32"), ("B", "bfloat16")):
        folder, _, _, weights = folders[(name, dtype)]
        cfg = CONFIGS[name][0]
        n = 4 * state_space.SCAN_CHUNK + 37
        requests = {"long": tokens(cfg, n + 9, 61), "short": tokens(cfg, 5, 62), "mid": tokens(cfg, 2 * state_space.SCAN_CHUNK + 8, 63)}
        ref = {rid: plain_logits(cfg, weights, ids) for rid, ids in requests.items()}
        trace = [{"step": 0, "entries": [{"id": "long", "tokens": requests["long"][:n], "want": [0, n // 2, n - 1]},
                                         {"id": "short", "tokens": requests["short"], "want": [4]},
                                         {"id": "mid", "tokens": requests["mid"][:-3], "want": [100]}], "end": ["short"]}]
        for i in range(n, n + 9):
            entries = [{"id": "long", "tokens": [requests["long"][i]], "want": [0]}]
            if i < n + 3:
                entries.append({"id": "mid", "tokens": [requests["mid"][i - n - 3]], "want": [0]})
            trace.append({"step": len(trace), "entries": entries, "end": ["mid"] if i == n + 2 else (["long"] if i == n + 8 else [])})
        runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16))
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
        check(rows, ref, dtype)
        assert runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [8, 32, 64])
@pytest.mark.parametrize("name", ["A", "B"])
def test_other_page_sizes(folders, name, page_size, dtype):
    """Pages of 32 and 64 tokens are kept in the matrix-core kernel's own order in bfloat16."""
    folder, requests, ref, _ = folders[(name, dtype)]
    trace = replay.mixed(requests, seed=3)
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, page_size), page_size=page_size)
    rows = replay.collect(trace, replay.run_trace(runner, trace), CONFIGS[name][0]["vocab"])
    check(rows, ref, dtype)
    assert runner.cache.idle()


def test_the_stream_after_every_layer(folders):
    from halite_amd.parts import block

    folder, requests, _, weights = folders[("A", "float32")]
    ids = requests["r1"]
    want = []
    P.forward(P.ZAB_A, weights, ids, layers_out=want)
    runner = make_runner(folder, "float32", 256)
    seen, inner = [], block.PostNormBlock.forward

    def forward(self, h, pending, ctx, run):
        out = inner(self, h, pending, ctx, run)
        seen.append(h.clone())
        return out

    block.PostNormBlock.forward = forward
    try:
        trace = replay.whole({"r1": ids})
        replay.run_trace(runner, trace)
    finally:
        block.PostNormBlock.forward = inner
    assert len(seen) == len(want) == 3
    for got, w in zip(seen, want):
        assert float((got.cpu() - w.float()).abs().max()) < 5e-5 * max(1.0, float(w.abs().max()))


# -- keys made loud -----------------------------------------------------------------------------

LOUD, ASK = 7, 11


def loud_biased_model():
    """One attention layer whose scores are dominated by one pair of tokens: the key of
    token LOUD and the query of token ASK have one large entry, so ASK's attention is all on
    LOUD wherever LOUD is visible, whatever lies between and however far back it is (the
    bias table is small beside it).  The values are the keys, so LOUD's value is loud too."""
    cfg = P.model_cfg(64, 61, [P.attention_layer(2, 1, 16, 1.5, 20, 0.2, 32)])
    w = P.random_weights(cfg, {0: 8}, seed=77)
    e = w["embed"].to(F)
    # (no louder: the norm over the whole projection would make that entry as large in
    # every token's key as it is in LOUD's)
    w["l0.mix.k"][0] = (e[LOUD] / (e[LOUD] @ e[LOUD])).float()
    for head in range(2):
        w["l0.mix.q"][head * 16] = (e[ASK] / (e[ASK] @ e[ASK])).float()
    w["l0.mix.rel"] *= 0.2
    w["l0.mix.o"] *= 3.0
    return cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}, {0: 8}


def loud_chunked_model(chunk):
    """The same for the attention inside chunks: the loud entry sits in a dimension that is
    not rotated and passes the convolutions unmixed (their last tap is 1, the others 0, on
    that channel)."""
    left = P.left_cfg(2, 1, 16, 16, 0.25, 3, chunk, 8)
    cfg = P.model_cfg(32, 61, [P.parallel_layer(left, P.right_cfg(2, 8, 8, 1, 2, 1), 1.0, 0.3)])
    w = P.random_weights(cfg, {}, seed=78)
    e = w["embed"].to(F)
    row = 8  # the first entry of a head that does not rotate
    w["l0.mix.left.k"][row] = (6.0 * e[LOUD] / (e[LOUD] @ e[LOUD])).float()
    w["l0.mix.left.k.conv"][row] = torch.tensor([0.0, 0.0, 1.0])
    for head in range(2):
        w["l0.mix.left.q"][head * 16 + row] = (6.0 * e[ASK] / (e[ASK] @ e[ASK])).float()
        w["l0.mix.left.q.conv"][head * 16 + row] = torch.tensor([0.0, 0.0, 1.0])
    w["l0.mix.left.o"] *= 3.0
    return cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}, {}


def loud_sequence(cfg, n, loud_at, ask_at, seed):
    ids = [t if t not in (LOUD, ASK) else 1 for t in tokens(cfg, n, seed)]
    for p in loud_at:
        ids[p] = LOUD
    for p in ask_at:
        ids[p] = ASK
    return ids


def replay_all(cfg, w, requests, dtype, tmp_path, tail=80, page_size=16):
    ref = {rid: plain_logits(cfg, w, ids) for rid, ids in requests.items()}
    folder = P.write_model_folder(str(tmp_path), cfg, w, DT[dtype])
    for make in (replay.whole, lambda q: replay.tail_one_by_one(q, tail=tail), replay.portions,
                 lambda q: replay.portions(q, sizes=(15, 1, 32, 2, 1, 1, 16, 64)), replay.mixed):
        trace = make(requests)
        runner = make_runner(folder, dtype, replay.peak_tokens(trace, page_size), page_size=page_size)
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
        check(rows, ref, dtype)
        assert runner.cache.idle()
    return ref


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [16, 32])
def test_a_loud_key_far_back_and_at_the_first_positions(dtype, page_size, tmp_path):
    """LOUD at position 3 (and, in a second request, at position 0) among hundreds of keys,
    ASK right behind it and hundreds of tokens later, beyond the bias table's last distance
    and across many pages."""
    cfg, w, _ = loud_biased_model()
    requests = {"far": loud_sequence(cfg, 400, [3], [4, 200, 255, 256, 399], 2),
                "first": loud_sequence(cfg, 300, [0], [1, 150, 299], 3)}
    ref = replay_all(cfg, w, requests, dtype, tmp_path, page_size=page_size)
    quiet = plain_logits(cfg, w, [1 if t == LOUD else t for t in requests["far"]])
    assert float((ref["far"][399] - quiet[399]).abs().max()) > 0.2 * float(ref["far"].abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunk", [32, 24])
@pytest.mark.parametrize("page_size", [16, 32])
def test_loud_keys_on_both_sides_of_a_chunks_edge(dtype, chunk, page_size, tmp_path):
    """With pages of 16: LOUD at the last position of a chunk and at the first of the next
    (for chunks of 32 those are a page's last and first slot), ASK just behind each, at the
    chunk's last position and at the first of the chunk after."""
    cfg, w, _ = loud_chunked_model(chunk)
    last, first = 2 * chunk - 1, 3 * chunk
    ask_at = [last + 1, last + 2, first + 1, first + chunk - 1, first + chunk, first + chunk + 1]
    requests = {"edges": loud_sequence(cfg, 5 * chunk, [last, first], ask_at, 4),
                "start": loud_sequence(cfg, 2 * chunk + 3, [0], [1, chunk - 1, chunk, chunk + 1], 5)}
    ref = replay_all(cfg, w, requests, dtype, tmp_path, tail=2 * chunk + 5, page_size=page_size)
    r = ref["edges"]  # the plain model itself tells the two sides of an edge far apart
    assert float((r[first + chunk - 1] - r[first + chunk]).abs().max()) > 0.1 * float(r.abs().max())


# -- long decoding, slots and pages that serve again ------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_long_decoding_beside_requests_that_come_and_go(folders, dtype, graphs):
    """A short prompt and 200 tokens decoded one by one (chunks pass, the recurrence runs on)
    beside short requests that take the freed slot and pages one after the other."""
    folder, _, _, weights = folders[("A", dtype)]
    cfg = P.ZAB_A
    ids, other = tokens(cfg, 215, 41), tokens(cfg, 30, 42)
    ref = {"long": plain_logits(cfg, weights, ids)}
    short = plain_logits(cfg, weights, other)
    trace = [{"step": 0, "entries": [{"id": "long", "tokens": ids[:15], "want": list(range(15))}], "end": []}]
    for i in range(15, 215):
        entries = [{"id": "long", "tokens": [ids[i]], "want": [0]}]
        j, rid = (i - 15) % 40, f"other{(i - 15) // 40}"
        if j < 30:
            entries.append({"id": rid, "tokens": [other[j]], "want": [0]})
            ref[rid] = short
        trace.append({"step": len(trace), "entries": entries,
                      "end": (["long"] if i == 214 else []) + ([rid] if j == 29 else [])})
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16), graphs=graphs)
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
    check(rows, ref, dtype)
    assert runner.cache.idle()
    if graphs:
        assert runner.graphs_allowed and runner.graph_replays > 100


def test_pages_behind_a_chunk_are_given_back(folders):
    """The chunked layers' group holds the pages of the chunk at hand only; the layers
    without a chunk hold every page."""
    folder, _, _, _ = folders[("A", "float32")]
    runner = make_runner(folder, "float32", 1024)
    chunked = [g for g in runner.cache.groups if g.need.chunk is not None]
    others = [g for g in runner.cache.groups if g.need.chunk is None]
    assert len(chunked) == 1 and len(others) == 1 and chunked[0].need.chunk == 24
    ids = tokens(P.ZAB_A, 200, 9)
    trace = replay.portions({"r": ids}, sizes=(50, 1, 1, 30))
    slots = {}
    held = []
    from halite_amd.engine.batch import Segment

    for step in trace:
        e = step["entries"][0]
        if "r" not in slots:
            slots["r"] = runner.admit()
        s = slots["r"]
        runner.step([Segment(s, runner.cache.length(s), e["tokens"], [])])
        n = runner.cache.length(s)
        held.append((n, chunked[0].pool.capacity - chunked[0].pool.available, others[0].pool.capacity - others[0].pool.available))
        runner.cache.check()
    for n, few, every in held:
        assert every == -(-n // 16)
        assert few == -(-n // 16) - (n - n % 24) // 16  # the pages from the one that holds the chunk's start
    runner.free(slots["r"])
    assert runner.cache.idle()


# -- through the engine's entry point ----------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    folder, _, _, weights = folders[(name, dtype)]
    cfg = CONFIGS[name][0]
    prompts = [tokens(cfg, n, 500 + n) for n in (5, 17, 33, 2, 48, 9)]
    engine = InferenceEngine.from_pretrained(
        folder, ServerConfig(kv_cache_num_tokens=1024, page_size=16, max_seqs_per_forward=3, chunked_prefill_size=20,
                             max_tokens_per_forward=24),
        ModelConfig(dtype=dtype),
    )
    params = {"max_new_tokens": 12, "temperature": 0.0}
    results = engine.infer_batch([(i, p, params) for i, p in enumerate(prompts)])
    for r, prompt in zip(results, prompts):
        ids = list(prompt)
        for step, tok in enumerate(r.output_ids[0]):
            logits = plain_logits(cfg, weights, ids)[-1]
            best = int(torch.argmax(logits))
            if tok != best:  # 16 bits may turn a near tie; anything else is a fault
                gap = float(logits[best] - logits[tok])
                assert gap < (1e-4 if dtype == "float32" else 0.05), f"request {r.id} token {step}: {tok} for {best}, gap {gap}"
            ids.append(tok)
        assert len(r.output_ids[0]) == 12


# -- the programs: generation from the command line, the random-weights mode, trace replay -----


def test_command_line_and_replay_program(folders, tmp_path):
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, _, _, weights = folders[("A", "float32")]
    cfg = P.ZAB_A
    cmd = [sys.executable, os.path.join(root, "bin", "halite_generate"), "--model", folder, "--prompt-ids", "5,17,3,90,9",
           "sampling.temperature=0", "sampling.max_new_tokens=5", "model.dtype=float32", "server.kv_cache_num_tokens=256"]
    proc = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().split("\n")[-1])
    ids = [5, 17, 3, 90, 9]
    for tok in rec["output_ids"][0]:
        assert tok == int(torch.argmax(plain_logits(cfg, weights, ids)[-1]))
        ids.append(tok)
    assert len(ids) == 10
    # the random-weights mode: a configuration without tensors states the rows of its bias
    # tables; the folder it writes holds the design's own keys, and the engine reads the rows
    # back from the tensors
    stated = json.loads(json.dumps(P.ZAB_C))
    for i, n in P.ZAB_C_BIAS.items():
        stated["layers"][i]["mixer"]["bias_buckets"] = n
    cfgfile, out = tmp_path / "c.json", tmp_path / "rand"
    cfgfile.write_text(json.dumps(stated))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "halite_make_random_model"), "--config", str(cfgfile),
                           "--out", str(out), "--seed", "3", "--dtype", "bfloat16", "--std", "0.1"], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "bias_buckets" not in (out / "config.json").read_text()
    # the replay program on that folder: a prompt in two portions and a decoded token, beside a
    # second request; two slots, so the third request takes the one that was freed
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3, 4, 5], "want": [4]}, {"id": "b", "tokens": [7], "want": [0]}], "end": ["b"]},
        {"step": 1, "entries": [{"id": "a", "tokens": [6, 7], "want": []}, {"id": "c", "tokens": [9, 8], "want": [1]}], "end": ["c"]},
        {"step": 2, "entries": [{"id": "a", "tokens": [8], "want": [0]}], "end": ["a"]},
    ]
    logits = tmp_path / "logits"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(out), "--dtype", "float32",
                           "--out", str(logits), "--max-tokens", "128", "--slots", "2"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    from safetensors.torch import load_file

    stored = {k: v.float() for k, v in load_file(str(out / "model.safetensors")).items()}
    want = plain_logits(P.ZAB_C, stored, [1, 2, 3, 4, 5, 6, 7, 8])
    got0 = torch.from_numpy(np.fromfile(logits / "0.f32", dtype="<f4").reshape(2, -1))
    got1 = torch.from_numpy(np.fromfile(logits / "1.f32", dtype="<f4").reshape(1, -1))
    got2 = torch.from_numpy(np.fromfile(logits / "2.f32", dtype="<f4").reshape(1, -1))
    scale = max(1.0, float(want.abs().max()))
    assert float((got0[0] - want[4]).abs().max()) < 5e-5 * scale and float((got2[0] - want[7]).abs().max()) < 5e-5 * scale
    assert float((got0[1] - plain_logits(P.ZAB_C, stored, [7])[0]).abs().max()) < 5e-5 * scale
    assert float((got1[0] - plain_logits(P.ZAB_C, stored, [9, 8])[1]).abs().max()) < 5e-5 * scale
    # a third live request has no slot
    steps[0]["entries"].append({"id": "x", "tokens": [3], "want": []})
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(out), "--dtype", "float32",
                           "--out", str(logits), "--max-tokens", "128", "--slots", "2"],
                          input=json.dumps(steps[0]) + "\n", cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 1 and "slots" in proc.stderr
