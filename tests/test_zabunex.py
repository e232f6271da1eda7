"""Zabunex without a GPU: the configuration and what is read from tensors' shapes, the
table of tensor names and the loader, the model as data, the page bookkeeping of a
chunked group, and the plain implementation's own pins."""

import json
import os

import pytest
import torch

import plain_zabunex as P
from halite_amd.cache import CacheManager
from halite_amd.config import parse_config, read_config
from halite_amd.config.registry import ConfigError
from halite_amd.parts import Decoder
from halite_amd.parts.base import PagedKVNeed
from halite_amd.weights import load_weights
from halite_amd.weights.loader import WeightError

CONFIGS = {"A": (P.ZAB_A, P.ZAB_A_BIAS), "B": (P.ZAB_B, P.ZAB_B_BIAS), "C": (P.ZAB_C, P.ZAB_C_BIAS)}


def test_the_bias_rows_come_from_the_tensor(tmp_path):
    cfg, rows = CONFIGS["A"]
    arch, parsed = parse_config(cfg)
    assert arch.name == "Zabunex" and parsed.layers[0].mixer.bias_buckets is None
    with pytest.raises(ConfigError, match="bias_buckets"):
        arch.to_spec(parsed)  # the file alone does not say how many rows the table has
    folder = P.write_model_folder(str(tmp_path), cfg, P.random_weights(cfg, rows, 1))
    arch, parsed = read_config(folder)
    assert [getattr(l.mixer, "bias_buckets", None) for l in parsed.layers] == [12, None, 12]
    spec = arch.to_spec(parsed)
    assert spec.layers["l0"].parts["mixer"].params()["distance_bias"] == {"buckets": 12, "max_distance": 40}
    # what is written back is the design's own keys
    written = parsed.to_json_dict()
    assert "bias_buckets" not in json.dumps(written) and written["layers"][1]["mixer"]["left"]["mask"] == {"size": 24}
    # a configuration without a folder states the rows itself
    stated = json.loads(json.dumps(cfg))
    for i, n in rows.items():
        stated["layers"][i]["mixer"]["bias_buckets"] = n
    assert parse_config(stated)[0].to_spec(parse_config(stated)[1]) == spec


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][0]["mixer"].update(vdim=8),  # values that are the keys have their size
    lambda c: c["layers"][0]["mixer"].update(kv_heads=3),
    lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=7),
    lambda c: c["layers"][1]["mixer"]["left"].pop("mask"),
    lambda c: c["layers"][1].update(type="recurrent"),
    lambda c: c["layers"][0]["mlp"].update(kind="gated"),
    lambda c: c.pop("norm"),
])
def test_configurations_that_are_refused(bad):
    cfg = json.loads(json.dumps(P.ZAB_A))
    bad(cfg)
    with pytest.raises(ConfigError):
        parse_config(cfg)


def test_sizes_written_as_floats_without_a_fraction():
    cfg = json.loads(json.dumps(P.ZAB_A))
    cfg["width"], cfg["layers"][0]["mixer"]["bias_max"], cfg["layers"][1]["mixer"]["left"]["mask"]["size"] = 64.0, 40.0, 24.0
    _, parsed = parse_config(cfg)
    assert (parsed.width, parsed.layers[0].mixer.bias_max, parsed.layers[1].mixer.left.mask.size) == (64, 40, 24)
    assert all(type(v) is int for v in (parsed.width, parsed.layers[0].mixer.bias_max))
    cfg["width"] = 64.5
    with pytest.raises(ConfigError):
        parse_config(cfg)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_model_as_data_and_its_tensors(name, tmp_path):
    cfg, rows = CONFIGS[name]
    weights = P.random_weights(cfg, rows, 2)
    folder = P.write_model_folder(str(tmp_path), cfg, weights)
    arch, parsed = read_config(folder)
    spec = arch.to_spec(parsed)
    assert [l.arrangement for l in spec.layers.values()] == ["post_norm"] * len(cfg["layers"])
    model = Decoder(spec, torch.float32, "cpu")
    load_weights(model, arch.weight_map(parsed), folder)
    for i, layer in enumerate(cfg["layers"]):
        block = model.layers[f"l{i}"]
        assert (block.ff is None) == (layer["mlp"] is None)
        if layer["type"] == "attention":
            m = block.mixer
            nq = layer["mixer"]["heads"] * layer["mixer"]["dim"]
            assert torch.equal(m.w_qkv[:nq], weights[f"l{i}.mix.q"]) and torch.equal(m.w_qkv[nq:], weights[f"l{i}.mix.k"])
            assert m.rule.sink and m.rule.chunk == 0 and m.bias_table.shape == (layer["mixer"]["heads"], layer["mixer"]["bias_max"] + 1)
            rel, far = weights[f"l{i}.mix.rel"], layer["mixer"]["bias_max"]
            for n in (0, 1, rows[i] // 2, far - 1, far):
                assert torch.equal(m.bias_table[:, n], rel[P.distance_bucket(n, rows[i], far)])
            assert m.state_need() == {} and m.cache_need().chunk is None
        else:
            (ln, left, ls), (rn, right, rs) = block.mixer.members
            l, r = layer["mixer"]["left"], layer["mixer"]["right"]
            assert (ln, rn, ls, rs) == ("left", "right", layer["mixer"]["left_scale"], layer["mixer"]["right_scale"])
            nq, nk = l["heads"] * l["dim"], l["kv_heads"] * l["dim"]
            assert torch.equal(left.w_qkv[nq + nk :], weights[f"l{i}.mix.left.v"])
            assert torch.equal(left.w_conv[nq : nq + nk], weights[f"l{i}.mix.left.k.conv"])
            assert not left.rule.sink and left.rule.bias is None and left.rule.chunk == l["mask"]["size"]
            need = block.mixer.cache_need()
            assert need.chunk == l["mask"]["size"] and need.n_kv_heads == l["kv_heads"] and need.head_dim >= max(l["dim"], l["vdim"])
            states = block.mixer.state_need()
            assert states["right.state"].shape == (r["heads"], r["state"], r["vdim"])
            assert ("left.conv" in states) == (l["conv"] > 1) and ("right.conv" in states) == (r["conv"] > 1)
            if l["conv"] > 1:
                assert states["left.conv"].shape == (l["conv"] - 1, nq + nk + l["kv_heads"] * l["vdim"])
            assert torch.equal(right.A_log, weights[f"l{i}.mix.right.A_log"])
            cos, sin = left.position.tables(50)
            f = l["rot"]["base"] ** (-2.0 * 1 / l["rot"]["dims"]) / l["rot"]["scaling"]["factor"] if l["rot"]["dims"] > 2 else None
            if f is not None:
                assert abs(float(cos[37, 1]) - torch.cos(torch.tensor(37 * f, dtype=torch.float64)).item()) < 1e-7
    # a tensor that is missing and one that nobody knows are both named
    from safetensors.torch import save_file

    broken = dict(weights)
    broken.pop("l1.norm1")
    broken["l0.mix.v"] = torch.zeros(3)
    save_file({k: v.to(torch.bfloat16) for k, v in broken.items()}, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_weights(Decoder(spec, torch.float32, "cpu"), arch.weight_map(parsed), folder)
    assert "l1.norm1" in e.value.missing and "l0.mix.v" in e.value.unexpected


def test_pages_of_a_chunked_group():
    """Chunks of 24 positions over pages of 16: the pages before the one that holds the start
    of the chunk of the next token go back; a group with a window and a chunk keeps the
    fewer."""
    needs = {0: PagedKVNeed(2, 16, None, 24), 1: PagedKVNeed(2, 16), 2: PagedKVNeed(2, 16, 20, 24)}
    cache = CacheManager(needs, page_size=16, num_pages=40, n_slots=2, allocate=False)
    chunked, plain, both = cache.groups
    slot = cache.admit()
    held = lambda g: g.pool.capacity - g.pool.available  # noqa: E731
    for new_len in (10, 23, 24, 25, 47, 48, 100, 101, 167, 168, 169):
        cache.reserve([(slot, new_len)])
        cache.advance(slot, new_len)
        cache.check()
        last = (new_len - 1) // 16
        assert held(plain) == last + 1
        assert held(chunked) == last + 1 - min(last + 1, (new_len - new_len % 24) // 16)
        oldest = max(new_len - new_len % 24, new_len - 20 + 1, 0)
        assert held(both) == last + 1 - min(last + 1, oldest // 16)
    # a long portion needs the pages of its own first token's chunk on
    assert chunked.pages_missing(slot, 169, 400) == (399 // 16) - (168 // 16) + 1 - held(chunked)
    cache.free(slot)
    assert cache.idle()


# -- the plain implementation's own pins -------------------------------------------------------------


def test_plain_attention_written_twice():
    for name, (cfg, rows) in CONFIGS.items():
        w = P.random_weights(cfg, rows, 3)
        ids = torch.randint(0, cfg["vocab"], (45,), generator=torch.Generator().manual_seed(1)).tolist()
        a, b = P.forward(cfg, w, ids, fast=True), P.forward(cfg, w, ids, fast=False)
        assert float((a - b).abs().max()) < 1e-10


def test_plain_pieces_against_library_routines():
    g = torch.Generator().manual_seed(4)
    u, w, b = torch.randn(30, 6, generator=g, dtype=torch.float64), torch.randn(6, 4, generator=g, dtype=torch.float64), torch.randn(6, generator=g, dtype=torch.float64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (3, 0)), w[:, None, :], b, groups=6)[0].T
    assert float((P.short_convolution(u, w, b) - want).abs().max()) < 1e-12
    x = torch.randn(9, 7, generator=g, dtype=torch.float64)
    assert float((P.softplus(x) - torch.nn.functional.softplus(x)).abs().max()) < 1e-12
    assert float((P.rms_norm(x, torch.ones(7, dtype=torch.float64), 1e-6) - torch.nn.functional.rms_norm(x, (7,), eps=1e-6)).abs().max()) < 1e-12
    # the sink: a softmax over the scores and one more score of 0, whose weight is dropped
    q, k, v = (torch.randn(5, 2, 4, generator=g, dtype=torch.float64) for _ in range(3))
    mask = torch.ones(5, 5, dtype=torch.bool).tril()
    got = P.attend_fast(q, k, v, 0.5, mask, sink=True)
    s = torch.einsum("ihd,jhd->hij", q, k) * 0.5
    s = torch.cat([s.masked_fill(~mask[None], float("-inf")), torch.zeros(2, 5, 1, dtype=torch.float64)], dim=-1)
    want = torch.einsum("hij,jhd->ihd", torch.softmax(s, -1)[..., :5], v)
    assert float((got - want).abs().max()) < 1e-12
    # a rotation keeps lengths, turns by the difference of positions only, and leaves the rest
    r = P.rotate_leading(torch.randn(12, 2, 10, generator=g, dtype=torch.float64), 6, 100.0, 2.0)
    y = torch.ones(12, 2, 10, dtype=torch.float64)
    ry = P.rotate_leading(y, 6, 100.0, 2.0)
    assert float((ry.norm(dim=-1) - y.norm(dim=-1)).abs().max()) < 1e-12 and torch.equal(ry[..., 6:], y[..., 6:])
    d1, d2 = (ry[3, 0] * ry[7, 0]).sum(), (ry[5, 0] * ry[9, 0]).sum()
    assert abs(float(d1 - d2)) < 1e-12 and r.shape == (12, 2, 10)


def test_plain_recurrence_in_two_halves():
    g = torch.Generator().manual_seed(5)
    T, heads, Pd, G, N = 20, 4, 3, 2, 5
    x, Bm, Cm = torch.randn(T, heads, Pd, generator=g, dtype=torch.float64), torch.randn(T, G, N, generator=g, dtype=torch.float64), torch.randn(T, G, N, generator=g, dtype=torch.float64)
    dt, bias, a_log, skip = (torch.randn(T, heads, generator=g, dtype=torch.float64), torch.randn(heads, generator=g, dtype=torch.float64),
                             torch.randn(heads, generator=g, dtype=torch.float64), torch.randn(heads, generator=g, dtype=torch.float64))
    y, S = P.selective_scan(x, Bm, Cm, dt, bias, a_log, skip)
    y1, S1 = P.selective_scan(x[:8], Bm[:8], Cm[:8], dt[:8], bias, a_log, skip)
    y2, S2 = P.selective_scan(x[8:], Bm[8:], Cm[8:], dt[8:], bias, a_log, skip, S=S1)
    assert float((torch.cat([y1, y2]) - y).abs().max()) < 1e-12 and float((S2 - S).abs().max()) < 1e-12
    # the same as a sum over all earlier tokens with the products of the decays between
    step = P.softplus(dt + bias)
    decay = torch.exp(-torch.exp(a_log) * step)
    t, hd = 13, 3
    total = sum(torch.prod(decay[j + 1 : t + 1, hd]) * step[j, hd] * (Cm[t, hd // 2] @ Bm[j, hd // 2]) * x[j, hd] for j in range(t + 1))
    assert float((total + skip[hd] * x[t, hd] - y[t, hd]).abs().max()) < 1e-12
