"""Kavuvik without a GPU: its ``config.json``, the model description made from it, the
tensor names of a folder, and the random-weights mode."""

import copy
import json
import os

import pytest
import torch

import plain_kavuvik as P
from halite_amd.cache import CacheManager
from halite_amd.config import ConfigError, KavuvikConfig, get_architecture, parse_config, read_config
from halite_amd.parts import Decoder
from halite_amd.weights import ModelFiles, WeightError, expand_weight_map, load_weights, write_random_model


@pytest.mark.parametrize("raw", [P.KAV_A, P.KAV_B, P.KAV_C])
def test_the_description_follows_the_file(raw):
    arch, cfg = parse_config(raw)
    assert arch.name == "Kavuvik" and isinstance(cfg, KavuvikConfig) and cfg.architectures == ["Kavuvik"]
    spec = arch.to_spec(cfg)
    assert spec.vocab_size == raw["vocab"] and spec.hidden_size == raw["width"]
    assert spec.embedding.params()["scale"] == raw["embedding"]["scale"]
    assert spec.head.params()["logit_scale"] == raw["logit_scale"]
    assert [r.layer for r in spec.order] == [f"l{i}" for i in range(len(raw["layers"]))]
    for i, layer in enumerate(raw["layers"]):
        parts = spec.layers[f"l{i}"].parts
        assert spec.layers[f"l{i}"].arrangement == "parallel"
        m, mine = layer["mixer"], parts["mixer"].params()
        assert (mine["n_heads"], mine["nope_dim"], mine["rope_dim"], mine["v_dim"], mine["q_rank"], mine["kv_rank"]) == \
            (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"])
        assert mine["scale"] == m["scale"] and mine["window"] == (m["mask"]["size"] if "mask" in m else None)
        assert mine["eps"] == raw["norm"]["eps"] and mine["output_gate"] is True
        rope = spec.positions[mine["position"]].params()
        assert (rope["rotary_dim"], rope["theta"], rope["interleaved"]) == (m["rot"]["dims"], m["rot"]["base"], False)
        assert parts["mixer_norm"].params()["round_before_weight"] is False
        if layer["mlp"] is None:
            assert "ff" not in parts and "ff_norm" not in parts
            continue
        f, ff = layer["mlp"], parts["ff"].params()
        assert (ff["n_experts"], ff["top_k"], ff["expert"]["intermediate_size"], ff["expert"]["limit"]) == \
            (f["router"]["experts"], f["router"]["top"], f["expert"]["ff"], f["expert"]["limit"])
        assert ff["expert"]["alpha"] == 1.702 and ff["score"] == "sigmoid" and ff["norm_eps"] == 1e-20
        assert (ff["shared"] is None) == ("shared" not in f)
        if "shared" in f:
            assert (ff["shared"]["intermediate_size"], ff["shared"]["limit"]) == (f["shared"]["ff"], f["shared"]["limit"])


def test_what_a_file_must_not_say():
    for change, match in (
        (lambda c: c["layers"][0].__setitem__("type", "convolution"), "latent_attention"),
        (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 9), "top"),
        (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 18), "rot.dims"),
        (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
        (lambda c: c.pop("logit_scale"), "logit_scale"),
        (lambda c: c.__setitem__("vocab", 0), "vocab"),
    ):
        raw = copy.deepcopy(P.KAV_A)
        change(raw)
        with pytest.raises(ConfigError, match=match):
            parse_config(raw)
    with pytest.raises(ConfigError, match="unknown architecture"):
        parse_config({"architecture": "Kavuvix"})
    # the same key that names a list of architectures elsewhere is understood too
    raw = copy.deepcopy(P.KAV_A)
    raw["architectures"] = [raw.pop("architecture")]
    with pytest.raises(ConfigError):  # ... but this design's files say 'architecture'
        parse_config(raw)


@pytest.mark.parametrize("raw", [P.KAV_A, P.KAV_B, P.KAV_C])
def test_tensor_names_and_shapes_of_a_folder(raw, tmp_path):
    """The plain model's own list of names and shapes is what the framework's table and
    parts come to, and a folder written by the random-weights mode holds exactly those."""
    arch, cfg = parse_config(raw)
    model = Decoder(arch.to_spec(cfg), torch.float32, "cpu")
    by_path = {s.path: tuple(s.decl.shape) for s in model.param_slots()}
    table = expand_weight_map(arch.weight_map(cfg), list(model.spec.layers))
    assert {name: by_path[path] for name, path in table.items()} == P.tensor_shapes(raw)
    assert sorted(table.values()) == sorted(by_path)
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=3, dtype="bfloat16")
    files = ModelFiles(folder)
    assert {n: tuple(files.shape_of(n)) for n in files.names()} == P.tensor_shapes(raw)
    assert {files.dtype_of(n) for n in files.names()} == {"BF16"}
    files.close()
    again_arch, again = read_config(folder)
    assert again_arch is arch and again == cfg
    load_weights(model, arch.weight_map(cfg), folder)  # fills the parts' packed tensors through their views
    mixer = model.layers["l0"].mixer
    q_rank = raw["layers"][0]["mixer"]["q_rank"]
    assert torch.equal(mixer.w_down[:q_rank], files_tensor(folder, "l0.mix.dq"))
    assert mixer.w_ukt.shape == (mixer.p.n_heads, mixer.p.kv_rank, mixer.p.nope_dim)
    assert torch.equal(mixer.w_ukt[0].T, files_tensor(folder, "l0.mix.uk")[: mixer.p.nope_dim])


def files_tensor(folder, name):
    from safetensors.torch import load_file

    return load_file(os.path.join(folder, "model.safetensors"))[name].float()


def test_a_folder_that_does_not_fit(tmp_path):
    arch, cfg = parse_config(P.KAV_B)
    weights = P.random_weights(P.KAV_B, seed=1)
    weights["l1.mlp.e9.gate"] = weights["l1.mlp.e0.gate"]
    del weights["l2.mlp.shared.down"]
    weights["l0.mix.g"] = weights["l0.mix.g"][:-1]
    weights["l0.norm2"] = torch.ones(80)  # a norm that nothing reads may be there
    folder = P.write_model_folder(str(tmp_path), P.KAV_B, weights)
    with pytest.raises(WeightError) as e:
        load_weights(Decoder(arch.to_spec(cfg), torch.float32, "cpu"), arch.weight_map(cfg), folder)
    assert e.value.missing == ["l2.mlp.shared.down"] and e.value.unexpected == ["l1.mlp.e9.gate"]
    assert [w[0] for w in e.value.wrong_shape] == ["l0.mix.g"]


def test_cache_groups_hold_one_latent_row_a_token():
    """A layer's pages hold, per token, one row of rotated part + latent (in steps of 16) as a
    key and as a value, whatever the number of heads; layers of equal needs share a group."""
    arch, cfg = parse_config(P.KAV_A)
    model = Decoder(arch.to_spec(cfg), torch.bfloat16, "cpu")
    needs = {i: model.mixer_of_run(i).cache_need() for i in range(2)}
    assert needs[0] == needs[1] and (needs[0].n_kv_heads, needs[0].head_dim, needs[0].window) == (1, 48, 20)
    cache = CacheManager(needs, page_size=16, num_pages=5, n_slots=2, dtype=torch.bfloat16, allocate=False)
    assert [g.runs for g in cache.groups] == [[0, 1]]
    assert CacheManager.bytes_per_page(needs, 16, torch.bfloat16) == 2 * (2 * 16 * 48) * 2
    heads = copy.deepcopy(P.KAV_A)
    heads["layers"][1]["mixer"]["heads"] = 7
    arch, cfg = parse_config(heads)
    model = Decoder(arch.to_spec(cfg), torch.bfloat16, "cpu")
    assert model.mixer_of_run(0).cache_need() == model.mixer_of_run(1).cache_need()


def test_the_architecture_is_found_by_name():
    arch = get_architecture("Kavuvik")
    assert arch.config_cls is KavuvikConfig
    assert json.loads(json.dumps(KavuvikConfig(**P.KAV_C).to_json_dict()))["architecture"] == "Kavuvik"
