"""Zabunex: a decoder whose layers norm what a part returns, not what it reads
(``x += norm(mixer(x))``, ``x += norm(ff(x))``), listed one by one in ``config.json``.  A
layer's mixer is either an attention without rotation (queries and keys normed over the
whole projection, the values the keys themselves, a temperature on the queries, a learned
bias by distance, a sink in the softmax) or two mixers side by side whose results are
added with a constant each: an attention inside chunks of positions (short convolutions on
q, k, v, partial rotation with stretched positions) and a state-space recurrence.  The
feed-forward is two products around the square of relu.
"""

from __future__ import annotations

from ..config.registry import Architecture, ConfigError, register_architecture
from ..config.spec import LayerRun, LayerSpec, ModelSpec, PartSpec
from ..config.zabunex import ZabunexAttentionLayer, ZabunexConfig

# The design has no longest request; the position tables are made for this many positions
# unless the folder states ``max_positions``.
DEFAULT_MAX_POSITIONS = 1 << 18


def _rope_name(m) -> str:
    return f"rope_{m.rot.dims}_of_{m.dim}_base_{m.rot.base!r}_by_{m.rot.scaling.factor!r}"


def _biased_attention(cfg, m, i) -> PartSpec:
    if m.bias_buckets is None:
        raise ConfigError(
            f"layer {i}: the rows of the bias table are the first dimension of the tensor 'l{i}.mix.rel'; "
            "a configuration that is used without the folder's tensors states them as 'bias_buckets'"
        )
    return PartSpec(
        kind="normed_attention", hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, qk_dim=m.dim,
        v_dim=m.vdim, scale=m.scale, eps=cfg.norm.eps, values_from_keys=True,
        q_temperature=dict(coef=m.q_temp.coef, every=m.q_temp.every),
        distance_bias=dict(buckets=m.bias_buckets, max_distance=m.bias_max), sink=True,
    )


def zabunex_spec(cfg: ZabunexConfig) -> ModelSpec:
    max_positions = cfg.max_positions or DEFAULT_MAX_POSITIONS
    norm = PartSpec(kind="rmsnorm", size=cfg.width, eps=cfg.norm.eps, round_before_weight=False)
    positions, layers = {}, {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(layer, ZabunexAttentionLayer):
            mixer = _biased_attention(cfg, m, i)
        else:
            left, right = m.left, m.right
            name = _rope_name(left)
            positions.setdefault(name, PartSpec(
                kind="rope", head_dim=left.dim, rotary_dim=left.rot.dims, theta=left.rot.base, interleaved=False,
                max_positions=max_positions, scaling=dict(kind="linear", factor=left.rot.scaling.factor),
                angles="float64",
            ))
            mixer = PartSpec(
                kind="sum", names=["left", "right"], scales=[m.left_scale, m.right_scale],
                mixers=[
                    dict(kind="normed_attention", hidden_size=cfg.width, n_heads=left.heads, n_kv_heads=left.kv_heads,
                         qk_dim=left.dim, v_dim=left.vdim, scale=left.scale, eps=cfg.norm.eps, conv_taps=left.conv,
                         position=name, chunk=left.mask.size),
                    dict(kind="state_space", hidden_size=cfg.width, n_heads=right.heads, head_dim=right.vdim,
                         state_size=right.state, groups=right.groups, conv_taps=right.conv,
                         norm_parts=right.norm_groups, eps=cfg.norm.eps),
                ],
            )
        parts = dict(mixer=mixer, mixer_norm=norm)
        if layer.mlp is not None:
            parts["ff"] = PartSpec(kind="dense", hidden_size=cfg.width, intermediate_size=layer.mlp.ff,
                                   activation="relu_squared")
            parts["ff_norm"] = norm
        layers[f"l{i}"] = LayerSpec(arrangement="post_norm", parts=parts)
    return ModelSpec(
        architecture="Zabunex",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_positions=max_positions,
        embedding=PartSpec(kind="embedding", vocab_size=cfg.vocab, size=cfg.width),
        positions=positions,
        layers=layers,
        order=[LayerRun(layer=name) for name in layers],
        final_norm=norm,
        head=PartSpec(kind="linear_head", vocab_size=cfg.vocab, size=cfg.width, tied=False),
    )


_ATTENTION_TENSORS = (("q", "q.weight"), ("k", "k.weight"), ("q.norm", "q_norm.weight"), ("k.norm", "k_norm.weight"),
                      ("rel", "distance_bias.weight"), ("o", "out.weight"))
_LEFT_TENSORS = (("q", "q.weight"), ("k", "k.weight"), ("v", "v.weight"), ("q.norm", "q_norm.weight"),
                 ("k.norm", "k_norm.weight"), ("q.conv", "q_conv.weight"), ("k.conv", "k_conv.weight"),
                 ("v.conv", "v_conv.weight"), ("o", "out.weight"))
_RIGHT_TENSORS = (("in", "in.weight"), ("conv", "conv.weight"), ("conv.b", "conv.bias"), ("dt_bias", "dt_bias"),
                  ("A_log", "A_log"), ("D", "D"), ("norm", "norm.weight"), ("o", "out.weight"))


def zabunex_weight_map(cfg: ZabunexConfig) -> dict[str, str | None]:
    """Tensor name in the folder -> parameter of a part, layer by layer."""
    table = {"embed": "embedding.weight", "final.norm": "final_norm.weight", "head": "head.weight"}
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}.", f"layers.l{i}."
        table[src + "norm1"] = dst + "mixer_norm.weight"
        if isinstance(layer, ZabunexAttentionLayer):
            for theirs, ours in _ATTENTION_TENSORS:
                table[f"{src}mix.{theirs}"] = f"{dst}mixer.{ours}"
        else:
            for theirs, ours in _LEFT_TENSORS:
                table[f"{src}mix.left.{theirs}"] = f"{dst}mixer.left.{ours}"
            for theirs, ours in _RIGHT_TENSORS:
                table[f"{src}mix.right.{theirs}"] = f"{dst}mixer.right.{ours}"
        if layer.mlp is None:
            table[src + "norm2"] = None  # a norm without a reader may be stored all the same
            continue
        table[src + "norm2"] = dst + "ff_norm.weight"
        table[src + "mlp.up"] = dst + "ff.linear_up.weight"
        table[src + "mlp.down"] = dst + "ff.linear_out.weight"
    return table


def zabunex_complete(cfg: ZabunexConfig, shape_of) -> ZabunexConfig:
    """Fills in what the folder's tensors say and the file does not: the rows of every
    attention layer's bias table."""
    layers = []
    for i, layer in enumerate(cfg.layers):
        if isinstance(layer, ZabunexAttentionLayer):
            shape = shape_of(f"l{i}.mix.rel")
            if shape is not None and len(shape) == 2:
                layer = layer.model_copy(update={"mixer": layer.mixer.model_copy(update={"bias_buckets": int(shape[0])})})
        layers.append(layer)
    return cfg.model_copy(update={"layers": layers})


ZABUNEX = register_architecture(
    Architecture(
        name="Zabunex",
        config_cls=ZabunexConfig,
        to_spec=zabunex_spec,
        weight_map=zabunex_weight_map,
        complete_from_tensors=zabunex_complete,
    )
)
