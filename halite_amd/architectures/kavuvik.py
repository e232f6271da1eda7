"""Kavuvik: a decoder of parallel blocks.  Every layer adds, to the same rows of the
stream, a latent attention (queries through a latent of their own, keys and values from
one cached latent and a rotated key part shared by the heads, a sliding window, a sigmoid
gate on the heads' output) and a mixture of clamped gated experts with sigmoid routing and
an expert that every token uses; the embedding and the logits carry a multiplier each.
The layers are listed one by one in ``config.json`` and may differ in every size.
"""

from __future__ import annotations

from ..config.kavuvik import KavuvikConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

# The design has no longest request; the position tables are made for this many positions
# unless the folder states ``max_positions``.
DEFAULT_MAX_POSITIONS = 1 << 18
# The multiplier inside the experts' sigmoid is the design's, not the file's.
EXPERT_ALPHA = 1.702
# What is added to the sum of the chosen scores before it divides them.
ROUTER_NORM_EPS = 1e-20


def _rope_name(m) -> str:
    return f"rope_{m.rot.dims}_of_{m.rot_dim + m.kv_rank}_base_{m.rot.base!r}"


def kavuvik_spec(cfg: KavuvikConfig) -> ModelSpec:
    max_positions = cfg.max_positions or DEFAULT_MAX_POSITIONS
    norm = PartSpec(kind="rmsnorm", size=cfg.width, eps=cfg.norm.eps, round_before_weight=False)
    positions, layers = {}, {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        name = _rope_name(m)
        # the rotated vector is the rotated part alone, of which the first rot.dims rotate
        positions.setdefault(name, PartSpec(
            kind="rope", head_dim=m.rot_dim, rotary_dim=m.rot.dims, theta=m.rot.base,
            interleaved=False, max_positions=max_positions,
        ))
        parts = dict(
            mixer_norm=norm,
            mixer=PartSpec(
                kind="latent_attention", hidden_size=cfg.width, n_heads=m.heads, nope_dim=m.dim,
                rope_dim=m.rot_dim, v_dim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale,
                eps=cfg.norm.eps, position=name, window=m.mask.size if m.mask is not None else None,
                output_gate=True,
            ),
        )
        if layer.mlp is not None:
            f = layer.mlp
            gate = lambda e: dict(intermediate_size=e.ff, limit=e.limit, alpha=EXPERT_ALPHA)  # noqa: E731
            parts["ff_norm"] = norm
            parts["ff"] = PartSpec(
                kind="moe", hidden_size=cfg.width, n_experts=f.router.experts, top_k=f.router.top,
                expert=gate(f.expert), shared=gate(f.shared) if f.shared is not None else None,
                score="sigmoid", normalize=True, norm_eps=ROUTER_NORM_EPS,
            )
        layers[f"l{i}"] = LayerSpec(arrangement="parallel", parts=parts)
    return ModelSpec(
        architecture="Kavuvik",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_positions=max_positions,
        embedding=PartSpec(kind="embedding", vocab_size=cfg.vocab, size=cfg.width, scale=cfg.embedding.scale),
        positions=positions,
        layers=layers,
        order=[LayerRun(layer=name) for name in layers],
        final_norm=norm,
        head=PartSpec(kind="linear_head", vocab_size=cfg.vocab, size=cfg.width, tied=False, logit_scale=cfg.logit_scale),
    )


def kavuvik_weight_map(cfg: KavuvikConfig) -> dict[str, str | None]:
    """Tensor name in the folder -> parameter of a part, layer by layer (the layers differ,
    so no pattern stands for all of them)."""
    table = {"embed": "embedding.weight", "final.norm": "final_norm.weight", "head": "head.weight"}
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}.", f"layers.l{i}."
        table[src + "norm1"] = dst + "mixer_norm.weight"
        for theirs, ours in (("dq", "dq.weight"), ("dq.norm", "dq_norm.weight"), ("uq", "uq.weight"),
                             ("dkv", "dkv.weight"), ("dkv.norm", "dkv_norm.weight"), ("uk", "uk.weight"),
                             ("uv", "uv.weight"), ("g", "gate.weight"), ("o", "out.weight")):
            table[f"{src}mix.{theirs}"] = f"{dst}mixer.{ours}"
        if layer.mlp is None:
            table[src + "norm2"] = None  # a norm without a reader may be stored all the same
            continue
        table[src + "norm2"] = dst + "ff_norm.weight"
        table[src + "mlp.router"] = dst + "ff.router.weight"
        for e in range(layer.mlp.router.experts):
            for proj in ("gate", "up", "down"):
                table[f"{src}mlp.e{e}.{proj}"] = f"{dst}ff.experts.{e}.{proj}.weight"
        if layer.mlp.shared is not None:
            for proj in ("gate", "up", "down"):
                table[f"{src}mlp.shared.{proj}"] = f"{dst}ff.shared.{proj}.weight"
    return table


KAVUVIK = register_architecture(
    Architecture(
        name="Kavuvik",
        config_cls=KavuvikConfig,
        to_spec=kavuvik_spec,
        weight_map=kavuvik_weight_map,
    )
)
