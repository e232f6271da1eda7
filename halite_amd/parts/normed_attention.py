"""Self-attention over the paged cache whose queries and keys are normed over the whole
projection, with pieces that a design may switch on one by one.

* ``q`` and ``k`` are divided by the root mean square of their whole row (all heads at
  once) and multiplied by a weight of that size (float32 arithmetic).
* ``values_from_keys``: there is no value projection; the values are the keys as they were
  projected, before their norm.
* ``conv_taps``: a short causal convolution over time on every channel of q, k and v, right
  after the projection; its last inputs are per-request state.
* ``position``: a rotary encoding of the leading entries of every query and key head.
* ``q_temperature``: queries are multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``.
* ``distance_bias``: a learned table ``[rows, heads]`` indexed by a bucket of the distance
  between query and key is added to the scaled score.
* ``window`` / ``chunk``: how far back a query sees, and whether only inside its own chunk
  of positions.
* ``sink``: the softmax's denominator has one more term of score 0.

The key and value heads may differ in size; pages hold heads of the larger size (in steps
of 16), the rest zero.  The result is float32 (the accumulators of the output projection).
"""

from __future__ import annotations

import math

import numpy as np
import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt, model_validator

from ..kernels import attention as attention_kernels
from ..kernels import ops
from .base import MIXERS, Mixer, PagedKVNeed, ParamDecl, RotaryPositionEncoding, StateNeed


class QueryTemperature(BaseModel):
    coef: float
    every: StrictInt = Field(gt=0)


class DistanceBias(BaseModel):
    buckets: StrictInt = Field(gt=1)
    """Rows of the table: the first half is one distance each, the second half spaced evenly
    in the logarithm of the distance up to ``max_distance``; further keys use the last row."""
    max_distance: StrictInt = Field(gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.max_distance <= self.buckets // 2:
            raise ValueError(f"max_distance {self.max_distance} must exceed half of the {self.buckets} buckets")
        return self


def distance_buckets(buckets: int, max_distance: int) -> np.ndarray:
    """Row of the bias table for every distance ``0 .. max_distance`` (beyond: the last)."""
    half = buckets // 2
    n = np.arange(max_distance + 1, dtype=np.int64)
    ratio = np.log(np.maximum(n, 1).astype(np.float64) / half) / np.log(max_distance / half)
    far = half + np.floor(ratio * (buckets - half)).astype(np.int64)
    return np.where(n < half, n, np.minimum(buckets - 1, far))


class NormedAttentionParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    n_kv_heads: StrictInt = Field(gt=0)
    qk_dim: StrictInt = Field(gt=0)
    v_dim: StrictInt = Field(gt=0)
    scale: float = Field(gt=0)
    eps: float = Field(gt=0)
    values_from_keys: StrictBool = False
    conv_taps: StrictInt | None = Field(default=None, gt=0, le=16)
    position: str | None = None
    q_temperature: QueryTemperature | None = None
    distance_bias: DistanceBias | None = None
    window: StrictInt | None = Field(default=None, gt=0)
    chunk: StrictInt | None = Field(default=None, gt=0)
    sink: StrictBool = False

    @model_validator(mode="after")
    def _check(self):
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.n_heads} heads are not a multiple of {self.n_kv_heads} kv heads")
        if self.values_from_keys and self.v_dim != self.qk_dim:
            raise ValueError(f"values that are the keys have their size: v_dim {self.v_dim}, qk_dim {self.qk_dim}")
        return self


@MIXERS.register("normed_attention")
class NormedAttention(Mixer):
    Params = NormedAttentionParams
    graph_safe = True

    def __init__(self, params, build):
        super().__init__(params, build)
        p = params
        self.head_dim = -(-max(p.qk_dim, p.v_dim) // 16) * 16
        self.n_q, self.n_k = p.n_heads * p.qk_dim, p.n_kv_heads * p.qk_dim
        self.n_v = 0 if p.values_from_keys else p.n_kv_heads * p.v_dim
        self.position = None
        if p.position is not None:
            if p.position not in build.positions:
                raise ValueError(f"attention names position encoding {p.position!r}, which the model does not define")
            self.position = build.positions[p.position]
            if not isinstance(self.position, RotaryPositionEncoding):
                raise ValueError(f"position encoding {p.position!r} is not a RotaryPositionEncoding")
            if self.position.rotary_dim > p.qk_dim:
                raise ValueError("the position encoding rotates more elements than a head has")
        self.bias_table = None

    def param_decls(self):
        p = self.p
        d = p.hidden_size
        decls = {"q.weight": ParamDecl((self.n_q, d)), "k.weight": ParamDecl((self.n_k, d))}
        if not p.values_from_keys:
            decls["v.weight"] = ParamDecl((self.n_v, d))
        decls["q_norm.weight"] = ParamDecl((self.n_q,), init="ones")
        decls["k_norm.weight"] = ParamDecl((self.n_k,), init="ones")
        if p.conv_taps is not None:
            decls["q_conv.weight"] = ParamDecl((self.n_q, p.conv_taps))
            decls["k_conv.weight"] = ParamDecl((self.n_k, p.conv_taps))
            if not p.values_from_keys:
                decls["v_conv.weight"] = ParamDecl((self.n_v, p.conv_taps))
        if p.distance_bias is not None:
            decls["distance_bias.weight"] = ParamDecl((p.distance_bias.buckets, p.n_heads))
        decls["out.weight"] = ParamDecl((d, p.n_heads * p.v_dim))
        return decls

    def allocate(self, dtypes):
        p = self.p
        dev = self.build.device
        projections = ["q", "k"] + ([] if p.values_from_keys else ["v"])
        if len({dtypes[f"{n}.weight"] for n in projections}) != 1:
            raise ValueError("q, k and v weights are stored with different element types")
        if dtypes["q_norm.weight"] != dtypes["k_norm.weight"]:
            raise ValueError("the norms of q and k are stored with different element types")
        rows = {"q": self.n_q, "k": self.n_k, "v": self.n_v}
        total = sum(rows[n] for n in projections)
        # one product for q, k and v; one convolution over all their channels
        self.w_qkv = torch.empty((total, p.hidden_size), dtype=dtypes["q.weight"], device=dev)
        self.w_conv = None
        if p.conv_taps is not None:
            if len({dtypes[f"{n}_conv.weight"] for n in projections}) != 1:
                raise ValueError("the convolutions of q, k and v are stored with different element types")
            self.w_conv = torch.empty((total, p.conv_taps), dtype=dtypes["q_conv.weight"], device=dev)
        out, at = {}, 0
        for n in projections:
            out[f"{n}.weight"] = self.w_qkv[at : at + rows[n]]
            if self.w_conv is not None:
                out[f"{n}_conv.weight"] = self.w_conv[at : at + rows[n]]
            at += rows[n]
        decls = self.param_decls()
        for name in decls:
            if name not in out:
                t = torch.empty(decls[name].shape, dtype=dtypes[name], device=dev)
                setattr(self, "w_" + name.split(".")[0], t)
                out[name] = t
        return out

    def finalize(self):
        p = self.p
        self.t_qkv = self.t_out = None
        if self.build.tiled_weights and self.w_qkv.is_cuda and self.w_qkv.dtype == torch.bfloat16:
            if p.hidden_size % 8 == 0:
                self.t_qkv = ops.tile_weight(self.w_qkv)
            if (p.n_heads * p.v_dim) % 8 == 0 and self.w_out.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.w_out)
        if p.distance_bias is not None:
            # the table by distance, [heads, max_distance + 1] float32: what the kernels add
            rows = torch.from_numpy(distance_buckets(p.distance_bias.buckets, p.distance_bias.max_distance))
            table = self.w_distance_bias.float()[rows.to(self.w_distance_bias.device)]
            self.bias_table = table.t().contiguous()
        self.rule = ops.ScoreRule(
            chunk=p.chunk or 0, bias=self.bias_table, sink=p.sink,
            bias_log2=None if self.bias_table is None else (self.bias_table.double() * math.log2(math.e)).float().contiguous(),
        )

    def cache_need(self):
        p = self.p
        return PagedKVNeed(p.n_kv_heads, self.head_dim, p.window, p.chunk)

    def prepare(self, ctx, run):
        group = ctx.cache.groups[run.kv.group_id]
        if attention_kernels.mfma_supported(self.build.dtype, self.head_dim, group.page_size):
            ctx.plan_attention(group.group_id, self.p.n_heads, self.p.n_kv_heads, self.p.window or 0, self.head_dim,
                               chunk=self.p.chunk or 0)

    def state_need(self):
        if self.p.conv_taps is None or self.p.conv_taps == 1:
            return {}
        return {"conv": StateNeed((self.p.conv_taps - 1, self.w_rows()))}

    def w_rows(self) -> int:
        return self.n_q + self.n_k + self.n_v

    def forward(self, x, ctx, run):
        p = self.p
        kv = run.kv
        group = ctx.group(kv.group_id)
        n, D = x.shape[0], self.head_dim
        a = ops.linear(x, self.w_qkv, out_dtype=torch.float32, tiled=self.t_qkv)
        if p.conv_taps is not None and p.conv_taps > 1:
            a = ops.short_conv_through(a, self.w_conv, None, run.state["conv"], ctx, torch.float32)
        elif p.conv_taps == 1:
            a = ops.short_conv(a, self.w_conv, None, a.new_zeros((1, 0, a.shape[1])), ctx.token_seg, ctx.seg_q_start,
                               ctx.token_slot, torch.float32)
        q, k = a[:, : self.n_q], a[:, self.n_q : self.n_q + self.n_k]
        v = None if p.values_from_keys else a[:, self.n_q + self.n_k :]
        temp = p.q_temperature
        # without a rotation the kernel that norms and packs appends to the pages itself
        appends_here = self.position is None and run.appends
        pages = dict(token_seg=ctx.token_seg, block_table=group.block_table, k_pages=kv.k, v_pages=kv.v,
                     page_size=group.page_size, tiled=kv.tiled)
        packed = ops.qk_norm_pack(
            q, k, v, self.w_q_norm, self.w_k_norm, p.eps, p.n_heads, p.n_kv_heads, p.qk_dim, p.v_dim, D, x.dtype,
            positions=ctx.positions, temp_coef=temp.coef if temp else 0.0, temp_every=temp.every if temp else 0,
            **(pages if appends_here else {}),
        )
        if self.position is not None:
            cos, sin = self.position.tables(ctx.max_position + 1)
            ops.rope_append(packed, ctx.positions, cos, sin, p.n_heads, p.n_kv_heads if run.appends else 0, D,
                            self.position.rotary_dim, self.position.interleaved, **pages)
        out = ctx.attention(packed, packed.shape[1], kv, group, p.n_heads, p.scale, p.window or 0, rule=self.rule)
        if D != p.v_dim:
            heads = torch.empty((n, p.n_heads * p.v_dim), dtype=out.dtype, device=out.device)
            ops.head_cols(out, D, 0, heads, p.v_dim, 0, p.v_dim, p.n_heads)
            out = heads
        return ops.linear(out, self.w_out, out_dtype=torch.float32, tiled=self.t_out)
