"""Typed configuration of the Zabunex decoder, read from its own ``config.json`` keys.

Every size and every constant that can differ between two models of the design is a key
of the file (or the shape of a tensor) and has no default here.  The number of rows of an
attention layer's bias table is not a key of the file: it is the first dimension of the
layer's ``mix.rel`` tensor and is filled in from the folder's tensors
(``complete_from_tensors``); a configuration that is used without a folder (random
weights) states it as ``bias_buckets``.
"""

from __future__ import annotations

from typing import Annotated, Literal, Union

from pydantic import BaseModel, BeforeValidator, ConfigDict, Field, StrictInt, model_validator


def _whole_number(v):
    """A size that a writer stored as a float without a fraction (64.0) is that integer;
    anything else goes to the strict check as it is."""
    if isinstance(v, float) and v.is_integer():
        return int(v)
    return v


Size = Annotated[StrictInt, BeforeValidator(_whole_number)]


class _Keys(BaseModel):
    # sizes and constants are typed strictly; keys the design does not have are passed over
    model_config = ConfigDict(extra="ignore")


class ZabunexNorm(_Keys):
    eps: float = Field(gt=0)


class ZabunexQueryTemperature(_Keys):
    coef: float
    every: Size = Field(gt=0)


class ZabunexBiasedAttention(_Keys):
    heads: Size = Field(gt=0)
    kv_heads: Size = Field(gt=0)
    dim: Size = Field(gt=0)
    vdim: Size = Field(gt=0)
    scale: float = Field(gt=0)
    bias_max: Size = Field(gt=0)
    q_temp: ZabunexQueryTemperature
    bias_buckets: Size | None = Field(default=None, gt=1)

    @model_validator(mode="after")
    def _check(self):
        if self.vdim != self.dim:
            raise ValueError(f"the values are the keys, so vdim {self.vdim} must equal dim {self.dim}")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} kv_heads")
        return self


class ZabunexRotationScaling(_Keys):
    factor: float = Field(gt=0)


class ZabunexRotation(_Keys):
    base: float = Field(gt=0)
    dims: Size = Field(gt=0)
    scaling: ZabunexRotationScaling


class ZabunexMask(_Keys):
    size: Size = Field(gt=0)


class ZabunexChunkedAttention(_Keys):
    heads: Size = Field(gt=0)
    kv_heads: Size = Field(gt=0)
    dim: Size = Field(gt=0)
    vdim: Size = Field(gt=0)
    scale: float = Field(gt=0)
    conv: Size = Field(gt=0)
    mask: ZabunexMask
    rot: ZabunexRotation

    @model_validator(mode="after")
    def _check(self):
        if self.rot.dims % 2 or self.rot.dims > self.dim:
            raise ValueError(f"rot.dims {self.rot.dims} must be even and at most dim {self.dim}")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} kv_heads")
        return self


class ZabunexStateSpace(_Keys):
    heads: Size = Field(gt=0)
    vdim: Size = Field(gt=0)
    state: Size = Field(gt=0)
    groups: Size = Field(gt=0)
    conv: Size = Field(gt=0)
    norm_groups: Size = Field(gt=0)


class ZabunexParallelMixer(_Keys):
    left: ZabunexChunkedAttention
    right: ZabunexStateSpace
    left_scale: float
    right_scale: float


class ZabunexDense(_Keys):
    kind: Literal["dense"]
    ff: Size = Field(gt=0)


class ZabunexAttentionLayer(_Keys):
    type: Literal["attention"]
    mixer: ZabunexBiasedAttention
    mlp: ZabunexDense | None = None


class ZabunexParallelLayer(_Keys):
    type: Literal["parallel"]
    mixer: ZabunexParallelMixer
    mlp: ZabunexDense | None = None


ZabunexLayer = Annotated[Union[ZabunexAttentionLayer, ZabunexParallelLayer], Field(discriminator="type")]


class ZabunexConfig(BaseModel):
    """``config.json`` of a Zabunex folder."""

    model_config = ConfigDict(extra="ignore")

    architecture: Literal["Zabunex"]
    vocab: Size = Field(gt=0)
    width: Size = Field(gt=0)
    norm: ZabunexNorm
    layers: list[ZabunexLayer] = Field(min_length=1)
    max_positions: Size | None = Field(default=None, gt=0)
    """Not a key of the design (a request may be as long as the cache allows); a folder may
    state it to bound the position tables."""
    stop_token_ids: tuple[int, ...] = ()

    @property
    def architectures(self) -> list[str]:
        return [self.architecture]

    def to_json_dict(self) -> dict:
        d = self.model_dump(exclude_none=True)
        if not self.stop_token_ids:
            d.pop("stop_token_ids")
        for layer in d["layers"]:
            layer["mixer"].pop("bias_buckets", None)  # the tensor's shape says it
            layer.setdefault("mlp", None)
        return d
