"""Typed configuration of the Kavuvik decoder, read from its own ``config.json`` keys.

Every size and every constant that can differ between two models of the design is a key
of the file and has no default here; what may be absent is what has a meaning when it
is: a layer without ``mlp`` has no feed-forward, a mixer without ``mask`` looks back to the
first token, a mixture without ``shared`` has no expert that every token uses.
"""

from __future__ import annotations

from typing import Literal

from pydantic import BaseModel, ConfigDict, Field, StrictInt, model_validator


class _Strict(BaseModel):
    # sizes and constants are typed strictly; keys the design does not have are passed over
    model_config = ConfigDict(extra="ignore")


class KavuvikEmbedding(_Strict):
    scale: float


class KavuvikNorm(_Strict):
    eps: float = Field(gt=0)


class KavuvikRotation(_Strict):
    base: float = Field(gt=0)
    dims: StrictInt = Field(gt=0)


class KavuvikMask(_Strict):
    size: StrictInt = Field(gt=0)


class KavuvikLatentMixer(_Strict):
    heads: StrictInt = Field(gt=0)
    dim: StrictInt = Field(gt=0)
    rot_dim: StrictInt = Field(gt=0)
    vdim: StrictInt = Field(gt=0)
    q_rank: StrictInt = Field(gt=0)
    kv_rank: StrictInt = Field(gt=0)
    scale: float = Field(gt=0)
    rot: KavuvikRotation
    mask: KavuvikMask | None = None

    @model_validator(mode="after")
    def _check(self):
        if self.rot.dims % 2 or self.rot.dims > self.rot_dim:
            raise ValueError(f"rot.dims {self.rot.dims} must be even and at most rot_dim {self.rot_dim}")
        return self


class KavuvikExpert(_Strict):
    ff: StrictInt = Field(gt=0)
    limit: float = Field(gt=0)


class KavuvikRouter(_Strict):
    experts: StrictInt = Field(gt=0)
    top: StrictInt = Field(gt=0)


class KavuvikMoE(_Strict):
    kind: Literal["moe"]
    expert: KavuvikExpert
    router: KavuvikRouter
    shared: KavuvikExpert | None = None

    @model_validator(mode="after")
    def _check(self):
        if self.router.top > self.router.experts:
            raise ValueError(f"router.top {self.router.top} of {self.router.experts} experts")
        return self


class KavuvikLayer(_Strict):
    type: Literal["latent_attention"]
    mixer: KavuvikLatentMixer
    mlp: KavuvikMoE | None = None


class KavuvikConfig(BaseModel):
    """``config.json`` of a Kavuvik folder."""

    model_config = ConfigDict(extra="ignore")

    architecture: Literal["Kavuvik"]
    vocab: StrictInt = Field(gt=0)
    width: StrictInt = Field(gt=0)
    embedding: KavuvikEmbedding
    norm: KavuvikNorm
    layers: list[KavuvikLayer] = Field(min_length=1)
    logit_scale: float
    max_positions: StrictInt | None = Field(default=None, gt=0)
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
        return d
