"""Typed configuration of the Vepitar decoder, read from its own ``config.json`` keys.

Every size and every constant that can differ between two models of the design is a key
of the file (or the shape of a tensor) and has no default here; a key that the file leaves
out switches its mechanism off (no convolution, no window, one copy of the stream, a
residual multiplier of one).  The rank of a delta-rule layer's decay projection is not a
key of the file: it is the first dimension of the layer's ``mix.w1`` tensor and is filled in
from the folder's tensors (``complete_from_tensors``); a configuration that is used without
a folder (random weights) states it as ``decay_rank``.
"""

from __future__ import annotations

from typing import Annotated, Literal, Union

from pydantic import BaseModel, ConfigDict, Field, model_validator

from .zabunex import Size, _Keys


class VepitarNorm(_Keys):
    eps: float = Field(gt=0)


class VepitarMask(_Keys):
    size: Size = Field(gt=0)


class VepitarDeltaMixer(_Keys):
    heads: Size = Field(gt=0)
    dim: Size = Field(gt=0)
    decay_rank: Size | None = Field(default=None, gt=0)


class VepitarAttentionMixer(_Keys):
    heads: Size = Field(gt=0)
    kv_heads: Size = Field(gt=0)
    dim: Size = Field(gt=0)
    vdim: Size = Field(gt=0)
    scale: float = Field(gt=0)
    conv: Size | None = Field(default=None, gt=0)
    mask: VepitarMask | None = None

    @model_validator(mode="after")
    def _check(self):
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} kv_heads")
        return self


class VepitarDense(_Keys):
    kind: Literal["dense"]
    ff: Size = Field(gt=0)


class VepitarExpert(_Keys):
    ff: Size = Field(gt=0)


class VepitarRouter(_Keys):
    experts: Size = Field(gt=0)
    top: Size = Field(gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.top > self.experts:
            raise ValueError(f"top {self.top} of {self.experts} experts")
        return self


class VepitarMoE(_Keys):
    kind: Literal["moe"]
    expert: VepitarExpert
    router: VepitarRouter


VepitarMlp = Annotated[Union[VepitarDense, VepitarMoE], Field(discriminator="kind")]


class VepitarDeltaLayer(_Keys):
    type: Literal["general_delta"]
    mixer: VepitarDeltaMixer
    mlp: VepitarMlp | None = None


class VepitarAttentionLayer(_Keys):
    type: Literal["attention"]
    mixer: VepitarAttentionMixer
    mlp: VepitarMlp | None = None


VepitarLayer = Annotated[Union[VepitarDeltaLayer, VepitarAttentionLayer], Field(discriminator="type")]


class VepitarConfig(BaseModel):
    """``config.json`` of a Vepitar folder."""

    model_config = ConfigDict(extra="ignore")

    architecture: Literal["Vepitar"]
    vocab: Size = Field(gt=0)
    width: Size = Field(gt=0)
    norm: VepitarNorm
    layers: list[VepitarLayer] = Field(min_length=1)
    residual_mult: float | None = None
    """What a part's result is multiplied by on its way into the stream (absent: one)."""
    streams: Size | None = Field(default=None, gt=0, le=8)
    """Copies of the residual stream with learned read, write and mixing weights per part
    (absent: one stream and the plain residual sum)."""
    max_positions: Size | None = Field(default=None, gt=0)
    """Not a key of the design (a request may be as long as the cache allows)."""
    stop_token_ids: tuple[int, ...] = ()

    @property
    def architectures(self) -> list[str]:
        return [self.architecture]

    def to_json_dict(self) -> dict:
        d = self.model_dump(exclude_none=True)
        if not self.stop_token_ids:
            d.pop("stop_token_ids")
        for layer in d["layers"]:
            layer["mixer"].pop("decay_rank", None)  # the tensor's shape says it
            layer.setdefault("mlp", None)
        return d
