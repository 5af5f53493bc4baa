"""Typed configuration of the Diporax decoder, read from its own ``config.json`` keys.

Every size and every constant that can differ between two models of the design is a key
of the file and has no default here; a key that the file leaves out switches its mechanism
off (no convolution, no cap on the scores, no blending of values, no stretched frequencies,
no shared expert, no per-layer token input).  Whether an attention's projections carry
biases is not a key of the file: the folder's tensors say it (``complete_from_tensors``);
a configuration that is used without a folder (random weights) states it as ``bias``.
"""

from __future__ import annotations

from typing import Annotated, Literal, Union

from pydantic import BaseModel, ConfigDict, Field, StrictBool, model_validator

from .zabunex import Size, _Keys


class DiporaxNorm(_Keys):
    eps: float = Field(gt=0)


class DiporaxRotScaling(_Keys):
    factor: float = Field(gt=0)
    original: Size = Field(gt=0)
    fast: float = Field(gt=0)
    slow: float = Field(gt=0)


class DiporaxRot(_Keys):
    base: float = Field(gt=1)
    dims: Size = Field(gt=0)
    scaling: DiporaxRotScaling | None = None


class DiporaxAttentionMixer(_Keys):
    heads: Size = Field(gt=0)
    kv_heads: Size = Field(gt=0)
    dim: Size = Field(gt=0)
    vdim: Size = Field(gt=0)
    scale: float = Field(gt=0)
    rot: DiporaxRot | None = None
    conv: Size | None = Field(default=None, gt=0)
    softcap: float | None = Field(default=None, gt=0)
    v_mix: StrictBool = False
    bias: StrictBool | None = None
    """Not a key of the design: the tensors ``mix.q.b`` and their like say it."""

    @model_validator(mode="after")
    def _check(self):
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} kv_heads")
        if self.rot is not None and (self.rot.dims % 2 or self.rot.dims > self.dim):
            raise ValueError(f"rot.dims {self.rot.dims} must be even and at most dim {self.dim}")
        return self


class DiporaxLatentMixer(_Keys):
    heads: Size = Field(gt=0)
    dim: Size = Field(gt=0)
    rot_dim: Size = Field(gt=0)
    vdim: Size = Field(gt=0)
    q_rank: Size = Field(gt=0)
    kv_rank: Size = Field(gt=0)
    scale: float = Field(gt=0)
    rot: DiporaxRot

    @model_validator(mode="after")
    def _check(self):
        if self.rot_dim % 2:
            raise ValueError(f"rot_dim {self.rot_dim} must be even")
        return self


class DiporaxLightningMixer(_Keys):
    heads: Size = Field(gt=0)
    dim: Size = Field(gt=0)
    vdim: Size = Field(gt=0)
    decay: list[float]

    @model_validator(mode="after")
    def _check(self):
        if len(self.decay) != self.heads:
            raise ValueError(f"{len(self.decay)} decays for {self.heads} heads")
        return self


class DiporaxExpert(_Keys):
    ff: Size = Field(gt=0)


class DiporaxRouter(_Keys):
    experts: Size = Field(gt=0)
    top: Size = Field(gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.top > self.experts:
            raise ValueError(f"top {self.top} of {self.experts} experts")
        return self


class DiporaxMoE(_Keys):
    kind: Literal["moe"]
    expert: DiporaxExpert
    router: DiporaxRouter
    shared: DiporaxExpert | None = None


class DiporaxAttentionLayer(_Keys):
    type: Literal["attention"]
    mixer: DiporaxAttentionMixer
    mlp: DiporaxMoE | None = None


class DiporaxLatentLayer(_Keys):
    type: Literal["latent_attention"]
    mixer: DiporaxLatentMixer
    mlp: DiporaxMoE | None = None


class DiporaxLightningLayer(_Keys):
    type: Literal["lightning"]
    mixer: DiporaxLightningMixer
    mlp: DiporaxMoE | None = None


DiporaxLayer = Annotated[Union[DiporaxAttentionLayer, DiporaxLatentLayer, DiporaxLightningLayer],
                         Field(discriminator="type")]


class DiporaxTokenSide(_Keys):
    dim: Size = Field(gt=0)


class DiporaxConfig(BaseModel):
    """``config.json`` of a Diporax folder."""

    model_config = ConfigDict(extra="ignore")

    architecture: Literal["Diporax"]
    vocab: Size = Field(gt=0)
    width: Size = Field(gt=0)
    norm: DiporaxNorm
    layers: list[DiporaxLayer] = Field(min_length=1)
    token_side: DiporaxTokenSide | None = None
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
            layer["mixer"].pop("bias", None)  # the folder's tensors say it
            layer.setdefault("mlp", None)
        return d
