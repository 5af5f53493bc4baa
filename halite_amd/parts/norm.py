"""RMSNorm (src/halite/nn/normalization.py:13-57)."""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt, model_validator

from ..kernels import ops
from .base import NORMS, Norm, ParamDecl


class RMSNormParams(BaseModel):
    size: StrictInt = Field(gt=0)
    eps: float = Field(gt=0)
    round_before_weight: StrictBool = True
    """True: the normalised value is rounded to the activation type before the weight
    multiplies it (the reference's order).  False: ``x * rstd * w`` in float32 and one
    rounding at the end."""
    weight_offset: float = 0.0
    """The stored weight is the multiplier's distance from this: the norm multiplies by
    ``weight_offset + weight`` (float32; only in the unrounded order)."""

    layer_scale: StrictBool = False
    """True: a second tensor ``scale`` of the norm's size multiplies the result element by
    element (a learned scale on what a part adds to the stream); the two are multiplied once,
    in float32, when the weights are loaded (only in the unrounded order)."""

    @model_validator(mode="after")
    def _check(self):
        if self.weight_offset != 0.0 and self.round_before_weight:
            raise ValueError("a weight stored as a distance is added up in float32: round_before_weight must be false")
        if self.layer_scale and (self.round_before_weight or self.weight_offset != 0.0):
            raise ValueError("a layer scale comes with the unrounded order and a plain weight")
        return self


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """``weight * (x * rsqrt(mean(x^2) + eps))``: statistics and scaling in float32,
    the normalised value rounded to the activation type before the weight
    multiplies it (normalization.py:48-55).  The residual add that precedes the
    norm in a block (src/halite/transformers/block.py:56-74) is fused in."""

    Params = RMSNormParams
    graph_safe = True

    def param_decls(self):
        decls = {"weight": ParamDecl((self.p.size,), init="ones")}
        if self.p.layer_scale:
            decls["scale"] = ParamDecl((self.p.size,), init="ones")
        return decls

    def finalize(self):
        # what multiplies the normalised rows: the weight, or weight * scale in float32 (exact
        # for two 16-bit factors)
        self.multiplier = self.weight.float() * self.scale.float() if self.p.layer_scale else self.weight

    def forward(self, h, delta=None, rows=None):
        if self.p.layer_scale:
            if delta is not None:
                ops.residual_add(h, delta)
            return ops.rmsnorm_exact(h, self.multiplier, self.p.eps, self.build.dtype, rows=rows)
        if not self.p.round_before_weight:
            if delta is not None:
                ops.residual_add(h, delta)
            if self.p.weight_offset != 0.0:
                return ops.streams_step(h.view(1, *h.shape), read=True, norm_weight=self.weight, offset=self.p.weight_offset,
                                        eps=self.p.eps, dtype=self.build.dtype, rows=rows)
            return ops.rmsnorm_exact(h, self.weight, self.p.eps, self.build.dtype, rows=rows)
        if isinstance(delta, ops.NormedRows):
            # the product before has added its result into h and prepared these rows
            if delta.weight is not self.weight or rows is not None:
                raise ValueError("rows were prepared for another norm")
            return delta
        return ops.rmsnorm(h, self.weight, self.p.eps, self.build.dtype, delta=delta, rows=rows)

    def foldable(self, h):
        if self.build.dtype != torch.bfloat16 or not h.is_cuda or not self.p.round_before_weight:
            return None
        return ops.NextNorm(h, self.weight, self.p.eps)
