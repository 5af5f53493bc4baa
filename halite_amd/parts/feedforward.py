"""The gated feed-forward (src/halite/transformers/feedforward.py:175-225)."""

from __future__ import annotations

import torch
from typing import Literal

from pydantic import BaseModel, Field, StrictBool, StrictInt, field_validator

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamDecl


class GatedParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    intermediate_size: StrictInt = Field(gt=0)
    activation: str = "silu"
    float32_result: StrictBool = False
    """True: the last product's float32 sums come back unrounded (for an arrangement that
    adds them into the float32 stream itself)."""

    @field_validator("activation")
    @classmethod
    def _known(cls, v):
        if v != "silu":
            raise ValueError(f"activation {v!r}: only 'silu' has a kernel")
        return v


@FEED_FORWARDS.register("gated")
class GatedFeedForward(FeedForward):
    """``linear_out(linear_proj(x) * silu(linear_gate(x)))`` without biases
    (feedforward.py:204-212).  Gate and up weights live in one tensor
    ``[2F, d]`` (gate first) so that one product serves both; the activation and
    the multiply are float32 on the accumulators or on the product's output."""

    Params = GatedParams
    graph_safe = True
    takes_normed_rows = True
    folds_next_norm = True

    def param_decls(self):
        f, d = self.p.intermediate_size, self.p.hidden_size
        return {
            "linear_gate.weight": ParamDecl((f, d)),
            "linear_proj.weight": ParamDecl((f, d)),
            "linear_out.weight": ParamDecl((d, f)),
        }

    def allocate(self, dtypes):
        f, d = self.p.intermediate_size, self.p.hidden_size
        dev = self.build.device
        if dtypes["linear_gate.weight"] != dtypes["linear_proj.weight"]:
            raise ValueError("gate and up weights are stored with different element types")
        self.w_gate_up = torch.empty((2 * f, d), dtype=dtypes["linear_gate.weight"], device=dev)
        self.w_out = torch.empty((d, f), dtype=dtypes["linear_out.weight"], device=dev)
        return {
            "linear_gate.weight": self.w_gate_up[:f],
            "linear_proj.weight": self.w_gate_up[f:],
            "linear_out.weight": self.w_out,
        }

    def finalize(self):
        self.t_gate = self.t_up = self.t_out = None
        f = self.p.intermediate_size
        if self.build.tiled_weights and self.w_gate_up.is_cuda:
            if self.w_gate_up.dtype == torch.bfloat16:
                self.t_gate = ops.tile_weight(self.w_gate_up[:f])
                self.t_up = ops.tile_weight(self.w_gate_up[f:])
            if self.w_out.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.w_out)

    def forward(self, x, ctx, then=None):
        f = self.p.intermediate_size
        w = self.w_gate_up
        if self.p.float32_result:
            return self._forward_float32_result(x)
        # The gated product with SiLU·mul in its epilogue beats the library product and a
        # kernel for SiLU·mul up to 16 rows, and at 17 to 32 rows on matrices of up to 64 M
        # elements (measured in captured graphs: 50 against 56 us at 14336 x 4096, 23 against
        # 25 at 8192 x 3072, 202 against 179 at 28672 x 8192).
        m, d = x.shape
        small = (self.t_gate is not None and x.dtype == torch.bfloat16 and d % 8 == 0
                 and (m <= ops.SKINNY_ROWS or (m <= ops.FUSED_ROWS and f * d <= ops.GATED_MID_ELEMENTS)))
        if isinstance(x, ops.NormedRows):
            if small:
                act = ops.gemm_bf16_skinny_norm(x, self.t_gate, (f, d), w_up_tiled=self.t_up)
                return ops.linear(act, self.w_out, tiled=self.t_out, next_norm=then)
            x = x.materialize()
        if small:
            act = ops.gemm_bf16_skinny(x, self.t_gate, w_up=self.t_up, tiled_shape=(f, d))
            return ops.linear(act, self.w_out, tiled=self.t_out, next_norm=then)
        fused = (
            w.dtype == torch.bfloat16
            and x.dtype == torch.bfloat16
            and ops.skinny_pays(x.shape[0], f, x.shape[1], False)
            and x.shape[1] % 8 == 0
            and (f * x.shape[1]) % 8 == 0
        )
        if fused:
            act = ops.gemm_bf16_skinny(x, w[:f], w_up=w[f:])
        else:
            act = ops.silu_mul(ops.linear(x, w))
        return ops.linear(act, self.w_out, tiled=self.t_out, next_norm=then)


    def _forward_float32_result(self, x):
        f = self.p.intermediate_size
        m, d = x.shape
        if self.t_gate is not None and x.dtype == torch.bfloat16 and d % 8 == 0 and m <= ops.SKINNY_ROWS:
            act = ops.gemm_bf16_skinny(x, self.t_gate, w_up=self.t_up, tiled_shape=(f, d))
        else:
            act = ops.silu_mul(ops.linear(x, self.w_gate_up))
        return ops.linear(act, self.w_out, out_dtype=torch.float32, tiled=self.t_out)


class DenseParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    intermediate_size: StrictInt = Field(gt=0)
    activation: Literal["relu_squared"] = "relu_squared"


@FEED_FORWARDS.register("dense")
class DenseFeedForward(FeedForward):
    """``linear_out(act(linear_up(x)))`` without biases and without a gate; ``act`` is the
    square of relu.  The result is float32 (the accumulators of the second product as they
    are), for an arrangement that norms or adds it in float32."""

    Params = DenseParams
    graph_safe = True

    def param_decls(self):
        f, d = self.p.intermediate_size, self.p.hidden_size
        return {"linear_up.weight": ParamDecl((f, d)), "linear_out.weight": ParamDecl((d, f))}

    def finalize(self):
        self.t_up = self.t_out = None
        if self.build.tiled_weights and self.linear_up_weight.is_cuda and self.linear_up_weight.dtype == torch.bfloat16:
            if self.p.hidden_size % 8 == 0:
                self.t_up = ops.tile_weight(self.linear_up_weight)
            if self.p.intermediate_size % 8 == 0 and self.linear_out_weight.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.linear_out_weight)

    def forward(self, x, ctx, then=None):
        m, d = x.shape
        if self.t_up is not None and x.dtype == torch.bfloat16 and m <= ops.SKINNY_ROWS and d % 8 == 0:
            # few rows: the activation is the product's epilogue
            act = ops.gemm_bf16_skinny(x, self.t_up, tiled_shape=tuple(self.linear_up_weight.shape), relu_squared=True)
        else:
            act = ops.relu_squared(ops.linear(x, self.linear_up_weight, tiled=self.t_up))
        return ops.linear(act, self.linear_out_weight, out_dtype=torch.float32, tiled=self.t_out)
