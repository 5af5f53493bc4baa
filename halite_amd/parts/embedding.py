"""Token embedding and output head (src/halite/transformers/embedding.py:7-51;
src/halite/transformers/feedforward.py:72-114)."""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Embedding, Head, ParamDecl


class EmbeddingParams(BaseModel):
    vocab_size: StrictInt = Field(gt=0)
    size: StrictInt = Field(gt=0)
    scale: float = 1.0
    """Every row is multiplied by this on its way into the stream (in float32)."""
    norm_eps: float | None = Field(default=None, gt=0)
    """With a value: a tensor ``norm.weight`` of the rows' size, and every row enters the
    stream as ``x / sqrt(mean(x^2) + norm_eps) * weight`` (float32)."""
    side_size: StrictInt | None = Field(default=None, gt=0)
    """With a value: a second table ``side.weight`` ``[vocab_size, side_size]`` of which parts of
    the layers read column ranges by token (``BuildContext.embedding.side_weight``)."""


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Embedding):
    """Row lookup (embedding.py:36-44) into the float32 residual stream, times ``scale``
    (1 in the reference's models)."""

    Params = EmbeddingParams
    graph_safe = True

    def param_decls(self):
        decls = {"weight": ParamDecl((self.p.vocab_size, self.p.size))}
        if self.p.norm_eps is not None:
            decls["norm.weight"] = ParamDecl((self.p.size,), init="ones")
        if self.p.side_size is not None:
            decls["side.weight"] = ParamDecl((self.p.vocab_size, self.p.side_size))
        return decls

    def forward(self, tokens, out=None):
        if self.p.norm_eps is None:
            return ops.embedding(tokens, self.weight, out=out, scale=self.p.scale)
        x = ops.rmsnorm_exact(ops.embedding(tokens, self.weight, scale=self.p.scale), self.norm_weight, self.p.norm_eps,
                              torch.float32)
        if out is None:
            return x
        out.copy_(x)
        return out


class LinearHeadParams(BaseModel):
    vocab_size: StrictInt = Field(gt=0)
    size: StrictInt = Field(gt=0)
    tied: StrictBool = False
    logit_scale: float = 1.0
    """The float32 logits are multiplied by this."""


@HEADS.register("linear_head")
class LinearHead(Head):
    """Bias-free projection to the vocabulary with float32 logits
    (src/halite/transformers/infer/postprocessor.py:45-57).  When ``tied`` the
    weight is the embedding's table itself
    (src/halite/transformers/transformer.py:59-61), bound by the model builder."""

    Params = LinearHeadParams
    graph_safe = True

    def param_decls(self):
        if self.p.tied:
            return {}
        return {"weight": ParamDecl((self.p.vocab_size, self.p.size))}

    def bind(self, embedding):
        if self.p.tied:
            self.weight = embedding.weight

    def finalize(self):
        self.t_weight = None
        if self.build.tiled_weights and self.weight.dtype == torch.bfloat16 and self.weight.is_cuda:
            self.t_weight = ops.tile_weight(self.weight)

    def forward(self, x):
        return ops.scale_(ops.linear(x, self.weight, out_dtype=torch.float32, tiled=self.t_weight), self.p.logit_scale)
