"""What a layer adds for the token itself: a small projection of the stream, through
``gelu_tanh``, gates the token's row of a table, and a second projection brings the gated
row back to the stream's width:

    y = W_proj (gelu_tanh(W_gate x) * table[token, col0 : col0 + size])

The table belongs to the model's embedding (``EmbeddingParams.side_size``): one table for
the whole model, of which every layer reads a column range of its own.  The result is
float32 (the accumulators of the second projection); a block norms and adds it as it does
for its other parts.
"""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictInt

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamDecl


class TokenGatedParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    size: StrictInt = Field(gt=0)
    """Columns of the table that the part reads, and rows of ``gate.weight``."""
    col0: StrictInt = Field(ge=0)
    """The first of those columns."""


@FEED_FORWARDS.register("token_gated")
class TokenGated(FeedForward):
    Params = TokenGatedParams
    graph_safe = True

    def __init__(self, params, build):
        super().__init__(params, build)
        emb = build.embedding
        side = getattr(getattr(emb, "p", None), "side_size", None)
        if side is None or params.col0 + params.size > side:
            raise ValueError(
                f"a token-gated part reads columns {params.col0}..{params.col0 + params.size} of the embedding's "
                f"side table, which has {side or 'none'}"
            )

    def param_decls(self):
        p = self.p
        return {"gate.weight": ParamDecl((p.size, p.hidden_size)), "proj.weight": ParamDecl((p.hidden_size, p.size))}

    def forward(self, x, ctx):
        p = self.p
        g = ops.linear(x, self.gate_weight, out_dtype=torch.float32)
        gated = ops.token_gate(g, self.build.embedding.side_weight, p.col0, ctx.tokens, x.dtype)
        return ops.linear(gated, self.proj_weight, out_dtype=torch.float32)
