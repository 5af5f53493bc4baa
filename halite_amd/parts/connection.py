"""Hyper-connections: the residual stream is kept in several copies, and every part has
learned weights for how its input is read from them, how its result is written to each of
them, and how the copies mix among themselves on the way:

    u = sum_s in[s] x_s;  y = part(norm(u));  x_t <- sum_s mix[s, t] x_s + mult * out[t] * y

(all copies at once from the old ones; ``mix`` is indexed [from, to]).  All copies start as
the embedding's output and the model's one stream at the end is their sum.  Without learned
weights (``learned`` false) the part is the plain residual sum ``x <- x + mult * y`` on one
copy.  Copies, sums and the norm that follows a read are float32; the write of one part and
the read and norm of the next are one kernel.
"""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt, model_validator

from ..kernels import ops
from .base import CONNECTIONS, Connection, ParamDecl
from .norm import RMSNorm


class HyperConnectionParams(BaseModel):
    streams: StrictInt = Field(gt=0, le=8)
    mult: float = 1.0
    """What the part's result is multiplied by on its way into the copies."""
    learned: StrictBool = True

    @model_validator(mode="after")
    def _check(self):
        if not self.learned and self.streams != 1:
            raise ValueError("several copies of the stream need learned weights")
        return self


@CONNECTIONS.register("hyper_connection")
class HyperConnection(Connection):
    Params = HyperConnectionParams
    graph_safe = True

    @property
    def copies(self) -> int:
        return self.p.streams

    def param_decls(self):
        if not self.p.learned:
            return {}
        s = self.p.streams
        return {"in": ParamDecl((s,), init="ones"), "out": ParamDecl((s,), init="ones"), "mix": ParamDecl((s, s))}

    def allocate(self, dtypes):
        if len(set(dtypes.values())) > 1:
            raise ValueError("a connection's in, out and mix are stored with different element types")
        dev = self.build.device
        out = {}
        for name, decl in self.param_decls().items():
            t = torch.empty(decl.shape, dtype=dtypes[name], device=dev)
            setattr(self, "w_" + name, t)
            out[name] = t
        return out

    def finalize(self):
        if not self.p.learned:
            dev = self.build.device
            self.w_in = torch.ones(1, dtype=torch.float32, device=dev)
            self.w_out = torch.ones(1, dtype=torch.float32, device=dev)
            self.w_mix = torch.ones((1, 1), dtype=torch.float32, device=dev)

    @staticmethod
    def _write_args(pending):
        if pending is None:
            return {}
        y, link = pending
        if y.dtype != torch.float32:
            y = y.float()
        return dict(y=y, mix=link.w_mix, out=link.w_out, mult=link.p.mult)

    def step(self, x, pending, norm):
        if not isinstance(norm, RMSNorm) or norm.p.round_before_weight:
            raise ValueError("a connection's read is normed by an RMSNorm in the unrounded order")
        return ops.streams_step(x, read=True, inw=self.w_in, norm_weight=norm.weight, offset=norm.p.weight_offset,
                                eps=norm.p.eps, dtype=self.build.dtype, **self._write_args(pending))

    def leave(self, x, pending, rows):
        if pending is not None:
            ops.streams_step(x, **self._write_args(pending))
        return ops.streams_step(x, read=True, rows=rows)
