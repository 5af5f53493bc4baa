"""The generalized delta rule: a recurrence with a matrix state per head.  Every token
decays the state ``S`` (key channel x value channel) per key channel, erases a part of what
lies along its unit key, writes its key and value, and reads with ``r``:

    S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,   o_t = S_t^T r_t,
    w_t = exp(-decay_rate * sigmoid(decay.bias + W_up tanh(W_down x_t))),
    a_t = sigmoid(W_a x_t + a.bias),   u_t = k_t / sqrt(sum(k_t^2) + unit_eps)   (per head),

where both middle terms read the old state.  Every head's ``o`` is divided by its root mean
square, multiplied by a weight and by ``sigmoid(W_gate x)``, and projected out.  Per request
the mixer keeps the state (float32, zero at the start); it has no paged cache.  Decays,
removal rates, unit keys, the state and the norm are float32.
"""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictInt

from ..kernels import ops
from .base import MIXERS, Mixer, ParamDecl, StateNeed


class GeneralDeltaParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    head_dim: StrictInt = Field(gt=0, le=256)
    decay_rank: StrictInt = Field(gt=0, le=1024)
    decay_rate: float = Field(gt=0)
    unit_eps: float = Field(ge=0)
    eps: float = Field(gt=0)


@MIXERS.register("general_delta")
class GeneralDelta(Mixer):
    Params = GeneralDeltaParams
    graph_safe = True

    # the order of the projections in the one product that makes them all
    _PROJECTIONS = ("r", "k", "v", "a", "gate")

    def __init__(self, params, build):
        super().__init__(params, build)
        self.inner = params.n_heads * params.head_dim

    def param_decls(self):
        p = self.p
        d, n = p.hidden_size, self.inner
        decls = {f"{name}.weight": ParamDecl((n, d)) for name in self._PROJECTIONS}
        decls["decay_down.weight"] = ParamDecl((p.decay_rank, d))
        decls["decay_up.weight"] = ParamDecl((n, p.decay_rank))
        decls["decay.bias"] = ParamDecl((n,))
        decls["a.bias"] = ParamDecl((n,))
        decls["norm.weight"] = ParamDecl((n,), init="ones")
        decls["out.weight"] = ParamDecl((d, n))
        return decls

    def allocate(self, dtypes):
        p = self.p
        dev = self.build.device
        names = [f"{name}.weight" for name in self._PROJECTIONS] + ["decay_down.weight"]
        if len({dtypes[n] for n in names}) != 1:
            raise ValueError("the projections of a delta-rule mixer are stored with different element types")
        if len({dtypes["decay_up.weight"], dtypes["decay.bias"], dtypes["a.bias"]}) != 1:
            raise ValueError("decay_up, decay.bias and a.bias are stored with different element types")
        n = self.inner
        # one product for r, k, v, a, the gate and the decay's inner projection
        self.w_in = torch.empty((5 * n + p.decay_rank, p.hidden_size), dtype=dtypes["r.weight"], device=dev)
        out = {f"{name}.weight": self.w_in[i * n : (i + 1) * n] for i, name in enumerate(self._PROJECTIONS)}
        out["decay_down.weight"] = self.w_in[5 * n :]
        for name in ("decay_up.weight", "decay.bias", "a.bias", "norm.weight", "out.weight"):
            t = torch.empty(self.param_decls()[name].shape, dtype=dtypes[name], device=dev)
            setattr(self, "w_" + name.replace(".", "_"), t)
            out[name] = t
        return out

    def finalize(self):
        self.t_in = self.t_out = None
        if self.build.tiled_weights and self.w_in.is_cuda and self.w_in.dtype == torch.bfloat16:
            if self.p.hidden_size % 8 == 0:
                self.t_in = ops.tile_weight(self.w_in)
            if self.inner % 8 == 0 and self.w_out_weight.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.w_out_weight)

    def state_need(self):
        p = self.p
        return {"state": StateNeed((p.n_heads, p.head_dim, p.head_dim))}

    def forward(self, x, ctx, run):
        p = self.p
        n = self.inner
        a = ops.linear(x, self.w_in, out_dtype=torch.float32, tiled=self.t_in)
        r, k, v, a_raw, gate = (a[:, i * n : (i + 1) * n] for i in range(5))
        x1 = a[:, 5 * n :]
        o = ops.delta_rule(r, k, v, a_raw, x1, self.w_decay_up_weight, self.w_decay_bias, self.w_a_bias,
                           run.state["state"], ctx.seg_q_start, ctx.seg_q_len, ctx.token_slot, p.decay_rate, p.unit_eps)
        y = ops.head_norm_gate(o, gate, self.w_norm_weight, p.eps, p.n_heads, x.dtype)
        return ops.linear(y, self.w_out_weight, out_dtype=torch.float32, tiled=self.t_out)
