"""A linear attention with one constant decay per head (the "lightning" form): per head a
state ``S`` of ``qk_dim x v_dim`` numbers, zero when a request starts, that every token decays
and writes to, ``S_t = decay_h S_(t-1) + k_t v_t^T``, and reads from, ``o_t = S_t^T q_t``, with
``q = act(W_q x)``, ``k = act(W_k x)``, ``v = act(W_v x)`` (``act`` SiLU) and no other scale.
The concatenated heads are divided by the root mean square of the whole row, multiplied by a
weight and by ``sigmoid(W_g x)`` element by element, and projected out.

Per request the mixer keeps the state (float32); it has no paged cache.  The recurrence is
the state-space scan's with constant decays and unit step sizes (keys in the place of its
``B``, queries of its ``C``, one group a head), so prompts are cut into chunks that are walked
side by side in the same way.  Decays, state, sums over the state, norm and gate are float32.
"""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictInt, model_validator

from ..kernels import ops
from .base import MIXERS, Mixer, ParamDecl, StateNeed
from .state_space import plan_scan_chunks, scan_arrays


class DecayAttentionParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    qk_dim: StrictInt = Field(gt=0, le=256)
    v_dim: StrictInt = Field(gt=0)
    decay: list[float]
    """One number in (0, 1] a head."""
    eps: float = Field(gt=0)

    @model_validator(mode="after")
    def _check(self):
        if len(self.decay) != self.n_heads:
            raise ValueError(f"{len(self.decay)} decays for {self.n_heads} heads")
        if any(not 0.0 < d <= 1.0 for d in self.decay):
            raise ValueError("a head's decay lies in (0, 1]")
        return self


@MIXERS.register("decay_attention")
class DecayAttention(Mixer):
    Params = DecayAttentionParams
    graph_safe = True

    def __init__(self, params, build):
        super().__init__(params, build)
        p = params
        self.inner = p.n_heads * p.v_dim
        self.n_qk = p.n_heads * p.qk_dim

    def param_decls(self):
        p = self.p
        d = p.hidden_size
        return {
            "v.weight": ParamDecl((self.inner, d)), "k.weight": ParamDecl((self.n_qk, d)),
            "q.weight": ParamDecl((self.n_qk, d)), "gate.weight": ParamDecl((self.inner, d)),
            "norm.weight": ParamDecl((self.inner,), init="ones"), "out.weight": ParamDecl((d, self.inner)),
        }

    def allocate(self, dtypes):
        p = self.p
        dev = self.build.device
        names = ("v", "k", "q", "gate")
        if len({dtypes[f"{n}.weight"] for n in names}) != 1:
            raise ValueError("q, k, v and gate weights are stored with different element types")
        rows = {"v": self.inner, "k": self.n_qk, "q": self.n_qk, "gate": self.inner}
        # one product, its rows in the scan's order: values, keys, queries; then the gate
        self.w_in = torch.empty((sum(rows.values()), p.hidden_size), dtype=dtypes["q.weight"], device=dev)
        out, at = {}, 0
        for n in names:
            out[f"{n}.weight"] = self.w_in[at : at + rows[n]]
            at += rows[n]
        self.w_norm = torch.empty((self.inner,), dtype=dtypes["norm.weight"], device=dev)
        self.w_out = torch.empty((p.hidden_size, self.inner), dtype=dtypes["out.weight"], device=dev)
        out["norm.weight"], out["out.weight"] = self.w_norm, self.w_out
        return out

    def finalize(self):
        p = self.p
        self.decay = torch.tensor(p.decay, dtype=torch.float64).float().to(self.build.device)
        self.t_in = self.t_out = None
        if self.build.tiled_weights and self.w_in.is_cuda and self.w_in.dtype == torch.bfloat16:
            if p.hidden_size % 8 == 0:
                self.t_in = ops.tile_weight(self.w_in)
            if self.inner % 8 == 0 and self.w_out.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.w_out)

    def state_need(self):
        p = self.p
        return {"state": StateNeed((p.n_heads, p.qk_dim, p.v_dim))}

    def prepare(self, ctx, run):
        plan_scan_chunks(ctx)  # (the state-space scan's cut, shared by the step's layers)

    def forward(self, x, ctx, run):
        p = self.p
        n_act = self.inner + 2 * self.n_qk
        a = ops.linear(x, self.w_in, out_dtype=torch.float32, tiled=self.t_in)
        # (SiLU of values, keys and queries where the scan reads them: float32 in either mode)
        y = ops.ssd_scan(a[:, :n_act], None, None, None, None, run.state["state"], ctx.seg_q_start, ctx.seg_q_len,
                         ctx.token_slot, p.n_heads, fixed_decay=self.decay, in_silu=True, **scan_arrays(ctx))
        gated = ops.head_norm_gate(y, a[:, n_act:], self.w_norm, p.eps, 1, x.dtype)
        return ops.linear(gated, self.w_out, out_dtype=torch.float32, tiled=self.t_out)
