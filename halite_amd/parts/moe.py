"""A mixture of small gated feed-forward layers with a router, and an optional expert
that every token uses.

The router's logits are a float32 product; a kernel turns them into the chosen experts
and their weights, a second one sorts the (token, choice) pairs by expert on the device,
and two grouped products run all experts at once on the sorted rows: gate and up with the
activation in the epilogue, then down.  A last kernel adds the weighted results into the
float32 stream.  Nothing is read back to the host, so a step's launches depend on its
number of tokens alone.
"""

from __future__ import annotations

import math
from typing import Literal

import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt, model_validator

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamDecl


class ClampedGate(BaseModel):
    """``g = min(W_gate x, limit)``, ``u = clamp(W_up x, -limit, limit)``,
    ``y = g * sigmoid(alpha * g) * (u + up_shift)``.  Without a limit, with ``alpha`` 1 and
    ``up_shift`` 0 that is the plain gate ``silu(W_gate x) * (W_up x)``."""

    intermediate_size: StrictInt = Field(gt=0)
    limit: float | None = Field(gt=0)
    """None: neither product is held to a limit."""
    alpha: float = 1.702
    up_shift: float = 1.0

    @property
    def limit_or_inf(self) -> float:
        return math.inf if self.limit is None else self.limit


class SquaredRelu(BaseModel):
    """An expert without a gate: ``W_down relu(W_up x)^2``."""

    kind: Literal["relu_squared"]
    intermediate_size: StrictInt = Field(gt=0)


class MoEParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_experts: StrictInt = Field(gt=0)
    top_k: StrictInt = Field(gt=0)
    expert: ClampedGate | SquaredRelu
    shared: ClampedGate | None = None
    score: Literal["sigmoid", "softmax"] = "sigmoid"
    normalize: StrictBool = True
    """The chosen scores are divided by their sum (+ ``norm_eps``)."""
    norm_eps: float = 1e-20
    float32_result: StrictBool = False
    """True: without a stream to add into, the float32 sum comes back unrounded."""
    shared_gate: StrictBool = False
    """True: the shared expert's result is multiplied by ``sigmoid(w . x)``, one number a
    token, with a tensor ``shared_gate.weight`` ``[1, hidden_size]`` (float32 arithmetic)."""

    @model_validator(mode="after")
    def _check(self):
        if self.top_k > self.n_experts:
            raise ValueError(f"top_k {self.top_k} of {self.n_experts} experts")
        if self.shared is not None and isinstance(self.expert, SquaredRelu):
            raise ValueError("a shared expert comes with gated experts")
        if self.shared_gate and self.shared is None:
            raise ValueError("a gate for the shared expert without a shared expert")
        return self


@FEED_FORWARDS.register("moe")
class MixtureOfExperts(FeedForward):
    Params = MoEParams
    graph_safe = True
    adds_to_stream = True

    @property
    def gated(self) -> bool:
        return isinstance(self.p.expert, ClampedGate)

    def param_decls(self):
        p = self.p
        d, f = p.hidden_size, p.expert.intermediate_size
        decls = {"router.weight": ParamDecl((p.n_experts, d))}
        for e in range(p.n_experts):
            if self.gated:
                decls[f"experts.{e}.gate.weight"] = ParamDecl((f, d))
            decls[f"experts.{e}.up.weight"] = ParamDecl((f, d))
            decls[f"experts.{e}.down.weight"] = ParamDecl((d, f))
        if p.shared is not None:
            fs = p.shared.intermediate_size
            decls["shared.gate.weight"] = ParamDecl((fs, d))
            decls["shared.up.weight"] = ParamDecl((fs, d))
            decls["shared.down.weight"] = ParamDecl((d, fs))
        if p.shared_gate:
            decls["shared_gate.weight"] = ParamDecl((1, d))
        return decls

    def allocate(self, dtypes):
        p = self.p
        d, f, n, dev = p.hidden_size, p.expert.intermediate_size, p.n_experts, self.build.device
        kinds = {dt for name, dt in dtypes.items() if name not in ("router.weight", "shared_gate.weight")}
        if p.shared_gate and dtypes["shared_gate.weight"] != dtypes["router.weight"]:
            raise ValueError("the router and the shared expert's gate are stored with different element types")
        if len(kinds) != 1:
            raise ValueError("the experts' weights are stored with different element types")
        dt = kinds.pop()
        # all experts in one tensor per projection: the grouped products index them by expert
        self.w_gate = torch.empty((n, f, d), dtype=dt, device=dev) if self.gated else None
        self.w_up = torch.empty((n, f, d), dtype=dt, device=dev)
        self.w_down = torch.empty((n, d, f), dtype=dt, device=dev)
        # the router's rows, and behind them the shared expert's gate: one product for both
        self.w_router = torch.empty((n + (1 if p.shared_gate else 0), d), dtype=dtypes["router.weight"], device=dev)
        out = {"router.weight": self.w_router[:n]}
        if p.shared_gate:
            out["shared_gate.weight"] = self.w_router[n:]
        for e in range(n):
            if self.gated:
                out[f"experts.{e}.gate.weight"] = self.w_gate[e]
            out[f"experts.{e}.up.weight"] = self.w_up[e]
            out[f"experts.{e}.down.weight"] = self.w_down[e]
        if p.shared is not None:
            fs = p.shared.intermediate_size
            # gate and up in one tensor, gate first: one library product serves both for many rows
            self.ws_gate_up = torch.empty((2 * fs, d), dtype=dt, device=dev)
            self.ws_down = torch.empty((d, fs), dtype=dt, device=dev)
            out["shared.gate.weight"], out["shared.up.weight"] = self.ws_gate_up[:fs], self.ws_gate_up[fs:]
            out["shared.down.weight"] = self.ws_down
        return out

    def finalize(self):
        self.t_shared_down = None
        if (self.p.shared is not None and self.build.tiled_weights and self.ws_down.is_cuda
                and self.ws_down.dtype == torch.bfloat16 and self.ws_down.shape[1] % 8 == 0):
            self.t_shared_down = ops.tile_weight(self.ws_down)

    def forward(self, x, ctx, add_to=None):
        p = self.p
        n, d = x.shape
        h = add_to if add_to is not None else torch.empty((n, d), dtype=torch.float32, device=x.device)
        z = ops.linear(x, self.w_router, out_dtype=torch.float32)
        shared_gate = z[:, p.n_experts:] if p.shared_gate else None
        z = z[:, : p.n_experts]
        routing = dict(softmax=p.score == "softmax", normalize=p.normalize, norm_eps=p.norm_eps)
        if n <= ops.ROUTE_SORT_MAX_TOKENS:  # few tokens: one workgroup routes and sorts
            idx, wgt, offsets, tiles, order = ops.moe_route_sort(z, p.top_k, p.n_experts, **routing)
        else:
            idx, wgt = ops.moe_route(z, p.top_k, **routing)
            offsets, tiles, order = ops.moe_sort(idx, p.n_experts)
        pairs = n * p.top_k
        # rows in the sorted order: row i belongs to pair order[i] = token * top_k + choice
        act = torch.empty((pairs, p.expert.intermediate_size), dtype=x.dtype, device=x.device)
        if self.gated:
            ops.grouped_gemm(x, self.w_gate, act, n_rows=pairs, w_up=self.w_up, limit=p.expert.limit_or_inf,
                             alpha=p.expert.alpha, up_shift=p.expert.up_shift, group_offsets=offsets, tile_offsets=tiles, row_src=order, src_div=p.top_k)
        else:
            ops.grouped_gemm(x, self.w_up, act, n_rows=pairs, relu_squared=True,
                             group_offsets=offsets, tile_offsets=tiles, row_src=order, src_div=p.top_k)
        y = torch.empty((pairs, d), dtype=torch.float32, device=x.device)
        ops.grouped_gemm(act, self.w_down, y, n_rows=pairs, group_offsets=offsets, tile_offsets=tiles, row_dst=order)
        if p.shared is not None:
            fs = p.shared.intermediate_size
            if x.dtype == torch.bfloat16 and n <= 16:
                # few rows: the grouped product of one group, activation in its epilogue
                acts = torch.empty((n, fs), dtype=x.dtype, device=x.device)
                ops.grouped_gemm(x, self.ws_gate_up[:fs].view(1, fs, d), acts, n_rows=n, w_up=self.ws_gate_up[fs:].view(1, fs, d),
                                 limit=p.shared.limit_or_inf, alpha=p.shared.alpha, up_shift=p.shared.up_shift)
            else:
                acts = ops.clamped_gate_mul(ops.linear(x, self.ws_gate_up), p.shared.limit_or_inf, p.shared.alpha,
                                            p.shared.up_shift)
            # the shared expert's result rides along with the weighted sum
            extra = ops.linear(acts, self.ws_down, out_dtype=torch.float32, tiled=self.t_shared_down)
        ops.moe_combine(h, y, wgt, extra if p.shared is not None else None, extra_gate=shared_gate,
                        overwrite=add_to is None)
        if add_to is not None:
            return None
        return h if p.float32_result else h.to(x.dtype)
