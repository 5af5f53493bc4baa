"""A selective state-space mixer with a scalar decay per head (the "state-space duality"
form): per head a state ``S`` of ``state_size x head_dim`` numbers that every token decays
and writes to, ``S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T``, and reads from,
``y_t = S_t^T C_t + D x_t``, with ``dt_t = softplus(dt_raw_t + dt_bias)``.

One projection gives ``[z | x | B | C | dt_raw]``; ``x``, ``B`` and ``C`` pass a short causal
convolution with bias and SiLU; ``B`` and ``C`` are shared by the heads of a group; the
heads' results are gated by ``silu(z)``, normed in ``norm_parts`` equal parts of the row and
projected out.  Per request the mixer keeps the state (float32) and the convolution's last
inputs; it has no paged cache.  Decays, step sizes, state, gate and norm are float32.
"""

from __future__ import annotations

import numpy as np
import torch
from pydantic import BaseModel, Field, StrictInt, model_validator

from ..kernels import ops
from .base import MIXERS, Mixer, ParamDecl, StateNeed


# Tokens of a chunk of the recurrence where a step's longest segment has at least two of them.
SCAN_CHUNK = 64


def plan_scan_chunks(ctx) -> None:
    """Long segments are cut into chunks that are walked side by side; the cut depends on
    the segments' token counts alone and is shared by every layer of the step that scans
    (``scan_arrays`` gives a layer the arrays, if the step has them)."""
    lens = ctx.seg_q_len_host
    if ctx.static is not None or len(lens) == 0 or int(lens.max()) < 2 * SCAN_CHUNK:
        return
    per_seg = -(-lens.astype(np.int64) // SCAN_CHUNK)
    first = np.concatenate(([0], np.cumsum(per_seg)[:-1]))

    def chunks():
        seg = np.repeat(np.arange(len(lens)), per_seg)
        k = np.arange(int(per_seg.sum())) - first[seg]
        t0 = ctx.seg_q_start_host[seg] + k * SCAN_CHUNK
        n = np.minimum(SCAN_CHUNK, lens[seg] - k * SCAN_CHUNK)
        return np.stack((t0, n, seg, np.zeros_like(seg)), axis=1)

    ctx.add_array(f"scan_chunks_{SCAN_CHUNK}", chunks)
    ctx.add_array(f"scan_seg_chunks_{SCAN_CHUNK}", lambda: np.stack((first, per_seg), axis=1))


def scan_arrays(ctx) -> dict:
    """``chunks`` and ``seg_chunks`` for ``ops.ssd_scan`` (None where the step is not cut)."""
    cut = ctx.has_array(f"scan_chunks_{SCAN_CHUNK}")
    return dict(chunks=ctx.array(f"scan_chunks_{SCAN_CHUNK}") if cut else None,
                seg_chunks=ctx.array(f"scan_seg_chunks_{SCAN_CHUNK}") if cut else None)


class StateSpaceParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    head_dim: StrictInt = Field(gt=0)
    state_size: StrictInt = Field(gt=0, le=256)
    groups: StrictInt = Field(gt=0)
    conv_taps: StrictInt = Field(gt=0, le=16)
    norm_parts: StrictInt = Field(gt=0)
    eps: float = Field(gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.n_heads % self.groups:
            raise ValueError(f"{self.n_heads} heads are not a multiple of {self.groups} groups")
        if (self.n_heads * self.head_dim) % self.norm_parts:
            raise ValueError(f"{self.n_heads * self.head_dim} channels do not split into {self.norm_parts} equal parts")
        return self


@MIXERS.register("state_space")
class StateSpace(Mixer):
    Params = StateSpaceParams
    graph_safe = True

    def __init__(self, params, build):
        super().__init__(params, build)
        p = params
        self.inner = p.n_heads * p.head_dim
        self.n_bc = p.groups * p.state_size
        self.conv_channels = self.inner + 2 * self.n_bc

    def param_decls(self):
        p = self.p
        return {
            "in.weight": ParamDecl((2 * self.inner + 2 * self.n_bc + p.n_heads, p.hidden_size)),
            "conv.weight": ParamDecl((self.conv_channels, p.conv_taps)),
            "conv.bias": ParamDecl((self.conv_channels,)),
            "dt_bias": ParamDecl((p.n_heads,)),
            "A_log": ParamDecl((p.n_heads,)),
            "D": ParamDecl((p.n_heads,), init="ones"),
            "norm.weight": ParamDecl((self.inner,), init="ones"),
            "out.weight": ParamDecl((p.hidden_size, self.inner)),
        }

    def allocate(self, dtypes):
        if dtypes["conv.weight"] != dtypes["conv.bias"]:
            raise ValueError("the convolution's weight and bias are stored with different element types")
        if len({dtypes["dt_bias"], dtypes["A_log"], dtypes["D"]}) != 1:
            raise ValueError("dt_bias, A_log and D are stored with different element types")
        return super().allocate(dtypes)

    def finalize(self):
        self.t_in = self.t_out = None
        if self.build.tiled_weights and self.in_weight.is_cuda and self.in_weight.dtype == torch.bfloat16:
            if self.p.hidden_size % 8 == 0:
                self.t_in = ops.tile_weight(self.in_weight)
            if self.inner % 8 == 0 and self.out_weight.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.out_weight)

    def state_need(self):
        p = self.p
        need = {"state": StateNeed((p.n_heads, p.state_size, p.head_dim))}
        if p.conv_taps > 1:
            need["conv"] = StateNeed((p.conv_taps - 1, self.conv_channels))
        return need

    def prepare(self, ctx, run):
        plan_scan_chunks(ctx)

    def forward(self, x, ctx, run):
        p = self.p
        inner = self.inner
        a = ops.linear(x, self.in_weight, out_dtype=torch.float32, tiled=self.t_in)
        z = a[:, :inner]
        u = a[:, inner : inner + self.conv_channels]
        dt_raw = a[:, inner + self.conv_channels :]
        conv_state = run.state["conv"] if p.conv_taps > 1 else a.new_zeros((1, 0, self.conv_channels))
        xbc = ops.short_conv_through(u, self.conv_weight, self.conv_bias, conv_state, ctx, x.dtype, silu=True)
        y = ops.ssd_scan(xbc, dt_raw, self.dt_bias, self.A_log, self.D, run.state["state"], ctx.seg_q_start,
                         ctx.seg_q_len, ctx.token_slot, p.groups, **scan_arrays(ctx))
        gated = ops.gated_part_norm(y, z, self.norm_weight, p.eps, p.norm_parts, x.dtype)
        return ops.linear(gated, self.out_weight, out_dtype=torch.float32, tiled=self.t_out)
