"""Self-attention over the paged cache without rotation and without softmax: a visible
key's weight is ``sigmoid(scale * q.k + bias[head])``, and the weights are not normalised
over the keys.

* ``conv_taps``: a short causal convolution over time on every channel of q, k and v, right
  after the projection; its last inputs are per-request state.
* every head of q and k is divided by its own root mean square, and so is every head of v
  (no weights; float32); keys and values are cached so.
* ``window``: a query sees itself and the ``window - 1`` tokens before it.
* every head's result is multiplied by ``sigmoid(W_gate x)`` of that head, one number a head.

The key and value heads may differ in size; pages hold heads of the larger size (in steps
of 16), the rest zero.  The result is float32 (the accumulators of the output projection).
"""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictInt, model_validator

from ..kernels import attention as attention_kernels
from ..kernels import ops
from .base import MIXERS, Mixer, PagedKVNeed, ParamDecl, StateNeed


class SigmoidAttentionParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    n_kv_heads: StrictInt = Field(gt=0)
    qk_dim: StrictInt = Field(gt=0)
    v_dim: StrictInt = Field(gt=0)
    scale: float = Field(gt=0)
    eps: float = Field(gt=0)
    conv_taps: StrictInt | None = Field(default=None, gt=0, le=16)
    window: StrictInt | None = Field(default=None, gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.n_heads} heads are not a multiple of {self.n_kv_heads} kv heads")
        return self


@MIXERS.register("sigmoid_attention")
class SigmoidAttention(Mixer):
    Params = SigmoidAttentionParams
    graph_safe = True

    def __init__(self, params, build):
        super().__init__(params, build)
        p = params
        self.head_dim = -(-max(p.qk_dim, p.v_dim) // 16) * 16
        self.n_q, self.n_k, self.n_v = p.n_heads * p.qk_dim, p.n_kv_heads * p.qk_dim, p.n_kv_heads * p.v_dim

    def attention_sizes(self):
        return self.p.n_heads, self.p.n_kv_heads, self.p.qk_dim

    def param_decls(self):
        p = self.p
        d = p.hidden_size
        decls = {"q.weight": ParamDecl((self.n_q, d)), "k.weight": ParamDecl((self.n_k, d)),
                 "v.weight": ParamDecl((self.n_v, d)), "gate.weight": ParamDecl((p.n_heads, d))}
        if p.conv_taps is not None:
            decls["q_conv.weight"] = ParamDecl((self.n_q, p.conv_taps))
            decls["k_conv.weight"] = ParamDecl((self.n_k, p.conv_taps))
            decls["v_conv.weight"] = ParamDecl((self.n_v, p.conv_taps))
        decls["score_bias"] = ParamDecl((p.n_heads,))
        decls["out.weight"] = ParamDecl((d, p.n_heads * p.v_dim))
        return decls

    def allocate(self, dtypes):
        p = self.p
        dev = self.build.device
        names = ("q", "k", "v", "gate")
        if len({dtypes[f"{n}.weight"] for n in names}) != 1:
            raise ValueError("q, k, v and gate weights are stored with different element types")
        rows = {"q": self.n_q, "k": self.n_k, "v": self.n_v, "gate": p.n_heads}
        # one product for q, k, v and the gate; one convolution over the channels of q, k and v
        self.w_in = torch.empty((sum(rows.values()), p.hidden_size), dtype=dtypes["q.weight"], device=dev)
        self.w_conv = None
        if p.conv_taps is not None:
            if len({dtypes[f"{n}_conv.weight"] for n in ("q", "k", "v")}) != 1:
                raise ValueError("the convolutions of q, k and v are stored with different element types")
            self.w_conv = torch.empty((self.n_q + self.n_k + self.n_v, p.conv_taps), dtype=dtypes["q_conv.weight"], device=dev)
        out, at = {}, 0
        for n in names:
            out[f"{n}.weight"] = self.w_in[at : at + rows[n]]
            if self.w_conv is not None and n != "gate":
                out[f"{n}_conv.weight"] = self.w_conv[at : at + rows[n]]
            at += rows[n]
        self.w_score_bias = torch.empty((p.n_heads,), dtype=dtypes["score_bias"], device=dev)
        self.w_out = torch.empty((p.hidden_size, p.n_heads * p.v_dim), dtype=dtypes["out.weight"], device=dev)
        out["score_bias"], out["out.weight"] = self.w_score_bias, self.w_out
        return out

    def finalize(self):
        p = self.p
        self.t_in = self.t_out = None
        if self.build.tiled_weights and self.w_in.is_cuda and self.w_in.dtype == torch.bfloat16:
            if p.hidden_size % 8 == 0:
                self.t_in = ops.tile_weight(self.w_in)
            if (p.n_heads * p.v_dim) % 8 == 0 and self.w_out.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.w_out)
        # the bias of a head as a table by distance with one entry, which is what the kernels add
        bias = self.w_score_bias.float().view(p.n_heads, 1).contiguous()
        self.rule = ops.ScoreRule(bias=bias, bias_log2=(bias.double() * 1.4426950408889634).float().contiguous(), sigmoid=True)

    def cache_need(self):
        return PagedKVNeed(self.p.n_kv_heads, self.head_dim, self.p.window)

    def state_need(self):
        if self.p.conv_taps is None or self.p.conv_taps == 1:
            return {}
        return {"conv": StateNeed((self.p.conv_taps - 1, self.n_q + self.n_k + self.n_v))}

    def prepare(self, ctx, run):
        group = ctx.cache.groups[run.kv.group_id]
        if attention_kernels.mfma_supported(self.build.dtype, self.head_dim, group.page_size):
            ctx.plan_attention(group.group_id, self.p.n_heads, self.p.n_kv_heads, self.p.window or 0, self.head_dim)

    def forward(self, x, ctx, run):
        p = self.p
        kv = run.kv
        group = ctx.group(kv.group_id)
        D = self.head_dim
        a = ops.linear(x, self.w_in, out_dtype=torch.float32, tiled=self.t_in)
        n_conv = self.n_q + self.n_k + self.n_v
        qkv, gate = a[:, :n_conv], a[:, n_conv:]
        if p.conv_taps is not None and p.conv_taps > 1:
            qkv = ops.short_conv_through(qkv, self.w_conv, None, run.state["conv"], ctx, torch.float32)
        elif p.conv_taps == 1:
            qkv = ops.short_conv(qkv, self.w_conv, None, a.new_zeros((1, 0, n_conv)), ctx.token_seg, ctx.seg_q_start,
                                 ctx.token_slot, torch.float32)
        q, k, v = qkv[:, : self.n_q], qkv[:, self.n_q : self.n_q + self.n_k], qkv[:, self.n_q + self.n_k :]
        pages = dict(positions=ctx.positions, token_seg=ctx.token_seg, block_table=group.block_table, k_pages=kv.k,
                     v_pages=kv.v, page_size=group.page_size, tiled=kv.tiled)
        packed = ops.head_norm_pack(q, k, v, p.eps, p.n_heads, p.n_kv_heads, p.qk_dim, p.v_dim, D, x.dtype,
                                    **(pages if run.appends else {}))
        out = ctx.attention(packed, packed.shape[1], kv, group, p.n_heads, p.scale, p.window or 0, rule=self.rule)
        heads = ops.head_gate_cols(out, D, gate, p.v_dim, p.n_heads)
        return ops.linear(heads, self.w_out, out_dtype=torch.float32, tiled=self.t_out)
