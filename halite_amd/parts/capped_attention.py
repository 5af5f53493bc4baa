"""Softmax self-attention over the paged cache with grouped heads and these pieces, each a
parameter:

* ``bias``: q, k and v projections with a bias each, added in the projection.
* ``conv_taps``: a short causal convolution over time on every channel of q, k and v, right
  after the projection (and its bias); its last inputs are per-request state, zeros before a
  request's first token.
* every head of q and k is divided by its own root mean square and multiplied by a weight of
  the head's size that all heads share (float32), before the rotation.
* ``position``: a rotary encoding of the leading entries of every query and key head.
* ``softcap``: the scaled score ``s`` becomes ``softcap * tanh(s / softcap)``.
* ``value_mix``: ``"first"``: the layer's values (as they are cached) are left for later layers of
  the same step under ``value_mix_name``; ``"blend"``: the layer's values become
  ``(1 - lambda) v + lambda v_first`` with the learned number ``value_mix.weight`` and the
  values that a ``"first"`` layer left for the same tokens; the blended values are cached.
* ``window``: a query sees itself and the ``window - 1`` tokens before it.
* every head's result is multiplied by ``sigmoid(W_gate x)`` of that head, one number a head.

The key and value heads may differ in size; pages hold heads of the larger size (in steps
of 16), the rest zero.  The result is float32 (the accumulators of the output projection).
"""

from __future__ import annotations

from typing import Literal

import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt, model_validator

from ..kernels import attention as attention_kernels
from ..kernels import ops
from .base import MIXERS, Mixer, PagedKVNeed, ParamDecl, RotaryPositionEncoding, StateNeed


class CappedAttentionParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    n_kv_heads: StrictInt = Field(gt=0)
    qk_dim: StrictInt = Field(gt=0)
    v_dim: StrictInt = Field(gt=0)
    scale: float = Field(gt=0)
    eps: float = Field(gt=0)
    bias: StrictBool = False
    conv_taps: StrictInt | None = Field(default=None, gt=0, le=16)
    position: str | None = None
    softcap: float | None = Field(default=None, gt=0)
    value_mix: Literal["first", "blend"] | None = None
    value_mix_name: str = "values"
    window: StrictInt | None = Field(default=None, gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.n_heads} heads are not a multiple of {self.n_kv_heads} kv heads")
        return self


@MIXERS.register("capped_attention")
class CappedAttention(Mixer):
    Params = CappedAttentionParams
    graph_safe = True

    def __init__(self, params, build):
        super().__init__(params, build)
        p = params
        self.head_dim = -(-max(p.qk_dim, p.v_dim) // 16) * 16
        self.n_q, self.n_k, self.n_v = p.n_heads * p.qk_dim, p.n_kv_heads * p.qk_dim, p.n_kv_heads * p.v_dim
        self.n_conv = self.n_q + self.n_k + self.n_v
        self.position = None
        if p.position is not None:
            if p.position not in build.positions:
                raise ValueError(f"attention names position encoding {p.position!r}, which the model does not define")
            self.position = build.positions[p.position]
            if not isinstance(self.position, RotaryPositionEncoding):
                raise ValueError(f"position encoding {p.position!r} is not a RotaryPositionEncoding")
            if self.position.rotary_dim > p.qk_dim:
                raise ValueError("the position encoding rotates more elements than a head has")

    def attention_sizes(self):
        return self.p.n_heads, self.p.n_kv_heads, self.p.qk_dim

    def param_decls(self):
        p = self.p
        d = p.hidden_size
        decls = {"q.weight": ParamDecl((self.n_q, d)), "k.weight": ParamDecl((self.n_k, d)),
                 "v.weight": ParamDecl((self.n_v, d)), "gate.weight": ParamDecl((p.n_heads, d))}
        if p.bias:
            decls.update({"q.bias": ParamDecl((self.n_q,)), "k.bias": ParamDecl((self.n_k,)),
                          "v.bias": ParamDecl((self.n_v,))})
        if p.conv_taps is not None:
            decls["q_conv.weight"] = ParamDecl((self.n_q, p.conv_taps))
            decls["k_conv.weight"] = ParamDecl((self.n_k, p.conv_taps))
            decls["v_conv.weight"] = ParamDecl((self.n_v, p.conv_taps))
        decls["q_norm.weight"] = ParamDecl((p.qk_dim,), init="ones")
        decls["k_norm.weight"] = ParamDecl((p.qk_dim,), init="ones")
        if p.value_mix == "blend":
            decls["value_mix.weight"] = ParamDecl(())
        decls["out.weight"] = ParamDecl((d, p.n_heads * p.v_dim))
        return decls

    def allocate(self, dtypes):
        p = self.p
        dev = self.build.device
        names = ("q", "k", "v", "gate")
        if len({dtypes[f"{n}.weight"] for n in names}) != 1:
            raise ValueError("q, k, v and gate weights are stored with different element types")
        if dtypes["q_norm.weight"] != dtypes["k_norm.weight"]:
            raise ValueError("the norms of q and k are stored with different element types")
        rows = {"q": self.n_q, "k": self.n_k, "v": self.n_v, "gate": p.n_heads}
        # one product for q, k, v and the gate; one bias row and one convolution over the
        # channels of q, k and v
        self.w_in = torch.empty((sum(rows.values()), p.hidden_size), dtype=dtypes["q.weight"], device=dev)
        self.w_conv = self.w_bias = None
        if p.conv_taps is not None:
            if len({dtypes[f"{n}_conv.weight"] for n in ("q", "k", "v")}) != 1:
                raise ValueError("the convolutions of q, k and v are stored with different element types")
            self.w_conv = torch.empty((self.n_conv, p.conv_taps), dtype=dtypes["q_conv.weight"], device=dev)
        if p.bias:
            if len({dtypes[f"{n}.bias"] for n in ("q", "k", "v")}) != 1:
                raise ValueError("the biases of q, k and v are stored with different element types")
            self.w_bias = torch.empty((self.n_conv,), dtype=dtypes["q.bias"], device=dev)
        out, at = {}, 0
        for n in names:
            out[f"{n}.weight"] = self.w_in[at : at + rows[n]]
            if n != "gate":
                if self.w_conv is not None:
                    out[f"{n}_conv.weight"] = self.w_conv[at : at + rows[n]]
                if self.w_bias is not None:
                    out[f"{n}.bias"] = self.w_bias[at : at + rows[n]]
            at += rows[n]
        decls = self.param_decls()
        for name in decls:
            if name not in out:
                t = torch.empty(decls[name].shape, dtype=dtypes[name], device=dev)
                setattr(self, "w_" + name.split(".")[0], t)
                out[name] = t
        return out

    def finalize(self):
        p = self.p
        self.t_in = self.t_out = None
        if self.build.tiled_weights and self.w_in.is_cuda and self.w_in.dtype == torch.bfloat16:
            if p.hidden_size % 8 == 0:
                self.t_in = ops.tile_weight(self.w_in)
            if (p.n_heads * p.v_dim) % 8 == 0 and self.w_out.dtype == torch.bfloat16:
                self.t_out = ops.tile_weight(self.w_out)
        self.rule = ops.ScoreRule(softcap=p.softcap) if p.softcap is not None else None
        # the blend's learned number is a constant once the weights are loaded
        self.blend = float(self.w_value_mix.float().cpu()) if p.value_mix == "blend" else 0.0

    def cache_need(self):
        return PagedKVNeed(self.p.n_kv_heads, self.head_dim, self.p.window)

    def state_need(self):
        if self.p.conv_taps is None or self.p.conv_taps == 1:
            return {}
        return {"conv": StateNeed((self.p.conv_taps - 1, self.n_conv))}

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
        qkv, gate = a[:, : self.n_conv], a[:, self.n_conv :]
        # (the biases go into the convolution's reads; without a convolution a pass of their own adds them)
        if p.conv_taps is not None and p.conv_taps > 1:
            qkv = ops.short_conv_through(qkv, self.w_conv, None, run.state["conv"], ctx, torch.float32, in_bias=self.w_bias)
        elif p.conv_taps == 1:
            qkv = ops.short_conv(qkv, self.w_conv, None, a.new_zeros((1, 0, self.n_conv)), ctx.token_seg, ctx.seg_q_start,
                                 ctx.token_slot, torch.float32, in_bias=self.w_bias)
        elif self.w_bias is not None:
            ops.bias_rows_(qkv, self.w_bias)
        q, k, v = qkv[:, : self.n_q], qkv[:, self.n_q : self.n_q + self.n_k], qkv[:, self.n_q + self.n_k :]
        other = None
        if p.value_mix is not None:
            left = ctx.__dict__.setdefault("values_left", {})
            if p.value_mix == "first":
                left[p.value_mix_name] = v  # (float32; kept alive for the step by this reference)
            else:
                other = left.get(p.value_mix_name)
                if other is None or other.shape != v.shape:
                    raise ValueError(f"no layer before this one left values {p.value_mix_name!r} of this layer's shape to blend with")
        pages = dict(token_seg=ctx.token_seg, block_table=group.block_table, k_pages=kv.k, v_pages=kv.v,
                     page_size=group.page_size, tiled=kv.tiled)
        appends_here = self.position is None and run.appends
        packed = ops.head_norm_pack(q, k, v, p.eps, p.n_heads, p.n_kv_heads, p.qk_dim, p.v_dim, D, x.dtype,
                                    w_q=self.w_q_norm, w_k=self.w_k_norm, norm_v=False, v_other=other, v_mix=self.blend,
                                    **(dict(positions=ctx.positions, **pages) if appends_here else {}))
        if self.position is not None:
            cos, sin = self.position.tables(ctx.max_position + 1)
            ops.rope_append(packed, ctx.positions, cos, sin, p.n_heads, p.n_kv_heads if run.appends else 0, D,
                            self.position.rotary_dim, self.position.interleaved, **pages)
        out = ctx.attention(packed, packed.shape[1], kv, group, p.n_heads, p.scale, p.window or 0, rule=self.rule)
        heads = ops.head_gate_cols(out, D, gate, p.v_dim, p.n_heads)
        return ops.linear(heads, self.w_out, out_dtype=torch.float32, tiled=self.t_out)
