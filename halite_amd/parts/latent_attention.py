"""Self-attention whose keys and values are projections of one small latent vector per
token, with a rotated key part shared by all heads.

Per token the cache holds the normed latent ``c`` (``kv_rank`` numbers) and the rotated
key part ``r`` (``rope_dim`` numbers), not keys and values of every head.  Head ``h`` has
the key ``[U_k,h c | r]`` and the value ``U_v,h c``; the score of a query ``[q_n | q_r]``
is ``q_n . U_k,h c + q_r . r``.  Since ``q_n . U_k,h c = (U_k,h^T q_n) . c``, the query is
taken into the latent's space once (``kv_rank`` numbers a head) and every head attends
over the *same* rows ``[r | c]``: attention with one key/value head of size
``rope_dim + kv_rank`` whose values are the keys' latent part, which is what the paged
attention kernels serve.  The weighted sum of latents comes back to ``v_dim`` numbers a
head through ``U_v,h`` afterwards.  So a token costs ``rope_dim + kv_rank`` cached numbers
(twice: as a key row and, transposed, as a value row, the layouts those kernels read),
whatever the number of heads.
"""

from __future__ import annotations

import torch
from pydantic import BaseModel, Field, StrictBool, StrictInt

from ..kernels import attention as attention_kernels
from ..kernels import ops
from .base import MIXERS, Mixer, PagedKVNeed, ParamDecl, RotaryPositionEncoding


class LatentAttentionParams(BaseModel):
    hidden_size: StrictInt = Field(gt=0)
    n_heads: StrictInt = Field(gt=0)
    nope_dim: StrictInt = Field(gt=0)
    """Query/key dimensions of a head that are not rotated."""
    rope_dim: StrictInt = Field(ge=0)
    """Rotated query dimensions of a head, and the size of the key part all heads share."""
    v_dim: StrictInt = Field(gt=0)
    q_rank: StrictInt = Field(gt=0)
    kv_rank: StrictInt = Field(gt=0)
    scale: float = Field(gt=0)
    eps: float = Field(gt=0)
    """Of the norms of the two latents."""
    position: str | None = None
    window: StrictInt | None = Field(default=None, gt=0)
    output_gate: StrictBool = False
    """The concatenated heads are multiplied by ``sigmoid(W_g x)`` before the output projection."""
    gate_per_head: StrictBool = False
    """With ``output_gate``: ``W_g`` has one row a head, and a head's result is multiplied by
    one number."""
    learned_sink: StrictBool = False
    """Every head's softmax has one more term in its denominator, ``exp(sink[head])`` with a
    tensor ``sink`` ``[n_heads]``: it has no key and no value and is not scaled."""
    float32_result: StrictBool = False
    """True: without a stream to add into, the output projection's float32 sums come back unrounded."""


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    """``c_q = norm(W_dq x)``, ``q = W_uq c_q`` (per head ``[nope_dim | rope_dim]``);
    ``[c' | r] = W_dkv x``, ``c = norm(c')``; rotation of ``q``'s rotated part and of ``r``;
    causal softmax attention inside ``window`` as described above (optionally with a learned
    sink a head); optional output gate; output projection."""

    Params = LatentAttentionParams
    graph_safe = True
    adds_to_stream = True

    def __init__(self, params, build):
        super().__init__(params, build)
        p = params
        # the size of the one key/value head that the attention kernels see, in steps of 16
        self.head_dim = -(-(p.rope_dim + p.kv_rank) // 16) * 16
        self.position = None
        if p.position is not None:
            if p.position not in build.positions:
                raise ValueError(f"latent attention names position encoding {p.position!r}, which the model does not define")
            self.position = build.positions[p.position]
            if not isinstance(self.position, RotaryPositionEncoding):
                raise ValueError(f"position encoding {p.position!r} is not a RotaryPositionEncoding")
            if self.position.rotary_dim > p.rope_dim:
                raise ValueError("the position encoding rotates more elements than the rotated part has")
        elif p.rope_dim:
            raise ValueError("a rotated part needs a position encoding")

    def param_decls(self):
        p = self.p
        d, h = p.hidden_size, p.n_heads
        decls = {
            "dq.weight": ParamDecl((p.q_rank, d)),
            "dq_norm.weight": ParamDecl((p.q_rank,), init="ones"),
            "uq.weight": ParamDecl((h * (p.nope_dim + p.rope_dim), p.q_rank)),
            "dkv.weight": ParamDecl((p.kv_rank + p.rope_dim, d)),
            "dkv_norm.weight": ParamDecl((p.kv_rank,), init="ones"),
            "uk.weight": ParamDecl((h * p.nope_dim, p.kv_rank)),
            "uv.weight": ParamDecl((h * p.v_dim, p.kv_rank)),
            "out.weight": ParamDecl((d, h * p.v_dim)),
        }
        if p.output_gate:
            decls["gate.weight"] = ParamDecl((h if p.gate_per_head else h * p.v_dim, d))
        if p.learned_sink:
            decls["sink"] = ParamDecl((h,))
        return decls

    def allocate(self, dtypes):
        p = self.p
        dev = self.build.device
        down = ["dq.weight", "dkv.weight"] + (["gate.weight"] if p.output_gate else [])
        if len({dtypes[n] for n in down}) != 1 or dtypes["dq_norm.weight"] != dtypes["dkv_norm.weight"]:
            raise ValueError("the down projections (and the two latent norms) are stored with different element types")
        decls = self.param_decls()
        rows = [decls[n].shape[0] for n in down]
        # one product serves the two down projections and the gate: [dq | dkv | gate] rows
        self.w_down = torch.empty((sum(rows), p.hidden_size), dtype=dtypes["dq.weight"], device=dev)
        out, at = {}, 0
        for n, r in zip(down, rows):
            out[n] = self.w_down[at : at + r]
            at += r
        for n in decls:
            if n not in out:
                t = torch.empty(decls[n].shape, dtype=dtypes[n], device=dev)
                setattr(self, "w_" + n.split(".")[0], t)
                out[n] = t
        return out

    def finalize(self):
        p = self.p
        h = p.n_heads
        # U_k of a head, transposed: the query's unrotated part times this is the query in
        # the latent's space
        self.w_ukt = self.w_uk.view(h, p.nope_dim, p.kv_rank).transpose(1, 2).contiguous()
        self.w_uv3 = self.w_uv.view(h, p.v_dim, p.kv_rank)
        self.rule = None
        if p.learned_sink:
            sinks = self.w_sink.float().contiguous()
            self.rule = ops.ScoreRule(sink=True, sink_values=sinks,
                                      sink_values_log2=(sinks.double() * 1.4426950408889634).float().contiguous())
        self.t_down = self.t_uq = self.t_out = None
        if self.build.tiled_weights and self.w_down.is_cuda:
            tile = lambda w: ops.tile_weight(w) if w.dtype == torch.bfloat16 and w.shape[1] % 8 == 0 else None  # noqa: E731
            self.t_down, self.t_uq, self.t_out = tile(self.w_down), tile(self.w_uq), tile(self.w_out)

    def attention_sizes(self):
        return None  # no (heads, key/value heads, head size) in the sense of the options that name them

    def cache_need(self):
        return PagedKVNeed(1, self.head_dim, self.p.window)

    def prepare(self, ctx, run):
        group = ctx.cache.groups[run.kv.group_id]
        if attention_kernels.mfma_supported(self.build.dtype, self.head_dim, group.page_size):
            ctx.plan_attention(group.group_id, self.p.n_heads, 1, self.p.window or 0, self.head_dim)

    def forward(self, x, ctx, run, add_to=None):
        p = self.p
        kv = run.kv
        group = ctx.group(kv.group_id)
        n, h, D = x.shape[0], p.n_heads, self.head_dim
        qh = p.nope_dim + p.rope_dim
        kv_col0 = p.q_rank
        gate_col0 = p.q_rank + p.kv_rank + p.rope_dim
        a = ops.linear(x, self.w_down, out_dtype=torch.float32, tiled=self.t_down)
        # rows [q of every head | the key row | the value row], each D wide, as the kernels
        # that rotate, append and attend take them: a head is [rotated part | latent | 0]
        packed = torch.empty((n, (h + 2) * D), dtype=x.dtype, device=x.device)
        cq = ops.latent_prep(a, 0, p.q_rank, kv_col0, p.kv_rank, p.rope_dim, D, self.w_dq_norm, self.w_dkv_norm,
                             p.eps, packed, h * D)
        q = ops.linear(cq, self.w_uq, tiled=self.t_uq)
        ops.grouped_gemm(q, self.w_ukt, packed, n_rows=n, x_group_cols=qh, y_group_cols=D, y_col0=p.rope_dim)
        ops.head_cols(q, qh, p.nope_dim, packed, D, 0, p.rope_dim, h,
                      zero_from=p.rope_dim + p.kv_rank, n_zero=D - p.rope_dim - p.kv_rank)
        if self.position is not None:
            cos, sin = self.position.tables(ctx.max_position + 1)
            rot = self.position.rotary_dim
        else:
            cos = sin = ctx.empty_f32
            rot = 0
        ops.rope_append(
            packed, ctx.positions, cos, sin, h, 1 if run.appends else 0, D, rot,
            self.position.interleaved if self.position is not None else False,
            token_seg=ctx.token_seg, block_table=group.block_table,
            k_pages=kv.k, v_pages=kv.v, page_size=group.page_size, tiled=kv.tiled,
        )
        latent = ctx.attention(packed, packed.shape[1], kv, group, h, p.scale, p.window or 0, rule=self.rule)
        heads = torch.empty((n, h * p.v_dim), dtype=x.dtype, device=x.device)
        ops.grouped_gemm(latent, self.w_uv3, heads, n_rows=n, x_group_cols=D, x_col0=p.rope_dim, y_group_cols=p.v_dim,
                         gate=a[:, gate_col0:] if p.output_gate else None, gate_per_group=p.gate_per_head)
        if add_to is not None:
            ops.linear_add(add_to, heads, self.w_out, tiled=self.t_out)
            return None
        return ops.linear(heads, self.w_out, out_dtype=torch.float32 if p.float32_result else None, tiled=self.t_out)
