"""Diporax: a decoder whose layers norm what a part returns (``x += scale * norm(part(x))``
with a learned scale per channel), listed one by one in ``config.json``.  The embedding's rows
are normed on their way in.  A layer's mixer is one of three: a softmax attention with biased
projections, short convolutions on q, k and v, a weighted norm per head on q and k, partial
rotation with stretched frequencies, capped scores, values blended with those of the first
such layer, and a gate per head; a latent attention (one normed latent and one shared rotated
key part per token, neighbouring pairs rotated) with a learned sink per head and a gate per
head; or a linear attention with one constant decay per head.  The feed-forward is a mixture
of SiLU-gated experts weighted by the softmax over the chosen logits, with a shared expert
behind a sigmoid gate of its own.  Every layer ends by adding, through a norm, a gated row
of a per-layer part of a second token table.
"""

from __future__ import annotations

import math

from ..config.diporax import DiporaxAttentionLayer, DiporaxConfig, DiporaxLatentLayer
from ..config.registry import Architecture, register_architecture
from ..config.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

# The design has no longest request; the position tables are made for this many positions
# unless the folder states ``max_positions``.
DEFAULT_MAX_POSITIONS = 1 << 18
# What a stretched rotation multiplies cosine and sine by: 1 + this times ln(factor).
ROT_MAGNITUDE_SLOPE = 0.1
# The name under which the first blending attention leaves its values for the later ones.
VALUES_NAME = "first_values"


def _rope(rot, dims: int, head: int, interleaved: bool, max_positions: int) -> tuple[str, PartSpec]:
    s = rot.scaling
    name = f"rope_{dims}_of_{head}_base_{rot.base!r}_{'pairs' if interleaved else 'halves'}"
    scaling, magnitude = None, 1.0
    if s is not None:
        name += f"_by_{s.factor!r}_{s.original}_{s.fast!r}_{s.slow!r}"
        scaling = dict(kind="ramp", factor=s.factor, original_context_len=s.original, fast_turns=s.fast, slow_turns=s.slow)
        magnitude = ROT_MAGNITUDE_SLOPE * math.log(s.factor) + 1.0
    return name, PartSpec(kind="rope", head_dim=head, rotary_dim=dims, theta=rot.base, interleaved=interleaved,
                          max_positions=max_positions, scaling=scaling, magnitude=magnitude, angles="float64")


def diporax_spec(cfg: DiporaxConfig) -> ModelSpec:
    max_positions = cfg.max_positions or DEFAULT_MAX_POSITIONS
    eps = cfg.norm.eps
    scaled_norm = PartSpec(kind="rmsnorm", size=cfg.width, eps=eps, round_before_weight=False, layer_scale=True)
    plain_norm = PartSpec(kind="rmsnorm", size=cfg.width, eps=eps, round_before_weight=False)
    positions, layers = {}, {}
    seen_values = False
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(layer, DiporaxAttentionLayer):
            position = None
            if m.rot is not None:
                position, spec = _rope(m.rot, m.rot.dims, m.dim, False, max_positions)
                positions.setdefault(position, spec)
            mix = None
            if m.v_mix:
                mix = "blend" if seen_values else "first"
                seen_values = True
            mixer = PartSpec(
                kind="capped_attention", hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, qk_dim=m.dim,
                v_dim=m.vdim, scale=m.scale, eps=eps, bias=bool(m.bias), conv_taps=m.conv, position=position,
                softcap=m.softcap, value_mix=mix, value_mix_name=VALUES_NAME,
            )
        elif isinstance(layer, DiporaxLatentLayer):
            position, spec = _rope(m.rot, m.rot_dim, m.rot_dim, True, max_positions)
            positions.setdefault(position, spec)
            mixer = PartSpec(
                kind="latent_attention", hidden_size=cfg.width, n_heads=m.heads, nope_dim=m.dim, rope_dim=m.rot_dim,
                v_dim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=eps, position=position,
                output_gate=True, gate_per_head=True, learned_sink=True, float32_result=True,
            )
        else:
            mixer = PartSpec(kind="decay_attention", hidden_size=cfg.width, n_heads=m.heads, qk_dim=m.dim, v_dim=m.vdim,
                             decay=list(m.decay), eps=eps)
        parts = dict(mixer=mixer, mixer_norm=scaled_norm)
        f = layer.mlp
        if f is not None:
            gate = dict(limit=None, alpha=1.0, up_shift=0.0)  # silu(gate) * up
            parts["ff"] = PartSpec(
                kind="moe", hidden_size=cfg.width, n_experts=f.router.experts, top_k=f.router.top,
                expert=dict(intermediate_size=f.expert.ff, **gate),
                shared=dict(intermediate_size=f.shared.ff, **gate) if f.shared is not None else None,
                shared_gate=f.shared is not None, score="softmax", normalize=True, norm_eps=0.0, float32_result=True,
            )
            parts["ff_norm"] = scaled_norm
        if cfg.token_side is not None:
            d = cfg.token_side.dim
            parts["side"] = PartSpec(kind="token_gated", hidden_size=cfg.width, size=d, col0=i * d)
            parts["side_norm"] = plain_norm
        layers[f"l{i}"] = LayerSpec(arrangement="post_norm", parts=parts)
    side = cfg.token_side.dim * len(cfg.layers) if cfg.token_side is not None else None
    return ModelSpec(
        architecture="Diporax",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_positions=max_positions,
        embedding=PartSpec(kind="embedding", vocab_size=cfg.vocab, size=cfg.width, norm_eps=eps, side_size=side),
        positions=positions,
        layers=layers,
        order=[LayerRun(layer=name) for name in layers],
        final_norm=plain_norm,
        head=PartSpec(kind="linear_head", vocab_size=cfg.vocab, size=cfg.width, tied=False),
    )


_ATTENTION_TENSORS = (("q", "q.weight"), ("k", "k.weight"), ("v", "v.weight"), ("q.norm", "q_norm.weight"),
                      ("k.norm", "k_norm.weight"), ("g", "gate.weight"), ("o", "out.weight"))
_BIAS_TENSORS = (("q.b", "q.bias"), ("k.b", "k.bias"), ("v.b", "v.bias"))
_CONV_TENSORS = (("q.conv", "q_conv.weight"), ("k.conv", "k_conv.weight"), ("v.conv", "v_conv.weight"))
_LATENT_TENSORS = (("dq", "dq.weight"), ("dq.norm", "dq_norm.weight"), ("uq", "uq.weight"), ("dkv", "dkv.weight"),
                   ("dkv.norm", "dkv_norm.weight"), ("uk", "uk.weight"), ("uv", "uv.weight"), ("sink", "sink"),
                   ("g", "gate.weight"), ("o", "out.weight"))
_LIGHTNING_TENSORS = (("q", "q.weight"), ("k", "k.weight"), ("v", "v.weight"), ("g", "gate.weight"),
                      ("norm", "norm.weight"), ("o", "out.weight"))
_EXPERT_TENSORS = (("gate", "gate.weight"), ("up", "up.weight"), ("down", "down.weight"))


def diporax_weight_map(cfg: DiporaxConfig) -> dict[str, str | None]:
    """Tensor name in the folder -> parameter of a part, layer by layer."""
    table = {"embed": "embedding.weight", "embed.norm": "embedding.norm.weight", "final.norm": "final_norm.weight",
             "head": "head.weight"}
    if cfg.token_side is not None:
        table["side.embed"] = "embedding.side.weight"
    seen_values = False
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}.", f"layers.l{i}."
        table[src + "norm1"] = dst + "mixer_norm.weight"
        table[src + "ls1"] = dst + "mixer_norm.scale"
        m = layer.mixer
        if isinstance(layer, DiporaxAttentionLayer):
            names = _ATTENTION_TENSORS + (_BIAS_TENSORS if m.bias else ()) + (_CONV_TENSORS if m.conv is not None else ())
            if m.v_mix:
                # the first blending layer's own number has no reader
                table[src + "mix.vmix"] = dst + "mixer.value_mix.weight" if seen_values else None
                seen_values = True
        elif isinstance(layer, DiporaxLatentLayer):
            names = _LATENT_TENSORS
        else:
            names = _LIGHTNING_TENSORS
        for theirs, ours in names:
            table[f"{src}mix.{theirs}"] = f"{dst}mixer.{ours}"
        f = layer.mlp
        if f is None:
            table[src + "norm2"] = table[src + "ls2"] = None  # stored without a reader, perhaps
        else:
            table[src + "norm2"] = dst + "ff_norm.weight"
            table[src + "ls2"] = dst + "ff_norm.scale"
            table[src + "mlp.router"] = dst + "ff.router.weight"
            for e in range(f.router.experts):
                for theirs, ours in _EXPERT_TENSORS:
                    table[f"{src}mlp.e{e}.{theirs}"] = f"{dst}ff.experts.{e}.{ours}"
            if f.shared is not None:
                for theirs, ours in _EXPERT_TENSORS:
                    table[f"{src}mlp.shared.{theirs}"] = f"{dst}ff.shared.{ours}"
                table[src + "mlp.shared.sg"] = dst + "ff.shared_gate.weight"
        if cfg.token_side is not None:
            table[src + "side.gate"] = dst + "side.gate.weight"
            table[src + "side.proj"] = dst + "side.proj.weight"
            table[src + "side.norm"] = dst + "side_norm.weight"
    return table


def diporax_complete(cfg: DiporaxConfig, shape_of) -> DiporaxConfig:
    """Fills in what the folder's tensors say and the file does not: whether an attention
    layer's projections have biases."""
    layers = []
    for i, layer in enumerate(cfg.layers):
        if isinstance(layer, DiporaxAttentionLayer) and layer.mixer.bias is None:
            has = shape_of(f"l{i}.mix.q.b") is not None
            layer = layer.model_copy(update={"mixer": layer.mixer.model_copy(update={"bias": has})})
        layers.append(layer)
    return cfg.model_copy(update={"layers": layers})


DIPORAX = register_architecture(
    Architecture(
        name="Diporax",
        config_cls=DiporaxConfig,
        to_spec=diporax_spec,
        weight_map=diporax_weight_map,
        complete_from_tensors=diporax_complete,
    )
)
