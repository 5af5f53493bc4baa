"""Vepitar: a pre-norm decoder whose layers are listed one by one in ``config.json`` and whose
residual stream may be kept in several copies with learned read, write and mixing weights
per part (hyper-connections).  A layer's mixer is either a generalized delta rule (a
recurrence with a matrix state per head: decay per key channel, erasure along the unit key)
or an attention without rotation and without softmax (short convolutions on q, k and v,
unit norms per head, a sliding window, sigmoid weights with a bias per head, a gate per
head).  The feed-forward is a gated dense layer or a mixture of small ungated experts with
the square of relu.  The norms' weights are stored as their distance from one, and the
logits are made with the embedding table.
"""

from __future__ import annotations

import math

from ..config.registry import Architecture, ConfigError, register_architecture
from ..config.spec import LayerRun, LayerSpec, ModelSpec, PartSpec
from ..config.vepitar import VepitarAttentionLayer, VepitarConfig, VepitarDense

# The design has no longest request and no position tables; the number only bounds what a
# caller may ask for, unless the folder states ``max_positions``.
DEFAULT_MAX_POSITIONS = 1 << 18
# Constants that the design fixes.
DECAY_RATE = math.exp(-0.5)  # a key channel's decay is exp(-DECAY_RATE * sigmoid(.))
UNIT_KEY_EPS = 1e-6  # added to the sum of a key's squares before the root
ROUTER_NORM_EPS = 1e-20  # added to the sum of the chosen scores before it divides them
NORM_WEIGHT_OFFSET = 1.0  # a norm multiplies by this plus its stored weight


def vepitar_spec(cfg: VepitarConfig) -> ModelSpec:
    max_positions = cfg.max_positions or DEFAULT_MAX_POSITIONS
    eps = cfg.norm.eps
    norm = PartSpec(kind="rmsnorm", size=cfg.width, eps=eps, round_before_weight=False, weight_offset=NORM_WEIGHT_OFFSET)
    link = PartSpec(kind="hyper_connection", streams=cfg.streams or 1, learned=cfg.streams is not None,
                    mult=1.0 if cfg.residual_mult is None else cfg.residual_mult)
    layers = {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(layer, VepitarAttentionLayer):
            mixer = PartSpec(
                kind="sigmoid_attention", hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, qk_dim=m.dim,
                v_dim=m.vdim, scale=m.scale, eps=eps, conv_taps=m.conv, window=m.mask.size if m.mask is not None else None,
            )
        else:
            if m.decay_rank is None:
                raise ConfigError(
                    f"layer {i}: the rank of the decay projection is the first dimension of the tensor 'l{i}.mix.w1'; "
                    "a configuration that is used without the folder's tensors states it as 'decay_rank'"
                )
            mixer = PartSpec(kind="general_delta", hidden_size=cfg.width, n_heads=m.heads, head_dim=m.dim,
                             decay_rank=m.decay_rank, decay_rate=DECAY_RATE, unit_eps=UNIT_KEY_EPS, eps=eps)
        parts = dict(mixer_norm=norm, mixer=mixer, mixer_link=link)
        f = layer.mlp
        if f is not None:
            parts["ff_norm"] = norm
            parts["ff_link"] = link
            if isinstance(f, VepitarDense):
                parts["ff"] = PartSpec(kind="gated", hidden_size=cfg.width, intermediate_size=f.ff, activation="silu",
                                       float32_result=True)
            else:
                parts["ff"] = PartSpec(
                    kind="moe", hidden_size=cfg.width, n_experts=f.router.experts, top_k=f.router.top,
                    expert=dict(kind="relu_squared", intermediate_size=f.expert.ff), score="softmax", normalize=True,
                    norm_eps=ROUTER_NORM_EPS, float32_result=True,
                )
        layers[f"l{i}"] = LayerSpec(arrangement="hyper_pre_norm", parts=parts)
    return ModelSpec(
        architecture="Vepitar",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_positions=max_positions,
        embedding=PartSpec(kind="embedding", vocab_size=cfg.vocab, size=cfg.width),
        positions={},
        layers=layers,
        order=[LayerRun(layer=name) for name in layers],
        final_norm=norm,
        head=PartSpec(kind="linear_head", vocab_size=cfg.vocab, size=cfg.width, tied=True),
    )


_DELTA_TENSORS = (("r", "r.weight"), ("k", "k.weight"), ("v", "v.weight"), ("g", "gate.weight"), ("a", "a.weight"),
                  ("a.b", "a.bias"), ("w1", "decay_down.weight"), ("w2", "decay_up.weight"), ("w0", "decay.bias"),
                  ("norm", "norm.weight"), ("o", "out.weight"))
_ATTENTION_TENSORS = (("q", "q.weight"), ("k", "k.weight"), ("v", "v.weight"), ("pb", "score_bias"),
                      ("g", "gate.weight"), ("o", "out.weight"))
_CONV_TENSORS = (("q.conv", "q_conv.weight"), ("k.conv", "k_conv.weight"), ("v.conv", "v_conv.weight"))
_LINK_TENSORS = (("in", "in"), ("out", "out"), ("mix", "mix"))


def vepitar_weight_map(cfg: VepitarConfig) -> dict[str, str | None]:
    """Tensor name in the folder -> parameter of a part, layer by layer."""
    table = {"embed": "embedding.weight", "final.norm": "final_norm.weight"}
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}.", f"layers.l{i}."
        table[src + "norm1"] = dst + "mixer_norm.weight"
        if isinstance(layer, VepitarAttentionLayer):
            names = _ATTENTION_TENSORS + (_CONV_TENSORS if layer.mixer.conv is not None else ())
        else:
            names = _DELTA_TENSORS
        for theirs, ours in names:
            table[f"{src}mix.{theirs}"] = f"{dst}mixer.{ours}"
        if cfg.streams is not None:
            for theirs, ours in _LINK_TENSORS:
                table[f"{src}hc1.{theirs}"] = f"{dst}mixer_link.{ours}"
        f = layer.mlp
        if f is None:
            # a norm and weights without a reader may be stored all the same
            table[src + "norm2"] = None
            for theirs, _ in _LINK_TENSORS:
                table[f"{src}hc2.{theirs}"] = None
            continue
        table[src + "norm2"] = dst + "ff_norm.weight"
        if cfg.streams is not None:
            for theirs, ours in _LINK_TENSORS:
                table[f"{src}hc2.{theirs}"] = f"{dst}ff_link.{ours}"
        if isinstance(f, VepitarDense):
            table[src + "mlp.gate"] = dst + "ff.linear_gate.weight"
            table[src + "mlp.up"] = dst + "ff.linear_proj.weight"
            table[src + "mlp.down"] = dst + "ff.linear_out.weight"
        else:
            table[src + "mlp.router"] = dst + "ff.router.weight"
            for e in range(f.router.experts):
                table[f"{src}mlp.e{e}.up"] = f"{dst}ff.experts.{e}.up.weight"
                table[f"{src}mlp.e{e}.down"] = f"{dst}ff.experts.{e}.down.weight"
    return table


def vepitar_complete(cfg: VepitarConfig, shape_of) -> VepitarConfig:
    """Fills in what the folder's tensors say and the file does not: the rank of every
    delta-rule layer's decay projection."""
    layers = []
    for i, layer in enumerate(cfg.layers):
        if not isinstance(layer, VepitarAttentionLayer):
            shape = shape_of(f"l{i}.mix.w1")
            if shape is not None and len(shape) == 2:
                layer = layer.model_copy(update={"mixer": layer.mixer.model_copy(update={"decay_rank": int(shape[0])})})
        layers.append(layer)
    return cfg.model_copy(update={"layers": layers})


VEPITAR = register_architecture(
    Architecture(
        name="Vepitar",
        config_cls=VepitarConfig,
        to_spec=vepitar_spec,
        weight_map=vepitar_weight_map,
        complete_from_tensors=vepitar_complete,
    )
)
