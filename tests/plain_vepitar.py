"""A plain, slow implementation of the Vepitar decoder: one function per mechanism, written
from the design's equations in float64 (or any torch dtype), sharing no code with the
framework.  Tests compare the framework with it.

Notation: ``h`` is a mixer's or feed-forward's input ``[T, width]`` for the ``T`` tokens of
one request, in order; weights are ``[out, in]`` and applied as ``h @ W.T``.  A model is a
dict ``cfg`` with the keys of ``config.json`` and a dict ``w`` of tensors by their names in
the folder.
"""

from __future__ import annotations

import json
import math
import os

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps)`` over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, weight, eps):
    """RMS norm whose stored weight is the distance from one."""
    return rms_unit(x, eps) * (1.0 + weight)


def short_conv(u: torch.Tensor, taps_weight: torch.Tensor) -> torch.Tensor:
    """Causal convolution over time on every channel: ``u`` [T, C], ``taps_weight``
    [C, taps]; the last tap multiplies the token itself, zeros before the first token."""
    T, C = u.shape
    taps = taps_weight.shape[1]
    padded = torch.cat([u.new_zeros((taps - 1, C)), u], 0)
    y = u.new_zeros((T, C))
    for t in range(T):
        for j in range(taps):
            y[t] += taps_weight[:, j] * padded[t + j]  # padded[t + j] is u[t - taps + 1 + j]
    return y


def sigmoid_window_attention(h, w, pre, m, eps):
    """Grouped heads, convolved and unit-normed q, k, v, a sliding window, and sigmoid
    weights that are not normalised over the keys; a gate per head on the result."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[pre + "q"].T, h @ w[pre + "k"].T, h @ w[pre + "v"].T
    if m.get("conv"):
        q, k, v = (short_conv(t, w[pre + n + ".conv"]) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    q = rms_unit(q.view(T, H, D), eps)
    k = rms_unit(k.view(T, G, D), eps)
    v = rms_unit(v.view(T, G, V), eps)
    gate = torch.sigmoid(h @ w[pre + "g"].T)  # [T, H]
    window = (m.get("mask") or {}).get("size")
    out = h.new_zeros((T, H, V))
    for i in range(T):
        lo = 0 if window is None else max(0, i - window + 1)
        for head in range(H):
            g = head // (H // G)
            s = (k[lo : i + 1, g] @ q[i, head]) * m["scale"] + w[pre + "pb"][head]
            out[i, head] = torch.sigmoid(s) @ v[lo : i + 1, g]
    out = out * gate[:, :, None]
    return out.reshape(T, H * V) @ w[pre + "o"].T


def delta_recurrence(r, k, v, decay, a, S, unit_eps=1e-6):
    """One head: ``r``, ``k``, ``v``, ``decay``, ``a`` [T, D]; ``S`` [D, D] (key channel x
    value channel) is the state before the first token.  Both middle terms read the old
    state.  Returns the reads [T, D] and the state after the last token."""
    S = S.clone()
    o = torch.zeros_like(v)
    for t in range(r.shape[0]):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum() + unit_eps)
        S = decay[t][:, None] * S - torch.outer(a[t] * u, u @ S) + torch.outer(k[t], v[t])
        o[t] = S.T @ r[t]
    return o, S


def delta_decay(h, w, pre):
    """Decay per key channel, between exp(-e^(-1/2)) and 1."""
    z = torch.tanh(h @ w[pre + "w1"].T) @ w[pre + "w2"].T + w[pre + "w0"]
    return torch.exp(-math.exp(-0.5) * torch.sigmoid(z))


def general_delta(h, w, pre, m, eps, state=None):
    """The generalized delta rule with its projections, the per-head norm, the gate and the
    output projection.  Returns the result and the states [H, D, D] after the last token."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ w[pre + "r"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, H, D)
    v = (h @ w[pre + "v"].T).view(T, H, D)
    decay = delta_decay(h, w, pre).view(T, H, D)
    a = torch.sigmoid(h @ w[pre + "a"].T + w[pre + "a.b"]).view(T, H, D)
    S = h.new_zeros((H, D, D)) if state is None else state
    o, left = h.new_zeros((T, H, D)), []
    for head in range(H):
        o[:, head], s = delta_recurrence(r[:, head], k[:, head], v[:, head], decay[:, head], a[:, head], S[head])
        left.append(s)
    o = rms_unit(o, eps).reshape(T, H * D) * w[pre + "norm"]
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, torch.stack(left)


def gated_feed_forward(h, w, pre):
    z = h @ w[pre + "gate"].T
    return (z * torch.sigmoid(z) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def routed_experts(h, w, pre, mlp, margins_out=None):
    """Softmax over all experts, the ``top`` largest, their scores over their sum.
    ``margins_out`` receives, per token, how far the last chosen expert's logit lies above
    the first that is not chosen."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = h @ w[pre + "router"].T
    if margins_out is not None and top < E:
        ranked = logits.sort(-1, descending=True).values
        margins_out.append(ranked[:, top - 1] - ranked[:, top])
    scores = torch.softmax(logits, -1)
    chosen_s, chosen = torch.topk(scores, top, dim=-1)
    weights = chosen_s / (chosen_s.sum(-1, keepdim=True) + 1e-20)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen[t, j])
            act = torch.relu(h[t] @ w[f"{pre}e{e}.up"].T) ** 2
            out[t] += weights[t, j] * (act @ w[f"{pre}e{e}.down"].T)
    return out


def feed_forward(h, w, pre, mlp, margins_out=None):
    if mlp["kind"] == "dense":
        return gated_feed_forward(h, w, pre)
    return routed_experts(h, w, pre, mlp, margins_out)


def connection_read(streams, w_in):
    """What a part reads from the copies of the stream: their sum weighted by ``in``."""
    return sum(w_in[s] * x for s, x in enumerate(streams))


def connection_write(streams, y, w_mix, w_out, mult):
    """All copies anew from the old ones: mixed among themselves (``mix`` [from, to]), plus
    the part's result times ``mult * out[to]``."""
    n = len(streams)
    return [sum(w_mix[s, t] * streams[s] for s in range(n)) + mult * w_out[t] * y for t in range(n)]


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out: list | None = None, round_inputs=None,
            margins_out: list | None = None):
    """Logits ``[T, vocab]`` of one request's tokens.  ``layers_out`` receives the stream
    after every layer (the sum of the copies where there are several).  ``round_inputs``: an
    element type that every part's normed input is rounded to on the way (how far the logits
    move then says how sensitive a position is to arithmetic in that type).  ``margins_out``
    receives every routed feed-forward's margins (see ``routed_experts``)."""
    w = {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in w.items()}
    eps = cfg["norm"]["eps"]
    m = cfg.get("residual_mult", 1.0)
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    n_streams = cfg.get("streams")
    streams = None if n_streams is None else [x.clone() for _ in range(n_streams)]
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        for q in (1, 2):
            if q == 2 and layer.get("mlp") is None:
                continue
            if streams is not None:
                hc = f"{pre}hc{q}."
                inp = connection_read(streams, w[hc + "in"])
            else:
                inp = x
            h = norm_around_zero(inp, w[f"{pre}norm{q}"], eps)
            if round_inputs is not None:
                h = h.to(round_inputs).to(dtype)
            if q == 2:
                y = feed_forward(h, w, pre + "mlp.", layer["mlp"], margins_out)
            elif layer["type"] == "attention":
                y = sigmoid_window_attention(h, w, pre + "mix.", layer["mixer"], eps)
            elif layer["type"] == "general_delta":
                y, _ = general_delta(h, w, pre + "mix.", layer["mixer"], eps)
            else:
                raise ValueError(layer["type"])
            if streams is not None:
                streams = connection_write(streams, y, w[hc + "mix"], w[hc + "out"], m)
            else:
                x = x + m * y
        if layers_out is not None:
            layers_out.append(sum(streams) if streams is not None else x.clone())
    if streams is not None:
        x = sum(streams)
    return norm_around_zero(x, w["final.norm"], eps) @ w["embed"].T


def tokens_with_clear_routing(cfg, w, tokens, margin=0.1, seed=0, tries=400):
    """``tokens`` with as few replaced as it takes for no router of the model to choose between
    two experts whose logits lie closer than ``margin``: arithmetic in 16 bits moves a logit by
    a few hundredths, and a choice that turns over makes another model of it.  The first
    token with such a call is drawn anew until there is none (earlier tokens stay as they are:
    the model is causal)."""
    gen = torch.Generator().manual_seed(seed)
    ids = list(tokens)
    for _ in range(tries):
        margins = []
        forward(cfg, w, ids, margins_out=margins)
        if not margins:
            return ids
        close = (torch.stack(margins).min(0).values < margin).nonzero()
        if close.numel() == 0:
            return ids
        ids[int(close[0])] = int(torch.randint(0, cfg["vocab"], (1,), generator=gen))
    raise RuntimeError("no sequence without a close call of a router")


# ---- configurations, tensors and folders for the tests ------------------------------------------


def delta_layer(heads, dim, mlp=None):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


def attention_layer(heads, kv_heads, dim, vdim, scale, conv=None, window=None, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv is not None:
        mixer["conv"] = conv
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def model_cfg(width, vocab, layers, streams=None, residual_mult=None, eps=1e-5):
    cfg = {"architecture": "Vepitar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        cfg["streams"] = streams
    if residual_mult is not None:
        cfg["residual_mult"] = residual_mult
    return cfg


def tensor_shapes(cfg, ranks) -> dict:
    """Name -> shape of every tensor of a folder; ``ranks``: layer -> rank of its decay projection."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,)}
    S = cfg.get("streams")
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        out[pre + "norm1"] = (W,)
        if layer["type"] == "general_delta":
            n = m["heads"] * m["dim"]
            for name in ("r", "k", "v", "g", "a"):
                out[f"{pre}mix.{name}"] = (n, W)
            out[pre + "mix.a.b"] = (n,)
            out[pre + "mix.w1"] = (ranks[i], W)
            out[pre + "mix.w2"] = (n, ranks[i])
            out[pre + "mix.w0"] = (n,)
            out[pre + "mix.norm"] = (n,)
            out[pre + "mix.o"] = (W, n)
        else:
            sizes = {"q": m["heads"] * m["dim"], "k": m["kv_heads"] * m["dim"], "v": m["kv_heads"] * m["vdim"]}
            for name, n in sizes.items():
                out[f"{pre}mix.{name}"] = (n, W)
                if m.get("conv"):
                    out[f"{pre}mix.{name}.conv"] = (n, m["conv"])
            out[pre + "mix.pb"] = (m["heads"],)
            out[pre + "mix.g"] = (m["heads"], W)
            out[pre + "mix.o"] = (W, m["heads"] * m["vdim"])
        links = ["hc1"]
        mlp = layer.get("mlp")
        if mlp is not None:
            links.append("hc2")
            out[pre + "norm2"] = (W,)
            if mlp["kind"] == "dense":
                out[pre + "mlp.gate"], out[pre + "mlp.up"], out[pre + "mlp.down"] = (mlp["ff"], W), (mlp["ff"], W), (W, mlp["ff"])
            else:
                out[pre + "mlp.router"] = (mlp["router"]["experts"], W)
                for e in range(mlp["router"]["experts"]):
                    out[f"{pre}mlp.e{e}.up"], out[f"{pre}mlp.e{e}.down"] = (mlp["expert"]["ff"], W), (W, mlp["expert"]["ff"])
        if S is not None:
            for hc in links:
                out[f"{pre}{hc}.in"], out[f"{pre}{hc}.out"], out[f"{pre}{hc}.mix"] = (S,), (S,), (S, S)
    return out


def random_weights(cfg, ranks, seed, std=0.12, stored=torch.bfloat16):
    """Matrices N(0, std); norm weights around zero (they are stored so), the per-head norm of
    the delta rule around one; convolutions, biases and connections of a size that counts;
    rounded to ``stored`` so that engine and plain model hold the same numbers."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, ranks).items():
        parts = name.split(".")
        last = parts[-1]
        r = lambda scale=1.0: scale * torch.randn(shape, generator=gen)  # noqa: E731
        if name == "embed":
            t = r(0.7)
        elif last == "conv":
            t = r(0.5)
        elif last in ("norm1", "norm2") or name == "final.norm":
            t = r(0.2)
        elif name.endswith("mix.norm"):
            t = 1.0 + r(0.2)
        elif last == "pb":
            t = -3.0 + r(0.5)
        elif last in ("b", "w0"):
            t = r(0.7)
        elif last == "w2":
            t = r(0.6)
        elif len(parts) > 1 and parts[-2] in ("hc1", "hc2"):
            t = (torch.eye(shape[0]) + r(0.3)) if last == "mix" else (0.8 + r(0.3))
        elif last in ("up", "down") and parts[-2][0] == "e":
            t = r(1.5 * std)
        elif last == "router":
            t = r(4 * std)
        else:
            t = r(std)
        out[name] = t.to(stored).float()
    return out


def write_model_folder(folder, cfg, weights, dtype=torch.bfloat16):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


# two copies of the stream; both kinds of mixer and of feed-forward; key and value heads of one size
VEP_A = model_cfg(64, 331, [
    delta_layer(4, 16, dense(96)),
    attention_layer(4, 2, 16, 16, 0.3, conv=4, window=24, mlp=moe(8, 2, 32)),
    delta_layer(4, 16, moe(8, 2, 32)),
], streams=2, residual_mult=0.7)
VEP_A_RANKS = {0: 8, 2: 8}
# three copies and no multiplier; the attention first and without a feed-forward; a window
# shorter than a page; every expert chosen, and one of three; an attention without convolution
# and without window; value heads larger and smaller than the keys'; one head of 48 channels
VEP_B = model_cfg(48, 257, [
    attention_layer(6, 3, 8, 24, 0.5, conv=2, window=7),
    delta_layer(2, 24, moe(5, 5, 24)),
    attention_layer(2, 2, 24, 8, 0.25, mlp=dense(40)),
    delta_layer(1, 48, moe(3, 1, 36)),
], streams=3)
VEP_B_RANKS = {1: 5, 3: 3}
# one stream and the plain residual sum; sizes that are multiples of nothing; five taps; a window
# one longer than two pages of 16
VEP_C = model_cfg(40, 203, [
    delta_layer(5, 8, dense(52)),
    attention_layer(5, 1, 12, 20, 0.2, conv=5, window=33, mlp=moe(6, 3, 20)),
    delta_layer(2, 20),
], eps=1e-6)
VEP_C_RANKS = {0: 6, 2: 2}
