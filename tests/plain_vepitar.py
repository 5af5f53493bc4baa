"""A plain, slow implementation of the Vepitar decoder: one function per mechanism, written
from the design's equations in float64 (or any torch dtype), sharing no code with the
framework.  Tests compare the framework with it.

Notation: ``h`` is a mixer's or feed-forward's input ``[T, width]`` for the ``T`` tokens of
one request, in order; weights are ``[out, in]`` and applied as ``h @ W.T``.  A model is a
dict ``cfg`` with the keys of ``config.json`` and a dict ``w`` of tensors by their names in
the folder.
"""

from __future__ import annotations

import math

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


def general_delta(h, w, pre, m, eps, state=None):
    """The generalized delta rule: per head a state ``S`` [dim, dim] (key channel x value
    channel) that every token decays per key channel, partly erases along its unit key and
    writes to.  Returns the result and the state after the last token."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ w[pre + "r"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, H, D)
    v = (h @ w[pre + "v"].T).view(T, H, D)
    lora = torch.tanh(h @ w[pre + "w1"].T) @ w[pre + "w2"].T + w[pre + "w0"]
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(lora)).view(T, H, D)
    a = torch.sigmoid(h @ w[pre + "a"].T + w[pre + "a.b"]).view(T, H, D)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = h.new_zeros((H, D, D)) if state is None else state.clone()
    o = h.new_zeros((T, H, D))
    for t in range(T):
        for head in range(H):
            old = S[head]
            erased = torch.outer(a[t, head] * u[t, head], u[t, head] @ old)
            S[head] = decay[t, head][:, None] * old - erased + torch.outer(k[t, head], v[t, head])
            o[t, head] = S[head].T @ r[t, head]
    o = rms_unit(o, eps).reshape(T, H * D) * w[pre + "norm"]
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, S


def gated_feed_forward(h, w, pre):
    z = h @ w[pre + "gate"].T
    return (z * torch.sigmoid(z) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def routed_experts(h, w, pre, mlp):
    """Softmax over all experts, the ``top`` largest, their scores over their sum."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    scores = torch.softmax(h @ w[pre + "router"].T, -1)
    chosen_s, chosen = torch.topk(scores, top, dim=-1)
    weights = chosen_s / (chosen_s.sum(-1, keepdim=True) + 1e-20)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen[t, j])
            act = torch.relu(h[t] @ w[f"{pre}e{e}.up"].T) ** 2
            out[t] += weights[t, j] * (act @ w[f"{pre}e{e}.down"].T)
    return out


def feed_forward(h, w, pre, mlp):
    if mlp["kind"] == "dense":
        return gated_feed_forward(h, w, pre)
    return routed_experts(h, w, pre, mlp)


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out: list | None = None):
    """Logits ``[T, vocab]`` of one request's tokens.  ``layers_out`` receives the stream
    after every layer (the sum of the copies where there are several)."""
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
                inp = sum(w[hc + "in"][s] * streams[s] for s in range(n_streams))
            else:
                inp = x
            h = norm_around_zero(inp, w[f"{pre}norm{q}"], eps)
            if q == 2:
                y = feed_forward(h, w, pre + "mlp.", layer["mlp"])
            elif layer["type"] == "attention":
                y = sigmoid_window_attention(h, w, pre + "mix.", layer["mixer"], eps)
            elif layer["type"] == "general_delta":
                y, _ = general_delta(h, w, pre + "mix.", layer["mixer"], eps)
            else:
                raise ValueError(layer["type"])
            if streams is not None:
                streams = [sum(w[hc + "mix"][s, t] * streams[s] for s in range(n_streams)) + m * w[hc + "out"][t] * y
                           for t in range(n_streams)]
            else:
                x = x + m * y
        if layers_out is not None:
            layers_out.append(sum(streams) if streams is not None else x.clone())
    if streams is not None:
        x = sum(streams)
    return norm_around_zero(x, w["final.norm"], eps) @ w["embed"].T
