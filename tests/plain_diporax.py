"""A plain, slow implementation of the Diporax decoder: one function per mechanism, written
from the design's equations in float64 (or any torch dtype), sharing no code with the
framework.  Tests compare the framework with it.

Notation: ``h`` is a part's input ``[T, width]`` for the ``T`` tokens of one request, in
order; weights are ``[out, in]`` and applied as ``h @ W.T``.  A model is a dict ``cfg`` with
the keys of ``config.json`` and a dict ``w`` of tensors by their names in the folder.
"""

from __future__ import annotations

import json
import math
import os

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps)`` over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def short_conv(u: torch.Tensor, taps_weight: torch.Tensor) -> torch.Tensor:
    """Causal convolution over time on every channel: ``u`` [T, C], ``taps_weight``
    [C, taps]; the last tap multiplies the token itself, zeros before the first token."""
    T, C = u.shape
    taps = taps_weight.shape[1]
    padded = torch.cat([u.new_zeros((taps - 1, C)), u], 0)
    y = u.new_zeros((T, C))
    for j in range(taps):
        y += taps_weight[:, j] * padded[j : j + T]  # padded[t + j] is u[t - taps + 1 + j]
    return y


def stretched_frequencies(rot: dict, dtype=torch.float64):
    """The rotation's frequencies ``base^(-2i/dims)``, and with ``scaling`` the blend of each
    with itself divided by ``factor`` along a ramp over the pair index; also the number that
    cosine and sine are multiplied by."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    s = rot.get("scaling")
    if not s:
        return f, 1.0

    def pair_of(turns):  # the pair index whose wavelength fits `turns` times into `original`
        return dims * math.log(s["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(s["fast"])), 0)
    hi = min(math.ceil(pair_of(s["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / s["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(s["factor"]) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict, interleaved: bool) -> torch.Tensor:
    """Rotates the first ``rot.dims`` entries of the last dimension of ``x`` [T, ..., D]:
    pairs ``(2i, 2i + 1)`` if ``interleaved``, else ``(i, i + dims/2)``."""
    dims = rot["dims"]
    f, mag = stretched_frequencies(rot, x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]
    cos, sin = torch.cos(a) * mag, torch.sin(a) * mag
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        u, v = x[..., : dims // 2], x[..., dims // 2 : dims]
        out[..., : dims // 2] = u * cos - v * sin
        out[..., dims // 2 : dims] = v * cos + u * sin
    return out


def capped_attention(h, w, pre, m, eps, v_first):
    """Grouped heads with biases, short convolutions, a norm per head on q and k, partial
    rotation, capped scores, values mixed with an earlier layer's, a gate per head.
    Returns the result and the values that were attended over (after mixing)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    proj = {}
    for n in ("q", "k", "v"):
        t = h @ w[pre + n].T
        if pre + n + ".b" in w:
            t = t + w[pre + n + ".b"]
        if m.get("conv"):
            t = short_conv(t, w[pre + n + ".conv"])
        proj[n] = t
    q = rms_unit(proj["q"].view(T, H, D), eps) * w[pre + "q.norm"]
    k = rms_unit(proj["k"].view(T, G, D), eps) * w[pre + "k.norm"]
    v = proj["v"].view(T, G, V)
    pos = torch.arange(T)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], False), rotate(k, pos, m["rot"], False)
    if m.get("v_mix") and v_first is not None:
        lam = w[pre + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    gate = torch.sigmoid(h @ w[pre + "g"].T)  # [T, H]
    cap = m.get("softcap")
    out = h.new_zeros((T, H, V))
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
        out[:, head] = torch.softmax(s, -1) @ v[:, g]
    out = out * gate[:, :, None]
    return out.reshape(T, H * V) @ w[pre + "o"].T, v


def latent_sink_attention(h, w, pre, m, eps):
    """Queries through a latent; keys and values of every head made from one normed latent
    per token plus one rotated key part that all heads share; a learned term without key
    and value in every head's softmax; a gate per head."""
    T = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_unit(h @ w[pre + "dq"].T, eps) * w[pre + "dq.norm"]
    q = (cq @ w[pre + "uq"].T).view(T, H, D + R)
    kv = h @ w[pre + "dkv"].T
    c = rms_unit(kv[:, :C], eps) * w[pre + "dkv.norm"]
    pos = torch.arange(T)
    rot = dict(m["rot"], dims=R)
    shared = rotate(kv[:, C:], pos, rot, True)  # [T, R]
    q_rot = rotate(q[..., D:], pos, rot, True)
    keys = (c @ w[pre + "uk"].T).view(T, H, D)
    vals = (c @ w[pre + "uv"].T).view(T, H, V)
    gate = torch.sigmoid(h @ w[pre + "g"].T)
    out = h.new_zeros((T, H, V))
    for head in range(H):
        s = (q[:, head, :D] @ keys[:, head].T + q_rot[:, head] @ shared.T) * m["scale"]
        s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
        s = torch.cat([s, w[pre + "sink"][head].expand(T, 1)], 1)  # the term without a key
        out[:, head] = torch.softmax(s, -1)[:, :T] @ vals[:, head]
    out = out * gate[:, :, None]
    return out.reshape(T, H * V) @ w[pre + "o"].T


def decayed_sum_attention(h, w, pre, m, eps):
    """A recurrence with a matrix state per head and one constant decay per head:
    ``S <- decay S + k v^T``, read by ``S^T q``; the heads normed together and gated."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[pre + "q"].T).view(T, H, D)
    k = silu(h @ w[pre + "k"].T).view(T, H, D)
    v = silu(h @ w[pre + "v"].T).view(T, H, V)
    out = h.new_zeros((T, H, V))
    for head in range(H):
        S = h.new_zeros((D, V))
        for t in range(T):
            S = m["decay"][head] * S + torch.outer(k[t, head], v[t, head])
            out[t, head] = S.T @ q[t, head]
    y = rms_unit(out.reshape(T, H * V), eps) * w[pre + "norm"]
    y = y * torch.sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T


def gated_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def routed_experts(h, w, pre, f):
    """The ``top`` experts with the largest router logits, weighted by the softmax over the
    chosen logits alone; and an expert for every token times a sigmoid of its own."""
    z = h @ w[pre + "router"].T
    top = f["router"]["top"]
    chosen = torch.topk(z, top, dim=-1)
    weights = torch.softmax(chosen.values, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen.indices[t, j])
            out[t] += weights[t, j] * gated_expert(h[t : t + 1], w, f"{pre}e{e}.")[0]
    if f.get("shared"):
        out = out + torch.sigmoid(h @ w[pre + "shared.sg"].T) * gated_expert(h, w, pre + "shared.")
    return out, chosen


def token_input(x, tokens, w, pre, table, eps):
    """What a layer adds for the token itself: a gated row of the layer's part of a table."""
    g = gelu_tanh(x @ w[pre + "side.gate"].T) * table[tokens]
    y = g @ w[pre + "side.proj"].T
    return rms_unit(y, eps) * w[pre + "side.norm"]


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out: list | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one request's tokens; ``layers_out`` collects the stream
    after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = rms_unit(w["embed"][tokens], eps) * w["embed.norm"]
    side = cfg.get("token_side")
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "attention":
            y, v = capped_attention(x, w, pre + "mix.", m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif layer["type"] == "latent_attention":
            y = latent_sink_attention(x, w, pre + "mix.", m, eps)
        elif layer["type"] == "lightning":
            y = decayed_sum_attention(x, w, pre + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_unit(y, eps) * w[pre + "norm1"] * w[pre + "ls1"]
        if layer.get("mlp"):
            y, _ = routed_experts(x, w, pre + "mlp.", layer["mlp"])
            x = x + rms_unit(y, eps) * w[pre + "norm2"] * w[pre + "ls2"]
        if side:
            d = side["dim"]
            x = x + token_input(x, tokens, w, pre, w["side.embed"][:, i * d : (i + 1) * d], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_unit(x, eps) * w["final.norm"]
    return x @ w["head"].T


def load_folder(folder: str):
    """``(cfg, w)`` of a model folder, read with the safetensors package."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, load_file(os.path.join(folder, "model.safetensors"))
