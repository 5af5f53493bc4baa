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
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    out, _ = decayed_state_walk(q, k, v, decay, h.new_zeros((H, D, V)))
    y = rms_unit(out.reshape(T, H * V), eps) * w[pre + "norm"]
    y = y * torch.sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T


def decayed_state_walk(q, k, v, decay, S):
    """``q``, ``k`` [T, H, D], ``v`` [T, H, V], ``decay`` [H], ``S`` [H, D, V] the state before
    the first token: ``S <- decay S + k v^T`` then the read ``S^T q``, token by token.
    Returns the reads [T, H, V] and the state after the last token."""
    out = v.new_zeros(v.shape)
    for t in range(q.shape[0]):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = (S * q[t][:, :, None]).sum(1)
    return out, S


def gated_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def routed_experts(h, w, pre, f, margins_out=None):
    """The ``top`` experts with the largest router logits, weighted by the softmax over the
    chosen logits alone; and an expert for every token times a sigmoid of its own.
    ``margins_out`` receives, per token, the distance between the last chosen logit and the
    first one left out (infinite where every expert is chosen)."""
    z = h @ w[pre + "router"].T
    top, n = f["router"]["top"], f["router"]["experts"]
    chosen = torch.topk(z, top, dim=-1)
    weights = torch.softmax(chosen.values, -1)
    if margins_out is not None:
        ranked = torch.sort(z, dim=-1, descending=True).values
        margins_out.append(ranked[:, top - 1] - ranked[:, top] if top < n else torch.full_like(z[:, 0], math.inf))
    out = torch.zeros_like(h)
    for e in range(n):
        for j in range(top):
            rows = (chosen.indices[:, j] == e).nonzero()[:, 0]
            if rows.numel():
                out[rows] += weights[rows, j : j + 1] * gated_expert(h[rows], w, f"{pre}e{e}.")
    if f.get("shared"):
        out = out + torch.sigmoid(h @ w[pre + "shared.sg"].T) * gated_expert(h, w, pre + "shared.")
    return out, chosen


def token_input(x, tokens, w, pre, table, eps):
    """What a layer adds for the token itself: a gated row of the layer's part of a table."""
    g = gelu_tanh(x @ w[pre + "side.gate"].T) * table[tokens]
    y = g @ w[pre + "side.proj"].T
    return rms_unit(y, eps) * w[pre + "side.norm"]


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out: list | None = None, round_inputs=None,
            margins_out: list | None = None, disturb: float = 0.0, seed: int = 0) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one request's tokens; ``layers_out`` collects the stream
    after every layer.  ``round_inputs``: an element type that every part's input is rounded
    to on the way (how far the logits move then says how sensitive a position is to arithmetic
    in that type); ``disturb``: a relative error that every entry of every part's input is moved by,
    drawn from ``seed``.  ``margins_out`` receives every router's margins (see ``routed_experts``)."""
    gen = torch.Generator().manual_seed(seed)

    def rounded(t):
        if round_inputs is not None:
            t = t.to(round_inputs).to(dtype)
        if disturb:  # every entry moved by a relative error of that size (what arithmetic in 16 bits has piled up by then)
            t = t * (1.0 + disturb * torch.randn(t.shape, generator=gen, dtype=dtype))
        return t

    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = rms_unit(w["embed"][tokens], eps) * w["embed.norm"]
    side = cfg.get("token_side")
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        xin = rounded(x)
        if layer["type"] == "attention":
            y, v = capped_attention(xin, w, pre + "mix.", m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif layer["type"] == "latent_attention":
            y = latent_sink_attention(xin, w, pre + "mix.", m, eps)
        elif layer["type"] == "lightning":
            y = decayed_sum_attention(xin, w, pre + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_unit(y, eps) * w[pre + "norm1"] * w[pre + "ls1"]
        if layer.get("mlp"):
            y, _ = routed_experts(rounded(x), w, pre + "mlp.", layer["mlp"], margins_out)
            x = x + rms_unit(y, eps) * w[pre + "norm2"] * w[pre + "ls2"]
        if side:
            d = side["dim"]
            x = x + token_input(rounded(x), tokens, w, pre, w["side.embed"][:, i * d : (i + 1) * d], eps)
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
def rot(base, dims, factor=None, original=64, fast=32.0, slow=1.0):
    out = {"base": base, "dims": dims}
    if factor is not None:
        out["scaling"] = {"factor": factor, "original": original, "fast": fast, "slow": slow}
    return out


def attention_layer(heads, kv_heads, dim, vdim, scale, conv=None, rot=None, softcap=None, v_mix=False, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    for key, value in (("conv", conv), ("rot", rot), ("softcap", softcap)):
        if value is not None:
            mixer[key] = value
    if v_mix:
        mixer["v_mix"] = True
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def latent_layer(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot, mlp=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
             "scale": scale, "rot": rot}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def lightning_layer(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def model_cfg(width, vocab, layers, side=None, eps=1e-5):
    cfg = {"architecture": "Diporax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if side is not None:
        cfg["token_side"] = {"dim": side}
    return cfg


def tensor_shapes(cfg) -> dict:
    """Name -> shape of every tensor of a folder."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "embed.norm": (W,), "final.norm": (W,), "head": (V, W)}
    side = cfg.get("token_side")
    if side:
        out["side.embed"] = (V, side["dim"] * len(cfg["layers"]))
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        out[pre + "norm1"], out[pre + "ls1"] = (W,), (W,)
        if layer["type"] == "attention":
            sizes = {"q": m["heads"] * m["dim"], "k": m["kv_heads"] * m["dim"], "v": m["kv_heads"] * m["vdim"]}
            for name, n in sizes.items():
                out[f"{pre}mix.{name}"], out[f"{pre}mix.{name}.b"] = (n, W), (n,)
                if m.get("conv"):
                    out[f"{pre}mix.{name}.conv"] = (n, m["conv"])
            out[pre + "mix.q.norm"], out[pre + "mix.k.norm"] = (m["dim"],), (m["dim"],)
            if m.get("v_mix"):
                out[pre + "mix.vmix"] = ()
            out[pre + "mix.g"], out[pre + "mix.o"] = (m["heads"], W), (W, m["heads"] * m["vdim"])
        elif layer["type"] == "latent_attention":
            H = m["heads"]
            out[pre + "mix.dq"], out[pre + "mix.dq.norm"] = (m["q_rank"], W), (m["q_rank"],)
            out[pre + "mix.uq"] = (H * (m["dim"] + m["rot_dim"]), m["q_rank"])
            out[pre + "mix.dkv"], out[pre + "mix.dkv.norm"] = (m["kv_rank"] + m["rot_dim"], W), (m["kv_rank"],)
            out[pre + "mix.uk"], out[pre + "mix.uv"] = (H * m["dim"], m["kv_rank"]), (H * m["vdim"], m["kv_rank"])
            out[pre + "mix.sink"], out[pre + "mix.g"], out[pre + "mix.o"] = (H,), (H, W), (W, H * m["vdim"])
        else:
            nk, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out[pre + "mix.q"], out[pre + "mix.k"], out[pre + "mix.v"] = (nk, W), (nk, W), (nv, W)
            out[pre + "mix.g"], out[pre + "mix.norm"], out[pre + "mix.o"] = (nv, W), (nv,), (W, nv)
        f = layer.get("mlp")
        if f is not None:
            out[pre + "norm2"], out[pre + "ls2"] = (W,), (W,)
            out[pre + "mlp.router"] = (f["router"]["experts"], W)
            groups = [(f"e{e}", f["expert"]["ff"]) for e in range(f["router"]["experts"])]
            if f.get("shared"):
                groups.append(("shared", f["shared"]["ff"]))
                out[pre + "mlp.shared.sg"] = (1, W)
            for name, ff in groups:
                out[f"{pre}mlp.{name}.gate"], out[f"{pre}mlp.{name}.up"], out[f"{pre}mlp.{name}.down"] = (ff, W), (ff, W), (W, ff)
        if side:
            out[pre + "side.gate"], out[pre + "side.proj"], out[pre + "side.norm"] = (side["dim"], W), (W, side["dim"]), (W,)
    return out


def random_weights(cfg, seed, std=0.12, stored=torch.bfloat16):
    """Matrices N(0, std); norm weights and layer scales around one and below; convolutions,
    biases, sinks and blends of a size that counts; rounded to ``stored`` so that engine and
    plain model hold the same numbers."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        parts = name.split(".")
        last = parts[-1]
        r = lambda scale=1.0: scale * torch.randn(shape, generator=gen)  # noqa: E731
        if name in ("embed", "side.embed"):
            t = r(0.7)
        elif last == "conv":
            t = r(0.5)
        elif last == "norm" or last in ("norm1", "norm2"):
            t = 1.0 + r(0.2)
        elif last in ("ls1", "ls2"):
            t = 0.5 + r(0.1)
        elif last == "vmix":
            t = torch.tensor(0.35) + r(0.05)
        elif last == "sink":
            t = r(1.5)
        elif last == "b":
            t = r(0.5)
        elif last in ("gate", "up", "down") and parts[-2] != "side":
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


# every mixer; grouped key/value heads; a lightning head whose values are longer than its keys;
# two blending attentions; stretched rotations of both pairings; a shared expert; token input
DIP_A = model_cfg(64, 331, [
    attention_layer(4, 2, 16, 16, 0.3, conv=4, rot=rot(1000.0, 8, factor=4.0), softcap=5.0, v_mix=True,
                    mlp=moe(8, 2, 32, shared=24)),
    lightning_layer(2, 16, 24, [0.9, 0.995], mlp=moe(8, 2, 32, shared=24)),
    attention_layer(4, 2, 16, 16, 0.3, conv=4, rot=rot(1000.0, 8, factor=4.0), softcap=5.0, v_mix=True,
                    mlp=moe(8, 2, 32, shared=24)),
    latent_layer(4, 16, 8, 16, 24, 32, 0.2, rot(1000.0, 8, factor=2.0, original=32), mlp=moe(8, 2, 32, shared=24)),
], side=8)
# the recurrence first; no token input; an attention without convolution, rotation, cap and blend and
# without a feed-forward; value heads larger and smaller than the keys'; a blend that starts at the
# fourth layer; a whole head rotated; every expert chosen, and one of three; no shared expert;
# rotations that are not stretched
DIP_B = model_cfg(48, 257, [
    lightning_layer(3, 8, 16, [0.5, 0.97, 1.0], mlp=moe(5, 5, 24)),
    attention_layer(6, 3, 8, 24, 0.5, conv=2),
    latent_layer(2, 24, 4, 8, 10, 20, 0.25, rot(50.0, 4), mlp=moe(3, 1, 36, shared=20)),
    attention_layer(2, 2, 24, 8, 0.25, rot=rot(200.0, 24), softcap=12.0, v_mix=True, mlp=moe(4, 2, 20)),
    attention_layer(2, 2, 24, 8, 0.25, conv=1, rot=rot(200.0, 24), v_mix=True),
])
# sizes that are multiples of nothing; five taps; one key/value head; one blending layer alone; one
# lightning head without decay and without a feed-forward; a latent row that pages pad
DIP_C = model_cfg(40, 203, [
    attention_layer(5, 1, 12, 20, 0.2, conv=5, rot=rot(77.0, 6, factor=8.0, original=16, fast=4.0, slow=0.5), softcap=30.0,
                    v_mix=True, mlp=moe(6, 3, 20, shared=28)),
    lightning_layer(1, 20, 12, [1.0]),
    latent_layer(3, 12, 6, 20, 7, 27, 0.3, rot(300.0, 6, factor=3.0, original=40), mlp=moe(6, 3, 20)),
], side=3, eps=1e-6)
