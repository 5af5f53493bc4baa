"""Vepitar without a GPU: the configuration and what is read from tensors' shapes, the
table of tensor names and the loader, the model as data, the random-weights mode, and the
plain implementation's own pins."""

import json
import math
import os

import pytest
import torch

import plain_vepitar as P
from halite_amd.config import parse_config, read_config
from halite_amd.config.registry import ConfigError
from halite_amd.parts import Decoder
from halite_amd.weights import load_weights, write_random_model
from halite_amd.weights.loader import WeightError

CONFIGS = {"A": (P.VEP_A, P.VEP_A_RANKS), "B": (P.VEP_B, P.VEP_B_RANKS), "C": (P.VEP_C, P.VEP_C_RANKS)}
F = torch.float64


def rand(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F)


def test_the_decay_rank_comes_from_the_tensor(tmp_path):
    cfg, ranks = CONFIGS["A"]
    arch, parsed = parse_config(cfg)
    assert arch.name == "Vepitar" and parsed.layers[0].mixer.decay_rank is None
    with pytest.raises(ConfigError, match="decay_rank"):
        arch.to_spec(parsed)  # the file alone does not say how wide the decay's inner projection is
    folder = P.write_model_folder(str(tmp_path), cfg, P.random_weights(cfg, ranks, 1))
    arch, parsed = read_config(folder)
    assert [getattr(l.mixer, "decay_rank", None) for l in parsed.layers] == [8, None, 8]
    spec = arch.to_spec(parsed)
    mixer = spec.layers["l0"].parts["mixer"].params()
    assert mixer["decay_rank"] == 8 and abs(mixer["decay_rate"] - math.exp(-0.5)) < 1e-15 and mixer["unit_eps"] == 1e-6
    written = parsed.to_json_dict()
    assert "decay_rank" not in json.dumps(written) and written["layers"][1]["mixer"]["mask"] == {"size": 24}
    assert written["residual_mult"] == 0.7 and written["streams"] == 2
    stated = json.loads(json.dumps(cfg))
    for i, n in ranks.items():
        stated["layers"][i]["mixer"]["decay_rank"] = n
    assert parse_config(stated)[0].to_spec(parse_config(stated)[1]) == spec


def test_keys_that_are_left_out_switch_their_mechanism_off():
    cfg = json.loads(json.dumps(P.VEP_C))
    for i, n in P.VEP_C_RANKS.items():
        cfg["layers"][i]["mixer"]["decay_rank"] = n
    arch, parsed = parse_config(cfg)
    spec = arch.to_spec(parsed)
    link = spec.layers["l0"].parts["mixer_link"].params()
    assert link["streams"] == 1 and link["learned"] is False and link["mult"] == 1.0
    assert "ff" not in spec.layers["l2"].parts and "ff_link" not in spec.layers["l2"].parts
    _, parsed_b = parse_config({**json.loads(json.dumps(P.VEP_B)),
                                "layers": [P.attention_layer(2, 2, 24, 8, 0.25, mlp=P.dense(40))]})
    att = arch.to_spec(parsed_b).layers["l0"].parts["mixer"].params()
    assert att["conv_taps"] is None and att["window"] is None and att["scale"] == 0.25
    names = arch.weight_map(parsed_b)
    assert "l0.mix.q.conv" not in names and names["l0.hc1.mix"] == "layers.l0.mixer_link.mix"
    assert "l0.hc1.in" not in arch.weight_map(parsed)  # one stream: no connection weights


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][1]["mixer"].update(kv_heads=3),
    lambda c: c["layers"][1]["mixer"].pop("scale"),
    lambda c: c["layers"][1]["mixer"].pop("vdim"),
    lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
    lambda c: c["layers"][0].update(type="recurrent"),
    lambda c: c["layers"][0]["mlp"].update(kind="gated"),
    lambda c: c["layers"][1]["mixer"].update(mask={"size": 0}),
    lambda c: c.update(streams=0),
    lambda c: c.update(layers=[]),
    lambda c: c.pop("norm"),
    lambda c: c.update(width=64.5),
])
def test_configurations_that_are_refused(bad):
    cfg = json.loads(json.dumps(P.VEP_A))
    bad(cfg)
    with pytest.raises(ConfigError):
        parse_config(cfg)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_model_as_data_and_its_tensors(name, tmp_path):
    cfg, ranks = CONFIGS[name]
    weights = P.random_weights(cfg, ranks, 2)
    folder = P.write_model_folder(str(tmp_path), cfg, weights)
    arch, parsed = read_config(folder)
    spec = arch.to_spec(parsed)
    assert [l.arrangement for l in spec.layers.values()] == ["hyper_pre_norm"] * len(cfg["layers"])
    model = Decoder(spec, torch.float32, "cpu")
    assert model.stream_copies == (cfg.get("streams") or 1)
    load_weights(model, arch.weight_map(parsed), folder)
    assert torch.equal(model.embedding.weight, weights["embed"])
    for i, layer in enumerate(cfg["layers"]):
        block = model.layers[f"l{i}"]
        m, mixer = layer["mixer"], block.mixer
        assert (block.ff is None) == (layer["mlp"] is None)
        if layer["type"] == "general_delta":
            n = m["heads"] * m["dim"]
            for j, t in enumerate(("r", "k", "v", "a", "g")):
                assert torch.equal(mixer.w_in[j * n : (j + 1) * n], weights[f"l{i}.mix.{t}"])
            assert torch.equal(mixer.w_in[5 * n :], weights[f"l{i}.mix.w1"]) and mixer.w_in.shape[0] == 5 * n + ranks[i]
            assert torch.equal(mixer.w_decay_up_weight, weights[f"l{i}.mix.w2"])
            assert torch.equal(mixer.w_a_bias, weights[f"l{i}.mix.a.b"])
            assert mixer.state_need()["state"].shape == (m["heads"], m["dim"], m["dim"])
            assert mixer.state_need()["state"].dtype == torch.float32 and mixer.cache_need() is None
        else:
            nq, nk, nv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            assert torch.equal(mixer.w_in[:nq], weights[f"l{i}.mix.q"])
            assert torch.equal(mixer.w_in[nq + nk : nq + nk + nv], weights[f"l{i}.mix.v"])
            assert torch.equal(mixer.w_in[nq + nk + nv :], weights[f"l{i}.mix.g"])
            need = mixer.cache_need()
            assert need.n_kv_heads == m["kv_heads"] and need.head_dim >= max(m["dim"], m["vdim"]) and need.head_dim % 16 == 0
            assert need.window == (m.get("mask") or {}).get("size")
            if m.get("conv", 1) > 1:
                assert torch.equal(mixer.w_conv[nq : nq + nk], weights[f"l{i}.mix.k.conv"])
                assert mixer.state_need()["conv"].shape == (m["conv"] - 1, nq + nk + nv)
            else:
                assert mixer.state_need() == {}
            assert mixer.rule.sigmoid and torch.equal(mixer.rule.bias[:, 0], weights[f"l{i}.mix.pb"])
        if cfg.get("streams"):
            assert torch.equal(block.mixer_link.w_mix, weights[f"l{i}.hc1.mix"])
            if block.ff is not None:
                assert torch.equal(block.ff_link.w_out, weights[f"l{i}.hc2.out"])
        if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
            e = layer["mlp"]["router"]["experts"] - 1
            assert block.ff.w_gate is None and torch.equal(block.ff.w_up[e], weights[f"l{i}.mlp.e{e}.up"])
            assert torch.equal(block.ff.w_down[0], weights[f"l{i}.mlp.e0.down"])
    # a tensor that is missing and one that nobody knows are both named
    from safetensors.torch import save_file

    broken = dict(weights)
    broken.pop("l1.norm1")
    broken["l0.mix.extra"] = torch.zeros(3)
    save_file({k: v.to(torch.bfloat16) for k, v in broken.items()}, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_weights(Decoder(spec, torch.float32, "cpu"), arch.weight_map(parsed), folder)
    assert "l1.norm1" in e.value.missing and "l0.mix.extra" in e.value.unexpected


def test_a_folder_of_random_weights(tmp_path):
    """The random-weights mode writes the design's own tensor names and keys, and the folder
    reads back to the same model as data."""
    stated = json.loads(json.dumps(P.VEP_B))
    for i, n in P.VEP_B_RANKS.items():
        stated["layers"][i]["mixer"]["decay_rank"] = n
    arch, parsed = parse_config(stated)
    folder = write_random_model(str(tmp_path / "m"), parsed, 3, "bfloat16", 0.1, arch)
    from safetensors import safe_open

    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        shapes = {k: tuple(f.get_slice(k).get_shape()) for k in f.keys()}
    assert shapes == {k: tuple(v) for k, v in P.tensor_shapes(P.VEP_B, P.VEP_B_RANKS).items()}
    arch2, back = read_config(folder)
    assert arch2.to_spec(back) == arch.to_spec(parsed)
    assert "decay_rank" not in open(os.path.join(folder, "config.json")).read()


# -- the plain implementation's own pins -------------------------------------------------------------


def test_plain_recurrence_in_two_halves_and_as_sums():
    T, D = 18, 6
    r, k, v = rand(T, D, seed=1), rand(T, D, seed=2), rand(T, D, seed=3)
    decay, a = torch.sigmoid(rand(T, D, seed=4)), torch.sigmoid(rand(T, D, seed=5))
    S0 = rand(D, D, seed=6)
    o, S = P.delta_recurrence(r, k, v, decay, a, S0)
    o1, S1 = P.delta_recurrence(r[:7], k[:7], v[:7], decay[:7], a[:7], S0)
    o2, S2 = P.delta_recurrence(r[7:], k[7:], v[7:], decay[7:], a[7:], S1)
    assert float((torch.cat([o1, o2]) - o).abs().max()) < 1e-12 and float((S2 - S).abs().max()) < 1e-12
    # nothing removed: a sum over the earlier tokens with the products of the decays between
    o0, _ = P.delta_recurrence(r, k, v, decay, torch.zeros_like(a), torch.zeros(D, D, dtype=F))
    t = 11
    want = sum((r[t] * torch.prod(decay[j + 1 : t + 1], 0) * k[j]).sum() * v[j] for j in range(t + 1))
    assert float((o0[t] - want).abs().max()) < 1e-12
    # no decay and all removed: what lay along the unit key is gone before the new pair is written
    one = torch.ones(1, D, dtype=F)
    _, S3 = P.delta_recurrence(r[:1], k[:1], v[:1], one, one, S0, unit_eps=0.0)
    u = k[0] / k[0].norm()
    assert float((u @ (S3 - torch.outer(k[0], v[0]))).abs().max()) < 1e-12
    # the transition as a matrix: diag(w) - (a u) u^T on the old state
    _, S4 = P.delta_recurrence(r[:1], k[:1], v[:1], decay[:1], a[:1], S0, unit_eps=0.0)
    M = torch.diag(decay[0]) - torch.outer(a[0] * u, u)
    assert float((S4 - (M @ S0 + torch.outer(k[0], v[0]))).abs().max()) < 1e-12


def test_plain_pieces_against_library_routines():
    u, w = rand(30, 6, seed=7), rand(6, 4, seed=8)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (3, 0)), w[:, None, :], groups=6)[0].T
    assert float((P.short_conv(u, w) - want).abs().max()) < 1e-12
    x = rand(9, 7, seed=9)
    assert float((P.rms_unit(x, 1e-6) - torch.nn.functional.rms_norm(x, (7,), eps=1e-6)).abs().max()) < 1e-12
    wz = rand(7, seed=10, scale=0.2)
    assert float((P.norm_around_zero(x, wz, 1e-6) - torch.nn.functional.rms_norm(x, (7,), 1 + wz, 1e-6)).abs().max()) < 1e-12
    # the decay lies between exp(-e^(-1/2)) and 1
    wd = {"w1": rand(3, 7, seed=11), "w2": rand(5, 3, seed=12, scale=5.0), "w0": rand(5, seed=13, scale=5.0)}
    d = P.delta_decay(x, wd, "")
    assert float(d.max()) <= 1.0 and float(d.min()) >= math.exp(-math.exp(-0.5)) and float(d.max() - d.min()) > 0.3


def test_plain_attention_as_matrices():
    """The loop over queries against masked matrices: the window's first and last key, heads
    that share keys, no sum to one."""
    T, W = 25, 20
    m = {"heads": 4, "kv_heads": 2, "dim": 3, "vdim": 5, "scale": 0.7, "conv": 3, "mask": {"size": 6}}
    w = {"q": rand(12, W, seed=1), "k": rand(6, W, seed=2), "v": rand(10, W, seed=3), "g": rand(4, W, seed=4),
         "o": rand(W, 20, seed=5), "pb": rand(4, seed=6), "q.conv": rand(12, 3, seed=7), "k.conv": rand(6, 3, seed=8),
         "v.conv": rand(10, 3, seed=9)}
    h = rand(T, W, seed=10)
    got = P.sigmoid_window_attention(h, w, "", m, 1e-5)
    q = P.rms_unit(P.short_conv(h @ w["q"].T, w["q.conv"]).view(T, 4, 3), 1e-5)
    k = P.rms_unit(P.short_conv(h @ w["k"].T, w["k.conv"]).view(T, 2, 3), 1e-5).repeat_interleave(2, 1)
    v = P.rms_unit(P.short_conv(h @ w["v"].T, w["v.conv"]).view(T, 2, 5), 1e-5).repeat_interleave(2, 1)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None]
    seen = (j <= i) & (i - j < 6)
    p = torch.sigmoid(torch.einsum("ihd,jhd->hij", q, k) * 0.7 + w["pb"][:, None, None]) * seen
    out = torch.einsum("hij,jhd->ihd", p, v) * torch.sigmoid(h @ w["g"].T)[:, :, None]
    assert float((got - out.reshape(T, 20) @ w["o"].T).abs().max()) < 1e-12
    assert float(p.sum(-1).max()) > 1.5  # the weights are not normalised
    m2 = {k_: v_ for k_, v_ in m.items() if k_ not in ("conv", "mask")}
    full = P.sigmoid_window_attention(h, w, "", {**m2, "mask": {"size": T}}, 1e-5)
    assert float((full - P.sigmoid_window_attention(h, w, "", m2, 1e-5)).abs().max()) == 0.0


def test_plain_connections_and_experts():
    x = [rand(5, 8, seed=s) for s in (1, 2, 3)]
    y = rand(5, 8, seed=4)
    eye, ones = torch.eye(3, dtype=F), torch.ones(3, dtype=F)
    new = P.connection_write(x, y, eye, ones, 0.5)  # nothing mixed: the plain residual sum on every copy
    assert all(float((n - (o + 0.5 * y)).abs().max()) < 1e-12 for n, o in zip(new, x))
    mix = rand(3, 3, seed=5)
    new = P.connection_write(x, torch.zeros_like(y), mix, ones, 1.0)  # [from, to]
    assert float((new[2] - (mix[0, 2] * x[0] + mix[1, 2] * x[1] + mix[2, 2] * x[2])).abs().max()) < 1e-12
    assert float((P.connection_read(x, torch.tensor([1.0, 0.0, 2.0], dtype=F)) - (x[0] + 2 * x[2])).abs().max()) < 1e-12
    # every expert chosen: the softmax itself weighs them; one chosen: its weight is 1
    h = rand(6, 8, seed=6)
    w = {"router": rand(4, 8, seed=7)}
    for e in range(4):
        w[f"e{e}.up"], w[f"e{e}.down"] = rand(5, 8, seed=10 + e), rand(8, 5, seed=20 + e)
    outs = torch.stack([(torch.relu(h @ w[f"e{e}.up"].T) ** 2) @ w[f"e{e}.down"].T for e in range(4)], 1)
    s = torch.softmax(h @ w["router"].T, -1)
    every = P.routed_experts(h, w, "", {"router": {"experts": 4, "top": 4}})
    assert float((every - (s[:, :, None] * outs).sum(1)).abs().max()) < 1e-12
    single = P.routed_experts(h, w, "", {"router": {"experts": 4, "top": 1}})
    assert float((single - outs[torch.arange(6), s.argmax(-1)]).abs().max()) < 1e-12


def test_plain_model_token_by_token_state():
    """The plain mixer's state argument: a sequence in two calls equals one call."""
    cfg, ranks = CONFIGS["A"]
    w = {k: v.to(F) for k, v in P.random_weights(cfg, ranks, 4).items()}
    h = rand(15, cfg["width"], seed=1)
    m = cfg["layers"][0]["mixer"]
    y, S = P.general_delta(h, w, "l0.mix.", m, 1e-5)
    y1, S1 = P.general_delta(h[:4], w, "l0.mix.", m, 1e-5)
    y2, S2 = P.general_delta(h[4:], w, "l0.mix.", m, 1e-5, state=S1)
    assert float((torch.cat([y1, y2]) - y).abs().max()) < 1e-12 and float((S2 - S).abs().max()) < 1e-12
