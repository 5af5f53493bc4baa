"""Diporax without a GPU: the configuration and what is read from the folder's tensors, keys
that switch a mechanism off when they are left out, the table of tensor names and the loader,
the model as data, the random-weights mode, and the plain implementation's own pins."""

import json
import math
import os

import pytest
import torch

import plain_diporax as P
from halite_amd.config import parse_config, read_config
from halite_amd.config.registry import ConfigError
from halite_amd.parts import Decoder
from halite_amd.weights import load_weights, write_random_model
from halite_amd.weights.loader import WeightError

CONFIGS = {"A": P.DIP_A, "B": P.DIP_B, "C": P.DIP_C}
F = torch.float64


def rand(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F)


def test_biases_are_told_by_the_tensors(tmp_path):
    arch, parsed = parse_config(P.DIP_A)
    assert arch.name == "Diporax" and parsed.layers[0].mixer.bias is None
    assert arch.to_spec(parsed).layers["l0"].parts["mixer"].params()["bias"] is False  # the file alone knows of none
    folder = P.write_model_folder(str(tmp_path), P.DIP_A, P.random_weights(P.DIP_A, 1))
    arch, parsed = read_config(folder)
    assert [getattr(l.mixer, "bias", None) for l in parsed.layers] == [True, None, True, None]
    spec = arch.to_spec(parsed)
    assert spec.layers["l2"].parts["mixer"].params()["bias"] is True
    written = parsed.to_json_dict()
    assert '"bias"' not in json.dumps(written) and written["token_side"] == {"dim": 8}
    assert written["layers"][0]["mixer"]["rot"]["scaling"]["factor"] == 4.0


def test_the_model_as_data():
    arch, parsed = parse_config(P.DIP_A)
    spec = arch.to_spec(parsed)
    assert [l.arrangement for l in spec.layers.values()] == ["post_norm"] * 4
    kinds = [l.parts["mixer"].kind for l in spec.layers.values()]
    assert kinds == ["capped_attention", "decay_attention", "capped_attention", "latent_attention"]
    first, third = spec.layers["l0"].parts["mixer"].params(), spec.layers["l2"].parts["mixer"].params()
    assert first["value_mix"] == "first" and third["value_mix"] == "blend" and first["softcap"] == 5.0
    assert first["position"] == third["position"] and len(spec.positions) == 2  # one table a distinct rotation
    rope = spec.positions[first["position"]].params()
    assert rope["interleaved"] is False and rope["rotary_dim"] == 8 and rope["scaling"]["kind"] == "ramp"
    assert abs(rope["magnitude"] - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    latent = spec.layers["l3"].parts["mixer"].params()
    assert latent["learned_sink"] and latent["gate_per_head"] and latent["rope_dim"] == 8 and "window" not in latent
    assert spec.positions[latent["position"]].params()["interleaved"] is True
    ff = spec.layers["l1"].parts["ff"].params()
    assert ff["score"] == "softmax" and ff["normalize"] and ff["norm_eps"] == 0.0 and ff["shared_gate"] is True
    assert ff["expert"]["limit"] is None and ff["expert"]["alpha"] == 1.0 and ff["expert"]["up_shift"] == 0.0
    assert [spec.layers[f"l{i}"].parts["side"].params()["col0"] for i in range(4)] == [0, 8, 16, 24]
    assert spec.embedding.params()["side_size"] == 32 and spec.embedding.params()["norm_eps"] == 1e-5
    assert spec.layers["l0"].parts["mixer_norm"].params()["layer_scale"] is True
    assert "layer_scale" not in spec.layers["l0"].parts["side_norm"].params()


def test_keys_that_are_left_out_switch_their_mechanism_off():
    arch, parsed = parse_config(P.DIP_B)
    spec = arch.to_spec(parsed)
    bare = spec.layers["l1"].parts["mixer"].params()
    assert bare["position"] is None and bare["softcap"] is None and bare["value_mix"] is None and bare["conv_taps"] == 2
    assert "ff" not in spec.layers["l1"].parts and "side" not in spec.layers["l0"].parts
    assert spec.embedding.params()["side_size"] is None
    assert spec.layers["l3"].parts["mixer"].params()["value_mix"] == "first"  # the first layer that says so
    assert spec.layers["l4"].parts["mixer"].params()["value_mix"] == "blend"
    assert spec.layers["l0"].parts["ff"].params()["shared"] is None and not spec.layers["l0"].parts["ff"].params()["shared_gate"]
    whole_head = spec.positions[spec.layers["l3"].parts["mixer"].params()["position"]].params()
    assert whole_head["scaling"] is None and whole_head["magnitude"] == 1.0 and whole_head["rotary_dim"] == 24
    names = arch.weight_map(parsed)
    assert "l1.mix.q.conv" in names and "l3.mix.q.conv" not in names and "side.embed" not in names
    assert names["l3.mix.vmix"] is None and names["l4.mix.vmix"] == "layers.l4.mixer.value_mix.weight"
    assert names["l1.norm2"] is None and "l0.mlp.shared.sg" not in names and names["l2.mlp.shared.sg"] == "layers.l2.ff.shared_gate.weight"


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][0]["mixer"].update(kv_heads=3),
    lambda c: c["layers"][0]["mixer"].pop("scale"),
    lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7),
    lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18),
    lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("original"),
    lambda c: c["layers"][1]["mixer"].update(decay=[0.5]),
    lambda c: c["layers"][3]["mixer"].pop("kv_rank"),
    lambda c: c["layers"][3]["mixer"].update(rot_dim=5),
    lambda c: c["layers"][0]["mlp"]["router"].update(top=9),
    lambda c: c["layers"][0].update(type="recurrent"),
    lambda c: c["layers"][0]["mlp"].update(kind="dense"),
    lambda c: c.update(token_side={"dim": 0}),
    lambda c: c.update(layers=[]),
    lambda c: c.pop("norm"),
    lambda c: c.update(width=64.5),
])
def test_configurations_that_are_refused(bad):
    cfg = json.loads(json.dumps(P.DIP_A))
    bad(cfg)
    with pytest.raises(ConfigError):
        parse_config(cfg)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_loader_and_the_tensors(name, tmp_path):
    cfg = CONFIGS[name]
    weights = P.random_weights(cfg, 2)
    folder = P.write_model_folder(str(tmp_path), cfg, weights)
    arch, parsed = read_config(folder)
    model = Decoder(arch.to_spec(parsed), torch.float32, "cpu")
    assert model.stream_copies is None
    load_weights(model, arch.weight_map(parsed), folder)
    assert torch.equal(model.embedding.weight, weights["embed"]) and torch.equal(model.embedding.norm_weight, weights["embed.norm"])
    if cfg.get("token_side"):
        assert torch.equal(model.embedding.side_weight, weights["side.embed"])
    for i, layer in enumerate(cfg["layers"]):
        block = model.layers[f"l{i}"]
        m, mixer = layer["mixer"], block.mixer
        assert (block.ff is None) == (layer["mlp"] is None) and (block.side is None) == (cfg.get("token_side") is None)
        assert torch.equal(block.mixer_norm.multiplier, weights[f"l{i}.norm1"] * weights[f"l{i}.ls1"])
        if layer["type"] == "attention":
            nq, nk, nv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            assert torch.equal(mixer.w_in[:nq], weights[f"l{i}.mix.q"]) and torch.equal(mixer.w_in[nq + nk + nv :], weights[f"l{i}.mix.g"])
            assert torch.equal(mixer.w_bias[nq : nq + nk], weights[f"l{i}.mix.k.b"])
            need = mixer.cache_need()
            assert need.n_kv_heads == m["kv_heads"] and need.head_dim >= max(m["dim"], m["vdim"]) and need.window is None
            if m.get("conv", 1) > 1:
                assert torch.equal(mixer.w_conv[nq + nk :], weights[f"l{i}.mix.v.conv"])
                assert mixer.state_need()["conv"].shape == (m["conv"] - 1, nq + nk + nv)
            else:
                assert mixer.state_need() == {}
            assert (mixer.rule is None) == ("softcap" not in m) and (mixer.rule is None or mixer.rule.softcap == m["softcap"])
            if mixer.p.value_mix == "blend":
                assert mixer.blend == float(weights[f"l{i}.mix.vmix"])
        elif layer["type"] == "latent_attention":
            assert torch.equal(mixer.w_down[: m["q_rank"]], weights[f"l{i}.mix.dq"])
            assert torch.equal(mixer.w_down[m["q_rank"] + m["kv_rank"] + m["rot_dim"] :], weights[f"l{i}.mix.g"])
            assert torch.equal(mixer.rule.sink_values, weights[f"l{i}.mix.sink"]) and mixer.rule.sink
            need = mixer.cache_need()
            assert need.n_kv_heads == 1 and need.head_dim >= m["kv_rank"] + m["rot_dim"] and need.head_dim % 16 == 0
        else:
            nk, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            assert torch.equal(mixer.w_in[:nv], weights[f"l{i}.mix.v"]) and torch.equal(mixer.w_in[nv + nk : nv + 2 * nk], weights[f"l{i}.mix.q"])
            assert mixer.state_need()["state"].shape == (m["heads"], m["dim"], m["vdim"]) and mixer.cache_need() is None
            assert torch.equal(mixer.decay, torch.tensor(m["decay"]).float())
        f = layer["mlp"]
        if f is not None:
            e = f["router"]["experts"]
            assert torch.equal(block.ff.w_router[:e], weights[f"l{i}.mlp.router"])
            assert torch.equal(block.ff.w_gate[e - 1], weights[f"l{i}.mlp.e{e - 1}.gate"])
            if f.get("shared"):
                assert torch.equal(block.ff.w_router[e:], weights[f"l{i}.mlp.shared.sg"])
                assert torch.equal(block.ff.ws_down, weights[f"l{i}.mlp.shared.down"])
    # a tensor that is missing and one that nobody knows are both named
    from safetensors.torch import save_file

    broken = dict(weights)
    broken.pop("l0.ls1")
    broken["l0.mix.extra"] = torch.zeros(3)
    save_file({k: v.to(torch.bfloat16) for k, v in broken.items()}, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_weights(Decoder(arch.to_spec(parsed), torch.float32, "cpu"), arch.weight_map(parsed), folder)
    assert "l0.ls1" in str(e.value) and "l0.mix.extra" in str(e.value)


def test_the_random_weights_mode(tmp_path):
    stated = json.loads(json.dumps(P.DIP_C))
    stated["layers"][0]["mixer"]["bias"] = True
    arch, parsed = parse_config(stated)
    folder = write_random_model(str(tmp_path / "m"), parsed, seed=4, dtype="bfloat16", std=0.1)
    arch2, again = read_config(folder)
    assert arch2.to_spec(again) == arch.to_spec(parsed)
    from safetensors.torch import load_file

    names = set(load_file(os.path.join(folder, "model.safetensors")))
    assert names == set(P.tensor_shapes(P.DIP_C)) - {"l0.mix.vmix"}  # (the first blending layer's own number has no reader)
    assert json.load(open(os.path.join(folder, "config.json")))["layers"][1]["mlp"] is None


# -- the plain implementation's own pins -----------------------------------------------------------


def test_the_recurrence_as_sums_and_in_halves():
    T, H, D, V = 13, 2, 5, 7
    q, k, v = rand(T, H, D, seed=1), rand(T, H, D, seed=2), rand(T, H, V, seed=3)
    decay = torch.tensor([0.8, 1.0], dtype=F)
    out, S = P.decayed_state_walk(q, k, v, decay, torch.zeros(H, D, V, dtype=F))
    for t in (0, 6, 12):
        for h in range(H):
            want = sum(decay[h] ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h] for j in range(t + 1))
            assert float((out[t, h] - want).abs().max()) < 1e-12
    first, mid = P.decayed_state_walk(q[:6], k[:6], v[:6], decay, torch.zeros(H, D, V, dtype=F))
    second, end = P.decayed_state_walk(q[6:], k[6:], v[6:], decay, mid)
    assert float((torch.cat([first, second]) - out).abs().max()) < 1e-12 and float((end - S).abs().max()) < 1e-12


def test_the_rotations_are_rotations():
    x, pos = rand(9, 3, 12, seed=1), torch.arange(9)
    plain = P.rot(100.0, 8)
    for interleaved in (False, True):
        y = P.rotate(x, pos, plain, interleaved)
        assert float((y[..., 8:] - x[..., 8:]).abs().max()) == 0.0 and float((y[0] - x[0]).abs().max()) < 1e-15
        assert float((y.norm(dim=-1) - x.norm(dim=-1)).abs().max()) < 1e-12
        # the product of two rotated vectors depends on the distance alone
        a, b = P.rotate(x[:1].expand(9, 3, 12), pos, plain, interleaved), P.rotate(x[1:2].expand(9, 3, 12), pos, plain, interleaved)
        assert float(((a[5] * b[3]).sum(-1) - (a[8] * b[6]).sum(-1)).abs().max()) < 1e-12
    # halves pair entry i with i + dims/2, neighbours 2i with 2i + 1: one is the other with the entries reordered
    order = [0, 4, 1, 5, 2, 6, 3, 7, 8, 9, 10, 11]
    assert float((P.rotate(x[..., order], pos, plain, True) - P.rotate(x, pos, plain, False)[..., order]).abs().max()) < 1e-12
    f, mag = P.stretched_frequencies(P.rot(10000.0, 16, factor=4.0, original=64, fast=32.0, slow=1.0))
    base = 10000.0 ** (-2.0 * torch.arange(8, dtype=F) / 16)
    assert abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-15 and float((f[0] - base[0]).abs()) == 0.0  # the fastest pair is kept
    assert float((f[-1] - base[-1] / 4.0).abs()) < 1e-18 and bool((f <= base).all()) and bool((f >= base / 4.0 - 1e-18).all())


def test_the_sink_is_one_more_term_of_the_denominator():
    cfg = P.model_cfg(16, 11, [P.latent_layer(2, 4, 2, 3, 5, 6, 0.7, P.rot(100.0, 2))])
    w = {k: v.to(F) for k, v in P.random_weights(cfg, 3, stored=torch.float32).items()}
    h = rand(6, 16, seed=2)
    m = cfg["layers"][0]["mixer"]
    with_sink = P.latent_sink_attention(h, w, "l0.mix.", m, 1e-5)
    none = P.latent_sink_attention(h, dict(w, **{"l0.mix.sink": torch.full((2,), -700.0, dtype=F)}), "l0.mix.", m, 1e-5)
    # the first token sees itself alone: without a sink its weight is 1, with one it is e^s / (e^s + e^sink)
    assert float((with_sink[0] - none[0]).abs().max()) > 1e-3
    heavy = P.latent_sink_attention(h, dict(w, **{"l0.mix.sink": torch.full((2,), 700.0, dtype=F)}), "l0.mix.", m, 1e-5)
    assert float(heavy.abs().max()) < 1e-200  # everything goes to the term without a value


def test_the_experts_weights_and_the_token_input():
    cfg = P.model_cfg(12, 9, [P.lightning_layer(1, 4, 4, [0.9], mlp=P.moe(4, 2, 6, shared=5))], side=3)
    w = {k: v.to(F) for k, v in P.random_weights(cfg, 7, stored=torch.float32).items()}
    h = rand(5, 12, seed=1)
    out, chosen = P.routed_experts(h, w, "l0.mlp.", cfg["layers"][0]["mlp"])
    z = h @ w["l0.mlp.router"].T
    for t in range(5):
        a, b = (int(e) for e in chosen.indices[t])
        wa = 1.0 / (1.0 + math.exp(float(z[t, b] - z[t, a])))  # two chosen: a sigmoid of their difference
        want = wa * P.gated_expert(h[t : t + 1], w, f"l0.mlp.e{a}.")[0] + (1 - wa) * P.gated_expert(h[t : t + 1], w, f"l0.mlp.e{b}.")[0]
        want = want + torch.sigmoid(h[t] @ w["l0.mlp.shared.sg"][0]) * P.gated_expert(h[t : t + 1], w, "l0.mlp.shared.")[0]
        assert float((out[t] - want).abs().max()) < 1e-12
    ids = torch.tensor([3, 3, 8, 0, 3])
    y = P.token_input(h, ids, w, "l0.", w["side.embed"][:, :3], 1e-12)
    assert float(((y / w["l0.side.norm"]) ** 2).mean(-1).sub(1).abs().max()) < 1e-6  # normed rows
    assert float((y[0] - y[1]).abs().max()) > 1e-3 and ids[0] == ids[1]  # the same token, gated by other rows
    assert float((P.gelu_tanh(torch.tensor([0.0, 1.0, -1.0], dtype=F)) - torch.tensor([0.0, 0.8411919906, -0.1588080094], dtype=F)).abs().max()) < 1e-9
