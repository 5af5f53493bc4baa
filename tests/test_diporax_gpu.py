"""Diporax on the GPU against the plain implementation in ``plain_diporax``: every new or
changed kernel alone, every mixer alone in a model of one layer, then whole models of three
configurations under the ways of cutting (whole, decoded tail, portions down to two tokens,
mixed batches over a pool of exactly the trace's peak, filled with NaN, whose pages and slots
serve again), keys made loud far back, at the first positions and on both sides of a page's
border (in prompts and decoded), a pair written to the recurrent state hundreds of tokens
before it is read, long decoding beside requests that come and go, the stream after every
layer, and greedy generation through the engine's entry point and the programs."""

import math

import pytest
import torch

import plain_diporax as P
import replay
from halite_amd.config import ModelConfig, ServerConfig
from halite_amd.engine import InferenceEngine
from halite_amd.engine.runner import ModelRunner
from halite_amd.kernels import ops

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 5e-5, "bfloat16": 2.5e-2}  # of the largest logit
CONFIGS = {"A": P.DIP_A, "B": P.DIP_B, "C": P.DIP_C}
LENGTHS = {"A": [5, 70, 33, 1, 130], "B": [90, 2, 41, 160], "C": [64, 17, 150, 3]}
F = torch.float64


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain_logits(cfg, weights, ids):
    return P.forward(cfg, weights, ids).float()


def make_runner(folder, dtype, pool_tokens, page_size=16, graphs=False):
    server = ServerConfig(kv_cache_num_tokens=pool_tokens, page_size=page_size, max_seqs_per_forward=4,
                          use_cudagraph=graphs)
    runner = ModelRunner.from_pretrained(folder, server, ModelConfig(dtype=dtype))
    for g in runner.cache.groups:  # a page that is read before it is written, or after its time, shows
        g.storage.fill_(float("nan"))
    return runner


def sensitivity(cfg, weights, requests, ref):
    """Per request and position: how far the plain model's logits move (of the largest logit)
    when every part's input is rounded to bfloat16."""
    out = {}
    for rid, ids in requests.items():
        moved = P.forward(cfg, weights, ids, round_inputs=torch.bfloat16).float()
        out[rid] = (moved - ref[rid]).abs().amax(-1) / max(1.0, float(ref[rid].abs().max()))
    return out


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        weights = P.random_weights(cfg, seed=5 + len(name) + ord(name))
        requests = {f"r{i}": P.tokens_with_clear_routing(cfg, weights, tokens(cfg, n, 300 + i)) for i, n in enumerate(LENGTHS[name])}
        ref = {rid: plain_logits(cfg, weights, ids) for rid, ids in requests.items()}
        sens = sensitivity(cfg, weights, requests, ref)
        for dtype in DT:
            folder = str(tmp_path_factory.mktemp(f"dip{name}_{dtype}"))
            P.write_model_folder(folder, cfg, weights, DT[dtype])
            out[(name, dtype)] = (folder, requests, ref, weights, sens)
    return out


def check(rows, ref, dtype, sens):
    """float32: every row within the tolerance.  bfloat16: the norms on the parts' results make a
    position whose result nearly cancels as sensitive to the roundings before it as the result is
    small; the plain model with rounded inputs says which positions those are.  So every row
    is finite and within five times the tolerance plus three times its position's sensitivity,
    and all but a few (4%, at least two) within the tolerance plus that."""
    if dtype == "float32":
        return replay.compare(rows, ref, TOL[dtype])
    n = over = 0
    for rid, by_pos in rows.items():
        scale = max(1.0, float(ref[rid].abs().max()))
        for p, row in by_pos.items():
            err = float((row - ref[rid][p]).abs().max()) / scale
            room = 3.0 * float(sens[rid][p])
            assert err <= 5 * TOL[dtype] + room, f"request {rid} position {p}: error {err:.3e} (sensitivity {float(sens[rid][p]):.3e})"
            n, over = n + 1, over + (err > TOL[dtype] + room)
    assert over <= max(2, 0.04 * n), f"{over} of {n} rows beyond the tolerance"


def rand(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def step_arrays(gpu, cuts, slots):
    """The step's arrays for segments of ``cuts`` tokens that belong to ``slots``."""
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)  # noqa: E731
    starts = [sum(cuts[:i]) for i in range(len(cuts))]
    seg = [i for i, n in enumerate(cuts) for _ in range(n)]
    slot = [slots[i] for i, n in enumerate(cuts) for _ in range(n)]
    return i32(seg), i32(starts), i32(cuts), i32(slot)


# -- kernels alone --------------------------------------------------------------------------


@pytest.mark.parametrize("stored", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 16, 16), (1, 48, 8), (3, 8, 24), (2, 20, 70), (2, 64, 64), (1, 130, 5)])
def test_constant_decays_in_steps(gpu, stored, shape):
    """The recurrence with one decay a head over two requests cut into steps of unequal sizes
    (single tokens, two, many), in slots that are not in order, against the whole sequences;
    the state is carried in float32 rows, the rows of other slots hold NaN.  Keys shorter and
    longer than the values, more value channels than a wave, a decay of exactly one."""
    H, N, Pv = shape
    T = {2: 47, 0: 23}
    decay = torch.tensor([1.0, 0.9, 0.999, 0.5][:H], dtype=F)
    rows = {s: rand(t, H * Pv + 2 * H * N, seed=10 + s).to(DT[stored]) for s, t in T.items()}
    want = {}
    for s, a in rows.items():
        b = a.to(F)
        v, k, q = b[:, : H * Pv].view(-1, H, Pv), b[:, H * Pv : H * Pv + H * N].view(-1, H, N), b[:, H * Pv + H * N :].view(-1, H, N)
        want[s] = P.decayed_state_walk(q, k, v, decay, torch.zeros(H, N, Pv, dtype=F))[0].reshape(T[s], H * Pv)
    state = torch.full((4, H, N, Pv), float("nan"), device=gpu)
    state[0].zero_(), state[2].zero_()
    at = {2: 0, 0: 0}
    dec = decay.float().to(gpu)
    for step in ({2: 1, 0: 2}, {2: 2}, {0: 1, 2: 1}, {0: 1, 2: 33}, {2: 1, 0: 1}, {2: 8, 0: 17}, {0: 1, 2: 1}):
        slots = list(step)
        cuts = [step[s] for s in slots]
        a = torch.cat([rows[s][at[s] : at[s] + step[s]] for s in slots]).to(gpu)
        _, starts, lens, slot = step_arrays(gpu, cuts, slots)
        y = ops.ssd_scan(a, None, None, None, None, state, starts, lens, slot, H, fixed_decay=dec).cpu()
        i = 0
        for s in slots:
            ref = want[s][at[s] : at[s] + step[s]]
            assert float((y[i : i + step[s]] - ref).abs().max()) < 3e-5 * max(1.0, float(want[s].abs().max())), (s, at[s])
            i += step[s]
            at[s] += step[s]
    assert at == T and bool(torch.isnan(state[1]).all()) and bool(torch.isnan(state[3]).all())


@pytest.mark.parametrize("in_silu", [False, True])
def test_constant_decays_over_chunks(gpu, in_silu):
    """A long portion cut into chunks that are walked side by side and joined by a carry,
    beside a short one, on states that are not zero; then single tokens on top.  With
    ``in_silu`` the rows are a view into wider float32 rows and go through SiLU as they are read."""
    H, N, Pv, chunk = 3, 24, 40, 64
    T = {1: 301, 3: 70}
    decay = torch.tensor([0.97, 1.0, 0.999], dtype=F)
    rows = {s: rand(t, H * Pv + 2 * H * N, seed=20 + s, scale=0.5) for s, t in T.items()}
    start = 0.3 * rand(4, H, N, Pv, seed=5)
    state = start.clone().to(gpu)
    want = {}
    for s, a in rows.items():
        b = P.silu(a.to(F)) if in_silu else a.to(F)
        v, k, q = b[:, : H * Pv].view(-1, H, Pv), b[:, H * Pv : H * Pv + H * N].view(-1, H, N), b[:, H * Pv + H * N :].view(-1, H, N)
        want[s] = P.decayed_state_walk(q, k, v, decay, start[s].to(F))[0].reshape(T[s], H * Pv)
    at = {1: 0, 3: 0}
    for step in ({1: 300, 3: 69}, {3: 1, 1: 1}):
        slots = list(step)
        cuts = [step[s] for s in slots]
        a = torch.cat([rows[s][at[s] : at[s] + step[s]] for s in slots]).to(gpu)
        if in_silu:
            a = torch.cat([a, torch.full((a.shape[0], 7), float("nan"), device=gpu)], 1)[:, : H * Pv + 2 * H * N]
        _, starts, lens, slot = step_arrays(gpu, cuts, slots)
        chunks = seg_chunks = None
        if max(cuts) >= 2 * chunk:
            per = [-(-n // chunk) for n in cuts]
            first = [sum(per[:i]) for i in range(len(per))]
            rows_ = [[sum(cuts[:s]) + c * chunk, min(chunk, cuts[s] - c * chunk), s, 0] for s in range(len(cuts)) for c in range(per[s])]
            chunks = torch.tensor(rows_, dtype=torch.int32, device=gpu)
            seg_chunks = torch.tensor([[f, n] for f, n in zip(first, per)], dtype=torch.int32, device=gpu)
        y = ops.ssd_scan(a, None, None, None, None, state, starts, lens, slot, H, fixed_decay=decay.float().to(gpu),
                         chunks=chunks, seg_chunks=seg_chunks, in_silu=in_silu).cpu()
        i = 0
        for s in slots:
            ref = want[s][at[s] : at[s] + step[s]]
            assert float((y[i : i + step[s]] - ref).abs().max()) < 3e-5 * max(1.0, float(want[s].abs().max())), (s, at[s])
            i += step[s]
            at[s] += step[s]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 16, 16), (6, 3, 8, 24, 32), (2, 2, 24, 8, 32), (5, 1, 12, 20, 32)])
def test_heads_normed_weighted_and_blended(gpu, dtype, shape):
    """q and k divided by each head's root mean square and multiplied by a weight of the head's
    size, the values left as they are or blended with another layer's; padded to the pages'
    head size."""
    H, K, dq, dv, D = shape
    t = 23
    q, k, v, other = rand(t, H * dq, seed=1, scale=2.0), rand(t, K * dq, seed=2, scale=0.3), rand(t, K * dv, seed=3), rand(t, K * dv, seed=4)
    wq, wk = (1 + 0.3 * rand(dq, seed=5)).to(DT[dtype]), (1 + 0.3 * rand(dq, seed=6)).to(DT[dtype])
    tol = 1e-5 if dtype == "float32" else 1e-2
    for blend in (None, 0.35):
        packed = ops.head_norm_pack(q.to(gpu), k.to(gpu), v.to(gpu), 1e-5, H, K, dq, dv, D, DT[dtype], w_q=wq.to(gpu),
                                    w_k=wk.to(gpu), norm_v=False, v_other=None if blend is None else other.to(gpu),
                                    v_mix=blend or 0.0)
        got = packed.float().cpu().view(t, H + 2 * K, D)
        want_v = v.to(F) if blend is None else (1 - blend) * v.to(F) + blend * other.to(F)
        for part, want, d in ((got[:, :H], P.rms_unit(q.to(F).view(t, H, dq), 1e-5) * wq.to(F), dq),
                              (got[:, H : H + K], P.rms_unit(k.to(F).view(t, K, dq), 1e-5) * wk.to(F), dq),
                              (got[:, H + K :], want_v.view(t, K, dv), dv)):
            assert float((part[..., :d] - want).abs().max()) < tol * float(want.abs().max())
            assert float(part[..., d:].abs().max() if D > d else 0.0) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_passes_over_rows(gpu, dtype):
    """A bias added to a column range of float32 rows in place; SiLU of a column range; the
    gated row of a token's part of a table (a token outside the table gives NaN, not a fault)."""
    t, c = 19, 70
    a, bias = rand(t, c + 9, seed=1), rand(c, seed=2).to(DT[dtype])
    ag = a.to(gpu)
    ops.bias_rows_(ag[:, 5 : 5 + c], bias.to(gpu))
    want = a.clone()
    want[:, 5 : 5 + c] += bias.float()
    assert float((ag.cpu() - want).abs().max()) < 1e-6
    got = ops.silu_rows(a.to(gpu)[:, 3 : 3 + c], DT[dtype]).float().cpu()
    ref = P.silu(a[:, 3 : 3 + c].to(F))
    assert float((got - ref).abs().max()) < (1e-6 if dtype == "float32" else 1e-2) * float(ref.abs().max())
    table, g = rand(31, 24, seed=3).to(DT[dtype]), rand(t, 6 + 8, seed=4, scale=2.0)
    ids = torch.randint(0, 31, (t,), generator=torch.Generator().manual_seed(5)).to(torch.int32)
    ids[4] = 31  # outside
    got = ops.token_gate(g.to(gpu)[:, 6:], table.to(gpu), 8, ids.to(gpu), DT[dtype]).float().cpu()
    ok = ids < 31
    ref = P.gelu_tanh(g[:, 6:].to(F))[ok] * table.to(F)[ids[ok].long(), 8:16]
    assert float((got[ok] - ref).abs().max()) < (2e-6 if dtype == "float32" else 1e-2) * float(ref.abs().max())
    assert bool(torch.isnan(got[4]).all())


def test_routing_weights_and_gates(gpu):
    """The softmax over the chosen logits alone, from a column range of wider rows; the plain
    SiLU gate as the clamped gate without limit and shift; the weighted sum with an extra row
    behind a sigmoid of its own."""
    t, E, top, d = 37, 11, 3, 20
    z = rand(t, E + 1, seed=1, scale=2.0)
    idx, wgt = ops.moe_route(z.to(gpu)[:, :E], top, softmax=True, normalize=True, norm_eps=0.0)
    chosen = torch.topk(z[:, :E].to(F), top, dim=-1)
    assert torch.equal(idx.cpu().long(), chosen.indices)
    assert float((wgt.cpu() - torch.softmax(chosen.values, -1)).abs().max()) < 1e-6
    # the same, and the pairs sorted by expert, from one launch
    idx2, wgt2, offsets, tiles, order = ops.moe_route_sort(z.to(gpu)[:, :E], top, E, softmax=True, normalize=True, norm_eps=0.0)
    assert torch.equal(idx2, idx) and torch.equal(wgt2, wgt)
    o, pairs, flat = offsets.cpu().tolist(), order.cpu().tolist(), idx.cpu().flatten().tolist()
    assert o[0] == 0 and o[E] == t * top and sorted(pairs) == list(range(t * top))
    assert all(flat[pairs[i]] == e for e in range(E) for i in range(o[e], o[e + 1]))
    assert tiles.cpu().tolist() == [sum(-(-(o[j + 1] - o[j]) // ops.GROUP_TILE_ROWS) for j in range(e)) for e in range(E + 1)]
    gu = rand(t, 2 * d, seed=2, scale=3.0)
    got = ops.clamped_gate_mul(gu.to(gpu), math.inf, 1.0, 0.0).cpu()
    assert float((got - P.silu(gu[:, :d].to(F)) * gu[:, d:].to(F)).abs().max()) < 1e-5
    h, y, extra = rand(t, d, seed=3), rand(t * top, d, seed=4), rand(t, d, seed=5)
    hg = h.to(gpu)
    ops.moe_combine(hg, y.to(gpu), wgt, extra.to(gpu), extra_gate=z.to(gpu)[:, E:])
    want = h.to(F) + (wgt.cpu().to(F)[:, :, None] * y.to(F).view(t, top, d)).sum(1) + torch.sigmoid(z[:, E:].to(F)) * extra.to(F)
    assert float((hg.cpu() - want).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(1, 1100), (3, 512), (1, 96), (2, 4096)])
def test_rows_normed_weighted_and_gated(gpu, dtype, shape):
    """The heads of a row (one head: the whole row) divided by their root mean square, times a
    weight and the sigmoid of a gate; narrow heads a wave each, wide ones a workgroup each."""
    H, D = shape
    t = 9
    y, a = rand(t, H * D, seed=1, scale=3.0), rand(t, 5 + H * D, seed=2)
    w = (1 + 0.2 * rand(H * D, seed=3)).to(DT[dtype])
    got = ops.head_norm_gate(y.to(gpu), a.to(gpu)[:, 5:], w.to(gpu), 1e-5, H, DT[dtype]).float().cpu()
    want = P.rms_unit(y.to(F).view(t, H, D), 1e-5).reshape(t, H * D) * w.to(F) * torch.sigmoid(a[:, 5:].to(F))
    assert float((got - want).abs().max()) < (1e-5 if dtype == "float32" else 2e-2) * float(want.abs().max())


@pytest.mark.parametrize("sizes", [(3, 4096, 4), (70, 40, 2), (300, 1024, 1), (1, 520, 3)])
def test_weighted_sum_of_the_chosen_experts(gpu, sizes):
    """Few tokens spread a row over several workgroups, many take one each: the same sums."""
    t, d, top = sizes
    h, y, wgt, extra, g = rand(t, d, seed=1), rand(t * top, d, seed=2), rand(t, top, seed=3).abs(), rand(t, d, seed=4), rand(t, 1, seed=5)
    hg = h.to(gpu)
    ops.moe_combine(hg, y.to(gpu), wgt.to(gpu), extra.to(gpu), extra_gate=g.to(gpu))
    want = h.to(F) + (wgt.to(F)[:, :, None] * y.to(F).view(t, top, d)).sum(1) + torch.sigmoid(g.to(F)) * extra.to(F)
    assert float((hg.cpu() - want).abs().max()) < 1e-5
    fresh = torch.full((t, d), float("nan"), device=gpu)  # written, not added to
    ops.moe_combine(fresh, y.to(gpu), wgt.to(gpu), extra.to(gpu), extra_gate=g.to(gpu), overwrite=True)
    assert float((fresh.cpu() - (want - h.to(F))).abs().max()) < 1e-5


def test_stretched_rotation_tables(gpu):
    """The rotary part's table against the plain frequencies: the ramp between fast and slow
    pairs, and cosine and sine times the stretch's magnitude."""
    from halite_amd.parts.base import BuildContext
    from halite_amd.parts.rope import Rope, RopeParams

    for r in (P.rot(1000.0, 8, factor=4.0), P.rot(77.0, 6, factor=8.0, original=16, fast=4.0, slow=0.5), P.rot(50.0, 4),
              P.rot(1000000.0, 48, factor=3.0, original=512, fast=16.0, slow=2.0)):
        s = r.get("scaling")
        params = RopeParams(head_dim=r["dims"], rotary_dim=r["dims"], theta=r["base"], max_positions=4096, angles="float64",
                            scaling=None if s is None else dict(kind="ramp", factor=s["factor"], original_context_len=s["original"],
                                                                fast_turns=s["fast"], slow_turns=s["slow"]),
                            magnitude=1.0 if s is None else 0.1 * math.log(s["factor"]) + 1.0)
        cos, sin = Rope(params, BuildContext(dtype=torch.float32, device=gpu, hidden_size=8)).tables(700)
        f, mag = P.stretched_frequencies(r)
        a = torch.arange(700, dtype=F)[:, None] * f[None, :]
        assert float((cos[:700].cpu() - torch.cos(a) * mag).abs().max()) < 1e-6
        assert float((sin[:700].cpu() - torch.sin(a) * mag).abs().max()) < 1e-6


# -- every mixer alone --------------------------------------------------------------------------

ONE_LAYER = {
    "attention": P.model_cfg(32, 97, [P.attention_layer(4, 2, 8, 12, 0.4, conv=3, rot=P.rot(500.0, 4, factor=3.0, original=16),
                                                        softcap=3.0)]),
    "attention_bare": P.model_cfg(32, 97, [P.attention_layer(3, 3, 8, 8, 0.4)]),
    "latent": P.model_cfg(32, 97, [P.latent_layer(3, 8, 4, 12, 9, 14, 0.4, P.rot(500.0, 4, factor=3.0, original=16))]),
    "lightning": P.model_cfg(32, 97, [P.lightning_layer(3, 8, 12, [0.8, 0.99, 1.0])]),
    "experts": P.model_cfg(32, 97, [P.lightning_layer(1, 8, 8, [0.9], mlp=P.moe(7, 2, 12, shared=10))]),
    "token_input": P.model_cfg(32, 97, [P.lightning_layer(1, 8, 8, [0.9])], side=5),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ONE_LAYER))
def test_one_layer_models(name, dtype, tmp_path):
    """A model of one layer for each mixer (the attention with and without its optional pieces),
    for the experts and for the token input: a prompt whole against token by token and portions."""
    cfg = ONE_LAYER[name]
    w = P.random_weights(cfg, seed=31)
    if name == "latent":
        w["l0.mix.sink"][:] = torch.tensor([2.0, -1.0, 0.5])  # sinks that count
    requests = {"a": P.tokens_with_clear_routing(cfg, w, tokens(cfg, 50, 1)), "b": P.tokens_with_clear_routing(cfg, w, tokens(cfg, 21, 2))}
    ref = {rid: plain_logits(cfg, w, ids) for rid, ids in requests.items()}
    sens = sensitivity(cfg, w, requests, ref)
    folder = P.write_model_folder(str(tmp_path), cfg, w, DT[dtype])
    for make in (replay.whole, lambda q: replay.tail_one_by_one(q, tail=50), replay.portions, replay.mixed):
        trace = make(requests)
        runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16))
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
        check(rows, ref, dtype, sens)
        assert runner.cache.idle()


def test_a_sink_and_a_cap_change_the_result(tmp_path):
    """The plain model itself: without the sink's term, or without the cap, the logits differ by
    much more than the tests' tolerance, so a kernel that left either out would show."""
    for name, key in (("latent", "sink"), ("attention", "softcap")):
        cfg = ONE_LAYER[name]
        w = P.random_weights(cfg, seed=31)
        ids = tokens(cfg, 40, 1)
        if key == "sink":
            w["l0.mix.sink"][:] = torch.tensor([2.0, -1.0, 0.5])
            other_w, other_cfg = dict(w, **{"l0.mix.sink": torch.full((3,), -60.0)}), cfg
        else:
            w["l0.mix.q.norm"] *= 4.0  # scores beyond the cap
            other_w = w
            other_cfg = P.model_cfg(32, 97, [dict(cfg["layers"][0], mixer={k: v for k, v in cfg["layers"][0]["mixer"].items() if k != key})])
        a, b = plain_logits(cfg, w, ids), plain_logits(other_cfg, other_w, ids)
        assert float((a - b).abs().max()) > 0.02 * float(a.abs().max())


# -- whole models -----------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed", "mixed2"])
def test_schedules(folders, name, dtype, schedule):
    folder, requests, ref, _, sens = folders[(name, dtype)]
    cfg = CONFIGS[name]
    make = {"whole": replay.whole, "tail": lambda q: replay.tail_one_by_one(q, tail=40), "portions": replay.portions,
            "mixed": replay.mixed, "mixed2": lambda q: replay.mixed(q, seed=7, decode_tail=30)}[schedule]
    trace = make(requests)
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16))
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
    check(rows, ref, dtype, sens)
    assert runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [8, 32, 64])
@pytest.mark.parametrize("name", ["A", "C"])
def test_other_page_sizes(folders, name, page_size, dtype):
    folder, requests, ref, _, sens = folders[(name, dtype)]
    trace = replay.mixed(requests, seed=3)
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, page_size), page_size=page_size)
    rows = replay.collect(trace, replay.run_trace(runner, trace), CONFIGS[name]["vocab"])
    check(rows, ref, dtype, sens)
    assert runner.cache.idle()


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_stream_after_every_layer(folders, name):
    from halite_amd.parts import block

    folder, requests, _, weights, _ = folders[(name, "float32")]
    cfg = CONFIGS[name]
    ids = requests["r1"]
    want = []
    P.forward(cfg, weights, ids, layers_out=want)
    runner = make_runner(folder, "float32", 256)
    seen, inner = [], block.PostNormBlock.forward

    def forward(self, h, pending, ctx, run):
        out = inner(self, h, pending, ctx, run)
        seen.append(h.clone())
        return out

    block.PostNormBlock.forward = forward
    try:
        replay.run_trace(runner, replay.whole({"r1": ids}))
    finally:
        block.PostNormBlock.forward = inner
    assert len(seen) == len(want) == len(cfg["layers"])
    for got, w in zip(seen, want):
        assert float((got.cpu() - w.float()).abs().max()) < 5e-5 * max(1.0, float(w.abs().max()))


# -- keys made loud -----------------------------------------------------------------------------

LOUD, ASK = 7, 11


def mark_embedding(w):
    """Channel 0 of the embedding is nonzero for LOUD alone and channel 1 for ASK alone (the
    embedding's norm keeps zeros), so a projection that reads one of them tells that token from
    all others."""
    w["embed"][:, :2] = 0.0
    w["embed"][LOUD, 0] = 3.0
    w["embed"][ASK, 1] = 3.0
    w["embed.norm"][:2] = 1.0


def loud_attention_model(kv_heads=1, conv=3):
    """One attention layer whose weights stand out for one pair of tokens: key channel 12 (which
    is not rotated) is large for LOUD and zero for every other token, query channel 12 large for
    ASK and zero otherwise (the biases of that channel are zero and the convolutions pass it
    unmixed), so after the norms per head ASK's score on LOUD is nearly ``scale * dim`` (under the
    cap) where all other scores are small: ASK attends to LOUD wherever it is."""
    cfg = P.model_cfg(64, 61, [P.attention_layer(2, kv_heads, 16, 24, 1.5, conv=conv, rot=P.rot(1000.0, 8, factor=2.0, original=32),
                                                 softcap=40.0)], side=4)
    w = P.random_weights(cfg, seed=77)
    mark_embedding(w)
    for n, heads in (("k", kv_heads), ("q", 2)):
        w[f"l0.mix.{n}"] *= 0.2
        w[f"l0.mix.{n}.b"] *= 0.2
        for head in range(heads):
            row = head * 16 + 12
            w[f"l0.mix.{n}"][row] = 0.0
            w[f"l0.mix.{n}"][row, 0 if n == "k" else 1] = 4.0
            w[f"l0.mix.{n}.b"][row] = 0.0
            if conv:
                w[f"l0.mix.{n}.conv"][row] = 0.0
                w[f"l0.mix.{n}.conv"][row, -1] = 1.0
    w["l0.mix.g"] *= 0.1
    w["l0.mix.o"] *= 3.0
    return cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}


def loud_latent_model():
    """One latent attention whose latent's entry 0 is large for LOUD and zero for every other
    token and whose query latent's entry 0 is large for ASK alone; every head's key and query
    read those entries in their channel 0 (not rotated)."""
    cfg = P.model_cfg(64, 61, [P.latent_layer(2, 16, 8, 24, 12, 24, 1.2, P.rot(1000.0, 8, factor=2.0, original=32))], side=4)
    w = P.random_weights(cfg, seed=78)
    mark_embedding(w)
    w["l0.mix.dkv"] *= 0.2
    w["l0.mix.dq"] *= 0.2
    w["l0.mix.dkv"][0], w["l0.mix.dq"][0] = 0.0, 0.0
    w["l0.mix.dkv"][0, 0], w["l0.mix.dq"][0, 1] = 4.0, 4.0
    w["l0.mix.dkv.norm"][0] = w["l0.mix.dq.norm"][0] = 1.0
    w["l0.mix.uk"][:, 0] = 0.0
    w["l0.mix.uq"][:, 0] = 0.0
    for head in range(2):
        w["l0.mix.uk"][head * 16, 0] = 1.0
        w["l0.mix.uq"][head * 24, 0] = 1.0
    w["l0.mix.g"] *= 0.1
    w["l0.mix.o"] *= 3.0
    return cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}


def loud_lightning_model():
    """One lightning layer that forgets next to nothing, whose key channel 0 is large for LOUD
    and zero for every other token (SiLU keeps zeros) and whose query channel 0 is large for ASK
    alone: what ASK reads is mostly LOUD's value, however long ago it was written."""
    cfg = P.model_cfg(64, 61, [P.lightning_layer(2, 16, 24, [0.9995, 1.0])], side=4)
    w = P.random_weights(cfg, seed=79)
    mark_embedding(w)
    for n, col in (("k", 0), ("q", 1)):
        w[f"l0.mix.{n}"] *= 0.1
        for head in range(2):
            w[f"l0.mix.{n}"][head * 16] = 0.0
            w[f"l0.mix.{n}"][head * 16, col] = 2.0
        w[f"l0.mix.{n}"][:, :2][[r for r in range(32) if r % 16]] = 0.0
    w["l0.mix.o"] *= 3.0
    return cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}


def loud_sequence(cfg, n, loud_at, ask_at, seed):
    ids = [t if t not in (LOUD, ASK) else 1 for t in tokens(cfg, n, seed)]
    for p in loud_at:
        ids[p] = LOUD
    for p in ask_at:
        ids[p] = ASK
    return ids


def replay_all(cfg, w, requests, dtype, tmp_path, tail=80, page_size=16):
    ref = {rid: plain_logits(cfg, w, ids) for rid, ids in requests.items()}
    sens = sensitivity(cfg, w, requests, ref) if dtype == "bfloat16" else None
    folder = P.write_model_folder(str(tmp_path), cfg, w, DT[dtype])
    for make in (replay.whole, lambda q: replay.tail_one_by_one(q, tail=tail), replay.portions,
                 lambda q: replay.portions(q, sizes=(15, 1, 32, 2, 1, 1, 16, 64)), replay.mixed):
        trace = make(requests)
        runner = make_runner(folder, dtype, replay.peak_tokens(trace, page_size), page_size=page_size)
        rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
        check(rows, ref, dtype, sens)
        assert runner.cache.idle()
    return ref


def quiet(ids):
    return [1 if t == LOUD else t for t in ids]


LOUD_MODELS = {"attention": loud_attention_model, "attention_two_kv": lambda: loud_attention_model(kv_heads=2, conv=None),
               "latent": loud_latent_model, "lightning": loud_lightning_model}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("model", list(LOUD_MODELS))
def test_a_loud_token_far_back_and_at_the_first_positions(model, dtype, tmp_path):
    """LOUD at position 3 (and at 0) among hundreds of tokens across many pages; ASK right
    behind it, far behind it, and at the last position."""
    cfg, w = LOUD_MODELS[model]()
    requests = {"far": loud_sequence(cfg, 400, [3], [4, 200, 255, 256, 399], 2),
                "first": loud_sequence(cfg, 300, [0], [1, 150, 299], 3)}
    ref = replay_all(cfg, w, requests, dtype, tmp_path)
    silent = plain_logits(cfg, w, quiet(requests["far"]))
    assert float((ref["far"][399] - silent[399]).abs().max()) > 0.1 * float(ref["far"].abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("model,page_size", [("attention", 16), ("latent", 16), ("attention", 32), ("latent", 64)])
def test_loud_keys_on_both_sides_of_a_pages_border(model, page_size, dtype, tmp_path):
    """LOUD in the last slot of a page and in the first slot of the next one, ASK in the slots
    around them and a few pages on; the schedules put these places into prompts and into
    decoded tokens."""
    cfg, w = LOUD_MODELS[model]()
    n = 4 * page_size + 9
    requests = {"last_slot": loud_sequence(cfg, n, [2 * page_size - 1], [2 * page_size, 2 * page_size + 1, 3 * page_size - 1, 3 * page_size, n - 1], 4),
                "first_slot": loud_sequence(cfg, n, [2 * page_size], [2 * page_size + 1, 3 * page_size - 1, 3 * page_size, n - 1], 5)}
    ref = replay_all(cfg, w, requests, dtype, tmp_path, tail=2 * page_size + 12, page_size=page_size)
    for rid in requests:
        silent = plain_logits(cfg, w, quiet(requests[rid]))
        assert float((ref[rid][n - 1] - silent[n - 1]).abs().max()) > 0.1 * float(ref[rid].abs().max())


# -- long decoding, slots and pages that serve again ------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_long_decoding_beside_requests_that_come_and_go(folders, dtype, graphs):
    """A short prompt and 200 tokens decoded one by one (the recurrence runs on, the blended
    values and the convolutions' inputs are carried) beside short requests that take the freed
    slot and pages one after the other."""
    folder, _, _, weights, _ = folders[("A", dtype)]
    cfg = P.DIP_A
    ids, other = (P.tokens_with_clear_routing(cfg, weights, tokens(cfg, n, seed)) for n, seed in ((215, 41), (30, 42)))
    ref = {"long": plain_logits(cfg, weights, ids)}
    short = plain_logits(cfg, weights, other)
    sens = sensitivity(cfg, weights, {"long": ids, "other": other}, {"long": ref["long"], "other": short})
    trace = [{"step": 0, "entries": [{"id": "long", "tokens": ids[:15], "want": list(range(15))}], "end": []}]
    for i in range(15, 215):
        entries = [{"id": "long", "tokens": [ids[i]], "want": [0]}]
        j, rid = (i - 15) % 40, f"other{(i - 15) // 40}"
        if j < 30:
            entries.append({"id": rid, "tokens": [other[j]], "want": [0]})
            ref[rid], sens[rid] = short, sens["other"]
        trace.append({"step": len(trace), "entries": entries,
                      "end": (["long"] if i == 214 else []) + ([rid] if j == 29 else [])})
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16), graphs=graphs)
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
    check(rows, ref, dtype, sens)
    assert runner.cache.idle()
    if graphs:
        assert runner.graphs_allowed and runner.graph_replays > 100


# -- through the engine's entry point ----------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    folder, _, _, weights, _ = folders[(name, dtype)]
    cfg = CONFIGS[name]
    prompts = [P.tokens_with_clear_routing(cfg, weights, tokens(cfg, n, 500 + n)) for n in (5, 17, 33, 2, 48, 9)]
    engine = InferenceEngine.from_pretrained(
        folder, ServerConfig(kv_cache_num_tokens=1024, page_size=16, max_seqs_per_forward=3, chunked_prefill_size=20,
                             max_tokens_per_forward=24),
        ModelConfig(dtype=dtype),
    )
    params = {"max_new_tokens": 12, "temperature": 0.0}
    results = engine.infer_batch([(i, p, params) for i, p in enumerate(prompts)])
    checked = 0
    for r, prompt in zip(results, prompts):
        ids = list(prompt)
        for step, tok in enumerate(r.output_ids[0]):
            margins = []
            logits = P.forward(cfg, weights, ids, margins_out=margins).float()[-1]
            if dtype == "bfloat16" and margins and float(torch.stack(margins).min()) < 0.1:
                break  # a router's close call among the generated tokens: 16 bits may take the other expert from here on
            best = int(torch.argmax(logits))
            if tok != best:  # 16 bits may turn a near tie; anything else is a fault
                gap = float(logits[best] - logits[tok])
                assert gap < (1e-4 if dtype == "float32" else 0.05), f"request {r.id} token {step}: {tok} for {best}, gap {gap}"
            ids.append(tok)
        assert len(r.output_ids[0]) == 12
        checked += len(ids) - len(prompt)
    # (a model with a router in every layer meets a close call among twelve generated tokens more
    # often than not; in 16 bits the comparison of a request ends there)
    assert checked >= (36 if dtype == "float32" else 12)


# -- the programs: generation from the command line, the random-weights mode, trace replay -----


def test_command_line_and_replay_program(folders, tmp_path):
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, _, _, weights, _ = folders[("A", "float32")]
    cfg = P.DIP_A
    cmd = [sys.executable, os.path.join(root, "bin", "halite_generate"), "--model", folder, "--prompt-ids", "5,17,3,90,9",
           "sampling.temperature=0", "sampling.max_new_tokens=5", "model.dtype=float32", "server.kv_cache_num_tokens=256"]
    proc = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().split("\n")[-1])
    ids = [5, 17, 3, 90, 9]
    for tok in rec["output_ids"][0]:
        assert tok == int(torch.argmax(plain_logits(cfg, weights, ids)[-1]))
        ids.append(tok)
    assert len(ids) == 10
    # the random-weights mode: a configuration without tensors states whether its attentions'
    # projections have biases; the folder it writes holds the design's own keys
    stated = json.loads(json.dumps(P.DIP_C))
    stated["layers"][0]["mixer"]["bias"] = True
    cfgfile, out = tmp_path / "c.json", tmp_path / "rand"
    cfgfile.write_text(json.dumps(stated))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "halite_make_random_model"), "--config", str(cfgfile),
                           "--out", str(out), "--seed", "3", "--dtype", "bfloat16", "--std", "0.1"], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert '"bias"' not in (out / "config.json").read_text()
    # the replay program on that folder: a prompt in two portions and a decoded token, beside a
    # second request; two slots, so the third request takes the one that was freed
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3, 4, 5], "want": [4]}, {"id": "b", "tokens": [7], "want": [0]}], "end": ["b"]},
        {"step": 1, "entries": [{"id": "a", "tokens": [6, 7], "want": []}, {"id": "c", "tokens": [9, 8], "want": [1]}], "end": ["c"]},
        {"step": 2, "entries": [{"id": "a", "tokens": [8], "want": [0]}], "end": ["a"]},
    ]
    logits = tmp_path / "logits"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(out), "--dtype", "float32",
                           "--out", str(logits), "--max-tokens", "128", "--slots", "2"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    from safetensors.torch import load_file

    stored = {k: v.float() for k, v in load_file(str(out / "model.safetensors")).items()}
    want = plain_logits(P.DIP_C, stored, [1, 2, 3, 4, 5, 6, 7, 8])
    got0 = torch.from_numpy(np.fromfile(logits / "0.f32", dtype="<f4").reshape(2, -1))
    got1 = torch.from_numpy(np.fromfile(logits / "1.f32", dtype="<f4").reshape(1, -1))
    got2 = torch.from_numpy(np.fromfile(logits / "2.f32", dtype="<f4").reshape(1, -1))
    scale = max(1.0, float(want.abs().max()))
    assert float((got0[0] - want[4]).abs().max()) < 5e-5 * scale and float((got2[0] - want[7]).abs().max()) < 5e-5 * scale
    assert float((got0[1] - plain_logits(P.DIP_C, stored, [7])[0]).abs().max()) < 5e-5 * scale
    assert float((got1[0] - plain_logits(P.DIP_C, stored, [9, 8])[1]).abs().max()) < 5e-5 * scale
