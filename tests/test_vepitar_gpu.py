"""Vepitar on the GPU against the plain implementation in ``plain_vepitar``: every new
kernel alone, then whole models of three configurations under the four ways of cutting
(whole, decoded tail, portions down to two tokens, mixed batches over a pool of exactly
the trace's peak, filled with NaN, whose pages and slots serve again), keys made loud far
back, at the first positions and on both sides of a window's edge (also where that edge is
a page's), a pair written to the recurrent state hundreds of tokens before it is read, long
decoding beside requests that come and go, the stream after every layer, and greedy
generation through the engine's entry point and the programs."""

import math

import pytest
import torch

import plain_vepitar as P
import replay
from halite_amd.config import ModelConfig, ServerConfig
from halite_amd.engine import InferenceEngine
from halite_amd.engine.runner import ModelRunner
from halite_amd.kernels import ops

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 5e-5, "bfloat16": 2.5e-2}  # of the largest logit
CONFIGS = {"A": (P.VEP_A, P.VEP_A_RANKS), "B": (P.VEP_B, P.VEP_B_RANKS), "C": (P.VEP_C, P.VEP_C_RANKS)}
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


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (cfg, ranks) in CONFIGS.items():
        weights = P.random_weights(cfg, ranks, seed=5 + len(name))
        requests = {f"r{i}": P.tokens_with_clear_routing(cfg, weights, tokens(cfg, n, 300 + i)) for i, n in enumerate(LENGTHS[name])}
        ref = {rid: plain_logits(cfg, weights, ids) for rid, ids in requests.items()}
        sens = sensitivity(cfg, weights, requests, ref)
        for dtype in DT:
            folder = str(tmp_path_factory.mktemp(f"vep{name}_{dtype}"))
            P.write_model_folder(folder, cfg, weights, DT[dtype])
            out[(name, dtype)] = (folder, requests, ref, weights, sens)
    return out


def sensitivity(cfg, weights, requests, ref):
    """Per request and position: how far the plain model's logits move (of the largest logit)
    when every part's input is rounded to bfloat16."""
    out = {}
    for rid, ids in requests.items():
        moved = P.forward(cfg, weights, ids, round_inputs=torch.bfloat16).float()
        out[rid] = (moved - ref[rid]).abs().amax(-1) / max(1.0, float(ref[rid].abs().max()))
    return out


def check(rows, ref, dtype, sens):
    """float32: every row within the tolerance.  bfloat16: the per-head norms make a position
    whose head nearly cancels (the first tokens of a recurrence, where one pair's sign decides)
    as sensitive to the roundings before it as that head is small; the plain model with
    rounded inputs says which positions those are.  So every row is finite and within five
    times the tolerance plus three times its position's sensitivity, and all but a few (4%,
    at least two) within the tolerance plus that."""
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
@pytest.mark.parametrize("shape", [(4, 16, 8), (1, 48, 3), (5, 8, 6), (2, 24, 5), (2, 64, 4), (3, 80, 2), (1, 132, 7),
                                   (3, 32, 4), (2, 128, 3)])
def test_delta_rule_in_steps(gpu, stored, shape):
    """The recurrence over two requests cut into steps of unequal sizes (single tokens, two,
    many, more than a block of the walk), in slots that are not in order, against the whole
    sequences; the state is carried in float32 rows, and the rows of other slots hold NaN.
    Heads of 8 to 132 channels: fewer than a wave's quarter holds, and more than one block of
    value channels; steps of single tokens alone take a kernel of their own for heads of 32,
    64 and 128."""
    H, D, rank = shape
    n = H * D
    T = {2: 47, 0: 23}
    w2, w0, ab = (rand(n, rank, seed=1, scale=0.8).to(DT[stored]), rand(n, seed=2, scale=1.5).to(DT[stored]),
                  rand(n, seed=3).to(DT[stored]))
    rows = {s: rand(t, 3 + 4 * n + rank, seed=10 + s) for s, t in T.items()}
    want = {}
    for s, a in rows.items():
        b = a[:, 3:].to(F)
        r, k, v, a_raw, x1 = b[:, :n], b[:, n : 2 * n], b[:, 2 * n : 3 * n], b[:, 3 * n : 4 * n], b[:, 4 * n :]
        decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(x1) @ w2.to(F).T + w0.to(F))).view(-1, H, D)
        rate = torch.sigmoid(a_raw + ab.to(F)).view(-1, H, D)
        o = torch.zeros(T[s], H, D, dtype=F)
        for h in range(H):
            o[:, h], _ = P.delta_recurrence(r.view(-1, H, D)[:, h], k.view(-1, H, D)[:, h], v.view(-1, H, D)[:, h],
                                            decay[:, h], rate[:, h], torch.zeros(D, D, dtype=F))
        want[s] = o.reshape(T[s], n)
    state = torch.full((4, H, D, D), float("nan"), device=gpu)
    state[0].zero_(), state[2].zero_()
    at = {2: 0, 0: 0}
    for step in ({2: 1, 0: 2}, {2: 2}, {0: 1, 2: 1}, {0: 1, 2: 33}, {2: 1, 0: 1}, {2: 8, 0: 17}, {0: 1, 2: 1}):
        slots = list(step)
        cuts = [step[s] for s in slots]
        a = torch.cat([rows[s][at[s] : at[s] + step[s]] for s in slots]).to(gpu)[:, 3:]  # rows that begin off 16 bytes
        _, starts, lens, slot = step_arrays(gpu, cuts, slots)
        y = ops.delta_rule(a[:, :n], a[:, n : 2 * n], a[:, 2 * n : 3 * n], a[:, 3 * n : 4 * n], a[:, 4 * n :], w2.to(gpu),
                           w0.to(gpu), ab.to(gpu), state, starts, lens, slot, math.exp(-0.5), 1e-6).cpu()
        i = 0
        for s in slots:
            ref = want[s][at[s] : at[s] + step[s]]
            assert float((y[i : i + step[s]] - ref).abs().max()) < 3e-5 * max(1.0, float(want[s].abs().max())), (s, at[s])
            i += step[s]
            at[s] += step[s]
    assert at == T and bool(torch.isnan(state[1]).all()) and bool(torch.isnan(state[3]).all())


@pytest.mark.parametrize("shape", [(2, 64, 40), (3, 24, 5), (1, 128, 33)])
def test_delta_rule_over_a_long_portion(gpu, shape):
    """Hundreds of tokens in one step (many blocks of the walk, and the kernel that makes the
    vectors of sixteen tokens at a time, with a rank that is no multiple of its tile) beside a
    short request, then a step of single tokens on top of the states they left."""
    H, D, rank = shape
    n = H * D
    T = {1: 301, 3: 6}
    w2, w0, ab = rand(n, rank, seed=1, scale=0.8), rand(n, seed=2, scale=1.5), rand(n, seed=3)
    rows = {s: rand(t, 4 * n + rank, seed=20 + s) for s, t in T.items()}
    want = {}
    for s, a in rows.items():
        b = a.to(F)
        r, k, v, a_raw = (b[:, i * n : (i + 1) * n].view(-1, H, D) for i in range(4))
        x1 = b[:, 4 * n :]
        decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(x1) @ w2.to(F).T + w0.to(F))).view(-1, H, D)
        rate = torch.sigmoid(a_raw + ab.to(F).view(H, D))
        o = torch.zeros(T[s], H, D, dtype=F)
        for h in range(H):
            o[:, h], _ = P.delta_recurrence(r[:, h], k[:, h], v[:, h], decay[:, h], rate[:, h], torch.zeros(D, D, dtype=F))
        want[s] = o.reshape(T[s], n)
    state = torch.zeros((4, H, D, D), device=gpu)
    at = {1: 0, 3: 0}
    for step in ({1: 300, 3: 5}, {3: 1, 1: 1}):
        slots = list(step)
        cuts = [step[s] for s in slots]
        a = torch.cat([rows[s][at[s] : at[s] + step[s]] for s in slots]).to(gpu)
        _, starts, lens, slot = step_arrays(gpu, cuts, slots)
        y = ops.delta_rule(a[:, :n], a[:, n : 2 * n], a[:, 2 * n : 3 * n], a[:, 3 * n : 4 * n], a[:, 4 * n :], w2.to(gpu),
                           w0.to(gpu), ab.to(gpu), state, starts, lens, slot, math.exp(-0.5), 1e-6).cpu()
        i = 0
        for s in slots:
            ref = want[s][at[s] : at[s] + step[s]]
            assert float((y[i : i + step[s]] - ref).abs().max()) < 3e-5 * max(1.0, float(want[s].abs().max())), (s, at[s])
            i += step[s]
            at[s] += step[s]


def test_delta_rule_over_many_requests(gpu):
    """So many segments that the walk takes its other layout for heads of 64 (sixteen value
    channels a wave): 170 requests of 2 to 11 tokens each on states that are not zero."""
    H, D, rank, R = 4, 64, 8, 170
    n = H * D
    w2, w0, ab = rand(n, rank, seed=1, scale=0.8), rand(n, seed=2, scale=1.5), rand(n, seed=3)
    lens = [2 + (7 * i) % 10 for i in range(R)]
    a = rand(sum(lens), 4 * n + rank, seed=4)
    start = 0.3 * rand(R, H, D, D, seed=5)
    state = start.clone().to(gpu)
    slots = list(range(R - 1, -1, -1))  # request i lives in slot R - 1 - i
    _, starts, cuts, slot = step_arrays(gpu, lens, slots)
    ag = a.to(gpu)
    y = ops.delta_rule(ag[:, :n], ag[:, n : 2 * n], ag[:, 2 * n : 3 * n], ag[:, 3 * n : 4 * n], ag[:, 4 * n :], w2.to(gpu),
                       w0.to(gpu), ab.to(gpu), state, starts, cuts, slot, math.exp(-0.5), 1e-6).cpu()
    left = state.cpu()
    t0 = 0
    for i in (0, 1, 57, 168, 169):  # a few of them against the plain recurrence
        b = a[t0 if i == 0 else sum(lens[:i]) : sum(lens[: i + 1])].to(F)
        r, k, v, a_raw = (b[:, j * n : (j + 1) * n].view(-1, H, D) for j in range(4))
        decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(b[:, 4 * n :]) @ w2.to(F).T + w0.to(F))).view(-1, H, D)
        rate = torch.sigmoid(a_raw + ab.to(F).view(H, D))
        for h in range(H):
            o, S = P.delta_recurrence(r[:, h], k[:, h], v[:, h], decay[:, h], rate[:, h], start[slots[i], h].to(F))
            got = y[sum(lens[:i]) : sum(lens[: i + 1]), h * D : (h + 1) * D]
            assert float((got - o).abs().max()) < 3e-5 * max(1.0, float(o.abs().max())), (i, h)
            assert float((left[slots[i], h] - S).abs().max()) < 3e-5 * max(1.0, float(S.abs().max())), (i, h)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 16), (1, 48), (5, 8), (3, 80), (2, 200)])
def test_norm_weight_and_gate_per_head(gpu, dtype, shape):
    H, D = shape
    t = 19
    y, a = rand(t, H * D, seed=1, scale=3.0), rand(t, 5 + H * D, seed=2)
    w = (1 + 0.2 * rand(H * D, seed=3)).to(DT[dtype])
    got = ops.head_norm_gate(y.to(gpu), a.to(gpu)[:, 5:], w.to(gpu), 1e-5, H, DT[dtype]).float().cpu()
    want = P.rms_unit(y.to(F).view(t, H, D), 1e-5).reshape(t, H * D) * w.to(F) * torch.sigmoid(a[:, 5:].to(F))
    assert float((got - want).abs().max()) < (1e-5 if dtype == "float32" else 2e-2) * float(want.abs().max())
    bare = ops.head_norm_gate(y.to(gpu), None, None, 1e-5, H, torch.float32).cpu()
    assert float((bare - P.rms_unit(y.to(F).view(t, H, D), 1e-5).reshape(t, H * D)).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(1, 7, 40), (2, 33, 64), (3, 5, 1028), (4, 3, 4100), (8, 2, 30)])
def test_copies_of_the_stream(gpu, dtype, sizes):
    """A write to all copies from the old ones ([from, to]), the read and the norm whose weight
    is stored around zero in the same pass; a read alone; the plain sum of chosen rows."""
    S, t, W = sizes
    x, y = rand(S, t, W, seed=1), rand(t, W, seed=2, scale=2.0)
    mix = (torch.eye(S) + 0.3 * rand(S, S, seed=3)).to(DT[dtype])
    out, inw = (0.8 + 0.3 * rand(S, seed=4)).to(DT[dtype]), (0.8 + 0.3 * rand(S, seed=5)).to(DT[dtype])
    wn = (0.2 * rand(W, seed=6)).to(DT[dtype])
    xg = x.to(gpu)
    got = ops.streams_step(xg, y=y.to(gpu), mix=mix.to(gpu), out=out.to(gpu), mult=0.7, read=True, inw=inw.to(gpu),
                           norm_weight=wn.to(gpu), offset=1.0, eps=1e-5, dtype=DT[dtype]).float().cpu()
    new = P.connection_write(list(x.to(F)), y.to(F), mix.to(F), out.to(F), 0.7)
    assert float((xg.cpu() - torch.stack(new)).abs().max()) < 3e-6 * float(torch.stack(new).abs().max())
    want = P.norm_around_zero(P.connection_read(new, inw.to(F)), wn.to(F), 1e-5)
    assert float((got - want).abs().max()) < (1e-5 if dtype == "float32" else 1.5e-2) * float(want.abs().max())
    # a read alone leaves the copies as they are
    before = xg.clone()
    u = ops.streams_step(xg, read=True, inw=inw.to(gpu)).cpu()
    assert float((u - P.connection_read(new, inw.to(F))).abs().max()) < 1e-5 and torch.equal(xg, before)
    rows = torch.tensor([t - 1, 0], dtype=torch.int32, device=gpu)
    total = ops.streams_step(xg, read=True, rows=rows).cpu()
    assert float((total - sum(new)[[t - 1, 0]]).abs().max()) < 1e-5
    # a write without a read
    ops.streams_step(xg, y=y.to(gpu), mix=mix.to(gpu), out=out.to(gpu), mult=1.0)
    again = P.connection_write(new, y.to(F), mix.to(F), out.to(F), 1.0)
    assert float((xg.cpu() - torch.stack(again)).abs().max()) < 5e-6 * float(torch.stack(again).abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 16, 16), (6, 3, 8, 24, 32), (2, 2, 24, 8, 32), (5, 1, 12, 20, 32), (3, 3, 64, 80, 80)])
@pytest.mark.parametrize("first", [5, 8])
def test_unit_heads_packed_and_gated(gpu, dtype, shape, first):
    """q, k and v divided by each head's root mean square and padded to the pages' head size;
    rows that begin at a multiple of four columns and rows that do not.  Then the heads'
    first entries times the sigmoid of one number a head."""
    H, K, dq, dv, D = shape
    t = 23
    a = rand(t, 8 + (H + K) * dq + K * dv + H, seed=7, scale=2.0)[:, 8 - first :].contiguous()
    q, k = a[:, first : first + H * dq], a[:, first + H * dq : first + (H + K) * dq]
    v = a[:, first + (H + K) * dq : first + (H + K) * dq + K * dv]
    ag = a.to(gpu)
    packed = ops.head_norm_pack(ag[:, first : first + H * dq], ag[:, first + H * dq : first + (H + K) * dq],
                                ag[:, first + (H + K) * dq : first + (H + K) * dq + K * dv], 1e-5, H, K, dq, dv, D, DT[dtype])
    got = packed.float().cpu().view(t, H + 2 * K, D)
    tol = 1e-5 if dtype == "float32" else 1e-2
    for part, src, n, d in ((got[:, :H], q, H, dq), (got[:, H : H + K], k, K, dq), (got[:, H + K :], v, K, dv)):
        want = P.rms_unit(src.to(F).view(t, n, d), 1e-5)
        assert float((part[..., :d] - want).abs().max()) < tol * float(want.abs().max())
        assert float(part[..., d:].abs().max() if D > d else 0.0) == 0.0
    gate = ag[:, first + (H + K) * dq + K * dv :]
    heads = ops.head_gate_cols(packed[:, : H * D].contiguous(), D, gate, dq, H).float().cpu().view(t, H, dq)
    want = got[:, :H, :dq].to(F) * torch.sigmoid(a[:, first + (H + K) * dq + K * dv :].to(F))[:, :, None]
    assert float((heads - want).abs().max()) < tol * float(want.abs().max())


# -- whole models -----------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed", "mixed2"])
def test_schedules(folders, name, dtype, schedule):
    folder, requests, ref, _, sens = folders[(name, dtype)]
    cfg = CONFIGS[name][0]
    make = {"whole": replay.whole, "tail": lambda q: replay.tail_one_by_one(q, tail=40), "portions": replay.portions,
            "mixed": replay.mixed, "mixed2": lambda q: replay.mixed(q, seed=7, decode_tail=30)}[schedule]
    trace = make(requests)
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, 16))
    rows = replay.collect(trace, replay.run_trace(runner, trace), cfg["vocab"])
    check(rows, ref, dtype, sens)
    assert runner.cache.idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [8, 32, 64])
@pytest.mark.parametrize("name", ["A", "B"])
def test_other_page_sizes(folders, name, page_size, dtype):
    folder, requests, ref, _, sens = folders[(name, dtype)]
    trace = replay.mixed(requests, seed=3)
    runner = make_runner(folder, dtype, replay.peak_tokens(trace, page_size), page_size=page_size)
    rows = replay.collect(trace, replay.run_trace(runner, trace), CONFIGS[name][0]["vocab"])
    check(rows, ref, dtype, sens)
    assert runner.cache.idle()


@pytest.mark.parametrize("name", ["A", "C"])
def test_the_stream_after_every_layer(folders, name):
    """The sum of the copies once a layer's last part has been written back."""
    from halite_amd.parts import block

    folder, requests, _, weights, _ = folders[(name, "float32")]
    cfg = CONFIGS[name][0]
    ids = requests["r1"]
    want = []
    P.forward(cfg, weights, ids, layers_out=want)
    runner = make_runner(folder, "float32", 256)
    seen, inner = [], block.HyperPreNormBlock.forward

    def forward(self, h, pending, ctx, run):
        out = inner(self, h, pending, ctx, run)
        seen.append(self.leave(h.clone(), out, None))
        return out

    block.HyperPreNormBlock.forward = forward
    try:
        replay.run_trace(runner, replay.whole({"r1": ids}))
    finally:
        block.HyperPreNormBlock.forward = inner
    assert len(seen) == len(want) == len(cfg["layers"])
    for got, w in zip(seen, want):
        assert float((got.cpu() - w.float()).abs().max()) < 5e-5 * max(1.0, float(w.abs().max()))


# -- keys made loud -----------------------------------------------------------------------------

LOUD, ASK = 7, 11


def mark_embedding(w):
    """Channel 0 of the embedding is nonzero for LOUD alone and channel 1 for ASK alone, so a
    projection that reads one of them tells that token from all others."""
    w["embed"][:, :2] = 0.0
    w["embed"][LOUD, 0] = 3.0
    w["embed"][ASK, 1] = 3.0


def loud_attention_model(window, conv=3, kv_heads=1, streams=2):
    """One attention layer whose weights stand out for one pair of tokens: key channel 0 is
    large for LOUD and zero for every other token, query channel 0 large for ASK and zero
    otherwise (the convolutions pass that channel unmixed), so after the unit norms ASK's
    score on LOUD is nearly ``scale * dim`` and its weight nearly 1 where all others' are
    ``sigmoid(bias)``, a few hundredths.  A single layer: a LOUD that ASK does not see leaves
    ASK's logits nearly as they are without it."""
    cfg = P.model_cfg(64, 61, [P.attention_layer(2, kv_heads, 16, 24, 0.6, conv=conv, window=window, mlp=P.dense(48))],
                      streams=streams, residual_mult=0.8)
    w = P.random_weights(cfg, {}, seed=77)
    mark_embedding(w)
    w["l0.norm1"][:2] = 0.0
    w["l0.mix.k"] *= 0.2
    w["l0.mix.q"] *= 0.2
    for head in range(kv_heads):
        w["l0.mix.k"][head * 16] = 0.0
        w["l0.mix.k"][head * 16, 0] = 4.0
    for head in range(2):
        w["l0.mix.q"][head * 16] = 0.0
        w["l0.mix.q"][head * 16, 1] = 4.0
    if conv:
        last = torch.zeros(conv)
        last[-1] = 1.0
        for head in range(kv_heads):
            w["l0.mix.k.conv"][head * 16] = last
        for head in range(2):
            w["l0.mix.q.conv"][head * 16] = last
    w["l0.mix.pb"][:] = -4.0
    w["l0.mix.g"] *= 0.1
    w["l0.mix.o"] *= 3.0
    return cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}


def loud_delta_model():
    """One delta-rule layer that forgets and removes next to nothing (decay and removal
    biases far down) and whose key channel 0 is large for LOUD, read channel 0 large for ASK
    and both zero otherwise: what ASK reads is LOUD's value, however long ago it was written."""
    cfg = P.model_cfg(64, 61, [P.delta_layer(2, 16, P.dense(48))], streams=2, residual_mult=0.8)
    w = P.random_weights(cfg, {0: 4}, seed=79)
    mark_embedding(w)
    w["l0.norm1"][:2] = 0.0
    w["l0.mix.k"] *= 0.3
    w["l0.mix.r"] *= 0.3
    for head in range(2):
        w["l0.mix.k"][head * 16] = 0.0
        w["l0.mix.k"][head * 16, 0] = 5.0
        w["l0.mix.r"][head * 16] = 0.0
        w["l0.mix.r"][head * 16, 1] = 5.0
    w["l0.mix.w0"][:] = -9.0
    w["l0.mix.w2"] *= 0.1
    w["l0.mix.a.b"][:] = -9.0
    w["l0.mix.a"] *= 0.1
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window,page_size", [(40, 16), (32, 16), (33, 32), (7, 16), (130, 64)])
def test_loud_keys_on_both_sides_of_a_windows_edge(dtype, window, page_size, tmp_path):
    """LOUD at one position, ASK at the last position that sees it and at the first that does
    not; for a window of two pages the edge is also a page's.  The schedules put both places
    into prompts and into decoded tokens.  A second request has LOUD at position 0 and at the
    window's first place."""
    cfg, w = loud_attention_model(window)
    p0 = 2 * window + 5
    n = p0 + 2 * window + 9
    requests = {"edge": loud_sequence(cfg, n, [p0], [p0 + 1, p0 + window - 1, p0 + window, p0 + window + 1], 2),
                "start": loud_sequence(cfg, window + 30, [0], [1, window - 1, window, window + 1], 3),
                "deep": loud_sequence(cfg, 3 * window + 2, [window + 1], [2 * window, 2 * window + 1, 3 * window + 1], 4)}
    ref = replay_all(cfg, w, requests, dtype, tmp_path, tail=window + 12, page_size=page_size)
    top = float(ref["edge"].abs().max())
    for rid, inside, outside in (("edge", p0 + window - 1, p0 + window), ("start", window - 1, window), ("deep", 2 * window, 2 * window + 1)):
        silent = plain_logits(cfg, w, quiet(requests[rid]))
        # (just outside, the convolutions still carry a little of the token into its neighbours' keys)
        assert float((ref[rid][inside] - silent[inside]).abs().max()) > 0.08 * top
        assert float((ref[rid][outside] - silent[outside]).abs().max()) < 0.01 * top


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kv_heads", [1, 2])
def test_a_loud_key_far_back_without_a_window(dtype, kv_heads, tmp_path):
    """No window and no convolution: LOUD at position 3 (and at 0) among hundreds of keys
    across many pages."""
    cfg, w = loud_attention_model(None, conv=None, kv_heads=kv_heads, streams=3)
    requests = {"far": loud_sequence(cfg, 400, [3], [4, 200, 255, 256, 399], 2),
                "first": loud_sequence(cfg, 300, [0], [1, 150, 299], 3)}
    ref = replay_all(cfg, w, requests, dtype, tmp_path)
    silent = plain_logits(cfg, w, quiet(requests["far"]))
    assert float((ref["far"][399] - silent[399]).abs().max()) > 0.15 * float(ref["far"].abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_pair_written_to_the_state_long_before_it_is_read(dtype, tmp_path):
    cfg, w = loud_delta_model()
    requests = {"far": loud_sequence(cfg, 420, [3], [4, 200, 419], 5),
                "first": loud_sequence(cfg, 260, [0], [1, 130, 259], 6)}
    ref = replay_all(cfg, w, requests, dtype, tmp_path)
    silent = plain_logits(cfg, w, quiet(requests["far"]))
    assert float((ref["far"][419] - silent[419]).abs().max()) > 0.15 * float(ref["far"].abs().max())


# -- long decoding, slots and pages that serve again ------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_long_decoding_beside_requests_that_come_and_go(folders, dtype, graphs):
    """A short prompt and 200 tokens decoded one by one (the window passes over decoded tokens,
    the recurrence runs on) beside short requests that take the freed slot and pages one
    after the other."""
    folder, _, _, weights, _ = folders[("A", dtype)]
    cfg = P.VEP_A
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


def test_pages_behind_the_window_are_given_back(folders):
    folder, _, _, _, _ = folders[("A", "float32")]
    runner = make_runner(folder, "float32", 1024)
    (group,) = runner.cache.groups
    assert group.need.window == 24
    from halite_amd.engine.batch import Segment

    slot = runner.admit()
    ids = tokens(P.VEP_A, 200, 9)
    pos = 0
    for n in (50, 1, 1, 30, 2, 100, 16):
        runner.step([Segment(slot, pos, ids[pos : pos + n], [])])
        pos += n
        runner.cache.check()
        held = group.pool.capacity - group.pool.available
        assert held == -(-pos // 16) - max(pos - 24 + 1, 0) // 16  # pages wholly before the next token's window went back
    runner.free(slot)
    assert runner.cache.idle()


# -- through the engine's entry point ----------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    folder, _, _, weights, _ = folders[(name, dtype)]
    cfg = CONFIGS[name][0]
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
    assert checked >= 36


# -- the programs: generation from the command line, the random-weights mode, trace replay -----


def test_command_line_and_replay_program(folders, tmp_path):
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, _, _, weights, _ = folders[("A", "float32")]
    cfg = P.VEP_A
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
    # the random-weights mode: a configuration without tensors states the rank of its decay
    # projections; the folder it writes holds the design's own keys
    stated = json.loads(json.dumps(P.VEP_C))
    for i, n in P.VEP_C_RANKS.items():
        stated["layers"][i]["mixer"]["decay_rank"] = n
    cfgfile, out = tmp_path / "c.json", tmp_path / "rand"
    cfgfile.write_text(json.dumps(stated))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "halite_make_random_model"), "--config", str(cfgfile),
                           "--out", str(out), "--seed", "3", "--dtype", "bfloat16", "--std", "0.1"], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "decay_rank" not in (out / "config.json").read_text()
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
    want = plain_logits(P.VEP_C, stored, [1, 2, 3, 4, 5, 6, 7, 8])
    got0 = torch.from_numpy(np.fromfile(logits / "0.f32", dtype="<f4").reshape(2, -1))
    got1 = torch.from_numpy(np.fromfile(logits / "1.f32", dtype="<f4").reshape(1, -1))
    got2 = torch.from_numpy(np.fromfile(logits / "2.f32", dtype="<f4").reshape(1, -1))
    scale = max(1.0, float(want.abs().max()))
    assert float((got0[0] - want[4]).abs().max()) < 5e-5 * scale and float((got2[0] - want[7]).abs().max()) < 5e-5 * scale
    assert float((got0[1] - plain_logits(P.VEP_C, stored, [7])[0]).abs().max()) < 5e-5 * scale
    assert float((got1[0] - plain_logits(P.VEP_C, stored, [9, 8])[1]).abs().max()) < 5e-5 * scale
