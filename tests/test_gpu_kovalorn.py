"""Kovalorn on the GPU against the plain model (`plain_kovalorn`): every mechanism alone, whole prompts, decoding
through the cache, portions down to two tokens, unequal batches, pages and slots used again, keys at the edges of
the window, of the kept first keys and of pages, far keys, long decoding, other sizes, and generation through the
engine's entry point."""
import math

import pytest
import torch

import kovalorn_util as u
import plain_kovalorn as plain

pytestmark = pytest.mark.gpu

_models = {}


def model_for(tmp_path_factory, name, cfg, seed, dtype, change=None):
    """(weights as the plain model reads them, loaded engine model); made once per (name, dtype)."""
    from ferrox_amd.engine.loading import load_model
    key = (name, dtype)
    if key not in _models:
        weights = u.make_weights(cfg, seed)
        if change:
            change(weights)
        folder = u.write_model(str(tmp_path_factory.mktemp(f"kovalorn_{name}")), cfg, weights)
        _models[key] = (weights, load_model(folder, dtype, "cuda:0"))
    return _models[key]


def runner_of(model, block_size=16, num_pages=24, max_seqs=4, **kw):
    from ferrox_amd.engine.runner import ModelRunner
    return ModelRunner(model, block_size=block_size, num_pages=num_pages, max_seqs=max_seqs, **kw)


def traced(dtype):
    import contextlib

    from ferrox_amd import debug
    return debug.trace_routing() if dtype == "bfloat16" else contextlib.nullcontext()


def run_and_check(cfg, weights, model, requests, schedule, dtype, what, **runner_kw):
    runner = runner_of(model, **runner_kw)
    with traced(dtype) as trace:
        got, chosen = u.run_schedule(runner, requests, schedule, trace)
    for key in runner.manager.groups:
        assert runner.manager.n_free_pages(key) == runner_kw.get("num_pages", 24), "pages were lost"
    return u.check_against_plain(cfg, weights, requests, got, dtype, chosen, what)


# ---------------------------------------------------------------------------
# each mechanism alone: models of one layer (two where a layer reads another's keys)
# ---------------------------------------------------------------------------
SINGLE = {
    "no_mask": u.config([u.attention_layer(heads=2, kv_heads=2, dim=16, vdim=16, window=0, scale=0.6)], logit_scale=1.0),
    "window": u.config([u.attention_layer(heads=4, kv_heads=1, dim=32, vdim=16, window=10, keep_first=0, scale=0.5)]),
    "window_kept": u.config([u.attention_layer(heads=4, kv_heads=2, dim=24, vdim=40, window=7, keep_first=4, scale=0.5)]),
    "kept_more_than_window": u.config([u.attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=3, keep_first=21, scale=0.7)]),
    "shared_keys": u.config([u.attention_layer(heads=4, kv_heads=2, dim=16, vdim=32, window=12, keep_first=2, scale=0.5),
                             u.attention_layer(heads=2, kv_heads=2, dim=16, vdim=32, window=30, keep_first=0, scale=0.9, kv_from=0)]),
    "dense": u.config([u.attention_layer(heads=1, kv_heads=1, dim=16, vdim=16, window=0, mlp=u.dense(40))]),
    "moe": u.config([u.attention_layer(heads=1, kv_heads=1, dim=16, vdim=16, window=0, mlp=u.moe(7, 3, 24, 1.4, 0))]),
    "moe_shared": u.config([u.attention_layer(heads=1, kv_heads=1, dim=16, vdim=16, window=0, mlp=u.moe(4, 1, 16, 0.6, 48))]),
    "moe_many": u.config([u.attention_layer(heads=1, kv_heads=1, dim=16, vdim=16, window=0, mlp=u.moe(70, 5, 8, 2.5, 8))]),
}


@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_alone(tmp_path_factory, name):
    cfg = SINGLE[name]
    weights, model = model_for(tmp_path_factory, name, cfg, 11, "float32")
    requests = {"a": u.random_tokens(cfg["vocab"], 37, 1), "b": u.random_tokens(cfg["vocab"], 5, 2)}
    run_and_check(cfg, weights, model, requests, [[("a", 37)], [("b", 5)]], "float32", name + " whole")
    cut = [[("a", 20), ("b", 2)], [("a", 2), ("b", 1)], [("a", 1), ("b", 1)]] + [[("a", 1)]] * 14 + [[("b", 1)]]
    run_and_check(cfg, weights, model, requests, cut, "float32", name + " cut")


def test_the_plain_model_shows_every_mechanism():
    """What the comparisons above can see: leaving a mechanism out of the plain model moves its logits far beyond
    the tests' limit, so an engine without it would fail them."""
    cfg = SINGLE["window_kept"]
    weights = u.make_weights(cfg, 11)
    tokens = u.random_tokens(cfg["vocab"], 37, 1)
    right = plain.forward(cfg, weights, tokens)

    def moved(other_cfg=None, other_weights=None):
        return float(u.row_errors(plain.forward(other_cfg or cfg, other_weights or weights, tokens), right).max())

    def with_mixer(**kw):
        layer = dict(cfg["layers"][0], mixer=dict(cfg["layers"][0]["mixer"], **kw))
        return dict(cfg, layers=[layer])

    bar = 100 * u.LIMIT["float32"]
    assert moved(with_mixer(mask={"size": 7, "keep_first": 0})) > bar            # the kept first keys
    assert moved(with_mixer(mask={"size": 7, "keep_first": 3})) > bar
    assert moved(with_mixer(mask={"size": 8, "keep_first": 4})) > bar            # the window, one position off
    assert moved(with_mixer(scale=0.55)) > bar
    assert moved(other_weights=dict(weights, **{"l0.mix.sink": weights["l0.mix.sink"] - 30.0})) > bar      # no sink
    assert moved(other_weights=dict(weights, **{"l0.mix.g": weights["l0.mix.g"] * 0})) > bar                 # no gate
    assert moved(other_weights=dict(weights, **{"l0.norm1": weights["l0.norm1"] - 1.0})) > bar               # weight not around zero
    assert moved(dict(cfg, logit_scale=1.0)) > bar


def attention_reference(q, k, v, scale, window, keep_first, sinks, gate):
    """float64 attention of one sequence from position 0: q [n, H, D], k [n, G, D], v [n, G, V]."""
    n, H, _ = q.shape
    G = k.shape[1]
    see = plain.visible(n, window or n, keep_first)
    out = torch.zeros(n, H, v.shape[2], dtype=torch.float64)
    for h in range(H):
        s = (q[:, h].double() @ k[:, h // (H // G)].double().T) * scale
        s = s.masked_fill(~see, -math.inf)
        e = torch.exp(s)
        den = e.sum(-1, keepdim=True) + (torch.exp(sinks[h].double()) if sinks is not None else 0.0)
        out[:, h] = (e / den) @ v[:, h // (H // G)].double()
    if gate is not None:
        out = out * torch.sigmoid(gate.double()).view(n, H, -1)
    return out


@pytest.mark.parametrize("dtype,hd,vd,bs", [
    ("float32", 24, 40, 16), ("bfloat16", 64, 64, 64), ("bfloat16", 128, 128, 64), ("bfloat16", 96, 96, 64),
    ("bfloat16", 32, 32, 16), ("bfloat16", 256, 256, 16), ("bfloat16", 48, 16, 16), ("bfloat16", 20, 20, 16)])
def test_attention_kernels_with_kept_keys_sinks_and_gate(dtype, hd, vd, bs):
    """The attention kernels alone, every variant that head sizes and page sizes select (matrix-unit kernels that
    stage through registers, that load straight into LDS, with items of 64 and of 128 queries, one wave a block, and
    the kernels for any shape): a prompt of 333 positions written into scattered pages, read as one portion, as a
    portion deep in the sequence, and as single queries, with windows whose start falls inside and outside the kept
    first keys and kept keys that span several tiles."""
    from ferrox_amd import debug, ops
    dt = getattr(torch, dtype)
    gen = torch.Generator().manual_seed(hd + vd)
    n, H, G = 333, 4, 2
    q = torch.randn(n, H, hd, generator=gen).to(dt)
    k = torch.randn(n, G, hd, generator=gen).to(dt)
    v = torch.randn(n, G, vd, generator=gen).to(dt)
    gate = torch.randn(n, H * vd, generator=gen).to(dt)
    sinks = torch.randn(H, generator=gen) + 1.0
    n_blocks = -(-n // bs)
    order = torch.randperm(n_blocks + 3, generator=gen)[:n_blocks].to(torch.int32)
    k_pages = torch.full((n_blocks + 3, G, bs, hd), float("nan")).to(dt)
    v_pages = torch.full((n_blocks + 3, G, vd, bs), float("nan")).to(dt)
    for t in range(n):
        k_pages[order[t // bs], :, t % bs] = k[t]
        v_pages[order[t // bs], :, :, t % bs] = v[t]
    dev = dict(device="cuda")
    qd, gd, kp, vp = q.view(n, -1).cuda(), gate.cuda(), k_pages.cuda(), v_pages.cuda()
    positions = torch.arange(n, dtype=torch.int32, **dev)
    tol = 2e-5 if dtype == "float32" else 2e-2
    for window, keep in ((40, 7), (100, 70), (64, 64), (20, 150), (50, 0), (0, 0)):
        want = attention_reference(q, k, v, 0.25, window, keep, sinks, gate).view(n, -1)
        table = order.clone()
        if window:      # pages that no query of the portions below sees hold no page id
            for b in range(n_blocks):
                if b * bs >= keep and (b + 1) * bs <= 200 - window:
                    table[b] = -1
        table_d = table.view(1, -1).cuda()
        common = (H, G, hd, bs, window, 0.25)
        extra = dict(v_dim=vd, keep_first=keep, sinks=sinks.cuda(), gate=gd)
        wide = ops.attention_tile_queries(dt, hd, bs)
        # (one and two groups of waves a block, where the kernel that loads straight into LDS has both)
        variants = [(64, 0)] + ([(64, 1), (wide, 1), (wide, 2)] if wide > 64 else [])
        for tile_q, groups in variants:
            with debug.kernel_switch("attention", "direct_groups", groups):
                for first in (0, 200) if window else (0,):
                    table_all = order.view(1, -1).cuda() if first == 0 else table_d
                    starts = list(range(first, n, tile_q))
                    item = lambda x: torch.tensor(x, dtype=torch.int32, **dev)      # noqa: E731
                    out = torch.zeros(n, H * vd, dtype=dt, **dev)
                    ops.attention_tiles(qd, out, kp, vp, table_all, positions, item([0] * len(starts)), item(starts),
                                        item([min(tile_q, n - s) for s in starts]), *common, tile_q=tile_q, **extra)
                    err = (out[first:].double().cpu() - want[first:]).abs().max()
                    assert float(err) < tol, (window, keep, tile_q, groups, first, float(err))
        toks = [200, 201, 263, 264, 332] if window else [0, 1, 63, 64, 332]
        for chunk in (None, 64):
            out = torch.zeros(n, H * vd, dtype=dt, **dev)
            ops.attention_decode(qd, out, kp, vp, table_d if window else order.view(1, -1).cuda(), positions,
                                 torch.zeros(len(toks), dtype=torch.int32, **dev), torch.tensor(toks, dtype=torch.int32, **dev),
                                 *common, max_kv_len=n, chunk=chunk, **extra)
            err = (out[toks].double().cpu() - want[toks]).abs().max()
            assert float(err) < tol, (window, keep, "decode", chunk, float(err))


def test_router_weights_with_a_floor_and_a_constant():
    """Sigmoid scores, the largest k, each over the sum of the chosen (+ a floor) times a constant, from all three
    launches that select experts; more than 64 experts take the kernel's second path."""
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(5)
    for E, k, T in ((8, 3, 9), (70, 5, 33), (3, 3, 2), (16, 1, 5)):
        logits = torch.randn(T, E, generator=gen) * 2
        s = torch.sigmoid(logits.double())
        val, want = torch.topk(s, k, dim=-1)
        want_w = val / (val.sum(-1, keepdim=True) + 1e-20) * 1.7
        ids, w, _ = ops.router_select(logits.cuda(), E, k, True, ops.GATE_SIGMOID, weighting=(1e-20, 1.7))
        assert ids.cpu().tolist() == want.tolist()
        assert torch.allclose(w.cpu().double(), want_w, atol=1e-6)
        routed = ops.route(logits.cuda(), E, k, True, ops.GATE_SIGMOID, weighting=(1e-20, 1.7))
        assert routed[0].cpu().tolist() == want.tolist() and torch.allclose(routed[1].cpu().double(), want_w, atol=1e-6)
    # scores that all vanish: the floor keeps the weights finite (zero over the floor, not zero over zero)
    ids, w, _ = ops.router_select(torch.full((2, 4), -200.0).cuda(), 4, 2, True, ops.GATE_SIGMOID, weighting=(1e-20, 1.5))
    assert torch.isfinite(w).all() and float(w.abs().max()) == 0.0


def test_norm_with_a_weight_around_zero_and_without_one():
    from ferrox_amd import ops
    from ferrox_amd.parts.norm import RMSNorm
    gen = torch.Generator().manual_seed(2)
    for H in (48, 300, 5000):
        x = torch.randn(7, H, generator=gen) * 3
        w = (0.1 * torch.randn(H, generator=gen)).to(torch.bfloat16)
        norm = RMSNorm(H, 1e-5, name="w", offset=1.0, gain=1.5)
        norm.load(lambda name: w.cuda())
        assert norm.weight.dtype == torch.float32
        got = ops.rmsnorm(x.cuda(), norm.weight, norm.eps, torch.float32).cpu().double()
        assert torch.allclose(got, plain.offset_norm(x.double(), w.double(), 1e-5) * 1.5, atol=1e-5)
        got = ops.rmsnorm(x.cuda(), None, 1e-5, torch.float32).cpu().double()
        assert torch.allclose(got, plain.unit_rms(x.double(), 1e-5), atol=1e-5)


# ---------------------------------------------------------------------------
# the model whole and cut
# ---------------------------------------------------------------------------
LENGTHS = [1, 2, 23, 50, 97]       # a single token, two, around the windows and the kept keys, across pages


def main_requests():
    return {f"r{n}": u.random_tokens(u.CFG_MAIN["vocab"], n, 40 + n) for n in LENGTHS}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts_and_decoding(tmp_path_factory, dtype):
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    run_and_check(u.CFG_MAIN, weights, model, reqs, [[(r, len(t))] for r, t in reqs.items()], dtype, "whole")
    # most of a prompt in one step, the last 40 tokens (or all but one) one by one: the windows of 9 to 50 positions
    # pass over decoded tokens, across the page borders at 16, 32, ...
    sched = []
    for r, t in reqs.items():
        first = max(1, len(t) - 40)
        sched += [[(r, first)]] + [[(r, 1)]] * (len(t) - first)
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "decode")
    # token by token from the first token on: the first tokens of a sequence, kept keys that are not there yet
    one = {"r50": reqs["r50"]}
    run_and_check(u.CFG_MAIN, weights, model, one, [[("r50", 1)]] * 50, dtype, "token by token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size(tmp_path_factory, dtype):
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    sizes = [2, 5, 2, 16, 1, 7, 24, 3, 2, 17, 1, 1, 9]
    sched = []
    for r, t in reqs.items():
        left, i = len(t), 0
        while left:
            n = min(sizes[i % len(sizes)], left)
            sched.append([(r, n)])
            left -= n
            i += 1
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_with_pages_and_slots_used_again(tmp_path_factory, dtype):
    """Up to three live requests under three slots and a pool of 14 pages of 16 (the requests' sum needs 18):
    portions beside single tokens, requests that pause, slots and pages taken again by later requests."""
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    reqs["s40"] = u.random_tokens(u.CFG_MAIN["vocab"], 40, 7)
    sched = [
        [("r97", 30), ("r23", 2), ("r1", 1)],
        [("r97", 3), ("r23", 1), ("r2", 2)],                    # r1's slot goes to r2
        [("r97", 1), ("r23", 18)],
        [("r23", 1), ("r50", 21)],                              # r97 pauses
        [("r97", 40), ("r23", 1), ("r50", 1)],                  # r23 ends
        [("r97", 1), ("r50", 27), ("s40", 2)],
        [("r97", 22), ("r50", 1), ("s40", 37)],                 # r97 and r50 end
        [("s40", 1)],
    ]
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "mixed", num_pages=14, max_seqs=3)
    # the same requests, each alone, give the same logits up to rounding: the batch changes nothing
    alone = runner_of(model, num_pages=14, max_seqs=3)
    mixed = runner_of(model, num_pages=14, max_seqs=3)
    got_alone, _ = u.run_schedule(alone, reqs, [[(r, len(t))] for r, t in reqs.items()])
    got_mixed, _ = u.run_schedule(mixed, reqs, sched)
    for r in reqs:
        assert float(u.row_errors(got_mixed[r], got_alone[r]).max()) <= 2 * u.LIMIT[dtype], r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_fused_head_norms_give_the_bits_of_the_separate_kernels(tmp_path_factory, dtype, monkeypatch):
    """The launch that norms the heads of q and k and writes the cache against the three launches it stands for
    (two norms over gathered heads, the cache write): the same logits bit for bit, prompts, portions and single
    tokens, also for the layers that have no keys of their own."""
    from ferrox_amd.parts import attention
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = {"a": u.random_tokens(u.CFG_MAIN["vocab"], 70, 1), "b": u.random_tokens(u.CFG_MAIN["vocab"], 9, 2)}
    sched = [[("a", 40), ("b", 2)], [("a", 1), ("b", 7)]] + [[("a", 1)]] * 12 + [[("a", 17)]]
    got = {}
    for fused in (True, False):
        monkeypatch.setattr(attention, "FUSE_HEAD_NORMS", fused)
        got[fused], _ = u.run_schedule(runner_of(model), reqs, sched)
    for r in reqs:
        assert torch.equal(got[True][r], got[False][r]), r


def test_used_pages_start_clean_and_passed_pages_come_back(tmp_path_factory):
    """One slot and four pages of 16: every request takes the pages that the one before left.  A layer that keeps
    the first 3 keys and a window of 20 holds a 150-token request in four pages (the first, and up to three under
    the window and the portion in progress), in portions of at most 8; the pages in between go back as the window
    passes, and come again for later positions."""
    cfg = u.config([u.attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=20, keep_first=3, scale=0.8, mlp=u.moe(3, 1, 16, 1.2, 0)),
                    u.attention_layer(heads=4, kv_heads=1, dim=16, vdim=16, window=11, keep_first=1, scale=0.8, kv_from=0)], width=32)
    weights, model = model_for(tmp_path_factory, "giveback", cfg, 8, "float32")
    reqs = {"z": u.random_tokens(cfg["vocab"], 150, 2), "y": u.random_tokens(cfg["vocab"], 60, 3)}
    sched = [[("z", 8)]] * 17 + [[("z", 1)]] * 14 + [[("y", 7)]] * 8 + [[("y", 2)]] * 2
    run_and_check(cfg, weights, model, reqs, sched, "float32", "give back", num_pages=4, max_seqs=1)


# ---------------------------------------------------------------------------
# where a fault hides behind random weights: peaked attention
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_the_edges_stand_out(tmp_path_factory, dtype):
    """A large score scale makes the softmax pick single keys, so that a key just inside the window or the kept
    first keys that is missed, or one just outside that is seen, moves the logits far beyond rounding.  The plain
    model itself must tell the cases apart.  Prompts end and decoding runs on both sides of the window's edge as it
    passes the kept keys (positions 5 + 30) and the page borders (16, 32, ...), and far from the start."""
    # (bfloat16 rounds q and k to 8 bits: under scale 2 over unit-RMS heads of 32 that alone moves the scores by a
    # tenth, so the bfloat16 run takes a smaller scale and a lower bar for the plain model's own sensitivity)
    scale, bar = {"float32": (2.0, 0.15), "bfloat16": (0.8, 0.09)}[dtype]
    cfg = u.config([u.attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, window=30, keep_first=5, scale=scale, mlp=u.moe(4, 2, 32, 1.0, 16)),
                    u.attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, window=47, keep_first=17, scale=scale, kv_from=0)], width=64)

    def no_sink(w):      # (a sink that takes no weight: the keys alone share the softmax, one of them stands out)
        for i in range(2):
            w[f"l{i}.mix.sink"] = w[f"l{i}.mix.sink"] - 6.0

    weights, model = model_for(tmp_path_factory, "peaked" + dtype, cfg, 21, dtype, change=no_sink)
    tokens = u.random_tokens(cfg["vocab"], 150, 5)
    right = plain.forward(cfg, weights, tokens)
    for layer, (size, keep) in ((0, (29, 5)), (0, (31, 5)), (0, (30, 4)), (0, (30, 6)), (1, (46, 17)), (1, (47, 16)), (1, (47, 18))):
        layers = list(cfg["layers"])
        layers[layer] = dict(layers[layer], mixer=dict(layers[layer]["mixer"], mask={"size": size, "keep_first": keep}))
        assert float(u.row_errors(plain.forward(dict(cfg, layers=layers), weights, tokens), right).max()) > bar, (layer, size, keep)
    reqs = {"p": tokens}
    for first in (1, 4, 5, 6, 29, 30, 31, 34, 35, 36, 63, 64, 65, 120):
        steps = min(14, 150 - first)
        sched = [[("p", first)]] + [[("p", 1)]] * steps
        if 150 - first - steps:
            sched.append([("p", 150 - first - steps)])
        run_and_check(cfg, weights, model, reqs, sched, dtype, f"edge {first}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path_factory, dtype):
    """A layer without a mask under a peaked softmax: queries deep in a 600-token sequence pick keys hundreds of
    positions back (the plain model without the keys beyond 400 positions differs far beyond the limit), across
    nine pages of 64, whole, in portions, and decoded one by one; a second layer reads the same keys under a window."""
    scale, bar = {"float32": (2.0, 0.15), "bfloat16": (0.8, 0.09)}[dtype]
    cfg = u.config([u.attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, window=0, scale=scale, mlp=u.dense(64)),
                    u.attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, window=70, keep_first=0, scale=scale, kv_from=0)], width=64)

    def no_sink(w):
        for i in range(2):
            w[f"l{i}.mix.sink"] = w[f"l{i}.mix.sink"] - 6.0

    weights, model = model_for(tmp_path_factory, "far" + dtype, cfg, 23, dtype, change=no_sink)
    tokens = u.random_tokens(cfg["vocab"], 600, 6)
    near = dict(cfg, layers=[dict(cfg["layers"][0], mixer=dict(cfg["layers"][0]["mixer"], mask={"size": 400, "keep_first": 0})),
                             cfg["layers"][1]])
    moved = u.row_errors(plain.forward(near, weights, tokens)[400:], plain.forward(cfg, weights, tokens)[400:])
    assert float(moved.max()) > bar, float(moved.max())
    reqs = {"f": tokens}
    for what, sched in (("whole", [[("f", 600)]]), ("decode", [[("f", 560)]] + [[("f", 1)]] * 40),
                        ("portions", [[("f", 37)]] * 16 + [[("f", 8)]])):
        run_and_check(cfg, weights, model, reqs, sched, dtype, "far " + what, block_size=64, num_pages=10)


def test_a_sink_that_takes_nearly_all(tmp_path_factory):
    """Sinks far above every score (the heads' outputs nearly vanish) and far below (no sink at all): neither
    overflows, both match the plain model."""
    cfg = SINGLE["window_kept"]
    for name, shift in (("high_sink", 60.0), ("low_sink", -90.0)):
        def change(w, shift=shift):
            w["l0.mix.sink"] = (w["l0.mix.sink"].float() + shift).to(torch.bfloat16)
        weights, model = model_for(tmp_path_factory, name, cfg, 12, "float32", change=change)
        reqs = {"a": u.random_tokens(cfg["vocab"], 40, 4)}
        run_and_check(cfg, weights, model, reqs, [[("a", 25)]] + [[("a", 1)]] * 15, "float32", name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_on_the_matrix_units(tmp_path_factory, dtype):
    """Sizes that take the bfloat16 kernels' matrix-unit paths (equal head sizes of 32, 64 and 128, widths in
    multiples of 64, pages of 64): a prompt, then 140 tokens one by one from recorded steps, the windows passing the
    kept first keys (of which one layer keeps more than two tiles), and two requests decoding side by side."""
    weights, model = model_for(tmp_path_factory, "mfma", u.CFG_MFMA, 17, dtype)
    reqs = {"x": u.random_tokens(u.CFG_MFMA["vocab"], 300, 3), "y": u.random_tokens(u.CFG_MFMA["vocab"], 150, 4)}
    sched = [[("x", 160)], [("y", 10)]] + [[("x", 1), ("y", 1)]] * 140
    run_and_check(u.CFG_MFMA, weights, model, reqs, sched, dtype, "long decode", block_size=64, num_pages=10)
    whole = [[("x", 300), ("y", 150)]]
    run_and_check(u.CFG_MFMA, weights, model, reqs, whole, dtype, "whole", block_size=64, num_pages=10)
    cut = [[("x", 130), ("y", 3)], [("x", 2), ("y", 140)], [("x", 150), ("y", 7)], [("x", 18)]]
    run_and_check(u.CFG_MFMA, weights, model, reqs, cut, dtype, "portions", block_size=64, num_pages=10)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_fit_no_vector(tmp_path_factory, dtype):
    """Head sizes, widths and a vocabulary that are no multiples of 16, 8 or 4: the kernels' guarded paths."""
    cfg = u.config([u.attention_layer(heads=3, kv_heads=3, dim=24, vdim=40, window=7, keep_first=2, scale=0.6, mlp=u.moe(3, 2, 20, 1.1, 12)),
                    u.attention_layer(heads=6, kv_heads=3, dim=24, vdim=40, window=19, keep_first=0, scale=0.5, kv_from=0, mlp=u.dense(30)),
                    u.attention_layer(heads=2, kv_heads=1, dim=18, vdim=6, window=0, scale=0.5)], width=70, vocab=151)
    weights, model = model_for(tmp_path_factory, "odd", cfg, 13, dtype)
    reqs = {"a": u.random_tokens(151, 45, 1), "b": u.random_tokens(151, 20, 2)}
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 17)]] + [[("a", 1), ("b", 1)]] + [[("a", 1)]] * 13
    run_and_check(cfg, weights, model, reqs, sched, dtype, "odd sizes")


# ---------------------------------------------------------------------------
# through the engine's own entry point: scheduler, sampling, recorded steps
# ---------------------------------------------------------------------------
def plain_greedy(cfg, weights, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_engine(tmp_path_factory):
    from ferrox_amd.engine.api import Engine
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, "float32")
    prompts = [u.random_tokens(u.CFG_MAIN["vocab"], n, 90 + n) for n in (3, 30, 1, 47)]
    want = [plain_greedy(u.CFG_MAIN, weights, p, 12) for p in prompts]
    assert len({t for w in want for t in w}) >= 6, "the expected continuations say too little"
    # steps of at most 16 tokens: prompts are cut into portions that run beside other requests' decoded tokens
    engine = Engine(model=model, block_size=16, num_pages=32, max_seqs=3, max_tokens_per_step=16, prefill_chunk=16)
    assert engine.generate(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True) == want
    # too few pages for all at once: requests wait, or are preempted and recomputed
    small = Engine(model=model, block_size=16, num_pages=6, max_seqs=4, max_tokens_per_step=32, prefill_chunk=32)
    assert small.generate(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True) == want


def test_command_line_and_replay(tmp_path_factory):
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from conftest import ROOT
    weights = u.make_weights(u.CFG_MAIN, 3)
    folder = u.write_model(str(tmp_path_factory.mktemp("kovalorn_cli")), u.CFG_MAIN, weights)
    prompt = u.random_tokens(u.CFG_MAIN["vocab"], 9, 77)
    want = plain_greedy(u.CFG_MAIN, weights, prompt, 6)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ferrox-amd"), "-m", folder, "--tokens",
                          ",".join(map(str, prompt)), "-n", "6", "--temp", "0", "--repeat-penalty", "1.0", "--ignore-eos", "--dtype", "float32",
                          "--block-size", "16", "--num-pages", "16"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert ",".join(map(str, want)) in out.stdout.replace(" ", ""), (out.stdout[-500:], want)
    # the step-by-step replay: two requests, a portion beside a single token, logits at chosen places
    a, b = u.random_tokens(u.CFG_MAIN["vocab"], 30, 1), u.random_tokens(u.CFG_MAIN["vocab"], 4, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:29], "want": []}, {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[3:], "want": [0]}, {"id": "a", "tokens": a[29:], "want": [0]}], "end": ["a", "b"]}]
    out_dir = str(tmp_path_factory.mktemp("kovalorn_replay"))
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                          "--out", out_dir, "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [line for line in run.stdout.split("\n") if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    pa, pb = plain.forward(u.CFG_MAIN, weights, a), plain.forward(u.CFG_MAIN, weights, b)
    V = u.CFG_MAIN["vocab"]
    for step, rows in ((0, [pa[0], pa[16]]), (1, [pb[2]]), (2, [pb[3], pa[29]])):
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, V).copy())
        assert got.shape[0] == len(rows)
        assert float(u.row_errors(got, torch.stack(rows)).max()) <= u.LIMIT["float32"]
