"""Rafilix on the GPU against the plain model (`plain_rafilix`): every mechanism alone, whole prompts, decoding
through the cache and the state slots, portions down to two tokens, unequal batches, pages and slots used again,
chunk and page edges, far keys, long decoding, other sizes, and generation through the engine's entry point."""
import pytest
import torch

import plain_rafilix as plain
import rafilix_util as u

pytestmark = pytest.mark.gpu

_models = {}


def model_for(tmp_path_factory, name, cfg, seed, dtype, **kw):
    """(folder weights as the plain model reads them, loaded engine model); made once per (name, dtype)."""
    from ferrox_amd.engine.loading import load_model
    key = (name, dtype)
    if key not in _models:
        weights = u.make_weights(cfg, seed, **kw)
        folder = u.write_model(str(tmp_path_factory.mktemp(f"rafilix_{name}")), cfg, weights)
        _models[key] = (weights, load_model(folder, dtype, "cuda:0"))
    return _models[key]


def runner_of(model, block_size=16, num_pages=24, max_seqs=4, **kw):
    from ferrox_amd.engine.runner import ModelRunner
    return ModelRunner(model, block_size=block_size, num_pages=num_pages, max_seqs=max_seqs, **kw)


def traced(dtype):
    from ferrox_amd import debug
    import contextlib
    return debug.trace_routing() if dtype == "bfloat16" else contextlib.nullcontext()


def run_and_check(cfg, weights, model, requests, schedule, dtype, what, **runner_kw):
    runner = runner_of(model, **runner_kw)
    with traced(dtype) as trace:
        got, chosen = u.run_schedule(runner, requests, schedule, trace)
    for key in runner.manager.groups:          # (a model of recurrent layers alone keeps no pages)
        assert runner.manager.n_free_pages(key) == runner_kw.get("num_pages", 24), "pages were lost"
    return u.check_against_plain(cfg, weights, requests, got, dtype, chosen, what)


# ---------------------------------------------------------------------------
# each mechanism alone: models of one layer
# ---------------------------------------------------------------------------
SINGLE = {
    "attention_plain": u.config([u.attention_layer(heads=2, kv_heads=2, dim=16, vdim=16, chunk=0, rot_dims=0, scale=0.6)]),
    "attention_chunked": u.config([u.attention_layer(heads=4, kv_heads=1, dim=32, vdim=16, chunk=10, rot_dims=0, scale=0.6)]),
    "attention_rotated": u.config([u.attention_layer(heads=4, kv_heads=2, dim=32, vdim=64, chunk=0, rot_dims=24,
                                                     scaling=(6.0, 1.0, 3.0, 40.0), base=500.0, scale=0.8)]),
    "delta": u.config([u.delta_layer(heads=4, kv_heads=2, dim=32, vdim=16, conv=3)]),
    "delta_wide_key": u.config([u.delta_layer(heads=2, kv_heads=1, dim=144, vdim=40, conv=1)]),
    "moe": u.config([u.attention_layer(heads=1, kv_heads=1, dim=16, vdim=16, chunk=0, rot_dims=0, mlp=u.moe(5, 3, 3, 40))]),
    "moe_identity_only": u.config([u.attention_layer(heads=1, kv_heads=1, dim=16, vdim=16, chunk=0, rot_dims=0,
                                                     mlp=u.moe(0, 3, 2, 8))]),
}


@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_alone(tmp_path_factory, name):
    cfg = SINGLE[name]
    weights, model = model_for(tmp_path_factory, name, cfg, 11, "float32")
    requests = {"a": u.random_tokens(cfg["vocab"], 37, 1), "b": u.random_tokens(cfg["vocab"], 5, 2)}
    # whole, then the same requests cut: a prompt portion, a portion of two, single tokens
    run_and_check(cfg, weights, model, requests, [[("a", 37)], [("b", 5)]], "float32", name + " whole")
    cut = [[("a", 20), ("b", 2)], [("a", 2), ("b", 1)], [("a", 1), ("b", 1)]] + [[("a", 1)]] * 14 + [[("b", 1)]]
    run_and_check(cfg, weights, model, requests, cut, "float32", name + " cut")


def test_scaled_frequencies_cover_all_three_bands():
    """The table of the rotation with wavelength-dependent scaling, against the plain formula; the test's
    constants put pairs into each of the three bands."""
    from ferrox_amd.parts.rope import scaled_frequencies
    got = scaled_frequencies(24, 500.0, (6.0, 1.0, 3.0, 40.0))
    want = plain.rotary_frequencies(24, 500.0, dict(factor=6.0, low=1.0, high=3.0, original=40.0))
    unscaled = plain.rotary_frequencies(24, 500.0, None)
    kept = sum(1 for a, b in zip(want, unscaled) if a == b)
    divided = sum(1 for a, b in zip(want, unscaled) if abs(a - b / 6.0) < 1e-15 and a != b)
    assert kept >= 1 and divided >= 1 and kept + divided < len(want), (kept, divided)
    assert max(abs(a - b) / b for a, b in zip(got, want)) < 1e-14


def test_router_selection_bias_and_identity_kernels():
    """The selection by score + bias with the scores as weights, and the combine that hands the input through
    for identity experts, against plain formulas; 70 router outputs take the kernel's path for more than 64."""
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(5)
    for E, k, T in ((8, 3, 9), (70, 5, 33), (3, 3, 2)):
        logits = torch.randn(T, E, generator=gen)
        bias = 0.3 * torch.randn(E, generator=gen)
        ids, w, _ = ops.router_select(logits.cuda(), E, k, False, selection_bias=bias.cuda())
        s = torch.softmax(logits.double(), -1)
        want = torch.topk(s + bias.double(), k, dim=-1).indices
        assert ids.cpu().tolist() == want.tolist()
        assert torch.allclose(w.cpu().double(), torch.gather(s, 1, want), atol=1e-6)
    T, H, k, E = 7, 40, 3, 4
    ids = torch.randint(0, E + 2, (T, k), generator=gen, dtype=torch.int32)
    w = torch.rand(T, k, generator=gen)
    y = torch.randn(T * k, H, generator=gen)
    x = torch.randn(T, H, generator=gen)
    y_dev = y.clone()
    y_dev[(ids.reshape(-1) >= E)] = float("nan")          # rows of identity pairs are never used
    mixed = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            mixed[t] += w[t, j].double() * (y[t * k + j].double() if ids[t, j] < E else x[t].double())
    nw = 1.0 + 0.1 * torch.randn(H, generator=gen)
    for post, want in ((None, mixed), ((nw.cuda(), 1e-5), plain.rms_norm(mixed, nw.double(), 1e-5))):
        h = torch.ones(T, H).cuda()
        ops.moe_combine_identity(h, y_dev.cuda(), ids.cuda(), w.cuda(), x.cuda(), E, post)
        assert torch.allclose(h.cpu().double(), 1.0 + want, atol=2e-5)


def test_stored_activation_of_the_product():
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(6)
    for M, N, K, dt in ((5, 24, 40, torch.float32), (70, 64, 128, torch.bfloat16), (300, 96, 64, torch.bfloat16)):
        a, w = torch.randn(M, K, generator=gen).to(dt), (torch.randn(N, K, generator=gen) / K ** 0.5).to(dt)
        got = ops.gemm(a.cuda(), w.cuda(), store_activation="relu2").float().cpu()
        want = torch.relu(a.double() @ w.double().T) ** 2
        assert torch.allclose(got.double(), want, atol=1e-5 if dt == torch.float32 else 3e-2, rtol=1e-2)


def test_pair_of_small_products():
    """The one-launch pair of float32 products for few rows against float64 products, and bit for bit against the
    float32 product kernel that takes more rows (a row must not change with the number of rows beside it)."""
    from ferrox_amd import ops
    gen = torch.Generator().manual_seed(8)
    for T, K0, N0, K1, N1 in ((1, 12, 40, 20, 7), (9, 128, 600, 64, 300), (32, 5, 3, 300, 257)):
        big = torch.randn(T, K0 + K1 + 3, generator=gen).cuda()
        x0, x1 = big[:, :K0], big[:, K0 + 3:]                       # rows with a stride of their own
        w0, w1 = torch.randn(N0, K0, generator=gen).cuda(), torch.randn(N1, K1, generator=gen).cuda()
        a, b = ops.small_rows_pair(x0, w0.t().contiguous(), x1, w1.t().contiguous())
        for got, x, w in ((a, x0, w0), (b, x1, w1)):
            want = x.double() @ w.double().T
            assert torch.allclose(got.double(), want, atol=1e-4 * float(want.abs().max()))
            assert torch.equal(got, ops.gemm(x, w, epilogue=ops.EPI_STORE_F32))


# ---------------------------------------------------------------------------
# the model whole and cut
# ---------------------------------------------------------------------------
LENGTHS = [1, 2, 23, 50, 97]       # a single token, two, below a chunk, across chunks and pages


def main_requests():
    return {f"r{n}": u.random_tokens(u.CFG_MAIN["vocab"], n, 40 + n) for n in LENGTHS}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts_and_decoding(tmp_path_factory, dtype):
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, dtype)
    reqs = main_requests()
    run_and_check(u.CFG_MAIN, weights, model, reqs, [[(r, len(t))] for r, t in reqs.items()], dtype, "whole")
    # most of a prompt in one step, the last 30 tokens (or all but one) one by one: across the chunk edges at 24 and
    # 48 or 72 and 96, and the page borders at 16, 32, ...
    sched = []
    for r, t in reqs.items():
        first = max(1, len(t) - 30)
        sched += [[(r, first)]] + [[(r, 1)]] * (len(t) - first)
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, dtype, "decode")
    # token by token from the first token on (the recurrence from its zero state, the first chunk from its start)
    one = {"r23": reqs["r23"]}
    run_and_check(u.CFG_MAIN, weights, model, one, [[("r23", 1)]] * 23, dtype, "token by token")


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
    """Up to three live requests under three slots and a pool of 14 pages of 16 (the requests' sum needs 18): portions beside single tokens, requests that pause, slots and pages taken again by later requests."""
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


def test_a_used_slot_and_used_pages_start_clean(tmp_path_factory):
    """One slot and just enough pages: every request takes the slot and the pages that the one before left."""
    weights, model = model_for(tmp_path_factory, "main", u.CFG_MAIN, 3, "float32")
    reqs = {f"q{i}": u.random_tokens(u.CFG_MAIN["vocab"], n, 70 + i) for i, n in enumerate([33, 48, 9, 40])}
    sched = []
    for r, t in reqs.items():
        sched += [[(r, len(t) - 3)]] + [[(r, 1)]] * 3
    run_and_check(u.CFG_MAIN, weights, model, reqs, sched, "float32", "one slot", num_pages=3, max_seqs=1)


# ---------------------------------------------------------------------------
# where a fault hides behind random weights: peaked attention, long memory
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_chunk_edges_and_page_borders_stand_out(tmp_path_factory, dtype):
    """A large score scale makes the softmax pick single keys, so that a key just inside the chunk (its first
    position) that is missed, or one just outside (the last of the chunk before) that is seen, moves the logits far
    beyond rounding: with scale 4 over normed heads of 32 the largest score leads by several units.  Prompts end and
    decoding runs on both sides of the chunk edges (40, 80) and the page borders (16, 32, ...)."""
    # (bfloat16 rounds q and k to 8 bits: with scale 4 that alone moves the scores by a tenth and the logits past any
    # bound that would still see a fault, so the bfloat16 run is made with scale 1.5 and a lower bar for the plain
    # model's own sensitivity, still three times the test's limit)
    scale, bar = {"float32": (4.0, 0.3), "bfloat16": (1.5, 0.12)}[dtype]
    cfg = u.config([u.attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, chunk=40, rot_dims=32, scale=scale,
                                      mlp=u.moe(4, 1, 2, 32)),
                    u.attention_layer(heads=2, kv_heads=1, dim=32, vdim=32, chunk=0, rot_dims=16, scale=scale)], width=64)
    weights, model = model_for(tmp_path_factory, "peaked" + dtype, cfg, 21, dtype)
    # the plain model itself must tell the cases apart: one position more or less in the chunk moves its logits
    tokens = u.random_tokens(cfg["vocab"], 90, 5)
    right = plain.forward(cfg, weights, tokens)
    for size in (39, 41):
        other = dict(cfg, layers=[dict(cfg["layers"][0], mixer=dict(cfg["layers"][0]["mixer"], mask={"size": size})),
                                  cfg["layers"][1]])
        assert float(u.row_errors(plain.forward(other, weights, tokens), right).max()) > bar
    reqs = {"p": tokens}
    for first in (39, 40, 41, 79, 80, 81, 1):
        sched = [[("p", first)]] + [[("p", 1)]] * min(12, 90 - first)
        left = 90 - first - min(12, 90 - first)
        if left:
            sched.append([("p", left)])
        run_and_check(cfg, weights, model, reqs, sched, dtype, f"edge {first}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_state_far_back_still_counts(tmp_path_factory, dtype):
    """Decays close to one (A_log around -4): what the first tokens wrote into the state is read 150 tokens later.
    The plain model shows it (another first token moves the last logits); the engine carries it through portions,
    single tokens and a pause, in a state slot that another request used before."""
    cfg = u.config([u.delta_layer(heads=4, kv_heads=2, dim=32, vdim=32, conv=4, mlp=u.moe(4, 2, 2, 32)),
                    u.delta_layer(heads=2, kv_heads=2, dim=64, vdim=16, conv=2)], width=64)
    weights, model = model_for(tmp_path_factory, "longmemory", cfg, 31, dtype, slow_decay=True)
    tokens = u.random_tokens(cfg["vocab"], 160, 9)
    changed = [(tokens[0] + 1) % cfg["vocab"]] + tokens[1:]
    moved = u.row_errors(plain.forward(cfg, weights, changed)[-1:], plain.forward(cfg, weights, tokens)[-1:])
    assert float(moved) > 100 * u.LIMIT["float32"], float(moved)      # (far above float32 rounding; bfloat16 runs the same path)
    reqs = {"before": u.random_tokens(cfg["vocab"], 20, 1), "long": tokens}
    sched = [[("before", 20)], [("long", 3)], [("long", 2)], [("long", 70)]] + [[("long", 1)]] * 40 + [[("long", 45)]]
    run_and_check(cfg, weights, model, reqs, sched, dtype, "long memory", max_seqs=1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_on_the_matrix_units(tmp_path_factory, dtype):
    """Sizes that take the bfloat16 kernels' matrix-unit paths (equal head sizes in multiples of 16, widths in
    multiples of 64, pages of 64): a prompt, then 140 tokens one by one from recorded steps, across chunk edges at
    40, 80, ... and 100, and two requests decoding side by side."""
    weights, model = model_for(tmp_path_factory, "mfma", u.CFG_MFMA, 17, dtype)
    reqs = {"x": u.random_tokens(u.CFG_MFMA["vocab"], 200, 3), "y": u.random_tokens(u.CFG_MFMA["vocab"], 150, 4)}
    sched = [[("x", 60)], [("y", 10)]] + [[("x", 1), ("y", 1)]] * 140
    run_and_check(u.CFG_MFMA, weights, model, reqs, sched, dtype, "long decode", block_size=64, num_pages=8)
    whole = [[("x", 200), ("y", 150)]]
    run_and_check(u.CFG_MFMA, weights, model, reqs, whole, dtype, "whole", block_size=64, num_pages=8)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_fit_no_vector(tmp_path_factory, dtype):
    """Head sizes, widths and a vocabulary that are no multiples of 16, 8 or 4: the kernels' guarded paths."""
    cfg = u.config([u.attention_layer(heads=3, kv_heads=3, dim=24, vdim=40, chunk=7, rot_dims=10, scale=0.6, mlp=u.moe(3, 1, 2, 20)),
                    u.delta_layer(heads=3, kv_heads=1, dim=30, vdim=10, conv=2, mlp=u.moe(2, 2, 1, 12)),
                    u.attention_layer(heads=2, kv_heads=1, dim=18, vdim=6, chunk=0, rot_dims=18, scale=0.5)], width=70, vocab=151)
    weights, model = model_for(tmp_path_factory, "odd", cfg, 13, dtype, decay_rank=5, gate_rank=7)
    reqs = {"a": u.random_tokens(151, 45, 1), "b": u.random_tokens(151, 20, 2)}
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 17)]] + [[("a", 1), ("b", 1)]] + [[("a", 1)]] * 13
    run_and_check(cfg, weights, model, reqs, sched, dtype, "odd sizes")


def test_pages_of_ended_chunks_are_given_back(tmp_path_factory):
    """A chunked layer needs the pages of the chunk in progress only: with every attention layer chunked, a prompt
    of 200 tokens runs in a pool of 5 pages of 16 (chunks of 40 span at most 4), in portions of at most a chunk."""
    cfg = u.config([u.attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, chunk=40, rot_dims=16, scale=1.0, mlp=u.moe(3, 1, 1, 16)),
                    u.delta_layer(heads=2, kv_heads=1, dim=16, vdim=16, conv=2)], width=32)
    weights, model = model_for(tmp_path_factory, "giveback", cfg, 8, "float32")
    reqs = {"z": u.random_tokens(cfg["vocab"], 200, 2)}
    sched = [[("z", 8)]] * 24 + [[("z", 1)]] * 8
    run_and_check(cfg, weights, model, reqs, sched, "float32", "give back", num_pages=5)


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
    # too few pages for all at once: requests wait, or are preempted and recomputed, state slot and all
    small = Engine(model=model, block_size=16, num_pages=6, max_seqs=4, max_tokens_per_step=32, prefill_chunk=32)
    assert small.generate(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True) == want


def test_command_line_generates(tmp_path_factory):
    import os
    import subprocess
    import sys
    from conftest import ROOT
    weights = u.make_weights(u.CFG_MAIN, 3)
    folder = u.write_model(str(tmp_path_factory.mktemp("rafilix_cli")), u.CFG_MAIN, weights)
    prompt = u.random_tokens(u.CFG_MAIN["vocab"], 9, 77)
    want = plain_greedy(u.CFG_MAIN, weights, prompt, 6)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ferrox-amd"), "-m", folder, "--tokens",
                          ",".join(map(str, prompt)), "-n", "6", "--temp", "0", "--repeat-penalty", "1.0", "--ignore-eos", "--dtype", "float32",
                          "--block-size", "16", "--num-pages", "16"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert ",".join(map(str, want)) in out.stdout.replace(" ", ""), (out.stdout[-500:], want)
    # without a folder: random weights of a named shape of the design (two of its layers)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ferrox-amd"), "--random-weights", "--config", "rafilix-2k",
                          "--layers", "2", "-s", "5", "--tokens", "1,2,3", "-n", "4", "--temp", "0", "--ignore-eos",
                          "--num-pages", "8"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert len(out.stdout.strip().split(",")) == 4, out.stdout[-300:]
