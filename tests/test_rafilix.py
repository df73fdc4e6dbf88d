"""Rafilix without a GPU: the plain model's own properties (so that the oracle of the GPU tests is itself held to
the design's equations), the configuration reader, the model description's tensor names, and the cache manager's
chunked groups."""
import math

import pytest
import torch

import plain_rafilix as plain
import rafilix_util as u
from ferrox_amd.cache.manager import CacheManager
from ferrox_amd.config.base import ConfigError
from ferrox_amd.config.rafilix import RafilixConfig
from ferrox_amd.engine.model import Model
from ferrox_amd.models.rafilix import build_spec


# ---- the plain model ---------------------------------------------------------
def test_chunk_visibility():
    assert plain.chunk_visible(5, 5, 4) and plain.chunk_visible(5, 4, 4) and not plain.chunk_visible(5, 3, 4)
    assert not plain.chunk_visible(4, 5, 4) and plain.chunk_visible(3, 0, 4) and not plain.chunk_visible(4, 3, 4)
    assert plain.chunk_visible(100, 0, None) and plain.chunk_visible(7, 0, 8) and not plain.chunk_visible(8, 7, 8)


def test_rotation_keeps_lengths_and_depends_on_distance_only():
    freqs = plain.rotary_frequencies(8, 100.0, dict(factor=4.0, low=1.0, high=2.0, original=16.0))
    gen = torch.Generator().manual_seed(0)
    q, k = torch.randn(12, generator=gen, dtype=torch.float64), torch.randn(12, generator=gen, dtype=torch.float64)
    a = plain.rotate_interleaved(q, 9, freqs, "exact") @ plain.rotate_interleaved(k, 4, freqs, "exact")
    b = plain.rotate_interleaved(q, 25, freqs, "exact") @ plain.rotate_interleaved(k, 20, freqs, "exact")
    assert abs(a - b) < 1e-12
    r = plain.rotate_interleaved(q, 9, freqs, "exact")
    assert abs(r.norm() - q.norm()) < 1e-12 and torch.equal(r[8:], q[8:])     # the last four dimensions pass
    assert torch.allclose(plain.rotate_interleaved(q, 0, freqs), q)


def test_frequency_scaling_bands():
    plainf = plain.rotary_frequencies(16, 10000.0, None)
    scaled = plain.rotary_frequencies(16, 10000.0, dict(factor=8.0, low=1.0, high=4.0, original=64.0))
    for f, s in zip(plainf, scaled):
        wavelength = 2 * math.pi / f
        if wavelength < 16.0:
            assert s == f
        elif wavelength > 64.0:
            assert s == f / 8.0
        else:
            assert f / 8.0 <= s <= f
    assert scaled[0] == 1.0 and scaled[-1] == plainf[-1] / 8.0 and any(f / 8.0 < s < f for f, s in zip(plainf, scaled))


def test_short_convolution_is_causal_and_starts_from_zeros():
    gen = torch.Generator().manual_seed(1)
    x, taps = torch.randn(9, 3, generator=gen, dtype=torch.float64), torch.randn(3, 4, generator=gen, dtype=torch.float64)
    y = plain.short_conv_silu(x, taps)
    z = taps[:, 3] * x[0]
    assert torch.allclose(y[0], z * torch.sigmoid(z))                 # the last column is the current token's
    x2 = x.clone()
    x2[6:] += 1.0
    assert torch.equal(plain.short_conv_silu(x2, taps)[:6], y[:6])
    z = taps[:, 3] * x[5] + taps[:, 2] * x[4] + taps[:, 1] * x[3] + taps[:, 0] * x[2]
    assert torch.allclose(y[5], z * torch.sigmoid(z))


def test_delta_rule_reads_back_what_it_wrote():
    """With beta = 1, no decay and orthogonal unit keys, the state stores v_t under k_t: reading with q = k_s returns
    v_s (times the query's scale), also after later writes; a decay of g on a key's channel shrinks it by g a step."""
    D, V = 4, 3
    S = torch.zeros(D, V, dtype=torch.float64)
    keys, vals = torch.eye(D, dtype=torch.float64), torch.arange(12, dtype=torch.float64).view(4, 3) + 1
    for t in range(3):
        S = S + torch.outer(keys[t], 1.0 * (vals[t] - S.T @ keys[t]))
    assert torch.allclose(S.T @ keys[1], vals[1])
    S = S + torch.outer(keys[1], 1.0 * (vals[3] - S.T @ keys[1]))       # a second write under the same key replaces
    assert torch.allclose(S.T @ keys[1], vals[3]) and torch.allclose(S.T @ keys[0], vals[0])
    g = torch.tensor([0.5, 1.0, 1.0, 1.0], dtype=torch.float64)
    assert torch.allclose((g.view(D, 1) * S).T @ keys[0], 0.5 * vals[0])


def test_identity_experts_and_selection_bias():
    gen = torch.Generator().manual_seed(2)
    f = u.moe(experts=2, identity=2, top=2, ff=6)
    w = {"router": torch.randn(4, 5, generator=gen, dtype=torch.float64),
         "correction": torch.zeros(4, dtype=torch.float64)}
    for e in range(2):
        w[f"e{e}.up"], w[f"e{e}.down"] = (torch.randn(6, 5, generator=gen, dtype=torch.float64),
                                          torch.randn(5, 6, generator=gen, dtype=torch.float64))
    h = torch.randn(3, 5, generator=gen, dtype=torch.float64)
    scores = torch.softmax(h @ w["router"].T, -1)
    w["correction"] = torch.tensor([-9.0, -9.0, 0.0, 0.0], dtype=torch.float64)        # the bias pushes both experts out
    ids, wt = plain.route(h, w, f["router"])
    assert sorted(ids[0].tolist()) == [2, 3] and torch.allclose(wt, torch.gather(scores, 1, ids))    # weights without the bias
    assert torch.allclose(plain.moe(h, w, f), h * (scores[:, 2] + scores[:, 3]).view(3, 1))          # not renormalised
    w["correction"] = torch.tensor([9.0, -9.0, -9.0, -9.0], dtype=torch.float64)
    only = dict(f, router=dict(f["router"], top=1))
    z = torch.relu(h @ w["e0.up"].T)
    assert torch.allclose(plain.moe(h, w, only), scores[:, :1] * ((z * z) @ w["e0.down"].T))


def test_plain_model_decodes_as_it_prefills():
    """The plain model is causal: the logits of a prefix are those of the whole prompt at the same positions."""
    weights = u.make_weights(u.CFG_MAIN, 3)
    tokens = u.random_tokens(u.CFG_MAIN["vocab"], 30, 4)
    whole = plain.forward(u.CFG_MAIN, weights, tokens)
    part = plain.forward(u.CFG_MAIN, weights, tokens[:26])
    assert float(u.row_errors(part, whole[:26]).max()) < 1e-12
    layers = []
    plain.forward(u.CFG_MAIN, weights, tokens[:5], layers_out=layers)
    assert len(layers) == len(u.CFG_MAIN["layers"]) and layers[0].shape == (5, u.CFG_MAIN["width"])


# ---- configuration and description ------------------------------------------------
def test_config_reads_every_layer_and_refuses_what_it_does_not_know():
    cfg = RafilixConfig.from_dict(u.CFG_MAIN)
    assert [l.type for l in cfg.layers] == ["channel_delta", "attention", "channel_delta", "attention"]
    a = cfg.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.chunk, a.scale) == (4, 2, 32, 48, 24, 0.7)
    assert a.rot.dims == 16 and a.rot.scaling == (4.0, 1.0, 4.0, 64.0)
    assert cfg.layers[3].mixer.chunk is None and cfg.layers[2].mlp is None and cfg.layers[0].mlp.identity == 3
    assert RafilixConfig.from_dict(cfg.to_dict()) == cfg
    bad = [
        (lambda c: c["layers"][0].update(type="conv"), "type"),
        (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
        (lambda c: c["layers"][1]["mixer"].update(heads=3), "kv_heads"),
        (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34), "dims"),
        (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
        (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
        (lambda c: c.pop("norm"), "norm"),
        (lambda c: c.update(layers=[]), "layers"),
    ]
    import copy
    for change, word in bad:
        c = copy.deepcopy(u.CFG_MAIN)
        change(c)
        with pytest.raises(ConfigError) as e:
            RafilixConfig.from_dict(c)
        assert word in str(e.value), (word, str(e.value))


def test_named_shape_of_the_design_reads():
    from ferrox_amd.config import presets
    from ferrox_amd.models.registry import resolve
    raw = presets.load("rafilix-2k")
    assert resolve(raw).name == "Rafilix"
    cfg = RafilixConfig.from_dict(raw)
    assert len(cfg.layers) == 8 and {l.type for l in cfg.layers} == {"attention", "channel_delta"}
    assert cfg.layers[1].mixer.decay_rank == cfg.layers[1].mixer.dim        # named in the file: no checkpoint gives it


def test_description_names_the_tensors_of_the_test_models():
    """The tensor names and shapes that the model description expects are those that the tests' own list gives
    (written from the design, not from the description); the low-rank sizes come from the tensors."""
    from ferrox_amd.engine.loading import TensorNames

    class Source:
        def __init__(self, shapes):
            self.shapes = shapes

        def names(self):
            return list(self.shapes)

        def info(self, name):
            return torch.bfloat16, self.shapes[name]

    for cfg in (u.CFG_MAIN, u.CFG_MFMA):
        shapes = u.tensor_shapes(cfg, decay_rank=12, gate_rank=20)
        model = Model(build_spec(RafilixConfig.from_dict(cfg), TensorNames(Source(shapes))))
        got = {n: tuple(s.shape) for n, s in model.named_params().items()}
        assert got == {n: tuple(s) for n, s in shapes.items()}
    groups = Model(build_spec(RafilixConfig.from_dict(u.CFG_MAIN), None)).cache_groups()
    assert groups == {("chunk", 24): ("chunk", 24), ("full",): None}


# ---- the cache manager's chunked groups ---------------------------------------------
def test_chunked_group_gives_back_the_pages_of_ended_chunks():
    mgr = CacheManager({("chunk", 24): ("chunk", 24), ("full",): None}, 10, 16, 2)
    assert mgr.admit("a") is not None
    assert mgr.extend("a", 23) and mgr.trim("a") == 0                     # the first chunk is still open
    assert mgr.extend("a", 24) and mgr.trim("a") == 1                     # position 24 starts a chunk: page 0 (0..15) goes
    assert mgr.table("a", ("chunk", 24))[:2] == [-1, mgr.table("a", ("chunk", 24))[1]] and mgr.table("a", ("chunk", 24))[1] >= 0
    assert mgr.extend("a", 100) and mgr.trim("a") == 5                    # 96 starts the chunk in progress: pages below 96 go
    assert [p >= 0 for p in mgr.table("a", ("chunk", 24))] == [False] * 6 + [True]
    assert all(p >= 0 for p in mgr.table("a", ("full",)))
    mgr.check_invariants()
    assert mgr.admit("b") is not None and mgr.extend("b", 48) and mgr.trim("b") == 3
    mgr.release("a"), mgr.release("b")
    mgr.check_invariants()
    assert mgr.n_free_pages(("chunk", 24)) == 10 and mgr.n_free_pages(("full",)) == 10
    with pytest.raises(ValueError):
        CacheManager({"x": ("window", 3)}, 4, 16, 1)
