"""Kovalorn without a GPU: the plain model's own properties, the configuration reader, the description's tensor
names, the cache groups that keep the first keys of a sequence beside a window."""
import math

import pytest
import torch

import kovalorn_util as u
import plain_kovalorn as plain
from ferrox_amd.cache.manager import CacheManager
from ferrox_amd.config.base import ConfigError
from ferrox_amd.config.kovalorn import KovalornConfig
from ferrox_amd.engine.model import Model
from ferrox_amd.models.kovalorn import build_spec, cache_retention
from ferrox_amd.models.registry import resolve


# ---------------------------------------------------------------------------
# the plain model
# ---------------------------------------------------------------------------
def test_visibility_of_window_and_kept_keys():
    see = plain.visible(12, 4, 2)
    assert see[11].tolist() == [True, True] + [False] * 6 + [True] * 4
    assert see[3].tolist() == [True] * 4 + [False] * 8            # the window still reaches the start
    assert see[0].tolist() == [True] + [False] * 11               # a kept key that is not there yet is not seen
    assert plain.visible(5, 5, 0).tolist() == torch.tril(torch.ones(5, 5)).bool().tolist()


def test_the_sink_takes_weight_and_brings_no_value():
    cfg = u.config([u.attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=0)])
    w = u.make_weights(cfg, 1)
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(6, 64, dtype=torch.float64)
    kv = plain.keys_values(h, w, "l0.mix.", m, 1e-6)
    # with one key (the first position) the softmax weight of the key is 1 / (1 + exp(sink - score))
    w_open = dict(w, **{"l0.mix.g": w["l0.mix.g"] * 0, "l0.mix.o": torch.eye(64)[:, :32].to(torch.bfloat16)})      # gate 1/2, identity out
    out = plain.attention(h[:1], w_open, "l0.mix.", m, 1e-6, (kv[0][:1], kv[1][:1]))
    q = plain.unit_rms((h[:1] @ w["l0.mix.q"].double().T).view(1, 2, 16), 1e-6)
    for a in range(2):
        score = float((q[0, a] * kv[0][0, 0]).sum()) * m["scale"]
        share = 1.0 / (1.0 + math.exp(float(w["l0.mix.sink"][a]) - score))
        assert torch.allclose(out[0, 16 * a:16 * a + 16], 0.5 * share * kv[1][0, 0], atol=1e-12)


def test_unit_heads_and_offset_norm():
    x = torch.randn(5, 3, 16, dtype=torch.float64) * 7
    assert torch.allclose((plain.unit_rms(x, 0.0) ** 2).mean(-1), torch.ones(5, 3, dtype=torch.float64))
    w = torch.zeros(16, dtype=torch.float64)
    assert torch.allclose(plain.offset_norm(x, w, 0.0), plain.unit_rms(x, 0.0))      # a stored weight of zero is a weight of one


def test_router_weights_sum_to_the_constant():
    h = torch.randn(9, 32, dtype=torch.float64)
    wr = torch.randn(7, 32)
    ids, wts = plain.router_choice(h, wr, 3, 1.7)
    assert torch.allclose(wts.sum(-1), torch.full((9,), 1.7, dtype=torch.float64))
    s = torch.sigmoid(h @ wr.double().T)
    assert all(set(ids[t].tolist()) == set(torch.argsort(s[t], descending=True)[:3].tolist()) for t in range(9))


def test_a_reader_of_another_layers_keys_sees_them():
    """Layer 1 reads layer 0's keys and values: changing layer 0's key projection changes layer 1's mixer even
    where layer 1's input is held fixed, and layer 1 has no such tensors of its own."""
    cfg = u.config([u.attention_layer(window=12), u.attention_layer(window=30, keep_first=0, kv_from=0)])
    shapes = u.tensor_shapes(cfg)
    assert "l0.mix.k" in shapes and "l1.mix.k" not in shapes and "l1.mix.v" not in shapes and "l1.mix.q" in shapes
    w = u.make_weights(cfg, 4)
    tokens = u.random_tokens(cfg["vocab"], 20, 1)
    a = plain.forward(cfg, w, tokens)
    b = plain.forward(cfg, dict(w, **{"l0.mix.v": w["l0.mix.v"] * 0}), tokens)
    assert float(u.row_errors(b, a).max()) > 0.01


# ---------------------------------------------------------------------------
# configuration and description
# ---------------------------------------------------------------------------
def test_configuration_reads_every_size_from_the_file():
    c = KovalornConfig.from_dict(u.CFG_MAIN)
    assert resolve(u.CFG_MAIN).name == "Kovalorn"
    assert (c.vocab, c.width, c.logit_scale, len(c.layers)) == (160, 64, 1.7, 6)
    m = c.layers[2].mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.window, m.keep_first, m.kv_from) == (6, 3, 16, 24, 50, 18, 1)
    assert c.layers[3].mixer.window is None and c.layers[3].mlp is None
    f = c.layers[1].mlp
    assert (f.ff, f.experts, f.top, f.scale, f.shared_ff) == (24, 6, 2, 1.3, 40)
    assert c.layers[2].mlp.shared_ff == 0 and c.layers[0].mlp.ff == 48
    assert c.to_dict()["layers"] == u.CFG_MAIN["layers"]


@pytest.mark.parametrize("change,complaint", [
    (lambda c: c["layers"][0].update(type="recurrent"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "multiple"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "earlier"),
    (lambda c: c["layers"][5]["mixer"].update(kv_from=2), "no keys and values of its own"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=1), "other key and value heads"),
    (lambda c: c["layers"][1]["mlp"].update(kind="conv"), "kind"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][0]["mixer"].update(dim=512), "attention kernels"),
])
def test_configuration_refusals(change, complaint):
    import copy
    raw = copy.deepcopy(u.CFG_MAIN)
    change(raw)
    with pytest.raises(ConfigError, match=complaint):
        KovalornConfig.from_dict(raw)


def test_tensor_names_and_shapes_of_the_description():
    for cfg in (u.CFG_MAIN, u.CFG_MFMA):
        model = Model(build_spec(KovalornConfig.from_dict(cfg)))
        assert {k: tuple(v.shape) for k, v in model.named_params().items()} == u.tensor_shapes(cfg)


def test_a_cache_holds_what_its_widest_reader_sees():
    c = KovalornConfig.from_dict(u.CFG_MAIN)
    need = cache_retention(c)
    assert need[1] == need[2] == need[5] == (50, 18)      # the owner's 37 / 0, its readers' 50 / 18 and 11 / 5
    assert need[0] == (20, 3)
    assert need[3] == need[4] == (None, 0)                 # a layer without a mask keeps every key, also for a windowed reader
    model = Model(build_spec(c))
    assert model.cache_groups() == {("window", 20, "keep", 3): ("keep", 20, 3), ("window", 50, "keep", 18): ("keep", 50, 18),
                                    ("full",): None}
    assert [e.cache for e in model.schedule] == [None, None, 1, None, 3, 1]


# ---------------------------------------------------------------------------
# pages of a window that keeps the first keys
# ---------------------------------------------------------------------------
def test_pages_under_the_window_go_back_and_the_first_stay():
    key = ("window", 10, "keep", 5)
    m = CacheManager({key: ("keep", 10, 5), ("window", 10): 10}, num_pages=12, block_size=4, n_slots=2)
    assert m.admit("a") is not None and m.extend("a", 41)
    assert m.trim("a") > 0
    kept, plain_window = m.table("a", key), m.table("a", ("window", 10))
    # every later query sees keys >= 41 - 10 + 1 = 32: pages 8.. stay in both; the pages of the first 5 keys stay in one
    assert [p >= 0 for p in plain_window] == [False] * 8 + [True] * 3
    assert [p >= 0 for p in kept] == [True, True] + [False] * 6 + [True] * 3
    m.check_invariants()
    assert m.extend("a", 48) and m.trim("a") >= 0
    assert [p >= 0 for p in m.table("a", key)][:3] == [True, True, False]
    m.release("a")
    m.check_invariants()
    assert m.n_free_pages(key) == 12 and m.n_free_pages(("window", 10)) == 12
    with pytest.raises(ValueError):
        CacheManager({"k": ("keep", 0, 3)}, num_pages=4, block_size=4, n_slots=1)
