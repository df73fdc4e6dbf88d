"""Helpers of the Kovalorn tests: small configurations, weights made in the test, and the comparison of the
engine's logits with the plain model (`plain_kovalorn`)."""
from __future__ import annotations

import torch

import plain_kovalorn as plain
from rafilix_util import random_tokens, row_errors, run_schedule, write_model  # noqa: F401  (schedules and files are alike)


def attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, window=24, keep_first=3, scale=0.3, kv_from=None, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        mixer["mask"] = {"size": window, "keep_first": keep_first}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=24, scale=1.3, shared_ff=40):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared_ff:
        out["shared"] = {"ff": shared_ff}
    return out


def config(layers, width=64, vocab=160, eps=1e-6, logit_scale=1.7):
    return {"architecture": "Kovalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": layers}


# Layers unlike each other: a dense and two sparse feed-forwards and none, one and several kv heads, key heads wider and
# narrower than value heads, a layer without a mask, readers of another layer's keys whose window is wider and
# narrower than the owner's, no kept keys, more kept keys than a page holds, top 1, no shared expert.
CFG_MAIN = config([
    attention_layer(heads=4, kv_heads=2, dim=32, vdim=16, window=20, keep_first=3, scale=0.3, mlp=dense(48)),
    attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, window=37, keep_first=0, scale=0.45, mlp=moe(6, 2, 24, 1.3, 40)),
    attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, window=50, keep_first=18, scale=0.4, kv_from=1, mlp=moe(5, 1, 16, 0.8, 0)),
    attention_layer(heads=2, kv_heads=1, dim=48, vdim=48, window=0, scale=0.25, mlp=None),
    attention_layer(heads=3, kv_heads=1, dim=48, vdim=48, window=9, keep_first=2, scale=0.3, kv_from=3, mlp=dense(24)),
    attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, window=11, keep_first=5, scale=0.5, kv_from=1, mlp=moe(3, 3, 8, 2.0, 8)),
], width=64, vocab=160)
# bfloat16 on the matrix units: equal head sizes in multiples of 16 (64 and 128 among them), widths in multiples of 64
CFG_MFMA = config([
    attention_layer(heads=4, kv_heads=2, dim=64, vdim=64, window=70, keep_first=9, scale=0.2, mlp=moe(8, 3, 64, 1.5, 128)),
    attention_layer(heads=4, kv_heads=2, dim=64, vdim=64, window=100, keep_first=70, scale=0.2, kv_from=0, mlp=dense(128)),
    attention_layer(heads=2, kv_heads=1, dim=128, vdim=128, window=33, keep_first=1, scale=0.15, mlp=moe(4, 2, 64, 1.0, 0)),
    attention_layer(heads=4, kv_heads=4, dim=32, vdim=32, window=150, keep_first=130, scale=0.3, mlp=None),
], width=128, vocab=256)


def tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a model's tensors, from its configuration."""
    W, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out.update({p + "mix.q": (H * D, W), p + "mix.sink": (H,), p + "mix.g": (H * V, W), p + "mix.o": (W, H * V)})
        if m.get("kv_from") is None:
            out.update({p + "mix.k": (G * D, W), p + "mix.v": (G * V, W)})
        f = layer.get("mlp")
        if not f:
            continue
        out[p + "norm2"] = (W,)
        gated = lambda q, ff: {q + "gate": (ff, W), q + "up": (ff, W), q + "down": (W, ff)}      # noqa: E731
        if f["kind"] == "dense":
            out.update(gated(p + "mlp.", f["ff"]))
        else:
            out[p + "mlp.router"] = (f["router"]["experts"], W)
            for e in range(f["router"]["experts"]):
                out.update(gated(p + f"mlp.e{e}.", f["expert"]["ff"]))
            if f.get("shared"):
                out.update(gated(p + "mlp.shared.", f["shared"]["ff"]))
    return out


def make_weights(cfg: dict, seed: int) -> dict:
    """Random weights, bfloat16 values, of a size that keeps every sublayer's output of order one: a missing key,
    a sink that is left out or a wrong expert then moves the logits."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if "norm" in last:
            t = 0.2 * torch.randn(shape, generator=gen)           # stored around zero
        elif last == "sink":
            t = 1.0 + torch.randn(shape, generator=gen)
        elif name == "embed":
            t = torch.randn(shape, generator=gen)
        elif last == "router":
            t = 3.0 * torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        else:
            t = 1.3 * torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


LIMIT = {"float32": 3e-5, "bfloat16": 4e-2}
MARGIN = 0.02      # a bfloat16 engine may exchange experts whose scores are this close


def check_against_plain(cfg, weights, requests, got, dtype, chosen=None, what=""):
    """Every position of every request against the plain model.  Under bfloat16 the plain model follows the
    engine's expert choices, which must be top choices of the plain router up to MARGIN."""
    worst = 0.0
    for r, tokens in requests.items():
        margins = []
        routing = chosen[r] if (chosen and chosen.get(r) is not None) else None
        want = plain.forward(cfg, weights, tokens, routing=routing, margins=margins)
        if routing is not None:
            assert max(margins, default=0.0) <= MARGIN, f"{what} {r}: an expert was chosen {max(margins):.3g} below the plain router's"
        err = row_errors(got[r], want)
        i = int(err.argmax())
        assert float(err[i]) <= LIMIT[dtype], (f"{what} request {r}: position {i} of {len(tokens)} is off by {float(err[i]):.3g} "
                                                f"(limit {LIMIT[dtype]:g}); first position over it: "
                                                f"{int((err > LIMIT[dtype]).nonzero()[0])}")
        worst = max(worst, float(err[i]))
    return worst
