"""Helpers of the Rafilix tests: small configurations, weights made in the test, schedules through the engine's
step function, and the comparison with the plain model (`plain_rafilix`)."""
from __future__ import annotations

import json
import os

import torch

import plain_rafilix as plain


def attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, chunk=24, rot_dims=None, base=10000.0, scaling=None,
                    scale=0.5, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        mixer["mask"] = {"size": chunk}
    if rot_dims is None:
        rot_dims = dim
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def delta_layer(heads=4, kv_heads=2, dim=32, vdim=16, conv=3, mlp=None):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp}


def moe(experts=5, identity=3, top=3, ff=40):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}


def config(layers, width=64, vocab=160, eps=1e-6):
    return {"architecture": "Rafilix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# three layers of each kind, sizes unlike each other: partial rotation with scaled frequencies, value heads wider and
# narrower than key heads, one kv head and several, key sizes on both sides of 64, one and three taps, top 1 and 3,
# with and without identity experts, a layer without feed-forward, a layer without mask
CFG_MAIN = config([
    delta_layer(heads=4, kv_heads=2, dim=32, vdim=16, conv=3, mlp=moe(5, 3, 3, 40)),
    attention_layer(heads=4, kv_heads=2, dim=32, vdim=48, chunk=24, rot_dims=16, scaling=(4.0, 1.0, 4.0, 64.0), scale=0.7,
                    mlp=moe(4, 0, 1, 24)),
    delta_layer(heads=2, kv_heads=2, dim=80, vdim=24, conv=2, mlp=None),
    attention_layer(heads=6, kv_heads=1, dim=16, vdim=16, chunk=0, rot_dims=16, scale=0.9, mlp=moe(3, 2, 2, 16)),
], width=64, vocab=160)
# bfloat16 on the matrix units: equal head sizes that are multiples of 16, widths that are multiples of 64
CFG_MFMA = config([
    attention_layer(heads=4, kv_heads=2, dim=64, vdim=64, chunk=40, rot_dims=64, scaling=(4.0, 1.0, 8.0, 96.0), scale=0.3,
                    mlp=moe(6, 1, 3, 64)),
    delta_layer(heads=4, kv_heads=4, dim=64, vdim=48, conv=3, mlp=moe(5, 3, 2, 64)),
    attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, chunk=100, rot_dims=32, scale=0.4, mlp=None),
], width=128, vocab=256)


def tensor_shapes(cfg: dict, decay_rank: int = 12, gate_rank: int = 20) -> dict:
    """Names and shapes of a model's tensors, from its configuration."""
    W, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            out.update({p + "mix.q": (H * D, W), p + "mix.k": (G * D, W), p + "mix.v": (G * V, W), p + "mix.o": (W, H * V),
                        p + "mix.q.norm": (D,), p + "mix.k.norm": (D,)})
        else:
            t = m["conv"]
            out.update({p + "mix.q": (G * D, W), p + "mix.q.conv": (G * D, t), p + "mix.k": (G * D, W), p + "mix.k.conv": (G * D, t),
                        p + "mix.v": (H * V, W), p + "mix.v.conv": (H * V, t), p + "mix.b": (H, W), p + "mix.A_log": (H,),
                        p + "mix.norm": (V,), p + "mix.a1": (decay_rank, W), p + "mix.a2": (H * D, decay_rank),
                        p + "mix.dt_bias": (H * D,), p + "mix.g1": (gate_rank, W), p + "mix.g2": (H * V, gate_rank),
                        p + "mix.o": (W, H * V)})
        f = layer.get("mlp")
        if f:
            r = f["router"]
            out[p + "norm2"] = out[p + "norm2b"] = (W,)
            out[p + "mlp.router"] = (r["experts"] + r["identity"], W)
            out[p + "mlp.correction"] = (r["experts"] + r["identity"],)
            for e in range(r["experts"]):
                out[p + f"mlp.e{e}.up"] = (f["expert"]["ff"], W)
                out[p + f"mlp.e{e}.down"] = (W, f["expert"]["ff"])
    return out


def make_weights(cfg: dict, seed: int, slow_decay: bool = False, **ranks) -> dict:
    """Random weights, bfloat16 values, of a size that keeps every sublayer's output of order one: a missing key,
    a lost state or a wrong expert then moves the logits."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, **ranks).items():
        last = name.split(".")[-1]
        if "norm" in last or last.startswith("norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=gen)
        elif last == "A_log":
            t = (-4.0 if slow_decay else -1.5) + 0.5 * torch.randn(shape, generator=gen)
        elif last == "dt_bias":
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last == "correction":
            t = 0.15 * torch.randn(shape, generator=gen)
        elif last == "embed" or name == "embed":
            t = torch.randn(shape, generator=gen)
        elif last == "router":
            t = 2.0 * torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        else:
            t = 1.3 * torch.randn(shape, generator=gen) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_model(folder: str, cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    return folder


def random_tokens(vocab: int, n: int, seed: int) -> list:
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=gen).tolist()


def run_schedule(runner, requests: dict, schedule: list, trace=None) -> tuple:
    """Feeds `requests` (id -> tokens) through the step function: `schedule` is a list of steps, a step a list of
    (id, number of next tokens).  Every position's logits are asked for.  A request is admitted at its first entry
    and released after its last token.  Returns (id -> float32 logits [len, vocab] on the CPU, id -> per feed-forward
    the chosen experts [len, top] if `trace` is an active routing trace)."""
    from ferrox_amd.engine.runner import StepEntry
    at = {r: 0 for r in requests}
    rows = {r: [] for r in requests}
    chosen = {r: None for r in requests}
    for step in schedule:
        entries = []
        for r, n in step:
            if r not in runner.manager:
                assert runner.admit(r), f"no slot for {r}"
            assert runner.reserve(r, n), f"no pages for {r}"
            entries.append(StepEntry(r, requests[r][at[r]:at[r] + n], list(range(n))))
        logits = runner.step(entries).float().cpu()
        calls = trace.read() if trace is not None else None
        o = 0
        for (r, n), e in zip(step, entries):
            rows[r].append(logits[o:o + n])
            if calls is not None:
                if chosen[r] is None:
                    chosen[r] = [[] for _ in calls]
                for c, ids in enumerate(calls):
                    chosen[r][c] += ids[o:o + n]
            o += n
            at[r] += n
            if at[r] == len(requests[r]):
                runner.release(r)
        runner.manager.check_invariants()
    assert all(at[r] == len(requests[r]) for r in requests), "the schedule does not cover every request"
    return {r: torch.cat(v) for r, v in rows.items()}, chosen


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per position: root mean square of the difference of the logits over that of the wanted logits (means taken off)."""
    d = got.double() - want.double()
    d = d - d.mean(dim=-1, keepdim=True)
    w = want.double() - want.double().mean(dim=-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


LIMIT = {"float32": 3e-5, "bfloat16": 4e-2}
MARGIN = 0.02      # a bfloat16 engine may exchange experts whose choice scores are this close


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
