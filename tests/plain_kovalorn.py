"""Kovalorn, written out plainly: one function per mechanism, float64, whole sequences, no cache.

The oracle of the tests.  It shares nothing with the package: weights come in as a dict
name -> tensor ([out, in] matrices), the configuration as the dict that config.json holds.

A layer is  x += mixer(N(x)); x += ff(N(x))  with N(x) = x / sqrt(mean(x^2) + eps) * (1 + w).
The mixer is grouped-query attention without positions in its scores: every head of q and k is
brought to unit root mean square, scores are (q.k) * scale over the keys j <= i that lie in the
window (i - j < W) or among the first F of the sequence, the softmax's denominator has one more
term exp(sink_h), the heads are gated by sigmoid(W_g x) and projected.  A layer may read another
layer's keys and values.  The feed-forward is a tanh-gelu gated one, or a mixture of silu-gated
experts chosen by the largest sigmoid scores, weighted by score / sum of the chosen * scale, plus
a shared expert.  The head is the embedding table, times a constant.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def offset_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * (1 + w), rows of x."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + w)


def unit_rms(x, eps):
    """Every row of the last dimension divided by its root mean square."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def visible(n: int, window: int, keep_first: int):
    """[n, n] bool: query i (row) sees key j (column)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & ((i - j < window) | (j < keep_first))


def keys_values(h, w, pre, m, eps):
    """Keys (normed) [n, G, dim] and values [n, G, vdim] that a layer with projections makes from its input rows."""
    n = h.shape[0]
    k = (h @ w[pre + "k"].to(F64).T).view(n, m["kv_heads"], m["dim"])
    v = (h @ w[pre + "v"].to(F64).T).view(n, m["kv_heads"], m["vdim"])
    return unit_rms(k, eps), v


def attention(h, w, pre, m, eps, kv):
    """The mixer's output [n, width] from its input rows h and the (keys, values) it reads."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ w[pre + "q"].to(F64).T).view(n, H, D), eps)
    k, v = kv
    mask = m.get("mask")
    see = visible(n, mask["size"], mask.get("keep_first", 0)) if mask else visible(n, n, 0)
    sink = w[pre + "sink"].to(F64)
    out = torch.zeros(n, H, V, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~see, -math.inf)
        top = torch.maximum(s.max(-1, keepdim=True).values, sink[a])
        e = torch.exp(s - top)
        out[:, a] = (e / (e.sum(-1, keepdim=True) + torch.exp(sink[a] - top))) @ v[:, g]
    gate = torch.sigmoid(h @ w[pre + "g"].to(F64).T)
    return (out.reshape(n, H * V) * gate) @ w[pre + "o"].to(F64).T


def gated(h, w, pre, act):
    return (act(h @ w[pre + "gate"].to(F64).T) * (h @ w[pre + "up"].to(F64).T)) @ w[pre + "down"].to(F64).T


def router_choice(h, w_router, top: int, scale: float):
    """(ids [n, top], weights [n, top]): the largest sigmoid scores, each over the sum of the chosen, times scale."""
    s = torch.sigmoid(h @ w_router.to(F64).T)
    val, ids = torch.topk(s, top, dim=-1)
    return ids, val / (val.sum(-1, keepdim=True) + 1e-20) * scale


def mixture(h, w, pre, f, routing=None, margins=None):
    r = f["router"]
    ids, wts = router_choice(h, w[pre + "router"], r["top"], r["scale"])
    if routing is not None:      # the choices of another run; the weights follow from this run's scores
        all_s = torch.sigmoid(h @ w[pre + "router"].to(F64).T)
        ids = torch.as_tensor(routing, dtype=torch.long)
        s = all_s.gather(1, ids)
        if margins is not None:  # how far below this run's last choice the other run's worst choice scores
            kth = torch.topk(all_s, r["top"], dim=-1).values[:, -1]
            margins.append(float((kth - s.min(-1).values).max()))
        wts = s / (s.sum(-1, keepdim=True) + 1e-20) * r["scale"]
    y = torch.zeros_like(h)
    for e in range(r["experts"]):
        rows, col = (ids == e).nonzero(as_tuple=True)
        if rows.numel():
            y[rows] += wts[rows, col, None] * gated(h[rows], w, f"{pre}e{e}.", silu)
    if f.get("shared"):
        y = y + gated(h, w, pre + "shared.", silu)
    return y, ids


def forward(cfg: dict, w: dict, tokens, routing=None, layers_out=None, margins=None):
    """float64 logits [n, vocab] of one sequence.  `routing`: per layer with a mixture, the expert ids to use
    (from a run whose close calls went the other way); `margins` then receives, per mixture, how far such a choice
    scores below this run's own.  `layers_out`: a list that receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    held = {}
    chosen = []
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        m, pre = layer["mixer"], f"l{i}."
        h = offset_norm(x, w[pre + "norm1"].to(F64), eps)
        if m.get("kv_from") is None:
            held[i] = keys_values(h, w, pre + "mix.", m, eps)
            kv = held[i]
        else:
            kv = held[m["kv_from"]]
        x = x + attention(h, w, pre + "mix.", m, eps, kv)
        f = layer.get("mlp")
        if f is not None:
            h = offset_norm(x, w[pre + "norm2"].to(F64), eps)
            if f["kind"] == "dense":
                x = x + gated(h, w, pre + "mlp.", gelu_tanh)
            else:
                y, ids = mixture(h, w, pre + "mlp.", f, None if routing is None else routing[len(chosen)], margins)
                chosen.append(ids)
                x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    x = offset_norm(x, w["final.norm"].to(F64), eps)
    return (x @ w["embed"].to(F64).T) * cfg.get("logit_scale", 1.0)
