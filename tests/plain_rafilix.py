"""Plain, slow Rafilix: whole sequences, no cache, one function per mechanism.

The oracle of the Rafilix tests.  It shares no code with the package under
test: weights are a dict of CPU torch tensors, every formula is written out,
loops stand where a loop is the clearest way to say it.  Arithmetic runs in
`dtype` (float64 by default).

The design, in this file's notation.  A layer is
    x <- x + N1b(mixer(N1(x))),   x <- x + N2b(ff(N2(x)))
with N(x) = x / sqrt(mean(x^2) + eps) * w.  The mixer is either chunked
grouped-query attention (`attention`) or a gated delta rule whose decay acts
per key channel (`channel_delta`); the feed-forward is a mixture of experts
whose last router outputs are identity experts.  The head is the embedding
table applied to the normed residual.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


# --------------------------------------------------------------------------
# rotation
# --------------------------------------------------------------------------
def rotary_frequencies(dims: int, base: float, scaling: dict | None) -> list:
    """f_i = base^(-2i/dims), i < dims/2, then the wavelength-dependent scaling: with L = 2 pi / f,
    f stays where L < original/high, becomes f/factor where L > original/low, and in between is
    (1 - s) f/factor + s f with s = (original/L - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < orig / high:
                pass
            elif wavelength > orig / low:
                f = f / factor
            else:
                s = (orig / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate_interleaved(vec: torch.Tensor, pos: int, freqs: list, angles: str = "float32") -> torch.Tensor:
    """Pairs (2i, 2i+1) of the first 2*len(freqs) entries of the last dimension turn by pos * f_i;
    the rest passes.  angles="float32": frequency and product rounded to float32, as a 32-bit
    implementation has them; "exact": float64."""
    import numpy as np
    out = vec.clone()
    for i, f in enumerate(freqs):
        a = float(np.float32(pos) * np.float32(f)) if angles == "float32" else pos * f
        c, s = math.cos(a), math.sin(a)
        u, v = vec[..., 2 * i], vec[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


# --------------------------------------------------------------------------
# mixers
# --------------------------------------------------------------------------
def chunk_visible(i: int, j: int, size: int | None) -> bool:
    """Query position i sees key position j."""
    return j <= i and (not size or i // size == j // size)


def attention(h: torch.Tensor, w: dict, m: dict, eps: float, first_pos: int = 0, angles: str = "float32") -> torch.Tensor:
    """h [T, width] -> [T, width].  `w`: the mixer's tensors by their short names (q, k, v, o, q.norm, k.norm)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(T, H, D)
    k = (h @ w["k"].T).view(T, G, D)
    v = (h @ w["v"].T).view(T, G, V)
    q = rms_norm(q, w["q.norm"], eps)
    k = rms_norm(k, w["k.norm"], eps)
    rot = m.get("rot")
    if rot and rot.get("dims", 0) > 0:
        freqs = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q = torch.stack([rotate_interleaved(q[t], first_pos + t, freqs, angles) for t in range(T)])
        k = torch.stack([rotate_interleaved(k[t], first_pos + t, freqs, angles) for t in range(T)])
    size = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            js = [j for j in range(T) if chunk_visible(first_pos + i, first_pos + j, size)]
            s = (k[js, g] @ q[i, hd]) * m["scale"]          # one score per visible key
            p = torch.softmax(s, dim=0)
            out[i, hd] = p @ v[js, g]
    return out.reshape(T, H * V) @ w["o"].T


def short_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y[t, c] = silu(sum_j taps[c, n-1-j] x[t-j, c]), zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(n):
            if t - j >= 0:
                y[t] += taps[:, n - 1 - j] * x[t - j]
    return y * torch.sigmoid(y)


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


def channel_delta(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel.  Per head, with S [dim, vdim] from zero:
        S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ w["q"].T, w["q.conv"]).view(T, G, D)
    k = short_conv_silu(h @ w["k"].T, w["k.conv"]).view(T, G, D)
    v = short_conv_silu(h @ w["v"].T, w["v.conv"]).view(T, H, V)
    q = unit(q) * D ** -0.5
    k = unit(k)
    beta = torch.sigmoid(h @ w["b"].T)                                           # [T, H]
    a = (h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]                               # [T, H*D]
    g = torch.exp(-torch.exp(w["A_log"]).view(1, H, 1) * torch.nn.functional.softplus(a).view(T, H, D))
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        kv = hd // (H // G)
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(T):
            S = g[t, hd].view(D, 1) * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, hd] = S.T @ q[t, kv]
    out = out / torch.sqrt((out * out).mean(dim=-1, keepdim=True) + eps) * w["norm"] * gate
    return out.reshape(T, H * V) @ w["o"].T


# --------------------------------------------------------------------------
# feed-forward
# --------------------------------------------------------------------------
def route(h: torch.Tensor, w: dict, r: dict, chosen=None):
    """ids [T, top] and weights [T, top]: softmax over all router outputs, the `top` largest of
    (score + correction) chosen, weighted by the score itself.  `chosen`: ids to take instead of the
    router's own choice (the weights are still this router's scores)."""
    s = torch.softmax(h @ w["router"].T, dim=-1)
    choice = s + w["correction"]
    ids = torch.topk(choice, r["top"], dim=-1).indices if chosen is None else torch.as_tensor(chosen, dtype=torch.int64)
    return ids, torch.gather(s, 1, ids)


def choice_margin(h: torch.Tensor, w: dict, r: dict, ids) -> float:
    """How far `ids` are from being the router's top choices: the largest amount by which a choice score that
    was left out exceeds one that was taken (0 or less: `ids` are a valid top set)."""
    s = torch.softmax(h @ w["router"].T, dim=-1) + w["correction"]
    ids = torch.as_tensor(ids, dtype=torch.int64)
    taken = torch.zeros_like(s, dtype=torch.bool).scatter_(1, ids, True)
    worst_taken = torch.where(taken, s, torch.full_like(s, float("inf"))).min(dim=-1).values
    best_left = torch.where(taken, torch.full_like(s, float("-inf")), s).max(dim=-1).values
    return float((best_left - worst_taken).max())


def moe(h: torch.Tensor, w: dict, f: dict, routing=None, margins=None) -> torch.Tensor:
    """`routing`: the ids [T, top] to use instead of the router's own choice (`margins`, a list, then receives how
    far they are from it).  Experts e < experts are down_e(relu(up_e h)^2); router outputs experts .. experts+identity-1 hand h through."""
    r = f["router"]
    E = r["experts"]
    ids, weights = route(h, w, r, routing)
    if routing is not None and margins is not None:
        margins.append(choice_margin(h, w, r, routing))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            if e >= E:
                y = h[t]
            else:
                z = torch.relu(w[f"e{e}.up"] @ h[t])
                y = w[f"e{e}.down"] @ (z * z)
            out[t] += weights[t, j] * y
    return out


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: dict, tokens: list, dtype=torch.float64, angles: str = "float32", layers_out=None,
            routing=None, margins=None):
    """Logits [T, vocab] of one sequence from position 0.  `layers_out`: a list that receives the residual
    stream after every layer.  `routing`: per layer with a feed-forward, in order, the ids [T, top] to use instead
    of the router's own choice; `margins` then receives how far each is from that choice."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    n_ff = 0
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, W[p + "norm1"], eps)
        mix = {"attention": attention, "channel_delta": channel_delta}[layer["type"]]
        kw = {"angles": angles} if layer["type"] == "attention" else {}
        x = x + rms_norm(mix(h, sub(W, p + "mix."), layer["mixer"], eps, **kw), W[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = rms_norm(x, W[p + "norm2"], eps)
            y = moe(h, sub(W, p + "mlp."), layer["mlp"], routing[n_ff] if routing else None, margins)
            n_ff += 1
            x = x + rms_norm(y, W[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["embed"].T
