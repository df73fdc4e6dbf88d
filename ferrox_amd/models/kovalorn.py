"""Kovalorn as a list of parts.

Every layer is a pre-norm block, x += mixer(norm1(x)); x += ff(norm2(x)), whose norms store their weight around
zero.  The mixer is grouped-query attention without positions in its scores: unit-RMS heads of q and k, a sliding
window beside the kept first keys of the sequence, a sink logit per head in the softmax's denominator, an output
gate; a layer may read an earlier layer's keys and values instead of making its own.  The feed-forward is a
tanh-gelu gated one or a mixture of silu-gated experts under sigmoid scores with a shared expert.  The head is the
embedding table, its logits times a constant.  Tensor names are the checkpoint's: `l<i>.norm1`, `l<i>.mix.q`,
`l<i>.mlp.e<j>.up`, `embed`, `final.norm`.
"""
from __future__ import annotations

from ..config.kovalorn import DenseConfig, KovalornConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

GATED_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def _norm(width: int, eps: float, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": width, "eps": eps, "name": name, "offset": 1.0})


def cache_retention(cfg: KovalornConfig) -> dict:
    """layer -> (window or None, kept first keys) that the pages of its cache must hold: a layer with keys of its
    own serves its own mask and those of the layers that read its cache, which may be wider."""
    need = {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        owner = i if m.kv_from is None else m.kv_from
        window, keep = need.get(owner, (0, 0))
        if m.window is None or window is None:
            need[owner] = (None, 0)
        else:
            need[owner] = (max(window, m.window), max(keep, m.keep_first))
    return {i: need[i if layer.mixer.kv_from is None else layer.mixer.kv_from] for i, layer in enumerate(cfg.layers)}


def build_spec(cfg: KovalornConfig, tensor_names=None) -> ModelSpec:
    W, eps = cfg.width, cfg.eps
    retain = cache_retention(cfg)
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        mixer = PartSpec("paged_attention", {
            "hidden_size": W, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_dim": m.vdim,
            "bias": False, "scale": m.scale, "window": m.window, "keep_first": m.keep_first,
            "position": PartSpec("none", {"head_dim": m.dim}),
            "qk_norm": PartSpec("rmsnorm", {"size": m.dim, "eps": eps, "weight": False}),
            "sink": True, "out_gate": True, "own_kv": m.kv_from is None, "retain": retain[i],
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "gate": "g"},
        }, prefix="mix.")
        parts = {"norm1": _norm(W, eps, "norm1"), "mixer": mixer}
        f = layer.mlp
        if f is not None:
            parts["norm2"] = _norm(W, eps, "norm2")
            if isinstance(f, DenseConfig):
                parts["ffn"] = PartSpec("gated_mlp", {"hidden_size": W, "intermediate_size": f.ff, "activation": "gelu_tanh",
                                                      "names": GATED_NAMES}, prefix="mlp.")
            else:
                parts["ffn"] = PartSpec("sparse_moe", {
                    "hidden_size": W, "n_experts": f.experts, "top_k": f.top, "expert_intermediate_size": f.ff,
                    "norm_topk_prob": True, "gating": "sigmoid", "shared_intermediate_size": f.shared_ff,
                    "shared_gate": False, "activation": "silu", "weight_scale": f.scale, "renorm_eps": 1e-20,
                    "names": {"router": "router", "gate": "e{}.gate", "up": "e{}.up", "down": "e{}.down",
                              "shared": "shared.", "shared_names": GATED_NAMES},
                }, prefix="mlp.")
        layers.append(LayerSpec("prenorm", f"l{i}.", parts))
    return ModelSpec(
        hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "embed"}),
        layers=layers,
        schedule=[ScheduleEntry(i, cache=layer.mixer.kv_from) for i, layer in enumerate(cfg.layers)],
        # (the logits' constant rides on the rows in front of the head, which is linear: no kernel of its own)
        final_norm=PartSpec("rmsnorm", {"size": W, "eps": eps, "name": "final.norm", "offset": 1.0, "gain": cfg.logit_scale}),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": "embed"}),
        max_positions=cfg.max_positions,
        eos_token_id=cfg.eos_token_id,
    )
