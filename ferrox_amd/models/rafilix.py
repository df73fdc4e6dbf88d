"""Rafilix as a list of parts.

Every layer is a block with a norm before and after each sublayer,
    x += norm1b(mixer(norm1(x)));  x += norm2b(ff(norm2(x)))
whose mixer is either chunked grouped-query attention (per-head q/k norms,
interleaved rotary positions with wavelength-dependent frequency scaling, key
and value heads of different sizes) or a gated delta rule with per-channel
decay, and whose feed-forward, where the layer has one, is a mixture of
ungated relu^2 experts with identity experts and a selection bias.  The head
is the embedding table.  Tensor names are the checkpoint's: `l<i>.norm1`,
`l<i>.mix.q`, `l<i>.mlp.e<j>.up`, `embed`, `final.norm`.
"""
from __future__ import annotations

from ..config.rafilix import RafilixConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _norm(width: int, eps: float, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": width, "eps": eps, "name": name})


def build_spec(cfg: RafilixConfig, tensor_names=None) -> ModelSpec:
    W, eps = cfg.width, cfg.eps
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "attention":
            position = PartSpec("none", {"head_dim": m.dim})
            if m.rot is not None:
                position = PartSpec("rope_scaled", {"head_dim": m.dim, "theta": m.rot.base, "rotary_dim": m.rot.dims,
                                                    "interleaved": True, "scaling": m.rot.scaling})
            mixer = PartSpec("paged_attention", {
                "hidden_size": W, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_dim": m.vdim,
                "bias": False, "scale": m.scale, "chunk": m.chunk, "position": position,
                "qk_norm": PartSpec("rmsnorm", {"size": m.dim, "eps": eps, "name": "norm"}),
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.", "k_norm": "k."},
            }, prefix="mix.")
        else:
            shapes = getattr(tensor_names, "shapes", {})
            ranks = {}
            for arg, tensor, given in (("decay_rank", f"l{i}.mix.a1", m.decay_rank), ("gate_rank", f"l{i}.mix.g1", m.gate_rank)):
                shape = shapes.get(tensor)
                ranks[arg] = int(shape[0]) if shape else (given or max(16, m.dim // 4))
            mixer = PartSpec("channel_delta", {
                "hidden_size": W, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "key_dim": m.dim, "v_dim": m.vdim,
                "conv_taps": m.conv, "norm_eps": eps, **ranks,
            }, prefix="mix.")
        parts = {"norm1": _norm(W, eps, "norm1"), "mixer": mixer, "norm1b": _norm(W, eps, "norm1b")}
        if layer.mlp is not None:
            f = layer.mlp
            parts.update({
                "norm2": _norm(W, eps, "norm2"),
                "ffn": PartSpec("routed_experts", {
                    "hidden_size": W, "n_experts": f.experts, "n_identity": f.identity, "top_k": f.top,
                    "expert_intermediate_size": f.ff, "activation": "relu2", "gating": "softmax", "renorm": False,
                    "selection_bias": True,
                }, prefix="mlp."),
                "norm2b": _norm(W, eps, "norm2b"),
            })
        layers.append(LayerSpec("sandwich", f"l{i}.", parts))
    return ModelSpec(
        hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "embed"}),
        layers=layers,
        schedule=[ScheduleEntry(i) for i in range(len(layers))],
        final_norm=PartSpec("rmsnorm", {"size": W, "eps": eps, "name": "final.norm"}),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": "embed"}),
        max_positions=cfg.max_positions,
        eos_token_id=cfg.eos_token_id,
    )
