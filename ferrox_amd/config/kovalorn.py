"""Typed configuration of the Kovalorn design, read from config.json.

    {"architecture": "Kovalorn", "vocab": V, "width": W, "norm": {"eps": e}, "logit_scale": s,
     "layers": [{"type": "attention", "mixer": {...}, "mlp": {...} | null}, ...]}

Every layer entry carries its own sizes, so layers of different sizes may follow each other in any order.
`attention` mixer: heads, kv_heads, dim (a query and key head), vdim (a value head), scale (of the scores),
mask {size, keep_first} (a sliding window of `size` positions beside the first `keep_first` of the sequence;
without `mask` a query sees every earlier key), optional kv_from (the layer whose keys and values this one reads
instead of making its own).
`mlp`: kind "dense" with ff, or kind "moe" with expert {ff}, router {experts, top, scale} and optionally
shared {ff}.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .. import limits
from .base import ConfigError, ConfigReader
from .rafilix import _section

MIXER_TYPES = ("attention",)
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class GatedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None          # positions of the sliding window, None: every earlier key
    keep_first: int             # first positions of a sequence that stay visible beside the window
    kv_from: int | None         # the layer whose keys and values are read, None: its own


@dataclass(frozen=True)
class DenseConfig:
    ff: int


@dataclass(frozen=True)
class SigmoidMoeConfig:
    ff: int
    experts: int
    top: int
    scale: float
    shared_ff: int              # 0: no shared expert


@dataclass(frozen=True)
class KovalornLayer:
    type: str
    mixer: GatedAttentionConfig
    mlp: object                 # DenseConfig, SigmoidMoeConfig or None


def _attention(r: ConfigReader, index: int) -> GatedAttentionConfig:
    heads, kv = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
    if heads % kv:
        raise ConfigError(f"{r.where}: heads {heads} is not a multiple of kv_heads {kv}")
    dim, vdim = r.integer("dim", minimum=1), r.integer("vdim", minimum=1)
    for name, v in (("dim", dim), ("vdim", vdim)):
        if v > limits.HEAD_DIM_MAX:
            raise ConfigError(f"{r.where}: {name} {v} is more than the attention kernels' {limits.HEAD_DIM_MAX}")
    window, keep = None, 0
    mr = _section(r, "mask", required=False)
    if mr is not None:
        window = mr.integer("size", minimum=1)
        keep = mr.integer("keep_first", 0, minimum=0)
    kv_from = r.optional_integer("kv_from", minimum=0)
    if kv_from is not None and kv_from >= index:
        raise ConfigError(f"{r.where}: kv_from {kv_from} must name an earlier layer than this one ({index})")
    return GatedAttentionConfig(heads, kv, dim, vdim, r.number("scale", positive=True), window, keep, kv_from)


def _mlp(r: ConfigReader):
    kind = r.string("kind")
    if kind not in MLP_KINDS:
        raise ConfigError(f"{r.where}: feed-forward kind '{kind}' is not one of {', '.join(MLP_KINDS)}")
    if kind == "dense":
        return DenseConfig(r.integer("ff", minimum=1))
    ff = _section(r, "expert").integer("ff", minimum=1)
    rr = _section(r, "router")
    experts, top = rr.integer("experts", minimum=1), rr.integer("top", minimum=1)
    if top > experts:
        raise ConfigError(f"{rr.where}: top {top} of {experts} experts")
    if experts > limits.MOE_MAX_EXPERTS or top > limits.MOE_MAX_TOP_K:
        raise ConfigError(f"{rr.where}: the routing kernels take up to {limits.MOE_MAX_EXPERTS} experts "
                          f"and {limits.MOE_MAX_TOP_K} per token")
    sr = _section(r, "shared", required=False)
    return SigmoidMoeConfig(ff, experts, top, rr.number("scale", 1.0, positive=True),
                            sr.integer("ff", minimum=1) if sr is not None else 0)


@dataclass(frozen=True)
class KovalornConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: tuple
    raw: dict = field(default_factory=dict, compare=False, repr=False)
    eos_token_id: int | tuple | None = None
    max_positions: int = 32768            # the design names no limit; the optional key `max_positions` does (it sizes the default cache)
    defaulted_keys: tuple = field(default=(), compare=False)

    architecture = "Kovalorn"
    model_type = "kovalorn"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "KovalornConfig":
        r = ConfigReader(raw, where)
        vocab, width = r.integer("vocab", minimum=1), r.integer("width", minimum=1)
        eps = _section(r, "norm").number("eps", positive=True)
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError(f"{where}: key 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(entries):
            lr = ConfigReader(entry, f"{where}: layers[{i}]")
            kind = lr.string("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{lr.where}: type '{kind}' is not one of {', '.join(MIXER_TYPES)}")
            mixer = _attention(_section(lr, "mixer"), i)
            if mixer.kv_from is not None:
                owner = layers[mixer.kv_from].mixer
                if owner.kv_from is not None:
                    raise ConfigError(f"{lr.where}: kv_from {mixer.kv_from} names a layer that has no keys and values of its own")
                if (owner.kv_heads, owner.dim, owner.vdim) != (mixer.kv_heads, mixer.dim, mixer.vdim):
                    raise ConfigError(f"{lr.where}: kv_from {mixer.kv_from} names a layer with other key and value heads")
            fr = _section(lr, "mlp", required=False)
            layers.append(KovalornLayer(kind, mixer, _mlp(fr) if fr is not None else None))
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = tuple(int(e) for e in eos)
        return cls(vocab, width, eps, r.number("logit_scale", 1.0, positive=True), tuple(layers), copy.deepcopy(raw), eos,
                   r.integer("max_positions", 32768, minimum=1), tuple(r.defaulted))

    def to_dict(self) -> dict:
        out = copy.deepcopy(self.raw)
        out.setdefault("architecture", self.architecture)
        return out
