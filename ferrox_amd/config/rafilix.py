"""Typed configuration of the Rafilix design, read from config.json.

The file names no global sizes beyond `vocab`, `width` and `norm.eps`: every
layer entry of `layers` carries its own mixer and feed-forward sizes, so layers
of different kinds and sizes may follow each other in any order.

    {"architecture": "Rafilix", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "attention" | "channel_delta", "mixer": {...}, "mlp": {...} | null}, ...]}

`attention` mixer: heads, kv_heads, dim, vdim, scale, optional rot {base, dims,
scaling {factor, low, high, original}}, optional mask {size}.
`channel_delta` mixer: heads, kv_heads, dim, vdim, conv (taps of the short convolution); the inner sizes of its
two low-rank projections are those of the checkpoint's tensors (`decay_rank` / `gate_rank` may name them for a
model made without a checkpoint; without both, a quarter of dim, at least 16).
`mlp`: kind "moe", expert {ff}, router {experts, identity, top}.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .. import limits
from .base import ConfigError, ConfigReader

MIXER_TYPES = ("attention", "channel_delta")


def _section(r: ConfigReader, key: str, required: bool = True):
    v = r.raw.get(key)
    if v is None:
        if required:
            raise ConfigError(f"{r.where}: required key '{key}' is missing")
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: key '{key}' must be an object, got {v!r}")
    return ConfigReader(v, f"{r.where}: {key}")


@dataclass(frozen=True)
class RotaryConfig:
    dims: int
    base: float
    scaling: tuple | None       # (factor, low, high, original) or None


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryConfig | None
    chunk: int | None           # positions per chunk of the chunked mask, None: plain causal


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int | None = None     # inner sizes of the two low-rank projections: the checkpoint's tensors give
    gate_rank: int | None = None      # them; these optional keys serve a model that is made without a checkpoint


@dataclass(frozen=True)
class MoeConfig:
    ff: int
    experts: int
    identity: int
    top: int


@dataclass(frozen=True)
class RafilixLayer:
    type: str
    mixer: object
    mlp: MoeConfig | None


def _heads(r: ConfigReader):
    heads, kv = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
    if heads % kv:
        raise ConfigError(f"{r.where}: heads {heads} is not a multiple of kv_heads {kv}")
    return heads, kv, r.integer("dim", minimum=1), r.integer("vdim", minimum=1)


def _attention(r: ConfigReader) -> AttentionConfig:
    heads, kv, dim, vdim = _heads(r)
    for name, v in (("dim", dim), ("vdim", vdim)):
        if v > limits.HEAD_DIM_MAX:
            raise ConfigError(f"{r.where}: {name} {v} is more than the attention kernels' {limits.HEAD_DIM_MAX}")
    rot = None
    rr = _section(r, "rot", required=False)
    if rr is not None:
        dims = rr.integer("dims", minimum=0)
        if dims % 2 or dims > dim:
            raise ConfigError(f"{rr.where}: dims {dims} must be even and at most dim {dim}")
        scaling = None
        sr = _section(rr, "scaling", required=False)
        if sr is not None:
            scaling = (sr.number("factor", positive=True), sr.number("low", positive=True),
                       sr.number("high", positive=True), sr.number("original", positive=True))
            if not scaling[2] > scaling[1]:
                raise ConfigError(f"{sr.where}: high {scaling[2]} must be above low {scaling[1]}")
        rot = RotaryConfig(dims, rr.number("base", positive=True), scaling) if dims else None
    mr = _section(r, "mask", required=False)
    chunk = mr.integer("size", minimum=1) if mr is not None else None
    return AttentionConfig(heads, kv, dim, vdim, r.number("scale", positive=True), rot, chunk)


def _channel_delta(r: ConfigReader) -> ChannelDeltaConfig:
    heads, kv, dim, vdim = _heads(r)
    return ChannelDeltaConfig(heads, kv, dim, vdim, r.integer("conv", minimum=1),
                              r.optional_integer("decay_rank", minimum=1), r.optional_integer("gate_rank", minimum=1))


def _moe(r: ConfigReader) -> MoeConfig:
    kind = r.string("kind", "moe")
    if kind != "moe":
        raise ConfigError(f"{r.where}: feed-forward kind '{kind}' is not one this design has (moe)")
    ff = _section(r, "expert").integer("ff", minimum=1)
    rr = _section(r, "router")
    experts, identity = rr.integer("experts", minimum=0), rr.integer("identity", 0, minimum=0)
    top = rr.integer("top", minimum=1)
    if experts + identity < 1 or top > experts + identity:
        raise ConfigError(f"{rr.where}: top {top} of {experts} experts and {identity} identity experts")
    if experts + identity > limits.MOE_MAX_EXPERTS or top > limits.MOE_MAX_TOP_K:
        raise ConfigError(f"{rr.where}: the routing kernels take up to {limits.MOE_MAX_EXPERTS} router outputs "
                          f"and {limits.MOE_MAX_TOP_K} per token")
    return MoeConfig(ff, experts, identity, top)


@dataclass(frozen=True)
class RafilixConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    raw: dict = field(default_factory=dict, compare=False, repr=False)
    eos_token_id: int | tuple | None = None
    max_positions: int = 32768            # the design names no limit; the optional key `max_positions` does (it sizes the default cache)
    defaulted_keys: tuple = field(default=(), compare=False)

    architecture = "Rafilix"
    model_type = "rafilix"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "RafilixConfig":
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
            mr = _section(lr, "mixer")
            mixer = _attention(mr) if kind == "attention" else _channel_delta(mr)
            fr = _section(lr, "mlp", required=False)
            layers.append(RafilixLayer(kind, mixer, _moe(fr) if fr is not None else None))
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = tuple(int(e) for e in eos)
        return cls(vocab, width, eps, tuple(layers), copy.deepcopy(raw), eos,
                   r.integer("max_positions", 32768, minimum=1), tuple(r.defaulted))

    def to_dict(self) -> dict:
        out = copy.deepcopy(self.raw)
        out.setdefault("architecture", self.architecture)
        return out
