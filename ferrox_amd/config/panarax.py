"""Typed configuration of the Panarax design, read from config.json.

    {"architecture": "Panarax", "vocab": V, "width": W, "max_positions": P, "norm": {"eps": e}, "canon": {"taps": n},
     "layers": [{"type": "rglru" | "lightning" | "parallel", "mixer": {...},
                 "mlp": {"kind": "dense", "ff": F} | {"kind": "moe", "expert": {"ff": F, "limit": L},
                         "router": {"experts": E, "top": k}} | null}, ...]}

Every layer entry carries its own sizes, so layers of different kinds and sizes may follow each other in any order.
`rglru` mixer: width, blocks, conv.  `lightning` mixer: heads, dim, vdim, decay (one number a head).
`parallel` mixer: left {heads, kv_heads, dim, vdim, scale, q_temp {coef, every}} (softmax attention),
right {heads, dim, vdim, gate_cap} (matrix memory).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .. import limits
from .base import ConfigError, ConfigReader
from .rafilix import _section

MIXER_TYPES = ("rglru", "lightning", "parallel")


@dataclass(frozen=True)
class RglruConfig:
    width: int
    blocks: int
    conv: int


@dataclass(frozen=True)
class LightningConfig:
    heads: int
    dim: int
    vdim: int
    decay: tuple


@dataclass(frozen=True)
class SoftmaxAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp: tuple | None         # (coef, every) or None


@dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class SideBySideConfig:
    left: SoftmaxAttentionConfig
    right: MatrixMemoryConfig


@dataclass(frozen=True)
class DenseConfig:
    ff: int


@dataclass(frozen=True)
class MoeConfig:
    experts: int
    top: int
    ff: int
    limit: float


@dataclass(frozen=True)
class PanaraxLayer:
    type: str
    mixer: object
    mlp: object        # DenseConfig, MoeConfig or None


def _rglru(r: ConfigReader) -> RglruConfig:
    width, blocks, conv = r.integer("width", minimum=1), r.integer("blocks", minimum=1), r.integer("conv", minimum=1)
    if width % blocks:
        raise ConfigError(f"{r.where}: width {width} is not cut into {blocks} equal blocks")
    if conv > 16:
        raise ConfigError(f"{r.where}: conv {conv} is more than the convolution kernel's 16 taps")
    return RglruConfig(width, blocks, conv)


def _recurrent_dim(r: ConfigReader, dim: int) -> int:
    if dim > 256:
        raise ConfigError(f"{r.where}: dim {dim} is more than the recurrence kernel's 256 key channels a head")
    return dim


def _lightning(r: ConfigReader) -> LightningConfig:
    heads = r.integer("heads", minimum=1)
    decay = r.raw.get("decay")
    if not isinstance(decay, list) or len(decay) != heads or any(isinstance(d, bool) or not isinstance(d, (int, float))
                                                                 or not 0.0 < d <= 1.0 for d in decay):
        raise ConfigError(f"{r.where}: key 'decay' must list {heads} numbers in (0, 1], one a head, got {decay!r}")
    return LightningConfig(heads, _recurrent_dim(r, r.integer("dim", minimum=1)), r.integer("vdim", minimum=1),
                           tuple(float(d) for d in decay))


def _parallel(r: ConfigReader) -> SideBySideConfig:
    lr, rr = _section(r, "left"), _section(r, "right")
    heads, kv = lr.integer("heads", minimum=1), lr.integer("kv_heads", minimum=1)
    if heads % kv:
        raise ConfigError(f"{lr.where}: heads {heads} is not a multiple of kv_heads {kv}")
    dim, vdim = lr.integer("dim", minimum=1), lr.integer("vdim", minimum=1)
    if max(dim, vdim) > limits.HEAD_DIM_MAX:
        raise ConfigError(f"{lr.where}: head sizes {dim} / {vdim} are more than the attention kernels' {limits.HEAD_DIM_MAX}")
    temp = None
    tr = _section(lr, "q_temp", required=False)
    if tr is not None:
        temp = (tr.number("coef"), tr.integer("every", minimum=1))
    left = SoftmaxAttentionConfig(heads, kv, dim, vdim, lr.number("scale", positive=True), temp)
    right = MatrixMemoryConfig(rr.integer("heads", minimum=1), _recurrent_dim(rr, rr.integer("dim", minimum=1)),
                               rr.integer("vdim", minimum=1), rr.number("gate_cap", positive=True))
    return SideBySideConfig(left, right)


def _mlp(r: ConfigReader | None):
    if r is None:
        return None
    kind = r.string("kind", "dense")
    if kind == "dense":
        return DenseConfig(r.integer("ff", minimum=1))
    if kind != "moe":
        raise ConfigError(f"{r.where}: feed-forward kind '{kind}' is not one this design has (dense, moe)")
    er, rr = _section(r, "expert"), _section(r, "router")
    experts, top = rr.integer("experts", minimum=1), rr.integer("top", minimum=1)
    if top > experts:
        raise ConfigError(f"{rr.where}: top {top} of {experts} experts")
    if experts > limits.MOE_MAX_EXPERTS or top > limits.MOE_MAX_TOP_K:
        raise ConfigError(f"{rr.where}: the routing kernels take up to {limits.MOE_MAX_EXPERTS} experts and "
                          f"{limits.MOE_MAX_TOP_K} per token")
    return MoeConfig(experts, top, er.integer("ff", minimum=1), er.number("limit", positive=True))


@dataclass(frozen=True)
class PanaraxConfig:
    vocab: int
    width: int
    eps: float
    canon_taps: int
    max_positions: int
    layers: tuple
    raw: dict = field(default_factory=dict, compare=False, repr=False)
    eos_token_id: int | tuple | None = None
    defaulted_keys: tuple = field(default=(), compare=False)

    architecture = "Panarax"
    model_type = "panarax"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "PanaraxConfig":
        r = ConfigReader(raw, where)
        vocab, width = r.integer("vocab", minimum=1), r.integer("width", minimum=1)
        eps = _section(r, "norm").number("eps", positive=True)
        cr = _section(r, "canon", required=False)
        taps = cr.integer("taps", minimum=1) if cr is not None else 0
        if taps > 16:
            raise ConfigError(f"{where}: canon.taps {taps} is more than the convolution kernel's 16 taps")
        # the learned position vectors are a table of this many rows; no sequence is longer
        max_positions = r.integer("max_positions", minimum=1)
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
            mixer = {"rglru": _rglru, "lightning": _lightning, "parallel": _parallel}[kind](mr)
            layers.append(PanaraxLayer(kind, mixer, _mlp(_section(lr, "mlp", required=False))))
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = tuple(int(e) for e in eos)
        return cls(vocab, width, eps, taps, max_positions, tuple(layers), copy.deepcopy(raw), eos, tuple(r.defaulted))

    def to_dict(self) -> dict:
        out = copy.deepcopy(self.raw)
        out.setdefault("architecture", self.architecture)
        return out
