"""Typed configuration of the Fokinex design, read from config.json.

    {"architecture": "Fokinex", "vocab": V, "width": W, "norm": {"eps": e}, "embedding": {"scale": s},
     "layers": [{"type": "latent_attention" | "parallel", "mixer": {...}, "mlp": {"kind": "dense", "ff": F} | null}, ...]}

Every layer entry carries its own sizes, so layers of different kinds and sizes may follow each other in any order.
`latent_attention` mixer: heads, dim (unrotated query/key dimensions a head), rot_dim (rotated ones), vdim, q_rank,
kv_rank, scale, optional rot {base, dims, scaling {factor, original, fast, slow}}, optional mask {size}, optional
kv_from (the layer whose latents this one reads instead of making its own).
`parallel` mixer: left {heads, kv_heads, dim, vdim, scale, softcap, mask {size}} (attention), right {heads, kv_heads,
dim, vdim, conv} (gated delta rule), left_scale, right_scale.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .. import limits
from .base import ConfigError, ConfigReader
from .rafilix import _section

MIXER_TYPES = ("latent_attention", "parallel")


@dataclass(frozen=True)
class RampedRotaryConfig:
    dims: int
    base: float
    scaling: tuple | None       # (factor, original, fast, slow) or None


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: RampedRotaryConfig | None
    window: int | None
    kv_from: int | None


@dataclass(frozen=True)
class CappedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None
    window: int | None


@dataclass(frozen=True)
class HeadDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: CappedAttentionConfig
    right: HeadDeltaConfig
    left_scale: float
    right_scale: float
    kv_from = None


@dataclass(frozen=True)
class DenseConfig:
    ff: int


@dataclass(frozen=True)
class FokinexLayer:
    type: str
    mixer: object
    mlp: DenseConfig | None


def _window(r: ConfigReader):
    mr = _section(r, "mask", required=False)
    return mr.integer("size", minimum=1) if mr is not None else None


def _latent(r: ConfigReader, index: int) -> LatentAttentionConfig:
    heads, dim = r.integer("heads", minimum=1), r.integer("dim", minimum=1)
    rot_dim, vdim = r.integer("rot_dim", minimum=0), r.integer("vdim", minimum=1)
    q_rank, kv_rank = r.integer("q_rank", minimum=1), r.integer("kv_rank", minimum=1)
    if kv_rank + rot_dim > limits.HEAD_DIM_MAX_ANY:
        raise ConfigError(f"{r.where}: kv_rank {kv_rank} + rot_dim {rot_dim} is more than the attention kernels' {limits.HEAD_DIM_MAX_ANY}")
    rot = None
    rr = _section(r, "rot", required=False)
    if rr is not None:
        dims = rr.integer("dims", minimum=0)
        if dims % 2 or dims > rot_dim:
            raise ConfigError(f"{rr.where}: dims {dims} must be even and at most rot_dim {rot_dim}")
        scaling = None
        sr = _section(rr, "scaling", required=False)
        if sr is not None:
            scaling = (sr.number("factor", positive=True), sr.number("original", positive=True),
                       sr.number("fast", positive=True), sr.number("slow", positive=True))
        base = rr.number("base", positive=True)
        if scaling is not None and base == 1.0:
            raise ConfigError(f"{rr.where}: a base of 1 has no wavelengths to scale")
        rot = RampedRotaryConfig(dims, base, scaling) if dims else None
    kv_from = r.optional_integer("kv_from", minimum=0)
    if kv_from is not None and kv_from >= index:
        raise ConfigError(f"{r.where}: kv_from {kv_from} must name an earlier layer than this one ({index})")
    return LatentAttentionConfig(heads, dim, rot_dim, vdim, q_rank, kv_rank, r.number("scale", positive=True), rot,
                                 _window(r), kv_from)


def _heads(r: ConfigReader):
    heads, kv = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
    if heads % kv:
        raise ConfigError(f"{r.where}: heads {heads} is not a multiple of kv_heads {kv}")
    return heads, kv, r.integer("dim", minimum=1), r.integer("vdim", minimum=1)


def _parallel(r: ConfigReader) -> ParallelMixerConfig:
    lr, rr = _section(r, "left"), _section(r, "right")
    heads, kv, dim, vdim = _heads(lr)
    if vdim != dim:
        raise ConfigError(f"{lr.where}: the keys are the values, so vdim {vdim} must equal dim {dim}")
    if dim > limits.HEAD_DIM_MAX:
        raise ConfigError(f"{lr.where}: dim {dim} is more than the attention kernels' {limits.HEAD_DIM_MAX}")
    cap = lr.raw.get("softcap")
    left = CappedAttentionConfig(heads, kv, dim, vdim, lr.number("scale", positive=True),
                                 lr.number("softcap", positive=True) if cap is not None else None, _window(lr))
    rh, rkv, rdim, rvdim = _heads(rr)
    if rdim > 256:
        raise ConfigError(f"{rr.where}: dim {rdim} is more than the recurrence kernel's 256 key channels a head")
    conv = rr.integer("conv", minimum=1)
    if conv > 16:
        raise ConfigError(f"{rr.where}: conv {conv} is more than the convolution kernel's 16 taps")
    return ParallelMixerConfig(left, HeadDeltaConfig(rh, rkv, rdim, rvdim, conv), r.number("left_scale", 1.0), r.number("right_scale", 1.0))


@dataclass(frozen=True)
class FokinexConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    layers: tuple
    raw: dict = field(default_factory=dict, compare=False, repr=False)
    eos_token_id: int | tuple | None = None
    max_positions: int = 32768            # the design names no limit; the optional key `max_positions` does (it sizes the default cache)
    defaulted_keys: tuple = field(default=(), compare=False)

    architecture = "Fokinex"
    model_type = "fokinex"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "FokinexConfig":
        r = ConfigReader(raw, where)
        vocab, width = r.integer("vocab", minimum=1), r.integer("width", minimum=1)
        eps = _section(r, "norm").number("eps", positive=True)
        er = _section(r, "embedding", required=False)
        emb_scale = er.number("scale", 1.0) if er is not None else 1.0
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
            if kind == "latent_attention":
                mixer = _latent(mr, i)
                if mixer.kv_from is not None:
                    owner = layers[mixer.kv_from]
                    if owner.type != "latent_attention" or owner.mixer.kv_from is not None:
                        raise ConfigError(f"{lr.where}: kv_from {mixer.kv_from} names a layer that has no latents of its own")
                    if (owner.mixer.kv_rank, owner.mixer.rot_dim, owner.mixer.rot) != (mixer.kv_rank, mixer.rot_dim, mixer.rot):
                        raise ConfigError(f"{lr.where}: kv_from {mixer.kv_from} names a layer with another latent size or rotation")
            else:
                mixer = _parallel(mr)
            fr = _section(lr, "mlp", required=False)
            mlp = None
            if fr is not None:
                fkind = fr.string("kind", "dense")
                if fkind != "dense":
                    raise ConfigError(f"{fr.where}: feed-forward kind '{fkind}' is not one this design has (dense)")
                mlp = DenseConfig(fr.integer("ff", minimum=1))
            layers.append(FokinexLayer(kind, mixer, mlp))
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = tuple(int(e) for e in eos)
        return cls(vocab, width, eps, emb_scale, tuple(layers), copy.deepcopy(raw), eos,
                   r.integer("max_positions", 32768, minimum=1), tuple(r.defaulted))

    def to_dict(self) -> dict:
        out = copy.deepcopy(self.raw)
        out.setdefault("architecture", self.architecture)
        return out
