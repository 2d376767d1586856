"""Typed configuration of the Metitar decoder: layers whose mixer is attention over a shared low-rank latent or a
recurrence with a bounded forget gate (HGRN2), each read through a short causal convolution of the residual stream,
with a dense feed-forward of normed powers or a mixture of experts, sublayer outputs layer-normed before they are
added, and a per-layer token input.

config.json keys: ``architecture`` ("Metitar"), ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``,
``logit_scale``, ``canon.taps`` (absent: no input convolution), ``token_side.dim`` (absent: no per-layer token input)
and ``layers``, a list with one object per layer: ``type`` ("latent_attention" or "hgrn2"), ``mixer`` with that
mixer's sizes, and ``mlp`` (``{"kind": "dense", "ff": ...}``, ``{"kind": "moe", ...}`` or null).

``mixer`` of latent attention: ``heads``, ``dim`` (unrotated query/key channels a head), ``rot_dim`` (rotated ones),
``vdim``, ``kv_rank``, ``q_rank``, ``scale``, ``rot`` (``base``, ``dims``, optional ``scaling`` with ``factor``,
``original``, ``fast``, ``slow``) and optionally ``kv_from``, the layer whose kept latent it reads.  ``mixer`` of
HGRN2: ``heads``, ``dim``, ``vdim``.  ``mlp`` of kind moe: ``router`` (``experts``, ``top``), ``expert`` (``ff``) and
optionally ``shared`` (``ff``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import ConfigError, KeyReader, ModelConfig


@dataclass(frozen=True)
class RampedScaling:
    """Frequency rescaling by a linear ramp over the channel index between the channels that make ``fast`` and
    ``slow`` turns over ``original`` positions."""
    factor: float
    original: int
    fast: float
    slow: float

    @classmethod
    def read(cls, keys: KeyReader) -> "RampedScaling":
        return cls(factor=keys.number("factor", positive=True), original=keys.integer("original", minimum=1),
                   fast=keys.number("fast", positive=True), slow=keys.number("slow", positive=True))

    def to_dict(self) -> dict[str, Any]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class MetitarLatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: RampedScaling | None = None
    kv_from: int | None = None

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "MetitarLatentAttention":
        rot = keys.sub("rot")
        rot_dim = keys.integer("rot_dim", minimum=0)
        if rot is None and rot_dim > 0:
            raise ConfigError(f"{where}: required key 'rot' is missing")
        scaling = rot.sub("scaling") if rot is not None else None
        dim = keys.integer("dim", minimum=1)
        out = cls(heads=keys.integer("heads", minimum=1), dim=dim, rot_dim=rot_dim, vdim=keys.integer("vdim", minimum=1),
                  kv_rank=keys.integer("kv_rank", minimum=1), q_rank=keys.integer("q_rank", minimum=1),
                  scale=keys.number("scale", (dim + rot_dim) ** -0.5),
                  rot_base=rot.number("base", positive=True) if rot is not None else 10000.0,
                  rot_dims=rot.integer("dims", rot_dim, minimum=0) if rot is not None else 0,
                  rot_scaling=RampedScaling.read(scaling) if scaling is not None else None,
                  kv_from=keys.optional_integer("kv_from", minimum=0))
        out.check(where)
        return out

    def check(self, where: str) -> None:
        if self.rot_dims % 2 or self.rot_dims > self.rot_dim:
            raise ConfigError(f"{where}: 'rot.dims' ({self.rot_dims}) must be even and at most 'rot_dim' ({self.rot_dim})")

    def rotation(self) -> tuple:
        """What two layers must share to share a kept latent."""
        return (self.kv_rank, self.rot_dim, self.rot_base, self.rot_dims, self.rot_scaling)

    def to_dict(self) -> dict[str, Any]:
        rot: dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_dict()
        out: dict[str, Any] = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                               "kv_rank": self.kv_rank, "q_rank": self.q_rank, "scale": self.scale, "rot": rot}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class MetitarHGRN2:
    heads: int
    dim: int
    vdim: int

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "MetitarHGRN2":
        return cls(heads=keys.integer("heads", minimum=1), dim=keys.integer("dim", minimum=1),
                   vdim=keys.integer("vdim", minimum=1))

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}


@dataclass(frozen=True)
class MetitarDense:
    ff: int

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class MetitarExperts:
    experts: int
    top: int
    ff: int
    shared_ff: int | None = None

    def check(self, where: str) -> None:
        if self.top > self.experts:
            raise ConfigError(f"{where}: 'top' ({self.top}) is more than the {self.experts} experts")

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff},
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


def read_mlp(keys: KeyReader, where: str) -> "MetitarDense | MetitarExperts":
    kind = keys.string("kind")
    if kind == "dense":
        return MetitarDense(ff=keys.integer("ff", minimum=1))
    if kind != "moe":
        raise ConfigError(f"{where}: 'kind' must be 'dense' or 'moe', got {kind!r}")
    router, expert, shared = keys.sub("router"), keys.sub("expert"), keys.sub("shared")
    if router is None or expert is None:
        raise ConfigError(f"{where}: a mixture of experts needs 'router' and 'expert'")
    out = MetitarExperts(experts=router.integer("experts", minimum=1), top=router.integer("top", minimum=1),
                         ff=expert.integer("ff", minimum=1),
                         shared_ff=shared.integer("ff", minimum=1) if shared else None)
    out.check(where)
    return out


LAYER_TYPES = ("latent_attention", "hgrn2")


@dataclass(frozen=True)
class MetitarLayer:
    type: str
    mixer: "MetitarLatentAttention | MetitarHGRN2"
    mlp: "MetitarDense | MetitarExperts | None" = None

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class MetitarConfig(ModelConfig):
    architecture: ClassVar[str] = "Metitar"

    vocab: int
    width: int
    layers: tuple[MetitarLayer, ...]
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    token_side_dim: int | None = None
    canon_taps: int | None = None

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: 'vocab' and 'width' must be >= 1 and 'layers' must not be empty")
        object.__setattr__(self, "layers", tuple(self.layers))
        for index, layer in enumerate(self.layers):
            where = f"config.json:layers[{index}]"
            if layer.type not in LAYER_TYPES:
                raise ConfigError(f"{where}: 'type' must be one of {LAYER_TYPES}, got {layer.type!r}")
            if (layer.type == "latent_attention") != isinstance(layer.mixer, MetitarLatentAttention):
                raise ConfigError(f"{where}: the mixer's sizes do not belong to a layer of type {layer.type!r}")
            if isinstance(layer.mlp, MetitarExperts):
                layer.mlp.check(where + ":mlp")
            if layer.type != "latent_attention":
                continue
            layer.mixer.check(where + ":mixer")
            source = layer.mixer.kv_from
            if source is None:
                continue
            if not 0 <= source < index or self.layers[source].type != "latent_attention":
                raise ConfigError(f"{where}:mixer: 'kv_from' ({source}) must name an earlier latent-attention layer")
            lender = self.layers[source].mixer
            if lender.kv_from is not None:
                raise ConfigError(f"{where}:mixer: layer {source} keeps no latent of its own to read ('kv_from' of 'kv_from')")
            if lender.rotation() != layer.mixer.rotation():
                raise ConfigError(f"{where}:mixer: 'kv_rank', 'rot_dim' and 'rot' must equal those of layer {source}, whose latent it reads")

    @classmethod
    def from_dict(cls, data: dict[str, Any]) -> "MetitarConfig":
        keys = KeyReader(data)
        raw_layers = keys.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for index, raw in enumerate(raw_layers):
            where = f"config.json:layers[{index}]"
            layer = KeyReader(raw, where)
            kind = layer.string("type")
            mixer = layer.sub("mixer")
            if kind not in LAYER_TYPES:
                raise ConfigError(f"{where}: 'type' must be one of {LAYER_TYPES}, got {kind!r}")
            if mixer is None:
                raise ConfigError(f"{where}: required key 'mixer' is missing")
            sizes = (MetitarLatentAttention.read(mixer, where + ":mixer") if kind == "latent_attention"
                     else MetitarHGRN2.read(mixer, where + ":mixer"))
            mlp = layer.sub("mlp")
            layers.append(MetitarLayer(type=kind, mixer=sizes, mlp=None if mlp is None else read_mlp(mlp, where + ":mlp")))
        norm, embedding, side, canon = keys.sub("norm"), keys.sub("embedding"), keys.sub("token_side"), keys.sub("canon")
        return cls(vocab=keys.integer("vocab", minimum=1), width=keys.integer("width", minimum=1), layers=tuple(layers),
                   norm_eps=norm.number("eps", 1e-5, positive=True) if norm else 1e-5,
                   embedding_scale=embedding.number("scale", 1.0) if embedding else 1.0,
                   logit_scale=keys.number("logit_scale", 1.0),
                   token_side_dim=side.integer("dim", minimum=1) if side else None,
                   canon_taps=canon.integer("taps", minimum=1) if canon else None)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                               "logit_scale": self.logit_scale, "layers": [layer.to_dict() for layer in self.layers]}
        if self.token_side_dim is not None:
            out["token_side"] = {"dim": self.token_side_dim}
        if self.canon_taps is not None:
            out["canon"] = {"taps": self.canon_taps}
        return out
