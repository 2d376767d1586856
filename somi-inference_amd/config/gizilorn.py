"""Typed configuration of the Gizilorn decoder: pre-norm layers around several residual streams (hyper-connections),
whose mixer is grouped-query attention with mixed heads (capped scores, a window, a softmax whose denominator
holds an extra 1, values turned by their position) or attention over a shared low-rank latent (a window, a sigmoid gate on
the heads' outputs, optionally reading the latent an earlier layer kept), with a dense feed-forward whose activation
has two learned numbers; the embedded rows are RMS-normed.

config.json keys: ``architecture`` ("Gizilorn"), ``vocab``, ``width``, ``norm.eps``, ``streams`` (absent, with no
``hc*`` tensors in the checkpoint: the plain residual sum) and ``layers``, a list with one object per layer: ``type`` ("attention" or
"latent_attention"), ``mixer`` with that mixer's sizes, and ``mlp`` (``{"kind": "dense", "ff": ...}`` or null).

``mixer`` of attention: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``softcap`` (absent: scores are not
capped), ``rot`` (``base``, ``dims``), ``mask.size`` (absent: every earlier token is seen).  ``mixer`` of latent
attention: ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``kv_rank``, ``scale``, ``rot`` (``base``, ``dims``),
``mask.size`` and optionally ``kv_from``, the layer whose kept latent it reads.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import ConfigError, KeyReader, ModelConfig


def _window(keys: KeyReader) -> int | None:
    mask = keys.sub("mask")
    return mask.optional_integer("size", minimum=1) if mask is not None else None


@dataclass(frozen=True)
class GizilornAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    softcap: float | None = None
    window: int | None = None

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "GizilornAttention":
        rot = keys.sub("rot")
        if rot is None:
            raise ConfigError(f"{where}: required key 'rot' is missing")
        dim = keys.integer("dim", minimum=1)
        heads = keys.integer("heads", minimum=1)
        out = cls(heads=heads, kv_heads=keys.integer("kv_heads", heads, minimum=1), dim=dim,
                  vdim=keys.integer("vdim", dim, minimum=1), scale=keys.number("scale", dim ** -0.5),
                  rot_base=rot.number("base", positive=True), rot_dims=rot.integer("dims", dim, minimum=0),
                  softcap=keys.number("softcap", positive=True) if keys.has("softcap") else None, window=_window(keys))
        out.check(where)
        return out

    def check(self, where: str) -> None:
        if self.heads % self.kv_heads:
            raise ConfigError(f"{where}: 'heads' ({self.heads}) must be a multiple of 'kv_heads' ({self.kv_heads})")
        if self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ConfigError(f"{where}: 'rot.dims' ({self.rot_dims}) must be even and at most 'dim' ({self.dim})")
        if self.vdim % 2:
            raise ConfigError(f"{where}: 'vdim' ({self.vdim}) must be even: the values turn in pairs")

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class GizilornLatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: int | None = None
    kv_from: int | None = None

    @classmethod
    def read(cls, keys: KeyReader, where: str) -> "GizilornLatentAttention":
        rot = keys.sub("rot")
        rot_dim = keys.integer("rot_dim", minimum=0)
        if rot is None and rot_dim > 0:
            raise ConfigError(f"{where}: required key 'rot' is missing")
        dim = keys.integer("dim", minimum=1)
        out = cls(heads=keys.integer("heads", minimum=1), dim=dim, rot_dim=rot_dim, vdim=keys.integer("vdim", minimum=1),
                  kv_rank=keys.integer("kv_rank", minimum=1), scale=keys.number("scale", (dim + rot_dim) ** -0.5),
                  rot_base=rot.number("base", positive=True) if rot is not None else 10000.0,
                  rot_dims=rot.integer("dims", rot_dim, minimum=0) if rot is not None else 0,
                  window=_window(keys), kv_from=keys.optional_integer("kv_from", minimum=0))
        out.check(where)
        return out

    def check(self, where: str) -> None:
        if self.rot_dims % 2 or self.rot_dims > self.rot_dim:
            raise ConfigError(f"{where}: 'rot.dims' ({self.rot_dims}) must be even and at most 'rot_dim' ({self.rot_dim})")

    def kept(self) -> tuple:
        """What two layers must share to share a kept latent."""
        return (self.kv_rank, self.rot_dim, self.rot_base, self.rot_dims)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                               "kv_rank": self.kv_rank, "scale": self.scale,
                               "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class GizilornDense:
    ff: int

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


LAYER_TYPES = ("attention", "latent_attention")


@dataclass(frozen=True)
class GizilornLayer:
    type: str
    mixer: "GizilornAttention | GizilornLatentAttention"
    mlp: "GizilornDense | None" = None

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class GizilornConfig(ModelConfig):
    architecture: ClassVar[str] = "Gizilorn"

    vocab: int
    width: int
    layers: tuple[GizilornLayer, ...]
    norm_eps: float = 1e-6
    streams: int | None = None       # None: one stream and the plain residual sum (no hyper-connection tensors)

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: 'vocab' and 'width' must be >= 1 and 'layers' must not be empty")
        if self.streams is not None and self.streams < 1:
            raise ConfigError(f"config.json: 'streams' must be >= 1, got {self.streams}")
        object.__setattr__(self, "layers", tuple(self.layers))
        for index, layer in enumerate(self.layers):
            where = f"config.json:layers[{index}]"
            if layer.type not in LAYER_TYPES:
                raise ConfigError(f"{where}: 'type' must be one of {LAYER_TYPES}, got {layer.type!r}")
            if (layer.type == "latent_attention") != isinstance(layer.mixer, GizilornLatentAttention):
                raise ConfigError(f"{where}: the mixer's sizes do not belong to a layer of type {layer.type!r}")
            layer.mixer.check(where + ":mixer")
            if layer.type != "latent_attention" or layer.mixer.kv_from is None:
                continue
            source = layer.mixer.kv_from
            if not 0 <= source < index or self.layers[source].type != "latent_attention":
                raise ConfigError(f"{where}:mixer: 'kv_from' ({source}) must name an earlier latent-attention layer")
            lender = self.layers[source].mixer
            if lender.kv_from is not None:
                raise ConfigError(f"{where}:mixer: layer {source} keeps no latent of its own to read ('kv_from' of 'kv_from')")
            if lender.kept() != layer.mixer.kept():
                raise ConfigError(f"{where}:mixer: 'kv_rank', 'rot_dim' and 'rot' must equal those of layer {source}, whose latent it reads")

    def fitted_to(self, shapes: dict[str, tuple[int, ...]]) -> "GizilornConfig":
        """Whether the layers have connection tensors is what the checkpoint says where config.json says one stream or
        nothing: one stream without such tensors is the plain residual sum, and tensors of one stream without the key
        are connections of one stream."""
        import dataclasses
        has = any(".hc1." in name for name in shapes)
        if self.streams == 1 and not has:
            return dataclasses.replace(self, streams=None)
        if self.streams is None and has:
            count = next(shape[0] for name, shape in shapes.items() if name.endswith(".hc1.in"))
            return dataclasses.replace(self, streams=int(count))
        return self

    @classmethod
    def from_dict(cls, data: dict[str, Any]) -> "GizilornConfig":
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
            sizes = (GizilornLatentAttention.read(mixer, where + ":mixer") if kind == "latent_attention"
                     else GizilornAttention.read(mixer, where + ":mixer"))
            mlp = layer.sub("mlp")
            dense = None
            if mlp is not None:
                if mlp.string("kind", "dense") != "dense":
                    raise ConfigError(f"{where}:mlp: 'kind' must be 'dense', got {mlp.string('kind')!r}")
                dense = GizilornDense(ff=mlp.integer("ff", minimum=1))
            layers.append(GizilornLayer(type=kind, mixer=sizes, mlp=dense))
        norm = keys.sub("norm")
        return cls(vocab=keys.integer("vocab", minimum=1), width=keys.integer("width", minimum=1), layers=tuple(layers),
                   norm_eps=norm.number("eps", 1e-6, positive=True) if norm else 1e-6,
                   streams=keys.optional_integer("streams", minimum=1))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "layers": [layer.to_dict() for layer in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        return out
