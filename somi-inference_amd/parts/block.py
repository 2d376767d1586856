"""Arrangements of a layer's parts around the residual stream."""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import VECTOR, Init, WeightSpec
from .base import Block, BorrowedCache, CompositeSpec, LayerCache, Part, PartSpec
from .registry import build_part
from .residual import ResidualStream


class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += feed_forward(norm2(h)).

    Reference: somi_inference/models/qwen2.py:325-339.  ``names`` gives the
    sub-prefixes of the four parts under the layer's prefix (an empty one puts a
    part's tensors directly under the layer's).  A layer without a feed-forward
    (``feed_forward=None``) has the first sublayer only.
    """
    graph_safe = True

    DEFAULT_NAMES = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                     "ffn_norm": "post_attention_layernorm", "feed_forward": "mlp"}

    def __init__(self, prefix: str, mixer: PartSpec, feed_forward: PartSpec | None, mixer_norm: PartSpec,
                 ffn_norm: PartSpec | None = None, names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        sub = dict(self.DEFAULT_NAMES)
        sub.update(names or {})
        self.mixer_norm = build_part("norm", mixer_norm, prefix=self.name(sub["mixer_norm"]))
        self.mixer = build_part("mixer", mixer, prefix=self.name(sub["mixer"]))
        self.ffn_norm = self.feed_forward = None
        if feed_forward is not None:
            if ffn_norm is None:
                raise ValueError(f"{prefix}: a feed-forward needs its norm")
            self.ffn_norm = build_part("norm", ffn_norm, prefix=self.name(sub["ffn_norm"]))
            self.feed_forward = build_part("feed_forward", feed_forward, prefix=self.name(sub["feed_forward"]))

    def parts(self) -> list[Part]:
        parts = [self.mixer_norm, self.mixer]
        return parts + [self.ffn_norm, self.feed_forward] if self.feed_forward is not None else parts

    def forward(self, stream: ResidualStream, step, cache: LayerCache | None) -> None:
        x = stream.normed(self.mixer_norm, lazy=getattr(self.mixer, "takes_normed_rows", False))
        stream.add(self.mixer.forward(x, step, cache))
        if self.feed_forward is None:
            return
        x = stream.normed(self.ffn_norm, lazy=getattr(self.feed_forward, "takes_normed_rows", False))
        stream.add(self.feed_forward.forward(x, step))


class ParallelBlock(Block):
    """One norm, and mixer and feed-forward side by side: with x' = norm(h), ``h += mult * (mixer(x') + ff(x'))``;
    then, if the layer has one, a per-layer token input adds to h from the token itself (``token_input``, a part of
    the category of that name with ``add_to(h, x, step, mult)``).  The sum is float32; a layer without a feed-forward
    adds the mixer alone.  ``names``: the sub-prefixes of the norm, the mixer, the feed-forward and the token input."""

    DEFAULT_NAMES = {"norm": "input_layernorm", "mixer": "self_attn", "feed_forward": "mlp", "token_input": "token_input"}

    def __init__(self, prefix: str, mixer: PartSpec, feed_forward: PartSpec | None, norm: PartSpec,
                 residual_mult: float = 1.0, token_input: PartSpec | None = None,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        sub = dict(self.DEFAULT_NAMES)
        sub.update(names or {})
        self.residual_mult = float(residual_mult)
        self.norm = build_part("norm", norm, prefix=self.name(sub["norm"]))
        self.mixer = build_part("mixer", mixer, prefix=self.name(sub["mixer"]))
        self.feed_forward = (build_part("feed_forward", feed_forward, prefix=self.name(sub["feed_forward"]))
                             if feed_forward is not None else None)
        self.token_input = (build_part("token_input", token_input, prefix=self.name(sub["token_input"]))
                            if token_input is not None else None)
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts())

    def parts(self) -> list[Part]:
        return [part for part in (self.norm, self.mixer, self.feed_forward, self.token_input) if part is not None]

    def forward(self, stream: ResidualStream, step, cache: LayerCache | None) -> None:
        x = stream.normed(self.norm)
        mixed = _float32_rows(self.mixer.forward(x, step, cache))
        fed = _float32_rows(self.feed_forward.forward(x, step)) if self.feed_forward is not None else None
        h = stream.settle()
        with stage("residual add"):
            copy = ops.scaled_add(h, mixed, fed, self.residual_mult,
                                  self.runtime.dtype if self.token_input is not None else None)
        if self.token_input is not None:
            self.token_input.add_to(h, copy, step, self.residual_mult)


class OutputNormBlock(Block):
    """The norm sits on a sublayer's output, and the sublayers read the stream itself:

        h += norm1(mixer(f(h)));   h += norm2(feed_forward(h));   then, if the layer has one, the per-layer token input,

    where f is the identity or an input filter (``input_conv``, a part of that category with ``forward(h, step, cache)``
    and ``state_spec()``: what the mixer reads is then a function of the stream's rows and of the request's kept
    state).  The norms are any that offer ``add_normed``.  A layer without a feed-forward has the first sublayer only.
    ``names``: the sub-prefixes of the two norms, the mixer, the feed-forward, the input filter and the token input."""

    DEFAULT_NAMES = {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "feed_forward": "mlp",
                     "input_conv": "input_conv", "token_input": "token_input"}

    def __init__(self, prefix: str, mixer: PartSpec, feed_forward: PartSpec | None, mixer_norm: PartSpec,
                 ffn_norm: PartSpec | None = None, input_conv: PartSpec | None = None, token_input: PartSpec | None = None,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        sub = dict(self.DEFAULT_NAMES)
        sub.update(names or {})
        self.mixer_norm = build_part("norm", mixer_norm, prefix=self.name(sub["mixer_norm"]))
        self.mixer = build_part("mixer", mixer, prefix=self.name(sub["mixer"]))
        self.ffn_norm = self.feed_forward = None
        if feed_forward is not None:
            if ffn_norm is None:
                raise ValueError(f"{prefix}: a feed-forward needs its norm")
            self.ffn_norm = build_part("norm", ffn_norm, prefix=self.name(sub["ffn_norm"]))
            self.feed_forward = build_part("feed_forward", feed_forward, prefix=self.name(sub["feed_forward"]))
        self.input_conv = (build_part("input_conv", input_conv, prefix=self.name(sub["input_conv"]))
                           if input_conv is not None else None)
        self.token_input = (build_part("token_input", token_input, prefix=self.name(sub["token_input"]))
                            if token_input is not None else None)
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts())

    def parts(self) -> list[Part]:
        return [part for part in (self.input_conv, self.mixer, self.mixer_norm, self.feed_forward, self.ffn_norm,
                                  self.token_input) if part is not None]

    def cache_spec(self, borrow_from: int | None = None):
        """Without an input filter: the mixer's need.  With one: a composite of the filter's state (``input``) and the
        mixer's need (``mixer``), the latter borrowed from the earlier run if the mixer reads that run's cache."""
        if self.input_conv is None:
            return super().cache_spec(borrow_from)
        parts = [("input", self.input_conv.state_spec())]
        if borrow_from is not None:
            parts.append(("mixer", BorrowedCache(borrow_from, ("mixer",))))
        elif self.mixer.cache_spec() is not None:
            parts.append(("mixer", self.mixer.cache_spec()))
        return CompositeSpec(tuple(parts))

    def forward(self, stream: ResidualStream, step, cache: LayerCache | None) -> None:
        h = stream.settle()
        dtype = self.runtime.dtype
        mixer_cache = cache
        if self.input_conv is not None:
            with stage("input convolution"):
                x = self.input_conv.forward(h, step, cache.children.get("input") if cache is not None else None)
            mixer_cache = cache.children.get("mixer") if cache is not None else None
        else:
            x = h if dtype == torch.float32 else h.to(dtype)
        mixed = _rows(self.mixer.forward(x, step, mixer_cache))
        last = self.feed_forward is None and self.token_input is None
        with stage("output norm, residual add"):
            x = self.mixer_norm.add_normed(h, mixed, None if last else dtype)
        if self.feed_forward is not None:
            fed = _rows(self.feed_forward.forward(x, step))
            with stage("output norm, residual add"):
                x = self.ffn_norm.add_normed(h, fed, dtype if self.token_input is not None else None)
        if self.token_input is not None:
            self.token_input.add_to(h, x, step, 1.0)


class HyperConnectionBlock(Block):
    """A pre-norm layer around ``streams`` residual streams instead of one.  For sublayer q (the mixer, then the
    feed-forward) with its three tensors ``in`` [S], ``mix`` [S, S] (from, to) and ``out`` [S]:

        u = sum_s in[s] x_s;     y = sublayer(norm_q(u));     x_t <- sum_s mix[s, t] x_s + out[t] y    (all t at once).

    The streams are all equal to the embedded rows when the first such layer meets them, and what the model's final
    norm reads is their sum.  ``connections`` False: no such tensors; one stream with in = mix = out = 1, the plain
    residual sum.  Streams, their sums and the norms are float32; a sublayer's last product is computed into float32
    rows, and one kernel does a sublayer's write and the next sublayer's read and norm.  A layer without a feed-forward
    has the first sublayer only.  ``names``: the sub-prefixes of the two norms, the mixer, the feed-forward and the two
    sets of connection tensors."""

    DEFAULT_NAMES = {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "feed_forward": "mlp",
                     "mixer_streams": "hc1", "ffn_streams": "hc2"}

    def __init__(self, prefix: str, mixer: PartSpec, feed_forward: PartSpec | None, mixer_norm: PartSpec,
                 ffn_norm: PartSpec | None = None, streams: int = 1, connections: bool = True,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        sub = dict(self.DEFAULT_NAMES)
        sub.update(names or {})
        self.sub = sub
        self.streams, self.connections = int(streams), bool(connections)
        if not 1 <= self.streams <= ops.HC_MAX_STREAMS or (not self.connections and self.streams != 1):
            raise ValueError(f"{prefix}: 1 to {ops.HC_MAX_STREAMS} streams (one without connection tensors), got {streams}")
        self.mixer_norm = build_part("norm", mixer_norm, prefix=self.name(sub["mixer_norm"]))
        self.mixer = build_part("mixer", mixer, prefix=self.name(sub["mixer"]))
        self.ffn_norm = self.feed_forward = None
        if feed_forward is not None:
            if ffn_norm is None:
                raise ValueError(f"{prefix}: a feed-forward needs its norm")
            self.ffn_norm = build_part("norm", ffn_norm, prefix=self.name(sub["ffn_norm"]))
            self.feed_forward = build_part("feed_forward", feed_forward, prefix=self.name(sub["feed_forward"]))
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and not (getattr(norm, "fusable", False) and hasattr(norm, "eps")):
                raise ValueError(f"{prefix}: the kernel that reads the streams norms them by their root mean square")
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts())

    def parts(self) -> list[Part]:
        return [part for part in (self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward) if part is not None]

    def _connection_names(self) -> list[str]:
        subs = [self.sub["mixer_streams"]] + ([self.sub["ffn_streams"]] if self.feed_forward is not None else [])
        return [self.name(s) for s in subs] if self.connections else []

    def weight_specs(self):
        specs = super().weight_specs()
        s = self.streams
        for base in self._connection_names():
            specs += [WeightSpec(f"{base}.in", (s,), VECTOR, Init(1.0 / s, 0.1)),
                      WeightSpec(f"{base}.out", (s,), VECTOR, Init(1.0, 0.1)),
                      WeightSpec(f"{base}.mix", (s, s), VECTOR, Init(1.0 / s, 0.1))]
        return specs

    def load(self, fetch, runtime) -> None:
        super().load(fetch, runtime)
        self.links = []
        for base in self._connection_names():
            self.links.append((fetch(f"{base}.in"), fetch(f"{base}.mix").contiguous(), fetch(f"{base}.out")))
        if not self.connections:
            one = torch.ones((1,), dtype=torch.float32, device=runtime.device)
            self.links = [(one, one.view(1, 1), one)] * 2

    def forward(self, stream: ResidualStream, step, cache: LayerCache | None) -> None:
        lanes = stream.fan_out(self.streams)
        dtype = self.runtime.dtype
        first, second = self.links[0], (self.links[1] if self.feed_forward is not None else None)
        with stage("residual add, norm"):
            x = ops.hc_step(lanes, read=True, in_weights=first[0], norm_weight=self.mixer_norm.weight,
                            eps=self.mixer_norm.eps, out_dtype=dtype)
        y = _float32_product(self.mixer.forward(x, step, cache))
        if second is None:
            with stage("residual add, norm"):
                ops.hc_step(lanes, y=y, mix=first[1], out_weights=first[2])
            return
        with stage("residual add, norm"):
            x = ops.hc_step(lanes, y=y, mix=first[1], out_weights=first[2], read=True, in_weights=second[0],
                            norm_weight=self.ffn_norm.weight, eps=self.ffn_norm.eps, out_dtype=dtype)
        y = _float32_product(self.feed_forward.forward(x, step))
        with stage("residual add, norm"):
            ops.hc_step(lanes, y=y, mix=second[1], out_weights=second[2])


def _float32_product(y):
    """A sublayer's output for the float32 streams: a promised product is computed into float32 rows, so that its
    sums are not rounded before they are added; rows that exist stay as they are."""
    if hasattr(y, "projection"):
        with stage(y.projection.label):
            return linear_kernels.linear(y.x, y.projection.weight, y.projection.bias, torch.float32)
    return y


def _rows(y):
    """A sublayer's output as rows (a promised product is computed)."""
    return y.materialize() if hasattr(y, "materialize") else y


def _float32_rows(y):
    """A sublayer's output as float32 rows (a promised product is computed, 16-bit rows are widened)."""
    if hasattr(y, "materialize"):
        y = y.materialize()
    return y if y.dtype == torch.float32 else y.to(torch.float32)
