"""Arrangements of a layer's parts around the residual stream."""

from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.stages import stage
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


def _rows(y):
    """A sublayer's output as rows (a promised product is computed)."""
    return y.materialize() if hasattr(y, "materialize") else y


def _float32_rows(y):
    """A sublayer's output as float32 rows (a promised product is computed, 16-bit rows are widened)."""
    if hasattr(y, "materialize"):
        y = y.materialize()
    return y if y.dtype == torch.float32 else y.to(torch.float32)
