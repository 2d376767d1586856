"""A short causal convolution in front of a sublayer: what the sublayer reads is ``h + conv(h)``, with

    conv(h)[t, c] = sum_j taps[c, j] * h[t - (n - 1) + j, c],     j = 0 .. n - 1,   zeros before the sequence's start

per channel of the residual stream (no bias; the last tap weighs the current token).  A request's last ``n - 1`` input
rows are state of fixed size, kept in float32 in its state slot and carried from step to step, so a prompt cut into
portions, or decoded token by token, reads the same inputs as the whole prompt.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import VECTOR, Init, WeightSpec
from .base import Fetch, FixedStateSpec, LayerCache, Part, Runtime


class ShortConvInput(Part):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, taps: int) -> None:
        """The taps are the tensor named by the prefix itself, ``[hidden_size, taps]``."""
        super().__init__(prefix)
        if not 1 <= int(taps) <= ops.CONV_MAX_TAPS:
            raise ValueError(f"{prefix}: a convolution of {taps} taps; 1 to {ops.CONV_MAX_TAPS} are supported")
        self.hidden_size, self.taps = int(hidden_size), int(taps)

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.name(""), (self.hidden_size, self.taps), VECTOR, Init(0.0, 0.3))]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.weight = fetch(self.name(""))

    def state_spec(self) -> FixedStateSpec:
        return FixedStateSpec((max(self.taps - 1, 1), self.hidden_size), torch.float32)

    def forward(self, h: torch.Tensor, step, cache: LayerCache | None) -> torch.Tensor:
        """h: the float32 residual rows -> ``h + conv(h)`` in the compute dtype; the request's kept rows advance."""
        if cache is None or cache.state is None:
            raise ValueError(f"{self.prefix}: the input convolution needs a state slot per request")
        return ops.input_conv(h, self.weight, cache.state, step, self.runtime.dtype)
