"""Norms: RMSNorm (reference: somi_inference/models/qwen2.py:46-62), a norm without statistics, layer norm."""

from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import VECTOR, Init, WeightSpec
from .base import Fetch, Norm, Runtime


class RMSNorm(Norm):
    """y = w * x * rsqrt(mean(x^2) + eps), no mean subtraction, no bias
    (qwen2.py:55-62).  Square, mean, rsqrt and scale are float32."""
    graph_safe = True
    fusable = True        # weight * (h / sqrt(mean(h^2) + eps)): what a projection can apply while it loads h

    def __init__(self, prefix: str, hidden_size: int, eps: float,
                 init: tuple[float, float] = (1.0, 0.1), tensor: str = "weight") -> None:
        """``tensor``: what the checkpoint calls the scale under the part's prefix."""
        super().__init__(prefix)
        self.tensor = str(tensor)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self._init = Init(*init)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.name(self.tensor), (self.hidden_size,), VECTOR, self._init)]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.weight = fetch(self.name(self.tensor))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, self.runtime.dtype)

    def add_forward(self, h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, self.runtime.dtype, delta=delta)

    def add_normed(self, h: torch.Tensor, y: torch.Tensor, copy_dtype: torch.dtype | None = None) -> torch.Tensor | None:
        y = y if y.dtype == torch.float32 else y.to(torch.float32)
        return ops.normed_add(h, y, self.weight, self.eps, 1.0, copy_dtype)


class DynamicTanh(Norm):
    """y = tanh(alpha * x) * w + b: a norm that computes no mean and no variance.  ``alpha`` is one stored number,
    ``w`` and ``b`` vectors; the tensors are ``<tensor>``, ``<tensor>.alpha`` and ``<tensor>.b`` under the prefix.
    float32 throughout, rounded once to the compute dtype."""
    graph_safe = True
    fusable = False       # not a row scale: no projection applies it while it loads its rows

    def __init__(self, prefix: str, hidden_size: int, tensor: str = "weight", alpha_init: float = 0.5) -> None:
        super().__init__(prefix)
        self.tensor = str(tensor)
        self.hidden_size = int(hidden_size)
        self.alpha_init = float(alpha_init)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        name = self.name(self.tensor)
        return [WeightSpec(name, (self.hidden_size,), VECTOR, Init(1.0, 0.1)),
                WeightSpec(f"{name}.b", (self.hidden_size,), VECTOR, Init(0.0, 0.1)),
                WeightSpec(f"{name}.alpha", (), VECTOR, Init(self.alpha_init, 0.0))]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        name = self.name(self.tensor)
        self.weight, self.bias = fetch(name), fetch(f"{name}.b")
        self.alpha = fetch(f"{name}.alpha").reshape(1).contiguous()      # stays on the device: the kernel reads it

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return ops.dynamic_tanh(h, self.weight, self.bias, self.alpha, self.runtime.dtype)


class LayerNorm(Norm):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * w + b, the variance being the mean of the squared deviations; the
    tensors are ``<tensor>`` and ``<tensor>.b`` under the prefix.  Statistics and the result are float32, rounded once
    to the compute dtype."""
    graph_safe = True
    fusable = False       # the mean makes it more than a row scale: no projection applies it while it loads its rows

    def __init__(self, prefix: str, hidden_size: int, eps: float, tensor: str = "weight") -> None:
        super().__init__(prefix)
        self.tensor = str(tensor)
        self.hidden_size, self.eps = int(hidden_size), float(eps)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        name = self.name(self.tensor)
        return [WeightSpec(name, (self.hidden_size,), VECTOR, Init(1.0, 0.1)),
                WeightSpec(f"{name}.b", (self.hidden_size,), VECTOR, Init(0.0, 0.1))]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        name = self.name(self.tensor)
        self.weight, self.bias = fetch(name), fetch(f"{name}.b")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return ops.layernorm(h, self.weight, self.bias, self.eps, self.runtime.dtype)

    def add_normed(self, h: torch.Tensor, y: torch.Tensor, copy_dtype: torch.dtype | None = None) -> torch.Tensor | None:
        return ops.layernorm_add(h, y, self.weight, self.bias, self.eps, copy_dtype)
