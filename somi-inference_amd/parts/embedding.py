"""Token embedding and LM head.

Reference: somi_inference/models/qwen2.py:360,382 (lookup) and
somi_inference/models/qwen2_adapter.py:60-62 (logits = h . E^T with the
embedding matrix, no bias).  The reference always ties the head; here a head
has a matrix of its own unless it is told to use the embedding's.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..weights.spec import MATRIX, VECTOR, Init, WeightSpec
from .base import Fetch, Part, Runtime


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, prefix: str, vocab_size: int, hidden_size: int, tensor: str = "weight",
                 scale: float | None = None, norm_tensor: str | None = None, norm_eps: float = 1e-6) -> None:
        """``tensor``: what the checkpoint calls the table under the part's prefix.  ``scale``: a factor on the
        embedded rows (a head tied to the table multiplies by the table itself, without it).  ``norm_tensor``: the
        embedded rows are RMS-normed, ``x / sqrt(mean(x^2) + norm_eps) * w``, with the weight of that name (float32 in,
        float32 out)."""
        super().__init__(prefix)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tensor = str(tensor)
        self.scale = float(scale) if scale is not None and float(scale) != 1.0 else None
        self.norm_tensor, self.norm_eps = (str(norm_tensor) if norm_tensor else None), float(norm_eps)
        self.weight: torch.Tensor | None = None
        self.norm_weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        specs = [WeightSpec(self.name(self.tensor), (self.vocab_size, self.hidden_size), MATRIX)]
        if self.norm_tensor:
            specs.append(WeightSpec(self.name(self.norm_tensor), (self.hidden_size,), VECTOR, Init(1.0, 0.1)))
        return specs

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.weight = fetch(self.name(self.tensor))
        if self.norm_tensor:
            self.norm_weight = fetch(self.name(self.norm_tensor))

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        """[N] int32 -> [N, H] float32 (the residual stream starts in float32)."""
        h = ops.embedding(self.weight, token_ids)
        if self.scale is not None:
            ops.scale_(h, self.scale)
        if self.norm_weight is not None:
            h = ops.hc_step(h.unsqueeze(0), read=True, norm_weight=self.norm_weight, eps=self.norm_eps)
        return h


class LMHead(Part):
    """logits = x . W^T in float32, for the rows that were asked for only, times ``scale`` if there is one; with
    ``softcap`` c the logits are then bounded smoothly, c * tanh(logits / c)."""
    graph_safe = True

    def __init__(self, prefix: str, vocab_size: int, hidden_size: int, tied: bool = False,
                 softcap: float | None = None, tensor: str = "weight", scale: float | None = None) -> None:
        super().__init__(prefix)
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.softcap = float(softcap) if softcap else None
        if self.softcap is not None and not self.softcap > 0.0:
            raise ValueError(f"{prefix}: a soft cap must be > 0, got {softcap}")
        self.tensor = str(tensor)
        self.scale = float(scale) if scale is not None and float(scale) != 1.0 else None
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        if self.tied:
            return []
        return [WeightSpec(self.name(self.tensor), (self.vocab_size, self.hidden_size), MATRIX)]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        if not self.tied:
            self.weight = fetch(self.name(self.tensor))

    def tie(self, embedding: TokenEmbedding) -> None:
        self.weight = embedding.weight

    def flops(self, tokens: int, attended: int = 0) -> float:
        """Of the logits of ``tokens`` rows."""
        return 2.0 * tokens * self.vocab_size * self.hidden_size

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = linear_kernels.linear(x, self.weight, None, torch.float32)
        if self.scale is not None:
            ops.scale_(logits, self.scale)
        if self.softcap is not None:
            ops.softcap_(logits, self.softcap)
        return logits
