"""HGRN2: linear attention whose forget gate also decides what is written.

With q = silu(W_q h) (``heads x key_dim``), v = W_v h (``heads x value_dim``) and, per head and key channel, a forget
gate bounded below by a learned vector,

    f_t = lower + (1 - lower) * sigmoid(W_f h_t + b)
    S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T                  (per head; S: key_dim x value_dim, from zero)
    o_t = S_t^T q_t

(no key and no scale: what the gate does not keep, it writes).  Each head's o is RMS-normed over its value channels
with one weight shared by the heads, the heads are concatenated and projected by W_o.  The state lives in float32 in
the request's state slot and is carried from step to step; the gate, the recurrence and the norm are float32 in both
engines.  The recurrence is the gated-linear-attention kernel with alpha = f, k = 1 - f and a query scale of one.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, Init, WeightSpec
from .base import Fetch, FixedStateSpec, LayerCache, Mixer, Runtime
from .linear import Projection


class HGRN2(Mixer):
    graph_safe = True

    ROLES = {"q": "q", "f": "f", "f_bias": "f.b", "lower": "lower", "v": "v", "norm": "norm", "o": "o"}

    def __init__(self, prefix: str, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, eps: float,
                 names: dict[str, str] | None = None, suffix: str = "weight") -> None:
        """``names``: role -> the checkpoint's name under the prefix (``f_bias``, ``lower`` and ``norm`` are whole names,
        the matrices are followed by ``suffix`` unless it is empty)."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix = str(suffix)
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim, self.eps = int(key_dim), int(value_dim), float(eps)

    def _matrix(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def weight_specs(self) -> list[WeightSpec]:
        qk, vv, h = self.num_heads * self.key_dim, self.num_heads * self.value_dim, self.hidden_size
        return [
            WeightSpec(self._matrix("q"), (qk, h), MATRIX),
            WeightSpec(self._matrix("f"), (qk, h), MATRIX),
            WeightSpec(self.name(self.names["f_bias"]), (qk,), VECTOR, Init(1.0, 1.0)),
            WeightSpec(self.name(self.names["lower"]), (qk,), VECTOR, Init(0.5, 0.1)),
            WeightSpec(self._matrix("v"), (vv, h), MATRIX),
            WeightSpec(self.name(self.names["norm"]), (self.value_dim,), VECTOR, Init(1.0, 0.1)),
            WeightSpec(self._matrix("o"), (h, vv), MATRIX),
        ]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.inputs = Projection.stacked([fetch(self._matrix(role)) for role in ("q", "f", "v")], label="q/f/v")
        self.out = Projection(fetch(self._matrix("o")), label="o")
        self.gate_bias, self.lower = fetch(self.name(self.names["f_bias"])), fetch(self.name(self.names["lower"]))
        self.norm_weight = fetch(self.name(self.names["norm"]))

    def flops(self, tokens: int, attended: int) -> float:
        recurrence = 4.0 * self.num_heads * self.key_dim * self.value_dim * tokens
        return self.inputs.flops(tokens) + self.out.flops(tokens) + recurrence

    def cache_spec(self) -> FixedStateSpec:
        return FixedStateSpec((self.num_heads, self.key_dim, self.value_dim), torch.float32)

    def forward(self, x, step, cache: LayerCache | None):
        if cache is None or cache.state is None:
            raise ValueError(f"{self.prefix}: the recurrence needs a state slot per request")
        if hasattr(x, "materialize"):
            x = x.materialize()
        qk = self.num_heads * self.key_dim
        with stage(self.inputs.label):
            rows = linear_kernels.linear(x, self.inputs.weight, None, torch.float32)     # [N, q | f's sums | v], float32
        with stage("forget gates"):
            keep = ops.bounded_forget_(rows, qk, self.gate_bias, self.lower)            # rows: [silu(q) | 1 - f | v]
        with stage("recurrence"):
            o = ops.gla_scan(rows[:, :qk], rows[:, qk:2 * qk], rows[:, 2 * qk:], keep, step.entry_start, step.state_slots,
                             cache.state, 1.0)
        with stage("norm"):
            y = ops.gla_norm_gate(o, self.norm_weight, None, self.eps, out_dtype=self.runtime.dtype)
        with stage(self.out.label):
            return linear_kernels.linear(y, self.out.weight, None, torch.float32)
