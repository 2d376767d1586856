"""Mixture of experts: a router picks a few small gated feed-forwards per token; a shared one may run for all.

Router: ``z = W_r x`` in float32 and scores ``s = softmax(z)`` over all experts, or ``s = sigmoid(z)`` expert by expert
(``scores``).  The experts come in ``groups`` equal runs of neighbours; a run scores as its best expert, and only
experts of the ``keep`` best runs can be chosen.  Of those the ``top`` with the largest s are taken, weighted by s over
the sum of the chosen scores (+ 1e-20) or by s as it is (``normalize``).  An expert is

    g = min(W_gate x, limit);  u = clamp(W_up x, -limit, limit);  y = W_down (g sigmoid(alpha g) (u + shift))

without biases (no ``limit``, alpha 1 and shift 0: the plain ``silu(W_gate x) * (W_up x)``); the output is the weighted
sum of the chosen experts' outputs or, with ``weight_on="input"``, the sum of the experts applied to ``w x`` (the
weight then scales the float32 sums of gate and up before the unit, which is not the same thing since the unit is not
linear); plus the shared expert's (the same form with sizes and a limit of its own).  The (token, expert) pairs are sorted by expert on the device, so that an
expert's rows are one block of the products' input; nothing of it is read by the host.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, WeightSpec
from .base import FeedForward, Fetch, Runtime
from .linear import Projection


class ClampedGLU:
    """The constants of the experts' gated unit."""

    def __init__(self, limit: float | None, alpha: float = 1.702, shift: float = 1.0) -> None:
        self.limit = float(limit) if limit is not None else float("inf")       # no limit: nothing is clamped
        self.alpha, self.shift = float(alpha), float(shift)
        if not self.limit > 0.0:
            raise ValueError(f"a clamp limit must be > 0, got {limit}")


class RoutedExperts(FeedForward):
    graph_safe = True

    ROLES = {"router": "router", "expert": "e", "shared": "shared", "gate": "gate", "up": "up", "down": "down"}

    SCORES = ("softmax", "sigmoid")
    WEIGHT_ON = ("output", "input")

    def __init__(self, prefix: str, hidden_size: int, num_experts: int, top: int, expert_size: int, limit: float | None,
                 groups: int = 1, keep_groups: int = 1, shared_size: int | None = None, shared_limit: float | None = None,
                 alpha: float = 1.702, shift: float = 1.0, names: dict[str, str] | None = None, suffix: str = "weight",
                 scores: str = "softmax", normalize: bool = True, weight_on: str = "output") -> None:
        """``names``: ``router``, the experts' stem (``e`` gives ``e0``, ``e1``, ...), ``shared``, and the three matrices
        of an expert; ``suffix`` follows a matrix's name (empty: nothing)."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix = str(suffix)
        self.hidden_size, self.num_experts, self.top = int(hidden_size), int(num_experts), int(top)
        self.expert_size = int(expert_size)
        self.groups, self.keep_groups = int(groups), int(keep_groups)
        if self.groups < 1 or self.num_experts % self.groups or not 1 <= self.keep_groups <= self.groups:
            raise ValueError(f"{prefix}: {groups} groups (keep {keep_groups}) do not divide {num_experts} experts")
        if not 1 <= self.top <= self.keep_groups * (self.num_experts // self.groups):
            raise ValueError(f"{prefix}: top {top} does not fit the experts of {keep_groups} kept groups")
        if scores not in self.SCORES or weight_on not in self.WEIGHT_ON:
            raise ValueError(f"{prefix}: scores {scores!r} (one of {self.SCORES}), weight_on {weight_on!r} (one of {self.WEIGHT_ON})")
        self.scores, self.normalize, self.weight_on = scores, bool(normalize), weight_on
        self.unit = ClampedGLU(limit, alpha, shift)
        self.shared_size = int(shared_size) if shared_size else None
        self.shared_unit = ClampedGLU(shared_limit if shared_limit is not None else limit, alpha, shift) if self.shared_size else None

    def _matrix(self, *parts: str) -> str:
        name = ".".join(parts)
        return self.name(f"{name}.{self.suffix}" if self.suffix else name)

    def _expert(self, index: int) -> str:
        return f"{self.names['expert']}{index}"

    def weight_specs(self) -> list[WeightSpec]:
        h, f = self.hidden_size, self.expert_size
        specs = [WeightSpec(self._matrix(self.names["router"]), (self.num_experts, h), VECTOR)]
        for e in range(self.num_experts):
            specs += [WeightSpec(self._matrix(self._expert(e), self.names["gate"]), (f, h), MATRIX),
                      WeightSpec(self._matrix(self._expert(e), self.names["up"]), (f, h), MATRIX),
                      WeightSpec(self._matrix(self._expert(e), self.names["down"]), (h, f), MATRIX)]
        if self.shared_size:
            s = self.names["shared"]
            specs += [WeightSpec(self._matrix(s, self.names["gate"]), (self.shared_size, h), MATRIX),
                      WeightSpec(self._matrix(s, self.names["up"]), (self.shared_size, h), MATRIX),
                      WeightSpec(self._matrix(s, self.names["down"]), (h, self.shared_size), MATRIX)]
        return specs

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.router = fetch(self._matrix(self.names["router"]))            # float32: the router is computed in 32-bit
        gate_up, down = [], []
        for e in range(self.num_experts):
            gate_up.append(torch.cat([fetch(self._matrix(self._expert(e), self.names[role])) for role in ("gate", "up")], dim=0))
            down.append(fetch(self._matrix(self._expert(e), self.names["down"])))
        self.gate_up = torch.stack(gate_up).contiguous()                  # [experts, 2 F, H], gate rows first
        self.down = torch.stack(down).contiguous()                        # [experts, H, F]
        self.shared_gate_up = self.shared_down = None
        if self.shared_size:
            s = self.names["shared"]
            self.shared_gate_up = Projection.stacked([fetch(self._matrix(s, self.names[role])) for role in ("gate", "up")],
                                                     label="shared gate_up")
            self.shared_down = Projection(fetch(self._matrix(s, self.names["down"])), label="shared down")

    def flops(self, tokens: int, attended: int) -> float:
        routed = 6.0 * tokens * self.top * self.expert_size * self.hidden_size
        shared = 6.0 * tokens * (self.shared_size or 0) * self.hidden_size
        return routed + shared + 2.0 * tokens * self.num_experts * self.hidden_size

    def forward(self, x, step=None) -> torch.Tensor:
        if hasattr(x, "materialize"):
            x = x.materialize()
        with stage("router"):
            chosen, weight = ops.moe_route(x, self.router, self.top, self.groups, self.keep_groups, self.scores,
                                           self.normalize)
            # bfloat16: the products run on the matrix cores, in tiles sized by the rows an expert gets in this step
            mfma = ops.moe_mfma_supported(x, self.gate_up, self.down)
            rows = ops.moe_tile_rows(chosen.numel(), self.num_experts, mfma)
            order, _, tiles = ops.moe_align(chosen, self.num_experts, rows)
        with stage("experts gate_up"):
            act = ops.moe_gate_up(x, self.gate_up, tiles, order, self.top, self.unit.limit, self.unit.alpha, self.unit.shift,
                                  tile_rows=rows, mfma=mfma, input_weight=weight if self.weight_on == "input" else None)
        with stage("experts down"):
            pairs = ops.moe_down(act, self.down, tiles, order, weight if self.weight_on == "output" else None, self.top,
                                 tile_rows=rows, mfma=mfma)
        shared = None
        if self.shared_size:
            unit = self.shared_unit
            gate_up = self.shared_gate_up(x)
            with stage("activation"):
                gated = ops.clamped_glu(gate_up, unit.limit, unit.alpha, unit.shift)
            shared = self.shared_down(gated)
        with stage("experts' sum"):
            return ops.moe_combine(pairs, self.top, shared)
