"""Dense gated feed-forward (SwiGLU and its kin).  Reference: somi_inference/models/qwen2.py:209-229."""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, Init, WeightSpec
from .base import FeedForward, Fetch, Runtime
from .linear import NormedRows, Projection


class SwiGLU(FeedForward):
    """y = down(act(gate(x)) * up(x)), no biases; ``activation`` is SiLU (the reference's) or the tanh form of GELU;
    in bfloat16 either is taken into the gate_up product's end.  gate and up are stacked
    into one ``[2I, H]`` matrix, gate rows first, as the reference merges them at load
    (somi_inference/models/qwen2_adapter.py:183-190, 244-248; qwen2.py:228 chunks the result)."""
    graph_safe = True
    takes_normed_rows = True

    ROLES = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int,
                 names: dict[str, str] | None = None, activation: str = "silu", suffix: str = "weight") -> None:
        """``names``: what the checkpoint calls this part's matrices, role -> name under the prefix.  Roles:
        ``gate``, ``up``, ``down`` (defaults ``gate_proj``, ``up_proj``, ``down_proj``), and ``gate_up`` for a
        checkpoint that stores gate and up as one ``[2I, H]`` matrix, gate rows first.  ``suffix``: what follows a
        matrix's name in the checkpoint (empty: nothing)."""
        super().__init__(prefix)
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"{prefix}: unknown activation {activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.activation, self.suffix = activation, str(suffix)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        unknown = set(names or {}) - set(self.ROLES) - {"gate_up"}
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)} and 'gate_up'")
        self.names = {**self.ROLES, **(names or {})}

    def weight_specs(self) -> list[WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        down = WeightSpec(self._tensor("down"), (h, i), MATRIX)
        if "gate_up" in self.names:
            return [WeightSpec(self._tensor("gate_up"), (2 * i, h), MATRIX), down]
        return [WeightSpec(self._tensor("gate"), (i, h), MATRIX), WeightSpec(self._tensor("up"), (i, h), MATRIX), down]

    def _tensor(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    INTERLEAVE = 16       # rows per block when gate and up are interleaved for the fused kernel

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        if "gate_up" in self.names:
            gate, up = fetch(self._tensor("gate_up")).chunk(2, dim=0)
        else:
            gate, up = (fetch(self._tensor(role)) for role in ("gate", "up"))
        # The layout of the merged matrix is private.  In bfloat16 the rows are interleaved in blocks of 16
        # (gate 0..15, up 0..15, gate 16..31, ...), so that the decode kernel has gate and up of the same
        # columns in one workgroup and applies the gate in its epilogue.
        self.interleaved = (runtime.dtype == torch.bfloat16 and self.intermediate_size % self.INTERLEAVE == 0
                            and self.hidden_size % 8 == 0)
        if self.interleaved:
            b, h = self.INTERLEAVE, self.hidden_size
            merged = torch.stack([gate.view(-1, b, h), up.view(-1, b, h)], dim=1).reshape(-1, h).contiguous()
            self.gate_up = Projection(merged, label="gate_up")
        else:
            self.gate_up = Projection.stacked([gate, up], label="gate_up")
        self.down = Projection(fetch(self._tensor("down")), label="down")

    def flops(self, tokens: int, attended: int) -> float:
        return self.gate_up.flops(tokens) + self.down.flops(tokens)

    def forward(self, x, step=None):
        if not self.interleaved:
            projected = self.gate_up(x)                 # rows that are still to be normed are normed by the product
            with stage("activation"):
                if self.activation == "silu":
                    return self.down.deferred(ops.silu_mul(projected))
                return self.down.deferred(ops.act_mul(projected, self.activation))
        if isinstance(x, NormedRows):
            if self.gate_up.fusable(x.h.shape[0]):
                # norm, gate_up and SiLU . up in one kernel
                with stage(self.gate_up.label):
                    gated = linear_kernels.linear_scaled(x.weighted, x.norm.eps, x.stats, self.gate_up.weight,
                                                         swiglu=self.activation)
                return self.down.deferred(gated)
            x = x.materialize()
        if x.data_ptr() % 16 == 0:
            with stage(self.gate_up.label):
                return self.down.deferred(linear_kernels.linear_swiglu(x, self.gate_up.weight, self.activation))
        projected = self.gate_up(x)
        with stage("activation"):
            if self.activation == "silu":
                return self.down.deferred(ops.silu_mul(projected, block=self.INTERLEAVE))
            return self.down.deferred(ops.act_mul(projected, self.activation, block=self.INTERLEAVE))


class PolyNormFF(FeedForward):
    """y = down(act(up(x))) without a gate, act a polynomial of normed powers with four learned numbers (a, b, c, e):

        act(z) = a N(z) + b N(z^2) + c N(z^3) + e,      N(u) = u / sqrt(mean(u^2) + eps) over a token's values,

    powers taken element by element.  The up product leaves float32 sums, the three mean squares are float32, the
    activation is rounded once to the compute dtype."""
    graph_safe = True

    ROLES = {"up": "up", "down": "down", "act": "act"}

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, eps: float,
                 names: dict[str, str] | None = None, suffix: str = "weight") -> None:
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix = str(suffix)
        self.hidden_size, self.intermediate_size, self.eps = int(hidden_size), int(intermediate_size), float(eps)

    def _tensor(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def weight_specs(self) -> list[WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return [WeightSpec(self._tensor("up"), (i, h), MATRIX), WeightSpec(self._tensor("down"), (h, i), MATRIX),
                WeightSpec(self.name(self.names["act"]), (4,), VECTOR, Init(0.3, 0.3))]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.up = Projection(fetch(self._tensor("up")), label="up")
        self.down = Projection(fetch(self._tensor("down")), label="down")
        self.coefficients = fetch(self.name(self.names["act"]))

    def flops(self, tokens: int, attended: int) -> float:
        return self.up.flops(tokens) + self.down.flops(tokens)

    def forward(self, x, step=None):
        if hasattr(x, "materialize"):
            x = x.materialize()
        with stage(self.up.label):
            z = linear_kernels.linear(x, self.up.weight, None, torch.float32)
        with stage("activation"):
            a = ops.poly_norm(z, self.coefficients, self.eps, self.runtime.dtype)
        with stage(self.down.label):
            return linear_kernels.linear(a, self.down.weight, None, torch.float32)


class ActivatedFF(FeedForward):
    """y = down(act(up(x) + b_up)) + b_down without a gate, act an element-wise unit with stored numbers of its own.

    ``activation`` "xielu": with the two stored numbers (p, q) of the ``act`` tensor,

        act(z) = softplus(p) z^2 + z / 2                          for z > 0,
                 (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2     for z <= 0.

    The up product leaves float32 sums (bias added), the unit is float32 and rounded once to the compute dtype; the
    down product leaves float32 sums for the residual streams."""
    graph_safe = True

    ROLES = {"up": "up", "down": "down", "act": "act"}
    ACTIVATIONS = {"xielu": 2}          # name -> how many numbers it stores

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "xielu", bias: bool = True,
                 names: dict[str, str] | None = None, suffix: str = "weight", bias_suffix: str = "bias") -> None:
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"{prefix}: unknown activation {activation!r}; known: {sorted(self.ACTIVATIONS)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix, self.bias_suffix = str(suffix), str(bias_suffix)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation, self.bias = activation, bool(bias)

    def _tensor(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def _bias(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.bias_suffix}")

    def weight_specs(self) -> list[WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        specs = [WeightSpec(self._tensor("up"), (i, h), MATRIX), WeightSpec(self._tensor("down"), (h, i), MATRIX),
                 WeightSpec(self.name(self.names["act"]), (self.ACTIVATIONS[self.activation],), VECTOR, Init(0.3, 0.3))]
        if self.bias:
            specs += [WeightSpec(self._bias("up"), (i,), VECTOR), WeightSpec(self._bias("down"), (h,), VECTOR)]
        return specs

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.up = Projection(fetch(self._tensor("up")), fetch(self._bias("up")) if self.bias else None, label="up")
        self.down = Projection(fetch(self._tensor("down")), fetch(self._bias("down")) if self.bias else None, label="down")
        self.numbers = fetch(self.name(self.names["act"]))

    def flops(self, tokens: int, attended: int) -> float:
        return self.up.flops(tokens) + self.down.flops(tokens)

    def forward(self, x, step=None):
        if hasattr(x, "materialize"):
            x = x.materialize()
        with stage(self.up.label):
            z = linear_kernels.linear(x, self.up.weight, self.up.bias, torch.float32)
        with stage("activation"):
            a = ops.xielu(z, self.numbers, self.runtime.dtype)
        return self.down.deferred(a)
