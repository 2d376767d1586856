"""Grouped-query attention whose heads' softmax weights are mixed by a matrix before they meet the values.

With H query heads over G key/value heads (query head h reads key/value head ``h // (H / G)``), ``dim`` query/key
channels and ``value_dim`` value channels a head:

    s_g(i, j) = scale * q_g(i) . k(j),   then, with a cap c,  s <- c * tanh(s / c)
    p_g(i, j) = exp(s_g(i, j)) / (extra + sum_j' exp(s_g(i, j')))        extra = 1: as if one more key of score 0 and value 0 were seen
    w_h(i, j) = sum_g T[h, g] p_g(i, j)                                  T: the ``talk`` matrix [H, H]
    o_h(i)    = sum_j w_h(i, j) v(j)                                     v of head h's own key/value head

over the keys ``max(0, i - window + 1) <= j <= i``, then ``W_o`` on the concatenated heads.  q and k are rotated by their
positions on their first ``rotary_dim`` channels (the position part says which channels turn together).  With
``value_rotation`` the value of position j is rotated by j over all its channels, with frequencies ``theta^(-2m /
value_dim)`` of their own, before it is cached, and a head's output at position i is turned back by i; the values then
enter the sum rotated by ``j - i``.

Every one of these is a parameter (no cap, no sink, no mix, no window and plain values give ordinary attention).  The
projections leave float32 sums, the rotations, scores, softmax, mix and weighted sum are float32 in both engines; q and
the cached keys and values take the engine's type.  A layer that ``shares_cache`` has no k/v projections and reads the
pages an earlier layer wrote.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, Init, WeightSpec
from .base import PAGE, Fetch, LayerCache, Mixer, PagedSpec, PageTensor, PartSpec, Runtime
from .linear import Projection
from .registry import build_part


class MixedHeadsAttention(Mixer):
    graph_safe = True
    PORTION_TOKENS = 4     # a step whose longest entry has this many tokens runs the kernel with several tokens a workgroup

    ROLES = {"q": "q", "k": "k", "v": "v", "o": "o", "talk": "talk", "position": "rotary_emb"}

    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, value_dim: int,
                 position: PartSpec, scale: float | None = None, softcap: float | None = None, window: int | None = None,
                 sink_one: bool = False, head_mix: bool = False, value_rotation: dict | None = None,
                 qkv_bias: bool = False, shares_cache: bool = False, names: dict[str, str] | None = None,
                 suffix: str = "weight", bias_suffix: str = "bias") -> None:
        """``sink_one``: one is added to the softmax's denominator.  ``head_mix``: the part has a ``talk`` tensor.
        ``value_rotation``: None or ``{"theta": ..., "pairing": "half" | "neighbours"}``.  ``names``: role -> the
        checkpoint's name under the prefix; a matrix's name is followed by ``suffix`` unless it is empty, its bias is
        ``<name>.<bias_suffix>``."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix, self.bias_suffix = str(suffix), str(bias_suffix)
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"{prefix}: {num_heads} query heads are no multiple of {num_kv_heads} key/value heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.value_dim = int(dim), int(value_dim)
        self.scale = float(scale) if scale is not None else self.dim ** -0.5
        self.softcap = float(softcap) if softcap else 0.0
        if self.softcap < 0.0:
            raise ValueError(f"{prefix}: a cap on the scores must be > 0, got {softcap}")
        self.window = int(window) if window else None
        self.sink_one, self.head_mix = bool(sink_one), bool(head_mix)
        self.qkv_bias, self.shares_cache = bool(qkv_bias), bool(shares_cache)
        self.position = build_part("position", position, prefix=self.name(self.names["position"]))
        if getattr(self.position, "amplitude", 1.0) != 1.0:
            raise ValueError(f"{prefix}: this part's kernels take no amplitude on the rotation's cosines and sines")
        self.value_rotation = None
        if value_rotation:
            theta, pairing = float(value_rotation["theta"]), str(value_rotation.get("pairing", "half"))
            if self.value_dim % 2 or theta <= 0.0 or pairing not in ops.PAIRINGS:
                raise ValueError(f"{prefix}: rotated values need an even size, a base > 0 and a known pairing, got "
                                 f"{self.value_dim} and {value_rotation}")
            self.value_rotation = {"theta": theta, "pairing": pairing}

    def _matrix(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def _bias(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.bias_suffix}")

    # ------------------------------------------------------------------ weights
    def _projections(self) -> list[tuple[str, int]]:
        q = [("q", self.num_heads * self.dim)]
        if self.shares_cache:
            return q
        return q + [("k", self.num_kv_heads * self.dim), ("v", self.num_kv_heads * self.value_dim)]

    def weight_specs(self) -> list[WeightSpec]:
        specs = []
        for role, width in self._projections():
            specs.append(WeightSpec(self._matrix(role), (width, self.hidden_size), MATRIX))
            if self.qkv_bias:
                specs.append(WeightSpec(self._bias(role), (width,), VECTOR))
        if self.head_mix:
            specs.append(WeightSpec(self.name(self.names["talk"]), (self.num_heads, self.num_heads), VECTOR, Init(0.0, 0.3)))
        specs.append(WeightSpec(self._matrix("o"), (self.hidden_size, self.num_heads * self.value_dim), MATRIX))
        return specs + self.position.weight_specs()

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        roles = [role for role, _ in self._projections()]
        self.qkv = Projection.stacked([fetch(self._matrix(r)) for r in roles],
                                      [fetch(self._bias(r)) for r in roles] if self.qkv_bias else None, label="q/k/v")
        self.talk = fetch(self.name(self.names["talk"])).contiguous() if self.head_mix else None
        self.out = Projection(fetch(self._matrix("o")), label="o")
        self.position.load(fetch, runtime)
        table = self.position.rotation_table()
        self.inv_freq, self.rot_dims = (table[0], int(table[1])) if table is not None else (None, 0)
        self.pairing = getattr(self.position, "pairing", "half")
        self.value_freq = None
        if self.value_rotation:
            exponents = torch.arange(0, self.value_dim, 2, dtype=torch.float64) / self.value_dim
            self.value_freq = (1.0 / (self.value_rotation["theta"] ** exponents)).to(torch.float32).to(runtime.device)

    def flops(self, tokens: int, attended: int) -> float:
        """The projections; q.k twice (the keys are walked once for the softmax's sums and once for the weights), the
        mix of the heads' weights, and the weights times the values, over the (token, key) pairs the step's tokens see."""
        heads = self.num_heads
        mix = 2.0 * heads * heads if self.head_mix else 0.0
        return (self.qkv.flops(tokens) + self.out.flops(tokens)
                + attended * (4.0 * heads * self.dim + mix + 2.0 * heads * self.value_dim))

    # -------------------------------------------------------------------- cache
    def cache_spec(self) -> PagedSpec | None:
        """Keys by token, ``[pages, kv_heads, page, dim]``; values transposed inside a page, ``[pages, kv_heads,
        value_dim, page]`` (consecutive positions of one channel adjacent: the operand layout of weights times values)."""
        if self.shares_cache:
            return None
        return PagedSpec((PageTensor("k", (self.num_kv_heads, PAGE, self.dim)),
                          PageTensor("v", (self.num_kv_heads, self.value_dim, PAGE))), self.window)

    # ------------------------------------------------------------------ forward
    def forward(self, x, step, cache: LayerCache | None):
        if cache is None or cache.tensors.get("k") is None:
            raise ValueError(f"{self.prefix}: attention needs a paged cache")
        if cache.writes == self.shares_cache:
            raise ValueError(f"{self.prefix}: a layer keeps keys and values of its own or reads another layer's, not both")
        if hasattr(x, "materialize"):
            x = x.materialize()
        view = step.paged[cache.group]
        keys, values = cache.tensors["k"], cache.tensors["v"]
        with stage(self.qkv.label):
            rows = linear_kernels.linear(x, self.qkv.weight, self.qkv.bias, torch.float32)
        with stage("position encoding, k/v into pages"):
            q = ops.mixed_attention_store(
                rows, step.positions, None if self.shares_cache else view.slot_mapping, self.inv_freq, self.rot_dims,
                self.pairing, self.value_freq, (self.value_rotation or {}).get("pairing", "half"), self.num_heads,
                self.num_kv_heads, self.dim, self.value_dim, None if self.shares_cache else keys,
                None if self.shares_cache else values, self.runtime.dtype)
        with stage("mixed attention"):
            attended = self.attend(q, keys, values, step, view)
        return self.out.deferred(attended)

    def attend(self, q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, step, view) -> torch.Tensor:
        """[N, heads * dim] rotated queries -> [N, heads * value_dim], over the pages of each token's request.  bfloat16
        sizes the matrix-core kernel is built for take it; float32 and other sizes take the plain kernel."""
        pairing = (self.value_rotation or {}).get("pairing", "half")
        if ops.mixed_attention_mfma_supported(q, keys, values, self.num_heads):
            return ops.mixed_attention_mfma(q, keys, values, view.block_table, step.token_entry, step.positions,
                                            self.num_heads, self.window or 0, self.scale, self.softcap,
                                            1.0 if self.sink_one else 0.0, self.talk, self.value_freq, pairing,
                                            portions=step.max_entry_len >= self.PORTION_TOKENS,
                                            max_context=step.max_context)
        return ops.mixed_attention_plain(q, keys, values, view.block_table, step.token_entry, step.positions,
                                         self.num_heads, self.window or 0, self.scale, self.softcap,
                                         1.0 if self.sink_one else 0.0, self.talk, self.value_freq,
                                         (self.value_rotation or {}).get("pairing", "half"))
