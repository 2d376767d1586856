"""Attention over a shared low-rank latent, with a sink in the softmax.

Per token the layer keeps ONE vector for all heads: ``[c | r]`` with ``c = rms_norm(W_dkv h)[:rank] * w`` the latent
and ``r`` the last ``rot`` rows of ``W_dkv h``, rotated by the token's position: a key part that all heads share.  A
head's key is ``[U_h c | r]`` and its value ``V_h c``; queries come through a latent of their own, ``q = W_uq
(rms_norm(W_dq h) * w_q)``, head by head ``[dim plain | rot rotated]``.  With the configuration's ``scale``,

    score(i, j) = scale * (q_plain(i) . U_h c(j) + q_rot(i) . r(j)),      j <= i,
    p(i, j)     = exp(score(i, j)) / (sum_j' exp(score(i, j')) + exp(sink_h)),
    o_h(i)      = V_h sum_j p(i, j) c(j),

then ``W_o`` on the concatenated heads.  The sink is a learned number per head that only stands in the denominator.
Because U_h and V_h are linear, the kernels never expand keys or values: ``a_h = U_h^T q_plain`` is computed per query
(a per-head product), the attention runs on the kept vectors themselves (one key/value head of ``rank + rot`` key
channels whose first ``rank`` are the values), and V_h is applied to the weighted sum.  Norms, angles, scores and
softmax are float32 in both engines.

A layer that ``shares_cache`` has no W_dkv: it reads the vectors an earlier layer kept (the plan's ``cache_from``) with
its own U, V, queries and sink.

Variants, each a parameter: no query latent (``q_rank`` None: ``q = W_q h``), no sink (a softmax over the keys alone), a
``window`` of keys a token sees (itself included), a sigmoid gate on the concatenated heads before ``W_o`` (``sigmoid(W_g
h)`` of the mixer's own input), and the rotation's pairing (what the position part says).
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


class LatentAttention(Mixer):
    graph_safe = True
    PORTION_TOKENS = 8     # a step whose longest entry has this many tokens runs the kernel that shares a workgroup among tokens

    ROLES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
             "uv": "uv", "sink": "sink", "g": "g", "o": "o", "position": "rotary_emb"}

    def __init__(self, prefix: str, hidden_size: int, num_heads: int, dim: int, rot_dim: int, value_dim: int, kv_rank: int,
                 q_rank: int | None, scale: float, eps: float, position: PartSpec, shares_cache: bool = False,
                 page_size: int | None = None, names: dict[str, str] | None = None, suffix: str = "weight",
                 sink: bool = True, window: int | None = None, kept_window: "int | None | str" = "same",
                 gate: bool = False) -> None:
        """``position``: the rotation of the ``rot_dim`` channels (a rotary encoding of head size ``rot_dim``, or none).
        ``names``: role -> the checkpoint's name under the prefix (``dq_norm``, ``dkv_norm`` and ``sink`` are whole
        names; the matrices are followed by ``suffix`` unless it is empty).  ``q_rank`` None: no query latent, the
        queries are one product of the input (role ``q``).  ``sink`` False: no sink.  ``window``: the keys a token sees,
        itself included (None: all).  ``kept_window``: how long a token's kept row stays in the cache, where layers that
        read this layer's cache see further back than it does itself ("same": as long as ``window`` says; None: for
        ever).  ``gate``: the concatenated heads are multiplied by ``sigmoid(W_g h)`` (role ``g``) before ``W_o``."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix = str(suffix)
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.dim, self.rot_dim, self.value_dim = int(dim), int(rot_dim), int(value_dim)
        self.kv_rank, self.q_rank = int(kv_rank), (int(q_rank) if q_rank is not None else None)
        self.scale, self.eps = float(scale), float(eps)
        self.shares_cache = bool(shares_cache)
        self.page_size = int(page_size) if page_size else None
        self.has_sink, self.has_gate = bool(sink), bool(gate)
        self.window = int(window) if window else None
        self.kept_window = self.window if kept_window == "same" else (int(kept_window) if kept_window else None)
        if self.kept_window is not None and (self.window is None or self.window > self.kept_window):
            raise ValueError(f"{prefix}: a token sees {self.window or 'all'} keys but rows are kept for {self.kept_window}")
        self.position = build_part("position", position, prefix=self.name(self.names["position"]))
        self.pairing = getattr(self.position, "pairing", "half")
        self.rot_dims = int(getattr(self.position, "rotary_dim", 0))
        if self.rot_dims > self.rot_dim:
            raise ValueError(f"{prefix}: {self.rot_dims} rotated channels do not fit a key part of {self.rot_dim}")

    # ------------------------------------------------------------------ weights
    def _matrix(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def weight_specs(self) -> list[WeightSpec]:
        h, heads, rank = self.hidden_size, self.num_heads, self.kv_rank
        if self.q_rank is None:
            specs = [WeightSpec(self._matrix("q"), (heads * (self.dim + self.rot_dim), h), MATRIX)]
        else:
            specs = [
                WeightSpec(self._matrix("dq"), (self.q_rank, h), MATRIX),
                WeightSpec(self.name(self.names["dq_norm"]), (self.q_rank,), VECTOR, Init(1.0, 0.1)),
                WeightSpec(self._matrix("uq"), (heads * (self.dim + self.rot_dim), self.q_rank), MATRIX),
            ]
        if not self.shares_cache:
            specs += [WeightSpec(self._matrix("dkv"), (rank + self.rot_dim, h), MATRIX),
                      WeightSpec(self.name(self.names["dkv_norm"]), (rank,), VECTOR, Init(1.0, 0.1))]
        specs += [
            WeightSpec(self._matrix("uk"), (heads * self.dim, rank), MATRIX),
            WeightSpec(self._matrix("uv"), (heads * self.value_dim, rank), MATRIX),
        ]
        if self.has_sink:
            specs.append(WeightSpec(self.name(self.names["sink"]), (heads,), VECTOR, Init(0.0, 1.0)))
        if self.has_gate:
            specs.append(WeightSpec(self._matrix("g"), (heads * self.value_dim, h), MATRIX))
        specs.append(WeightSpec(self._matrix("o"), (h, heads * self.value_dim), MATRIX))
        return specs + self.position.weight_specs()

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.position.load(fetch, runtime)
        # one product of the input for everything that reads it: [query latent or queries | latent and shared key part |
        # gate], float32 sums, so that nothing is rounded before the norms, the rotation and the sigmoid
        down = [fetch(self._matrix("q" if self.q_rank is None else "dq"))]
        down += [] if self.shares_cache else [fetch(self._matrix("dkv"))]
        down += [fetch(self._matrix("g"))] if self.has_gate else []
        self.down = Projection.stacked(down, label="q/dkv/g" if self.q_rank is None else "dq/dkv")
        self.q_width = self.num_heads * (self.dim + self.rot_dim) if self.q_rank is None else self.q_rank
        self.q_norm = None if self.q_rank is None else fetch(self.name(self.names["dq_norm"]))
        self.c_norm = None if self.shares_cache else fetch(self.name(self.names["dkv_norm"]))
        self.up_q = None if self.q_rank is None else Projection(fetch(self._matrix("uq")), label="uq")
        heads, rank = self.num_heads, self.kv_rank
        # U_h^T per head, [heads, rank, dim]: the query's plain part goes to the latent's side
        self.key_maps = fetch(self._matrix("uk")).view(heads, self.dim, rank).transpose(1, 2).contiguous()
        self.value_maps = fetch(self._matrix("uv")).view(heads, self.value_dim, rank).contiguous()
        self.sink = fetch(self.name(self.names["sink"])) if self.has_sink else None
        self.out = Projection(fetch(self._matrix("o")), label="o")
        table = self.position.rotation_table() if self.rot_dims else None
        self.inv_freq = table[0] if table is not None else None
        self.amplitude = float(getattr(self.position, "amplitude", 1.0))

    def flops(self, tokens: int, attended: int) -> float:
        heads, rank = self.num_heads, self.kv_rank
        per_head = 2.0 * tokens * heads * rank * (self.dim + self.value_dim)
        attention = 2.0 * attended * heads * (2 * rank + self.rot_dim)
        up_q = self.up_q.flops(tokens) if self.up_q is not None else 0.0
        return self.down.flops(tokens) + up_q + per_head + attention + self.out.flops(tokens)

    # -------------------------------------------------------------------- cache
    def cache_spec(self) -> PagedSpec:
        """A token's row [c | r], and c once more transposed inside its page (consecutive positions of one channel
        adjacent: the operand layout of the weights-times-latents product on the matrix cores)."""
        return PagedSpec((PageTensor("latent", (PAGE, self.kv_rank + self.rot_dim)),
                          PageTensor("latent_t", (self.kv_rank, PAGE))), self.kept_window, self.page_size)

    # ------------------------------------------------------------------ forward
    def attend(self, queries: torch.Tensor, latent: torch.Tensor, step, view, latent_t: torch.Tensor | None = None) -> torch.Tensor:
        """The weighted sums of the kept latents for ``queries`` [N, heads, rank + rot] (the plain part already on the
        latent's side) -> [N, heads, rank].  bfloat16 sizes the matrix-core kernel is built for take it (it reads the
        transposed pages ``latent_t``); float32 and other sizes take the plain kernel."""
        if latent_t is not None and ops.latent_attention_mfma_supported(queries, latent, self.kv_rank):
            return ops.latent_attention_mfma(queries, latent, latent_t, view.block_table, step.token_entry, step.positions,
                                             self.kv_rank, self.scale, self.sink, step.max_context,
                                             portions=step.max_entry_len >= self.PORTION_TOKENS, window=self.window or 0)
        return ops.latent_attention_plain(queries, latent, view.block_table, step.token_entry, step.positions,
                                          self.kv_rank, self.scale, self.sink, window=self.window or 0)

    def forward(self, x, step, cache: LayerCache | None):
        if cache is None or "latent" not in cache.tensors:
            raise ValueError(f"{self.prefix}: latent attention needs a paged cache of latents")
        if cache.writes == self.shares_cache:
            raise ValueError(f"{self.prefix}: a layer keeps latents of its own or reads another layer's, not both")
        if hasattr(x, "materialize"):
            x = x.materialize()
        view = step.paged[cache.group]
        latent, latent_t = cache.tensors["latent"], cache.tensors.get("latent_t")
        heads, rank, rot, dtype = self.num_heads, self.kv_rank, self.rot_dim, self.runtime.dtype
        n = x.shape[0]
        with stage(self.down.label):
            rows = linear_kernels.linear(x, self.down.weight, None, torch.float32)
        with stage("latent norms, rotation, cache write"):
            q_latent = ops.latent_prepare(rows, self.q_width, rank, rot, self.q_norm, self.c_norm, self.eps, self.inv_freq,
                                          self.rot_dims, self.amplitude, step.positions,
                                          None if self.shares_cache else view.slot_mapping,
                                          None if self.shares_cache else latent, dtype,
                                          None if self.shares_cache else latent_t, pairing=self.pairing)
        # without a query latent the rows' first columns are the queries: their plain part as rounded by the kernel
        # above, their rotated part straight from the float32 sums
        q = self.up_q(q_latent) if self.up_q is not None else q_latent
        with stage("queries to the latent's side"):
            queries = torch.empty((n, heads, rank + rot), dtype=dtype, device=q.device)
            ops.head_linear(q.view(n, heads, self.dim + rot)[:, :, :self.dim], self.key_maps, out=queries[:, :, :rank])
            if rot:
                ops.latent_place(q if self.up_q is not None else rows[:, :self.q_width], heads, self.dim, rot, rank,
                                 self.inv_freq, self.rot_dims, self.amplitude, step.positions, queries, pairing=self.pairing)
        with stage("attention"):
            mixed = self.attend(queries, latent, step, view, latent_t)
        with stage("values from the latent"):
            values = ops.head_linear(mixed, self.value_maps).view(n, heads * self.value_dim)
        if self.has_gate:
            with stage("output gate"):
                values = ops.sigmoid_gate(values, rows[:, rows.shape[1] - heads * self.value_dim:])
        with stage(self.out.label):
            return linear_kernels.linear(values, self.out.weight, None, torch.float32)
