"""Differential attention over the paged cache, with a sliding window that keeps a request's first tokens.

Every head has two attention maps (two queries, two keys) over one set of values.  With a1 and a2 the maps'
outputs, ``o = a1 - lambda * a2`` with one number lambda for the layer,
``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff``; o is then divided by its root mean square over the head's value
channels and multiplied by ``1 - diff``.  Query head h reads key/value head ``h // (heads / kv_heads)``.  A token at
position i sees the keys j <= i with ``i - j < window`` or ``j < keep_first``.  Keys are cached after their rotation,
so a layer may read the keys and values of an earlier layer (``shares_cache``) with queries, mask and lambda of its
own.

Cache pages: K ``[pages, 2 kv_heads, page, key_dim]`` (the two maps of key/value head g at 2g and 2g + 1) and V
``[pages, kv_heads, value_dim, page]``.
"""

from __future__ import annotations

import torch

from ..kernels import diff_attention as diff_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, VECTOR, WeightSpec
from .base import PAGE, Fetch, LayerCache, Mixer, PagedSpec, PageTensor, PartSpec, Runtime
from .linear import Projection
from .registry import build_part


class DifferentialAttention(Mixer):
    graph_safe = True
    takes_normed_rows = True      # x only goes through the q/k/v projection, which norms rows while loading them
    entry_split = diff_kernels.DECODE_PORTION

    ROLES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj", "lq1": "lambda_q1", "lk1": "lambda_k1",
             "lq2": "lambda_q2", "lk2": "lambda_k2", "position": "rotary_emb"}

    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
                 position: PartSpec, scale: float, diff: float, eps: float, window: int | None = None,
                 keep_first: int = 0, shares_cache: bool = False,
                 reader_masks: tuple[tuple[int | None, int], ...] = (), names: dict[str, str] | None = None,
                 suffix: str = "weight") -> None:
        """``window``, ``keep_first``: this layer's mask (window None: every earlier key).  ``reader_masks``: the
        (window, keep_first) of the layers that read this layer's cache, so that the cache keeps what they see.
        ``names``: role -> the checkpoint's name under the prefix; ``suffix`` follows a matrix's name (empty: nothing)."""
        super().__init__(prefix)
        unknown = set(names or {}) - set(self.ROLES)
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)}")
        self.names = {**self.ROLES, **(names or {})}
        self.suffix = str(suffix)
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"heads ({num_heads}) must be divisible by kv_heads ({num_kv_heads})")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.diff, self.eps = float(scale), float(diff), float(eps)
        self.window = int(window) if window else None
        self.keep_first = int(keep_first)
        self.shares_cache = bool(shares_cache)
        self.reader_masks = tuple((int(w) if w else None, int(k)) for w, k in reader_masks)
        self.position = build_part("position", position, prefix=self.name(self.names["position"]))
        if getattr(self.position, "amplitude", 1.0) != 1.0:
            raise ValueError(f"{prefix}: this part's kernels take no amplitude on the rotation's cosines and sines")
        self.lam = 0.0

    # ------------------------------------------------------------------ weights
    def _matrix(self, role: str) -> str:
        return self.name(f"{self.names[role]}.{self.suffix}" if self.suffix else self.names[role])

    def _projections(self) -> list[tuple[str, int]]:
        q_width = self.num_heads * 2 * self.key_dim
        if self.shares_cache:
            return [("q", q_width)]
        return [("q", q_width), ("k", self.num_kv_heads * 2 * self.key_dim), ("v", self.num_kv_heads * self.value_dim)]

    def weight_specs(self) -> list[WeightSpec]:
        specs = [WeightSpec(self._matrix(role), (width, self.hidden_size), MATRIX) for role, width in self._projections()]
        specs.append(WeightSpec(self._matrix("o"), (self.hidden_size, self.num_heads * self.value_dim), MATRIX))
        specs += [WeightSpec(self.name(self.names[role]), (self.key_dim,), VECTOR) for role in ("lq1", "lk1", "lq2", "lk2")]
        return specs + self.position.weight_specs()

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.qkv = Projection.stacked([fetch(self._matrix(role)) for role, _ in self._projections()], label="q/k/v")
        self.out = Projection(fetch(self._matrix("o")), label="o")
        lq1, lk1, lq2, lk2 = (fetch(self.name(self.names[role])).to(torch.float32) for role in ("lq1", "lk1", "lq2", "lk2"))
        self.lam = float((torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum())).item()) + self.diff
        self.position.load(fetch, runtime)

    def flops(self, tokens: int, attended: int) -> float:
        """The projections, and for both maps q.k (key_dim channels) and p.v (value_dim channels) over the (token, key)
        pairs the step's tokens see (an upper bound where the window hides some)."""
        return (self.qkv.flops(tokens) + self.out.flops(tokens)
                + 4.0 * self.num_heads * (self.key_dim + self.value_dim) * attended)

    # -------------------------------------------------------------------- cache
    def cache_spec(self) -> PagedSpec | None:
        if self.shares_cache:
            return None
        masks = ((self.window, self.keep_first),) + self.reader_masks
        window = None if any(w is None for w, _ in masks) else max(w for w, _ in masks)
        keep_first = max(k for _, k in masks) if window is not None else 0
        return PagedSpec((PageTensor("k", (2 * self.num_kv_heads, PAGE, self.key_dim)),
                          PageTensor("v", (self.num_kv_heads, self.value_dim, PAGE))), window, None, keep_first)

    # ------------------------------------------------------------------ forward
    def forward(self, x, step, cache: LayerCache | None):
        if cache is None or cache.k is None:
            raise ValueError(f"{self.prefix}: attention needs a paged cache")
        k_shape = (2 * self.num_kv_heads, self.key_dim)
        if (cache.k.shape[1], cache.k.shape[3]) != k_shape or tuple(cache.v.shape[1:3]) != (self.num_kv_heads, self.value_dim):
            raise ValueError(f"{self.prefix}: the cache's pages {tuple(cache.k.shape)} / {tuple(cache.v.shape)} do not fit "
                             f"{self.num_kv_heads} key/value heads of {self.key_dim} and {self.value_dim} channels")
        view = step.paged[cache.group]
        own = not self.shares_cache
        qkv = self.qkv(x)                               # [N, 2 H dk (+ 2 G dk + G dv)]
        rotation = self.position.rotation_table()
        inv_freq, rotary_dim = rotation if rotation is not None else (None, 0)
        with stage("position encoding, k/v into pages"):
            ops.rope_kv_store_general(qkv, step.positions, view.slot_mapping if own else None, inv_freq, rotary_dim,
                                      getattr(self.position, "pairing", "half") == "neighbours",
                                      2 * self.num_heads, 2 * self.num_kv_heads if own else 0, self.key_dim,
                                      self.num_kv_heads if own else 0, self.value_dim,
                                      cache.k if own else None, cache.v if own else None)
        with stage("attention"):
            attended = diff_kernels.diff_attention(
                qkv, self.num_heads, cache.k, cache.v, view.block_table, step, window=self.window or 0,
                keep_first=self.keep_first, scale=self.scale, lam=self.lam, eps=self.eps, out_scale=1.0 - self.diff)
        return self.out.deferred(attended)
