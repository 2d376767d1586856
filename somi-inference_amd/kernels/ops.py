"""Python faces of the HIP entry points.

Each function checks on the host what its kernel assumes (device, dtype,
contiguity, shapes), launches on torch's current stream and raises
:class:`KernelError` with the library's message on failure.  There is no
fallback to a library or CPU implementation: the product path fails loudly
when the extension cannot be built or loaded.
"""

from __future__ import annotations

import ctypes

import torch

from ..csrc import build as _build

F32, BF16 = 0, 1


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


def library() -> ctypes.CDLL:
    return _build.load()


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"unsupported dtype {dtype}; kernels take float32 and bfloat16")


GATED = {"silu": 1, "gelu_tanh": 2}      # the activations the gated products take into their ends


def gate_code(swiglu: "bool | str | None") -> int:
    """0: no gate; 1: SiLU (also for True); 2: the tanh form of GELU."""
    if not swiglu:
        return 0
    if swiglu is True:
        return 1
    if swiglu not in GATED:
        raise KernelError(f"unknown gate activation {swiglu!r}; known: {sorted(GATED)}")
    return GATED[swiglu]


_compute_units: dict[int, int] = {}


def compute_units() -> int:
    """Compute units of the current device, asked once per device."""
    device = torch.cuda.current_device()
    if device not in _compute_units:
        count = library().somi_compute_units()
        if count <= 0:
            raise KernelError("the device does not report its compute units")
        _compute_units[device] = count
    return _compute_units[device]


def _stream() -> ctypes.c_void_p:
    # the raw handle of torch's current stream on the current device, without building a Stream object
    # (torch.cuda.current_stream() costs several microseconds, and every launch asks)
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _ptr(t: torch.Tensor | None) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(library().somi_last_error().decode("utf-8", "replace"))


def _need(t: torch.Tensor, name: str, dtype: torch.dtype | None = None, shape: tuple | None = None) -> None:
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: must live on the GPU (there is no CPU path), got {t.device}")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")


def _v_shape(k_cache: torch.Tensor) -> tuple:
    pages, nkv, page_size, head_dim = k_cache.shape
    return (pages, nkv, head_dim, page_size)


def embedding(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """h[t] = table[ids[t]] as float32.  table: [V, H]; ids: [N] int32."""
    _need(table, "embedding table")
    _need(ids, "token ids", torch.int32)
    vocab, hidden = table.shape
    n = ids.numel()
    if out is None:
        out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    _need(out, "embedding out", torch.float32, (n, hidden))
    _check(library().somi_embedding(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(out),
                                    n, hidden, vocab, _stream()))
    return out


def gather_rows(src: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """out[r] = src[rows[r]] for a float32 matrix."""
    _need(src, "gather source", torch.float32)
    _need(rows, "row indices", torch.int32)
    out = torch.empty((rows.numel(), src.shape[1]), dtype=torch.float32, device=src.device)
    _check(library().somi_gather_rows_f32(_ptr(src), _ptr(rows), _ptr(out), rows.numel(), src.shape[1], _stream()))
    return out


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            delta: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """out = rmsnorm(h (+ delta)) * weight; with delta, h is updated in place (h += delta)."""
    _need(h, "residual stream", torch.float32)
    n, hidden = h.shape
    _need(weight, "norm weight", torch.float32, (hidden,))
    if delta is not None:
        _need(delta, "residual delta", out_dtype, (n, hidden))
    if out is None:
        out = torch.empty((n, hidden), dtype=out_dtype, device=h.device)
    _need(out, "norm out", out_dtype, (n, hidden))
    _check(library().somi_rmsnorm(_ptr(h), _ptr(delta), _ptr(weight), ctypes.c_float(eps), _ptr(out),
                                  dtype_code(out_dtype), n, hidden, _stream()))
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> None:
    _need(h, "residual stream", torch.float32)
    _need(delta, "residual delta", None, tuple(h.shape))
    _check(library().somi_residual_add(_ptr(h), _ptr(delta), dtype_code(delta.dtype),
                                       ctypes.c_int64(h.numel()), _stream()))


def linear_plain(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
                 out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x @ weight.T (+ bias) with the plain float32-accumulating kernel.  weight: [N, K]."""
    _need(x, "linear input")
    m, k = x.shape
    _need(weight, "linear weight", x.dtype)
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"linear: input has {k} features, weight expects {weight.shape[1]}")
    if bias is not None:
        _need(bias, "linear bias", torch.float32, (n,))
    out_dtype = out_dtype or x.dtype
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _check(library().somi_linear_plain(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), dtype_code(x.dtype),
                                       dtype_code(out_dtype), m, n, k, _stream()))
    return out


def linear_skinny(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
                  out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x @ weight.T (+ bias) for at most 64 bfloat16 rows on the matrix cores (weight streamed once)."""
    _need(x, "linear input", torch.bfloat16)
    m, k = x.shape
    _need(weight, "linear weight", torch.bfloat16)
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"linear: input has {k} features, weight expects {weight.shape[1]}")
    if bias is not None:
        _need(bias, "linear bias", torch.float32, (n,))
    out_dtype = out_dtype or x.dtype
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _check(library().somi_linear_skinny(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), dtype_code(out_dtype),
                                        m, n, k, _stream()))
    return out


def rope_kv_store(qkv: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                  inv_freq: torch.Tensor | None, rotary_dim: int, nq: int, nkv: int, head_dim: int,
                  k_cache: torch.Tensor | None, v_cache: torch.Tensor | None) -> None:
    """Rotate q (in place) and k, and store k and v in their cache pages.

    qkv: [N, (nq + 2 nkv) * D]; k cache: [pages, nkv, page_size, D]; v cache: [pages, nkv, D, page_size];
    slots: [N] int32.
    """
    _need(qkv, "qkv")
    n = qkv.shape[0]
    if qkv.shape[1] != (nq + 2 * nkv) * head_dim:
        raise KernelError(f"rope_kv_store: qkv width {qkv.shape[1]} != (nq + 2 nkv) * D = {(nq + 2 * nkv) * head_dim}")
    _need(positions, "positions", torch.int32, (n,))
    page_size = 0
    if nkv > 0:
        _need(slots, "slot mapping", torch.int32, (n,))
        _need(k_cache, "k cache", qkv.dtype)
        if k_cache.dim() != 4:
            raise KernelError("rope_kv_store: the k cache must be [pages, kv_heads, page_size, head_dim]")
        _need(v_cache, "v cache", qkv.dtype, _v_shape(k_cache))
        if k_cache.dim() != 4 or k_cache.shape[1] != nkv or k_cache.shape[3] != head_dim:
            raise KernelError(f"rope_kv_store: cache shape {tuple(k_cache.shape)} != [pages, {nkv}, page, {head_dim}]")
        page_size = k_cache.shape[2]
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
    _check(library().somi_rope_kv_store(_ptr(qkv), dtype_code(qkv.dtype), ctypes.c_int64(qkv.shape[1]),
                                        _ptr(positions), _ptr(slots), _ptr(inv_freq), rotary_dim, n, nq, nkv,
                                        head_dim, _ptr(k_cache), _ptr(v_cache), page_size, _stream()))


def paged_attention_plain(q: torch.Tensor, q_stride: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                          block_table: torch.Tensor, token_entry: torch.Tensor, positions: torch.Tensor,
                          nq: int, window: int, scale: float) -> torch.Tensor:
    """Causal attention of every token over its request's cached keys (plain float32 kernel).

    q: a tensor whose row t holds the nq query heads of token t first (row stride q_stride elements).
    """
    _need(q, "q")
    n = q.shape[0]
    _need(k_cache, "k cache", q.dtype)
    if k_cache.dim() != 4:
        raise KernelError("paged_attention: the k cache must be [pages, kv_heads, page_size, head_dim]")
    _need(v_cache, "v cache", q.dtype, _v_shape(k_cache))
    _, nkv, page_size, head_dim = k_cache.shape
    if q_stride < nq * head_dim or q.shape[1] < nq * head_dim:
        raise KernelError("paged_attention: q rows are narrower than nq * head_dim")
    _need(block_table, "block table", torch.int32)
    _need(token_entry, "token entries", torch.int32, (n,))
    _need(positions, "positions", torch.int32, (n,))
    out = torch.empty((n, nq * head_dim), dtype=q.dtype, device=q.device)
    _check(library().somi_paged_attention_plain(
        _ptr(q), dtype_code(q.dtype), ctypes.c_int64(q_stride), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
        block_table.shape[1], _ptr(token_entry), _ptr(positions), n, nq, nkv, head_dim, page_size, window,
        ctypes.c_float(scale), _ptr(out), _stream()))
    return out


def attention_decode(q: torch.Tensor, q_stride: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     block_table: torch.Tensor, token_entry: torch.Tensor, positions: torch.Tensor,
                     nq: int, window: int, scale: float, split_len: int, num_splits: int,
                     out: torch.Tensor, token_list: torch.Tensor | None = None) -> None:
    """MFMA attention of the listed tokens (all when ``token_list`` is None) over their pages, written
    into ``out`` ([N, nq * D] bfloat16).  The keys of a request are cut into ``num_splits`` ranges of
    ``split_len`` positions that run in parallel and are merged afterwards."""
    _need(q, "q", torch.bfloat16)
    n = q.shape[0]
    _need(k_cache, "k cache", torch.bfloat16)
    if k_cache.dim() != 4:
        raise KernelError("attention_decode: the k cache must be [pages, kv_heads, page_size, head_dim]")
    _need(v_cache, "v cache", torch.bfloat16, _v_shape(k_cache))
    _, nkv, page_size, head_dim = k_cache.shape
    if q_stride < nq * head_dim or q.shape[1] < nq * head_dim:
        raise KernelError("attention_decode: q rows are narrower than nq * head_dim")
    _need(block_table, "block table", torch.int32)
    _need(token_entry, "token entries", torch.int32, (n,))
    _need(positions, "positions", torch.int32, (n,))
    _need(out, "attention out", torch.bfloat16, (n, nq * head_dim))
    n_list = n
    if token_list is not None:
        _need(token_list, "token list", torch.int32)
        n_list = token_list.numel()
    part_acc = part_ml = None
    if num_splits > 1:
        part_acc = torch.empty((n_list * nq * num_splits, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_list * nq * num_splits, 2), dtype=torch.float32, device=q.device)
    _check(library().somi_attention_decode(
        _ptr(q), ctypes.c_int64(q_stride), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
        _ptr(token_list), _ptr(token_entry), _ptr(positions), n_list, nq, nkv, head_dim, page_size, window,
        ctypes.c_float(scale), split_len, num_splits, _ptr(out), _ptr(part_acc), _ptr(part_ml), _stream()))


def attention_prefill(q: torch.Tensor, q_stride: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_table: torch.Tensor, entry_start: torch.Tensor, entry_first_position: torch.Tensor,
                      max_entry_len: int, nq: int, window: int, scale: float, out: torch.Tensor,
                      max_context: int = 0, shape: int = 0, entry_len: torch.Tensor | None = None) -> None:
    """MFMA causal attention of every token of every portion over its request's pages, into ``out``
    ([N, nq * D] bfloat16).  entry_start: [E + 1] int32 offsets of the portions in the flat batch;
    entry_first_position: [E] int32.  ``max_context``: the longest context a portion ends at, a hint for the
    launch shape (0: unknown).  ``shape``: 0 lets the launcher choose; 1 (64 queries a workgroup), 2 (the same
    with a query block's keys split over two wavefronts) or 3 (128 queries) asks for that shape of the 16 x 16 LDS
    kernel; 4 (128 queries, two key splits) or 5 (256 queries) for that shape of the 32 x 32 tile kernel (head sizes 64
    and 128, pages of 8 keys or more).
    ``entry_len``: [E] int32 lengths that stand for the offsets' own; 0 leaves a portion out (its rows of ``out`` are
    not written)."""
    _need(q, "q", torch.bfloat16)
    n = q.shape[0]
    _need(k_cache, "k cache", torch.bfloat16)
    if k_cache.dim() != 4:
        raise KernelError("attention_prefill: the k cache must be [pages, kv_heads, page_size, head_dim]")
    _need(v_cache, "v cache", torch.bfloat16, _v_shape(k_cache))
    _, nkv, page_size, head_dim = k_cache.shape
    if q_stride < nq * head_dim or q.shape[1] < nq * head_dim:
        raise KernelError("attention_prefill: q rows are narrower than nq * head_dim")
    _need(block_table, "block table", torch.int32)
    entries = block_table.shape[0]
    _need(entry_start, "entry offsets", torch.int32, (entries + 1,))
    _need(entry_first_position, "entry first positions", torch.int32, (entries,))
    if entry_len is not None:
        _need(entry_len, "entry lengths", torch.int32, (entries,))
    _need(out, "attention out", torch.bfloat16, (n, nq * head_dim))
    if not 0 <= max_entry_len <= n:
        raise KernelError(f"attention_prefill: longest portion {max_entry_len} does not fit {n} tokens")
    _check(library().somi_attention_prefill(
        _ptr(q), ctypes.c_int64(q_stride), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
        _ptr(entry_start), _ptr(entry_first_position), _ptr(entry_len), entries, max_entry_len, max(0, int(max_context)), int(shape), nq, nkv,
        head_dim, page_size, window, ctypes.c_float(scale), _ptr(out), _stream()))


def silu_mul(gate_up: torch.Tensor, block: int = 0) -> torch.Tensor:
    """silu(gate) * up.  block == 0: gate_up = [gate | up]; block == b: gate and up columns interleaved
    in blocks of b columns (gate 0..b-1, up 0..b-1, gate b..2b-1, ...)."""
    _need(gate_up, "gate_up")
    n, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError(f"silu_mul: width {two_i} is odd")
    out = torch.empty((n, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(library().somi_silu_mul(_ptr(gate_up), _ptr(out), dtype_code(gate_up.dtype), n, two_i // 2, block,
                                   _stream()))
    return out


def linear_skinny_swiglu(x: torch.Tensor, weight: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """act(x @ gate.T) * (x @ up.T) in one kernel for at most 64 bfloat16 rows, act SiLU or the tanh form of GELU.
    weight: [2 I, K] with gate and up rows interleaved in blocks of 16."""
    _need(x, "linear input", torch.bfloat16)
    m, k = x.shape
    _need(weight, "gate_up weight", torch.bfloat16)
    if weight.shape[1] != k or weight.shape[0] % 32:
        raise KernelError(f"linear_skinny_swiglu: weight {tuple(weight.shape)} does not fit input width {k}")
    inter = weight.shape[0] // 2
    out = torch.empty((m, inter), dtype=x.dtype, device=x.device)
    _check(library().somi_linear_skinny_gated(_ptr(x), _ptr(weight), _ptr(out), dtype_code(x.dtype), m, inter, k,
                                              gate_code(activation), _stream()))
    return out


# 136 MB per device: partial sums of a split K (a kernel splits less if it is short) and, in the streamed many-rows
# product, two slots of a 256 x 256 tile's sums for each of 256 workgroups
MID_WORKSPACE_FLOATS = 34 << 20
_mid_workspaces: dict[torch.device, torch.Tensor] = {}


def _mid_workspace(device: torch.device) -> torch.Tensor:
    """One workspace per device, shared by every launch: the launches of a device run on one stream."""
    held = _mid_workspaces.get(device)
    if held is None:
        held = _mid_workspaces[device] = torch.empty((MID_WORKSPACE_FLOATS,), dtype=torch.float32, device=device)
    return held


FUSED_MAX_ROWS = 64       # what the products fused with the residual add and the norm take


def _stats_width(rows: int) -> int:
    return 16 * ((rows + 15) // 16)


stats_width = _stats_width          # columns of the row statistics of this many rows


def _big_operands(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, what: str) -> tuple[int, int, int]:
    """Checks what the many-rows kernel assumes of its operands; x may be a view with a row stride of its own."""
    for t, name in ((x, "input"), (weight, "weight")):
        if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.bfloat16 or t.dim() != 2 or t.stride(1) != 1:
            raise KernelError(f"{what}: the {name} must be a bfloat16 matrix on the GPU with contiguous rows")
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"{what}: input has {k} features, weight expects {weight.shape[1]}")
    if k % 8 or x.stride(0) % 8 or weight.stride(0) % 8 or x.data_ptr() % 16 or weight.data_ptr() % 16:
        raise KernelError(f"{what}: K = {k} and the row strides must be multiples of 8 and the operands aligned to 16 bytes")
    if bias is not None:
        _need(bias, "linear bias", torch.float32, (n,))
    return m, n, k


def big_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """The many-rows kernel takes these operands (bfloat16, K a multiple of 8, 16-byte alignment)."""
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1
            and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def linear_big(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, *, swiglu: "bool | str" = False,
               eps: float = 0.0, stats: torch.Tensor | None = None, tile: int = 0,
               out: torch.Tensor | None = None, split_k: bool = True) -> torch.Tensor:
    """s * (x @ weight.T) (+ bias) -> bfloat16 for any number of rows, on 256-row tiles of the matrix cores.
    With ``stats`` ([blocks, width >= M] partial sums of squares, from :func:`linear_big_residual` or
    :func:`linear_residual`) the rows are scaled by s = 1 / sqrt(stats.sum(0) / K + eps): the product of
    RMS-normed rows when x holds ``norm_weight * h``.  With ``swiglu`` weight is [2 I, K] with gate and up rows
    interleaved in blocks of 16 and the result is act(s g) * (s u) -> [M, I] (True or "silu": SiLU; "gelu_tanh").  ``tile``: 0 lets the launcher
    choose the tile width, 128 or 256 asks for it.  ``split_k``: the ungated form may share a tile's K among
    workgroups (through the device's workspace) where its tiles alone would leave most of the device idle."""
    m, n, k = _big_operands(x, weight, bias, "linear_big")
    if swiglu and (n % 32 or bias is not None):
        raise KernelError(f"linear_big: the gated form needs an even number of 16-row blocks and no bias, got N = {n}")
    row_scale = None
    if stats is not None:
        _need(stats, "row statistics", torch.float32)
        if stats.dim() != 2 or stats.shape[1] < m:
            raise KernelError(f"linear_big: row statistics must be [blocks, >= {m}], got {tuple(stats.shape)}")
        row_scale = torch.empty((m,), dtype=torch.float32, device=x.device)
        _check(library().somi_row_scale(_ptr(stats), stats.shape[0], stats.shape[1], m, k, ctypes.c_float(eps),
                                        _ptr(row_scale), _stream()))
    cols = n // 2 if swiglu else n
    if out is None:
        out = torch.empty((m, cols), dtype=torch.bfloat16, device=x.device)
    _need(out, "linear_big out", torch.bfloat16, (m, cols))
    workspace = _mid_workspace(x.device) if split_k else None
    _check(library().somi_linear_big(_ptr(x), ctypes.c_int64(x.stride(0)), _ptr(weight), ctypes.c_int64(weight.stride(0)),
                                     _ptr(bias), _ptr(out), m, n, k, _ptr(row_scale), gate_code(swiglu), int(tile),
                                     _ptr(workspace), ctypes.c_int64(workspace.numel() if workspace is not None else 0),
                                     _stream()))
    return out


def linear_big_residual(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, h: torch.Tensor,
                        next_norm_weight: torch.Tensor | None = None, tile: int = 0, split_k: bool = True
                        ) -> tuple[torch.Tensor, torch.Tensor | None]:
    """h += x @ weight.T (+ bias) in float32, in place, for any number of rows.  Returns the row statistics
    ``[blocks, 16 ceil(M / 16)]`` (sums of squares of the new h, each over the 64 columns of one wavefront) and,
    with ``next_norm_weight``, the rows ``bfloat16(next_norm_weight * h)``: what :func:`linear_big` scales.
    ``split_k``: the 128-row tile may split K over workgroups (through the device's workspace) where its tiles alone
    would leave most of the device idle."""
    m, n, k = _big_operands(x, weight, bias, "linear_big_residual")
    _need(h, "residual stream", torch.float32, (m, n))
    lib = library()
    blocks = lib.somi_linear_big_stats_blocks(m, n, k, int(tile))
    stats = torch.empty((blocks, _stats_width(m)), dtype=torch.float32, device=x.device)
    weighted = None
    if next_norm_weight is not None:
        _need(next_norm_weight, "norm weight", torch.float32, (n,))
        weighted = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    workspace = _mid_workspace(x.device) if split_k else None
    _check(lib.somi_linear_big_residual(_ptr(x), ctypes.c_int64(x.stride(0)), _ptr(weight), ctypes.c_int64(weight.stride(0)),
                                        _ptr(bias), _ptr(h), _ptr(next_norm_weight), _ptr(weighted), _ptr(stats),
                                        stats.shape[1], m, n, k, int(tile), _ptr(workspace),
                                        ctypes.c_int64(workspace.numel() if workspace is not None else 0), _stream()))
    return stats, weighted


def linear_big_f32(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, tile: int = 0,
                   out: torch.Tensor | None = None) -> torch.Tensor:
    """x @ weight.T (+ bias) as float32 for any number of bfloat16 rows (logits of many rows at once: the weight is
    read once, and no result passes through bfloat16)."""
    m, n, k = _big_operands(x, weight, bias, "linear_big_f32")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _need(out, "linear_big_f32 out", torch.float32, (m, n))
    workspace = _mid_workspace(x.device)
    _check(library().somi_linear_big_f32(_ptr(x), ctypes.c_int64(x.stride(0)), _ptr(weight), ctypes.c_int64(weight.stride(0)),
                                         _ptr(bias), _ptr(out), m, n, k, int(tile), _ptr(workspace),
                                         ctypes.c_int64(workspace.numel()), _stream()))
    return out


def linear_big_rope_store(x: torch.Tensor, eps: float, stats: torch.Tensor | None, weight: torch.Tensor,
                          bias: torch.Tensor | None, positions: torch.Tensor, slots: torch.Tensor,
                          inv_freq: torch.Tensor, nq: int, nkv: int, head_dim: int, k_cache: torch.Tensor,
                          v_cache: torch.Tensor, tile: int = 0) -> torch.Tensor:
    """The q/k/v product of many bfloat16 rows where it shares a tile's K among workgroups
    (:func:`linear_big_splits` > 1), with the rows' scales (from ``stats``, as :func:`linear_big` takes them), the
    rotary encoding of q and k and the store of k and v into their cache pages in the kernel that adds the splits'
    sums -> q [M, nq * D], rotated.  Arguments as :func:`linear_rope_store`."""
    n = (nq + 2 * nkv) * head_dim
    m, n_w, k = _big_operands(x, weight, bias, "linear_big_rope_store")
    if n_w != n:
        raise KernelError(f"linear_big_rope_store: the weight has {n_w} rows, {nq} + 2 x {nkv} heads of {head_dim} are {n}")
    row_scale = None
    if stats is not None:
        _need(stats, "row statistics", torch.float32)
        if stats.dim() != 2 or stats.shape[1] < m:
            raise KernelError(f"linear_big_rope_store: row statistics must be [blocks, >= {m}], got {tuple(stats.shape)}")
        row_scale = torch.empty((m,), dtype=torch.float32, device=x.device)
        _check(library().somi_row_scale(_ptr(stats), stats.shape[0], stats.shape[1], m, k, ctypes.c_float(eps),
                                        _ptr(row_scale), _stream()))
    _need(positions, "positions", torch.int32, (m,))
    _need(slots, "slot mapping", torch.int32, (m,))
    _need(inv_freq, "inv_freq", torch.float32, (head_dim // 2,))
    _need(k_cache, "k cache", torch.bfloat16)
    if k_cache.dim() != 4 or k_cache.shape[1] != nkv or k_cache.shape[3] != head_dim:
        raise KernelError(f"linear_big_rope_store: cache shape {tuple(k_cache.shape)} != [pages, {nkv}, page, {head_dim}]")
    _need(v_cache, "v cache", torch.bfloat16, _v_shape(k_cache))
    q = torch.empty((m, nq * head_dim), dtype=torch.bfloat16, device=x.device)
    workspace = _mid_workspace(x.device)
    _check(library().somi_linear_big_rope_store(
        _ptr(x), ctypes.c_int64(x.stride(0)), _ptr(weight), ctypes.c_int64(weight.stride(0)), _ptr(bias), _ptr(q), m, k,
        _ptr(row_scale), _ptr(positions), _ptr(slots), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), nq, nkv, head_dim,
        k_cache.shape[2], int(tile), _ptr(workspace), ctypes.c_int64(workspace.numel()), _stream()))
    return q


BIG_TILE_STREAM, BIG_TILE_NO_STREAM = 1000, 2000      # added to a tile code: ask for the streamed form, or forbid it


def linear_big_splits(m: int, n: int, k: int, tile: int = 0) -> int:
    """Workgroups that share a tile's K in :func:`linear_big_residual` for these sizes (1: K is not split)."""
    return library().somi_linear_big_splits(m, n, k, int(tile), ctypes.c_int64(MID_WORKSPACE_FLOATS))


def linear_big_streams(m: int, n: int, k: int, tile: int = 0, units: int = 0) -> int:
    """Workgroups that the (tile, stage) units of the many-rows product are dealt out to for these sizes (0: tiles
    are handed out whole), on a device of ``units`` compute units (0: the current device)."""
    return library().somi_linear_big_streams(m, n, k, int(tile), ctypes.c_int64(MID_WORKSPACE_FLOATS), int(units))


def linear_big_tail(m: int, n: int, k: int, units: int = 0) -> tuple[int, int]:
    """(columns, splits): the last columns of a many-rows product (plain or gated, tile code 0) that run as a product
    of their own with K shared among workgroups, where whole rounds of 256 x 128 tiles leave a tail too small to fill
    the device; (0, 1) where the product runs whole.  ``units``: the device's compute units (0: the current device)."""
    splits = ctypes.c_int(1)
    columns = library().somi_linear_big_tail(m, n, k, ctypes.c_int64(MID_WORKSPACE_FLOATS), int(units), ctypes.byref(splits))
    return columns, splits.value


def residual_stats_blocks(m: int, n: int, k: int, mid: bool) -> int:
    """Rows of the statistics that :func:`linear_residual` writes for these sizes."""
    lib = library()
    return lib.somi_linear_mid_residual_tiles(m, n, k) if mid else lib.somi_linear_residual_blocks(m, n)


def linear_residual(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, h: torch.Tensor,
                    next_norm_weight: torch.Tensor | None = None, mid: bool = False
                    ) -> tuple[torch.Tensor, torch.Tensor | None]:
    """h += x @ weight.T (+ bias) in float32, in place, for at most 64 bfloat16 rows.  Returns the row statistics
    ``[workgroups, 16 ceil(M / 16)]`` (per workgroup and row the sum of squares of the new h over the workgroup's
    columns) and, with ``next_norm_weight``, the rows ``bfloat16(next_norm_weight * h)`` that :func:`linear_scaled`
    reads.  ``mid``: by the kernel that shares x inside a workgroup and splits K over workgroups."""
    _need(x, "linear input", torch.bfloat16)
    m, k = x.shape
    _need(weight, "linear weight", torch.bfloat16)
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"linear: input has {k} features, weight expects {weight.shape[1]}")
    if bias is not None:
        _need(bias, "linear bias", torch.float32, (n,))
    _need(h, "residual stream", torch.float32, (m, n))
    lib = library()
    blocks = residual_stats_blocks(m, n, k, mid)
    stats_stride = 0                    # rows of the statistics follow each other
    stats = torch.empty((blocks, _stats_width(m)), dtype=torch.float32, device=x.device)
    weighted = None
    if next_norm_weight is not None:
        _need(next_norm_weight, "norm weight", torch.float32, (n,))
        weighted = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    if mid:
        workspace = _mid_workspace(x.device)
        _check(lib.somi_linear_mid_residual(_ptr(x), _ptr(weight), _ptr(bias), _ptr(h), _ptr(stats), stats_stride,
                                            _ptr(next_norm_weight), _ptr(weighted), m, n, k, _ptr(workspace),
                                            ctypes.c_int64(workspace.numel()), _stream()))
    else:
        _check(lib.somi_linear_residual(_ptr(x), _ptr(weight), _ptr(bias), _ptr(h), _ptr(stats), stats_stride,
                                        _ptr(next_norm_weight), _ptr(weighted), m, n, k, _stream()))
    return stats, weighted


def linear_scaled(x: torch.Tensor, eps: float, stats: torch.Tensor, weight: torch.Tensor,
                  bias: torch.Tensor | None = None, swiglu: "bool | str" = False, mid: bool = False) -> torch.Tensor:
    """s * (x @ weight.T) (+ bias) -> bfloat16 with the row scales s = 1 / sqrt(stats.sum(0) / K + eps): the
    product of RMS-normed rows when x holds ``norm_weight * h`` and stats the sums of squares of h, both from
    :func:`linear_residual`.  At most 64 rows.  With ``swiglu`` weight is [2 I, K] with gate and up rows
    interleaved in blocks of 16 and the result is silu(s g) * (s u) for the gate and up products g, u.
    ``mid``: by the kernel that shares x inside a workgroup and splits K over workgroups."""
    _need(x, "linear input", torch.bfloat16)
    m, k = x.shape
    _need(weight, "linear weight", torch.bfloat16)
    n = weight.shape[0]
    if weight.shape[1] != k or (swiglu and n % 32):
        raise KernelError(f"linear_scaled: weight {tuple(weight.shape)} does not fit input width {k}")
    if bias is not None:
        _need(bias, "linear bias", torch.float32, (n,))
    _need(stats, "row statistics", torch.float32)
    if stats.dim() != 2 or stats.shape[1] != _stats_width(m):
        raise KernelError(f"linear_scaled: row statistics must be [blocks, {_stats_width(m)}], got {tuple(stats.shape)}")
    out = torch.empty((m, n // 2 if swiglu else n), dtype=torch.bfloat16, device=x.device)
    if mid:
        workspace = _mid_workspace(x.device)
        _check(library().somi_linear_mid_scaled(_ptr(x), ctypes.c_float(eps), _ptr(stats), stats.shape[0],
                                                _ptr(weight), _ptr(bias), _ptr(out), m, n, k, gate_code(swiglu),
                                                _ptr(workspace), ctypes.c_int64(workspace.numel()), _stream()))
    else:
        _check(library().somi_linear_scaled(_ptr(x), ctypes.c_float(eps), _ptr(stats), stats.shape[0], _ptr(weight),
                                            _ptr(bias), _ptr(out), m, n, k, gate_code(swiglu), _stream()))
    return out


def linear_rope_store(x: torch.Tensor, eps: float, stats: torch.Tensor | None, weight: torch.Tensor,
                      bias: torch.Tensor | None, positions: torch.Tensor, slots: torch.Tensor, inv_freq: torch.Tensor,
                      nq: int, nkv: int, head_dim: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      out: torch.Tensor | None = None) -> torch.Tensor:
    """The q/k/v product of at most 64 bfloat16 rows with the rotary encoding of q and k and the store of k and v
    into their cache pages in its end -> q [M, nq * D], rotated.  weight: [(nq + 2 nkv) * D, K], q heads, k
    heads, v heads.  With ``stats`` x holds ``norm_weight * h`` and the sums are scaled per row as in
    :func:`linear_scaled` (``stats`` may be the columns of these rows in the table of more rows); without, x is
    used as it is.  The whole head is rotated (inv_freq: [D / 2]); D must be a multiple of 32."""
    _need(x, "linear input", torch.bfloat16)
    m, k = x.shape
    _need(weight, "q/k/v weight", torch.bfloat16, ((nq + 2 * nkv) * head_dim, k))
    if bias is not None:
        _need(bias, "q/k/v bias", torch.float32, (weight.shape[0],))
    stats_stride = 0
    if stats is not None:
        if not isinstance(stats, torch.Tensor) or not stats.is_cuda or stats.dtype != torch.float32:
            raise KernelError("linear_rope_store: row statistics must be a float32 tensor on the GPU")
        if stats.dim() != 2 or stats.shape[1] != _stats_width(m) or stats.stride(1) != 1 or stats.stride(0) % 4:
            raise KernelError(f"linear_rope_store: row statistics must be [blocks, {_stats_width(m)}] with rows of "
                              f"consecutive floats, got {tuple(stats.shape)} with strides {stats.stride()}")
        stats_stride = stats.stride(0)
    _need(positions, "positions", torch.int32, (m,))
    _need(slots, "slot mapping", torch.int32, (m,))
    _need(inv_freq, "inv_freq", torch.float32, (head_dim // 2,))
    _need(k_cache, "k cache", torch.bfloat16)
    if k_cache.dim() != 4 or k_cache.shape[1] != nkv or k_cache.shape[3] != head_dim:
        raise KernelError(f"linear_rope_store: cache shape {tuple(k_cache.shape)} != [pages, {nkv}, page, {head_dim}]")
    _need(v_cache, "v cache", torch.bfloat16, _v_shape(k_cache))
    if out is None:
        q = torch.empty((m, nq * head_dim), dtype=torch.bfloat16, device=x.device)
    else:
        _need(out, "q", torch.bfloat16, (m, nq * head_dim))
        q = out
    _check(library().somi_linear_rope_store(_ptr(x), ctypes.c_float(eps), _ptr(stats),
                                            stats.shape[0] if stats is not None else 0, stats_stride, _ptr(weight), _ptr(bias),
                                            _ptr(q), _ptr(positions), _ptr(slots), _ptr(inv_freq), _ptr(k_cache),
                                            _ptr(v_cache), nq, nkv, head_dim, k_cache.shape[2], m, k, _stream()))
    return q


def linear_mid(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
               out_dtype: torch.dtype | None = None, swiglu: "bool | str" = False) -> torch.Tensor:
    """x @ weight.T (+ bias) for at most 64 bfloat16 rows, x shared by the wavefronts of a workgroup, K split
    over workgroups where the columns do not fill the device.  With ``swiglu`` weight is [2 I, K] with gate and
    up rows interleaved in blocks of 16 and the result is silu(x @ gate.T) * (x @ up.T)."""
    _need(x, "linear input", torch.bfloat16)
    m, k = x.shape
    _need(weight, "linear weight", torch.bfloat16)
    n = weight.shape[0]
    if weight.shape[1] != k or (swiglu and n % 32):
        raise KernelError(f"linear_mid: weight {tuple(weight.shape)} does not fit input width {k}")
    if bias is not None:
        _need(bias, "linear bias", torch.float32, (n,))
    out_dtype = out_dtype or x.dtype
    out = torch.empty((m, n // 2 if swiglu else n), dtype=out_dtype, device=x.device)
    workspace = _mid_workspace(x.device)
    _check(library().somi_linear_mid(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), dtype_code(out_dtype), m, n, k,
                                     gate_code(swiglu), _ptr(workspace), ctypes.c_int64(workspace.numel()), _stream()))
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor) -> torch.Tensor:
    """One token per row: argmax where temperature is 0, else an inverse-CDF draw from softmax(logits / T)."""
    _need(logits, "logits", torch.float32)
    rows, vocab = logits.shape
    _need(temperature, "temperature", torch.float32, (rows,))
    _need(uniform, "uniform", torch.float32, (rows,))
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    workspace = torch.empty((max(1, library().somi_sample_workspace_floats(rows, vocab)),), dtype=torch.float32,
                            device=logits.device)
    _check(library().somi_sample(_ptr(logits), rows, vocab, _ptr(temperature), _ptr(uniform), _ptr(out),
                                 _ptr(workspace), _stream()))
    return out


def repetition_penalty(logits_row: torch.Tensor, ids: torch.Tensor, penalty: float) -> None:
    """In place on one row of float32 logits; ids: distinct int32 token ids."""
    _need(logits_row, "logits row", torch.float32)
    _need(ids, "penalised ids", torch.int32)
    _check(library().somi_repetition_penalty(_ptr(logits_row), logits_row.numel(), _ptr(ids), ids.numel(),
                                             ctypes.c_float(penalty), _stream()))


def repetition_penalty_rows(logits: torch.Tensor, offsets: torch.Tensor, ids: torch.Tensor, penalties: torch.Tensor,
                            most_ids: int) -> None:
    """In place on [rows, vocab] float32 logits: row r's distinct ids are ids[offsets[r]:offsets[r + 1]], its
    penalty penalties[r] (1 leaves the row alone).  ``most_ids``: the largest number of ids a row has."""
    _need(logits, "logits", torch.float32)
    rows, vocab = logits.shape
    _need(offsets, "penalty offsets", torch.int32, (rows + 1,))
    _need(ids, "penalised ids", torch.int32)
    _need(penalties, "penalties", torch.float32, (rows,))
    if most_ids < 0 or most_ids > ids.numel():
        raise KernelError(f"repetition_penalty_rows: most_ids={most_ids} does not fit {ids.numel()} ids")
    _check(library().somi_repetition_penalty_rows(_ptr(logits), rows, vocab, _ptr(offsets), _ptr(ids), _ptr(penalties),
                                                  int(most_ids), _stream()))


def sample_filter(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor) -> None:
    """Top-k, then top-p on softmax(logits / T), in place on [rows, vocab] float32 logits: what a rule removes
    becomes -inf.  top_k: int32 (-1: off), top_p: float32 (1: off); rows with temperature 0 are left alone."""
    _need(logits, "logits", torch.float32)
    rows, vocab = logits.shape
    _need(temperature, "temperature", torch.float32, (rows,))
    _need(top_k, "top_k", torch.int32, (rows,))
    _need(top_p, "top_p", torch.float32, (rows,))
    _check(library().somi_sample_filter(_ptr(logits), rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                        _stream()))


def probe_stream_shapes() -> list[str]:
    """Names of the launch shapes of the streaming read (lanes a workgroup, loads in flight a lane, workgroups a
    compute unit, cache hints): a measurement runs each and reports the best."""
    lib = library()
    lib.somi_probe_stream_shape_name.restype = ctypes.c_char_p
    return [lib.somi_probe_stream_shape_name(i).decode() for i in range(lib.somi_probe_stream_shapes())]


def probe_stream_read(buffer: torch.Tensor, shape: str | int = 0) -> None:
    """Streams ``buffer`` (any dtype, contiguous, a multiple of 16 bytes) once through the compute units in the named
    launch shape: the time of this call is what reading that many bytes costs on this machine."""
    _need(buffer, "probe buffer")
    size = buffer.numel() * buffer.element_size()
    lib = library()
    index = probe_stream_shapes().index(shape) if isinstance(shape, str) else int(shape)
    sink = torch.zeros((max(1, lib.somi_probe_stream_blocks(index)),), dtype=torch.int32, device=buffer.device)
    _check(lib.somi_probe_stream_read(_ptr(buffer), ctypes.c_int64(size), index, _ptr(sink), _stream()))


def probe_mfma(iters: int, device: torch.device | str = "cuda:0", dense: bool = True) -> float:
    """Runs ``iters`` rounds of four bfloat16 32 x 32 x 16 matrix instructions on every wavefront slot the launch
    fills (two per SIMD); returns the flops the launch does.  ``dense``: operands with every mantissa bit in use, as
    real activations and weights have them (the clock under matrix instructions goes with what the operands toggle);
    otherwise small integers."""
    sink = torch.zeros((1,), dtype=torch.float32, device=device)
    flops = ctypes.c_double(0.0)
    _check(library().somi_probe_mfma(int(iters), 1 if dense else 0, _ptr(sink), ctypes.byref(flops), _stream()))
    return float(flops.value)


ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def act_mul(gate_up: torch.Tensor, activation: str, block: int = 0) -> torch.Tensor:
    """act(gate) * up; ``activation``: one of ACTIVATIONS.  block == 0: gate_up = [gate columns | up columns]; block ==
    b: gate and up columns interleaved in blocks of b columns, as for :func:`silu_mul`."""
    _need(gate_up, "gate_up")
    if activation not in ACTIVATIONS:
        raise KernelError(f"act_mul: unknown activation {activation!r}; known: {sorted(ACTIVATIONS)}")
    n, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError(f"act_mul: width {two_i} is odd")
    out = torch.empty((n, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(library().somi_act_mul(_ptr(gate_up), _ptr(out), dtype_code(gate_up.dtype), n, two_i // 2,
                                  ACTIVATIONS[activation], int(block), _stream()))
    return out


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap), in place on float32 values."""
    _need(x, "logits", torch.float32)
    _check(library().somi_softcap(_ptr(x), ctypes.c_float(cap), ctypes.c_int64(x.numel()), _stream()))
    return x


def rope_kv_store_general(qkv: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                          inv_freq: torch.Tensor | None, rotary_dim: int, pairs: bool, nq: int, nk: int, dk: int,
                          nv: int, dv: int, k_cache: torch.Tensor | None, v_cache: torch.Tensor | None) -> None:
    """Rotate the nq query heads (in place) and the nk key heads of size dk of every row of ``qkv`` ([N, >= (nq + nk) dk
    + nv dv]: queries, keys, values side by side) and store keys and values in their pages.  ``pairs``: the rotation
    pairs channel 2j with 2j + 1 instead of j with j + rotary_dim / 2.  k cache: [pages, nk, page, dk]; v cache:
    [pages, nv, dv, page]; nk == nv == 0 rotates the queries only."""
    _need(qkv, "qkv")
    n = qkv.shape[0]
    if qkv.shape[1] < (nq + nk) * dk + nv * dv:
        raise KernelError(f"rope_kv_store_general: rows of {qkv.shape[1]} are narrower than {(nq + nk) * dk + nv * dv}")
    _need(positions, "positions", torch.int32, (n,))
    page_size = 0
    if nk or nv:
        _need(slots, "slot mapping", torch.int32, (n,))
        _need(k_cache, "k cache", qkv.dtype)
        _need(v_cache, "v cache", qkv.dtype)
        if k_cache.dim() != 4 or k_cache.shape[1] != nk or k_cache.shape[3] != dk:
            raise KernelError(f"rope_kv_store_general: k cache {tuple(k_cache.shape)} != [pages, {nk}, page, {dk}]")
        page_size = k_cache.shape[2]
        if tuple(v_cache.shape) != (k_cache.shape[0], nv, dv, page_size):
            raise KernelError(f"rope_kv_store_general: v cache {tuple(v_cache.shape)} != "
                              f"[{k_cache.shape[0]}, {nv}, {dv}, {page_size}]")
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
    _check(library().somi_rope_kv_store_general(
        _ptr(qkv), dtype_code(qkv.dtype), ctypes.c_int64(qkv.shape[1]), _ptr(positions), _ptr(slots), _ptr(inv_freq),
        int(rotary_dim), 1 if pairs else 0, n, nq, nk, dk, nv, dv, _ptr(k_cache if nk else None),
        _ptr(v_cache if nv else None), page_size, _stream()))


def diff_attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                         token_entry: torch.Tensor, positions: torch.Tensor, nq: int, window: int, keep_first: int,
                         scale: float, lam: float, eps: float, out_scale: float,
                         out: torch.Tensor | None = None, token_list: torch.Tensor | None = None) -> torch.Tensor:
    """Differential attention of the listed tokens (all when ``token_list`` is None) over their requests' pages with the
    plain float32 kernel: per head two softmax maps over the same values, a1 - lam * a2, divided by its root mean
    square over the head's value channels, times ``out_scale`` -> [N, nq * dv].  q: row t holds token t's 2 nq
    query maps of dk channels first; k cache: [pages, 2 nkv, page, dk]; v cache: [pages, nkv, dv, page].  A token
    sees the keys within ``window`` positions (0: all) and the first ``keep_first`` of its request."""
    _need(q, "q")
    n = q.shape[0]
    _need(k_cache, "k cache", q.dtype)
    _need(v_cache, "v cache", q.dtype)
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.shape[1] != 2 * v_cache.shape[1]:
        raise KernelError("diff_attention: caches must be k [pages, 2 kv_heads, page, dk] and v [pages, kv_heads, dv, page]")
    pages, nkv, dv, page_size = v_cache.shape
    dk = k_cache.shape[3]
    if k_cache.shape[0] != pages or k_cache.shape[2] != page_size:
        raise KernelError(f"diff_attention: k cache {tuple(k_cache.shape)} and v cache {tuple(v_cache.shape)} disagree")
    if q.shape[1] < 2 * nq * dk:
        raise KernelError("diff_attention: q rows are narrower than 2 * heads * dk")
    _need(block_table, "block table", torch.int32)
    _need(token_entry, "token entries", torch.int32, (n,))
    _need(positions, "positions", torch.int32, (n,))
    if out is None:
        out = torch.empty((n, nq * dv), dtype=q.dtype, device=q.device)
    _need(out, "attention out", q.dtype, (n, nq * dv))
    n_list = n
    if token_list is not None:
        _need(token_list, "token list", torch.int32)
        n_list = token_list.numel()
    _check(library().somi_diff_attention_plain(
        _ptr(q), dtype_code(q.dtype), ctypes.c_int64(q.shape[1]), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
        block_table.shape[1], _ptr(token_list), _ptr(token_entry), _ptr(positions), n_list, nq, nkv, dk, dv, page_size,
        int(window), int(keep_first), ctypes.c_float(scale), ctypes.c_float(lam), ctypes.c_float(eps),
        ctypes.c_float(out_scale), _ptr(out), _stream()))
    return out


def gla_alpha_(z: torch.Tensor, tau: float) -> torch.Tensor:
    """z <- sigmoid(z)^(1 / tau), in place on float32 values (through the logarithm: exp(-softplus(-z) / tau))."""
    _need(z, "decay sums", torch.float32)
    _check(library().somi_gla_alpha(_ptr(z), ctypes.c_float(tau), ctypes.c_int64(z.numel()), _stream()))
    return z


def gla_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alpha: torch.Tensor, entry_start: torch.Tensor,
             state_slots: torch.Tensor, state: torch.Tensor, q_scale: float, lanes: int = 0) -> torch.Tensor:
    """The recurrence S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T (q_t * q_scale) per head over the tokens of every entry,
    from and into ``state[state_slots[e]]`` ([slots, heads, dim, vdim] float32) -> o [N, heads, vdim] float32.
    q, k: [N, heads * dim] and v: [N, heads * vdim], views of one matrix (one row stride).  ``lanes``: lanes that share a
    column of the state (4 or 16; 0: the launcher chooses by the model's sizes and the device)."""
    slots, heads, dim, vdim = state.shape
    _need(state, "recurrent state", torch.float32)
    n = q.shape[0]
    for t, name, width in ((q, "q", heads * dim), (k, "k", heads * dim), (v, "v", heads * vdim)):
        if (not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != q.dtype or t.dim() != 2 or t.stride(1) != 1
                or t.stride(0) != q.stride(0) or tuple(t.shape) != (n, width)):
            raise KernelError(f"gla_scan: {name} must be [{n}, {width}] of {q.dtype} with the row stride of q")
    _need(alpha, "decays", torch.float32, (n, heads * dim))
    entries = state_slots.numel()
    _need(entry_start, "entry offsets", torch.int32, (entries + 1,))
    _need(state_slots, "state slots", torch.int32, (entries,))
    o = torch.empty((n, heads, vdim), dtype=torch.float32, device=q.device)
    _check(library().somi_gla_scan(_ptr(q), _ptr(k), _ptr(v), dtype_code(q.dtype), ctypes.c_int64(q.stride(0)),
                                   _ptr(alpha), _ptr(entry_start), _ptr(state_slots), _ptr(state), entries, heads, dim,
                                   vdim, ctypes.c_float(q_scale), int(lanes), _ptr(o), _stream()))
    return o


def gla_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor | None, eps: float,
                  out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """o / sqrt(mean(o^2) + eps) * weight * silu(gate) per head -> [N, heads * vdim] in the gate's dtype.  o: [N, heads,
    vdim] float32; weight: [vdim] float32; gate: [N, heads * vdim] (a view with a row stride of its own is fine), or None
    for a mixer without a gate (the result is then in ``out_dtype``)."""
    _need(o, "recurrence output", torch.float32)
    n, heads, vdim = o.shape
    _need(weight, "norm weight", torch.float32, (vdim,))
    if gate is None:
        if out_dtype is None:
            raise KernelError("gla_norm_gate: without a gate the result's dtype must be named")
        y = torch.empty((n, heads * vdim), dtype=out_dtype, device=o.device)
        _check(library().somi_gla_norm_gate(_ptr(o), _ptr(weight), None, dtype_code(out_dtype), ctypes.c_int64(0),
                                            ctypes.c_float(eps), _ptr(y), n, heads, vdim, _stream()))
        return y
    if (not isinstance(gate, torch.Tensor) or not gate.is_cuda or gate.dim() != 2 or gate.stride(1) != 1
            or tuple(gate.shape) != (n, heads * vdim)):
        raise KernelError(f"gla_norm_gate: the gate must be [{n}, {heads * vdim}] on the GPU with contiguous rows")
    y = torch.empty((n, heads * vdim), dtype=gate.dtype, device=o.device)
    _check(library().somi_gla_norm_gate(_ptr(o), _ptr(weight), _ptr(gate), dtype_code(gate.dtype),
                                        ctypes.c_int64(gate.stride(0)), ctypes.c_float(eps), _ptr(y), n, heads, vdim,
                                        _stream()))
    return y


def bounded_forget_(rows: torch.Tensor, width: int, bias: torch.Tensor, lower: torch.Tensor) -> torch.Tensor:
    """For a recurrence whose forget gate also decides what is written: rows [N, q (width) | z (width) | ...] of float32
    sums, in place q <- silu(q) and z <- 1 - f with f = lower + (1 - lower) sigmoid(z + bias); returns f [N, width]."""
    _need(rows, "projected rows", torch.float32)
    n = rows.shape[0]
    if rows.dim() != 2 or rows.shape[1] < 2 * width:
        raise KernelError(f"bounded_forget: rows of {tuple(rows.shape)} do not hold two runs of {width} channels")
    _need(bias, "gate bias", torch.float32, (width,))
    _need(lower, "lower bounds", torch.float32, (width,))
    decay = torch.empty((n, width), dtype=torch.float32, device=rows.device)
    _check(library().somi_bounded_forget(_ptr(rows), ctypes.c_int64(rows.stride(0)), _ptr(bias), _ptr(lower), _ptr(decay), n,
                                         int(width), _stream()))
    return decay


def diff_attention_mfma_supported(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor) -> bool:
    """The matrix-core kernel takes these operands: bfloat16, key and value sizes it is built for, pages of a multiple
    of 4 keys, rows aligned to 8 bytes."""
    wide = k_cache.shape[3] % 32 == 0          # such key sizes are read sixteen bytes at a time
    return (q.dtype == torch.bfloat16 and q.shape[1] % (8 if wide else 4) == 0 and q.data_ptr() % (16 if wide else 8) == 0
            and bool(library().somi_diff_attention_mfma_supported(k_cache.shape[3], v_cache.shape[2], k_cache.shape[2])))


def diff_attention_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, nq: int,
                        window: int, keep_first: int, scale: float, lam: float, eps: float, out_scale: float,
                        out: torch.Tensor, *, entry_start: torch.Tensor | None = None,
                        entry_first_position: torch.Tensor | None = None, entry_len: torch.Tensor | None = None,
                        max_entry_len: int = 0, token_list: torch.Tensor | None = None,
                        token_entry: torch.Tensor | None = None, positions: torch.Tensor | None = None) -> None:
    """Differential attention on the matrix cores into ``out`` ([N, nq * dv] bfloat16); operands as
    :func:`diff_attention_plain`.  Either the portions of a step (``entry_start`` [E + 1], ``entry_first_position`` [E],
    ``max_entry_len``; ``entry_len`` [E] stands for the offsets' own lengths, 0 leaves a portion out), or listed tokens
    (``token_entry`` and ``positions`` [N]; ``token_list`` names the tokens to run, None: all)."""
    _need(q, "q", torch.bfloat16)
    n = q.shape[0]
    _need(k_cache, "k cache", torch.bfloat16)
    _need(v_cache, "v cache", torch.bfloat16)
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.shape[1] != 2 * v_cache.shape[1]:
        raise KernelError("diff_attention: caches must be k [pages, 2 kv_heads, page, dk] and v [pages, kv_heads, dv, page]")
    pages, nkv, dv, page_size = v_cache.shape
    dk = k_cache.shape[3]
    if k_cache.shape[0] != pages or k_cache.shape[2] != page_size:
        raise KernelError(f"diff_attention: k cache {tuple(k_cache.shape)} and v cache {tuple(v_cache.shape)} disagree")
    if q.shape[1] < 2 * nq * dk:
        raise KernelError("diff_attention: q rows are narrower than 2 * heads * dk")
    _need(block_table, "block table", torch.int32)
    _need(out, "attention out", torch.bfloat16, (n, nq * dv))
    listed = entry_start is None
    entries, n_list = block_table.shape[0], 0
    if listed:
        _need(token_entry, "token entries", torch.int32, (n,))
        _need(positions, "positions", torch.int32, (n,))
        n_list = n
        if token_list is not None:
            _need(token_list, "token list", torch.int32)
            n_list = token_list.numel()
    else:
        _need(entry_start, "entry offsets", torch.int32, (entries + 1,))
        _need(entry_first_position, "entry first positions", torch.int32, (entries,))
        if entry_len is not None:
            _need(entry_len, "entry lengths", torch.int32, (entries,))
        if not 0 <= max_entry_len <= n:
            raise KernelError(f"diff_attention: longest portion {max_entry_len} does not fit {n} tokens")
    _check(library().somi_diff_attention_mfma(
        _ptr(q), ctypes.c_int64(q.shape[1]), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
        1 if listed else 0, _ptr(entry_start), _ptr(entry_first_position), _ptr(entry_len), entries, int(max_entry_len),
        _ptr(token_list), _ptr(token_entry), _ptr(positions), n_list, nq, nkv, dk, dv, page_size, int(window),
        int(keep_first), ctypes.c_float(scale), ctypes.c_float(lam), ctypes.c_float(eps), ctypes.c_float(out_scale),
        _ptr(out), _stream()))


# ------------------------------------------------------------------ the parallel block, its norm and its joins
def dynamic_tanh(h: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, alpha: torch.Tensor,
                 out_dtype: torch.dtype) -> torch.Tensor:
    """tanh(alpha * h) * weight + bias over float32 rows -> rows in ``out_dtype``; ``alpha`` is one float32 number on
    the device."""
    _need(h, "residual rows", torch.float32)
    n, hidden = h.shape
    _need(weight, "norm weight", torch.float32, (hidden,))
    _need(bias, "norm bias", torch.float32, (hidden,))
    _need(alpha, "norm alpha", torch.float32)
    if alpha.numel() != 1:
        raise KernelError("dynamic_tanh: alpha is one number")
    out = torch.empty((n, hidden), dtype=out_dtype, device=h.device)
    _check(library().somi_dyt(_ptr(h), _ptr(weight), _ptr(bias), _ptr(alpha), _ptr(out), dtype_code(out_dtype), n, hidden,
                              _stream()))
    return out


def scaled_add(h: torch.Tensor, a: torch.Tensor, b: torch.Tensor | None, mult: float,
               copy_dtype: torch.dtype | None = None) -> torch.Tensor | None:
    """h += mult * (a + b) in place on float32 rows (``b`` may be None); with ``copy_dtype`` the new rows are also
    returned in that dtype."""
    _need(h, "residual rows", torch.float32)
    _need(a, "delta", torch.float32, tuple(h.shape))
    if b is not None:
        _need(b, "second delta", torch.float32, tuple(h.shape))
    copy = torch.empty(h.shape, dtype=copy_dtype, device=h.device) if copy_dtype is not None else None
    _check(library().somi_scaled_add(_ptr(h), _ptr(a), _ptr(b), ctypes.c_float(mult), _ptr(copy),
                                     dtype_code(copy_dtype) if copy_dtype is not None else 0, ctypes.c_int64(h.numel()),
                                     _stream()))
    return copy


def normed_pair_mean(left: torch.Tensor, right: torch.Tensor, left_weight: torch.Tensor, right_weight: torch.Tensor,
                     eps: float) -> torch.Tensor:
    """(left / rms(left) * left_weight + right / rms(right) * right_weight) / 2 per row -> float32."""
    _need(left, "left rows")
    n, width = left.shape
    _need(right, "right rows", left.dtype, (n, width))
    _need(left_weight, "left weight", torch.float32, (width,))
    _need(right_weight, "right weight", torch.float32, (width,))
    out = torch.empty((n, width), dtype=torch.float32, device=left.device)
    _check(library().somi_normed_pair_mean(_ptr(left), _ptr(right), dtype_code(left.dtype), _ptr(left_weight),
                                           _ptr(right_weight), ctypes.c_float(eps), _ptr(out), n, width, _stream()))
    return out


def normed_add(h: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, mult: float,
               copy_dtype: torch.dtype | None = None) -> torch.Tensor | None:
    """h += mult * y / rms(y) * weight in place on float32 rows; with ``copy_dtype`` the new rows are also returned."""
    _need(h, "residual rows", torch.float32)
    n, width = h.shape
    _need(y, "rows to add", torch.float32, (n, width))
    _need(weight, "norm weight", torch.float32, (width,))
    copy = torch.empty(h.shape, dtype=copy_dtype, device=h.device) if copy_dtype is not None else None
    _check(library().somi_normed_add(_ptr(h), _ptr(y), _ptr(weight), ctypes.c_float(eps), ctypes.c_float(mult), _ptr(copy),
                                     dtype_code(copy_dtype) if copy_dtype is not None else 0, n, width, _stream()))
    return copy


def gated_table_rows(gate: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, offset: int) -> torch.Tensor:
    """gelu_tanh(gate[t, c]) * table[ids[t], offset + c] -> [N, dim] in the gate's dtype."""
    _need(gate, "gate rows")
    n, dim = gate.shape
    _need(table, "table", gate.dtype)
    _need(ids, "token ids", torch.int32, (n,))
    if table.dim() != 2 or offset < 0 or offset + dim > table.shape[1]:
        raise KernelError(f"gated_table_rows: columns {offset}..{offset + dim} do not fit a table of {tuple(table.shape)}")
    out = torch.empty_like(gate)
    _check(library().somi_gated_table_rows(_ptr(gate), _ptr(table), dtype_code(gate.dtype), _ptr(ids), table.shape[0],
                                           table.shape[1], int(offset), dim, _ptr(out), n, _stream()))
    return out


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """x *= factor in place on float32 values."""
    _need(x, "values", torch.float32)
    _check(library().somi_scale_f32(_ptr(x), ctypes.c_float(factor), ctypes.c_int64(x.numel()), _stream()))
    return x


def qk_norm_store(rows: torch.Tensor, slots: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor, eps: float,
                  nq: int, nkv: int, head_dim: int, tied: bool, k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    """RMS norm of a token's whole q projection (in place) and whole k projection (into the key pages), each with a
    weight of the projection's size; the value pages get the row's value heads or, ``tied``, the keys as projected.
    rows: [N, (nq + nkv (+ nkv)) * D]."""
    _need(rows, "q/k rows")
    n = rows.shape[0]
    if rows.shape[1] != (nq + (1 if tied else 2) * nkv) * head_dim:
        raise KernelError(f"qk_norm_store: rows of {rows.shape[1]} do not hold {nq} + {nkv} heads of {head_dim}")
    _need(slots, "slot mapping", torch.int32, (n,))
    _need(q_weight, "q norm weight", torch.float32, (nq * head_dim,))
    _need(k_weight, "k norm weight", torch.float32, (nkv * head_dim,))
    _need(k_cache, "k cache", rows.dtype)
    if k_cache.dim() != 4 or k_cache.shape[1] != nkv or k_cache.shape[3] != head_dim:
        raise KernelError(f"qk_norm_store: cache shape {tuple(k_cache.shape)} != [pages, {nkv}, page, {head_dim}]")
    _need(v_cache, "v cache", rows.dtype, _v_shape(k_cache))
    _check(library().somi_qk_norm_store(_ptr(rows), dtype_code(rows.dtype), ctypes.c_int64(rows.shape[1]), _ptr(slots),
                                        _ptr(q_weight), _ptr(k_weight), ctypes.c_float(eps), n, nq, nkv, head_dim,
                                        1 if tied else 0, _ptr(k_cache), _ptr(v_cache), k_cache.shape[2], _stream()))


# ------------------------------------------------------------------------------------------ the gated delta rule
DELTA_MAX_TAPS = 9


def delta_prepare(rows: torch.Tensor, ab: torch.Tensor, taps: torch.Tensor, conv_state: torch.Tensor, step,
                  a_log: torch.Tensor, dt_bias: torch.Tensor, groups: int, heads: int, dim: int, vdim: int
                  ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """What the recurrence reads, in float32: (qkv [N, 2 G dim + H vdim], beta [N, H], decay [N, H]).  rows: the tokens'
    projections [q | k | v | ...]; ab: [N, 2 H] float32 (beta's, then the decay's projection); taps: [C, taps] float32;
    conv_state: [slots, taps - 1, C] float32, read and then advanced by the step's entries."""
    _need(rows, "projected rows")
    n = rows.shape[0]
    channels = 2 * groups * dim + heads * vdim
    if rows.shape[1] < channels:
        raise KernelError(f"delta_prepare: rows of {rows.shape[1]} hold fewer than {channels} channels")
    _need(ab, "beta/decay projections", torch.float32, (n, 2 * heads))
    _need(taps, "convolution taps", torch.float32)
    if taps.dim() != 2 or taps.shape[0] != channels or not 1 <= taps.shape[1] <= DELTA_MAX_TAPS:
        raise KernelError(f"delta_prepare: taps {tuple(taps.shape)} != [{channels}, 1..{DELTA_MAX_TAPS}]")
    width = taps.shape[1]
    _need(conv_state, "convolution state", torch.float32)
    if tuple(conv_state.shape[1:]) != (max(width - 1, 1), channels):
        raise KernelError(f"delta_prepare: convolution state {tuple(conv_state.shape)} != [slots, {max(width - 1, 1)}, {channels}]")
    entries = step.state_slots.numel()
    _need(step.token_entry, "token entries", torch.int32, (n,))
    _need(step.entry_start, "entry offsets", torch.int32, (entries + 1,))
    _need(a_log, "decay rates", torch.float32, (heads,))
    _need(dt_bias, "decay biases", torch.float32, (heads,))
    qkv = torch.empty((n, channels), dtype=torch.float32, device=rows.device)
    beta = torch.empty((n, heads), dtype=torch.float32, device=rows.device)
    decay = torch.empty((n, heads), dtype=torch.float32, device=rows.device)
    _check(library().somi_delta_prepare(
        _ptr(rows), dtype_code(rows.dtype), ctypes.c_int64(rows.stride(0)), _ptr(ab), _ptr(taps), width, _ptr(conv_state),
        _ptr(step.token_entry), _ptr(step.entry_start), _ptr(step.state_slots), _ptr(a_log), _ptr(dt_bias), n, entries,
        groups, heads, dim, vdim, _ptr(qkv), _ptr(beta), _ptr(decay), _stream()))
    return qkv, beta, decay


def delta_scan(qkv: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor, entry_start: torch.Tensor,
               state_slots: torch.Tensor, state: torch.Tensor, groups: int, lanes: int = 0) -> torch.Tensor:
    """The recurrence S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q per head over every entry's tokens, from
    and into ``state[state_slots[e]]`` ([slots, heads, dim, vdim] float32) -> o [N, heads, vdim] float32.  ``lanes``: lanes that
    share a column of the state (4 or 16; 0: the launcher chooses by the model's sizes and the device)."""
    _need(state, "recurrent state", torch.float32)
    _, heads, dim, vdim = state.shape
    n = qkv.shape[0]
    _need(qkv, "q/k/v", torch.float32, (n, 2 * groups * dim + heads * vdim))
    _need(beta, "beta", torch.float32, (n, heads))
    _need(decay, "decay", torch.float32, (n, heads))
    entries = state_slots.numel()
    _need(entry_start, "entry offsets", torch.int32, (entries + 1,))
    _need(state_slots, "state slots", torch.int32, (entries,))
    o = torch.empty((n, heads, vdim), dtype=torch.float32, device=qkv.device)
    _check(library().somi_delta_scan(_ptr(qkv), _ptr(beta), _ptr(decay), _ptr(entry_start), _ptr(state_slots), _ptr(state),
                                     entries, groups, heads, dim, vdim, int(lanes), _ptr(o), _stream()))
    return o


# ------------------------------------------------------------------------------------------ mixture of experts
MOE_TILE_ROWS = 16           # sorted rows of a tile of the plain products
MOE_MFMA_ROWS = 64           # ... of the matrix-core products
MOE_BIG_ROWS = 128           # ... and of the matrix-core products that stage the rows through LDS (experts with many rows)


MOE_FEW_ROWS = 16            # ... of the matrix-core products of steps of a few tokens (an expert's one or two rows)


def moe_tile_rows(pairs: int, experts: int, mfma: bool) -> int:
    """Rows of a tile for a step of ``pairs`` (token, expert) pairs: the plain products' where the matrix-core ones do
    not apply; else the small tile while an expert has a few rows on average, the large one once it has a middle
    tile's worth."""
    if not mfma:
        return MOE_TILE_ROWS
    if pairs <= experts * MOE_FEW_ROWS // 2:
        return MOE_FEW_ROWS
    return MOE_BIG_ROWS if pairs >= experts * MOE_MFMA_ROWS else MOE_MFMA_ROWS


def moe_mfma_supported(x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor) -> bool:
    """The matrix-core products take these operands: bfloat16, both K (the width and the experts' size) multiples of 8,
    rows aligned to 16 bytes."""
    return (x.dtype == torch.bfloat16 and gate_up.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and down.shape[2] % 8 == 0
            and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and gate_up.data_ptr() % 16 == 0 and down.data_ptr() % 16 == 0)


ROUTER_SCORES = {"softmax": 0, "sigmoid": 1}


def moe_route(x: torch.Tensor, router: torch.Tensor, top: int, groups: int, keep: int, scores: str = "softmax",
              normalize: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    """Chosen experts [N, top] int32 and their weights [N, top] float32: float32 scores (``scores``: the softmax over all
    experts, or each expert's own sigmoid), the ``keep`` best of ``groups`` runs of neighbouring experts, the ``top`` best
    experts of those; weights over their sum (``normalize``) or the scores as they are."""
    _need(x, "rows")
    n, width = x.shape
    _need(router, "router", torch.float32)
    if router.dim() != 2 or router.shape[1] != width:
        raise KernelError(f"moe_route: router {tuple(router.shape)} does not fit rows of {width}")
    if scores not in ROUTER_SCORES:
        raise KernelError(f"moe_route: unknown scores {scores!r}; known: {sorted(ROUTER_SCORES)}")
    chosen = torch.empty((n, top), dtype=torch.int32, device=x.device)
    weight = torch.empty((n, top), dtype=torch.float32, device=x.device)
    logits = torch.empty((n, router.shape[0]), dtype=torch.float32, device=x.device)     # the router's sums, if it tiles them
    _check(library().somi_moe_route(_ptr(x), dtype_code(x.dtype), ctypes.c_int64(x.stride(0)), _ptr(router), _ptr(logits), n,
                                    width, router.shape[0], int(top), int(groups), int(keep), ROUTER_SCORES[scores],
                                    1 if normalize else 0, _ptr(chosen), _ptr(weight), _stream()))
    return chosen, weight


def moe_align(chosen: torch.Tensor, experts: int, tile_rows: int = MOE_TILE_ROWS) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The (token, expert) pairs sorted by expert: (order [pairs] int32, offsets [experts + 1] int32, tiles [T, 3] int32
    = (expert or -1, first sorted row, rows) for row tiles of ``tile_rows``)."""
    _need(chosen, "chosen experts", torch.int32)
    pairs = chosen.numel()
    max_tiles = library().somi_moe_max_tiles(pairs, int(experts), int(tile_rows))
    order = torch.empty((pairs,), dtype=torch.int32, device=chosen.device)
    offsets = torch.empty((experts + 1,), dtype=torch.int32, device=chosen.device)
    tiles = torch.empty((max_tiles, 3), dtype=torch.int32, device=chosen.device)
    _check(library().somi_moe_align(_ptr(chosen), pairs, int(experts), int(tile_rows), max_tiles, _ptr(order), _ptr(offsets),
                                    _ptr(tiles), _stream()))
    return order, offsets, tiles


def moe_gate_up(x: torch.Tensor, gate_up: torch.Tensor, tiles: torch.Tensor, order: torch.Tensor, top: int,
                limit: float, alpha: float, shift: float, tile_rows: int = MOE_TILE_ROWS, mfma: bool = False,
                input_weight: torch.Tensor | None = None) -> torch.Tensor:
    """act[p] = glu(W_gate[e] x[t], W_up[e] x[t]) for the sorted pairs p = (t, e); gate_up: [experts, 2 F, K], gate rows
    first -> [pairs, F].  ``input_weight`` [pairs] float32: the pair's weight multiplies the expert's input (both float32
    sums are scaled by it before the unit)."""
    _need(x, "rows")
    _need(gate_up, "gate/up matrices", x.dtype)
    experts, two_f, k = gate_up.shape
    if x.shape[1] != k or two_f % 2:
        raise KernelError(f"moe_gate_up: matrices {tuple(gate_up.shape)} do not fit rows of {x.shape[1]}")
    pairs = order.numel()
    if input_weight is not None:
        _need(input_weight, "pair weights", torch.float32)
        if input_weight.numel() != pairs:
            raise KernelError(f"moe_gate_up: {input_weight.numel()} weights for {pairs} pairs")
    act = torch.empty((pairs, two_f // 2), dtype=x.dtype, device=x.device)
    if mfma:
        _check(library().somi_moe_product_mfma(_ptr(x), ctypes.c_int64(x.stride(0)), _ptr(gate_up), 1, _ptr(tiles), tiles.shape[0],
                                               int(tile_rows), _ptr(order), _ptr(input_weight), int(top), two_f // 2, k, ctypes.c_float(limit),
                                               ctypes.c_float(alpha), ctypes.c_float(shift), _ptr(act), _stream()))
        return act
    _check(library().somi_moe_product(_ptr(x), ctypes.c_int64(x.stride(0)), _ptr(gate_up), dtype_code(x.dtype), 1, _ptr(tiles),
                                      tiles.shape[0], _ptr(order), _ptr(input_weight), int(top), two_f // 2, k, ctypes.c_float(limit),
                                      ctypes.c_float(alpha), ctypes.c_float(shift), _ptr(act), _stream()))
    return act


def moe_down(act: torch.Tensor, down: torch.Tensor, tiles: torch.Tensor, order: torch.Tensor, weight: torch.Tensor | None,
             top: int, tile_rows: int = MOE_TILE_ROWS, mfma: bool = False) -> torch.Tensor:
    """y[pair] = weight[pair] * W_down[e] act[p] -> [pairs, width] float32, at the pairs' own places (``weight`` None: the
    products as they are)."""
    _need(act, "activations")
    _need(down, "down matrices", act.dtype)
    experts, width, k = down.shape
    if act.shape[1] != k:
        raise KernelError(f"moe_down: matrices {tuple(down.shape)} do not fit activations of {act.shape[1]}")
    if weight is not None:
        _need(weight, "pair weights", torch.float32)
    y = torch.empty((order.numel(), width), dtype=torch.float32, device=act.device)
    if mfma:
        _check(library().somi_moe_product_mfma(_ptr(act), ctypes.c_int64(act.stride(0)), _ptr(down), 0, _ptr(tiles), tiles.shape[0],
                                               int(tile_rows), _ptr(order), _ptr(weight), int(top), width, k, ctypes.c_float(0.0),
                                               ctypes.c_float(0.0), ctypes.c_float(0.0), _ptr(y), _stream()))
        return y
    _check(library().somi_moe_product(_ptr(act), ctypes.c_int64(act.stride(0)), _ptr(down), dtype_code(act.dtype), 0, _ptr(tiles),
                                      tiles.shape[0], _ptr(order), _ptr(weight), int(top), width, k, ctypes.c_float(0.0),
                                      ctypes.c_float(0.0), ctypes.c_float(0.0), _ptr(y), _stream()))
    return y


def moe_combine(y: torch.Tensor, top: int, shared: torch.Tensor | None) -> torch.Tensor:
    """out[t] = sum_j y[t * top + j] (+ shared[t]) -> [N, width] float32."""
    _need(y, "expert outputs", torch.float32)
    pairs, width = y.shape
    n = pairs // top
    if shared is not None:
        _need(shared, "shared expert rows", None, (n, width))
    out = torch.empty((n, width), dtype=torch.float32, device=y.device)
    _check(library().somi_moe_combine(_ptr(y), _ptr(shared), dtype_code(shared.dtype) if shared is not None else 0, n, int(top),
                                      width, _ptr(out), _stream()))
    return out


def clamped_glu(gate_up: torch.Tensor, limit: float, alpha: float, shift: float) -> torch.Tensor:
    """g' sigmoid(alpha g') (u' + shift) with g' = min(g, limit), u' = clamp(u, -limit, limit) on rows [g | u]."""
    _need(gate_up, "gate/up rows")
    n, two_f = gate_up.shape
    out = torch.empty((n, two_f // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(library().somi_clamped_glu(_ptr(gate_up), dtype_code(gate_up.dtype), n, two_f // 2, ctypes.c_float(limit),
                                      ctypes.c_float(alpha), ctypes.c_float(shift), _ptr(out), _stream()))
    return out


# ------------------------------------------------------------------ layer norm, the input convolution, normed powers
def layernorm(h: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """(h - mean) / sqrt(var + eps) * weight + bias over float32 rows -> rows in ``out_dtype``."""
    _need(h, "residual rows", torch.float32)
    n, width = h.shape
    _need(weight, "norm weight", torch.float32, (width,))
    _need(bias, "norm bias", torch.float32, (width,))
    out = torch.empty((n, width), dtype=out_dtype, device=h.device)
    _check(library().somi_layernorm(_ptr(h), _ptr(weight), _ptr(bias), ctypes.c_float(eps), _ptr(out), dtype_code(out_dtype),
                                    n, width, _stream()))
    return out


def layernorm_add(h: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float,
                  copy_dtype: torch.dtype | None = None) -> torch.Tensor | None:
    """h += layer_norm(y) * weight + bias in place on float32 rows; with ``copy_dtype`` the new rows are also returned in
    that dtype."""
    _need(h, "residual rows", torch.float32)
    n, width = h.shape
    _need(y, "rows to add", None, (n, width))
    _need(weight, "norm weight", torch.float32, (width,))
    _need(bias, "norm bias", torch.float32, (width,))
    copy = torch.empty(h.shape, dtype=copy_dtype, device=h.device) if copy_dtype is not None else None
    _check(library().somi_layernorm_add(_ptr(h), _ptr(y), dtype_code(y.dtype), _ptr(weight), _ptr(bias), ctypes.c_float(eps),
                                        _ptr(copy), dtype_code(copy_dtype) if copy_dtype is not None else 0, n, width,
                                        _stream()))
    return copy


CONV_MAX_TAPS = 17


def input_conv(h: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, step, out_dtype: torch.dtype) -> torch.Tensor:
    """h + conv(h) over time per channel -> [N, C] in ``out_dtype``.  h: [N, C] float32 rows of the step; taps: [C, taps]
    float32, the last tap on the current token; state: [slots, max(taps - 1, 1), C] float32, a request's last inputs,
    read and then advanced by the step's entries."""
    _need(h, "residual rows", torch.float32)
    n, channels = h.shape
    _need(taps, "convolution taps", torch.float32)
    if taps.dim() != 2 or taps.shape[0] != channels or not 1 <= taps.shape[1] <= CONV_MAX_TAPS:
        raise KernelError(f"input_conv: taps {tuple(taps.shape)} != [{channels}, 1..{CONV_MAX_TAPS}]")
    width = taps.shape[1]
    _need(state, "convolution state", torch.float32)
    if tuple(state.shape[1:]) != (max(width - 1, 1), channels):
        raise KernelError(f"input_conv: state {tuple(state.shape)} != [slots, {max(width - 1, 1)}, {channels}]")
    entries = step.state_slots.numel()
    _need(step.token_entry, "token entries", torch.int32, (n,))
    _need(step.entry_start, "entry offsets", torch.int32, (entries + 1,))
    out = torch.empty((n, channels), dtype=out_dtype, device=h.device)
    _check(library().somi_input_conv(_ptr(h), _ptr(taps), width, _ptr(state), _ptr(step.token_entry), _ptr(step.entry_start),
                                     _ptr(step.state_slots), n, entries, channels, _ptr(out), dtype_code(out_dtype),
                                     _stream()))
    return out


def poly_norm(z: torch.Tensor, coefficients: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e per row with N the division by the row's root mean square; z: [N, F] float32;
    coefficients: (a, b, c, e) float32 on the device."""
    _need(z, "rows", torch.float32)
    _need(coefficients, "coefficients", torch.float32, (4,))
    out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
    _check(library().somi_poly_norm(_ptr(z), _ptr(coefficients), ctypes.c_float(eps), _ptr(out), dtype_code(out_dtype),
                                    z.shape[0], z.shape[1], _stream()))
    return out


# ------------------------------------------------------------------------------------------ attention over a latent
def head_linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[t, h, :] = weight[h] x[t, h, :].  x: [N, heads, K] (a view whose last dimension is contiguous); weight:
    [heads, n_out, K]; out: [N, heads, n_out], likewise a view if given."""
    heads, n_out, k = weight.shape
    _need(weight, "per-head matrices", x.dtype)
    if not x.is_cuda or x.dim() != 3 or x.shape[1] != heads or x.shape[2] != k or x.stride(2) != 1:
        raise KernelError(f"head_linear: rows {tuple(x.shape)} do not fit matrices {tuple(weight.shape)}")
    n = x.shape[0]
    if out is None:
        out = torch.empty((n, heads, n_out), dtype=x.dtype, device=x.device)
    if out.dtype != x.dtype or tuple(out.shape) != (n, heads, n_out) or out.stride(2) != 1:
        raise KernelError(f"head_linear: the result must be [{n}, {heads}, {n_out}] of {x.dtype}")
    _check(library().somi_head_linear(_ptr(x), ctypes.c_int64(x.stride(0)), ctypes.c_int64(x.stride(1)), _ptr(weight),
                                      dtype_code(x.dtype), n, heads, n_out, k, _ptr(out), ctypes.c_int64(out.stride(0)),
                                      ctypes.c_int64(out.stride(1)), _stream()))
    return out


PAIRINGS = {"half": 0, "neighbours": 1}      # which channels of a rotation turn together: i with i + dims / 2, or 2i with 2i + 1


def pairing_code(pairing: str) -> int:
    if pairing not in PAIRINGS:
        raise KernelError(f"unknown pairing {pairing!r}; known: {sorted(PAIRINGS)}")
    return PAIRINGS[pairing]


def latent_prepare(rows: torch.Tensor, q_rank: int, rank: int, rot: int, q_weight: torch.Tensor | None,
                   c_weight: torch.Tensor | None, eps: float, inv_freq: torch.Tensor | None, rot_dims: int, amplitude: float,
                   positions: torch.Tensor, slots: torch.Tensor | None, latent: torch.Tensor | None,
                   out_dtype: torch.dtype, latent_t: torch.Tensor | None = None, pairing: str = "half") -> torch.Tensor:
    """From float32 rows [query latent (q_rank) | latent as projected (rank) | shared key part (rot)]: the RMS-normed
    query latent -> [N, q_rank] in ``out_dtype`` (without ``q_weight`` the first ``q_rank`` values are the queries
    themselves and are only rounded); and, with ``latent`` ([pages, page, rank + rot]), the RMS-normed
    latent and the rotated key part into the tokens' slots (``latent_t`` [pages, rank, page]: the latent once more,
    transposed inside its page)."""
    _need(rows, "projected rows", torch.float32)
    n = rows.shape[0]
    if q_weight is not None:
        _need(q_weight, "query latent's norm weight", torch.float32, (q_rank,))
    _need(positions, "positions", torch.int32, (n,))
    if latent is not None:
        _need(latent, "kept latents", out_dtype)
        if latent.dim() != 3 or latent.shape[2] != rank + rot:
            raise KernelError(f"latent_prepare: cache shape {tuple(latent.shape)} != [pages, page, {rank + rot}]")
        _need(c_weight, "latent's norm weight", torch.float32, (rank,))
        _need(slots, "slot mapping", torch.int32, (n,))
        if rot_dims:
            _need(inv_freq, "rotation frequencies", torch.float32, (rot_dims // 2,))
        if latent_t is not None:
            _need(latent_t, "transposed latents", out_dtype, (latent.shape[0], rank, latent.shape[1]))
    elif latent_t is not None:
        raise KernelError("latent_prepare: transposed pages without the pages")
    q_latent = torch.empty((n, q_rank), dtype=out_dtype, device=rows.device)
    _check(library().somi_latent_prepare(_ptr(rows), ctypes.c_int64(rows.stride(0)), n, int(q_rank), int(rank), int(rot),
                                         _ptr(q_weight), _ptr(c_weight), ctypes.c_float(eps), _ptr(inv_freq), int(rot_dims),
                                         ctypes.c_float(amplitude), pairing_code(pairing), _ptr(positions), _ptr(slots),
                                         _ptr(q_latent),
                                         _ptr(latent), _ptr(latent_t), latent.shape[1] if latent is not None else 0,
                                         dtype_code(out_dtype), _stream()))
    return q_latent


def latent_place(q: torch.Tensor, heads: int, dim: int, rot: int, rank: int, inv_freq: torch.Tensor | None, rot_dims: int,
                 amplitude: float, positions: torch.Tensor, queries: torch.Tensor, pairing: str = "half") -> None:
    """The rotated part of every head of q ([N, heads * (dim + rot)], head by head [dim | rot]; of the queries' type or
    float32, and possibly the first columns of wider rows) turned by its position and written to ``queries[t, h,
    rank:]`` ([N, heads, rank + rot])."""
    if not isinstance(q, torch.Tensor) or not q.is_cuda or q.dim() != 2 or q.stride(1) != 1 or q.shape[1] != heads * (dim + rot):
        raise KernelError(f"latent_place: projected queries must be rows of {heads * (dim + rot)} values on the GPU")
    if q.dtype not in (torch.float32, queries.dtype):
        raise KernelError(f"latent_place: projected queries are float32 or {queries.dtype}, got {q.dtype}")
    _need(queries, "query rows", None, (q.shape[0], heads, rank + rot))
    _need(positions, "positions", torch.int32, (q.shape[0],))
    if rot_dims:
        _need(inv_freq, "rotation frequencies", torch.float32, (rot_dims // 2,))
    _check(library().somi_latent_place(_ptr(q), dtype_code(q.dtype), ctypes.c_int64(q.stride(0)), dtype_code(queries.dtype),
                                       q.shape[0], int(heads), int(dim), int(rot), int(rank),
                                       _ptr(inv_freq), int(rot_dims), ctypes.c_float(amplitude), pairing_code(pairing),
                                       _ptr(positions), _ptr(queries), _stream()))


def latent_attention_plain(queries: torch.Tensor, latent: torch.Tensor, block_table: torch.Tensor, token_entry: torch.Tensor,
                           positions: torch.Tensor, rank: int, scale: float, sink: torch.Tensor | None,
                           window: int = 0) -> torch.Tensor:
    """Causal softmax attention with a sink over kept latents: queries [N, heads, rank + rot] against the rows of
    ``latent`` ([pages, page, rank + rot]) of each token's request up to its own position; the values are the rows' first
    ``rank`` channels -> [N, heads, rank].  ``sink`` None: a softmax over the keys alone.  ``window``: how many keys a
    token sees, itself included (0: all)."""
    _need(queries, "query rows")
    n, heads, width = queries.shape
    _need(latent, "kept latents", queries.dtype)
    if latent.dim() != 3 or latent.shape[2] != width or not 0 < rank <= width:
        raise KernelError(f"latent_attention: cache {tuple(latent.shape)} does not fit queries of {width} (rank {rank})")
    _need(block_table, "block table", torch.int32)
    _need(token_entry, "token entries", torch.int32, (n,))
    _need(positions, "positions", torch.int32, (n,))
    if sink is not None:
        _need(sink, "sinks", torch.float32, (heads,))
    if window < 0:
        raise KernelError(f"latent_attention: a window of {window} keys")
    out = torch.empty((n, heads, rank), dtype=queries.dtype, device=queries.device)
    _check(library().somi_latent_attention_plain(_ptr(queries), dtype_code(queries.dtype), _ptr(latent), _ptr(block_table),
                                                 block_table.shape[1], _ptr(token_entry), _ptr(positions), n, heads,
                                                 int(rank), width - int(rank), latent.shape[1], int(window),
                                                 ctypes.c_float(scale), _ptr(sink), _ptr(out), _stream()))
    return out


def latent_attention_mfma_supported(queries: torch.Tensor, latent: torch.Tensor, rank: int) -> bool:
    """The matrix-core kernel takes these operands: bfloat16, a latent and a whole row of multiples of 16 channels (up to
    512 and 576), pages of a power of two of at least 8 tokens."""
    return (queries.dtype == torch.bfloat16 and latent.dtype == torch.bfloat16
            and bool(library().somi_latent_attention_mfma_supported(int(rank), latent.shape[2] - int(rank), latent.shape[1])))


LATENT_SPLIT_KEYS = 64          # a key split of the matrix-core kernel is whole tiles of this many keys
LATENT_MAX_SPLITS = 64


def latent_attention_mfma(queries: torch.Tensor, latent: torch.Tensor, latent_t: torch.Tensor, block_table: torch.Tensor,
                          token_entry: torch.Tensor, positions: torch.Tensor, rank: int, scale: float,
                          sink: torch.Tensor | None, max_context: int, portions: bool = False, window: int = 0) -> torch.Tensor:
    """:func:`latent_attention_plain` on the matrix cores (bfloat16).  ``latent_t``: [pages, rank, page], the latents
    transposed inside their pages.  ``max_context``: the longest context of the step, known to the host; a step of few
    tokens splits every token's keys over several workgroups, so that the device is busy.  ``portions``: the step holds
    prompt portions: four consecutive tokens share a workgroup, so that it reads a tile of kept rows once for all of
    them (tokens of other requests in such a group are taken one after another)."""
    _need(queries, "query rows", torch.bfloat16)
    n, heads, width = queries.shape
    _need(latent, "kept latents", torch.bfloat16)
    if latent.dim() != 3 or latent.shape[2] != width or not 0 < rank <= width:
        raise KernelError(f"latent_attention: cache {tuple(latent.shape)} does not fit queries of {width} (rank {rank})")
    _need(latent_t, "transposed latents", torch.bfloat16, (latent.shape[0], rank, latent.shape[1]))
    _need(block_table, "block table", torch.int32)
    _need(token_entry, "token entries", torch.int32, (n,))
    _need(positions, "positions", torch.int32, (n,))
    if sink is not None:
        _need(sink, "sinks", torch.float32, (heads,))
    groups = n * ((heads + 15) // 16)
    seen = int(max_context) if window <= 0 else min(int(max_context), int(window) + LATENT_SPLIT_KEYS - 1)
    tiles = max(1, (seen + LATENT_SPLIT_KEYS - 1) // LATENT_SPLIT_KEYS)
    splits = 1 if portions else max(1, min(LATENT_MAX_SPLITS, tiles, (2 * compute_units()) // max(groups, 1)))
    out = torch.empty((n, heads, rank), dtype=torch.bfloat16, device=queries.device)
    part = torch.empty((n * heads * splits * (rank + 2),), dtype=torch.float32, device=queries.device) if splits > 1 else None
    _check(library().somi_latent_attention_mfma(_ptr(queries), _ptr(latent), _ptr(latent_t), _ptr(block_table),
                                                block_table.shape[1], _ptr(token_entry), _ptr(positions), n, heads,
                                                int(rank), width - int(rank), latent.shape[1], int(window),
                                                ctypes.c_float(scale), _ptr(sink), splits, 1 if portions else 0, _ptr(out),
                                                _ptr(part), _stream()))
    return out


# ------------------------------------------------------------------------------------------ several residual streams
HC_MAX_STREAMS = 8


def hc_step(lanes: torch.Tensor, *, y: torch.Tensor | None = None, mix: torch.Tensor | None = None,
            out_weights: torch.Tensor | None = None, read: bool = False, in_weights: torch.Tensor | None = None,
            norm_weight: torch.Tensor | None = None, eps: float = 0.0, out_dtype: torch.dtype = torch.float32,
            copies: int = 1) -> torch.Tensor | None:
    """What lies between two sublayers of a layer with several residual streams, in one launch.  ``lanes``: [S, N, W]
    float32, updated in place.  With ``y`` ([N, W], float32 or bfloat16): ``x_t <- sum_s mix[s, t] x_s + out_weights[t]
    y`` for all t at once.  With ``read``: returns ``sum_s in_weights[s] x_s`` of the new streams (weights of 1 without
    ``in_weights``), RMS-normed with ``norm_weight`` and ``eps`` if given, in ``out_dtype``, ``copies`` times over
    ([copies, N, W]; [N, W] for one copy)."""
    _need(lanes, "residual streams", torch.float32)
    if lanes.dim() != 3:
        raise KernelError(f"hc_step: the streams are [S, N, W], got {tuple(lanes.shape)}")
    streams, n, width = lanes.shape
    if y is not None:
        _need(y, "sublayer output", None, (n, width))
        _need(mix, "stream mix", torch.float32, (streams, streams))
        _need(out_weights, "stream output weights", torch.float32, (streams,))
    if in_weights is not None:
        _need(in_weights, "stream input weights", torch.float32, (streams,))
    if norm_weight is not None:
        _need(norm_weight, "norm weight", torch.float32, (width,))
    out = None
    if read:
        out = torch.empty((copies, n, width) if copies != 1 else (n, width), dtype=out_dtype, device=lanes.device)
    elif y is None:
        raise KernelError("hc_step: neither a write nor a read")
    _check(library().somi_hc_step(_ptr(lanes), streams, ctypes.c_int64(n), width, _ptr(mix), _ptr(out_weights), _ptr(y),
                                  dtype_code(y.dtype) if y is not None else 0, _ptr(in_weights), 1 if read else 0,
                                  _ptr(norm_weight), ctypes.c_float(eps), _ptr(out), dtype_code(out_dtype), int(copies),
                                  _stream()))
    return out


# ------------------------------------------------------------------------------------------ attention with mixed heads
def mixed_attention_store(rows: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                          inv_freq: torch.Tensor | None, rot_dims: int, pairing: str, value_freq: torch.Tensor | None,
                          value_pairing: str, heads: int, kv_heads: int, dim: int, vdim: int,
                          k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, out_dtype: torch.dtype) -> torch.Tensor:
    """From float32 rows [q (heads * dim) | k (kv_heads * dim) | v (kv_heads * vdim)] as projected: q with its first
    ``rot_dims`` channels a head rotated -> [N, heads * dim] in ``out_dtype``; k rotated likewise and v, rotated over all
    its channels with ``value_freq`` ([vdim / 2]) if given, into the tokens' slots of ``k_cache`` [pages, kv_heads, page,
    dim] and ``v_cache`` [pages, kv_heads, vdim, page] (transposed inside a page).  Without the caches the rows hold q only."""
    _need(rows, "projected rows", torch.float32)
    n = rows.shape[0]
    _need(positions, "positions", torch.int32, (n,))
    page = 0
    if k_cache is not None:
        _need(k_cache, "key pages", out_dtype)
        pages, page = k_cache.shape[0], k_cache.shape[2]
        if tuple(k_cache.shape) != (pages, kv_heads, page, dim):
            raise KernelError(f"mixed_attention_store: key pages {tuple(k_cache.shape)} != [pages, {kv_heads}, page, {dim}]")
        _need(v_cache, "value pages", out_dtype, (pages, kv_heads, vdim, page))
        _need(slots, "slot mapping", torch.int32, (n,))
    if rows.shape[1] != heads * dim + (kv_heads * (dim + vdim) if k_cache is not None else 0):
        raise KernelError(f"mixed_attention_store: rows of {rows.shape[1]} values do not hold the projections")
    if rot_dims:
        _need(inv_freq, "rotation frequencies", torch.float32, (rot_dims // 2,))
    if value_freq is not None:
        _need(value_freq, "value rotation frequencies", torch.float32, (vdim // 2,))
    q = torch.empty((n, heads * dim), dtype=out_dtype, device=rows.device)
    _check(library().somi_mixed_attention_store(_ptr(rows), ctypes.c_int64(rows.stride(0)), n, _ptr(positions), _ptr(slots),
                                                _ptr(inv_freq), int(rot_dims), pairing_code(pairing), _ptr(value_freq),
                                                pairing_code(value_pairing), int(heads), int(kv_heads), int(dim), int(vdim),
                                                _ptr(q), _ptr(k_cache), _ptr(v_cache), int(page), dtype_code(out_dtype),
                                                _stream()))
    return q


def mixed_attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                          token_entry: torch.Tensor, positions: torch.Tensor, heads: int, window: int, scale: float,
                          softcap: float, denominator_extra: float, talk: torch.Tensor | None,
                          value_freq: torch.Tensor | None, value_pairing: str = "half") -> torch.Tensor:
    """Attention of every token over its request's pages up to its own position (``window`` keys back, itself included;
    0: all): scores ``scale q . k``, capped smoothly at ``softcap`` if > 0; a softmax per head whose denominator also
    holds ``denominator_extra`` (0 or 1); the heads' weights mixed by ``talk`` ([heads, heads], to x from) if given; a
    head's mixed weights times the values of its own key/value head; with ``value_freq`` the result turned back by the
    query's position.  q: [N, heads * dim]; out: [N, heads * vdim]."""
    _need(q, "queries")
    n = q.shape[0]
    _need(k_cache, "key pages", q.dtype)
    pages, kv_heads, page, dim = k_cache.shape
    if q.shape[1] != heads * dim or heads % kv_heads:
        raise KernelError(f"mixed_attention: queries {tuple(q.shape)} do not fit {heads} heads over key pages {tuple(k_cache.shape)}")
    _need(v_cache, "value pages", q.dtype)
    if v_cache.dim() != 4 or tuple(v_cache.shape[:2]) != (pages, kv_heads) or v_cache.shape[3] != page:
        raise KernelError(f"mixed_attention: value pages {tuple(v_cache.shape)} do not fit key pages {tuple(k_cache.shape)}")
    vdim = v_cache.shape[2]
    _need(block_table, "block table", torch.int32)
    _need(token_entry, "token entries", torch.int32, (n,))
    _need(positions, "positions", torch.int32, (n,))
    if talk is not None:
        _need(talk, "head mix", torch.float32, (heads, heads))
    if value_freq is not None:
        _need(value_freq, "value rotation frequencies", torch.float32, (vdim // 2,))
    out = torch.empty((n, heads * vdim), dtype=q.dtype, device=q.device)
    _check(library().somi_mixed_attention_plain(_ptr(q), dtype_code(q.dtype), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                                block_table.shape[1], _ptr(token_entry), _ptr(positions), n, int(heads),
                                                kv_heads, dim, vdim, page, int(window), ctypes.c_float(scale),
                                                ctypes.c_float(softcap), ctypes.c_float(denominator_extra), _ptr(talk),
                                                _ptr(value_freq), pairing_code(value_pairing), _ptr(out), _stream()))
    return out


def mixed_attention_mfma_supported(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, heads: int) -> bool:
    """The matrix-core kernel takes these operands: bfloat16, at most 16 query heads a key/value head, key channels a
    multiple of 8 (up to 256), value channels a multiple of 16, pages of a multiple of 8 tokens, and sizes whose tiles
    fit a compute unit's LDS."""
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16 or q.data_ptr() % 16:
        return False
    return bool(library().somi_mixed_attention_mfma_supported(int(heads), k_cache.shape[1], k_cache.shape[3],
                                                              v_cache.shape[2], k_cache.shape[2]))


MIXED_SPLIT_KEYS = 64          # a key split of the matrix-core kernel holds at least this many keys
MIXED_MAX_SPLITS = 64


def mixed_attention_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                         token_entry: torch.Tensor, positions: torch.Tensor, heads: int, window: int, scale: float,
                         softcap: float, denominator_extra: float, talk: torch.Tensor | None,
                         value_freq: torch.Tensor | None, value_pairing: str = "half", portions: bool = False,
                         max_context: int = 0, group_tokens: int = 0) -> torch.Tensor:
    """:func:`mixed_attention_plain` on the matrix cores (bfloat16).  ``portions``: the step holds prompt portions, and
    consecutive tokens share a workgroup (as many as fill 16 query slots a key/value head), so that it reads a tile of
    keys once for all of them; otherwise a workgroup serves one token, and where the step's tokens are few a token's
    keys are dealt out to several workgroups (``max_context``: the longest context of the step, known to the host)."""
    _need(q, "queries", torch.bfloat16)
    n = q.shape[0]
    _need(k_cache, "key pages", torch.bfloat16)
    pages, kv_heads, page, dim = k_cache.shape
    if q.shape[1] != heads * dim or heads % kv_heads:
        raise KernelError(f"mixed_attention: queries {tuple(q.shape)} do not fit {heads} heads over key pages {tuple(k_cache.shape)}")
    _need(v_cache, "value pages", torch.bfloat16)
    if v_cache.dim() != 4 or tuple(v_cache.shape[:2]) != (pages, kv_heads) or v_cache.shape[3] != page:
        raise KernelError(f"mixed_attention: value pages {tuple(v_cache.shape)} do not fit key pages {tuple(k_cache.shape)}")
    vdim = v_cache.shape[2]
    _need(block_table, "block table", torch.int32)
    _need(token_entry, "token entries", torch.int32, (n,))
    _need(positions, "positions", torch.int32, (n,))
    if talk is not None:
        _need(talk, "head mix", torch.float32, (heads, heads))
    if value_freq is not None:
        _need(value_freq, "value rotation frequencies", torch.float32, (vdim // 2,))
    splits = 1
    if not portions and n > 0:
        seen = int(max_context) if window <= 0 else min(int(max_context), int(window) + 31)
        splits = max(1, min(MIXED_MAX_SPLITS, seen // MIXED_SPLIT_KEYS, (2 * compute_units()) // n))
    out = torch.empty((n, heads * vdim), dtype=torch.bfloat16, device=q.device)
    stats = part = None
    if splits > 1:
        stats = torch.empty((n * splits * heads * 2,), dtype=torch.float32, device=q.device)
        part = torch.empty((n * splits * heads * vdim,), dtype=torch.float32, device=q.device)
    _check(library().somi_mixed_attention_mfma(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
                                               _ptr(token_entry), _ptr(positions), n, int(heads), kv_heads, dim, vdim, page,
                                               int(window), ctypes.c_float(scale), ctypes.c_float(softcap),
                                               ctypes.c_float(denominator_extra), _ptr(talk), _ptr(value_freq),
                                               pairing_code(value_pairing), 1 if portions else 0, splits, _ptr(stats),
                                               _ptr(part), _ptr(out), int(group_tokens), _stream()))
    return out


# ------------------------------------------------------------------------------------------ activations and gates
def xielu(z: torch.Tensor, pq: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """softplus(p) z^2 + z / 2 for z > 0 and (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2 otherwise; z: float32; pq: the
    two stored numbers, float32 on the device."""
    _need(z, "rows", torch.float32)
    _need(pq, "activation numbers", torch.float32, (2,))
    out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
    _check(library().somi_xielu(_ptr(z), _ptr(pq), _ptr(out), dtype_code(out_dtype), ctypes.c_int64(z.numel()), _stream()))
    return out


def sigmoid_gate(x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """x * sigmoid(gate) element by element; x: [N, W]; gate: float32 [N, W], possibly columns of wider rows."""
    _need(x, "gated rows")
    n, width = x.shape
    if not gate.is_cuda or gate.dtype != torch.float32 or tuple(gate.shape) != (n, width) or gate.stride(1) != 1:
        raise KernelError(f"sigmoid_gate: the gate is float32 rows of {width} values on the GPU, got {tuple(gate.shape)} {gate.dtype}")
    out = torch.empty_like(x)
    _check(library().somi_sigmoid_gate(_ptr(x), dtype_code(x.dtype), _ptr(gate), ctypes.c_int64(gate.stride(0)), _ptr(out),
                                       ctypes.c_int64(n), width, _stream()))
    return out
