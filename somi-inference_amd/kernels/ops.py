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


def linear_skinny_swiglu(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """silu(x @ gate.T) * (x @ up.T) in one kernel for at most 64 bfloat16 rows.  weight: [2 I, K] with
    gate and up rows interleaved in blocks of 16."""
    _need(x, "linear input", torch.bfloat16)
    m, k = x.shape
    _need(weight, "gate_up weight", torch.bfloat16)
    if weight.shape[1] != k or weight.shape[0] % 32:
        raise KernelError(f"linear_skinny_swiglu: weight {tuple(weight.shape)} does not fit input width {k}")
    inter = weight.shape[0] // 2
    out = torch.empty((m, inter), dtype=x.dtype, device=x.device)
    _check(library().somi_linear_skinny_swiglu(_ptr(x), _ptr(weight), _ptr(out), dtype_code(x.dtype), m, inter, k,
                                               _stream()))
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


def linear_big(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, *, swiglu: bool = False,
               eps: float = 0.0, stats: torch.Tensor | None = None, tile: int = 0,
               out: torch.Tensor | None = None, split_k: bool = True) -> torch.Tensor:
    """s * (x @ weight.T) (+ bias) -> bfloat16 for any number of rows, on 256-row tiles of the matrix cores.
    With ``stats`` ([blocks, width >= M] partial sums of squares, from :func:`linear_big_residual` or
    :func:`linear_residual`) the rows are scaled by s = 1 / sqrt(stats.sum(0) / K + eps): the product of
    RMS-normed rows when x holds ``norm_weight * h``.  With ``swiglu`` weight is [2 I, K] with gate and up rows
    interleaved in blocks of 16 and the result is silu(s g) * (s u) -> [M, I].  ``tile``: 0 lets the launcher
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
                                     _ptr(bias), _ptr(out), m, n, k, _ptr(row_scale), 1 if swiglu else 0, int(tile),
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
                  bias: torch.Tensor | None = None, swiglu: bool = False, mid: bool = False) -> torch.Tensor:
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
                                                _ptr(weight), _ptr(bias), _ptr(out), m, n, k, 1 if swiglu else 0,
                                                _ptr(workspace), ctypes.c_int64(workspace.numel()), _stream()))
    else:
        _check(library().somi_linear_scaled(_ptr(x), ctypes.c_float(eps), _ptr(stats), stats.shape[0], _ptr(weight),
                                            _ptr(bias), _ptr(out), m, n, k, 1 if swiglu else 0, _stream()))
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
               out_dtype: torch.dtype | None = None, swiglu: bool = False) -> torch.Tensor:
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
                                     1 if swiglu else 0, _ptr(workspace), ctypes.c_int64(workspace.numel()), _stream()))
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
