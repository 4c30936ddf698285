"""Python face of the HIP kernels: one function per kernel, each checking on the
host that the operands have the shapes, types and layout that the kernel and its
grid assume, before anything is launched.  Tensors are torch tensors on the GPU;
torch is the allocator and gives the stream.
"""

from __future__ import annotations

import contextlib
import ctypes
import dataclasses
import json
import os
import warnings
from pathlib import Path

import torch

from .library import KernelError, call, library_path, load

__all__ = [
    "KernelError",
    "LIBRARY_PRODUCTS_TABLE",
    "PREFILL_TILE_TOKENS",
    "QueryTiles",
    "attention",
    "attention_calls",
    "forced_product",
    "hipblaslt_build",
    "library_product_bucket",
    "noting_library_products",
    "open_gemm_library",
    "prefers_skinny",
    "prepare_products",
    "product_calls",
    "query_tiles_host",
    "embedding_gather",
    "library_path",
    "linear",
    "linear_normed",
    "linear_silu_mul",
    "can_fuse_norm",
    "can_prepare_norm",
    "can_use_prepared_norm",
    "linear_norm_ahead",
    "linear_prepared",
    "can_accumulate",
    "load",
    "qk_norm_rope_append",
    "residual_add",
    "rmsnorm",
    "rope_table",
    "sample_rows",
    "silu_mul",
    "time_library_product",
]

_DTYPE_CODES = {torch.float32: 0, torch.bfloat16: 1}


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 storage, not {dtype}.") from None


def _check(tensor: torch.Tensor, name: str, *, dtype: torch.dtype | None = None, shape: tuple | None = None) -> None:
    if not isinstance(tensor, torch.Tensor):
        raise KernelError(f"{name} must be a tensor.")
    if not tensor.is_cuda:
        raise KernelError(f"{name} must live on the GPU (got {tensor.device}); there is no CPU path.")
    if not tensor.is_contiguous():
        raise KernelError(f"{name} must be contiguous.")
    if dtype is not None and tensor.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, not {tensor.dtype}.")
    if shape is not None and tuple(tensor.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, not {tuple(tensor.shape)}.")


def _ptr(tensor: torch.Tensor | None) -> int | None:
    return None if tensor is None else tensor.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream of the current device as a raw handle (the short way where
    torch offers it: this is called once per kernel)."""

    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def embedding_gather(token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """``out[t] = table[token_ids[t]]`` as float32 ``[N, hidden]`` (the residual stream)."""

    _check(token_ids, "token_ids", dtype=torch.int32)
    _check(table, "table")
    if token_ids.ndim != 1 or table.ndim != 2 or token_ids.numel() == 0:
        raise KernelError("embedding_gather takes token_ids [N>0] and table [vocab, hidden].")
    vocab, hidden = table.shape
    out = torch.empty((token_ids.numel(), hidden), dtype=torch.float32, device=table.device)
    call("ms_embedding_gather", _ptr(token_ids), _ptr(table), _ptr(out), token_ids.numel(), hidden, vocab,
         _code(table.dtype), _stream())
    return out


def rmsnorm(
    x: torch.Tensor,
    weight: torch.Tensor,
    eps: float,
    *,
    delta: torch.Tensor | None = None,
    rows: torch.Tensor | None = None,
    write_back: bool = False,
) -> torch.Tensor:
    """RMSNorm over the last dimension of ``x [n, dim]``.

    ``x`` is float32 (the residual stream) or of the weight's type.  With
    ``delta`` the norm is taken of ``x + delta``; ``write_back`` stores that sum
    into ``x``.  With ``rows`` (int32) output row ``r`` reads input row
    ``rows[r]``.  The output has the weight's type."""

    _check(weight, "weight")
    _check(x, "x")
    if x.ndim != 2 or weight.ndim != 1 or x.shape[1] != weight.numel():
        raise KernelError(f"rmsnorm: x {tuple(x.shape)} does not match weight {tuple(weight.shape)}.")
    if x.dtype != torch.float32 and x.dtype != weight.dtype:
        raise KernelError("rmsnorm: x must be float32 or of the weight's type.")
    n_in, dim = x.shape
    if delta is not None:
        _check(delta, "delta", dtype=weight.dtype, shape=(n_in, dim))
    if rows is not None:
        _check(rows, "rows", dtype=torch.int32)
        if rows.ndim != 1:
            raise KernelError("rmsnorm: rows must be one-dimensional.")
    n_out = n_in if rows is None else rows.numel()
    if n_out == 0:
        raise KernelError("rmsnorm: no rows.")
    out = torch.empty((n_out, dim), dtype=weight.dtype, device=x.device)
    call("ms_rmsnorm", _ptr(x), _ptr(delta), _ptr(weight), _ptr(out), _ptr(rows), n_out, dim, float(eps),
         int(x.dtype == torch.float32), int(write_back), _code(weight.dtype), _stream())
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> None:
    """``h += delta`` with ``h`` float32."""

    _check(h, "h", dtype=torch.float32)
    _check(delta, "delta", shape=tuple(h.shape))
    if h.ndim != 2 or h.numel() == 0:
        raise KernelError("residual_add takes h [n>0, dim>0].")
    call("ms_residual_add", _ptr(h), _ptr(delta), h.shape[0], h.shape[1], _code(delta.dtype), _stream())


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """cos and sin of ``float(position) * inv_freq`` in float32, ``[N, half]`` each:
    made once per step, read by every layer."""

    _check(positions, "positions", dtype=torch.int32)
    _check(inv_freq, "inv_freq", dtype=torch.float32)
    if positions.ndim != 1 or inv_freq.ndim != 1 or positions.numel() == 0 or inv_freq.numel() == 0:
        raise KernelError("rope_table takes positions [N>0] and inv_freq [half>0].")
    shape = (positions.numel(), inv_freq.numel())
    cos = torch.empty(shape, dtype=torch.float32, device=positions.device)
    sin = torch.empty(shape, dtype=torch.float32, device=positions.device)
    call("ms_rope_table", _ptr(positions), _ptr(inv_freq), _ptr(cos), _ptr(sin), shape[0], shape[1], _stream())
    return cos, sin


def qk_norm_rope_append(
    packed: torch.Tensor,
    *,
    num_q_heads: int,
    num_kv_heads: int,
    head_dim: int,
    q_weight: torch.Tensor | None,
    k_weight: torch.Tensor | None,
    eps: float,
    rope: tuple[torch.Tensor, torch.Tensor] | None,
    slot_mapping: torch.Tensor | None = None,
    key_pool: torch.Tensor | None = None,
    value_pool: torch.Tensor | None = None,
) -> torch.Tensor | None:
    """Per-head norm of q and k, rotation, and the cache write, in one kernel.

    ``packed [N, (num_q_heads + 2*num_kv_heads) * head_dim]`` holds q heads, then
    k heads, then v heads.  ``rope``: the (cos, sin) tables of :func:`rope_table` for
    these N tokens, or None for no rotation.  Returns q ``[N, num_q_heads, head_dim]`` (None when
    there are no q heads); with ``slot = page * block_size + offset`` from
    ``slot_mapping`` (int32), k goes to ``key_pool[page, kv_head, offset, :]`` and v,
    transposed, to ``value_pool[page, kv_head, :, offset]``."""

    _check(packed, "packed")
    heads = num_q_heads + 2 * num_kv_heads
    if packed.ndim != 2 or packed.shape[1] != heads * head_dim or packed.shape[0] == 0:
        raise KernelError(
            f"qk_norm_rope_append: packed {tuple(packed.shape)} is not [N, {heads} * {head_dim}]."
        )
    n = packed.shape[0]
    dtype = packed.dtype
    for name, weight in (("q_weight", q_weight), ("k_weight", k_weight)):
        if weight is not None:
            _check(weight, name, dtype=dtype, shape=(head_dim,))
    cos = sin = None
    if rope is not None:
        cos, sin = rope
        _check(cos, "rope cos", dtype=torch.float32, shape=(n, head_dim // 2))
        _check(sin, "rope sin", dtype=torch.float32, shape=(n, head_dim // 2))
    block_size = 0
    if num_kv_heads > 0:
        if slot_mapping is None or key_pool is None or value_pool is None:
            raise KernelError("qk_norm_rope_append: a cache write needs slot_mapping and both pools.")
        _check(slot_mapping, "slot_mapping", dtype=torch.int32, shape=(n,))
        _check(key_pool, "key_pool", dtype=dtype)
        if key_pool.ndim != 4 or key_pool.shape[1] != num_kv_heads or key_pool.shape[3] != head_dim:
            raise KernelError(
                f"qk_norm_rope_append: pool {tuple(key_pool.shape)} is not "
                f"[pages, {num_kv_heads}, block_size, {head_dim}]."
            )
        block_size = key_pool.shape[2]
        _check(value_pool, "value_pool", dtype=dtype, shape=_value_pool_shape(key_pool))
    q_out = None
    if num_q_heads > 0:
        q_out = torch.empty((n, num_q_heads, head_dim), dtype=dtype, device=packed.device)
    call("ms_qk_norm_rope_append", _ptr(packed), _ptr(q_weight), _ptr(k_weight), _ptr(cos), _ptr(sin),
         _ptr(slot_mapping), _ptr(q_out), _ptr(key_pool), _ptr(value_pool), n, num_q_heads, num_kv_heads,
         head_dim, block_size, float(eps), _code(dtype), _stream())
    return q_out


def _value_pool_shape(key_pool: torch.Tensor) -> tuple[int, ...]:
    pages, kv_heads, block_size, head_dim = key_pool.shape
    return (pages, kv_heads, head_dim, block_size)


# Tokens of one sequence that one workgroup of the tiled attention kernel serves.
PREFILL_TILE_TOKENS = 64


@dataclasses.dataclass
class QueryTiles:
    """The tokens after the single-token prefix of a batch, cut into tiles of at most
    ``PREFILL_TILE_TOKENS`` consecutive tokens of one sequence (what the tiled
    attention kernel walks)."""

    count: int
    seq: torch.Tensor       # int32 [count]: the tile's sequence (row of the block tables)
    token: torch.Tensor     # int32 [count]: index of the tile's first token in the batch
    length: torch.Tensor    # int32 [count]: 1..PREFILL_TILE_TOKENS
    first: torch.Tensor     # int32 [count]: position of the tile's first token; the others follow one by one
    by_keys: bool = False   # the tiles stand in the order of the keys they walk, fewest first


def query_tiles_host(query_lens, query_start, decode_prefix: int, first_positions, *, by_keys: bool = True):
    """The tiles of a batch as four lists (sequence, first token, length, position of the
    first token): every sequence after the first ``decode_prefix`` is cut into runs of at
    most ``PREFILL_TILE_TOKENS`` tokens.  ``first_positions``: the position of every
    sequence's first token of the step.  ``by_keys``: the tiles are put in the order of
    the keys they walk, fewest first (``QueryTiles.by_keys``): the kernel then hands the
    long ones out first and may give a workgroup a long and a short one."""

    tiles: list[tuple[int, int, int, int]] = []
    for index in range(decode_prefix, len(query_lens)):
        base, length, first = query_start[index], query_lens[index], first_positions[index]
        for start in range(0, length, PREFILL_TILE_TOKENS):
            count = min(PREFILL_TILE_TOKENS, length - start)
            tiles.append((first + start + count, index, base + start, count))
    if by_keys:
        tiles.sort()
    return [t[1] for t in tiles], [t[2] for t in tiles], [t[3] for t in tiles], [t[0] - t[3] for t in tiles]


# calls of attention() served by each kernel since the import; a bfloat16 call that no
# matrix-core kernel takes is served by the generic one, many times slower, and is
# reported once per geometry
attention_calls = {"decode": 0, "prefill": 0, "generic": 0}
_reported_fallbacks: set = set()


def _report_fallback(head_dim: int, block_size: int, reason: str) -> None:
    key = (head_dim, block_size, reason)
    if key not in _reported_fallbacks:
        _reported_fallbacks.add(key)
        warnings.warn(
            f"attention with head size {head_dim} and pages of {block_size} keys: {reason} "
            "(correct, but far slower than the matrix-core kernels; they take head sizes in steps of 16 "
            "up to 256 for single tokens, up to 128 for runs of tokens, and pages of a multiple of 16 keys).",
            RuntimeWarning, stacklevel=3,
        )


# Workgroups that the key-split attention aims to launch: two per compute unit, so that
# short batches still fill the chip (256 units on MI355X: 512).
_DECODE_MAX_SPLITS = 64
_decode_target_workgroups: int | None = None


def _decode_target() -> int:
    global _decode_target_workgroups
    if _decode_target_workgroups is None:
        _decode_target_workgroups = 2 * int(load().ms_device_compute_units())
    return _decode_target_workgroups


def decode_splits(num_tokens: int, num_kv_heads: int, group: int, max_context: int) -> int:
    """How many parts the keys of each row are cut into: enough workgroups to fill
    the chip, at least 160 keys per part (with shorter parts the kernel that joins
    them costs more than the parts save: measured with one and two rows at a context
    of 2,100)."""

    rows = num_tokens * num_kv_heads * ((group + 15) // 16)
    by_chip = -(-_decode_target() // rows)
    by_keys = max(1, max_context // 160)
    return max(1, min(by_chip, by_keys, _DECODE_MAX_SPLITS))


def attention(
    q: torch.Tensor,
    key_pool: torch.Tensor,
    value_pool: torch.Tensor,
    *,
    block_table: torch.Tensor,
    seq_of_token: torch.Tensor,
    positions: torch.Tensor,
    scale: float,
    window: int | None = None,
    decode_prefix: int = 0,
    tiles=None,
    max_context: int | None = None,
    splits: int | None = None,
) -> torch.Tensor:
    """Causal attention of ``q [N, heads, head_dim]`` over the paged cache
    (``key_pool [pages, kv_heads, block_size, head_dim]``, ``value_pool [pages,
    kv_heads, head_dim, block_size]``).

    Token ``t`` belongs to sequence ``seq_of_token[t]``, stands at absolute
    position ``positions[t]`` and sees the keys ``lo..positions[t]`` of that
    sequence through ``block_table [S, max_blocks]`` (int32), ``lo`` being 0 or
    ``positions[t] - window + 1``.  The caller guarantees that every page the
    table names for those keys lies inside the pool.

    float32 runs the generic kernel, whose result for a position is bit-identical
    for any batch.  bfloat16 runs the matrix-core kernels where they take the
    geometry: the first ``decode_prefix`` tokens are single tokens of their
    sequences and go to the key-split kernel (``max_context``, the largest
    position + 1, sizes the split; ``splits`` overrides it); the other tokens go,
    cut into ``tiles`` (a ``QueryTiles``: at most 64 consecutive tokens of one
    sequence each), to the tiled kernel.  Without ``tiles`` and ``decode_prefix``
    the generic kernel serves every token."""

    _check(q, "q")
    if q.ndim != 3 or q.shape[0] == 0:
        raise KernelError("attention: q must be [N>0, heads, head_dim].")
    n, heads, head_dim = q.shape
    _check(key_pool, "key_pool", dtype=q.dtype)
    if key_pool.ndim != 4 or key_pool.shape[3] != head_dim:
        raise KernelError(f"attention: pool {tuple(key_pool.shape)} is not [pages, kv_heads, block_size, {head_dim}].")
    _check(value_pool, "value_pool", dtype=q.dtype, shape=_value_pool_shape(key_pool))
    _, kv_heads, block_size, _ = key_pool.shape
    if heads % kv_heads != 0:
        raise KernelError(f"attention: {heads} query heads are not a multiple of {kv_heads} kv heads.")
    _check(block_table, "block_table", dtype=torch.int32)
    if block_table.ndim != 2 or block_table.shape[1] == 0:
        raise KernelError("attention: block_table must be [S, max_blocks>0].")
    _check(seq_of_token, "seq_of_token", dtype=torch.int32, shape=(n,))
    _check(positions, "positions", dtype=torch.int32, shape=(n,))
    window = 0 if window is None else int(window)
    if window < 0:
        raise KernelError("attention: window must be positive or None.")
    if not 0 <= decode_prefix <= n:
        raise KernelError("attention: decode_prefix lies outside the batch.")
    out = torch.empty_like(q)
    lib = load()
    max_blocks = block_table.shape[1]
    covered = decode_prefix == n or (tiles is not None and tiles.count > 0)
    if q.dtype == torch.bfloat16 and covered and lib.ms_attention_decode_supported(head_dim, block_size):
        tiled = lib.ms_attention_prefill_supported(head_dim, block_size)
        single = decode_prefix if tiled else n          # without the tiled kernel every token is served as a single one
        if not tiled and decode_prefix < n:
            _report_fallback(head_dim, block_size, "runs of tokens are served token by token by the single-token kernel")
        if single > 0:
            attention_calls["decode"] += 1
            if splits is None:
                splits = decode_splits(single, kv_heads, heads // kv_heads, max_context or max_blocks * block_size)
            partial_o = partial_ml = None
            if splits > 1:
                partial_o = torch.empty((single, heads, splits, head_dim), dtype=torch.float32, device=q.device)
                partial_ml = torch.empty((single, heads, splits, 2), dtype=torch.float32, device=q.device)
            call("ms_attention_decode", _ptr(q), _ptr(key_pool), _ptr(value_pool), _ptr(block_table),
                 _ptr(seq_of_token), _ptr(positions), _ptr(out), _ptr(partial_o), _ptr(partial_ml), single, heads,
                 kv_heads, head_dim, block_size, max_blocks, float(scale), window, int(splits), _stream())
        if tiled and decode_prefix < n:
            attention_calls["prefill"] += 1
            for name in ("seq", "token", "length", "first"):
                _check(getattr(tiles, name), f"tiles.{name}", dtype=torch.int32, shape=(tiles.count,))
            call("ms_attention_prefill", _ptr(q), _ptr(key_pool), _ptr(value_pool), _ptr(block_table),
                 _ptr(tiles.seq), _ptr(tiles.token), _ptr(tiles.length), _ptr(tiles.first), _ptr(out), tiles.count, int(tiles.by_keys),
                 heads, kv_heads, head_dim, block_size, max_blocks, float(scale), window, _stream())
        return out
    attention_calls["generic"] += 1
    if q.dtype == torch.bfloat16 and not lib.ms_attention_decode_supported(head_dim, block_size):
        _report_fallback(head_dim, block_size, "no matrix-core kernel takes this geometry, the generic kernel serves it")
    call("ms_attention_generic", _ptr(q), _ptr(key_pool), _ptr(value_pool), _ptr(block_table), _ptr(seq_of_token),
         _ptr(positions), _ptr(out), n, heads, kv_heads, head_dim, block_size, max_blocks, float(scale),
         window, _code(q.dtype), _stream())
    return out


_EPILOGUE_BF16, _EPILOGUE_F32, _EPILOGUE_ADD_F32, _EPILOGUE_SILU_MUL = 0, 1, 2, 3
# This library's product takes up to SKINNY_KERNEL_ROWS rows; the norm as its prologue
# up to SKINNY_MAX_ROWS rows.
SKINNY_MAX_ROWS = 16
SKINNY_KERNEL_ROWS = 64
# The largest matrices whose product takes the norm as its prologue (plain, and with the
# gated activation as its epilogue); beyond them the norm is a kernel of its own.
FUSED_NORM_BYTES = 64 << 20
FUSED_NORM_GATED_BYTES = 48 << 20


_GEMM_WORKSPACE_BYTES = 64 << 20
_gemm_workspaces: dict[int, torch.Tensor] = {}
_gemm_library_opened = False
# The table of pinned solutions: for a matrix [n, k], an output type and a bucket of
# row counts, the solution of hipBLASLt that was fastest when the table was measured
# (``python -m miniserve_amd.ops.tune``).  It holds for one build of the library, which
# the table names; with another build, or for a shape the table lacks, the library's own
# first choice runs.  Either way nothing is timed in a serving process, and the same
# model gives the same 32-bit sums in every process.
LIBRARY_PRODUCTS_TABLE = Path(__file__).resolve().parent / "library_products.json"


def _loaded_hipblaslt() -> str:
    """Path of the hipBLASLt that this process has loaded (torch's): the product for
    many rows binds to that copy, not to a second one."""

    with open("/proc/self/maps") as maps:
        for line in maps:
            path = line.rsplit(" ", 1)[-1].strip()
            if "libhipblaslt" in path.rsplit("/", 1)[-1]:
                return path
    raise KernelError("no hipBLASLt is loaded in this process (torch on ROCm brings it).")


def hipblaslt_build(path: str) -> str:
    """What names a build of the library in the table of pins: its file's name and size."""

    real = os.path.realpath(path)
    return f"{os.path.basename(real)}:{os.path.getsize(real)}"


def open_gemm_library() -> str:
    """Binds the product for many rows to the process's hipBLASLt and sets the pinned
    solutions; returns the library's path.  Done once."""

    global _gemm_library_opened
    path = _loaded_hipblaslt()
    if not _gemm_library_opened:
        call("ms_gemm_library_open", path.encode())
        if LIBRARY_PRODUCTS_TABLE.is_file():
            table = json.loads(LIBRARY_PRODUCTS_TABLE.read_text())
            if table.get("library") == hipblaslt_build(path):
                for n, k, out_float, bucket, solution in table.get("pins", ()):
                    call("ms_gemm_library_pin", int(n), int(k), int(out_float), int(bucket), int(solution))
        _gemm_library_opened = True
    return path


def _gemm_workspace(device: torch.device) -> torch.Tensor:
    index = device.index if device.index is not None else torch.cuda.current_device()
    workspace = _gemm_workspaces.get(index)
    if workspace is None:
        workspace = _gemm_workspaces[index] = torch.empty(_GEMM_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return workspace


def prepare_products(device: torch.device | str) -> None:
    """What the matrix products allocate and set up once per process and device (the
    library's binding, its pins and its workspace), done now: an engine calls this before
    it sizes its cache pool from the free memory, so that no step allocates for them."""

    open_gemm_library()
    _gemm_workspace(torch.device(device))


def _library_product(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, accumulate: bool) -> None:
    """``out (+)= x @ weight^T`` through hipBLASLt; bfloat16 in, bfloat16 or float32 out."""

    if not _gemm_library_opened:
        open_gemm_library()
    workspace = _gemm_workspace(x.device)
    m, k = x.shape
    product_calls["library"] += 1
    if _noted_library_products is not None:
        _noted_library_products.add((m, weight.shape[0], k, int(out.dtype == torch.float32)))
    call("ms_gemm_library", _ptr(x), _ptr(weight), _ptr(out), m, weight.shape[0], k, int(out.dtype == torch.float32),
         int(accumulate), _ptr(workspace), _GEMM_WORKSPACE_BYTES, _stream())


_noted_library_products: set | None = None


@contextlib.contextmanager
def noting_library_products(into: set):
    """Inside the block every product that hipBLASLt serves adds ``(m, n, k, out is
    float32)`` to ``into`` (for the tool that measures the table of pins)."""

    global _noted_library_products
    previous, _noted_library_products = _noted_library_products, into
    try:
        yield into
    finally:
        _noted_library_products = previous


def time_library_product(m: int, n: int, k: int, *, out_float32: bool = False, flush: torch.Tensor | None = None,
                         device: torch.device | str = "cuda:0") -> list[tuple[int, float]]:
    """For the tool that measures the table of pins: (solution, milliseconds) of every
    candidate that hipBLASLt offers for ``x [m, k] @ w [n, k]^T``, each timed from
    flushed caches (``flush``: a tensor larger than the caches, overwritten before every
    run); 0 ms marks a candidate that did not run."""

    open_gemm_library()
    device = torch.device(device)
    x = torch.randn((m, k), device=device).to(torch.bfloat16)
    w = (torch.randn((n, k), device=device) * 0.02).to(torch.bfloat16)
    out = torch.empty((m, n), dtype=torch.float32 if out_float32 else torch.bfloat16, device=device)
    workspace = _gemm_workspace(device)
    capacity = 16
    solutions = (ctypes.c_int * capacity)()
    milliseconds = (ctypes.c_float * capacity)()
    count = ctypes.c_int(0)
    call("ms_gemm_library_time", _ptr(x), _ptr(w), _ptr(out), m, n, k, int(out_float32), _ptr(workspace),
         _GEMM_WORKSPACE_BYTES, _ptr(flush), 0 if flush is None else flush.numel() * flush.element_size(),
         solutions, milliseconds, capacity, ctypes.byref(count), _stream())
    return [(int(solutions[i]), float(milliseconds[i])) for i in range(count.value)]


def library_product_bucket(m: int) -> int:
    """The bucket of row counts that shares one pinned solution."""

    return int(load().ms_gemm_library_bucket(int(m)))


# Which of the two products serves a call that both can serve is a fixed rule of the
# shape, so that the same model gives the same logits in every run and in recorded and
# eager steps alike.  The rule is fitted to timings on MI355X of both products inside
# recorded graphs over matrices that no cache holds (as a decode step meets its
# weights), for the matrices of the 0.6B, 8B and 32B sizes and 1 to 64 rows: this
# library's product streams a small matrix faster, the more so the fewer the rows;
# hipBLASLt, with the fastest of its candidates for the shape, streams a large one
# faster; the fused forms (norm as prologue, activation as epilogue) save one or two
# kernels of some 5 us each.  Which of its candidates the library runs is fixed as
# well (the table of pins above, else its first choice), so two processes that run the
# same model on the same steps give the same bits.
_MIB = 1 << 20
product_calls = {"skinny": 0, "library": 0}     # calls served by each since the import
_forced_product: str | None = None


@contextlib.contextmanager
def forced_product(which: str | None):
    """Inside the block every product that both kernels can serve goes to ``which``
    (``"skinny"``: this library's, up to ``SKINNY_KERNEL_ROWS`` rows; ``"library"``:
    hipBLASLt, and nothing is fused into a product) instead of following the rule.
    For tests and measurements."""

    global _forced_product
    if which not in (None, "skinny", "library"):
        raise ValueError("forced_product takes 'skinny', 'library' or None.")
    previous, _forced_product = _forced_product, which
    try:
        yield
    finally:
        _forced_product = previous


def prefers_skinny(m: int, n: int, k: int, *, fused: bool = False) -> bool:
    """The rule: whether this library's product is taken for ``x [m, k] @ w [n, k]^T``
    (``fused``: with a norm or an activation that would otherwise be kernels of their own)."""

    if m > SKINNY_KERNEL_ROWS:
        return False
    if _forced_product is not None:
        return _forced_product == "skinny"
    size = 2 * n * k
    if size <= 16 * _MIB:                       # the matrices of a small model
        return True
    if m > SKINNY_MAX_ROWS:
        return False
    if size <= 40 * _MIB:                       # middle sizes
        return True
    if n >= 65536:                              # a head: many short rows
        return m <= 8
    return fused and size <= 256 * _MIB


def _skinny_is_faster(x: torch.Tensor, weight: torch.Tensor, gated: bool) -> bool:
    m, k = x.shape
    n = weight.shape[0]
    epilogue = _EPILOGUE_SILU_MUL if gated else _EPILOGUE_BF16
    if m > SKINNY_KERNEL_ROWS or not load().ms_gemm_skinny_supported(m, n, k, epilogue):
        return False
    return prefers_skinny(m, n, k, fused=gated)


def _skinny(x: torch.Tensor, weight: torch.Tensor, epilogue: int, out: torch.Tensor) -> None:
    m, k = x.shape
    n = weight.shape[0]
    bf16_out = out if out.dtype == torch.bfloat16 else None
    f32_out = out if out.dtype == torch.float32 else None
    product_calls["skinny"] += 1
    call("ms_gemm_skinny", _ptr(x), _ptr(weight), _ptr(bf16_out), _ptr(f32_out), m, n, k, epilogue, _stream())


def linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    *,
    accumulate_into: torch.Tensor | None = None,
    out_float32: bool = False,
) -> torch.Tensor:
    """``x [M, K] @ weight [N, K]^T``.

    float32: this library's FMA kernel (true 32-bit; row results do not depend on
    M).  bfloat16: this library's matrix-core kernel that streams the weights once, or
    the library matrix product (hipBLASLt, the copy that torch has loaded), by the
    fixed rule of :func:`prefers_skinny`; beyond ``SKINNY_KERNEL_ROWS`` rows always
    the latter.  All with 32-bit accumulation.  ``accumulate_into`` (float32
    ``[M, N]``) receives ``+=`` and is returned; ``out_float32`` returns the
    32-bit sums without a rounding to bfloat16 in between."""

    _check(x, "x")
    _check(weight, "weight", dtype=x.dtype)
    if x.ndim != 2 or weight.ndim != 2 or x.shape[1] != weight.shape[1] or x.shape[0] == 0:
        raise KernelError(f"linear: x {tuple(x.shape)} does not match weight {tuple(weight.shape)}.")
    m, k = x.shape
    n = weight.shape[0]
    if accumulate_into is not None:
        _check(accumulate_into, "accumulate_into", dtype=torch.float32, shape=(m, n))
    if x.dtype == torch.float32:
        out = accumulate_into if accumulate_into is not None else torch.empty((m, n), dtype=torch.float32, device=x.device)
        call("ms_gemm_f32", _ptr(x), _ptr(weight), _ptr(out), m, n, k, int(accumulate_into is not None), _stream())
        return out
    _code(x.dtype)
    if _skinny_is_faster(x, weight, False):
        if accumulate_into is not None:
            _skinny(x, weight, _EPILOGUE_ADD_F32, accumulate_into)
            return accumulate_into
        out = torch.empty((m, n), dtype=torch.float32 if out_float32 else torch.bfloat16, device=x.device)
        _skinny(x, weight, _EPILOGUE_F32 if out_float32 else _EPILOGUE_BF16, out)
        return out
    if accumulate_into is not None:
        _library_product(x, weight, accumulate_into, True)
        return accumulate_into
    out = torch.empty((m, n), dtype=torch.float32 if out_float32 else torch.bfloat16, device=x.device)
    _library_product(x, weight, out, False)
    return out


def can_accumulate(rows: int, weight: torch.Tensor) -> bool:
    """Whether ``linear(..., accumulate_into=...)`` adds in the product's own epilogue
    (else it would cost a kernel more than handing the sum to the next norm)."""

    return weight.dtype in (torch.float32, torch.bfloat16)


def can_fuse_norm(rows: int, weight: torch.Tensor, *, gated: bool = False) -> bool:
    """Whether :func:`linear_normed` runs as one kernel for this many rows.  The norm as
    a prologue makes every workgroup read the 32-bit rows and the norm's weight beside its
    share of the matrix, which costs more than a norm kernel of its own once the matrix
    is large (measured on MI355X at 8 rows, fused against product + norm kernel: 48 MiB,
    16 us against 13 + 5; 100 MiB, 38 against 23 + 7; with the gated activation 48 MiB,
    17.5 against 12 + 5; 95 MiB, 39 against 24 + 5; 192 MiB, 50 against 42 + 5)."""

    n, k = weight.shape
    epilogue = _EPILOGUE_SILU_MUL if gated else _EPILOGUE_BF16
    if _forced_product is None and 2 * n * k > (FUSED_NORM_GATED_BYTES if gated else FUSED_NORM_BYTES):
        return False
    return (
        weight.dtype == torch.bfloat16
        and rows <= SKINNY_MAX_ROWS
        and bool(load().ms_gemm_skinny_supported(rows, n, k, epilogue))
        and prefers_skinny(rows, n, k, fused=True)
    )


def linear_normed(
    residual: torch.Tensor, norm_weight: torch.Tensor, eps: float, weight: torch.Tensor, *, gated: bool = False
) -> torch.Tensor:
    """``RMSNorm(residual) @ weight^T`` in one kernel (``gated``: then SiLU(gate) * up of
    the two halves of the result): the norm of the float32 ``residual [M, K]`` is the
    product's prologue.  Only where :func:`can_fuse_norm` says so."""

    _check(residual, "residual", dtype=torch.float32)
    _check(weight, "weight", dtype=torch.bfloat16)
    if residual.ndim != 2 or weight.ndim != 2 or residual.shape[1] != weight.shape[1] or residual.shape[0] == 0:
        raise KernelError(f"linear_normed: residual {tuple(residual.shape)} does not match weight {tuple(weight.shape)}.")
    m, k = residual.shape
    n = weight.shape[0]
    _check(norm_weight, "norm_weight", dtype=torch.bfloat16, shape=(k,))
    if not can_fuse_norm(m, weight, gated=gated):
        raise KernelError("linear_normed: this shape is not served by the fused kernel.")
    out = torch.empty((m, n // 2 if gated else n), dtype=torch.bfloat16, device=residual.device)
    product_calls["skinny"] += 1
    call("ms_gemm_skinny_normed", _ptr(residual), _ptr(norm_weight), float(eps), _ptr(weight), _ptr(out), m, n, k,
         _EPILOGUE_SILU_MUL if gated else _EPILOGUE_BF16, _stream())
    return out


def can_prepare_norm(rows: int, weight: torch.Tensor) -> bool:
    """Whether :func:`linear_norm_ahead` serves ``rows`` rows against ``weight``: where
    ``linear(..., accumulate_into=...)`` would run this library's product."""

    n, k = weight.shape
    return (
        weight.dtype == torch.bfloat16
        and rows <= SKINNY_KERNEL_ROWS
        and bool(load().ms_gemm_skinny_supported(rows, n, k, _EPILOGUE_ADD_F32))
        and prefers_skinny(rows, n, k)
    )


def can_use_prepared_norm(rows: int, weight: torch.Tensor, *, gated: bool = False) -> bool:
    """Whether :func:`linear_prepared` is the form to take for ``rows`` rows against
    ``weight``: where this library's product serves the shape and the norm would otherwise
    be a kernel of its own.  Measured on MI355X, pairs of (+= product, norm, product) in
    recorded graphs over matrices that no cache holds, in us, as (norm kernel | norm as
    prologue | prepared): 1024 wide into 6144 rows, 8 rows 13.0 | 11.1 | 11.7, 64 rows
    18.7 | - | 17.2; 4096 wide into 24576 rows, 8 rows 58.7 | 63.9 | 56.5, 16 rows
    66.0 | 73.6 | 68.1.  A small matrix with few rows keeps the prologue; every workgroup
    of the prepared form reads all rows' partial sums (as many as the product before had
    workgroups), which costs a large matrix more than the norm kernel from 16 rows on."""

    n, k = weight.shape
    epilogue = _EPILOGUE_SILU_MUL if gated else _EPILOGUE_BF16
    if not (
        weight.dtype == torch.bfloat16
        and rows <= SKINNY_KERNEL_ROWS
        and bool(load().ms_gemm_skinny_supported(rows, n, k, epilogue))
        and prefers_skinny(rows, n, k, fused=True)
    ):
        return False
    if _forced_product is not None:
        return True
    if can_fuse_norm(rows, weight, gated=gated):
        return False
    return rows <= 8 or 2 * n * k <= 16 * _MIB


def linear_norm_ahead(
    x: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor
) -> tuple[torch.Tensor, torch.Tensor]:
    """``residual += x @ weight^T`` as ``linear(..., accumulate_into=residual)``, and in the
    same kernel what the RMSNorm of the new ``residual`` needs: returns ``(weighted,
    squares)`` with ``weighted [M, N]`` = bfloat16(norm_weight * residual) and ``squares
    [G, M]``, every workgroup's sum of ``residual^2`` over its columns.
    :func:`linear_prepared` takes a product of that norm from the two."""

    _check(x, "x", dtype=torch.bfloat16)
    _check(weight, "weight", dtype=torch.bfloat16)
    if x.ndim != 2 or weight.ndim != 2 or x.shape[1] != weight.shape[1] or x.shape[0] == 0:
        raise KernelError(f"linear_norm_ahead: x {tuple(x.shape)} does not match weight {tuple(weight.shape)}.")
    m, k = x.shape
    n = weight.shape[0]
    _check(residual, "residual", dtype=torch.float32, shape=(m, n))
    _check(norm_weight, "norm_weight", dtype=torch.bfloat16, shape=(n,))
    if not can_prepare_norm(m, weight):
        raise KernelError("linear_norm_ahead: this shape is not served by this library's product.")
    groups = int(load().ms_gemm_skinny_groups(m, n))
    weighted = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    squares = torch.empty((groups, m), dtype=torch.float32, device=x.device)
    product_calls["skinny"] += 1
    call("ms_gemm_skinny_norm_ahead", _ptr(x), _ptr(weight), _ptr(residual), m, n, k, _ptr(norm_weight),
         _ptr(weighted), _ptr(squares), _stream())
    return weighted, squares


def linear_prepared(
    weighted: torch.Tensor, squares: torch.Tensor, eps: float, weight: torch.Tensor, *, gated: bool = False
) -> torch.Tensor:
    """``RMSNorm(residual) @ weight^T`` (``gated``: then SiLU(gate) * up of the two halves)
    from what :func:`linear_norm_ahead` left: the product of ``weighted`` with every sum
    scaled by ``1 / sqrt(sum of the row's squares / K + eps)``."""

    _check(weighted, "weighted", dtype=torch.bfloat16)
    _check(weight, "weight", dtype=torch.bfloat16)
    if weighted.ndim != 2 or weight.ndim != 2 or weighted.shape[1] != weight.shape[1] or weighted.shape[0] == 0:
        raise KernelError(f"linear_prepared: x {tuple(weighted.shape)} does not match weight {tuple(weight.shape)}.")
    m, k = weighted.shape
    n = weight.shape[0]
    if squares.ndim != 2 or squares.shape[0] == 0:
        raise KernelError(f"linear_prepared: squares {tuple(squares.shape)} are not [groups, {m}].")
    _check(squares, "squares", dtype=torch.float32, shape=(squares.shape[0], m))
    if not can_use_prepared_norm(m, weight, gated=gated):
        raise KernelError("linear_prepared: this shape is not served by this library's product.")
    out = torch.empty((m, n // 2 if gated else n), dtype=torch.bfloat16, device=weighted.device)
    product_calls["skinny"] += 1
    call("ms_gemm_skinny_scaled", _ptr(weighted), _ptr(weight), _ptr(out), None, m, n, k,
         _EPILOGUE_SILU_MUL if gated else _EPILOGUE_BF16, _ptr(squares), int(squares.shape[0]), float(eps), _stream())
    return out


def linear_silu_mul(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``silu(x Wg^T) * (x Wu^T)`` for ``weight [2 I, K]`` = gate rows, then up rows ->
    ``[M, I]``.  bfloat16 with few rows (as in :func:`linear`): one kernel, the
    activation in the product's epilogue; otherwise the product and :func:`silu_mul`."""

    _check(x, "x")
    _check(weight, "weight", dtype=x.dtype)
    if x.ndim != 2 or weight.ndim != 2 or x.shape[1] != weight.shape[1] or x.shape[0] == 0 or weight.shape[0] % 2:
        raise KernelError(f"linear_silu_mul: x {tuple(x.shape)} does not match weight {tuple(weight.shape)}.")
    m, k = x.shape
    n = weight.shape[0]
    if x.dtype == torch.bfloat16 and _skinny_is_faster(x, weight, True):
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
        _skinny(x, weight, _EPILOGUE_SILU_MUL, out)
        return out
    return silu_mul(linear(x, weight))


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` of ``gate_up [N, 2*I]`` (gate columns first) -> ``[N, I]``."""

    _check(gate_up, "gate_up")
    if gate_up.ndim != 2 or gate_up.shape[1] % 2 != 0 or gate_up.numel() == 0:
        raise KernelError("silu_mul takes gate_up [N>0, 2*I].")
    rows, width = gate_up.shape
    out = torch.empty((rows, width // 2), dtype=gate_up.dtype, device=gate_up.device)
    call("ms_silu_mul", _ptr(gate_up), _ptr(out), rows, width // 2, _code(gate_up.dtype), _stream())
    return out


# Vocabulary from which a sampled row is handled by many workgroups.
SAMPLE_CHUNKED_FROM = 8192


def sample_rows(
    logits: torch.Tensor,
    *,
    temperature: torch.Tensor | None = None,
    top_k: torch.Tensor | None = None,
    top_p: torch.Tensor | None = None,
    uniform: torch.Tensor | None = None,
    top_p_alone: bool = True,
) -> torch.Tensor:
    """One token per row of float32 ``logits [R, V]`` -> int32 ``[R]``.

    ``temperature`` None or 0 in a row: argmax.  Otherwise temperature, top-k
    (0 = off), top-p (1 = off), then the inverse CDF at ``uniform[r]`` in token
    order.  A row with a non-finite logit gives -1.  ``top_p_alone``: False when the
    caller knows that no row has top-p without top-k (a few small launches are spared)."""

    _check(logits, "logits", dtype=torch.float32)
    if logits.ndim != 2 or logits.numel() == 0:
        raise KernelError("sample_rows takes logits [R>0, V>0].")
    rows, vocab = logits.shape
    if temperature is not None:
        _check(temperature, "temperature", dtype=torch.float32, shape=(rows,))
        if uniform is None:
            raise KernelError("sample_rows: sampling needs uniform numbers.")
        _check(uniform, "uniform", dtype=torch.float32, shape=(rows,))
        if top_k is not None:
            _check(top_k, "top_k", dtype=torch.int32, shape=(rows,))
        if top_p is not None:
            _check(top_p, "top_p", dtype=torch.float32, shape=(rows,))
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    if temperature is None and vocab >= 4096:
        # all rows greedy: two stages, so that many workgroups share the read of a row
        chunks = 64
        chunk_max = torch.empty((rows, chunks), dtype=torch.float32, device=logits.device)
        chunk_index = torch.empty((rows, chunks), dtype=torch.int32, device=logits.device)
        call("ms_argmax_rows", _ptr(logits), _ptr(chunk_max), _ptr(chunk_index), _ptr(out), rows, vocab, chunks,
             _stream())
        return out
    if temperature is not None and vocab >= SAMPLE_CHUNKED_FROM and rows <= 65535:
        # a long row: its passes are shared by many workgroups; between the stages small tables and room for
        # the list of the tokens that can stay
        workspace = torch.empty(int(load().ms_sample_rows_workspace_bytes(rows, vocab)), dtype=torch.uint8, device=logits.device)
        call("ms_sample_rows_chunked", _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
             _ptr(out), _ptr(workspace), workspace.numel(), rows, vocab, int(bool(top_p_alone) and top_p is not None), _stream())
        return out
    call("ms_sample_rows", _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform), _ptr(out),
         rows, vocab, _stream())
    return out
