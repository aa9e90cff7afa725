"""Python faces of the HIP entry points.

Every function checks on the host what the kernel and its grid assume (device,
dtype, contiguity, shapes, index ranges that are known on the host) and raises
``ValueError`` with the offending value otherwise: a kernel is never launched
on operands it was not written for.  Kernels run on torch's current stream.
"""

from __future__ import annotations

import contextlib

from typing import Optional

import torch

from .library import load_library

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
_ERRORS = {1: "bad argument (a size or option the kernel does not take)", 2: "kernel launch failed",
           3: "more than the entry point's fixed scratch memory holds", 4: "the library's device memory was not found"}


class KernelError(RuntimeError):
    pass


_COMPUTE_UNITS: dict[int, int] = {}


def compute_units(device: "torch.device | int | None" = None) -> int:
    """Compute units of the GPU the kernels run on, asked of the device once (the plans that spread
    workgroups over the units are made from it); 256, an MI355X's, where no GPU is visible."""
    if not torch.cuda.is_available():
        return 256
    index = torch.cuda.current_device() if device is None else torch.device(device).index if not isinstance(device, int) else device
    index = torch.cuda.current_device() if index is None else index
    if index not in _COMPUTE_UNITS:
        _COMPUTE_UNITS[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _COMPUTE_UNITS[index]


def _code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise ValueError(f"kernels take float32 or bfloat16, got {dtype}") from None


def _gpu(name: str, tensor: torch.Tensor, dtype: Optional[torch.dtype] = None, dims: Optional[int] = None) -> None:
    if not tensor.is_cuda:
        raise ValueError(f"{name} must live on the GPU, is on {tensor.device}")
    if not tensor.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None:
        if not (tensor.dtype == dtype):
            raise ValueError(f"{name} must be {dtype}, is {tensor.dtype}")
    if dims is not None:
        if not (tensor.dim() == dims):
            raise ValueError(f"{name} must have {dims} dims, has shape {tuple(tensor.shape)}")


# Arguments go to the library as plain Python numbers: the entry points' argument types are declared
# when the library is loaded (kernels/library.py), and ctypes converts them itself.
def _ptr(tensor: Optional[torch.Tensor]) -> Optional[int]:
    return None if tensor is None else tensor.data_ptr()


def _stream() -> int:
    # the raw handle of torch's current stream (also the capturing one), without building a Stream object
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _run(name: str, code: int) -> None:
    if code != 0:
        raise KernelError(f"{name}: {_ERRORS.get(code, f'error {code}')}")


_i = int
_f = float


def _check_pools(k_pool: torch.Tensor, v_pool: torch.Tensor, dtype: torch.dtype, kv_heads: int,
                 head_dim: int) -> int:
    """Keys [pages, Hkv, page_size, D], values transposed [pages, Hkv, D, page_size]; returns page_size."""
    _gpu("k_pool", k_pool, dtype, 4)
    _gpu("v_pool", v_pool, dtype, 4)
    pages, heads, page_size, dim = k_pool.shape
    if not (heads == kv_heads and dim == head_dim):
        raise ValueError(f"k_pool {tuple(k_pool.shape)} does not match Hkv={kv_heads}, D={head_dim}")
    if not (tuple(v_pool.shape) == (pages, kv_heads, head_dim, page_size)):
        raise ValueError(f"v_pool {tuple(v_pool.shape)} must be {(pages, kv_heads, head_dim, page_size)}")
    return page_size


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None,
          feed: Optional[torch.Tensor] = None, pool: Optional[torch.Tensor] = None, scale: float = 1.0,
          rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t] = float32(table[ids[t]]) * scale``; ids int32 [T] (already checked against the vocabulary).
    With ``feed`` (int32 [T]) and ``pool`` (int32): row t takes ``pool[feed[t]]`` as its id where
    ``feed[t] >= 0`` (tokens another kernel left on the device; ``feed[t]`` must index ``pool``).
    ``rows`` ([T, hidden] in the table's dtype) also takes the same values, rounded to that dtype."""
    _gpu("table", table, dims=2)
    _gpu("ids", ids, torch.int32, 1)
    vocab, hidden = table.shape
    tokens = ids.shape[0]
    if feed is not None:
        _gpu("feed", feed, torch.int32, 1)
        if pool is None or feed.shape[0] < tokens:
            raise ValueError("feed needs a pool and one entry per token")
        _gpu("pool", pool, torch.int32, 1)
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
    _gpu("out", out, torch.float32, 2)
    if not (out.shape == (tokens, hidden)):
        raise ValueError(f"out must be {(tokens, hidden)}, is {tuple(out.shape)}")
    if rows is not None:
        _gpu("rows", rows, table.dtype, 2)
        if not (rows.shape == (tokens, hidden)):
            raise ValueError(f"rows must be {(tokens, hidden)}, is {tuple(rows.shape)}")
    _run("cie_embed", load_library().cie_embed(_stream(), _i(_code(table.dtype)), _ptr(table), _ptr(ids), _ptr(feed),
                                               _ptr(pool if feed is not None else None), _ptr(out), _ptr(rows),
                                               _i(tokens), _i(hidden), _i(vocab), _f(scale)))
    return out


MAX_NORM_WIDTH = 16384  # a row of the norm kernels is held in 64 KB of LDS as float32


def add_rmsnorm(residual: torch.Tensor, branch: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``residual += branch`` (if given; written back unless ``rows``), then RMS-normalise.

    residual float32 [T, H]; branch and the result in ``out_dtype``; weight [H]
    in ``out_dtype`` or float32.  With ``rows`` (int32 [n]) only those rows are
    produced, in that order, and the residual is left as it is."""
    _gpu("residual", residual, torch.float32, 2)
    tokens, hidden = residual.shape
    _gpu("weight", weight, dims=1)
    if not (weight.shape[0] == hidden):
        raise ValueError(f"weight must be [{hidden}], is {tuple(weight.shape)}")
    if not (weight.dtype in (out_dtype, torch.float32)):
        raise ValueError(f"weight dtype {weight.dtype} does not fit {out_dtype}")
    if not (hidden <= MAX_NORM_WIDTH):
        raise ValueError(f"hidden size {hidden} exceeds the norm kernel's {MAX_NORM_WIDTH}")
    if not (eps > 0):
        raise ValueError(f"eps must be positive, is {eps}")
    if branch is not None:
        _gpu("branch", branch, out_dtype, 2)
        if not (branch.shape == residual.shape):
            raise ValueError(f"branch {tuple(branch.shape)} vs residual {tuple(residual.shape)}")
    if rows is not None:
        _gpu("rows", rows, torch.int32, 1)
        n_out = rows.shape[0]
    else:
        n_out = tokens
    if out is None:
        out = torch.empty((n_out, hidden), dtype=out_dtype, device=residual.device)
    _gpu("out", out, out_dtype, 2)
    if not (out.shape == (n_out, hidden)):
        raise ValueError(f"out must be {(n_out, hidden)}, is {tuple(out.shape)}")
    _run("cie_add_rmsnorm", load_library().cie_add_rmsnorm(
        _stream(), _i(_code(out_dtype)), _i(_code(weight.dtype)), _ptr(residual), _ptr(branch), _ptr(weight),
        _ptr(out), _ptr(rows), _i(n_out), _i(hidden), _f(eps), _i(0 if rows is not None else 1)))
    return out


def rmsnorm_from_sumsq(residual: torch.Tensor, sumsq: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """bf16 RMSNorm of float32 rows whose partial sums of squares ``sumsq`` [rows, parts] are known."""
    _gpu("residual", residual, torch.float32, 2)
    rows, hidden = residual.shape
    _gpu("sumsq", sumsq, torch.float32, 2)
    if not (sumsq.shape[0] >= rows):
        raise ValueError(f"sumsq has {sumsq.shape[0]} rows for {rows}")
    _gpu("weight", weight, dims=1)
    if not (weight.shape[0] == hidden and weight.dtype in (torch.bfloat16, torch.float32)):
        raise ValueError("norm weight does not fit")
    if not (eps > 0):
        raise ValueError(f"eps must be positive, is {eps}")
    out = torch.empty((rows, hidden), dtype=torch.bfloat16, device=residual.device)
    _run("cie_rmsnorm_from_sumsq", load_library().cie_rmsnorm_from_sumsq(
        _stream(), _i(_code(weight.dtype)), _ptr(residual), _ptr(sumsq), _i(sumsq.shape[1]), _ptr(weight), _ptr(out),
        _i(rows), _i(hidden), _f(eps)))
    return out


def rope_kv_write(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                  seq_of_token: torch.Tensor, seq_slot: torch.Tensor, block_table: torch.Tensor,
                  k_pool: torch.Tensor, v_pool: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int,
                  rotate: bool = True, write_kv: bool = True, rotary_dim: Optional[int] = None) -> None:
    """Rotate q (in place) and k, write k and v of every token into its cache slot.

    qkv [T, (Hq+2Hkv)*D]; the first ``rotary_dim`` dimensions of every head rotate (all of them if
    ``None``), dimension i with i + rotary_dim/2, the rest pass through; cos/sin float32
    [max_position, rotary_dim/2]; key pool [pages, Hkv, page_size, D] and value pool
    [pages, Hkv, D, page_size] in qkv's dtype; block_table int32 [slots, width]."""
    _gpu("qkv", qkv, dims=2)
    tokens = qkv.shape[0]
    if not (qkv.shape[1] == (q_heads + 2 * kv_heads) * head_dim):
        raise ValueError(f"qkv row is {qkv.shape[1]}, heads say {(q_heads + 2 * kv_heads) * head_dim}")
    rotary_dim = head_dim if rotary_dim is None else rotary_dim
    if rotate and not (0 < rotary_dim <= head_dim and rotary_dim % 2 == 0):
        raise ValueError(f"rotary_dim must be even and at most the head size {head_dim}, is {rotary_dim}")
    for name, table in (("cos", cos), ("sin", sin)):
        _gpu(name, table, torch.float32, 2)
        if rotate and not (table.shape[1] == rotary_dim // 2):
            raise ValueError(f"{name} must be [max_position, {rotary_dim // 2}]")
    if not (cos.shape == sin.shape):
        raise ValueError("cos and sin tables differ in shape")
    for name, meta in (("positions", positions), ("seq_of_token", seq_of_token)):
        _gpu(name, meta, torch.int32, 1)
        if not (meta.shape[0] >= tokens):
            raise ValueError(f"{name} has {meta.shape[0]} entries for {tokens} tokens")
    _gpu("seq_slot", seq_slot, torch.int32, 1)
    _gpu("block_table", block_table, torch.int32, 2)
    page_size = _check_pools(k_pool, v_pool, qkv.dtype, kv_heads, head_dim)
    _run("cie_rope_kv_write", load_library().cie_rope_kv_write(
        _stream(), _i(_code(qkv.dtype)), _ptr(qkv), _ptr(cos), _ptr(sin), _ptr(positions), _ptr(seq_of_token),
        _ptr(seq_slot), _ptr(block_table), _i(block_table.shape[1]), _ptr(k_pool), _ptr(v_pool), _i(tokens),
        _i(q_heads), _i(kv_heads), _i(head_dim), _i(rotary_dim if rotate else 0), _i(page_size),
        _i(1 if rotate else 0), _i(1 if write_kv else 0)))


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None, row_sumsq: Optional[torch.Tensor] = None,
             hidden: int = 0, eps: float = 0.0) -> torch.Tensor:
    """``silu(gate_up[:, :I]) * gate_up[:, I:]`` for gate_up [T, 2I].  With ``row_sumsq``
    [T, parts] (partial sums of squares of rows of ``hidden`` values) both halves of
    row t are first multiplied by ``rsqrt(sum(row_sumsq[t]) / hidden + eps)``: the
    1/rms that the rows of the product behind ``gate_up`` lacked."""
    _gpu("gate_up", gate_up, dims=2)
    tokens, twice = gate_up.shape
    if not (twice % 2 == 0):
        raise ValueError(f"gate_up row must be even, is {twice}")
    inter = twice // 2
    if out is None:
        out = torch.empty((tokens, inter), dtype=gate_up.dtype, device=gate_up.device)
    _gpu("out", out, gate_up.dtype, 2)
    if not (out.shape == (tokens, inter)):
        raise ValueError(f"out must be {(tokens, inter)}, is {tuple(out.shape)}")
    parts = 0
    if row_sumsq is not None:
        _gpu("row_sumsq", row_sumsq, torch.float32, 2)
        if not (row_sumsq.shape[0] >= tokens and hidden > 0 and eps > 0):
            raise ValueError("row_sumsq needs a row per token, the rows' width and a positive eps")
        parts = row_sumsq.shape[1]
    _run("cie_silu_mul", load_library().cie_silu_mul(_stream(), _i(_code(gate_up.dtype)), _ptr(gate_up),
                                                     _ptr(out), _i(tokens), _i(inter), _ptr(row_sumsq), _i(parts),
                                                     _i(hidden), _f(eps)))
    return out


def paged_attention_generic(q: torch.Tensor, q_row_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                            block_table: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor,
                            seq_slot: torch.Tensor, tokens: int, q_heads: int, kv_heads: int, head_dim: int,
                            window: Optional[int], scale: float,
                            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of each token over its request's cached keys (its own included).

    ``q`` is any tensor whose row ``t`` holds the token's q heads in its first
    ``q_heads*head_dim`` elements, rows ``q_row_stride`` elements apart (the
    fused qkv buffer qualifies).  Returns [tokens, q_heads*head_dim]."""
    if not (q.is_cuda and q.dim() == 2 and q.stride(1) == 1 and q.stride(0) == q_row_stride):
        raise ValueError(f"q must be 2-d on the GPU with unit inner stride and row stride {q_row_stride}")
    if not (q.shape[0] >= tokens and q.shape[1] >= q_heads * head_dim):
        raise ValueError(f"q {tuple(q.shape)} too small")
    if not (q_heads % kv_heads == 0):
        raise ValueError(f"{q_heads} query heads are no multiple of {kv_heads} key heads")
    if not (head_dim % 8 == 0 and head_dim <= 256):
        raise ValueError(f"head_dim must be a multiple of 8 up to 256, is {head_dim}")
    if not (q_row_stride % 8 == 0):
        raise ValueError(f"q row stride must be a multiple of 8, is {q_row_stride}")
    _check_pools(k_pool, v_pool, q.dtype, kv_heads, head_dim)
    _gpu("block_table", block_table, torch.int32, 2)
    for name, meta in (("positions", positions), ("seq_of_token", seq_of_token)):
        _gpu(name, meta, torch.int32, 1)
        if not (meta.shape[0] >= tokens):
            raise ValueError(f"{name} has {meta.shape[0]} entries for {tokens} tokens")
    _gpu("seq_slot", seq_slot, torch.int32, 1)
    if out is None:
        out = torch.empty((tokens, q_heads * head_dim), dtype=q.dtype, device=q.device)
    _gpu("out", out, q.dtype, 2)
    if not (out.shape == (tokens, q_heads * head_dim)):
        raise ValueError(f"out is {tuple(out.shape)}")
    _run("cie_paged_attention_generic", load_library().cie_paged_attention_generic(
        _stream(), _i(_code(q.dtype)), _ptr(q), _i(q_row_stride), _ptr(k_pool), _ptr(v_pool), _ptr(block_table),
        _i(block_table.shape[1]), _ptr(positions), _ptr(seq_of_token), _ptr(seq_slot), _ptr(out), _i(tokens),
        _i(q_heads), _i(kv_heads), _i(head_dim), _i(k_pool.shape[2]), _i(window or 0), _f(scale)))
    return out


MFMA_HEAD_DIMS = (32, 64, 96, 128, 256)
TILE_WAVES = 4  # waves per workgroup of the prompt form of the matrix-core attention
PROMPT_WAVES = 8  # ... and of its form with tiles of 128 rows whose keys and values go through LDS


def paged_attention_mfma(q: torch.Tensor, q_row_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                         block_table: torch.Tensor, tile_seq: Optional[torch.Tensor], tile_q0: Optional[torch.Tensor],
                         n_tiles: int,
                         seq_slot: torch.Tensor, seq_start: torch.Tensor, seq_q_len: torch.Tensor,
                         q_start_loc: torch.Tensor, out: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int,
                         window: Optional[int], scale: float, tokens_per_tile: int, row_tiles: int,
                         n_splits: int = 1, keys_per_split: int = 0,
                         max_context_dev: Optional[torch.Tensor] = None,
                         part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                         tile_waves: int = 1) -> None:
    """Matrix-core attention (bf16) for the tiles ``(tile_seq[i], tile_q0[i])``: tile i
    holds up to ``tokens_per_tile`` tokens of sequence ``tile_seq[i]`` from its
    ``tile_q0[i]``-th token of this step on (both ``None``: tile i starts sequence i, as in
    a step of single tokens; one dependent load less).  Rows of other tokens of ``out`` are left alone.
    With ``n_splits > 1`` every tile's keys are cut into parts of ``keys_per_split``
    (a multiple of 32; or, with ``max_context_dev``, derived on the device from the
    step's longest context) and merged through the workspaces.  ``tile_waves=4`` gives
    every tile (and every part of its keys) a workgroup of four waves that take the
    blocks of 32 keys in turn; it needs pages of at least 16 keys.  ``tile_waves=8`` (heads of up to
    128 dimensions) is the form whose waves share the tile's keys and values through LDS: with
    ``row_tiles=8`` tiles of 128 rows and eight waves, with ``row_tiles=4`` tiles of 64 rows and four
    waves, two such workgroups to a compute unit."""
    if not (
        q.is_cuda and q.dtype == torch.bfloat16 and q.dim() == 2 and q.stride(1) == 1 and q.stride(0) == q_row_stride
    ):
        raise ValueError("q must be a bf16 GPU matrix with unit inner stride")
    if not (q.shape[1] >= q_heads * head_dim and q_row_stride % 8 == 0):
        raise ValueError(f"q {tuple(q.shape)} does not fit")
    if not (head_dim in MFMA_HEAD_DIMS):
        raise ValueError(f"head_dim must be one of {MFMA_HEAD_DIMS}, is {head_dim}")
    if not (q_heads % kv_heads == 0):
        raise ValueError(f"{q_heads} query heads are no multiple of {kv_heads} key heads")
    group = q_heads // kv_heads
    if not (row_tiles in (1, 2, 4, 8) and 1 <= tokens_per_tile and tokens_per_tile * group <= 16 * row_tiles):
        raise ValueError(f"{tokens_per_tile} tokens of {group} heads do not fit {row_tiles} row tiles")
    page_size = _check_pools(k_pool, v_pool, torch.bfloat16, kv_heads, head_dim)
    if not (page_size >= 4 and page_size & (page_size - 1) == 0):
        raise ValueError(f"page size must be a power of two >= 4, is {page_size}")
    _gpu("block_table", block_table, torch.int32, 2)
    if (tile_seq is None) != (tile_q0 is None):
        raise ValueError("tile_seq and tile_q0 come together, or neither (tile i is then the first tile of sequence i)")
    for name, meta in (("tile_seq", tile_seq), ("tile_q0", tile_q0)):
        if meta is None:
            continue
        _gpu(name, meta, torch.int32, 1)
        if not (meta.shape[0] >= n_tiles):
            raise ValueError(f"{name} has {meta.shape[0]} entries for {n_tiles} tiles")
    if tile_seq is None and seq_q_len.shape[0] < n_tiles:
        raise ValueError(f"{n_tiles} tiles for {seq_q_len.shape[0]} sequences")
    for name, meta in (("seq_slot", seq_slot), ("seq_start", seq_start), ("seq_q_len", seq_q_len),
                       ("q_start_loc", q_start_loc)):
        _gpu(name, meta, torch.int32, 1)
    _gpu("out", out, torch.bfloat16, 2)
    if not (out.shape[1] == q_heads * head_dim and out.shape[0] <= q.shape[0]):
        raise ValueError(f"out is {tuple(out.shape)}")
    if not (1 <= n_splits <= 65535):
        raise ValueError(f"n_splits {n_splits} out of range")
    if not (
        (tile_waves == 1 and row_tiles <= 4)
        or (tile_waves == TILE_WAVES and scale > 0 and page_size >= 16 and row_tiles <= 4
            and (row_tiles == 1 or head_dim <= 128))
        or (tile_waves == PROMPT_WAVES and scale > 0 and page_size >= 16 and row_tiles in (4, 8) and head_dim <= 128)
    ):
        raise ValueError(f"tile_waves {tile_waves} with {n_splits} splits, {row_tiles} row tiles, head size {head_dim}, "
                         f"pages of {page_size}")
    if n_splits > 1:
        rows = 16 * row_tiles
        if not (part_o is not None and part_ml is not None):
            raise ValueError("split attention needs its workspaces")
        _gpu("part_o", part_o, torch.float32)
        _gpu("part_ml", part_ml, torch.float32)
        units = n_tiles * kv_heads * n_splits
        if not (part_o.numel() >= units * rows * head_dim and part_ml.numel() >= units * rows * 2):
            raise ValueError("attention workspaces are too small")
        if max_context_dev is not None:
            _gpu("max_context_dev", max_context_dev, torch.int32)
        else:
            if not (keys_per_split > 0 and keys_per_split % 32 == 0):
                raise ValueError(f"keys_per_split {keys_per_split} must be a multiple of 32")
    _run("cie_paged_attention_mfma", load_library().cie_paged_attention_mfma(
        _stream(), _ptr(q), _i(q_row_stride), _ptr(k_pool), _ptr(v_pool), _ptr(block_table),
        _i(block_table.shape[1]), _ptr(tile_seq), _ptr(tile_q0), _ptr(seq_slot), _ptr(seq_start), _ptr(seq_q_len),
        _ptr(q_start_loc), _ptr(out), _ptr(part_o), _ptr(part_ml), _i(n_tiles), _i(q_heads), _i(kv_heads),
        _i(head_dim), _i(page_size), _i(window or 0), _f(scale), _i(n_splits), _i(tokens_per_tile), _i(row_tiles),
        _i(keys_per_split), _ptr(max_context_dev), _i(tile_waves)))


def gemm_f32(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """True float32 ``a @ weight.T + bias``; a [M, K] (rows may be strided), weight [N, K]."""
    if not (a.is_cuda and a.dtype == torch.float32 and a.dim() == 2 and a.stride(1) == 1):
        raise ValueError("a must be a float32 GPU matrix with unit inner stride")
    _gpu("weight", weight, torch.float32, 2)
    m, k = a.shape
    n = weight.shape[0]
    if not (weight.shape[1] == k):
        raise ValueError(f"a is [{m},{k}] but weight is {tuple(weight.shape)}")
    if bias is not None:
        _gpu("bias", bias, torch.float32, 1)
        if not (bias.shape[0] == n):
            raise ValueError(f"bias must be [{n}]")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    _gpu("out", out, torch.float32, 2)
    if not (out.shape == (m, n)):
        raise ValueError(f"out must be {(m, n)}")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    _run("cie_gemm_f32", load_library().cie_gemm_f32(_stream(), _ptr(a), _ptr(weight), _ptr(bias), _ptr(out),
                                                     _i(m), _i(n), _i(k), _i(lda), _i(n)))
    return out


EPI_BF16, EPI_F32, EPI_SILU, EPI_RESID, EPI_PARTIAL = 0, 1, 2, 3, 4
EPI_ATOMIC = 7  # (the shared-rows form: parts of K add into a float32 stream with atomic adds)
FUSED_TARGET_WAVES = 2048
FUSED_MAX_ROWS = 64  # rows one workgroup of ``gemm_fused`` takes; more rows run as more workgroup rows
FUSED_PAIR_WORKGROUPS = 256  # workgroups that must remain when workgroups of many rows take two column tiles


def plan_fused(rows: int, column_tiles: int, k: int) -> tuple[int, int, int]:
    """(row tiles, waves per workgroup, column tiles per workgroup) of ``gemm_fused``
    for ``rows`` rows, ``column_tiles`` tiles of 16 columns and a K of ``k``.  16, 32 or 64 rows per workgroup (more rows: more workgroups,
    each streaming the weight again).  With more than 16 rows a workgroup takes
    two column tiles if that still leaves enough workgroups (each activation
    value a wave loads then meets two weight tiles).  As many waves share K as it
    takes to fill the GPU, each with at least one 128-wide slice."""
    row_tiles = 1 if rows <= 16 else 2 if rows <= 32 else 4
    pair = row_tiles > 1 and column_tiles >= 2 * FUSED_PAIR_WORKGROUPS
    groups = (-(-column_tiles // 2) if pair else column_tiles) * -(-rows // FUSED_MAX_ROWS)
    waves = 1 if row_tiles == 1 else 4
    while waves < 8 and groups * waves < FUSED_TARGET_WAVES and waves * 2 * 128 <= k:
        waves *= 2
    return row_tiles, waves, 2 if pair else 1


def gemm_fused(weight: torch.Tensor, epilogue: int, a: torch.Tensor, bias: Optional[torch.Tensor] = None,
               residual_out: Optional[torch.Tensor] = None, sumsq_out: Optional[torch.Tensor] = None,
               plan: Optional[tuple[int, int, int]] = None,
               norm_weight: Optional[torch.Tensor] = None, scaled_out: Optional[torch.Tensor] = None,
               row_sumsq: Optional[torch.Tensor] = None, eps: float = 0.0) -> torch.Tensor:
    """Few-row matrix product ``a @ weight.T`` (bf16 operands, float32 sums) fused
    with its neighbour.  ``epilogue``: ``EPI_BF16`` / ``EPI_F32`` return
    ``a W^T + bias``; ``EPI_SILU`` (weight = gate rows over up rows) returns
    ``silu(gate) * up`` [M, N/2]; ``EPI_RESID`` adds the product
    into ``residual_out`` (float32 [M, N]) and returns the partial sums of
    squares of its new rows [M, ceil(N/16)].  (Partial products of a cut K: :func:`gemm_shared_rows`.)
    An RMSNorm between an ``EPI_RESID`` product and an ``EPI_SILU`` product of up to 16
    rows can ride along: with ``norm_weight`` (float32 [N]) and ``scaled_out`` (bf16
    [M, N]) the former also writes the new residual times the weight, and the latter,
    given these rows as ``a`` with ``row_sumsq`` (the former's result) and ``eps``,
    multiplies its sums by each row's ``rsqrt(mean square + eps)`` before the SiLU."""
    _gpu("weight", weight, torch.bfloat16, 2)
    n, k = weight.shape
    if not (a.is_cuda and a.dtype == torch.bfloat16 and a.dim() == 2 and a.stride(1) == 1):
        raise ValueError("a must be a bf16 GPU matrix with unit inner stride")
    m = a.shape[0]
    if not (m >= 1 and a.shape[1] == k):
        raise ValueError(f"a {tuple(a.shape)} vs K={k}")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    if not (k % 8 == 0 and lda % 8 == 0):
        raise ValueError(f"K and the row stride must be multiples of 8, are {k} and {lda}")
    if not (a.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0):
        raise ValueError("operands must be 16-byte aligned")
    device = weight.device
    if bias is not None:
        _gpu("bias", bias, torch.bfloat16, 1)
        if not (bias.shape[0] == n and epilogue != EPI_SILU):
            raise ValueError("bias does not fit")
    columns = n // 2 if epilogue == EPI_SILU else n
    row_tiles, waves, column_tiles = plan or plan_fused(m, -(-columns // 16), k)
    if epilogue == EPI_SILU:
        column_tiles = 1 if row_tiles == 1 else 2  # always a gate tile with its up tile
    if not (
        row_tiles in (1, 2, 4) and waves in ((1, 2, 4, 8) if row_tiles == 1 else (4, 8))
        and column_tiles in ((1,) if row_tiles == 1 else (1, 2))
    ):
        raise ValueError(f"plan {(row_tiles, waves, column_tiles)} is not one the kernel has")
    residual = sumsq = None
    if epilogue == EPI_BF16:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    elif epilogue == EPI_F32:
        out = torch.empty((m, n), dtype=torch.float32, device=device)
    elif epilogue == EPI_SILU:
        if not (n % 2 == 0):
            raise ValueError(f"the SiLU epilogue needs an even N, got {n}")
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=device)
    elif epilogue == EPI_RESID:
        if not (residual_out is not None):
            raise ValueError("the residual epilogue needs the residual to add into")
        _gpu("residual_out", residual_out, torch.float32, 2)
        if not (residual_out.shape == (m, n)):
            raise ValueError(f"residual_out {tuple(residual_out.shape)} vs {(m, n)}")
        parts = -(-n // 16)
        if sumsq_out is None:
            sumsq_out = torch.empty((m, parts), dtype=torch.float32, device=device)
        _gpu("sumsq_out", sumsq_out, torch.float32, 2)
        if not (sumsq_out.shape[0] >= m and sumsq_out.shape[1] == parts):
            raise ValueError(f"sumsq_out {tuple(sumsq_out.shape)} must be [>= {m}, {parts}]")
        out, residual, sumsq = sumsq_out, residual_out, sumsq_out
    else:
        raise ValueError(f"unknown epilogue {epilogue}")
    if (norm_weight is None) != (scaled_out is None) or (scaled_out is not None and epilogue != EPI_RESID):
        raise ValueError("a scaled copy needs the norm's weight, its own rows and the residual epilogue")
    if scaled_out is not None:
        _gpu("norm_weight", norm_weight, torch.float32, 1)
        _gpu("scaled_out", scaled_out, torch.bfloat16, 2)
        if not (norm_weight.shape[0] == n and scaled_out.shape == (m, n)):
            raise ValueError(f"norm_weight {tuple(norm_weight.shape)} / scaled_out {tuple(scaled_out.shape)} vs {(m, n)}")
    parts_in = 0
    if row_sumsq is not None:
        _gpu("row_sumsq", row_sumsq, torch.float32, 2)
        if not (epilogue == EPI_SILU and row_tiles == 1 and m <= 16 and row_sumsq.shape[0] >= m and eps > 0):
            raise ValueError("rows that lack their scale go to the SiLU epilogue of up to 16 rows, with a positive eps")
        parts_in = row_sumsq.shape[1]
    _run("cie_gemm_fused", load_library().cie_gemm_fused(
        _stream(), _ptr(a), _i(lda), _ptr(weight), _ptr(bias), _ptr(None if epilogue == EPI_RESID else out),
        _ptr(residual), _ptr(sumsq), _i(m), _i(n), _i(k), _i(epilogue), _i(row_tiles), _i(waves), _i(column_tiles),
        _ptr(norm_weight), _ptr(scaled_out), _ptr(row_sumsq), _i(parts_in), _f(eps)))
    return out


SHARED_ROWS_MAX = 128  # rows of the form whose waves share the rows of A


def gemm_shared_rows(weight: torch.Tensor, epilogue: int, a: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     column_tiles: int = 2, waves: int = 4, k_parts: int = 1,
                     row_sumsq: Optional[torch.Tensor] = None, eps: float = 0.0,
                     add_into: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``a @ weight.T`` for 17 to 128 rows (it takes fewer too) in the form whose four waves per
    workgroup own columns and share each slice of ``a`` through LDS: ``EPI_BF16`` or ``EPI_F32`` (+ bias),
    ``EPI_SILU`` (weight = gate rows over up rows; with ``row_sumsq`` and ``eps`` the rows of ``a``
    lack their ``rsqrt(mean square + eps)``, as in :func:`gemm_fused`) or ``EPI_PARTIAL``
    (``k_parts`` float32 partial products [k_parts, M, N], bias in part 0) or ``EPI_ATOMIC``
    (each of the ``k_parts`` parts of K adds its products into ``add_into``, float32 [M, N], with the
    hardware's atomic float add: no partial products to sum afterwards, and no fixed order of the sums;
    ``add_into`` comes back).  ``column_tiles`` tiles of 16 columns per wave, ``waves`` waves per workgroup."""
    _gpu("weight", weight, torch.bfloat16, 2)
    n, k = weight.shape
    if not (a.is_cuda and a.dtype == torch.bfloat16 and a.dim() == 2 and a.stride(1) == 1):
        raise ValueError("a must be a bf16 GPU matrix with unit inner stride")
    m = a.shape[0]
    if not (1 <= m <= SHARED_ROWS_MAX and a.shape[1] == k):
        raise ValueError(f"a {tuple(a.shape)} vs K={k} and at most {SHARED_ROWS_MAX} rows")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    if not (k % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0):
        raise ValueError(f"K and the row stride must be multiples of 8 (are {k}, {lda}) and the operands 16-byte aligned")
    if epilogue not in (EPI_BF16, EPI_F32, EPI_SILU, EPI_PARTIAL, EPI_ATOMIC):
        raise ValueError(f"epilogue {epilogue} is not one this form has")
    if epilogue == EPI_F32:
        column_tiles = 2
    if not (1 <= k_parts <= 64 and (k_parts == 1 or epilogue in (EPI_PARTIAL, EPI_ATOMIC))):
        raise ValueError(f"k_parts {k_parts} does not fit the epilogue")
    if (epilogue == EPI_ATOMIC) != (add_into is not None):
        raise ValueError("the atomic epilogue, and only it, adds into a stream that the caller gives")
    if add_into is not None:
        _gpu("add_into", add_into, torch.float32, 2)
        if not (tuple(add_into.shape) == (m, n) and add_into.is_contiguous()):
            raise ValueError(f"add_into is {tuple(add_into.shape)}, the product [{m}, {n}]")
    if epilogue == EPI_SILU:
        column_tiles = 2
        if n % 2 or bias is not None:
            raise ValueError("the SiLU epilogue needs an even N and no bias")
    if column_tiles not in (1, 2) or waves not in (2, 3, 4):
        raise ValueError(f"column_tiles {column_tiles} not in (1, 2), or waves {waves} not in (2, 3, 4)")
    if bias is not None:
        _gpu("bias", bias, torch.bfloat16, 1)
        if bias.shape[0] != n:
            raise ValueError(f"bias must be [{n}]")
    parts_in = 0
    if row_sumsq is not None:
        _gpu("row_sumsq", row_sumsq, torch.float32, 2)
        if not (epilogue == EPI_SILU and row_sumsq.shape[0] >= m and eps > 0):
            raise ValueError("rows that lack their scale go to the SiLU epilogue, with a positive eps")
        parts_in = row_sumsq.shape[1]
    device = weight.device
    if epilogue == EPI_BF16:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    elif epilogue == EPI_F32:
        out = torch.empty((m, n), dtype=torch.float32, device=device)
    elif epilogue == EPI_SILU:
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=device)
    elif epilogue == EPI_ATOMIC:
        out = add_into
    else:
        out = torch.empty((k_parts, m, n), dtype=torch.float32, device=device)
    _run("cie_gemm_shared_rows", load_library().cie_gemm_shared_rows(
        _stream(), _ptr(a), _i(lda), _ptr(weight), _ptr(bias), _ptr(out), _i(m), _i(n), _i(k), _i(epilogue),
        _i(column_tiles), _i(waves), _i(k_parts), _ptr(row_sumsq), _i(parts_in), _f(eps)))
    return out


_WORKSPACES: dict[torch.device, torch.Tensor] = {}
LIBRARY_WORKSPACE_BYTES = 64 << 20
# Products of at least this many rows, in steps of 256 (full prompt portions), and of a power of two of rows
# from 32 on (the buckets of captured decode steps) are the shapes that recur: they time the library's
# candidate algorithms at their first call and keep the fastest; others take its first choice.
LIBRARY_TUNE_ROWS = 512
# Row counts whose products time every algorithm the library has, not only the heuristic's candidates (a few
# seconds for each shape, once in a process).  An engine names the sizes of its full prompt portions around its
# own steps (:func:`library_search`); outside of that nothing is searched, so one engine's choice does not
# reach another's steps.
_search_rows: frozenset = frozenset()


@contextlib.contextmanager
def library_search(rows):
    """While the block runs, library products of these row counts time every algorithm at a shape's first call."""
    global _search_rows
    previous, _search_rows = _search_rows, frozenset(rows)
    try:
        yield
    finally:
        _search_rows = previous


def _tune_level(rows: int) -> int:
    if rows >= LIBRARY_TUNE_ROWS and rows in _search_rows:
        return 2
    if (rows >= LIBRARY_TUNE_ROWS and rows % 256 == 0) or (rows >= 32 and rows & (rows - 1) == 0):
        return 1
    return 0


def gemm_library(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 out_dtype: torch.dtype = torch.bfloat16) -> Optional[torch.Tensor]:
    """``a @ weight.T + bias`` through the vendor library (hipBLASLt) with the
    descriptors and the chosen algorithm of every shape kept after its first call:
    bf16 operands and bias, float32 sums, bf16 result, or without bias a float32
    result.  For products with many rows.  Returns ``None`` if the library has no algorithm for the shape."""
    _gpu("weight", weight, torch.bfloat16, 2)
    n, k = weight.shape
    if not (a.is_cuda and a.dtype == torch.bfloat16 and a.dim() == 2 and a.stride(1) == 1):
        raise ValueError("a must be a bf16 GPU matrix with unit inner stride")
    m = a.shape[0]
    if not (m >= 1 and a.shape[1] == k):
        raise ValueError(f"a {tuple(a.shape)} vs K={k}")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    if out_dtype not in (torch.bfloat16, torch.float32) or (out_dtype == torch.float32 and bias is not None):
        raise ValueError(f"the result is bf16, or float32 without bias; asked for {out_dtype} with{'' if bias is not None else 'out'} bias")
    if bias is not None:
        _gpu("bias", bias, torch.bfloat16, 1)
        if bias.shape[0] != n:
            raise ValueError(f"bias must be [{n}]")
    device = weight.device
    workspace = _WORKSPACES.get(device)
    if workspace is None:
        # cleared once: algorithms that meet through flags in the workspace leave them cleared after each call
        workspace = _WORKSPACES[device] = torch.zeros(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    out = torch.empty((m, n), dtype=out_dtype, device=device)
    code = load_library().cie_gemm_library(
        _stream(), _ptr(a), _i(lda), _ptr(weight), _ptr(bias), _ptr(out), _i(m), _i(n), _i(k),
        _i(1 if out_dtype == torch.float32 else 0), _ptr(workspace), workspace.numel(),
        _i(_tune_level(m)))
    if code == 1:
        return None
    _run("cie_gemm_library", code)
    return out


QKV_SPLIT_PAIRS_BELOW = 128  # (as in the kernel library: below this many pairs of tiles, one tile a workgroup)


FOLDED_NORM_ROWS = 16      # the most rows whose norm the q/k/v product makes itself: one tile of rows
# (norm kernel + product against the product that makes its norm, us in a captured chain: 3B shape 1 / 8 / 16 rows
# 9.0 / 10.6 / 10.9 against 7.1 / 7.9 / 8.9; 7B 13.3 / 15.2 / 16.0 against 11.3 / 12.8 / 14.2; 14B 21.1 / 22.3 /
# 23.4 against 18.9 / 20.2 / 22.0; 0.5B 7.0 / 8.3 / 8.5 against 5.7 / 6.6 / 7.4.  Every workgroup makes the rows
# anew, which costs it about 1 us: the rows are read in whole 256-byte segments, four rows a load, and pass through
# the wave's staging area; with every lane reading the values of its own matrix operand it cost 2 to 6 us and lost
# from the 7B width on.)


def folds_norm(rows: int, k: int) -> bool:
    """Whether ``gemm_qkv_rope`` takes ``folded=`` for this many rows of ``k`` values."""
    return 1 <= rows <= FOLDED_NORM_ROWS and k >= 8 and k % 8 == 0


def gemm_qkv_rope(weight: torch.Tensor, a: Optional[torch.Tensor], bias: Optional[torch.Tensor], cos: torch.Tensor,
                  sin: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor, seq_slot: torch.Tensor,
                  block_table: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, q_heads: int,
                  kv_heads: int, head_dim: int, rotate: bool = True, write_kv: bool = True,
                  waves: Optional[int] = None, folded: Optional[tuple] = None) -> torch.Tensor:
    """The q/k/v product of a few rows (64 per workgroup) fused with what ``rope_kv_write`` does:
    ``a @ weight.T + bias`` for weight [(Hq+2Hkv)*D, K], queries and keys rotated
    by each row's position, keys and values written into the cache.  Returns the
    buffer [M, (Hq+2Hkv)*D] whose query columns hold the rotated queries (its key
    and value columns are not written).  Same results as ``gemm_fused`` followed
    by ``rope_kv_write``.  Head sizes in steps of 32.

    ``folded=(residual, norm_weight, eps)`` instead of ``a`` (``folds_norm`` says for which sizes): the rows
    are the RMSNorm of ``residual`` (float32 [M, K], float32 weight), made inside the product: a lane makes
    the values of its matrix operand from the stream, and the rows' 1/rms multiplies the sums."""
    _gpu("weight", weight, torch.bfloat16, 2)
    n, k = weight.shape
    if folded is not None:
        residual, norm_weight, eps = folded
        _gpu("residual", residual, torch.float32, 2)
        _gpu("norm_weight", norm_weight, torch.float32, 1)
        m = residual.shape[0]
        if a is not None or not folds_norm(m, k):
            raise ValueError(f"the product makes the norm of up to {FOLDED_NORM_ROWS} rows itself, not of {m} rows "
                             f"of {k}; and then takes no rows")
        if not (residual.shape == (m, k) and norm_weight.shape == (k,) and eps > 0):
            raise ValueError(f"residual {tuple(residual.shape)}, weight {tuple(norm_weight.shape)} do not fit rows of K={k}")
        if not (residual.is_contiguous() and norm_weight.is_contiguous()
                and residual.data_ptr() % 16 == 0 and norm_weight.data_ptr() % 16 == 0):
            raise ValueError("residual and weight must be contiguous and 16-byte aligned")
        lda = k
    else:
        if not (a.is_cuda and a.dtype == torch.bfloat16 and a.dim() == 2 and a.stride(1) == 1):
            raise ValueError("a must be a bf16 GPU matrix with unit inner stride")
        m = a.shape[0]
        if not (m >= 1 and a.shape[1] == k):
            raise ValueError(f"a {tuple(a.shape)}: rows of K={k}")
        lda = a.stride(0) if m > 1 else max(a.stride(0), k)
        if not (a.data_ptr() % 16 == 0):
            raise ValueError("operands must be 16-byte aligned")
    if not (k % 8 == 0 and lda % 8 == 0):
        raise ValueError(f"K and the row stride must be multiples of 8, are {k} and {lda}")
    if not (weight.data_ptr() % 16 == 0):
        raise ValueError("operands must be 16-byte aligned")
    if not (head_dim % 32 == 0):
        raise ValueError(f"the fused rotation takes head sizes in steps of 32, not {head_dim}")
    if not (n == (q_heads + 2 * kv_heads) * head_dim):
        raise ValueError(f"weight has {n} rows, heads say {(q_heads + 2 * kv_heads) * head_dim}")
    if bias is not None:
        _gpu("bias", bias, torch.bfloat16, 1)
        if not (bias.shape[0] == n):
            raise ValueError("bias does not fit")
    for name, table in (("cos", cos), ("sin", sin)):
        _gpu(name, table, torch.float32, 2)
        if not (table.shape[1] == head_dim // 2):
            raise ValueError(f"{name} must be [max_position, {head_dim // 2}]")
    if not (cos.shape == sin.shape):
        raise ValueError("cos and sin tables differ in shape")
    for name, meta in (("positions", positions), ("seq_of_token", seq_of_token)):
        _gpu(name, meta, torch.int32, 1)
        if not (meta.shape[0] >= m):
            raise ValueError(f"{name} has {meta.shape[0]} entries for {m} rows")
    _gpu("seq_slot", seq_slot, torch.int32, 1)
    _gpu("block_table", block_table, torch.int32, 2)
    page_size = _check_pools(k_pool, v_pool, torch.bfloat16, kv_heads, head_dim)
    if waves is None:
        _, waves, _ = plan_fused(m, n // 32, k)
        if m <= 16 and n // 32 < QKV_SPLIT_PAIRS_BELOW:
            waves = min(waves, 4)  # (the kernel then takes one tile a workgroup, twice the workgroups: 8.1 -> 7.2 us)
    if not (waves in ((1, 2, 4, 8) if m <= 16 else (4, 8))):
        raise ValueError(f"{waves} waves per workgroup with {m} rows is not a form the kernel has")
    out = torch.empty((m, n), dtype=torch.bfloat16, device=weight.device)
    if folded is not None:
        _run("cie_gemm_qkv_rope_folded_norm", load_library().cie_gemm_qkv_rope_folded_norm(
            _stream(), _ptr(residual), _ptr(norm_weight), _f(eps),
            _ptr(weight), _ptr(bias), _ptr(out), _i(m), _i(n), _i(k), _i(waves), _ptr(cos), _ptr(sin), _ptr(positions),
            _ptr(seq_of_token), _ptr(seq_slot), _ptr(block_table), _i(block_table.shape[1]), _ptr(k_pool), _ptr(v_pool),
            _i(q_heads), _i(kv_heads), _i(head_dim), _i(page_size), _i(1 if rotate else 0), _i(1 if write_kv else 0)))
        return out
    _run("cie_gemm_qkv_rope", load_library().cie_gemm_qkv_rope(
        _stream(), _ptr(a), _i(lda), _ptr(weight), _ptr(bias), _ptr(out), _i(m), _i(n), _i(k), _i(waves), _ptr(cos),
        _ptr(sin), _ptr(positions), _ptr(seq_of_token), _ptr(seq_slot), _ptr(block_table), _i(block_table.shape[1]),
        _ptr(k_pool), _ptr(v_pool), _i(q_heads), _i(kv_heads), _i(head_dim), _i(page_size),
        _i(1 if rotate else 0), _i(1 if write_kv else 0)))
    return out


ARGMAX_CHUNK = 2048


def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           uniform: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of float32 logits: argmax where the row's temperature
    is 0 (or none is given), else a draw with the row's uniform number."""
    _gpu("logits", logits, torch.float32, 2)
    rows, vocab = logits.shape
    if temperature is None and vocab >= 4 * ARGMAX_CHUNK:
        if out is None:
            out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
        chunks = -(-vocab // ARGMAX_CHUNK)
        chunk_val = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
        chunk_idx = torch.empty(rows * chunks, dtype=torch.int32, device=logits.device)
        _run("cie_argmax", load_library().cie_argmax(_stream(), _ptr(logits), _ptr(chunk_val), _ptr(chunk_idx),
                                                     _ptr(out), _i(rows), _i(vocab), _i(vocab), _i(ARGMAX_CHUNK)))
        return out
    if temperature is not None:
        _gpu("temperature", temperature, torch.float32, 1)
        if not (uniform is not None):
            raise ValueError("temperature sampling needs the uniform numbers")
        _gpu("uniform", uniform, torch.float32, 1)
        if not (temperature.shape[0] == rows and uniform.shape[0] == rows):
            raise ValueError("one temperature and one uniform per row")
    if out is None:
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    _gpu("out", out, torch.int32, 1)
    if not (out.shape[0] == rows):
        raise ValueError(f"out must be [{rows}]")
    if temperature is not None and vocab >= 4 * ARGMAX_CHUNK:
        # a row is taken by many workgroups (one per row reads a vocabulary of 150,000 in a quarter of a millisecond)
        parts = -(-vocab // ARGMAX_CHUNK)
        part_val = torch.empty(rows * parts, dtype=torch.float32, device=logits.device)
        part_idx = torch.empty(rows * parts, dtype=torch.int32, device=logits.device)
        part_sum = torch.empty(rows * parts, dtype=torch.float32, device=logits.device)
        _run("cie_sample_parts", load_library().cie_sample_parts(
            _stream(), _ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(part_val), _ptr(part_idx), _ptr(part_sum),
            _ptr(out), _i(rows), _i(vocab), _i(vocab), _i(ARGMAX_CHUNK)))
        return out
    _run("cie_sample", load_library().cie_sample(_stream(), _ptr(logits), _ptr(temperature), _ptr(uniform),
                                                 _ptr(out), _i(rows), _i(vocab), _i(vocab)))
    return out


# ---------------------------------------------------------------------------
# A stream that is averaged over the depth, block-diagonal products, compressed keys, recurrent mixers
def depth_stream(x: torch.Tensor, branch_a: Optional[torch.Tensor] = None, branch_b: Optional[torch.Tensor] = None,
                 mult: float = 1.0, history: Optional[torch.Tensor] = None, newest: int = -1,
                 weights: Optional[torch.Tensor] = None, gains: tuple = (), out_dtype: torch.dtype = torch.float32,
                 eps: float = 1e-6, want_stream: bool = True):
    """One layer boundary of a stream whose layers add two parallel branches and whose next input is a weighted
    average of what the embedding and every layer so far left:

    ``v = x + mult * (branch_a + branch_b)`` (float32; without branches ``v = x``); ``history[newest] = v``;
    with ``weights`` (float32 [terms]) ``v = sum_j weights[j] * history[j]``; then for every gain ``g`` in
    ``gains`` (up to two) the rows ``v / sqrt(mean(v^2) + eps) * g`` in ``out_dtype``.

    x float32 [T, H]; branches [T, H] in ``out_dtype``; history float32 [layers + 1, T, H].  Returns
    ``(stream or None, [normed rows per gain])``; the stream is a new tensor (``want_stream``) unless nothing changed it."""
    _gpu("x", x, torch.float32, 2)
    rows, hidden = x.shape
    if hidden > MAX_NORM_WIDTH:
        raise ValueError(f"rows of up to {MAX_NORM_WIDTH} numbers, not {hidden}")
    for name, branch in (("branch_a", branch_a), ("branch_b", branch_b)):
        if branch is not None:
            _gpu(name, branch, out_dtype, 2)
            if branch.shape != x.shape:
                raise ValueError(f"{name} {tuple(branch.shape)} vs the stream {tuple(x.shape)}")
    if branch_b is not None and branch_a is None:
        raise ValueError("a second branch needs a first")
    terms, stride = 0, 0
    if history is not None:
        _gpu("history", history, torch.float32, 3)
        if tuple(history.shape[1:]) != (rows, hidden) or not -1 <= newest < history.shape[0]:
            raise ValueError(f"history {tuple(history.shape)} does not hold rows of {tuple(x.shape)} at {newest}")
        stride = rows * hidden
    elif newest >= 0:
        raise ValueError("a place in the history needs the history")
    if weights is not None:
        _gpu("weights", weights, torch.float32, 1)
        terms = weights.shape[0]
        if history is None or terms > history.shape[0]:
            raise ValueError(f"{terms} weights for a history of {0 if history is None else history.shape[0]}")
    if len(gains) > 2 or not eps > 0:
        raise ValueError("at most two norms, and a positive eps")
    changed = branch_a is not None or terms > 0
    stream = torch.empty_like(x) if (want_stream and changed) else None
    outs = [torch.empty((rows, hidden), dtype=out_dtype, device=x.device) for _ in gains]
    g = [float(v) for v in gains] + [0.0, 0.0]
    _run("cie_depth_stream", load_library().cie_depth_stream(
        _stream(), _i(_code(out_dtype)), _ptr(x), _ptr(branch_a), _ptr(branch_b), _f(mult), _ptr(history), stride,
        _i(newest), _ptr(weights), _i(terms), _ptr(stream), _ptr(outs[0] if outs else None), _f(g[0]),
        _ptr(outs[1] if len(outs) > 1 else None), _f(g[1]), _i(rows), _i(hidden), _f(eps)))
    return (stream if stream is not None else (x if want_stream else None)), outs


def block_linear(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 a_block: Optional[int] = None, out: Optional[torch.Tensor] = None, out_offset: int = 0,
                 c_block: Optional[int] = None, out_dtype: Optional[torch.dtype] = None,
                 gate: Optional[torch.Tensor] = None, gate_offset: int = 0, a_offset: int = 0) -> torch.Tensor:
    """A block-diagonal product: ``out[m, b, :] = a[m, b, :] @ weight[b].T (+ bias[b])``, times
    ``sigmoid(gate[m, b, :])`` if a gate is given.

    ``a`` [M, >= a_offset + (B-1) * a_block + K] with unit inner stride (block b's K numbers start at column
    ``a_offset + b * a_block``; ``a_block`` defaults to K); ``weight`` [B, N, K]; ``bias`` [B, N].  The result goes to
    columns ``out_offset + b * c_block`` (``c_block`` defaults to N) of ``out``, a new [M, B * N] tensor of ``out_dtype``
    (float32 or ``a``'s type) if none is given.  ``gate`` is laid out like the default result from its column
    ``gate_offset`` on.  float32 sums in one fixed order; float32 operands give a true float32 product."""
    _gpu("weight", weight, a.dtype, 3)
    blocks, n, k = weight.shape
    if not (a.is_cuda and a.dim() == 2 and a.stride(1) == 1 and a.dtype in _CODES):
        raise ValueError("a must be a float32 or bfloat16 GPU matrix with unit inner stride")
    a_block = k if a_block is None else a_block
    m = a.shape[0]
    if a_offset < 0 or a_block < 0 or a.shape[1] < a_offset + (blocks - 1) * a_block + k:
        raise ValueError(f"a {tuple(a.shape)} does not hold {blocks} blocks of {k} numbers {a_block} apart from {a_offset}")
    lda = a.stride(0) if m > 1 else max(a.stride(0), a.shape[1])
    if bias is not None:
        _gpu("bias", bias, a.dtype, 2)
        if tuple(bias.shape) != (blocks, n):
            raise ValueError(f"bias must be {(blocks, n)}")
    c_block = n if c_block is None else c_block
    if out is None:
        out_dtype = out_dtype or a.dtype
        out = torch.empty((m, out_offset + (blocks - 1) * c_block + n), dtype=out_dtype, device=a.device)
    if not (out.is_cuda and out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == m
            and out.dtype in (torch.float32, a.dtype)):
        raise ValueError("out must be a GPU matrix of float32 or a's type with a row per row of a")
    if out_offset < 0 or c_block < n or out.shape[1] < out_offset + (blocks - 1) * c_block + n:
        raise ValueError(f"out {tuple(out.shape)} does not hold {blocks} blocks of {n} results {c_block} apart from {out_offset}")
    ldc = out.stride(0) if m > 1 else max(out.stride(0), out.shape[1])
    ldg = 0
    if gate is not None:
        if not (gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and gate.dtype == a.dtype and gate.shape[0] == m
                and gate.shape[1] >= gate_offset + blocks * n):
            raise ValueError("the gate must be a matrix of a's type with a row per row of a and a number per result")
        ldg = gate.stride(0) if m > 1 else max(gate.stride(0), gate.shape[1])
    esz_a, esz_c = a.element_size(), out.element_size()
    _run("cie_block_linear", load_library().cie_block_linear(
        _stream(), _i(_code(a.dtype)), _i(1 if out.dtype == torch.float32 else 0), a.data_ptr() + a_offset * esz_a, lda,
        a_block, _ptr(weight), _ptr(bias), out.data_ptr() + out_offset * esz_c, ldc, c_block,
        None if gate is None else gate.data_ptr() + gate_offset * esz_a, ldg, n, _i(m), _i(n), _i(k), _i(blocks)))
    return out


def latent_rows(proj: torch.Tensor, weight: torch.Tensor, heads: int, plain: int, turned: int, latent: int,
                width: int, eps: float) -> torch.Tensor:
    """Lay out the rows ``[T, (heads + 2) * width]`` that the rotation-and-cache-write kernel and the attention
    kernels read for a layer whose keys are compressed (``csrc/latent.hip``): per query head its turned part,
    room for its folded plain part and zeros; one key ``[turned part | normed latent | zeros]`` and one value
    ``[zeros | normed latent | zeros]``.  ``proj`` [T, heads * (plain + turned) + latent + turned]."""
    if not (proj.is_cuda and proj.dim() == 2 and proj.stride(1) == 1 and proj.dtype in _CODES):
        raise ValueError("proj must be a float32 or bfloat16 GPU matrix with unit inner stride")
    tokens = proj.shape[0]
    if proj.shape[1] != heads * (plain + turned) + latent + turned or width < turned + latent:
        raise ValueError(f"proj {tuple(proj.shape)} does not fit {heads} heads of {plain}+{turned} and a latent of {latent}+{turned}")
    _gpu("weight", weight, dims=1)
    if weight.shape[0] != latent or weight.dtype not in (proj.dtype, torch.float32):
        raise ValueError("the latent's norm weight does not fit")
    rows = torch.empty((tokens, (heads + 2) * width), dtype=proj.dtype, device=proj.device)
    ldp = proj.stride(0) if tokens > 1 else max(proj.stride(0), proj.shape[1])
    _run("cie_latent_rows", load_library().cie_latent_rows(
        _stream(), _i(_code(proj.dtype)), _i(_code(weight.dtype)), _ptr(proj), ldp, _ptr(weight), _ptr(rows), _i(tokens),
        _i(heads), _i(plain), _i(turned), _i(latent), _i(width), _f(eps)))
    return rows


RETENTION_ROWS = (4, 8, 16, 32)  # rows of a head's memory that one thread keeps in registers
RETENTION_SLICE = 64             # value columns of a head that one workgroup takes
RETENTION_LDS_FLOATS = 15 * 1024
RETENTION_ACTIVATIONS = {None: 0, "silu": 1}   # what queries, keys and values pass through on their way in
RETENTION_GATES = {"silu": 0, "sigmoid": 1}    # the function of the gate columns that multiplies the read-out
RETENTION_BLOCKS_FROM = 16       # tokens a sequence (on average) from which the walk goes in blocks on the matrix cores
RETENTION_BLOCKS_MAX_DIM = 160   # ... for heads whose queries, keys and values of a block fit the LDS
RETENTION_BLOCKS_MAX_BYTES = 2 << 30  # ... and whose blocks' sums fit this much scratch memory


def plan_retention(dim: int, vdim: int, units: int = 1) -> tuple[int, int, int, int, int]:
    """(rows per thread, groups of threads, parts of the rows, value columns per workgroup, tokens per chunk) of
    the retention kernel for heads of ``dim`` x ``vdim`` when ``units`` (sequence, head) pairs run: a workgroup takes
    up to 64 value columns and a part of a head's rows, as many parts as give every compute unit a workgroup;
    workgroups of up to 512 threads."""
    if dim < 1 or vdim < 1 or units < 1:
        raise ValueError("head sizes must be positive")
    piece = min(vdim, RETENTION_SLICE)
    slices = -(-vdim // piece)
    most_groups = max(1, 512 // (-(-piece // 8) * 8))
    parts = max(1, min(compute_units() // (units * slices), -(-dim // 4)))
    parts = max(parts, -(-dim // (most_groups * RETENTION_ROWS[-1])))  # (no more rows than a workgroup can keep)
    share = -(-dim // parts)  # rows of a part
    rows = next((r for r in RETENTION_ROWS if -(-share // r) <= most_groups), None)
    if rows is None:
        raise ValueError(f"heads of {dim} x {vdim} do not fit the retention kernel's registers")
    groups = -(-share // rows)
    parts = -(-dim // (groups * rows))
    per_token = 2 * groups * rows + piece + groups * piece
    threads = -(-piece * groups // 64) * 64
    # (what a chunk holds must fit the LDS, and what a thread fetches ahead of a chunk its registers:
    # six 16-byte pieces of queries and keys and twelve values).  Long chunks: the next chunk's numbers are on
    # their way from memory for as long as the walk over the current one takes.
    chunk = min(48, RETENTION_LDS_FLOATS // per_token, 6 * threads * 4 // (2 * groups * rows), 12 * threads // piece)
    if chunk < 1 or threads > 512:
        raise ValueError(f"heads of {dim} x {vdim} do not fit the retention kernel's LDS")
    return rows, groups, parts, piece, chunk


def retention(proj: torch.Tensor, offsets: tuple[int, int, int, int], cos: Optional[torch.Tensor],
              sin: Optional[torch.Tensor], rot: int, decay: torch.Tensor, state: torch.Tensor, seq_slot: torch.Tensor,
              positions: torch.Tensor, q_start_loc: torch.Tensor, sequences: int, heads: int, dim: int, vdim: int,
              eps: float, key_scale: float, longest_position: int, activation: Optional[str] = None,
              norm_span: int = 1, norm_weight: Optional[torch.Tensor] = None, gate: str = "silu") -> torch.Tensor:
    """Retention over a step's tokens (``csrc/recurrent.hip``; ``positions`` int32 [T] are the tokens' own).
    ``proj`` [T, ...] holds each token's queries, keys
    (heads x dim), values and gates (heads x vdim) from the columns ``offsets`` on; ``state`` float32
    [slots, heads, dim, vdim] is read and written at the sequences' slots; cos/sin float32 [positions, rot/2]
    must reach ``longest_position``.  ``activation="silu"``: queries, keys and values pass through silu on their way
    in.  The read-out is divided by its root mean square over runs of ``norm_span`` heads (1: each head alone;
    ``heads``: the token's whole row), multiplied by ``norm_weight`` (float32 [heads * vdim]) where given, and by
    ``silu`` or ``sigmoid`` (``gate``) of the gate columns.  Steps of ``RETENTION_BLOCKS_FROM`` tokens a sequence and more
    walk in blocks of 32 tokens on the matrix cores in float32 (heads of up to ``RETENTION_BLOCKS_MAX_DIM`` numbers a key,
    scratch of up to ``RETENTION_BLOCKS_MAX_BYTES``), others token by token: the same sums in another order.
    Returns [T, heads * vdim] in ``proj``'s type."""
    if activation not in RETENTION_ACTIVATIONS or gate not in RETENTION_GATES:
        raise ValueError(f"activation is one of {list(RETENTION_ACTIVATIONS)}, gate one of {list(RETENTION_GATES)}")
    if norm_span < 1 or heads % norm_span:
        raise ValueError(f"the norm's runs of {norm_span} heads do not divide {heads} heads")
    if norm_weight is not None:
        _gpu("norm_weight", norm_weight, torch.float32, 1)
        if norm_weight.shape[0] != heads * vdim:
            raise ValueError(f"norm_weight must be [{heads * vdim}], is {tuple(norm_weight.shape)}")
    if not (proj.is_cuda and proj.dim() == 2 and proj.stride(1) == 1 and proj.dtype in _CODES):
        raise ValueError("proj must be a float32 or bfloat16 GPU matrix with unit inner stride")
    tokens = proj.shape[0]
    q_off, k_off, v_off, g_off = offsets
    if max(q_off + heads * dim, k_off + heads * dim, v_off + heads * vdim, g_off + heads * vdim) > proj.shape[1]:
        raise ValueError(f"proj {tuple(proj.shape)} does not hold the heads at {offsets}")
    if rot:
        for name, table in (("cos", cos), ("sin", sin)):
            _gpu(name, table, torch.float32, 2)
            if table.shape[1] != rot // 2 or table.shape[0] <= longest_position:
                raise ValueError(f"{name} {tuple(table.shape)} does not reach position {longest_position} with {rot // 2} pairs")
    _gpu("decay", decay, torch.float32, 1)
    _gpu("state", state, torch.float32, 4)
    if decay.shape[0] != heads or tuple(state.shape[1:]) != (heads, dim, vdim):
        raise ValueError(f"decay {tuple(decay.shape)} / state {tuple(state.shape)} do not fit {heads} heads of {dim} x {vdim}")
    for name, meta, least in (("seq_slot", seq_slot, sequences), ("positions", positions, tokens),
                              ("q_start_loc", q_start_loc, sequences + 1)):
        _gpu(name, meta, torch.int32, 1)
        if meta.shape[0] < least:
            raise ValueError(f"{name} has {meta.shape[0]} entries, {least} are needed")
    rows, groups, parts, piece, chunk = plan_retention(dim, vdim, max(1, sequences * heads))
    # sequences that bring many tokens (prompts' portions) walk in blocks of 32 tokens on the matrix cores, float32
    # operands and sums, every block's own sums at once and only the memory itself in order; steps of few tokens a
    # sequence walk token by token.  (The same sums in another order.)
    padded, vdim16 = -(-dim // 16) * 16, -(-vdim // 16) * 16
    places = tokens // 32 + sequences + 1
    blocks = (tokens >= RETENTION_BLOCKS_FROM * max(sequences, 1) and dim <= RETENTION_BLOCKS_MAX_DIM
              and places * heads * padded * vdim16 * 4 <= RETENTION_BLOCKS_MAX_BYTES)
    sums = None
    if blocks:
        rows, groups, parts = 16, 1, padded // 16
        sums = torch.empty((places, heads, padded, vdim16), dtype=torch.float32, device=proj.device)
    turned = torch.empty((tokens, heads, 2, parts * groups * rows), dtype=torch.float32, device=proj.device)
    raw = torch.empty((2 if blocks else parts, tokens, heads * vdim), dtype=torch.float32, device=proj.device)
    out = torch.empty((tokens, heads * vdim), dtype=proj.dtype, device=proj.device)
    ldp = proj.stride(0) if tokens > 1 else max(proj.stride(0), proj.shape[1])
    _run("cie_retention", load_library().cie_retention(
        _stream(), _i(_code(proj.dtype)), _ptr(proj), ldp, _i(q_off), _i(k_off), _i(v_off), _i(g_off),
        _ptr(cos if rot else None), _ptr(sin if rot else None), _i(rot), _ptr(decay), _ptr(state), _ptr(seq_slot),
        _ptr(positions), _ptr(q_start_loc), _ptr(turned), _ptr(raw), _ptr(out), _i(tokens), _i(sequences), _i(heads), _i(dim), _i(vdim),
        _i(rows), _i(groups), _i(parts), _i(piece), _i(chunk), _f(eps), _f(key_scale),
        _i(RETENTION_ACTIVATIONS[activation]), _i(norm_span), _ptr(norm_weight), _i(RETENTION_GATES[gate]),
        _i(1 if blocks else 0), _ptr(sums)))
    return out


MAX_CONV_TAPS = 16


def causal_conv(x: torch.Tensor, taps_w: torch.Tensor, bias: Optional[torch.Tensor], past: torch.Tensor,
                seq_of_token: torch.Tensor, seq_slot: torch.Tensor, q_start_loc: torch.Tensor,
                activation: Optional[str] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Per channel, ``out[t] = act(sum_j taps_w[c, j] * x[t - (taps - 1) + j] + bias[c])`` within each sequence; the
    inputs before the step come from ``past`` (float32 [slots, max(taps - 1, 1), C], oldest first; zeros for a new
    sequence).  x [T, C] (a view with unit inner stride), taps_w [C, taps].  ``activation``: ``None`` or ``"silu"``;
    ``out_dtype``: x's type, or float32."""
    if not (x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and x.dtype in _CODES):
        raise ValueError("x must be a float32 or bfloat16 GPU matrix with unit inner stride")
    tokens, channels = x.shape
    _gpu("taps_w", taps_w, x.dtype, 2)
    taps = taps_w.shape[1]
    if taps_w.shape[0] != channels or not 1 <= taps <= MAX_CONV_TAPS:
        raise ValueError(f"taps {tuple(taps_w.shape)} for {channels} channels (up to {MAX_CONV_TAPS} taps)")
    if bias is not None:
        _gpu("bias", bias, x.dtype, 1)
        if bias.shape[0] != channels:
            raise ValueError(f"bias must be [{channels}]")
    _gpu("past", past, torch.float32, 3)
    if tuple(past.shape[1:]) != (max(taps - 1, 1), channels):
        raise ValueError(f"past {tuple(past.shape)} must be [slots, {max(taps - 1, 1)}, {channels}]")
    for name, meta in (("seq_of_token", seq_of_token), ("seq_slot", seq_slot), ("q_start_loc", q_start_loc)):
        _gpu(name, meta, torch.int32, 1)
    if seq_of_token.shape[0] < tokens:
        raise ValueError("one sequence index per token")
    if activation not in RETENTION_ACTIVATIONS or out_dtype not in (None, x.dtype, torch.float32):
        raise ValueError(f"activation {activation!r} / out_dtype {out_dtype} are none the convolution has")
    out = torch.empty((tokens, channels), dtype=out_dtype or x.dtype, device=x.device)
    ldx = x.stride(0) if tokens > 1 else max(x.stride(0), channels)
    _run("cie_causal_conv", load_library().cie_causal_conv(
        _stream(), _i(_code(x.dtype)), _ptr(x), ldx, _ptr(taps_w), _ptr(bias), _ptr(past), _ptr(seq_of_token),
        _ptr(seq_slot), _ptr(q_start_loc), _ptr(out), _i(tokens), _i(channels), _i(taps),
        _i(RETENTION_ACTIVATIONS[activation]), _i(1 if out.dtype == torch.float32 else 0)))
    return out


def conv_keep(x: torch.Tensor, past: torch.Tensor, seq_slot: torch.Tensor, q_start_loc: torch.Tensor, sequences: int,
              taps: int) -> None:
    """Moves a causal convolution's state on by a step's inputs ``x`` [T, C]: of what ``past`` (float32 [slots,
    max(taps - 1, 1), C]) held and the step's rows, the last ``taps - 1`` stay.  Runs behind the convolution."""
    if not (x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and x.dtype in _CODES):
        raise ValueError("x must be a float32 or bfloat16 GPU matrix with unit inner stride")
    tokens, channels = x.shape
    _gpu("past", past, torch.float32, 3)
    if tuple(past.shape[1:]) != (max(taps - 1, 1), channels) or not 1 <= taps <= MAX_CONV_TAPS:
        raise ValueError(f"past {tuple(past.shape)} must be [slots, {max(taps - 1, 1)}, {channels}]")
    for name, meta, least in (("seq_slot", seq_slot, sequences), ("q_start_loc", q_start_loc, sequences + 1)):
        _gpu(name, meta, torch.int32, 1)
        if meta.shape[0] < least:
            raise ValueError(f"{name} has {meta.shape[0]} entries for {sequences} sequences")
    ldx = x.stride(0) if tokens > 1 else max(x.stride(0), channels)
    _run("cie_conv_keep", load_library().cie_conv_keep(_stream(), _i(_code(x.dtype)), _ptr(x), ldx, _ptr(past),
                                                       _ptr(seq_slot), _ptr(q_start_loc), _i(sequences), _i(channels),
                                                       _i(taps)))


def gated_recurrence(y_pre: torch.Tensor, x_in: torch.Tensor, u: torch.Tensor, gates: torch.Tensor, block_width: int,
                     rate: torch.Tensor, state: torch.Tensor, past: torch.Tensor, seq_slot: torch.Tensor,
                     q_start_loc: torch.Tensor, sequences: int, taps: int, segments: int = 1) -> torch.Tensor:
    """The gated linear recurrence of ``csrc/recurrent.hip`` over a step's tokens: per channel
    ``a = exp(rate * sigmoid(r))``, ``S = a * S + sqrt(1 - a^2) * sigmoid(i) * u``, ``out = S * gelu_tanh(y_pre)``,
    with r and i from ``gates`` (float32 [T, 2C], per block of ``block_width`` channels its r then its i).  ``state``
    float32 [slots, C]; ``past`` float32 [slots, max(taps - 1, 1), C] is moved on with the step's ``x_in``.
    ``segments`` (1 to 16) stretches of a sequence's tokens run side by side and are joined by the recurrence's
    own linearity (for long portions; the result differs from the walk in order by float32 rounding only)."""
    tokens, channels = u.shape
    for name, t in (("y_pre", y_pre), ("x_in", x_in)):
        if not (t.is_cuda and t.dim() == 2 and t.stride(1) == 1 and t.dtype == u.dtype and tuple(t.shape) == (tokens, channels)):
            raise ValueError(f"{name} must be a [{tokens}, {channels}] view of u's type with unit inner stride")
    _gpu("u", u, dims=2)
    _gpu("gates", gates, torch.float32, 2)
    _gpu("rate", rate, torch.float32, 1)
    _gpu("state", state, torch.float32, 2)
    _gpu("past", past, torch.float32, 3)
    if (tuple(gates.shape) != (tokens, 2 * channels) or rate.shape[0] != channels or state.shape[1] != channels
            or tuple(past.shape[1:]) != (max(taps - 1, 1), channels) or channels % block_width
            or not 1 <= taps <= MAX_CONV_TAPS or not 1 <= segments <= 16):
        raise ValueError("gates, rate, state or past do not fit the channels")
    for name, meta, least in (("seq_slot", seq_slot, sequences), ("q_start_loc", q_start_loc, sequences + 1)):
        _gpu(name, meta, torch.int32, 1)
        if meta.shape[0] < least:
            raise ValueError(f"{name} has {meta.shape[0]} entries for {sequences} sequences")
    out = torch.empty((tokens, channels), dtype=u.dtype, device=u.device)
    ld = lambda t: t.stride(0) if tokens > 1 else max(t.stride(0), channels)
    _run("cie_gated_recurrence", load_library().cie_gated_recurrence(
        _stream(), _i(_code(u.dtype)), _ptr(y_pre), ld(y_pre), _ptr(x_in), ld(x_in), _ptr(u), _ptr(gates),
        _i(block_width), _ptr(rate), _ptr(state), _ptr(past), _ptr(seq_slot), _ptr(q_start_loc), _ptr(out),
        _i(sequences), _i(channels), _i(taps), _i(segments)))
    return out


# ---------------------------------------------------------------------------
WALK_ROWS = (4, 8, 16, 32, 64)   # rows of a memory that one thread of the walk keeps in registers
WALK_MAX_ROWS = 1024
WALK_LDS_BYTES = 48 * 1024
WALK_AHEAD_FROM = 4              # tokens a sequence (on average) from which the walk fetches a chunk's operands a chunk ahead
WALK_BLOCKS_FROM = 16            # tokens a sequence (on average) from which the first form of the walk goes in blocks
WALK_BLOCKS_MAX_BYTES = 2 << 30  # ... while the blocks' sums fit this much scratch memory


def plan_memory_walk(rows: int, cols: int, time_form: bool, units: int = 1) -> tuple[int, int, int, int]:
    """(rows per thread, row groups, columns per workgroup, tokens staged at once) of ``memory_walk`` for a memory
    of ``rows`` x ``cols`` per head, of which ``units`` (sequences x heads) are walked at once.  Rows per thread and
    row groups follow from ``rows`` alone (they fix the order of the read-out's sums): few rows a thread, so that a
    prompt of one sequence still brings several waves to every compute unit.  The columns are cut into more
    workgroups while these are fewer than the compute units."""
    if not (1 <= rows <= WALK_MAX_ROWS and cols >= 1):
        raise ValueError(f"a memory of {rows} x {cols}: up to {WALK_MAX_ROWS} rows")
    per_thread = next(n for n in WALK_ROWS if 16 * n >= rows)
    groups = -(-rows // per_thread)
    slice_cols = 16
    while slice_cols < min(cols, 64) and 2 * slice_cols * groups <= 512:
        slice_cols *= 2
    while slice_cols > 16 and units * -(-cols // slice_cols) < 2 * compute_units():
        slice_cols //= 2
    per_token = groups * (per_thread + 4)
    floats = (4 if time_form else 2) * per_token + slice_cols + groups * slice_cols
    chunk = max(1, min(16, (WALK_LDS_BYTES - 64) // (4 * floats)))
    # (a thread fetches the next chunk's operands into registers while it walks this one: 8 numbers of each row
    # operand and 4 values a thread)
    threads = -(-slice_cols * groups // 64) * 64
    chunk = max(1, min(chunk, 8 * threads // (groups * per_thread), 4 * threads // slice_cols))
    return per_thread, groups, slice_cols, chunk


def memory_walk(decay: torch.Tensor, in_rows: torch.Tensor, out_rows: torch.Tensor, values: torch.Tensor,
                state: torch.Tensor, seq_slot: torch.Tensor, q_start_loc: torch.Tensor, sequences: int, heads: int,
                rows: int, cols: int, heads_per_group: int = 1, bonus: Optional[torch.Tensor] = None,
                value_scale: Optional[torch.Tensor] = None, skip: Optional[torch.Tensor] = None,
                read_first: bool = False, log_decay: Optional[torch.Tensor] = None,
                blocks: Optional[bool] = None) -> torch.Tensor:
    """The walk of ``csrc/memory_walk.hip`` over a step's tokens: per head a float32 memory ``S`` [rows, cols] in
    ``state`` [slots, heads, rows, cols], ``S <- decay * S + in (x) (value * value_scale)`` token by token, and the
    read-out ``y = S^T out + skip * value`` behind the update, or (``read_first``) ``y = (S + (bonus * in) (x) value)^T
    out`` in front of it.  All operands float32 views with unit inner stride: ``decay`` [T, heads] (one per head and
    token) or [T, heads * rows]; ``in_rows``, ``out_rows`` [T, (heads / heads_per_group) * rows]; ``values``
    [T, heads * cols]; ``bonus`` [heads, rows]; ``value_scale`` [T, heads]; ``skip`` [heads].  Returns y, float32
    [T, heads * cols].  With ``log_decay`` (float32 [T, heads], the decays' logarithms; the first form only) sequences
    that bring ``WALK_BLOCKS_FROM`` tokens and more on average are walked in blocks of 32 tokens on the matrix cores
    (``blocks``: force it or forbid it); the sums come in another order, a difference of float32 rounding."""
    tokens = values.shape[0]
    groups_of_heads = heads // heads_per_group
    if heads % heads_per_group:
        raise ValueError(f"{heads} heads in groups of {heads_per_group}")
    per_row = bool(read_first)  # (the read-out in front of the update comes with a decay per row, the other form with one per head)
    for name, t, width in (("decay", decay, heads * rows if per_row else heads), ("in_rows", in_rows, groups_of_heads * rows),
                           ("out_rows", out_rows, groups_of_heads * rows), ("values", values, heads * cols)):
        if not (t.is_cuda and t.dtype == torch.float32 and t.dim() == 2 and t.stride(1) == 1 and tuple(t.shape) == (tokens, width)):
            raise ValueError(f"{name} must be a float32 GPU view [{tokens}, {width}] with unit inner stride, is {tuple(t.shape)} {t.dtype}")
    _gpu("state", state, torch.float32, 4)
    if tuple(state.shape[1:]) != (heads, rows, cols):
        raise ValueError(f"state {tuple(state.shape)} does not hold {heads} memories of {rows} x {cols}")
    if bonus is not None:
        _gpu("bonus", bonus, torch.float32, 2)
        if tuple(bonus.shape) != (heads, rows) or not read_first:
            raise ValueError("the bonus is [heads, rows] and comes with a read-out in front of the update")
    ld_scale = 0
    if value_scale is not None:
        if not (value_scale.is_cuda and value_scale.dtype == torch.float32 and tuple(value_scale.shape) == (tokens, heads)
                and value_scale.stride(1) == 1):
            raise ValueError(f"value_scale must be float32 [{tokens}, {heads}]")
        ld_scale = value_scale.stride(0)
    if skip is not None:
        _gpu("skip", skip, torch.float32, 1)
        if skip.shape[0] != heads:
            raise ValueError(f"skip must be [{heads}]")
    for name, meta, least in (("seq_slot", seq_slot, sequences), ("q_start_loc", q_start_loc, sequences + 1)):
        _gpu(name, meta, torch.int32, 1)
        if meta.shape[0] < least:
            raise ValueError(f"{name} has {meta.shape[0]} entries for {sequences} sequences")
    per_thread, row_groups, slice_cols, chunk = plan_memory_walk(rows, cols, per_row, sequences * heads)
    y = torch.empty((tokens, heads * cols), dtype=torch.float32, device=values.device)
    ld = lambda t: t.stride(0) if tokens > 1 else max(t.stride(0), t.shape[1])
    if blocks is None:
        blocks = tokens >= WALK_BLOCKS_FROM * max(sequences, 1)
    if blocks and log_decay is not None and not read_first and bonus is None and sequences > 0:
        padded, cols16 = -(-rows // 16) * 16, -(-cols // 16) * 16
        panel = min(cols16, 128)
        lds = 4 * (2 * 32 * (padded + 4) + 32 * (panel + 16 if panel % 32 == 0 else panel) + 32 * 36 + 36)
        places = tokens // 32 + sequences + 1
        scratch = places * heads * padded * cols16 * 4
        if lds <= 64 * 1024 and scratch <= WALK_BLOCKS_MAX_BYTES and tokens <= 32 * 65535:
            if not (log_decay.is_cuda and log_decay.dtype == torch.float32 and tuple(log_decay.shape) == (tokens, heads)
                    and log_decay.stride(1) == 1):
                raise ValueError(f"log_decay must be float32 [{tokens}, {heads}]")
            sums = torch.empty(places * heads * padded * cols16, dtype=torch.float32, device=values.device)
            totals = torch.empty(places * heads, dtype=torch.float32, device=values.device)
            _run("cie_memory_walk_blocks", load_library().cie_memory_walk_blocks(
                _stream(), _ptr(log_decay), ld(log_decay), _ptr(in_rows), ld(in_rows), _ptr(out_rows), ld(out_rows),
                _i(heads_per_group), _ptr(values), ld(values), _ptr(value_scale), ld_scale, _ptr(skip), _ptr(state),
                _ptr(seq_slot), _ptr(q_start_loc), _ptr(y), _ptr(sums), _ptr(totals), _i(tokens), _i(sequences), _i(heads),
                _i(rows), _i(cols)))
            return y
    _run("cie_memory_walk", load_library().cie_memory_walk(
        _stream(), _ptr(decay), ld(decay), _ptr(in_rows), ld(in_rows), _ptr(out_rows), ld(out_rows), _i(heads_per_group),
        _ptr(bonus), _ptr(values), ld(values), _ptr(value_scale), ld_scale, _ptr(skip), _ptr(state), _ptr(seq_slot),
        _ptr(q_start_loc), _ptr(y), _i(sequences), _i(heads), _i(rows), _i(cols), _i(per_thread), _i(row_groups),
        _i(slice_cols), _i(chunk), _i(1 if read_first else 0), _i(1 if tokens >= WALK_AHEAD_FROM * max(sequences, 1) else 0)))
    return y


def space_steps(raw: torch.Tensor, bias: torch.Tensor, a_log: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Step sizes and decays of a state-space layer: ``dt = softplus(raw + bias)``, ``exp(-exp(a_log) * dt)`` and the
    decay's logarithm ``-exp(a_log) * dt`` per token and head, all float32 [T, heads].  ``raw`` [T, heads] (a view
    with unit inner stride); bias, a_log float32."""
    if not (raw.is_cuda and raw.dim() == 2 and raw.stride(1) == 1 and raw.dtype in _CODES):
        raise ValueError("raw must be a float32 or bfloat16 GPU matrix with unit inner stride")
    tokens, heads = raw.shape
    for name, t in (("bias", bias), ("a_log", a_log)):
        _gpu(name, t, torch.float32, 1)
        if t.shape[0] != heads:
            raise ValueError(f"{name} must be [{heads}]")
    made = torch.empty((3, tokens, heads), dtype=torch.float32, device=raw.device)
    ld = raw.stride(0) if tokens > 1 else max(raw.stride(0), heads)
    _run("cie_space_steps", load_library().cie_space_steps(_stream(), _i(_code(raw.dtype)), _ptr(raw), ld, _ptr(bias),
                                                           _ptr(a_log), _ptr(made[0]), _ptr(made[1]), _ptr(made[2]),
                                                           _i(tokens), _i(heads)))
    return made[0], made[1], made[2]


def shift_mix(h: torch.Tensor, before: torch.Tensor, mu: torch.Tensor, seq_of_token: torch.Tensor,
              seq_slot: torch.Tensor, q_start_loc: torch.Tensor) -> torch.Tensor:
    """``mixes[s, t] = h[t] + (h[t - 1] - h[t]) * mu[s]`` within each sequence, [n_mix, T, W] in h's type; the row in
    front of a step's first token comes from ``before`` (float32 [slots, W]; zeros for a new sequence), which
    ``time_decay`` moves on.  ``mu`` float32 [n_mix, W]."""
    if not (h.is_cuda and h.dim() == 2 and h.stride(1) == 1 and h.dtype in _CODES):
        raise ValueError("h must be a float32 or bfloat16 GPU matrix with unit inner stride")
    tokens, width = h.shape
    _gpu("before", before, torch.float32, 2)
    _gpu("mu", mu, torch.float32, 2)
    if before.shape[1] != width or mu.shape[1] != width:
        raise ValueError(f"before {tuple(before.shape)} / mu {tuple(mu.shape)} do not fit rows of {width}")
    for name, meta in (("seq_of_token", seq_of_token), ("seq_slot", seq_slot), ("q_start_loc", q_start_loc)):
        _gpu(name, meta, torch.int32, 1)
    if seq_of_token.shape[0] < tokens:
        raise ValueError("one sequence index per token")
    mixes = torch.empty((mu.shape[0], tokens, width), dtype=h.dtype, device=h.device)
    ldh = h.stride(0) if tokens > 1 else max(h.stride(0), width)
    _run("cie_shift_mix", load_library().cie_shift_mix(_stream(), _i(_code(h.dtype)), _ptr(h), ldh, _ptr(before), _ptr(mu),
                                                       _ptr(seq_of_token), _ptr(seq_slot), _ptr(q_start_loc), _ptr(mixes),
                                                       _i(tokens), _i(width), _i(mu.shape[0])))
    return mixes


def time_decay(low: torch.Tensor, w2t: torch.Tensor, w0: torch.Tensor, h: torch.Tensor, before: torch.Tensor,
               seq_of_token: torch.Tensor, seq_slot: torch.Tensor, q_start_loc: torch.Tensor) -> torch.Tensor:
    """``exp(-exp(tanh(low) w2t + w0))``, float32 [T, C]: ``low`` float32 [T, rank], ``w2t`` [rank, C] in h's type
    (the second small product's weight, transposed), ``w0`` float32 [C].  Also leaves the last row of ``h`` of every
    sequence of the step in ``before`` (the token-shift state that ``shift_mix`` reads at the next step)."""
    _gpu("low", low, torch.float32, 2)
    tokens, rank = low.shape
    if not (h.is_cuda and h.dim() == 2 and h.stride(1) == 1 and h.dtype in _CODES and h.shape[0] == tokens):
        raise ValueError("h must be a float32 or bfloat16 GPU matrix with unit inner stride, a row per token")
    _gpu("w2t", w2t, h.dtype, 2)
    channels = w2t.shape[1]
    _gpu("w0", w0, torch.float32, 1)
    _gpu("before", before, torch.float32, 2)
    if w2t.shape[0] != rank or w0.shape[0] != channels or before.shape[1] != h.shape[1]:
        raise ValueError(f"w2t {tuple(w2t.shape)}, w0 {tuple(w0.shape)}, before {tuple(before.shape)} do not fit")
    for name, meta in (("seq_of_token", seq_of_token), ("seq_slot", seq_slot), ("q_start_loc", q_start_loc)):
        _gpu(name, meta, torch.int32, 1)
    decay = torch.empty((tokens, channels), dtype=torch.float32, device=low.device)
    ldh = h.stride(0) if tokens > 1 else max(h.stride(0), h.shape[1])
    _run("cie_time_decay", load_library().cie_time_decay(
        _stream(), _i(_code(h.dtype)), _ptr(low), _ptr(w2t), _ptr(w0), _ptr(decay), _i(tokens), _i(channels), _i(rank),
        _ptr(h), ldh, _ptr(before), _ptr(seq_of_token), _ptr(seq_slot), _ptr(q_start_loc), _i(h.shape[1])))
    return decay


def gated_group_norm(y: torch.Tensor, gate: Optional[torch.Tensor], weight: Optional[torch.Tensor], groups: int,
                     eps: float, out_dtype: torch.dtype, gate_first: bool) -> torch.Tensor:
    """The RMS norm of float32 rows ``y`` [T, W] in ``groups`` equal consecutive parts (each over its own root mean
    square), times ``weight`` (float32 [W]), with ``silu(gate)`` multiplied in front of the norm (``gate_first``) or
    behind it.  ``gate`` [T, W] in ``out_dtype`` (a view with unit inner stride)."""
    _gpu("y", y, torch.float32, 2)
    tokens, width = y.shape
    if groups < 1 or width % groups or not eps > 0 or width + groups > MAX_NORM_WIDTH:
        raise ValueError(f"{groups} groups over rows of {width} with eps {eps}")
    ldg = 0
    if gate is not None:
        if not (gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and gate.dtype == out_dtype
                and tuple(gate.shape) == (tokens, width)):
            raise ValueError(f"gate must be a [{tokens}, {width}] view of {out_dtype} with unit inner stride")
        ldg = gate.stride(0) if tokens > 1 else max(gate.stride(0), width)
    if weight is not None:
        _gpu("weight", weight, torch.float32, 1)
        if weight.shape[0] != width:
            raise ValueError(f"weight must be [{width}]")
    out = torch.empty((tokens, width), dtype=out_dtype, device=y.device)
    _run("cie_gated_group_norm", load_library().cie_gated_group_norm(
        _stream(), _i(_code(out_dtype)), _ptr(y), _ptr(gate), ldg, _ptr(weight), _ptr(out), _i(tokens), _i(width),
        _i(groups), _f(eps), _i(1 if gate_first else 0)))
    return out


# ---------------------------------------------------------------------------
def branch_norm_add(residual: torch.Tensor, branch: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                    out_dtype: torch.dtype, parts: Optional[torch.Tensor] = None, want_rows: bool = True,
                    branch_gate: Optional[torch.Tensor] = None, part_weight: Optional[torch.Tensor] = None,
                    branch2: Optional[torch.Tensor] = None, scales: tuple[float, float] = (1.0, 1.0),
                    next_weight: Optional[torch.Tensor] = None):
    """``residual += y / sqrt(mean(y^2) + eps) * weight`` with ``y = scales[0] * branch * sigmoid(branch_gate) +
    scales[1] * branch2 + sum_p part_weight[:, p] * parts[:, p]`` (whatever of it is given), row by row, in float32
    and in place.  ``branch``, ``branch2`` [T, H] float32 or ``out_dtype``; ``branch_gate`` float32 [T] (logits, any
    stride); ``parts`` float32 [T, P, H]; ``part_weight`` float32 [T, P]; ``weight`` float32 [H] as it multiplies.
    Returns the new stream rounded to ``out_dtype`` (``want_rows``), which is what a sublayer that reads the stream
    itself takes; with ``next_weight`` (float32 [H]) a pair of that and the RMS norm of the new stream under that
    weight, in ``out_dtype``."""
    _gpu("residual", residual, torch.float32, 2)
    tokens, hidden = residual.shape
    _gpu("weight", weight, torch.float32, 1)
    if not (weight.shape[0] == hidden and hidden <= MAX_NORM_WIDTH and eps > 0):
        raise ValueError(f"weight {tuple(weight.shape)}, hidden {hidden}, eps {eps} do not fit the norm kernel")
    if branch is None and parts is None and branch2 is None:
        raise ValueError("nothing to add")
    kinds = set()
    for name, t in (("branch", branch), ("branch2", branch2)):
        if t is not None:
            _gpu(name, t, dims=2)
            if not (t.shape == residual.shape and t.dtype in (torch.float32, out_dtype)):
                raise ValueError(f"{name} {tuple(t.shape)} {t.dtype} does not fit {tuple(residual.shape)} {out_dtype}")
            kinds.add(t.dtype)
    if len(kinds) > 1:
        raise ValueError("the two branches must be of one type")
    gate_stride = 1
    if branch_gate is not None:
        if not (branch_gate.is_cuda and branch_gate.dtype == torch.float32 and branch_gate.dim() == 1):
            raise ValueError("branch_gate must be a float32 GPU vector")
        if branch is None or branch_gate.shape[0] != tokens:
            raise ValueError("a gate comes with a branch, one logit per row")
        gate_stride = max(branch_gate.stride(0), 1)
    n_parts = 0
    if parts is not None:
        _gpu("parts", parts, torch.float32, 3)
        if not (parts.shape[0] == tokens and parts.shape[2] == hidden):
            raise ValueError(f"parts {tuple(parts.shape)} do not fit {tuple(residual.shape)}")
        n_parts = parts.shape[1]
    if part_weight is not None:
        _gpu("part_weight", part_weight, torch.float32)
        if parts is None or part_weight.numel() != tokens * n_parts:
            raise ValueError("part weights come with parts, one per part and row")
    normed = None
    if next_weight is not None:
        _gpu("next_weight", next_weight, torch.float32, 1)
        if next_weight.shape[0] != hidden:
            raise ValueError(f"next_weight must be [{hidden}]")
        normed = torch.empty((tokens, hidden), dtype=out_dtype, device=residual.device)
    rows = torch.empty((tokens, hidden), dtype=out_dtype, device=residual.device) if want_rows else None
    kind = kinds.pop() if kinds else torch.float32
    _run("cie_branch_norm_add", load_library().cie_branch_norm_add(
        _stream(), _i(_code(kind)), _i(_code(out_dtype)), _ptr(residual), _ptr(branch), _ptr(branch_gate),
        _i(gate_stride), _ptr(branch2), _f(scales[0]), _f(scales[1]), _ptr(parts), _ptr(part_weight), _i(n_parts),
        _ptr(weight), _ptr(rows), _i(tokens), _i(hidden), _f(eps), _ptr(next_weight), _ptr(normed)))
    return rows if next_weight is None else (rows, normed)


def group_norm_add(residual: torch.Tensor, branch: Optional[torch.Tensor], weight: torch.Tensor, groups: int, eps: float,
                   out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, branch_gate: Optional[torch.Tensor] = None,
                   parts: Optional[torch.Tensor] = None, part_weight: Optional[torch.Tensor] = None,
                   plus: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``residual += branch * sigmoid(branch_gate) + sum_p part_weight[:, p] * parts[:, p] + plus`` (whatever of it
    is given; float32, in place unless ``rows``), then the RMS norm of every row in ``groups`` equal consecutive
    parts, each over its own root mean square, the whole times ``weight`` (float32 [H]).  ``branch`` [T, H] float32
    or ``out_dtype``; ``branch_gate`` float32 [T] (logits; any stride); ``parts`` float32 [T, P, H]; ``part_weight`` float32
    [T, P]; ``plus`` float32 [T, H].  With ``rows`` (int32 [n]) only those rows come back, in that order."""
    _gpu("residual", residual, torch.float32, 2)
    tokens, hidden = residual.shape
    _gpu("weight", weight, torch.float32, 1)
    if not (weight.shape[0] == hidden and hidden + groups <= MAX_NORM_WIDTH and eps > 0):
        raise ValueError(f"weight {tuple(weight.shape)}, hidden {hidden}, eps {eps} do not fit the norm kernel")
    if groups < 1 or hidden % groups:
        raise ValueError(f"{groups} groups do not divide a row of {hidden}")
    if branch is not None:
        _gpu("branch", branch, dims=2)
        if not (branch.shape == residual.shape and branch.dtype in (torch.float32, out_dtype)):
            raise ValueError(f"branch {tuple(branch.shape)} {branch.dtype} does not fit {tuple(residual.shape)} {out_dtype}")
    gate_stride = 1
    if branch_gate is not None:
        # (one logit per row; the rows may lie apart, as the first column of a wider product's result does)
        if not (branch_gate.is_cuda and branch_gate.dtype == torch.float32 and branch_gate.dim() == 1):
            raise ValueError("branch_gate must be a float32 GPU vector")
        if branch is None or branch_gate.shape[0] != tokens:
            raise ValueError("a gate comes with a branch, one logit per row")
        gate_stride = max(branch_gate.stride(0), 1)
    n_parts = 0
    if parts is not None:
        _gpu("parts", parts, torch.float32, 3)
        if not (parts.shape[0] == tokens and parts.shape[2] == hidden):
            raise ValueError(f"parts {tuple(parts.shape)} do not fit {tuple(residual.shape)}")
        n_parts = parts.shape[1]
    if part_weight is not None:
        _gpu("part_weight", part_weight, torch.float32)
        if parts is None or part_weight.numel() != tokens * n_parts:
            raise ValueError("part weights come with parts, one per part and row")
    if plus is not None:
        _gpu("plus", plus, torch.float32, 2)
        if plus.shape != residual.shape:
            raise ValueError(f"plus {tuple(plus.shape)} vs residual {tuple(residual.shape)}")
    n_out = tokens
    if rows is not None:
        _gpu("rows", rows, torch.int32, 1)
        n_out = rows.shape[0]
    out = torch.empty((n_out, hidden), dtype=out_dtype, device=residual.device)
    _run("cie_group_norm_add", load_library().cie_group_norm_add(
        _stream(), _i(_code(branch.dtype if branch is not None else out_dtype)), _i(_code(out_dtype)), _ptr(residual),
        _ptr(branch), _ptr(branch_gate), _i(gate_stride), _ptr(parts), _ptr(part_weight), _i(n_parts), _ptr(plus), _ptr(weight),
        _ptr(out), _ptr(rows), _i(n_out), _i(hidden), _i(groups), _f(eps)))
    return out


def clamped_glu(gate_up: torch.Tensor, limit: float, alpha: float, offset: float, cubic: float = 0.0) -> torch.Tensor:
    """``g * sigmoid(alpha * (g + cubic * g^3)) * (u + offset)`` with ``g = min(gate, limit)``,
    ``u = clamp(up, -limit, limit)`` for gate_up [T, 2I] (gate half first).  ``cubic = 0`` is the plain sigmoid
    gate; ``alpha = 2 sqrt(2 / pi)`` with ``cubic = 0.044715`` is the tanh form of gelu."""
    _gpu("gate_up", gate_up, dims=2)
    tokens, twice = gate_up.shape
    if twice % 2 or not limit > 0:
        raise ValueError(f"gate_up rows must be even and the limit positive, got {twice}, {limit}")
    out = torch.empty((tokens, twice // 2), dtype=gate_up.dtype, device=gate_up.device)
    _run("cie_clamped_glu", load_library().cie_clamped_glu(_stream(), _i(_code(gate_up.dtype)), _ptr(gate_up), _ptr(out),
                                                           _i(tokens), _i(twice // 2), _f(limit), _f(alpha), _f(offset),
                                                           _f(cubic)))
    return out


def soft_cap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x <- cap * tanh(x / cap)`` in place on a float32 tensor."""
    _gpu("x", x, torch.float32)
    if not cap > 0:
        raise ValueError(f"the cap must be positive, got {cap}")
    _run("cie_soft_cap", load_library().cie_soft_cap(_stream(), _ptr(x), _i(x.numel()), _f(cap)))
    return x


# ---------------------------------------------------------------------------
NORM_MODES = {None: 0, "unit": 1, "weight": 2, "whole": 3}
SCORED_MFMA_DIMS = ((64, 64), (128, 128), (64, 128), (128, 64))  # (key, value) head sizes of the matrix-core form


def _check_kv_pools(k_pool: torch.Tensor, v_pool: torch.Tensor, dtype: torch.dtype, kv_heads: int, dim: int,
                    vdim: int) -> int:
    _gpu("k_pool", k_pool, dtype, 4)
    _gpu("v_pool", v_pool, dtype, 4)
    pages, heads, page_size, width = k_pool.shape
    if not (heads == kv_heads and width == dim and tuple(v_pool.shape) == (pages, kv_heads, vdim, page_size)):
        raise ValueError(f"pools {tuple(k_pool.shape)}, {tuple(v_pool.shape)} do not fit {kv_heads} heads of {dim} and {vdim}")
    return page_size


def heads_prepare(proj: torch.Tensor, offsets: tuple[int, int, int], q_heads: int, kv_heads: int, dim: int, vdim: int,
                  kernel_dim: int, kernel_vdim: int, norm: Optional[str], q_weight: Optional[torch.Tensor],
                  k_weight: Optional[torch.Tensor], eps: float, temperature: Optional[tuple[float, int]],
                  positions: torch.Tensor, seq_of_token: torch.Tensor, seq_slot: torch.Tensor,
                  block_table: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, tokens: int,
                  write_kv: bool = True, rotary: Optional[tuple] = None) -> torch.Tensor:
    """From projected rows ``proj`` [T, >= ...] (queries at column ``offsets[0]``, keys at ``offsets[1]``, values at
    ``offsets[2]``, heads of ``dim`` / ``dim`` / ``vdim`` numbers) to queries ``[T, q_heads * kernel_dim]`` and the
    token's cache entries: per-head RMS norm of queries and keys (``norm``: ``None``, ``"unit"`` or ``"weight"`` with
    float32 weights [dim]; or ``"whole"``: over all query heads together and over all key heads together, weights
    [q_heads * dim] and [kv_heads * dim]), the queries times ``1 + coef * ln(floor((p + 1) / every) + 1)`` (``temperature = (coef,
    every)``), heads zero-padded up to the kernels' sizes.  ``rotary = (cos, sin, rot, neighbours)``: after the norm
    the first ``rot`` numbers of every query and key head turn by the token's position, in pairs of neighbours
    ``(2i, 2i + 1)`` or of the halves ``(i, i + rot / 2)``; cos and sin are float32 ``[positions, rot / 2]`` and must
    reach every position of the step (the caller sees to that)."""
    if not (proj.is_cuda and proj.dim() == 2 and proj.stride(1) == 1):
        raise ValueError("proj must be 2-d on the GPU with unit inner stride")
    dtype = proj.dtype
    q_off, k_off, v_off = offsets
    need = q_off + q_heads * dim
    if write_kv:
        need = max(need, k_off + kv_heads * dim, v_off + kv_heads * vdim)
    if not (proj.shape[0] >= tokens and proj.shape[1] >= need and min(offsets) >= 0):
        raise ValueError(f"proj {tuple(proj.shape)} too small for {tokens} tokens of {need} numbers")
    if norm not in NORM_MODES:
        raise ValueError(f"norm must be one of {list(NORM_MODES)}, got {norm!r}")
    if norm in ("weight", "whole"):
        # ("whole": one root mean square over all query heads of a token and one over all its key heads, a weight per
        # number of the projection; a call that writes no keys needs no key weight)
        for name, w, heads in (("q_weight", q_weight, q_heads), ("k_weight", k_weight, kv_heads)):
            if w is None and name == "k_weight" and not write_kv:
                continue
            if w is None:
                raise ValueError(f"{name} is missing")
            _gpu(name, w, torch.float32, 1)
            if w.shape[0] != (dim if norm == "weight" else heads * dim):
                raise ValueError(f"{name} {tuple(w.shape)} does not fit heads of {dim} under the {norm!r} norm")
    if kernel_dim < dim or kernel_vdim < vdim:
        raise ValueError("the kernels' head sizes must hold the projection's")
    page_size = _check_kv_pools(k_pool, v_pool, dtype, kv_heads, kernel_dim, kernel_vdim)
    _gpu("block_table", block_table, torch.int32, 2)
    for name, meta in (("positions", positions), ("seq_of_token", seq_of_token)):
        _gpu(name, meta, torch.int32, 1)
        if not (meta.shape[0] >= tokens):
            raise ValueError(f"{name} has {meta.shape[0]} entries for {tokens} tokens")
    _gpu("seq_slot", seq_slot, torch.int32, 1)
    coef, every = temperature if temperature else (0.0, 0)
    if temperature and every < 1:
        raise ValueError("the temperature's period must be positive")
    cos = sin = None
    rot, neighbours = 0, False
    if rotary is not None:
        cos, sin, rot, neighbours = rotary
        if rot < 2 or rot % 2 or rot > dim:
            raise ValueError(f"{rot} turning numbers in heads of {dim}: even, at least 2, at most the head")
        for name, table in (("cos", cos), ("sin", sin)):
            _gpu(name, table, torch.float32, 2)
            if table.shape[1] != rot // 2 or not table.is_contiguous():
                raise ValueError(f"{name} {tuple(table.shape)} does not hold {rot // 2} pairs per position")
    q_out = torch.empty((tokens, q_heads * kernel_dim), dtype=dtype, device=proj.device)
    _run("cie_heads_prepare", load_library().cie_heads_prepare(
        _stream(), _i(_code(dtype)), _ptr(proj), _i(proj.stride(0)), _i(q_off), _i(k_off), _i(v_off), _ptr(q_weight),
        _ptr(k_weight), _i(NORM_MODES[norm]), _f(eps), _f(coef), _i(every), _ptr(positions), _ptr(seq_of_token),
        _ptr(seq_slot), _ptr(block_table), _i(block_table.shape[1]), _ptr(q_out), _ptr(k_pool), _ptr(v_pool),
        _i(tokens), _i(q_heads), _i(kv_heads), _i(dim), _i(vdim), _i(kernel_dim), _i(kernel_vdim), _i(page_size),
        _i(1 if write_kv else 0), _ptr(cos), _ptr(sin), _i(rot), _i(1 if neighbours else 0)))
    return q_out


def _check_score_shape(q_heads: int, slopes, sinks, softcap, window=None, chunk=None, keep_first=0) -> None:
    if chunk is not None and (chunk < 1 or window):
        raise ValueError(f"chunks hold at least one token and stand in a window's place, got chunk {chunk}, window {window}")
    if keep_first < 0 or (keep_first and not window):
        raise ValueError(f"kept first keys ({keep_first}) are a count and come with a window")
    for name, t in (("slopes", slopes), ("sinks", sinks)):
        if t is not None:
            _gpu(name, t, torch.float32, 1)
            if t.shape[0] != q_heads:
                raise ValueError(f"{name} must be [{q_heads}], is {tuple(t.shape)}")
    if softcap is not None and not softcap > 0:
        raise ValueError(f"the cap on the scores must be positive, got {softcap}")


def _check_gate(gate, tokens: int, q_heads: int, dtype: torch.dtype) -> int:
    if gate is None:
        return 0
    if not (gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and gate.dtype == dtype
            and gate.shape[0] >= tokens and gate.shape[1] >= q_heads):
        raise ValueError(f"gate {tuple(gate.shape)} {gate.dtype} does not hold {tokens} rows of {q_heads} heads")
    return gate.stride(0)


def scored_attention_generic(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, block_table: torch.Tensor,
                             positions: torch.Tensor, seq_of_token: torch.Tensor, seq_slot: torch.Tensor, tokens: int,
                             q_heads: int, kv_heads: int, dim: int, vdim: int, window: Optional[int], scale: float,
                             softcap: Optional[float] = None, slopes: Optional[torch.Tensor] = None,
                             sinks: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                             chunk: Optional[int] = None, keep_first: int = 0) -> torch.Tensor:
    """Attention of each token over its request's cached keys with shaped scores (see ``csrc/attention_scored.hip``;
    ``chunk``: a token sees the keys of its own chunk of that many positions, counted from position 0, up to itself;
    ``keep_first``: beside its window a token sees the first that many keys of its sequence):
    ``q`` [T, q_heads * dim]; returns [T, q_heads * vdim].  ``gate`` [T, >= q_heads] (a view is fine): head h's output
    is multiplied by ``sigmoid(gate[t, h])``.  float32 or bfloat16."""
    _gpu("q", q, dims=2)
    if not (q.shape == (tokens, q_heads * dim) and q_heads % kv_heads == 0 and dim % 8 == 0 and vdim % 8 == 0
            and dim <= 256 and vdim <= 256):
        raise ValueError(f"q {tuple(q.shape)} does not fit {tokens} tokens of {q_heads} heads of {dim} (multiples of 8 up to 256)")
    page_size = _check_kv_pools(k_pool, v_pool, q.dtype, kv_heads, dim, vdim)
    _gpu("block_table", block_table, torch.int32, 2)
    for name, meta in (("positions", positions), ("seq_of_token", seq_of_token)):
        _gpu(name, meta, torch.int32, 1)
        if not (meta.shape[0] >= tokens):
            raise ValueError(f"{name} has {meta.shape[0]} entries for {tokens} tokens")
    _gpu("seq_slot", seq_slot, torch.int32, 1)
    _check_score_shape(q_heads, slopes, sinks, softcap, window, chunk, keep_first)
    gate_stride = _check_gate(gate, tokens, q_heads, q.dtype)
    out = torch.empty((tokens, q_heads * vdim), dtype=q.dtype, device=q.device)
    _run("cie_scored_attention_generic", load_library().cie_scored_attention_generic(
        _stream(), _i(_code(q.dtype)), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), _i(block_table.shape[1]),
        _ptr(positions), _ptr(seq_of_token), _ptr(seq_slot), _ptr(gate), _i(gate_stride), _ptr(out), _i(tokens),
        _i(q_heads), _i(kv_heads), _i(dim), _i(vdim), _i(page_size), _i(window or 0), _f(scale), _f(softcap or 0.0),
        _ptr(slopes), _ptr(sinks), _i(chunk or 0), _i(keep_first)))
    return out


def scored_attention_mfma(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, block_table: torch.Tensor,
                          tile_seq: Optional[torch.Tensor], tile_q0: Optional[torch.Tensor], n_tiles: int,
                          seq_slot: torch.Tensor, seq_start: torch.Tensor, seq_q_len: torch.Tensor,
                          q_start_loc: torch.Tensor, tokens: int, q_heads: int, kv_heads: int, dim: int, vdim: int,
                          tokens_per_tile: int, row_tiles: int, window: Optional[int], scale: float,
                          softcap: Optional[float] = None, slopes: Optional[torch.Tensor] = None,
                          sinks: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                          n_splits: int = 1, keys_per_split: int = 0, chunk: Optional[int] = None,
                          keep_first: int = 0) -> torch.Tensor:
    """The same on the matrix cores (bfloat16, (dim, vdim) in ``SCORED_MFMA_DIMS``, pages of a power of two >= 4):
    tiles of ``tokens_per_tile`` consecutive tokens of one sequence (``tile_seq``, ``tile_q0`` int32 [n_tiles]; both
    ``None``: tile i is sequence i's first), whose rows times the heads per key head fill ``row_tiles`` tiles of 16.
    ``n_splits > 1``: every tile's keys in that many shares of ``keys_per_split`` (a multiple of 128; the shares must
    cover the longest range of keys a tile sees), a workgroup each, joined by a second kernel."""
    _gpu("q", q, torch.bfloat16, 2)
    if not (q.shape == (tokens, q_heads * dim) and q_heads % kv_heads == 0 and (dim, vdim) in SCORED_MFMA_DIMS):
        raise ValueError(f"q {tuple(q.shape)} / heads of {dim}, {vdim} are not what the matrix-core form takes")
    page_size = _check_kv_pools(k_pool, v_pool, q.dtype, kv_heads, dim, vdim)
    if page_size < 4 or page_size & (page_size - 1):
        raise ValueError(f"pages must hold a power of two >= 4 keys, hold {page_size}")
    group = q_heads // kv_heads
    if row_tiles not in (1, 2, 4) or tokens_per_tile < 1 or tokens_per_tile * group > 16 * row_tiles:
        raise ValueError(f"{tokens_per_tile} tokens of {group} heads do not fit {row_tiles} tiles of 16 rows")
    _gpu("block_table", block_table, torch.int32, 2)
    if (tile_seq is None) != (tile_q0 is None):
        raise ValueError("tile_seq and tile_q0 come together")
    if tile_seq is not None:
        for name, t in (("tile_seq", tile_seq), ("tile_q0", tile_q0)):
            _gpu(name, t, torch.int32, 1)
            if t.shape[0] < n_tiles:
                raise ValueError(f"{name} has {t.shape[0]} entries for {n_tiles} tiles")
    sequences = seq_slot.shape[0]
    for name, meta, least in (("seq_slot", seq_slot, 1), ("seq_start", seq_start, sequences),
                              ("seq_q_len", seq_q_len, sequences), ("q_start_loc", q_start_loc, sequences)):
        _gpu(name, meta, torch.int32, 1)
        if meta.shape[0] < least:
            raise ValueError(f"{name} has {meta.shape[0]} entries for {sequences} sequences")
    if tile_seq is None and n_tiles > sequences:
        raise ValueError(f"{n_tiles} tiles for {sequences} sequences")
    _check_score_shape(q_heads, slopes, sinks, softcap, window, chunk, keep_first)
    gate_stride = _check_gate(gate, tokens, q_heads, q.dtype)
    out = torch.empty((tokens, q_heads * vdim), dtype=q.dtype, device=q.device)
    part_o = part_ml = None
    if n_splits > 1:
        if keys_per_split < 128 or keys_per_split % 128:
            raise ValueError(f"shares of the keys are multiples of 128, got {keys_per_split}")
        units = n_tiles * kv_heads * n_splits * 16 * row_tiles
        part_o = torch.empty(units * vdim, dtype=torch.float32, device=q.device)
        part_ml = torch.empty(units * 2, dtype=torch.float32, device=q.device)
    elif n_splits != 1:
        raise ValueError("n_splits must be positive")
    _run("cie_scored_attention_mfma", load_library().cie_scored_attention_mfma(
        _stream(), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), _i(block_table.shape[1]), _ptr(tile_seq),
        _ptr(tile_q0), _i(n_tiles), _ptr(seq_slot), _ptr(seq_start), _ptr(seq_q_len), _ptr(q_start_loc), _ptr(gate),
        _i(gate_stride), _ptr(out), _i(q_heads), _i(kv_heads), _i(dim), _i(vdim), _i(page_size), _i(tokens_per_tile),
        _i(row_tiles), _i(window or 0), _f(scale), _f(softcap or 0.0), _ptr(slopes), _ptr(sinks), _i(n_splits),
        _i(keys_per_split), _ptr(part_o), _ptr(part_ml), _i(chunk or 0), _i(keep_first)))
    return out


# ---------------------------------------------------------------------------
MAX_EXPERTS = 1024
EXPERT_TILE_ROWS = (16, 32, 64, 128)  # rows of one expert that a workgroup of the matrix-core forms takes (128: through LDS)


class ExpertRoute:
    """What ``experts_route`` leaves on the device for the expert products of one step."""

    __slots__ = ("pair_expert", "pair_weight", "sorted", "tile_expert", "tile_begin", "tile_count", "n_tiles",
                 "max_tiles", "tile_rows", "top", "pairs", "real", "pair_expert_outputs")


MAX_EXPERT_GROUPS = 64


def experts_route(logits: torch.Tensor, top: int, tile_rows: int = 16, real: Optional[int] = None,
                  scoring: str = "sigmoid", correction: Optional[torch.Tensor] = None,
                  groups: Optional[tuple[int, int]] = None, normalize: bool = False, scale: float = 1.0) -> ExpertRoute:
    """Scores ``sigmoid(logits)`` (float32 [T, E]), the ``top`` largest per token (ranked by the logits, which order
    the scores and do not saturate; lowest index first among equals),
    and the (token, choice) pairs sorted by expert in tiles of at most ``tile_rows`` rows.  Nothing comes back to
    the host: grids are sized for ``max_tiles`` and the kernels read the true count.

    What else a router may ask for: ``scoring="softmax"`` (scores are the softmax over all E outputs);
    ``correction`` (float32 [E], added to the scores for the choice only); ``groups=(count, keep)`` (the outputs form
    ``count`` equal runs of neighbours, a run counts by its largest choice score, and only outputs of the ``keep``
    best runs can be chosen); ``normalize`` (the chosen scores divided by their sum + 1e-20, times ``scale``);
    ``real`` (only the first ``real`` outputs are experts with weights: pairs of the others get no tiles, and
    ``experts_forward`` hands their token's row on as it is)."""
    _gpu("logits", logits, torch.float32, 2)
    tokens, experts = logits.shape
    if not (1 <= top <= experts <= MAX_EXPERTS and tile_rows >= 1):
        raise ValueError(f"{top} of {experts} experts (at most {MAX_EXPERTS}) in tiles of {tile_rows}")
    real = experts if real is None else real
    if not 0 <= real <= experts or scoring not in ("sigmoid", "softmax"):
        raise ValueError(f"{real} experts of {experts} outputs with {scoring!r} scores")
    if correction is not None:
        _gpu("correction", correction, torch.float32, 1)
        if correction.shape[0] != experts:
            raise ValueError(f"correction must be [{experts}], is {tuple(correction.shape)}")
    count, keep = groups if groups else (1, 1)
    if count > 1 and not (count <= MAX_EXPERT_GROUPS and experts % count == 0 and 1 <= keep <= count
                          and top <= keep * (experts // count)):
        raise ValueError(f"{count} groups of which {keep} are kept do not fit {top} of {experts} outputs")
    route = ExpertRoute()
    pairs = tokens * top
    route.pairs, route.top, route.tile_rows, route.real = pairs, top, tile_rows, real
    route.pair_expert_outputs = experts  # how many outputs the router has; those from ``real`` on have no weights
    route.max_tiles = min(pairs, pairs // tile_rows + real)
    ints = torch.empty(2 * pairs + 3 * max(route.max_tiles, 1) + 1, dtype=torch.int32, device=logits.device)
    route.pair_expert, route.sorted = ints[:pairs], ints[pairs: 2 * pairs]
    base = 2 * pairs
    width = max(route.max_tiles, 1)
    route.tile_expert, route.tile_begin, route.tile_count = (ints[base + i * width: base + (i + 1) * width] for i in range(3))
    route.n_tiles = ints[base + 3 * width:]
    route.pair_weight = torch.empty(pairs, dtype=torch.float32, device=logits.device)
    _run("cie_experts_route", load_library().cie_experts_route(
        _stream(), _ptr(logits), _i(tokens), _i(experts), _i(top), _i(tile_rows), _ptr(route.pair_expert),
        _ptr(route.pair_weight), _ptr(route.sorted), _ptr(route.tile_expert), _ptr(route.tile_begin),
        _ptr(route.tile_count), _ptr(route.n_tiles), _i(real), _i(1 if scoring == "softmax" else 0), _ptr(correction),
        _i(count), _i(keep), _i(1 if normalize else 0), _f(scale)))
    return route


def experts_forward(x: torch.Tensor, route: ExpertRoute, w_gate_up: torch.Tensor, w_down: torch.Tensor, limit: float,
                    alpha: float, offset: float, mfma: bool, weight_input: bool = True) -> torch.Tensor:
    """The chosen experts' outputs, float32 ``[T, top, hidden]``: row (t, k) is expert ``k`` of token t run on
    ``weight * x[t]``, or, with ``weight_input=False``, on ``x[t]`` itself (whoever sums the rows then applies
    ``route.pair_weight``).  ``w_gate_up`` [E, 2 * ff, hidden] (gate rows first), ``w_down`` [E, hidden, ff].  A pair
    whose choice lies behind the experts that have weights (``route.real``) gets ``x[t]`` as its row."""
    _gpu("x", x, dims=2)
    tokens, hidden = x.shape
    _gpu("w_gate_up", w_gate_up, x.dtype, 3)
    _gpu("w_down", w_down, x.dtype, 3)
    experts, twice, _ = w_gate_up.shape
    ff = twice // 2
    if not (w_gate_up.shape == (experts, 2 * ff, hidden) and w_down.shape == (experts, hidden, ff)
            and tokens * route.top == route.pairs and experts == route.real):
        raise ValueError(f"expert weights {tuple(w_gate_up.shape)}, {tuple(w_down.shape)} do not fit rows {tuple(x.shape)}")
    if mfma and not (x.dtype == torch.bfloat16 and hidden % 8 == 0 and ff % 8 == 0 and route.tile_rows in EXPERT_TILE_ROWS):
        raise ValueError("the matrix-core form takes bfloat16, widths that are multiples of 8 and tiles of 16, 32, 64 or 128 rows")
    if not mfma and route.tile_rows > 16:
        raise ValueError("the plain form takes tiles of up to 16 rows")
    act = torch.empty((route.pairs, ff), dtype=x.dtype, device=x.device)
    parts = torch.empty((tokens, route.top, hidden), dtype=torch.float32, device=x.device)
    lib = load_library()
    rows_in = x
    pair_weight = route.pair_weight if weight_input else None
    if mfma and route.tile_rows == 128:
        # many rows an expert: the rows in sorted order, weights applied, for the form that stages tiles through LDS
        gathered = torch.empty((route.pairs, hidden), dtype=x.dtype, device=x.device)
        _run("cie_experts_gather", lib.cie_experts_gather(_stream(), _ptr(x), _ptr(gathered), _ptr(route.sorted),
                                                          _ptr(pair_weight), _i(route.pairs), _i(route.top), _i(hidden)))
        x = gathered
    _run("cie_experts_gate_up", lib.cie_experts_gate_up(
        _stream(), _i(_code(x.dtype)), _i(1 if mfma else 0), _ptr(x), _ptr(w_gate_up), _ptr(act), _ptr(route.sorted),
        _ptr(pair_weight), _ptr(route.tile_expert), _ptr(route.tile_begin), _ptr(route.tile_count),
        _ptr(route.n_tiles), _i(route.max_tiles), _i(route.tile_rows), _i(route.top), _i(hidden), _i(ff), _f(limit),
        _f(alpha), _f(offset)))
    _run("cie_experts_down", lib.cie_experts_down(
        _stream(), _i(_code(x.dtype)), _i(1 if mfma else 0), _ptr(act), _ptr(w_down), _ptr(parts), _ptr(route.sorted),
        _ptr(route.tile_expert), _ptr(route.tile_begin), _ptr(route.tile_count), _ptr(route.n_tiles),
        _i(route.max_tiles), _i(route.tile_rows), _i(route.top), _i(hidden), _i(ff)))
    if route.real < route.pair_expert_outputs:
        _run("cie_experts_identity", lib.cie_experts_identity(
            _stream(), _i(_code(rows_in.dtype)), _ptr(rows_in), _ptr(route.pair_expert), _i(route.real), _ptr(parts),
            _i(route.pairs), _i(route.top), _i(hidden)))
    return parts
