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
          feed: Optional[torch.Tensor] = None, pool: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t] = float32(table[ids[t]])``; ids int32 [T] (already checked against the vocabulary).
    With ``feed`` (int32 [T]) and ``pool`` (int32): row t takes ``pool[feed[t]]`` as its id where
    ``feed[t] >= 0`` (tokens another kernel left on the device; ``feed[t]`` must index ``pool``)."""
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
    _run("cie_embed", load_library().cie_embed(_stream(), _i(_code(table.dtype)), _ptr(table), _ptr(ids), _ptr(feed),
                                               _ptr(pool if feed is not None else None), _ptr(out), _i(tokens),
                                               _i(hidden), _i(vocab)))
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
