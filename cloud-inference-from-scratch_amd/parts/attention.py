"""Grouped-query softmax attention over the paged cache.

Reference: ``Qwen2Attention.project`` (src/cloud_engine/model.py:103-137),
``apply_rope`` (src/cloud_engine/attention.py:75-85), the KV write before the
read (src/cloud_engine/cache.py:398-413) and the ragged attention of
``kernel.py:324-405``: query head ``h`` reads KV head ``h // group``, scores are
``q.k / sqrt(D)``, a token sees every cached key up to itself.  Here q, k and v
are one fused product, rotation and cache write are one kernel, and sizes, bias
switches, scale, position encoding and an optional window are parameters.
"""

from __future__ import annotations

import math
import warnings
from typing import Optional

import torch

from ..cache.manager import PagedKV
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import Part, build_part, register_part
from .linear import FUSED_ROWS, FUSED_SMALL_ROWS, FUSED_SMALL_WEIGHT, RawRows, linear


class Attention(Part):
    graph_safe = True
    adds_to_residual = True
    folds_next_norm = True  # its output product can leave the next norm's rows short of their scale
    takes_raw_rows = True  # its first product can make the norm of a few rows itself
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qkv_bias: bool, out_bias: bool, position: PartSpec, window: Optional[int] = None,
                 scale: Optional[float] = None) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are no multiple of {num_kv_heads} key heads")
        if head_dim % 8 or head_dim > 256:
            raise ValueError(f"head_dim must be a multiple of 8 up to 256 for the attention kernels, got {head_dim}")
        if window is not None and window < 1:
            raise ValueError("window must be positive")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.qkv_bias = qkv_bias
        self.out_bias = out_bias
        self.window = window
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position = build_part("position", position)
        # A head size that the matrix-core attention does not take (80, 112, 40, ...) runs as the next one it does:
        # the projections' rows of a head are padded with zero rows, which changes no score and no output (the keys'
        # and values' extra dimensions are zeros in the cache, o_proj's extra columns are zeros), and costs that much
        # more cache.  The generic kernel, which takes every size, is 20 (decode) to 180 (a 2,048-token prompt) times
        # slower.  A variant that works on the projected heads (``shape_projection``) sees the heads as they are.
        self.kernel_head_dim = head_dim
        if type(self).shape_projection is Attention.shape_projection:
            self.kernel_head_dim = next((size for size in ops.MFMA_HEAD_DIMS if size >= head_dim), head_dim)

    def cache_need(self) -> PagedKV:
        return PagedKV(self.num_kv_heads, self.kernel_head_dim, self.window)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        q_out = self.num_heads * self.head_dim
        kv_out = self.num_kv_heads * self.head_dim
        out = {
            prefix + "q_proj.weight": TensorSpec((q_out, self.hidden_size)),
            prefix + "k_proj.weight": TensorSpec((kv_out, self.hidden_size)),
            prefix + "v_proj.weight": TensorSpec((kv_out, self.hidden_size)),
            prefix + "o_proj.weight": TensorSpec((self.hidden_size, q_out)),
        }
        if self.qkv_bias:
            out[prefix + "q_proj.bias"] = TensorSpec((q_out,))
            out[prefix + "k_proj.bias"] = TensorSpec((kv_out,))
            out[prefix + "v_proj.bias"] = TensorSpec((kv_out,))
        if self.out_bias:
            out[prefix + "o_proj.bias"] = TensorSpec((self.hidden_size,))
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        names = ("q_proj", "k_proj", "v_proj")
        extra = self.kernel_head_dim - self.head_dim

        def per_head(t: torch.Tensor) -> torch.Tensor:
            # [heads * head_dim, ...] -> [heads * kernel_head_dim, ...], each head followed by zero rows
            if not extra:
                return t
            heads = t.shape[0] // self.head_dim
            padded = t.new_zeros((heads, self.kernel_head_dim) + tuple(t.shape[1:]))
            padded[:, : self.head_dim] = t.reshape((heads, self.head_dim) + tuple(t.shape[1:]))
            return padded.reshape((heads * self.kernel_head_dim,) + tuple(t.shape[1:]))

        self.w_qkv = torch.cat([per_head(tensors[f"{prefix}{n}.weight"]) for n in names], dim=0).contiguous()
        self.b_qkv = (
            torch.cat([per_head(tensors[f"{prefix}{n}.bias"]) for n in names], dim=0).contiguous()
            if self.qkv_bias else None
        )
        self.w_o = per_head(tensors[prefix + "o_proj.weight"].t()).t().contiguous()
        self.b_o = tensors[prefix + "o_proj.bias"].contiguous() if self.out_bias else None
        self.cos, self.sin = self.position.tables(device)

    def warm_up(self, rows: int) -> None:
        blank = lambda width: torch.zeros((rows, width), dtype=self.w_qkv.dtype, device=self.w_qkv.device)
        linear(blank(self.hidden_size), self.w_qkv, self.b_qkv)
        linear(blank(self.num_heads * self.kernel_head_dim), self.w_o, self.b_o)

    def shape_projection(self, qkv: torch.Tensor, batch) -> torch.Tensor:
        """The seam between projection and rotation: what a variant of this mixer does to the projected
        rows ``[tokens, (query heads + 2 key heads) * head_dim]`` (bias added; queries first, then keys,
        then values) before they are rotated and the keys and values go to the cache, such as a norm over
        each query and key head.  The default does nothing, and only a mixer that leaves it so lets the
        projection's own kernel rotate and write the cache."""
        return qkv

    def forward(self, x, batch, view, writes: bool = True, residual: Optional[torch.Tensor] = None,
                next_norm=None):
        if batch.max_context > self.position.max_position and self.position.rotates:
            raise ValueError(
                f"position {batch.max_context - 1} is beyond the rotary table of {self.position.max_position}"
            )
        rows = x.shape[0]
        few = rows <= FUSED_ROWS or (rows <= FUSED_SMALL_ROWS and self.w_qkv.numel() <= FUSED_SMALL_WEIGHT)
        head_dim = self.kernel_head_dim  # what the kernels and the cache see
        # the projection's own kernel rotates whole heads only, and only an untouched projection
        rotary_dim = getattr(self.position, "rotary_dim", self.head_dim) if self.position.rotates else None
        untouched = (type(self).shape_projection is Attention.shape_projection
                     and rotary_dim in (None, head_dim) and head_dim == self.head_dim)
        if isinstance(x, RawRows):
            if untouched and head_dim % 32 == 0 and self.w_qkv.dtype == torch.bfloat16:
                # the product makes the norm of its rows itself
                qkv = ops.gemm_qkv_rope(
                    self.w_qkv, None, self.b_qkv, self.cos, self.sin, batch.positions, batch.seq_of_token,
                    batch.seq_slot, view.block_table, view.k_pool, view.v_pool, self.num_heads, self.num_kv_heads,
                    head_dim, rotate=self.position.rotates, write_kv=writes,
                    folded=(x.residual, x.norm.weight_f32, x.norm.eps))
                context = attend(qkv, batch, view, self.num_heads, self.num_kv_heads, head_dim,
                                 self.window, self.scale)
                return linear(context, self.w_o, self.b_o, into=residual, then_norm=next_norm)
            x = x.complete()
        if (x.dtype == torch.bfloat16 and few and untouched and head_dim % 32 == 0
                and x.shape[1] % 8 == 0 and (rows == 1 or x.stride(0) % 8 == 0)):
            # few rows (where the hand-written product is the faster one): its epilogue rotates and writes the cache
            qkv = ops.gemm_qkv_rope(self.w_qkv, x, self.b_qkv, self.cos, self.sin, batch.positions,
                                    batch.seq_of_token, batch.seq_slot, view.block_table, view.k_pool, view.v_pool,
                                    self.num_heads, self.num_kv_heads, head_dim,
                                    rotate=self.position.rotates, write_kv=writes)
        else:
            qkv = self.shape_projection(linear(x, self.w_qkv, self.b_qkv), batch)
            ops.rope_kv_write(qkv, self.cos, self.sin, batch.positions, batch.seq_of_token, batch.seq_slot,
                              view.block_table, view.k_pool, view.v_pool, self.num_heads, self.num_kv_heads,
                              head_dim, rotate=self.position.rotates, write_kv=writes, rotary_dim=rotary_dim)
        context = attend(qkv, batch, view, self.num_heads, self.num_kv_heads, head_dim,
                         self.window, self.scale)
        return linear(context, self.w_o, self.b_o, into=residual, then_norm=next_norm)


WIDE_DECODE_KEYS = 2048  # contexts from which decode rows go to the four-wave form
# (the four-wave form cuts long contexts for as many workgroups as the GPU has compute units)
FEW_DECODE_UNITS = 8  # (sequence, kv head) pairs below which they do not: parts of one wave fill the GPU better
MANY_DECODE_UNITS = 96  # (sequence, kv head) pairs from which decode rows take the four-wave form at any context
SHARED_DECODE_KEYS = 96  # contexts from which four waves share a decode row's keys without cutting them
SPLIT_MIN_KEYS = 32  # the fewest keys of a one-wave part
SPLIT_DECODE_KEYS = 192  # contexts from which the keys of decode rows are cut into parts at all
JOINED_DECODE_ROWS = 32  # up to this many single-token sequences beside prompt portions ride in the prompt form's launch
PROMPT_SPLIT_KEYS = 512  # the fewest keys of a part when a prompt portion's keys are cut
# (cutting a prompt form's keys aims at as many workgroups as the GPU has compute units)
# Tiles of 64 rows x kv heads (as a share of the compute units) from which prompt portions take the form that
# shares keys and values through LDS: enough to give most compute units a workgroup without cutting the keys (whose parts, 64 KB of sums per tile and kv head, cost that
# form more than they gain it: 512 tokens behind 1,536 keys, 7B heads, 60 us in two parts against 40 us in the form
# of four waves).  Measured at head size 128 (us, four waves -> eight): 2,048 tokens of one prompt 55.7 -> 51.4
# (3B heads), 101 -> 58 (7B), 144 -> 84 (14B); behind 2,048 keys 108 -> 91, 195 -> 135, 284 -> 201; beside 8 single
# tokens 108 -> 64, 138 -> 75, 182 -> 111.
EIGHT_WAVE_TILES = 0.75  # of the compute units
LARGE_TILES_ABOVE = 1.0  # tiles of 128 rows x kv heads (as a share of the compute units) above which that form takes them


_SAID_GENERIC: set = set()  # geometries whose bfloat16 attention was sent to the generic kernel, each said once


def plan_splits(units: int, max_keys: int, target_waves: int = 1024, min_keys: int = 128) -> tuple[int, int]:
    """How many parts to cut a decode tile's keys into so that the GPU is filled:
    (number of splits, keys per split as a multiple of 32)."""
    wanted = max(1, target_waves // max(units, 1))
    splits = min(wanted, max(1, max_keys // min_keys))
    if splits <= 1:
        return 1, 0
    per_split = -(-(-(-max_keys // splits)) // 32) * 32
    return -(-max_keys // per_split), per_split


def attend(qkv: torch.Tensor, batch, view, num_heads: int, num_kv_heads: int, head_dim: int,
           window: Optional[int], scale: float) -> torch.Tensor:
    """Pick the attention kernel for this step's rows.

    bfloat16 with a head size the matrix-core kernel takes: sequences that bring
    one token go to the split-context decode form, prompt portions to the tiled
    form with up to 64 rows per tile (four waves per tile where pages hold at
    least 16 keys, one wave otherwise).  Everything else (float32, other head
    sizes, groups of more than 16 heads, pages of fewer than 4 tokens): the
    generic kernel."""
    group = num_heads // num_kv_heads
    decode_tiles = 1 if group <= 16 else 2 if group <= 32 else 4  # 16-row tiles that hold one token's heads
    page_size = view.page_size
    cus = ops.compute_units()  # compute units of the GPU
    # (a token's heads of one key head share a tile: up to 64 rows, 16 where the head has 256 dimensions)
    if (qkv.dtype != torch.bfloat16 or head_dim not in ops.MFMA_HEAD_DIMS or group > (64 if head_dim <= 128 else 16)
            or page_size < 4 or page_size & (page_size - 1)):
        if qkv.dtype == torch.bfloat16 and (head_dim, group, page_size) not in _SAID_GENERIC:
            # right, and many times slower than the matrix-core forms: said once per geometry, not silently
            _SAID_GENERIC.add((head_dim, group, page_size))
            warnings.warn(f"bfloat16 attention with head size {head_dim}, {group} query heads per key head and pages of "
                          f"{page_size} takes the generic kernel (the matrix-core forms take head sizes "
                          f"{ops.MFMA_HEAD_DIMS}, up to 64 heads per key head, 16 at head size 256, and pages of a power "
                          f"of two >= 4)",
                          RuntimeWarning, stacklevel=2)
        return ops.paged_attention_generic(
            qkv, qkv.stride(0), view.k_pool, view.v_pool, view.block_table, batch.positions,
            batch.seq_of_token, batch.seq_slot, batch.tokens, num_heads, num_kv_heads, head_dim, window, scale)
    out = torch.empty((batch.tokens, num_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    common = (batch.seq_slot, batch.seq_start, batch.seq_q_len, batch.q_start_loc, out, num_heads, num_kv_heads,
              head_dim, window, scale)
    max_keys = batch.max_context if window is None else min(batch.max_context, window + 64)
    wide = page_size >= 16 and scale > 0
    # Prompt portions with enough rows take tiles of 128 rows and eight waves, whose keys and values pass
    # through LDS once per tile.  (A short portion behind a long context also has its keys cut into parts.)
    prompt_tokens = sum(n for n in batch.host_q_lens if n > 1)
    bound = batch.static_plan.max_keys if batch.static_plan is not None else max_keys
    cuts = max(1, bound // PROMPT_SPLIT_KEYS) if wide and window is None else 1  # (a window's keys stay whole)
    big_tiles = -(-prompt_tokens * group // 128) * num_kv_heads
    small_tiles = -(-prompt_tokens * group // 64) * num_kv_heads
    # That form has tiles of 128 rows for eight waves, and tiles of 64 rows for four, two such workgroups to a
    # compute unit, where the larger tiles would not give every unit more than one (isolated kernel, us, 128 rows
    # -> 64: 2,048 tokens of one prompt, 3B heads, 256 large tiles: 50.8 -> 46.8, 1,024 tokens 27.5 -> 24.8; 7B
    # heads, 456 large tiles: 55.3 -> 70.5; heads of 64 dimensions, where the softmax arithmetic per key is the same
    # and the products are half: 2,048 tokens 40.2 -> 33.0, against 43.1 in the form of four waves without LDS).
    eight = (wide and head_dim in (64, 128) and group <= 64 and small_tiles >= max(1, EIGHT_WAVE_TILES * cus))
    lds_row_tiles = 8 if head_dim == 128 and big_tiles > LARGE_TILES_ABOVE * cus else 4

    def decode_form(bound: int, units: int) -> tuple[int, dict]:
        # Decode rows, `units` (sequence, kv head) pairs over up to `bound` keys.  Long contexts: four waves
        # per (sequence, kv head, part of the keys) take the part's blocks in turn with their loads running
        # ahead (15.8 against 18.1 us for 8 x 4,096 keys).  A few pairs do not fill the GPU that way: they take the
        # one-wave form below, whose parts are smaller (one sequence of the 3B shape over 32,000 keys: 333 -> 363
        # tokens/s; from four sequences on the forms are level).
        if wide and bound >= WIDE_DECODE_KEYS and units >= FEW_DECODE_UNITS:
            return ops.TILE_WAVES, dict(target_waves=cus, min_keys=32 * ops.TILE_WAVES)
        # Many pairs fill the GPU by themselves: the same form with the keys whole or in large parts
        # (64 sequences x 2 heads x 256 keys: 9.2 us against 11.1 us with one wave per part)
        if wide and units >= MANY_DECODE_UNITS and bound >= SHARED_DECODE_KEYS:
            return ops.TILE_WAVES, dict(target_waves=4 * cus // ops.TILE_WAVES, min_keys=512)
        # Otherwise one wave per part, parts down to one block of 32 keys (8 x 256 keys: 7.3 us in 8 parts,
        # 10.2 us in 2; 8 x 512 keys: 8.1 us in 16 parts, 10.6 us in 4) ...
        if bound >= SPLIT_DECODE_KEYS:
            return 1, dict(target_waves=4 * cus, min_keys=SPLIT_MIN_KEYS)
        # ... and below some 200 keys, where the merge costs more than it saves, four waves that share a
        # sequence's few blocks inside one workgroup instead of one wave that takes them in turn
        # (8 x 128 keys: 6.5 against 6.9 us, 8 x 160: 7 against 11)
        return (ops.TILE_WAVES if wide and bound >= SHARED_DECODE_KEYS else 1), dict(target_waves=4 * cus, min_keys=bound + 1)

    plan = batch.static_plan
    longest_dev = None
    if plan is not None:
        # a captured step: grids are fixed, lengths live on the device.  Its first sequences bring one token
        # each (tile i is sequence i, no tile lists); the sizes of the keys' parts follow the step's longest
        # context, which the device knows, within the bound the step was captured for
        max_keys = plan.max_keys if window is None else min(plan.max_keys, window + 64)
        longest_dev = plan.max_context
        decode_rows = batch.sequences if plan.decode_rows is None else plan.decode_rows
        joined = wide and not eight and 0 < decode_rows <= JOINED_DECODE_ROWS and decode_rows < batch.sequences
        if decode_rows and not joined:
            decode_waves, split_options = decode_form(max_keys, decode_rows * num_kv_heads)
            n_splits, _ = plan_splits(decode_rows * num_kv_heads, max_keys, **split_options)
            part_o = part_ml = None
            if n_splits > 1:
                part_o, part_ml = _workspaces(qkv.device, decode_rows * num_kv_heads * n_splits, 16 * decode_tiles, head_dim)
            ops.paged_attention_mfma(qkv, qkv.stride(0), view.k_pool, view.v_pool, view.block_table, None,
                                     None, decode_rows, *common, tokens_per_tile=1, row_tiles=decode_tiles,
                                     n_splits=n_splits, max_context_dev=longest_dev, part_o=part_o, part_ml=part_ml,
                                     tile_waves=decode_waves)
        if decode_rows == batch.sequences:
            return out
        n_tiles = 0  # (of the eager decode form below)
    else:
        tile_seq, tile_q0, n_tiles = batch.tiles(1, decode=True)
        # A few single tokens beside prompt portions: one launch (and one merge) of the prompt form for all
        # sequences instead of two of each (8 decode rows and a 64-token portion of the 3B shape: 4.84 -> 4.49 ms
        # a step; 32 rows over 3,000 keys and 256 tokens: 8.9 -> 8.2 ms; with 64 such rows the forms are level)
        # (not beside the form of eight waves, where a tile of one token would leave six of them idle)
        joined = wide and not eight and 0 < n_tiles <= JOINED_DECODE_ROWS and n_tiles < batch.sequences
    if n_tiles and not joined:
        decode_waves, split_options = decode_form(max_keys, n_tiles * num_kv_heads)
        n_splits, per_split = plan_splits(n_tiles * num_kv_heads, max_keys, **split_options)
        part_o = part_ml = None
        if n_splits > 1:
            part_o, part_ml = _workspaces(qkv.device, n_tiles * num_kv_heads * n_splits, 16 * decode_tiles, head_dim)
        ops.paged_attention_mfma(qkv, qkv.stride(0), view.k_pool, view.v_pool, view.block_table, tile_seq, tile_q0,
                                 n_tiles, *common, tokens_per_tile=1, row_tiles=decode_tiles, n_splits=n_splits,
                                 keys_per_split=per_split, part_o=part_o, part_ml=part_ml, tile_waves=decode_waves)
    if wide:
        # the prompt forms: waves share a tile's keys.  More rows per tile re-use each key more often,
        # fewer tiles leave compute units idle: the most rows that still give most units a workgroup, where a
        # short portion behind a long context also has its keys cut (256 tokens behind 3,840 keys, 2 kv heads:
        # 34 us with 64 rows per tile and four parts, 48 us with 16 rows per tile and the keys whole)
        if eight:
            tile_waves, row_tiles = ops.PROMPT_WAVES, lds_row_tiles
        else:
            tile_waves = ops.TILE_WAVES
            row_tiles = 4 if head_dim <= 128 else 1
            while row_tiles > 1 and -(-prompt_tokens * group // (16 * row_tiles)) * num_kv_heads * cuts < 0.75 * cus:
                row_tiles //= 2
    else:
        # one wave per tile; fewer rows where that would leave SIMDs without a wave (about a thousand
        # waves fill the GPU) or where the accumulators of a wide head would spill
        tile_waves = 1
        row_tiles = 2 if head_dim > 128 else 4
        while row_tiles > 1 and (prompt_tokens * group // (16 * row_tiles)) * num_kv_heads < 4 * cus:
            row_tiles //= 2
    while 16 * row_tiles < group:
        row_tiles *= 2
    per_tile = (16 * row_tiles) // group
    tile_seq, tile_q0, n_tiles = batch.tiles(per_tile, decode=None if joined else False)
    if n_tiles:
        # few tiles and many keys: parts of the keys, about as many workgroups as compute units
        n_splits, per_split, part_o, part_ml = 1, 0, None, None
        wanted = min(cuts, int(cus / (n_tiles * num_kv_heads) + 0.5))
        if wanted > 1:
            per_split = -(-(-(-max_keys // wanted)) // 128) * 128
            n_splits = -(-max_keys // per_split)
        if n_splits > 1:
            part_o, part_ml = _workspaces(qkv.device, n_tiles * num_kv_heads * n_splits, 16 * row_tiles, head_dim)
        else:
            per_split = 0
        ops.paged_attention_mfma(qkv, qkv.stride(0), view.k_pool, view.v_pool, view.block_table, tile_seq, tile_q0,
                                 n_tiles, *common, tokens_per_tile=per_tile, row_tiles=row_tiles,
                                 n_splits=n_splits, keys_per_split=per_split, part_o=part_o, part_ml=part_ml,
                                 tile_waves=tile_waves, max_context_dev=longest_dev if n_splits > 1 else None)
    return out


def _workspaces(device: torch.device, units: int, rows: int, head_dim: int) -> tuple[torch.Tensor, torch.Tensor]:
    return (torch.empty(units * rows * head_dim, dtype=torch.float32, device=device),
            torch.empty(units * rows * 2, dtype=torch.float32, device=device))


register_part("mixer", "attention", Attention)
