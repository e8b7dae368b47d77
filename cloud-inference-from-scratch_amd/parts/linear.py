"""``x @ W^T + b`` for a Linear's weight ``[out, in]``, and its fused forms.

float32: the hand-written true-float32 kernel, always.  bfloat16 with up to
``FUSED_ROWS`` rows (decode steps, the output head), and up to 64 or 128 rows where
it is the faster one (a small weight, a long K): the hand-written
matrix-core kernels that stream the weight once and take over their neighbours'
work: a SiLU-gate behind (``epilogue="silu"``), the add into the float32
residual stream (``into=residual``), or float32 results for the logits.  They
come in two forms: waves that share K and own all rows (few rows; the q/k/v,
o_proj and head products), and waves that own columns and share the rows through
LDS (the SiLU-gate product up to 64 rows and every product whose K is cut).
bfloat16 with more rows: the vendor library's product (hipBLASLt through a
thin cached interface of this package), as the reference leaves its products to
a library (src/cloud_engine/model.py:89-137), with the small kernels around it.
"""

from __future__ import annotations

import weakref
from dataclasses import dataclass
from typing import Any, Optional, Union

import torch

from ..kernels import ops

# Rows up to which the hand-written fused bf16 kernel replaces the library product.  Measured on
# MI355X (3B shapes): up to 16 rows it beats the library by 1.5-2x; with 17 to 64 rows it wins where K
# is long and is cut into parts (the down product: 17-20 us against the library's 27-32 us); its gate/up
# product loses from 32 rows on (34 us against 26 + 5 us at 64 rows: every workgroup re-reads the rows of A).
FUSED_ROWS = 16
# ... and up to 128 rows (the down product alone, weight from memory, own kernel against the library, us: 3B shape at
# 72 / 96 / 128 rows 18.3 / 19.9 / 24.2 against 27.7 / 28.4 / 28.4; 7B 41.6 / 45.8 / 54.4 against 96 / 95 / 84; 14B
# 36.3 / 39.8 / 48.2 against 50.0 / 61.6 / 60.9: the library has no good algorithm for a long K and few rows, and at
# row counts that do not recur it takes its heuristic's first choice)
FUSED_PARTS_ROWS = 128
# With 17 to 128 rows it also wins where the weight is small (q/k/v and o_proj of the 3B shape: 7-9 us against
# the library's 12-18 us inside a step at up to 64 rows, 9.3 and 8.2 us against 9.5-12.4 and 9.1 us at 72 and 128
# rows, where the weight is streamed twice; and the rotation, the cache write, the residual add and the next
# norm ride along); from about 6M weight values on the library is faster (7B o_proj at 64 rows: 12.6 us against
# 11.1 us).
FUSED_SMALL_ROWS = 128
FUSED_SMALL_WEIGHT = 6 << 20
# float32 logits of more rows than this go to the library (the hand-written kernel streams the weight once per
# 64 rows; up to 64 rows it is one pass either way)
FUSED_LOGIT_ROWS = 64
# An ``into=`` product with fewer than this many 16-column tiles and a K of at least ``PART_MIN_K`` cuts K
# into parts for more workgroups (each part adds its products into the stream with atomic adds; ``plan_shared_parts``).
PART_BELOW_TILES = 512
PART_MIN_K = 4096
PART_K = 1024           # the shortest stretch of K a part takes


# SiLU-gate products of up to this many rows take the form whose waves own columns and share the rows of A
# through LDS (gate/up of the 3B shape at 32 / 64 rows: 21 / 24 us against the library's 26 / 27 us and 5 us
# for the SiLU kernel behind it; 14B: 50 / 56 against 55 / 62 + 6; 7B: level); from 65 to 96 rows, on six row tiles
# (3B / 7B / 14B at 72 rows: 28.3 / 67.7 / 63.7 us against 31.4 / 75.2 / 70.4 for the library and its SiLU kernel,
# at 96 rows 29.6 / 69.6 / 65.0 against 32.2 / 71.1 / 64.6); beyond that the library is level or ahead (3B at 128
# rows: 35 against 30 + 5 us; 7B: 111 against 66).
SHARED_SILU_ROWS = 96
# float32 logits take that form up to this many rows (the head of the 3B / 7B / 14B shape, us: 64 rows 156 against
# 173 in the form whose waves share K; 72 rows 165 / 239 / 333 against the library's 174 / 249 / 349; 96 rows
# 172 / 255 / 346 against 174 / 238 / 338)
SHARED_LOGIT_ROWS = 80


def plan_shared_silu(pairs: int) -> tuple[int, bool]:
    """Waves per workgroup (each wave takes one gate tile and its up tile) for the shared-rows SiLU product,
    and whether every workgroup then has a compute unit of its own.  A compute unit streams at most some
    30 GB/s however many loads it has under way, so what counts is the most pairs that meet on one unit:
    workgroups of four waves, or of three where that needs fewer turns (688 pairs of the 3B shape: 172
    workgroups of four or 230 of three, one turn each; 1,184 of the 7B shape: two turns of four waves or
    two of three, 70 against 61 us at 64 rows; 864 of the 14B shape: one turn of four, 56 against 81 us)."""
    best = None
    units = ops.compute_units()
    for waves in (4, 3, 2):
        turns = -(-(-(-pairs // waves)) // units)
        if best is None or turns * waves < best[0]:
            best = (turns * waves, waves, turns == 1)
    return best[1], best[2]


def plan_shared_parts(tiles: int, k: int) -> tuple[int, int, int]:
    """(column tiles per wave, waves, parts of K) of a cut product in the shared-rows form: workgroups of four
    waves, one tile of 16 columns per wave (two for a wide result), and as many parts as give about one
    workgroup per compute unit.  Measured at 8 / 64 rows (us; the form of waves that share K, at its best
    cut, beside it): 128 tiles, K 11,008: 8 parts 11.0 / 14.8 (13.2 / 17.7); 224 tiles, K 18,944: 4 parts
    26.1 / 35.3 (29.7 / 43.8); 320 tiles, K 13,824, two tiles per wave: 4 parts 28.6 / 38.7 (30.0 / 44.0)."""
    units = ops.compute_units()
    column_tiles = 1 if tiles <= units else 2
    waves = 4
    blocks = -(-tiles // (column_tiles * waves))
    parts = max(1, min(units // blocks, 16, k // PART_K))
    return column_tiles, waves, parts


@dataclass
class RowSumsq:
    """Stands where a branch output would: the branch was already added into the
    residual stream, and ``sumsq`` [rows, parts] holds partial sums of squares of
    the residual's rows (what an RMSNorm needs of them).  ``scaled``, if given, is
    the new residual times the weight of ``norm`` in bf16: that norm's output
    short of each row's 1/rms."""

    sumsq: torch.Tensor
    scaled: Optional[torch.Tensor] = None
    norm: Any = None


@dataclass
class ScaledRows:
    """Stands where an RMSNorm's output would: ``rows`` [M, hidden] bf16 lack the
    factor ``rsqrt(sum(sumsq[m]) / hidden + eps)`` of their row, which a product
    that reads them applies to its sums (a product is linear in its rows)."""

    rows: torch.Tensor
    sumsq: torch.Tensor
    eps: float
    residual: torch.Tensor
    norm: Any

    @property
    def shape(self):
        return self.rows.shape

    def complete(self) -> torch.Tensor:
        """The norm's output after all (for a reader that cannot apply the factor)."""
        return ops.rmsnorm_from_sumsq(self.residual, self.sumsq, self.norm.weight, self.eps)


@dataclass
class Added:
    """Stands where a branch output would: the branch was already added into the residual stream, and
    nothing else is known of the stream's rows (a product whose K was cut into parts, each of which added
    its share with atomic adds)."""


@dataclass
class RawRows:
    """Stands where an RMSNorm's output would, before anything was computed: the rows are the norm ``norm``
    of the float32 stream ``residual``.  Only a mixer that says ``takes_raw_rows`` is shown it (the attention
    part's q/k/v product then makes its rows itself, with up to ``ops.FOLDED_NORM_ROWS`` rows: every workgroup
    reads the few rows once, where a kernel of its own for the norm costs a decode layer 4.6 us)."""

    residual: torch.Tensor
    norm: Any
    dtype: torch.dtype = torch.bfloat16

    @staticmethod
    def fits(residual: torch.Tensor, dtype: torch.dtype) -> bool:
        rows, width = residual.shape
        return dtype == torch.bfloat16 and residual.is_cuda and ops.folds_norm(rows, width)

    @property
    def shape(self):
        return self.residual.shape

    def complete(self) -> torch.Tensor:
        """The norm's output after all."""
        return ops.add_rmsnorm(self.residual, None, self.norm.weight, self.norm.eps, self.dtype)


_WIDENED: dict[int, tuple["weakref.ref", torch.Tensor]] = {}


def _widened(weight: torch.Tensor) -> torch.Tensor:
    """``weight`` in float32, made at its first use (an output head of 150,000 rows is not copied every step)."""
    key = id(weight)
    kept = _WIDENED.get(key)
    if kept is not None and kept[0]() is weight:
        return kept[1]
    wide = weight.float()
    _WIDENED[key] = (weakref.ref(weight, lambda _gone, key=key: _WIDENED.pop(key, None)), wide)
    return wide


def _fusable(rows: int, k: int, row_stride: int, weight: torch.Tensor) -> bool:
    return weight.dtype == torch.bfloat16 and rows >= 1 and k % 8 == 0 and row_stride % 8 == 0


def linear(x: Union[torch.Tensor, ScaledRows], weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, epilogue: Optional[str] = None,
           into: Optional[torch.Tensor] = None, then_norm: Any = None) -> Union[torch.Tensor, RowSumsq, Added]:
    """``x @ weight.T + bias``.

    ``epilogue="silu"``: weight stacks gate rows over up rows; returns
    ``silu(gate) * up``.  ``into=residual``: the caller wants the result added to
    the float32 residual stream; if a fused kernel runs it adds it in place, and a
    :class:`RowSumsq` comes back, or (a product whose K was cut into parts that
    each add their share) an :class:`Added`; otherwise the plain
    result comes back and the caller adds it (the next norm kernel does).
    ``then_norm`` (with ``into``): the norm that follows, if it can be folded into
    this product and the next (``RMSNorm.folds_into_products``): the residual
    epilogue then also leaves that norm's output short of the rows' scale.
    ``x`` may be such rows (:class:`ScaledRows`): the SiLU product of few rows
    applies the scale itself, any other reader gets the completed rows."""
    if isinstance(x, ScaledRows):
        rows, k = x.rows.shape
        if epilogue == "silu" and weight.shape[0] % 2 == 0 and bias is None and weight.dtype == torch.bfloat16:
            if _fusable(rows, k, x.rows.stride(0) if rows > 1 else k, weight):
                waves, own_unit = plan_shared_silu(-(-weight.shape[0] // 32))
                if FUSED_ROWS < rows <= SHARED_SILU_ROWS or (rows <= FUSED_ROWS and own_unit):
                    return ops.gemm_shared_rows(weight, ops.EPI_SILU, x.rows, waves=waves, row_sumsq=x.sumsq, eps=x.eps)
                if rows <= FUSED_ROWS:
                    return ops.gemm_fused(weight, ops.EPI_SILU, x.rows, row_sumsq=x.sumsq, eps=x.eps)
            # more rows: the library's product of the rows as they are, the scale in the SiLU kernel behind it
            out = ops.gemm_library(x.rows, weight) if x.rows.stride(1) == 1 else None
            if out is not None:
                return ops.silu_mul(out, row_sumsq=x.sumsq, hidden=k, eps=x.eps)
        x = x.complete()
    rows, k = x.shape
    n = weight.shape[0]
    silu = epilogue == "silu"
    wants_f32 = out_dtype == torch.float32
    if rows == 0 and into is None:  # nothing to multiply: no kernel, and no widened copy of the weight
        return torch.empty((0, n // 2 if silu else n), dtype=torch.float32 if wants_f32 else x.dtype, device=x.device)
    fusable = _fusable(rows, k, x.stride(0) if rows > 1 else k, weight)
    cut_k = (into is not None and -(-n // 16) < PART_BELOW_TILES and k >= PART_MIN_K and into.is_contiguous()
             and tuple(into.shape) == (rows, n))
    if fusable and cut_k and rows <= FUSED_PARTS_ROWS:
        # (atomic adds cost the product nothing, measured against partial products written for the next norm
        # kernel to sum: 10.3 us either way for the 3B shape's down product at 8 rows; and the kernel that summed
        # them falls away)
        column_tiles, waves, parts = plan_shared_parts(-(-n // 16), k)
        ops.gemm_shared_rows(weight, ops.EPI_ATOMIC, x, bias=bias, column_tiles=column_tiles, waves=waves,
                             k_parts=parts, add_into=into)
        return Added()
    if fusable and silu and n % 2 == 0 and bias is None and into is None and not wants_f32 and rows <= SHARED_SILU_ROWS:
        waves, own_unit = plan_shared_silu(-(-n // 32))
        if rows > FUSED_ROWS or own_unit:
            return ops.gemm_shared_rows(weight, ops.EPI_SILU, x, waves=waves)
    if fusable and wants_f32 and FUSED_ROWS < rows <= SHARED_LOGIT_ROWS and into is None and not silu:
        # logits of 17 to 80 rows: the shared-rows form
        return ops.gemm_shared_rows(weight, ops.EPI_F32, x, bias=bias, waves=4)
    if fusable and wants_f32 and rows > FUSED_LOGIT_ROWS and into is None and not silu and bias is None:
        out = ops.gemm_library(x, weight, out_dtype=torch.float32)  # logits of many rows: one pass over the weight
        if out is not None:
            return out
    small = rows <= FUSED_SMALL_ROWS and n * k <= FUSED_SMALL_WEIGHT and not silu
    if fusable and (rows <= FUSED_ROWS or wants_f32 or small):
        if into is not None:
            if then_norm is not None:
                scaled = torch.empty((rows, n), dtype=torch.bfloat16, device=x.device)
                sumsq = ops.gemm_fused(weight, ops.EPI_RESID, x, bias=bias, residual_out=into,
                                       norm_weight=then_norm.weight_f32, scaled_out=scaled)
                return RowSumsq(sumsq, scaled, then_norm)
            return RowSumsq(ops.gemm_fused(weight, ops.EPI_RESID, x, bias=bias, residual_out=into))
        elif silu and n % 2 == 0:
            return ops.gemm_fused(weight, ops.EPI_SILU, x)
        elif not silu:
            return ops.gemm_fused(weight, ops.EPI_F32 if wants_f32 else ops.EPI_BF16, x, bias=bias)
    if weight.dtype == torch.float32:
        out = ops.gemm_f32(x, weight, bias)
    elif wants_f32:
        # a shape the kernel refuses (a width that is no multiple of 8): widened operands, exact products,
        # float32 sums; the widened weight is made once and kept for as long as the weight lives
        out = x.float() @ _widened(weight).t()
        out = out if bias is None else out + bias.float()
    else:
        out = ops.gemm_library(x, weight, bias) if x.is_cuda and x.stride(1) == 1 else None
        if out is None:  # a shape the library's own interface has no algorithm for
            out = torch.nn.functional.linear(x, weight, bias)
    return ops.silu_mul(out) if silu else out
