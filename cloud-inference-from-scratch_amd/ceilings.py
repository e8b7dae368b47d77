"""What this GPU reaches on the two resources the roofline figures divide by:
memory bandwidth (a device copy, a streaming read through the library's
matrix-vector product and through this package's few-row product) and bf16 matrix
throughput (a large square product through the library, untuned and tuned).
``cie ceilings`` prints one JSON record.  The published peaks of the MI355X
(8 TB/s, 2.5 PFLOP/s dense bf16) are what ``bench.py`` divides by; these are what
a kernel can actually be compared with on the box at hand.
"""

from __future__ import annotations

import json
import time
from typing import Any, Callable


def _time(run: Callable[[], Any], repeats: int) -> float:
    import torch

    run()
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(repeats):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - start) / repeats


def measure(device: str = "cuda:0") -> dict[str, Any]:
    import torch

    from .kernels import ops

    record: dict[str, Any] = {"device": torch.cuda.get_device_name(device)}
    # -- memory: a 1 GiB copy (reads and writes), and reads of a 1 GiB bf16 matrix by a matrix-vector product
    source = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    target = torch.empty_like(source)
    seconds = _time(lambda: target.copy_(source), 20)
    record["copy_1GiB_GBps"] = round(2 * source.numel() / seconds / 1e9, 1)
    del source, target
    rows, cols = 1 << 18, 2048
    matrix = torch.randn((rows, cols), device=device, dtype=torch.bfloat16)
    vector = torch.randn((cols,), device=device, dtype=torch.bfloat16)
    seconds = _time(lambda: torch.mv(matrix, vector), 20)
    record["read_1GiB_library_mv_GBps"] = round(matrix.numel() * 2 / seconds / 1e9, 1)
    one_row = vector.view(1, cols).contiguous()
    seconds = _time(lambda: ops.gemm_fused(matrix, ops.EPI_BF16, one_row), 20)
    record["read_1GiB_few_row_product_GBps"] = round(matrix.numel() * 2 / seconds / 1e9, 1)
    small = matrix[: 11008]  # 45 MB: one down projection of the 3B shape
    seconds = _time(lambda: ops.gemm_fused(small, ops.EPI_BF16, one_row), 50)
    record["read_45MB_few_row_product_GBps"] = round(small.numel() * 2 / seconds / 1e9, 1)
    del matrix
    # -- matrix cores: 8192^3 in bf16
    n = 8192
    a = torch.randn((n, n), device=device, dtype=torch.bfloat16)
    b = torch.randn((n, n), device=device, dtype=torch.bfloat16)
    flops = 2.0 * n * n * n
    seconds = _time(lambda: torch.nn.functional.linear(a, b), 10)
    record["bf16_8192_cubed_library_TFLOPs"] = round(flops / seconds / 1e12, 1)
    seconds = _time(lambda: ops.gemm_library(a, b), 10)  # a shape that times the library's candidates first
    record["bf16_8192_cubed_library_tuned_TFLOPs"] = round(flops / seconds / 1e12, 1)
    return record


def main(argv: list[str] | None = None) -> int:
    print(json.dumps(measure()))
    return 0
