"""The compiler's assembly of the kernels that use the matrix cores keeps a matrix product and the first use of its
result far enough apart along every path (tests/mfma_hazards.py says why that needs a test)."""

from __future__ import annotations

import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

import pytest

import mfma_hazards

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))

WAIT_STATES = 8  # what the compiler keeps between a 16 x 16 x 32 product and a read of its sums where it counts


def test_the_checker_sees_a_short_cut():
    """Pinned on a listing made by hand: straight code with enough instructions passes; a branch around them is found."""
    straight = ["v_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]", "s_nop 7", "v_accvgpr_read_b32 v8, a0", "s_endpgm"]
    assert mfma_hazards.short_paths(straight, WAIT_STATES) == []
    short_cut = ["v_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]", "s_cbranch_vccnz .L1",
                 "v_mfma_f32_16x16x32_bf16 a[4:7], v[0:3], v[4:7], a[4:7]", "s_nop 7", ".L1:", "s_nop 0",
                 "v_accvgpr_read_b32 v8, a0", "s_endpgm"]
    found = mfma_hazards.short_paths(short_cut, WAIT_STATES)
    assert [(distance, use) for distance, _, use in found] == [(2, "v_accvgpr_read_b32 v8, a0")]
    # a product that accumulates into the same registers may follow at once
    chain = ["v_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]", "v_mfma_f32_16x16x32_bf16 a[0:3], v[8:11], v[4:7], a[0:3]",
             "s_nop 7", "v_accvgpr_read_b32 v8, a0", "s_endpgm"]
    assert mfma_hazards.short_paths(chain, WAIT_STATES) == []
    assert mfma_hazards.registers("v[2:4], a7, s[0:1]") == {("v", 2), ("v", 3), ("v", 4), ("a", 7)}


def test_no_kernel_reads_a_product_before_it_has_finished(tmp_path):
    from cie_amd.kernels import library

    hipcc = library._hipcc()
    if hipcc is None:
        pytest.skip("no hipcc here")
    sources = [path for path in library.sources() if "__builtin_amdgcn_mfma" in path.read_text()]
    assert sources, "the kernels that use the matrix cores"

    def listing(path: Path) -> tuple[Path, str]:
        out = tmp_path / (path.stem + ".s")
        done = subprocess.run([hipcc, *library.HIPCC_FLAGS, "-I", str(library.CSRC), "-S", "--cuda-device-only",
                               "-o", str(out), str(path)], capture_output=True, text=True)
        assert done.returncode == 0, done.stderr[-2000:]
        return path, out.read_text()

    with ThreadPoolExecutor(max_workers=4) as pool:
        listings = list(pool.map(listing, sources))
    kernels = 0
    for path, assembly in listings:
        for name, body in mfma_hazards.kernels_of(assembly):
            if not any(line.startswith("v_mfma") for line in body):
                continue
            kernels += 1
            found = mfma_hazards.short_paths(body, WAIT_STATES)
            assert not found, (f"{path.name}: {name}: {len(found)} uses of a product's result within {WAIT_STATES} wait states; "
                               f"the nearest after {min(found)[0]}: {min(found)[1]} -> {min(found)[2]}")
    assert kernels > 100  # (every instantiation of the attention and product kernels)
