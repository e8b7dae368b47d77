"""The kernel library's host side without a GPU: the entry points' argument types are read from the sources."""

from __future__ import annotations

import ctypes

import pytest

from cie_amd.kernels import library


def test_signatures_of_all_entry_points_are_read_from_the_sources():
    found = library.entry_point_signatures()
    text = "".join(path.read_text() for path in library.sources())
    assert len(found) == text.count("CIE_API int ") >= 14
    # (stream, dtype, gate_up, out, tokens, intermediate, row_sumsq, parts, hidden, eps)
    p, i, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    assert found["cie_silu_mul"] == [p, i, p, p, i, i, p, i, i, f]
    assert found["cie_gemm_library"][-2:] == [ctypes.c_size_t, i]
    assert all(types[0] is p for types in found.values())  # every entry point takes the stream first


@pytest.mark.parametrize("params", ["void* stream, double x", "void* stream, unsigned int n", "void* stream, int"])
def test_a_parameter_that_is_not_understood_is_an_error(tmp_path, monkeypatch, params):
    source = tmp_path / "odd.hip"
    source.write_text(f"CIE_API int cie_odd({params}) {{ return 0; }}\n")
    monkeypatch.setattr(library, "sources", lambda: [source])
    with pytest.raises(library.KernelLibraryError, match="cie_odd"):
        library.entry_point_signatures()


def test_a_product_of_no_rows_launches_nothing_and_widens_nothing():
    """Steps of prompt portions that end before their prompts want no logits: the output head is given no
    rows.  No kernel runs (none could, here without a GPU) and the weight is not touched."""
    import torch

    from cie_amd.parts.linear import linear

    weight = torch.zeros((32, 16), dtype=torch.bfloat16)
    rows = torch.empty((0, 16), dtype=torch.bfloat16)
    logits = linear(rows, weight, None, out_dtype=torch.float32)
    assert logits.shape == (0, 32) and logits.dtype == torch.float32
    gated = linear(rows, weight, None, epilogue="silu")
    assert gated.shape == (0, 16) and gated.dtype == torch.bfloat16


def test_the_fallback_build_folder_must_be_this_users_own(tmp_path, monkeypatch):
    """The folder under the temporary directory has a name anyone can guess: one that others can write
    into (or that is no folder of this user's) is neither built into nor loaded from."""
    import os

    folder = tmp_path / "cie_amd_build_me"
    monkeypatch.setattr(library, "_fallback_dir", lambda: folder)
    assert library._build_dirs()[-1] == folder and folder.stat().st_mode & 0o777 == 0o700
    os.chmod(folder, 0o777)  # as if someone else had made it before us
    assert folder not in library._build_dirs()
    os.chmod(folder, 0o755)
    assert folder in library._build_dirs()
    folder.rmdir()
    folder.symlink_to(tmp_path)  # a link is no folder of ours, wherever it points
    assert folder not in library._build_dirs()


def test_cut_products_and_silu_products_plan_by_compute_units():
    """The cut of a long K: workgroups of four waves, about one for each compute unit, no part shorter than
    ``PART_K``; the SiLU product: the fewest pairs of tiles that meet on one compute unit.  The shapes that were
    measured keep their measured choice."""
    from cie_amd.parts.linear import plan_shared_parts, plan_shared_silu

    assert plan_shared_parts(128, 11008) == (1, 4, 8)     # the 3B down product
    assert plan_shared_parts(224, 18944) == (1, 4, 4)     # 7B
    assert plan_shared_parts(320, 13824) == (2, 4, 6)     # 14B
    assert plan_shared_parts(6, 328) == (1, 4, 1) and plan_shared_parts(3, 4096) == (1, 4, 4)
    assert plan_shared_parts(500, 1 << 20) == (2, 4, 4) and plan_shared_parts(1, 1 << 20) == (1, 4, 16)
    assert plan_shared_silu(688) == (3, True)      # 3B: 230 workgroups of three waves
    assert plan_shared_silu(1184) == (3, False)    # 7B: two turns either way, three waves are less per turn
    assert plan_shared_silu(864) == (4, True)      # 14B: 216 workgroups of four
    assert plan_shared_silu(1) == (2, True)        # a narrow one: no idle waves


def test_a_widened_head_is_made_once_and_let_go_with_its_weight():
    import gc

    import torch

    from cie_amd.parts import linear

    weight = torch.ones((5, 3), dtype=torch.bfloat16)
    first = linear._widened(weight)
    assert first.dtype == torch.float32 and linear._widened(weight) is first
    key = id(weight)
    del weight
    gc.collect()
    assert key not in linear._WIDENED
