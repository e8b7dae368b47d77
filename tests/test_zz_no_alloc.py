"""GPU: the entry point that allocates nothing, called through ctypes as a caller that cannot allocate
would call it, against the entry point with a workspace that it is a variant of."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

CHUNK = 2048
MAX_ENTRIES = 16384  # CIE_ARGMAX_STATIC_MAX_ENTRIES of csrc/cie_no_alloc.h
TOO_LARGE = 3


def both(library, logits: torch.Tensor, vocab: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(tokens by cie_argmax with a workspace, tokens by cie_argmax_static) for the first ``vocab`` columns."""
    rows, ld = logits.shape
    chunks = -(-vocab // CHUNK)
    stream = torch.cuda.current_stream().cuda_stream
    chunk_val = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
    chunk_idx = torch.empty(rows * chunks, dtype=torch.int32, device=logits.device)
    with_workspace = torch.full((rows,), -1, dtype=torch.int32, device=logits.device)
    without = torch.full((rows,), -2, dtype=torch.int32, device=logits.device)
    code = library.cie_argmax(stream, logits.data_ptr(), chunk_val.data_ptr(), chunk_idx.data_ptr(),
                              with_workspace.data_ptr(), rows, vocab, ld, CHUNK)
    assert code == 0
    code = library.cie_argmax_static(stream, logits.data_ptr(), without.data_ptr(), rows, vocab, ld, CHUNK)
    assert code == 0
    torch.cuda.synchronize()
    return with_workspace.cpu(), without.cpu()


def test_argmax_without_allocation_equals_argmax_with_a_workspace():
    from cie_amd.kernels import load_library

    library = load_library()
    assert isinstance(library, ctypes.CDLL)
    g = torch.Generator().manual_seed(5)
    # the first call: 40 rows of a vocabulary that is no multiple of the chunk (the last chunk is short)
    large = torch.randn((40, 151936), generator=g).cuda()
    large[3, 70000] = large[3, 9] = 50.0        # a tie: the lower index wins
    large[7, 151935] = 60.0                     # the maximum in the last, short chunk
    expected, got = both(library, large, 151936)
    assert torch.equal(got, expected) and torch.equal(got.long(), large.argmax(-1).cpu())
    assert int(got[3]) == 9 and int(got[7]) == 151935
    # the second call, right behind it, with fewer rows and a shorter vocabulary: the array still holds the
    # first call's partial results beyond what this call writes, and none of them may be read
    small = torch.randn((5, 9000), generator=g).cuda()
    small[:, 4097] -= 100.0
    expected, got = both(library, small, 9000)
    assert torch.equal(got, expected) and torch.equal(got.long(), small.argmax(-1).cpu())
    # columns beyond `vocab` of a wider row are not looked at
    padded = torch.randn((6, 5000), generator=g).cuda()
    padded[:, 4500:] = 99.0
    expected, got = both(library, padded, 4500)
    assert torch.equal(got, expected) and int(got.max()) < 4500


def test_sizes_beyond_the_fixed_scratch_are_refused_and_nothing_runs():
    from cie_amd.kernels import load_library

    library = load_library()
    stream = torch.cuda.current_stream().cuda_stream
    rows = 300
    vocab = 151936  # 75 chunks a row: 22,500 partial results, more than the array's 16,384
    assert rows * -(-vocab // CHUNK) > MAX_ENTRIES
    logits = torch.zeros((rows, vocab), dtype=torch.float32, device="cuda")
    out = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    assert library.cie_argmax_static(stream, logits.data_ptr(), out.data_ptr(), rows, vocab, vocab, CHUNK) == TOO_LARGE
    torch.cuda.synchronize()
    assert int(out.min()) == int(out.max()) == -7
    # at the limit it runs: 218 rows x 75 chunks = 16,350
    assert library.cie_argmax_static(stream, logits.data_ptr(), out.data_ptr(), 218, vocab, vocab, CHUNK) == 0
    torch.cuda.synchronize()
    assert int(out[:218].max()) == 0 and int(out[218:].min()) == -7
    assert library.cie_argmax_static(stream, logits.data_ptr(), out.data_ptr(), 4, vocab, vocab - 1, CHUNK) == 1
