"""GPU: each HIP kernel alone against a plain float32 torch reference of the same
operation, at sizes other than the tiny models' (odd widths, many heads and
groups, head sizes in steps of 16)."""

from __future__ import annotations

import math
import random

import pytest
import torch

import plain_qwen2

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.fixture(scope="module")
def ops():
    from cie_amd.kernels import ops as module

    return module


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops, dtype):
    table = rand((1000, 72), dtype, 1)
    ids = torch.tensor([0, 999, 5, 5, 321], dtype=torch.int32).cuda()
    out = ops.embed(table, ids)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, table.float()[ids.long()], rtol=0, atol=0)
    # rows 1 and 3 take their tokens from a pool on the device instead
    feed = torch.tensor([-1, 2, -1, 0, -1], dtype=torch.int32).cuda()
    pool = torch.tensor([77, 500, 901], dtype=torch.int32).cuda()
    fed = ops.embed(table, ids, feed=feed, pool=pool)
    expect = torch.tensor([0, 901, 5, 77, 321]).cuda()
    torch.testing.assert_close(fed, table.float()[expect], rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [72, 1000, 4104])
def test_add_rmsnorm(ops, dtype, hidden):
    residual = rand((7, hidden), torch.float32, 2, 3.0)
    branch = rand((7, hidden), dtype, 3)
    weight = rand((hidden,), dtype, 4) + 1
    eps = 1e-5
    expect_res = residual + branch.float()
    expect = plain_qwen2.rms_norm(expect_res, weight.float(), eps)
    out = ops.add_rmsnorm(residual, branch, weight, eps, dtype)
    torch.testing.assert_close(residual, expect_res, rtol=0, atol=0)  # the float32 sum is written back
    torch.testing.assert_close(out.float(), expect, **tol(dtype))
    # no branch, selected rows only, float32 weight beside bf16 activations
    rows = torch.tensor([6, 0, 3], dtype=torch.int32).cuda()
    before = residual.clone()
    out = ops.add_rmsnorm(residual, None, weight.float(), eps, dtype, rows=rows)
    torch.testing.assert_close(residual, before, rtol=0, atol=0)
    torch.testing.assert_close(out.float(), expect[rows.long()], **tol(dtype))


def test_rmsnorm_invariants(ops):
    """weight 1, tiny eps: every output row has RMS 1; scaling the input changes nothing."""
    x = rand((4, 200), torch.float32, 5, 2.0)
    ones = torch.ones(200, device="cuda")
    out = ops.add_rmsnorm(x.clone(), None, ones, 1e-12, torch.float32)
    torch.testing.assert_close(out.pow(2).mean(-1), torch.ones(4, device="cuda"), rtol=1e-5, atol=1e-5)
    out2 = ops.add_rmsnorm(x * 7.5, None, ones, 1e-12, torch.float32)
    torch.testing.assert_close(out, out2, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(ops, dtype):
    gate_up = rand((5, 2 * 333), dtype, 6, 2.0)
    g, u = gate_up.float()[:, :333], gate_up.float()[:, 333:]
    out = ops.silu_mul(gate_up)
    torch.testing.assert_close(out.float(), torch.nn.functional.silu(g) * u, **tol(dtype))
    zero_gate = torch.cat([torch.zeros(5, 333), torch.randn(5, 333)], dim=1).to(dtype).cuda()
    assert ops.silu_mul(zero_gate).abs().max().item() == 0.0


@pytest.mark.parametrize("shape", [(1, 40, 24), (5, 515, 96), (70, 130, 200), (130, 64, 17)])
def test_gemm_f32(ops, shape):
    m, n, k = shape
    a, w, b = rand((m, k), torch.float32, 7), rand((n, k), torch.float32, 8), rand((n,), torch.float32, 9)
    expect = (a.double() @ w.double().t() + b.double()).float()
    torch.testing.assert_close(ops.gemm_f32(a, w, b), expect, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ops.gemm_f32(a, w), (a.double() @ w.double().t()).float(), rtol=1e-5, atol=1e-5)
    # a row's result does not depend on the other rows of the batch (bitwise)
    assert torch.equal(ops.gemm_f32(a[:1].contiguous(), w, b), ops.gemm_f32(a, w, b)[:1])


@pytest.mark.parametrize("shape", [(1, 40, 24), (5, 515, 96), (16, 64, 128), (17, 130, 200), (33, 70, 1032),
                                   (64, 256, 264), (150, 99, 72)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gemm_fused_plain_any_size(ops, shape, out_dtype):
    """Plain product with bias: rows from 1 to more than a workgroup takes, column counts
    that are no multiple of 16, inner sizes that are no multiple of 128."""
    m, n, k = shape
    a, w, b = rand((m, k), torch.bfloat16, 10), rand((n, k), torch.bfloat16, 11), rand((n,), torch.bfloat16, 12)
    expect = a.double() @ w.double().t()
    epilogue = ops.EPI_F32 if out_dtype == torch.float32 else ops.EPI_BF16
    out = ops.gemm_fused(w, epilogue, a)
    assert out.dtype == out_dtype and out.shape == (m, n)
    if out_dtype == torch.float32:
        torch.testing.assert_close(out.double(), expect, rtol=1e-4, atol=1e-4 * math.sqrt(k))
    else:
        torch.testing.assert_close(out.double(), expect, rtol=1e-2, atol=1e-2 * math.sqrt(k))
    out = ops.gemm_fused(w, ops.EPI_F32, a, bias=b)
    torch.testing.assert_close(out.double(), expect + b.double(), rtol=1e-4, atol=1e-4 * math.sqrt(k))
    # rows given as a strided view (a slice of a wider buffer)
    wide = torch.zeros((m, k + 64), dtype=torch.bfloat16).cuda()
    wide[:, :k] = a
    torch.testing.assert_close(ops.gemm_fused(w, ops.EPI_F32, wide[:, :k]), ops.gemm_fused(w, ops.EPI_F32, a), rtol=0, atol=0)


def build_cache(dtype, lengths, kv_heads, head_dim, page_size, seed, shuffle=True):
    """Random keys/values for sequences of the given lengths, scattered over the
    pages of a pool in a shuffled order.  Returns pools, block table and the
    dense per-sequence tensors."""
    g = torch.Generator().manual_seed(seed)
    pages_per = [-(-n // page_size) for n in lengths]
    total = sum(pages_per) + 3
    order = torch.randperm(total, generator=g).tolist() if shuffle else list(range(total))
    width = max(pages_per) + 2
    table = torch.zeros((len(lengths) + 2, width), dtype=torch.int32)
    slots = list(range(len(lengths), 0, -1))  # slot != sequence index, on purpose
    k_pool = torch.zeros((total, kv_heads, page_size, head_dim))
    v_pool = torch.zeros_like(k_pool)
    dense = []
    cursor = 0
    for s, n in enumerate(lengths):
        k = torch.randn((n, kv_heads, head_dim), generator=g)
        v = torch.randn((n, kv_heads, head_dim), generator=g)
        k, v = k.to(dtype).float(), v.to(dtype).float()
        dense.append((k, v))
        for p in range(pages_per[s]):
            page = order[cursor]
            cursor += 1
            table[slots[s], p] = page
            rows = slice(p * page_size, min((p + 1) * page_size, n))
            count = rows.stop - rows.start
            k_pool[page, :, :count] = k[rows].transpose(0, 1)
            v_pool[page, :, :count] = v[rows].transpose(0, 1)
    # values are cached transposed: [page, head, head_dim, page_size]
    v_pool = v_pool.transpose(2, 3).contiguous()
    return k_pool.to(dtype).cuda(), v_pool.to(dtype).cuda(), table.cuda(), slots, dense


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geometry", [(4, 2, 16, 16), (16, 2, 128, 16), (6, 6, 48, 8), (8, 1, 64, 32), (5, 5, 80, 4)])
def test_paged_attention_generic(ops, dtype, geometry):
    """Ragged batch: a long prompt portion with context, a fresh prompt, single
    decode tokens at page edges.  Context/query sizes follow the reference's
    matrix (tests/remote_ragged_gpu_tests.py:118-121) scaled down."""
    q_heads, kv_heads, head_dim, page_size = geometry
    contexts = [0, 15, 16, 17, 127, 300, 1]
    q_lens = [7, 1, 1, 2, 16, 1, 33]
    lengths = [c + q for c, q in zip(contexts, q_lens)]
    k_pool, v_pool, table, slots, dense = build_cache(dtype, lengths, kv_heads, head_dim, page_size, seed=20)
    scale = 1.0 / math.sqrt(head_dim)
    g = torch.Generator().manual_seed(21)
    positions, seq_of_token, expected, qs = [], [], [], []
    for s, (c, n) in enumerate(zip(contexts, q_lens)):
        q = (torch.randn((n, q_heads, head_dim), generator=g) * 2).to(dtype).float()
        qs.append(q)
        positions += list(range(c, c + n))
        seq_of_token += [s] * n
        k, v = dense[s]
        expected.append(plain_qwen2.causal_attention(q, k, v, scale, past_len=c))
    q_all = torch.cat(qs).reshape(len(positions), q_heads * head_dim)
    stride = (q_heads + 2 * kv_heads) * head_dim  # as if q sat inside a fused qkv buffer
    buffer = torch.zeros((len(positions), stride))
    buffer[:, : q_heads * head_dim] = q_all
    buffer = buffer.to(dtype).cuda()
    out = ops.paged_attention_generic(
        buffer, stride, k_pool, v_pool, table, torch.tensor(positions, dtype=torch.int32).cuda(),
        torch.tensor(seq_of_token, dtype=torch.int32).cuda(), torch.tensor(slots, dtype=torch.int32).cuda(),
        len(positions), q_heads, kv_heads, head_dim, None, scale)
    torch.testing.assert_close(out.float().cpu(), torch.cat(expected), **tol(dtype))


def run_mfma(ops, q_all, contexts, q_lens, k_pool, v_pool, table, slots, q_heads, kv_heads, head_dim, window,
             scale, per_tile, row_tiles, n_splits=1, keys_per_split=0, decode_only=None, tile_waves=1,
             max_context_dev=None):
    """Drive the matrix-core kernel the way the attention part does: tiles of
    ``per_tile`` tokens for the chosen sequences; returns [tokens, Hq*D] (rows of
    sequences that were not chosen stay zero)."""
    tokens = sum(q_lens)
    as_dev = lambda values: torch.tensor(values, dtype=torch.int32).cuda()  # noqa: E731
    loc = [0]
    for n in q_lens:
        loc.append(loc[-1] + n)
    tile_seq, tile_q0 = [], []
    for s, n in enumerate(q_lens):
        if decode_only is not None and (n == 1) != decode_only:
            continue
        for first in range(0, n, per_tile):
            tile_seq.append(s)
            tile_q0.append(first)
    stride = (q_heads + 2 * kv_heads) * head_dim
    buffer = torch.zeros((tokens, stride))
    buffer[:, : q_heads * head_dim] = q_all
    buffer = buffer.to(torch.bfloat16).cuda()
    out = torch.zeros((tokens, q_heads * head_dim), dtype=torch.bfloat16).cuda()
    part_o = part_ml = None
    if n_splits > 1:
        units = len(tile_seq) * kv_heads * n_splits
        part_o = torch.full((units * 16 * row_tiles * head_dim,), float("nan")).cuda()
        part_ml = torch.full((units * 16 * row_tiles * 2,), float("nan")).cuda()
    ops.paged_attention_mfma(buffer, stride, k_pool, v_pool, table, as_dev(tile_seq), as_dev(tile_q0), len(tile_seq),
                             as_dev(slots), as_dev(contexts), as_dev(q_lens), as_dev(loc), out, q_heads, kv_heads,
                             head_dim, window, scale, per_tile, row_tiles, n_splits=n_splits,
                             keys_per_split=keys_per_split, part_o=part_o, part_ml=part_ml, tile_waves=tile_waves,
                             max_context_dev=max_context_dev)
    return out.float().cpu()


# (query heads, KV heads, head size, page size); 28/4 and 40/8 are the head counts of the 7B and 14B shapes
MFMA_GEOMETRY = [(16, 2, 128, 16), (4, 2, 32, 8), (3, 1, 32, 8), (6, 6, 64, 4), (16, 1, 96, 32), (12, 4, 256, 16),
                 (28, 4, 128, 16), (40, 8, 128, 64)]


@pytest.mark.parametrize("geometry", MFMA_GEOMETRY)
@pytest.mark.parametrize("row_tiles,tile_waves", [(1, 1), (2, 1), (4, 1), (1, 4), (2, 4), (4, 4), (8, 8), (4, 8)])
def test_paged_attention_mfma_ragged(ops, geometry, row_tiles, tile_waves):
    """The tiled forms (one wave per tile; four waves that share a tile's keys; eight waves per tile of
    128 rows with keys and values in LDS) on
    a ragged batch (reference matrix of contexts and query lengths,
    tests/remote_ragged_gpu_tests.py:118-121): portions with and without context,
    lengths that do not fill a tile, single tokens at page edges."""
    q_heads, kv_heads, head_dim, page_size = geometry
    group = q_heads // kv_heads
    if (group > 16 * row_tiles or (head_dim == 256 and row_tiles > (2 if tile_waves == 1 else 1))):
        pytest.skip("more heads per group than rows, or a variant the kernel refuses")
    if tile_waves >= 4:
        page_size = max(page_size, 16)  # these forms keep the 16 keys of a product in one page
    contexts = [0, 15, 16, 17, 127, 511, 1, 40, 100]
    q_lens = [7, 1, 2, 16, 1, 33, 64, 5, 200]
    lengths = [c + q for c, q in zip(contexts, q_lens)]
    k_pool, v_pool, table, slots, dense = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=70)
    scale = 1.0 / math.sqrt(head_dim)
    g = torch.Generator().manual_seed(71)
    qs, expected = [], []
    for s, (c, n) in enumerate(zip(contexts, q_lens)):
        q = (torch.randn((n, q_heads, head_dim), generator=g) * 2).to(torch.bfloat16).float()
        qs.append(q.reshape(n, -1))
        expected.append(plain_qwen2.causal_attention(q, *dense[s], scale, past_len=c))
    per_tile = (16 * row_tiles) // group
    out = run_mfma(ops, torch.cat(qs), contexts, q_lens, k_pool, v_pool, table, slots, q_heads, kv_heads, head_dim,
                   None, scale, per_tile, row_tiles, tile_waves=tile_waves)
    torch.testing.assert_close(out, torch.cat(expected), **tol(torch.bfloat16))


@pytest.mark.parametrize("geometry", MFMA_GEOMETRY)
@pytest.mark.parametrize("splits", [(1, 0), (3, 704), (16, 128), (64, 32)])
@pytest.mark.parametrize("tile_waves", [1, 4])
def test_paged_attention_mfma_decode_splits(ops, geometry, splits, tile_waves):
    """Single tokens over contexts up to 2047 (boundary lengths of
    tests/remote_gpu_tests.py:204), the keys cut into parts that are merged;
    parts beyond a short context are empty.  With one wave per part and with four
    (a part of 32 keys then leaves three of them without a key)."""
    q_heads, kv_heads, head_dim, page_size = geometry
    if tile_waves == 4:
        page_size = max(page_size, 16)
    n_splits, per_split = splits
    contexts = [0, 1, 15, 16, 17, 127, 128, 129, 1000, 2047]
    q_lens = [1] * len(contexts)
    lengths = [c + 1 for c in contexts]
    k_pool, v_pool, table, slots, dense = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=72)
    scale = 1.0 / math.sqrt(head_dim)
    g = torch.Generator().manual_seed(73)
    qs, expected = [], []
    for s, c in enumerate(contexts):
        q = (torch.randn((1, q_heads, head_dim), generator=g) * 2).to(torch.bfloat16).float()
        qs.append(q.reshape(1, -1))
        expected.append(plain_qwen2.causal_attention(q, *dense[s], scale, past_len=c))
    out = run_mfma(ops, torch.cat(qs), contexts, q_lens, k_pool, v_pool, table, slots, q_heads, kv_heads, head_dim,
                   None, scale, 1, 1, n_splits=n_splits, keys_per_split=per_split, tile_waves=tile_waves)
    torch.testing.assert_close(out, torch.cat(expected), **tol(torch.bfloat16))
    if n_splits > 1:
        # as in a captured step: the size of a part is derived on the device from the longest context,
        # here once the true one and once a loose bound
        for longest in (max(lengths), 3000):
            out = run_mfma(ops, torch.cat(qs), contexts, q_lens, k_pool, v_pool, table, slots, q_heads, kv_heads,
                           head_dim, None, scale, 1, 1, n_splits=n_splits, tile_waves=tile_waves,
                           max_context_dev=torch.tensor([longest], dtype=torch.int32).cuda())
            torch.testing.assert_close(out, torch.cat(expected), **tol(torch.bfloat16))


@pytest.mark.parametrize("geometry", [(16, 2, 128, 16), (6, 2, 32, 16), (5, 5, 64, 32)])
@pytest.mark.parametrize("row_tiles", [1, 2, 4, 8, -4])
@pytest.mark.parametrize("splits", [(3, 512), (5, 256), (9, 128)])
def test_paged_attention_mfma_prompt_portions_with_their_keys_cut(ops, geometry, row_tiles, splits):
    """Portions of prompts behind long contexts, tiles of 16 to 128 rows whose keys are cut into
    parts (some of them empty for the shorter sequences, some ending inside the portion); tiles of 128
    rows, and of 64 where ``row_tiles`` is given as -4, in the form that shares keys and values through LDS."""
    q_heads, kv_heads, head_dim, page_size = geometry
    through_lds = row_tiles in (8, -4)
    row_tiles = abs(row_tiles)
    group = q_heads // kv_heads
    if group > 16 * row_tiles:
        pytest.skip("the group does not fit the tile")
    n_splits, per_split = splits
    contexts, q_lens = [1000, 0, 300, 37], [40, 70, 9, 33]
    lengths = [c + n for c, n in zip(contexts, q_lens)]
    k_pool, v_pool, table, slots, dense = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=82)
    scale = 1.0 / math.sqrt(head_dim)
    g = torch.Generator().manual_seed(83)
    qs, expected = [], []
    for s, (c, n) in enumerate(zip(contexts, q_lens)):
        q = (torch.randn((n, q_heads, head_dim), generator=g) * 2).to(torch.bfloat16).float()
        qs.append(q.reshape(n, -1))
        expected.append(plain_qwen2.causal_attention(q, *dense[s], scale, past_len=c))
    per_tile = (16 * row_tiles) // group
    out = run_mfma(ops, torch.cat(qs), contexts, q_lens, k_pool, v_pool, table, slots, q_heads, kv_heads, head_dim,
                   None, scale, per_tile, row_tiles, n_splits=n_splits, keys_per_split=per_split,
                   tile_waves=8 if through_lds else 4)
    torch.testing.assert_close(out, torch.cat(expected), **tol(torch.bfloat16))


@pytest.mark.parametrize("window", [5, 32, 100])
def test_paged_attention_mfma_window(ops, window):
    q_heads, kv_heads, head_dim = 4, 2, 64
    contexts = [0, 90, 300, 33]
    q_lens = [40, 1, 17, 1]
    lengths = [c + q for c, q in zip(contexts, q_lens)]
    scale = 1.0 / math.sqrt(head_dim)
    for page_size, variants in ((8, ((1, 1),)), (16, ((4, 1), (4, 2), (8, 8), (8, 4))), (64, ((4, 4), (8, 8), (8, 4)))):
        k_pool, v_pool, table, slots, dense = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=74)
        g = torch.Generator().manual_seed(75)
        qs, expected = [], []
        for s, (c, n) in enumerate(zip(contexts, q_lens)):
            q = (torch.randn((n, q_heads, head_dim), generator=g) * 2).to(torch.bfloat16).float()
            qs.append(q.reshape(n, -1))
            expected.append(plain_qwen2.causal_attention(q, *dense[s], scale, past_len=c, window=window))
        want = torch.cat(expected)
        for tile_waves, row_tiles in variants:
            tiled = run_mfma(ops, torch.cat(qs), contexts, q_lens, k_pool, v_pool, table, slots, q_heads, kv_heads,
                             head_dim, window, scale, 8 * row_tiles, row_tiles, tile_waves=tile_waves)  # (groups of two)
            torch.testing.assert_close(tiled, want, **tol(torch.bfloat16))
        rows = [40, 58]  # the two single-token sequences
        for tile_waves in ((1,) if page_size < 16 else (1, 4)):
            split = run_mfma(ops, torch.cat(qs), contexts, q_lens, k_pool, v_pool, table, slots, q_heads, kv_heads,
                             head_dim, window, scale, 1, 1, n_splits=4, keys_per_split=32, decode_only=True,
                             tile_waves=tile_waves)
            torch.testing.assert_close(split[rows], want[rows], **tol(torch.bfloat16))


@pytest.mark.parametrize("geometry", [(16, 2, 128, 16), (16, 1, 96, 32), (12, 4, 256, 16), (6, 6, 64, 16)])
def test_paged_attention_mfma_decode_hundreds_of_parts(ops, geometry):
    """Two single tokens over 9,000 and 3,100 keys cut into parts of 32 and 64 keys: the merge sums
    up to 282 parts per row, most of them in its loop behind the parts it fetches early; one far key
    carries the weight of the first sequence, so a part lost or counted twice shows."""
    q_heads, kv_heads, head_dim, page_size = geometry
    group = q_heads // kv_heads
    lengths, far = [9000, 3100], 7777
    k_pool, v_pool, table, slots, dense = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=91)
    scale = 1.0 / math.sqrt(head_dim)
    g = torch.Generator().manual_seed(92)
    qs = [torch.stack([dense[0][0][far, h // group] * 2.0 for h in range(q_heads)])[None].to(torch.bfloat16).float(),
          (torch.randn((1, q_heads, head_dim), generator=g) * 2).to(torch.bfloat16).float()]
    contexts = [n - 1 for n in lengths]
    expected = torch.cat([plain_qwen2.causal_attention(q, *dense[s], scale, past_len=contexts[s])
                          for s, q in enumerate(qs)])
    for n_splits, per_split, tile_waves in [(282, 32, 1), (141, 64, 1), (71, 128, 4)]:
        out = run_mfma(ops, torch.cat([q.reshape(1, -1) for q in qs]), contexts, [1, 1], k_pool, v_pool, table, slots,
                       q_heads, kv_heads, head_dim, None, scale, 1, 1, n_splits=n_splits, keys_per_split=per_split,
                       tile_waves=tile_waves)
        torch.testing.assert_close(out, expected, **tol(torch.bfloat16))


@pytest.mark.parametrize("joined_rows", [0, 32])
@pytest.mark.parametrize("geometry", [(16, 2, 128, 16), (28, 4, 128, 16), (6, 2, 64, 32)])
def test_attention_planning_of_steps_with_single_tokens_beside_portions(ops, geometry, joined_rows, monkeypatch):
    """The planner of the attention part on a step as a scheduler makes it: four sequences that bring one
    token over 1 to 3,001 keys beside two prompt portions (one behind 2,000 cached keys), once with two
    launches (decode form and prompt form) and once with the single tokens riding in the prompt form's
    launch, against plain attention per sequence."""
    from cie_amd.engine.batch import PagedView, StepBatch
    from cie_amd.parts import attention

    monkeypatch.setattr(attention, "JOINED_DECODE_ROWS", joined_rows)
    q_heads, kv_heads, head_dim, page_size = geometry
    contexts = [0, 31, 600, 3000, 100, 2000]
    q_lens = [1, 1, 1, 1, 40, 70]
    lengths = [c + n for c, n in zip(contexts, q_lens)]
    k_pool, v_pool, table, slots, dense = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=95)
    scale = 1.0 / math.sqrt(head_dim)
    g = torch.Generator().manual_seed(96)
    total = sum(q_lens)
    width = (q_heads + 2 * kv_heads) * head_dim
    qkv = torch.zeros((total, width), dtype=torch.bfloat16)
    expected, row = [], 0
    for s, (c, n) in enumerate(zip(contexts, q_lens)):
        q = (torch.randn((n, q_heads, head_dim), generator=g) * 2).to(torch.bfloat16)
        qkv[row: row + n, : q_heads * head_dim] = q.reshape(n, -1)
        expected.append(plain_qwen2.causal_attention(q.float(), *dense[s], scale, past_len=c))
        row += n
    as_dev = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")  # noqa: E731
    loc = [0]
    for n in q_lens:
        loc.append(loc[-1] + n)
    positions = [c + i for c, n in zip(contexts, q_lens) for i in range(n)]
    seq_of_token = [s for s, n in enumerate(q_lens) for _ in range(n)]
    batch = StepBatch(tokens=total, sequences=len(q_lens), token_ids=as_dev([0] * total), positions=as_dev(positions),
                      seq_of_token=as_dev(seq_of_token), seq_slot=as_dev(slots), seq_start=as_dev(contexts),
                      seq_q_len=as_dev(q_lens), q_start_loc=as_dev(loc), logit_rows=as_dev([0]),
                      host_slots=list(slots), host_starts=contexts, host_q_lens=q_lens)
    view = PagedView(k_pool, v_pool, table, page_size)
    launches = []
    real = ops.paged_attention_mfma
    monkeypatch.setattr(ops, "paged_attention_mfma", lambda *a, **k: (launches.append(k["tokens_per_tile"]), real(*a, **k))[1])
    out = attention.attend(qkv.cuda(), batch, view, q_heads, kv_heads, head_dim, None, scale)
    assert len(launches) == (1 if joined_rows else 2), launches
    torch.testing.assert_close(out.float().cpu(), torch.cat(expected), **tol(torch.bfloat16))


def test_paged_attention_mfma_far_key(ops):
    """One key among two thousand carries the weight: output = its value row, in
    the tiled form and in every split layout."""
    q_heads, kv_heads, head_dim, page_size = 16, 2, 128, 16
    length, far = 2000, 1234
    k_pool, v_pool, table, slots, dense = build_cache(torch.bfloat16, [length], kv_heads, head_dim, page_size, seed=76)
    k, v = dense[0]
    q = torch.stack([k[far, h // 8] * 2.0 for h in range(q_heads)])[None].to(torch.bfloat16).float()
    scale = 1.0 / math.sqrt(head_dim)
    expect = plain_qwen2.causal_attention(q, k, v, scale, past_len=length - 1)
    for tile_waves in (1, 4):
        for n_splits, per_split in [(1, 0), (7, 288), (63, 32)]:
            out = run_mfma(ops, q.reshape(1, -1), [length - 1], [1], k_pool, v_pool, table, slots, q_heads, kv_heads,
                           head_dim, None, scale, 1, 1, n_splits=n_splits, keys_per_split=per_split,
                           tile_waves=tile_waves)
            torch.testing.assert_close(out, expect, **tol(torch.bfloat16))
            torch.testing.assert_close(out.view(q_heads, head_dim), v[far].repeat_interleave(8, dim=0), rtol=0.05, atol=0.05)
    # the prompt form: the last of 40 tokens asks for the far key; the four waves of its tile each see a
    # quarter of the keys and only one of them holds the key that counts
    q_many = torch.cat([torch.randn((39, q_heads, head_dim), generator=torch.Generator().manual_seed(77)), q])
    q_many = q_many.to(torch.bfloat16).float()
    expect = plain_qwen2.causal_attention(q_many, k, v, scale, past_len=length - 40)
    # (tiles of 128 rows, and of 64 a second time: the form through LDS, whose two halves each see every other block)
    for row_tiles, tile_waves in ((1, 4), (2, 4), (4, 4), (8, 8), (4, 8)):
        out = run_mfma(ops, q_many.reshape(40, -1), [length - 40], [40], k_pool, v_pool, table, slots, q_heads,
                       kv_heads, head_dim, None, scale, 2 * row_tiles, row_tiles, tile_waves=tile_waves)
        torch.testing.assert_close(out, expect, **tol(torch.bfloat16))
        torch.testing.assert_close(out[-1].view(q_heads, head_dim), v[far].repeat_interleave(8, dim=0), rtol=0.05, atol=0.05)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_and_window(ops, dtype):
    """One far key is made to dominate: the output must be its value row.  With a
    window that excludes it, it must vanish; the window's edge is exact."""
    q_heads, kv_heads, head_dim, page_size = 4, 2, 32, 8
    length, far = 400, 37
    k_pool, v_pool, table, slots, dense = build_cache(dtype, [length], kv_heads, head_dim, page_size, seed=30)
    k, v = dense[0]
    q = torch.zeros((1, q_heads, head_dim))
    for h in range(q_heads):
        q[0, h] = k[far, h // 2] * 4.0  # aligned with the far key, far larger score than any other
    q = q.to(dtype).float()
    scale = 1.0 / math.sqrt(head_dim)
    args = (k_pool, v_pool, table, torch.tensor([length - 1], dtype=torch.int32).cuda(),
            torch.tensor([0], dtype=torch.int32).cuda(), torch.tensor(slots, dtype=torch.int32).cuda(),
            1, q_heads, kv_heads, head_dim)
    qd = q.reshape(1, -1).to(dtype).cuda()
    full = ops.paged_attention_generic(qd, q_heads * head_dim, *args, None, scale).float().cpu()
    expect_full = plain_qwen2.causal_attention(q, k, v, scale, past_len=length - 1)
    torch.testing.assert_close(full, expect_full, **tol(dtype))
    # the far key carries nearly all the weight
    torch.testing.assert_close(full.reshape(q_heads, head_dim), v[far].repeat_interleave(2, dim=0), rtol=0.1, atol=0.1)
    for window in (length - far, length - far - 1):  # far key just inside / just outside
        got = ops.paged_attention_generic(qd, q_heads * head_dim, *args, window, scale).float().cpu()
        expect = plain_qwen2.causal_attention(q, k, v, scale, past_len=length - 1, window=window)
        torch.testing.assert_close(got, expect, **tol(dtype))
    assert (got - full).abs().max() > 0.1  # outside the window the answer changes


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geometry", [(4, 2, 16, 16), (3, 1, 48, 8), (16, 2, 128, 16)])
def test_rope_kv_write(ops, dtype, geometry):
    q_heads, kv_heads, head_dim, page_size = geometry
    theta, max_pos = 10000.0, 512
    lengths = [40, 3, 100]
    starts = [30, 0, 99]  # tokens of this step: positions start..length-1
    k_pool, v_pool, table, slots, _ = build_cache(dtype, lengths, kv_heads, head_dim, page_size, seed=40)
    k_before, v_before = k_pool.clone(), v_pool.clone()
    positions, seq_of_token = [], []
    for s, (start, n) in enumerate(zip(starts, lengths)):
        positions += list(range(start, n))
        seq_of_token += [s] * (n - start)
    t = len(positions)
    qkv = rand((t, (q_heads + 2 * kv_heads) * head_dim), dtype, 41)
    original = qkv.float().cpu()
    cos, sin = plain_qwen2.rope_tables(head_dim, max_pos, theta)
    half = head_dim // 2
    pos_t = torch.tensor(positions)
    ops.rope_kv_write(qkv, cos[:, :half].contiguous().cuda(), sin[:, :half].contiguous().cuda(),
                      torch.tensor(positions, dtype=torch.int32).cuda(),
                      torch.tensor(seq_of_token, dtype=torch.int32).cuda(),
                      torch.tensor(slots, dtype=torch.int32).cuda(), table, k_pool, v_pool,
                      q_heads, kv_heads, head_dim)
    q_in = original[:, : q_heads * head_dim].view(t, q_heads, head_dim)
    k_in = original[:, q_heads * head_dim: (q_heads + kv_heads) * head_dim].view(t, kv_heads, head_dim)
    v_in = original[:, (q_heads + kv_heads) * head_dim:].view(t, kv_heads, head_dim)
    q_expect = plain_qwen2.apply_rope(q_in, cos, sin, pos_t)
    k_expect = plain_qwen2.apply_rope(k_in, cos, sin, pos_t)
    torch.testing.assert_close(qkv.float().cpu()[:, : q_heads * head_dim].view(t, q_heads, head_dim), q_expect, **tol(dtype))
    table_h = table.cpu()
    touched = torch.zeros(k_pool.shape[:3], dtype=torch.bool)  # [page, head, row]
    for i, (pos, s) in enumerate(zip(positions, seq_of_token)):
        page = int(table_h[slots[s], pos // page_size])
        row = pos % page_size
        torch.testing.assert_close(k_pool[page, :, row].float().cpu(), k_expect[i], **tol(dtype))
        torch.testing.assert_close(v_pool[page, :, :, row].float().cpu(), v_in[i], rtol=0, atol=0)  # transposed
        touched[page, :, row] = True
    # nothing else in the pools moved
    untouched = ~touched.cuda()
    assert torch.equal(k_pool[untouched], k_before[untouched])
    assert torch.equal(v_pool.transpose(2, 3)[untouched], v_before.transpose(2, 3)[untouched])


@pytest.mark.parametrize("geometry", [(16, 2, 128, 16, 2048), (4, 2, 32, 8, 96), (3, 1, 64, 4, 328), (5, 5, 96, 32, 200)])
@pytest.mark.parametrize("rows", [1, 7, 16, 24, 40, 64, 72, 100, 128])
@pytest.mark.parametrize("waves", [None, 1, 8])
def test_gemm_qkv_rope_equals_product_then_rotation(ops, geometry, rows, waves):
    """The q/k/v product whose epilogue rotates and writes the cache, against the plain
    product followed by the rotation kernel (themselves checked against the plain
    implementation above): rotated queries, touched cache rows and untouched ones."""
    q_heads, kv_heads, head_dim, page_size, hidden = geometry
    n = (q_heads + 2 * kv_heads) * head_dim
    row_tiles = 1 if rows <= 16 else 2 if rows <= 32 else 4
    if waves == 1 and row_tiles > 1:
        waves = 4  # the fewest with more than 16 rows
    lengths = [40, 35, 100, 33][: max(1, min(4, rows))]  # every sequence has at least rows / 4 tokens
    k_pool, v_pool, table, slots, _ = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=44)
    k_two, v_two = k_pool.clone(), v_pool.clone()
    # the rows: the last tokens of the sequences in turn (decode rows), several per sequence when rows > sequences
    positions, seq_of_token = [], []
    for i in range(rows):
        s = i % len(lengths)
        positions.append(lengths[s] - 1 - i // len(lengths))
        seq_of_token.append(s)
    assert min(positions) >= 0
    a = rand((rows, hidden), torch.bfloat16, 45)
    w, b = rand((n, hidden), torch.bfloat16, 46, 0.3), rand((n,), torch.bfloat16, 47)
    cos, sin = plain_qwen2.rope_tables(head_dim, 512, 1e6)
    half = head_dim // 2
    cos, sin = cos[:, :half].contiguous().cuda(), sin[:, :half].contiguous().cuda()
    meta = (torch.tensor(positions, dtype=torch.int32).cuda(), torch.tensor(seq_of_token, dtype=torch.int32).cuda(),
            torch.tensor(slots, dtype=torch.int32).cuda(), table)
    fused = ops.gemm_qkv_rope(w, a, b, cos, sin, *meta, k_pool, v_pool, q_heads, kv_heads, head_dim, waves=waves)
    plain_qkv = ops.gemm_fused(w, ops.EPI_BF16, a, bias=b, plan=None if waves is None else (row_tiles, waves, 1))
    ops.rope_kv_write(plain_qkv, cos, sin, *meta, k_two, v_two, q_heads, kv_heads, head_dim)
    q_cols = q_heads * head_dim
    # one bf16 step at most (the two kernels may round a fused multiply-add differently)
    step = dict(rtol=2 ** -7, atol=1e-6)
    torch.testing.assert_close(fused[:, :q_cols].float(), plain_qkv[:, :q_cols].float(), **step)
    torch.testing.assert_close(k_pool.float(), k_two.float(), **step)
    assert torch.equal(v_pool, v_two)
    # without rotation and without cache writes
    k_before, v_before = k_pool.clone(), v_pool.clone()
    bare = ops.gemm_qkv_rope(w, a, b, cos, sin, *meta, k_pool, v_pool, q_heads, kv_heads, head_dim, rotate=False,
                             write_kv=False, waves=waves)
    if waves is None:  # the two plans may cut K differently: sums in another order
        torch.testing.assert_close(bare[:, :q_cols].float(), ops.gemm_fused(w, ops.EPI_BF16, a, bias=b)[:, :q_cols].float(), **step)
    else:
        same_plan = ops.gemm_fused(w, ops.EPI_BF16, a, bias=b, plan=(row_tiles, waves, 1))
        if row_tiles == 1:
            assert torch.equal(bare[:, :q_cols], same_plan[:, :q_cols])
        else:  # a pair of column tiles per workgroup here, one there: the waves' sums meet in another order
            torch.testing.assert_close(bare[:, :q_cols].float(), same_plan[:, :q_cols].float(), **step)
    assert torch.equal(k_pool, k_before) and torch.equal(v_pool, v_before)
    with pytest.raises(ValueError, match="steps of 32"):
        ops.gemm_qkv_rope(w[: 3 * 16], a, None, cos[:, :8].contiguous(), sin[:, :8].contiguous(), *meta,
                          k_pool[..., :16].contiguous(), v_pool[:, :, :16].contiguous(), 1, 1, 16)


@pytest.mark.parametrize("geometry", [(16, 2, 128, 16, 2048), (4, 2, 32, 8, 96), (3, 1, 64, 4, 328), (28, 4, 128, 16, 3584),
                                      (5, 5, 96, 32, 200), (64, 8, 128, 16, 8192)])
@pytest.mark.parametrize("rows", [1, 3, 8, 13, 16, 17])
@pytest.mark.parametrize("waves", [None, 1, 8])
def test_gemm_qkv_rope_that_makes_the_norm_itself(ops, geometry, rows, waves):
    """The q/k/v product of up to 16 rows that is given the float32 residual stream instead of normalised rows:
    the rotated queries and the cache against float64 arithmetic on the kernel's own operand rounding (rows are
    bf16(x * weight), their 1/rms multiplies the sums), and against the two kernels it replaces."""
    q_heads, kv_heads, head_dim, page_size, hidden = geometry
    if not ops.folds_norm(rows, hidden):
        with pytest.raises(ValueError, match="makes the norm of up to"):
            ops.gemm_qkv_rope(rand(((q_heads + 2 * kv_heads) * head_dim, hidden), torch.bfloat16, 1), None, None,
                              *([torch.zeros(1, device="cuda")] * 8), q_heads, kv_heads, head_dim,
                              folded=(torch.zeros((rows, hidden), device="cuda"), torch.ones(hidden, device="cuda"), 1e-6))
        return
    n = (q_heads + 2 * kv_heads) * head_dim
    eps = 1e-5
    lengths = [40, 35, 100, 33, 64, 1, 17, 90, 41, 36, 101, 34, 65, 2, 18, 91][:rows]
    k_pool, v_pool, table, slots, _ = build_cache(torch.bfloat16, lengths, kv_heads, head_dim, page_size, seed=61)
    k_two, v_two = k_pool.clone(), v_pool.clone()
    positions = [length - 1 for length in lengths]
    residual = rand((rows, hidden), torch.float32, 62, 2.0) * torch.linspace(0.2, 3.0, rows, device="cuda")[:, None]
    norm_weight = (1.0 + rand((hidden,), torch.float32, 64, 0.3)).contiguous()
    w, b = rand((n, hidden), torch.bfloat16, 65, 0.05), rand((n,), torch.bfloat16, 66)
    cos, sin = plain_qwen2.rope_tables(head_dim, 512, 1e6)
    half = head_dim // 2
    cos, sin = cos[:, :half].contiguous().cuda(), sin[:, :half].contiguous().cuda()
    meta = (torch.tensor(positions, dtype=torch.int32).cuda(), torch.arange(rows, dtype=torch.int32).cuda(),
            torch.tensor(slots, dtype=torch.int32).cuda(), table)
    before = residual.clone()
    fused = ops.gemm_qkv_rope(w, None, b, cos, sin, *meta, k_pool, v_pool, q_heads, kv_heads, head_dim,
                              waves=waves, folded=(residual, norm_weight, eps))
    assert torch.equal(residual, before)  # the stream is read only
    scale = torch.rsqrt(residual.double().pow(2).mean(-1, keepdim=True) + eps)
    operand = (residual * norm_weight).to(torch.bfloat16).double()  # the rows as the kernel rounds them
    unrotated = ((operand @ w.double().t()) * scale + b.double()).to(torch.bfloat16)
    ops.rope_kv_write(unrotated, cos, sin, *meta, k_two, v_two, q_heads, kv_heads, head_dim)
    q_cols = q_heads * head_dim
    # a bf16 step in a value before its rotation moves the rotated pair by that much of the larger of the two
    step = dict(rtol=2 ** -6, atol=2 ** -7 * float(unrotated.float().abs().max()))
    torch.testing.assert_close(fused[:, :q_cols].float(), unrotated[:, :q_cols].float(), **step)
    torch.testing.assert_close(k_pool.float(), k_two.float(), **step)
    torch.testing.assert_close(v_pool.float(), v_two.float(), **step)
    # ... and it agrees with the two kernels it replaces to the rounding of their different order
    normed = ops.add_rmsnorm(residual.clone(), None, norm_weight, eps, torch.bfloat16)
    two = ops.gemm_qkv_rope(w, normed, b, cos, sin, *meta, k_two, v_two, q_heads, kv_heads, head_dim)
    torch.testing.assert_close(fused[:, :q_cols].float(), two[:, :q_cols].float(), rtol=2 ** -5,
                               atol=2 ** -6 * float(unrotated.float().abs().max()))


def test_rope_shift_invariance():
    """Scores of rotated q and k depend on the distance of their positions only
    (pins sign and pairing of the rotation in the plain implementation)."""
    head_dim = 32
    cos, sin = plain_qwen2.rope_tables(head_dim, 600, 10000.0)
    g = torch.Generator().manual_seed(50)
    q = torch.randn((1, 1, head_dim), generator=g, dtype=torch.float64)
    k = torch.randn((1, 1, head_dim), generator=g, dtype=torch.float64)
    cos, sin = cos.double(), sin.double()

    def score(m, n):
        qm = plain_qwen2.apply_rope(q, cos, sin, torch.tensor([m]))
        kn = plain_qwen2.apply_rope(k, cos, sin, torch.tensor([n]))
        return (qm * kn).sum()

    assert abs(score(10, 3) - score(210, 203)) < 1e-3  # float32 tables limit the agreement
    assert abs(score(10, 3) - score(10, 4)) > 1e-3


def test_sample_greedy_and_temperature(ops):
    g = torch.Generator().manual_seed(60)
    logits = torch.randn((6, 1003), generator=g).cuda() * 3
    logits[2, 500] = logits[2, 17] = logits[2].max() + 1  # a tie: the lower index wins
    out = ops.sample(logits)
    assert out.tolist() == torch.argmax(logits, dim=-1).tolist()
    assert out[2].item() == 17
    temperature = torch.tensor([0.0, 0.7, 1.0, 1.3, 0.7, 2.0]).cuda()
    uniform = torch.tensor([0.3, 0.0, 0.999999, 0.5, 0.25, 0.75]).cuda()
    got = ops.sample(logits, temperature, uniform).tolist()
    assert got[0] == out[0].item()  # temperature 0 is greedy
    for r in range(1, 6):
        p = torch.softmax(logits[r].double() / temperature[r].double(), dim=-1).cpu()
        cdf = torch.cumsum(p, dim=0)
        u = float(uniform[r])
        lo = cdf[got[r] - 1].item() if got[r] > 0 else 0.0
        assert lo - 1e-5 <= u <= cdf[got[r]].item() + 1e-5, (r, got[r], lo, u, cdf[got[r]].item())


@pytest.mark.parametrize("vocab", [1024, 4099, 8192, 9001, 151936])
def test_sample_over_many_chunks(ops, vocab):
    """A vocabulary of many chunks of the kernel's walk (and one that ends inside a chunk, with rows that are
    not 16-byte aligned), and from 8,192 tokens on rows that many workgroups take in parts and a second kernel
    finishes: the token is the one whose share of [0, 1) holds the row's number, for numbers at the very start,
    inside and at the very end, and for a row whose weight sits in its last tokens."""
    g = torch.Generator().manual_seed(62)
    rows = 7
    logits = (torch.randn((rows, vocab), generator=g) * 2).cuda()
    logits[5, vocab - 3:] += 30.0       # nearly all weight in the last three tokens
    logits[6, : vocab - 1] -= 60.0      # all of it in the last one
    temperature = torch.tensor([0.7, 1.0, 1.5, 0.3, 1.0, 1.0, 1.0]).cuda()
    uniform = torch.tensor([0.0, 0.37, 0.999999, 0.5, 0.123456, 0.9, 0.4]).cuda()
    got = ops.sample(logits, temperature, uniform).tolist()
    for r in range(rows):
        p = torch.softmax(logits[r].double() / temperature[r].double(), dim=-1).cpu()
        cdf = torch.cumsum(p, dim=0)
        u = float(uniform[r])
        lo = cdf[got[r] - 1].item() if got[r] > 0 else 0.0
        assert 0 <= got[r] < vocab and lo - 2e-5 <= u <= cdf[got[r]].item() + 2e-5, (r, got[r], lo, u, cdf[got[r]].item())
    assert got[5] >= vocab - 3 and got[6] == vocab - 1
    # the same draw whatever else is in the batch: row 1 alone
    assert ops.sample(logits[1:2], temperature[1:2], uniform[1:2]).tolist() == [got[1]]
    # rows without a temperature among the others: the first index of the largest logit
    logits[3, vocab - 1] = logits[3, 5] = logits[3].max() + 1
    mixed = temperature.clone()
    mixed[3] = mixed[0] = 0.0
    again = ops.sample(logits, mixed, uniform).tolist()
    assert again[3] == 5 and again[0] == int(torch.argmax(logits[0])) and again[1] == got[1] and again[6] == got[6]


@pytest.mark.parametrize("vocab", [3000, 40000])
def test_sample_with_a_number_next_to_one_never_draws_a_token_without_probability(ops, vocab):
    """The row's number is the largest below 1 and the target may round past the running sums (they are made
    in another order than the total): the token then is the last one that has any probability, never the
    last of a chunk or part whose tail lies so far below the maximum that its terms are zero.  Many rows
    with their weight in the first tokens, spread over several chunks (and, in the large vocabulary, two parts)."""
    g = torch.Generator().manual_seed(64)
    rows = 256
    logits = torch.full((rows, vocab), -1.0e4)
    heads = torch.randint(1500, 2600, (rows,), generator=g)
    for r in range(rows):
        logits[r, : heads[r]] = torch.randn(int(heads[r]), generator=g) * 0.5
    temperature = torch.full((rows,), 1.0)
    uniform = torch.full((rows,), 1.0 - 2.0 ** -24)
    assert float(uniform[0]) < 1.0
    got = ops.sample(logits.cuda(), temperature.cuda(), uniform.cuda()).tolist()
    for r in range(rows):
        p = torch.softmax(logits[r].double(), dim=-1)
        assert p[got[r]] > 0, (r, got[r], int(heads[r]))
        assert got[r] >= int(heads[r]) - 3, (r, got[r], int(heads[r]))  # and it is (next to) the last such token


def test_sample_frequencies(ops):
    """Empirical frequencies on a four-token vocabulary follow softmax(l / T)."""
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0]]).repeat(4000, 1).cuda()
    g = torch.Generator().manual_seed(61)
    uniform = torch.rand(4000, generator=g).cuda()
    temperature = torch.full((4000,), 0.8).cuda()
    got = ops.sample(logits, temperature, uniform)
    freq = torch.bincount(got.long().cpu(), minlength=4).double() / 4000
    expect = torch.softmax(torch.tensor([0.0, 1.0, 2.0, -1.0]).double() / 0.8, dim=0)
    assert (freq - expect).abs().max() < 0.03


@pytest.mark.parametrize("shape", [(1, 64, 128), (8, 2560, 2048), (16, 96, 328), (17, 208, 1032), (40, 66, 264),
                                   (64, 2048, 1408), (70, 48, 96)])
@pytest.mark.parametrize("plan", [None, "few", "many", "paired"])
def test_gemm_fused_epilogues(ops, shape, plan):
    """The fused few-row product: SiLU-gate and residual-accumulate epilogues, for every plan the
    kernel has (the fewest and the most waves per workgroup, partial tiles summed through LDS;
    one or two column tiles per workgroup with more than 16 rows; more than 64 rows as several
    rows of workgroups), against float64 products."""
    m, n, k = shape
    row_tiles = 1 if m <= 16 else 2 if m <= 32 else 4
    if plan == "paired" and row_tiles == 1:
        pytest.skip("workgroups of 16 rows take one column tile")
    chosen = {None: None, "few": (row_tiles, 1 if row_tiles == 1 else 4, 1), "many": (row_tiles, 8, 1),
              "paired": (row_tiles, 8, 2)}[plan]
    a, w = rand((m, k), torch.bfloat16, 80), rand((n, k), torch.bfloat16, 81, 0.3)
    b = rand((n,), torch.bfloat16, 82)
    exact = a.double() @ w.double().t()
    gate, up = exact[:, : n // 2], exact[:, n // 2:]
    out = ops.gemm_fused(w, ops.EPI_SILU, a, plan=chosen)
    assert out.shape == (m, n // 2) and out.dtype == torch.bfloat16
    want = torch.nn.functional.silu(gate) * up
    torch.testing.assert_close(out.double(), want, rtol=1e-2, atol=1e-2 * float(want.abs().max()))
    plain_out = ops.gemm_fused(w, ops.EPI_F32, a, bias=b, plan=chosen)
    torch.testing.assert_close(plain_out.double(), exact + b.double(), rtol=1e-4, atol=2e-4 * math.sqrt(k))
    residual = rand((m, n), torch.float32, 83, 2.0)
    before = residual.clone()
    parts = -(-n // 16)
    sumsq = torch.full((m + 2, parts), float("nan")).cuda()
    assert ops.gemm_fused(w, ops.EPI_RESID, a, bias=b, residual_out=residual, sumsq_out=sumsq, plan=chosen) is sumsq
    want = before.double() + exact + b.double()
    torch.testing.assert_close(residual.double(), want, rtol=1e-4, atol=2e-4 * math.sqrt(k))
    padded = torch.zeros((m, parts * 16), dtype=torch.float64).cuda()
    padded[:, :n] = want
    torch.testing.assert_close(sumsq[:m].double(), padded.pow(2).view(m, parts, 16).sum(-1), rtol=1e-4, atol=1e-3)
    assert torch.isnan(sumsq[m:]).all()


def test_gemm_fused_random_shapes(ops):
    """Seeded random shapes (rows to 70, any column count, K any multiple of 8) through every
    epilogue, against float64 products: the edges of row tiles, column tiles and K slices in
    combinations the hand-picked shapes do not hold."""
    rng = random.Random(1234)
    for case in range(40):
        m, n, k = rng.randint(1, 70), 2 * rng.randint(1, 150), 8 * rng.randint(1, 180)
        k_parts = rng.choice([1, 1, 2, 3, 5])
        a, w = rand((m, k), torch.bfloat16, 300 + case), rand((n, k), torch.bfloat16, 400 + case, 0.3)
        b = rand((n,), torch.bfloat16, 500 + case)
        exact = a.double() @ w.double().t()
        tag = f"case {case}: m={m} n={n} k={k} parts={k_parts}"
        out = ops.gemm_fused(w, ops.EPI_F32, a, bias=b)
        torch.testing.assert_close(out.double(), exact + b.double(), rtol=1e-4, atol=2e-4 * math.sqrt(k), msg=lambda t: f"{tag}: {t}")
        parts = ops.gemm_shared_rows(w, ops.EPI_PARTIAL, a, bias=b, k_parts=k_parts, column_tiles=1 + case % 2, waves=2 + case % 3)
        torch.testing.assert_close(parts.double().sum(0), exact + b.double(), rtol=1e-4, atol=2e-4 * math.sqrt(k),
                                   msg=lambda t: f"{tag}: {t}")
        gated = ops.gemm_fused(w, ops.EPI_SILU, a)
        want = torch.nn.functional.silu(exact[:, : n // 2]) * exact[:, n // 2:]
        torch.testing.assert_close(gated.double(), want, rtol=1e-2, atol=1e-2 * float(want.abs().max()) + 1e-6,
                                   msg=lambda t: f"{tag}: {t}")
        residual = rand((m, n), torch.float32, 600 + case, 2.0)
        want = residual.double() + exact + b.double()
        sumsq = ops.gemm_fused(w, ops.EPI_RESID, a, bias=b, residual_out=residual)
        torch.testing.assert_close(residual.double(), want, rtol=1e-4, atol=2e-4 * math.sqrt(k), msg=lambda t: f"{tag}: {t}")
        torch.testing.assert_close(sumsq.double().sum(-1), want.pow(2).sum(-1), rtol=1e-3, atol=1e-3, msg=lambda t: f"{tag}: {t}")


@pytest.mark.parametrize("shape", [(1, 64, 256), (8, 2048, 11008), (13, 96, 328), (16, 48, 1032), (40, 200, 1032),
                                   (64, 2048, 2752), (5, 50, 264), (8, 3584, 1024), (72, 2048, 11008), (100, 200, 1032),
                                   (128, 96, 328)])
@pytest.mark.parametrize("k_parts", [1, 3, 4])
def test_gemm_fused_partial_products_and_their_norm(ops, shape, k_parts):
    """K cut into parts: the float32 partial products sum to the product (bias once); and the same parts added
    into a float32 stream with atomic adds leave the stream plus the product there, twice in a row."""
    m, n, k = shape
    a, w, b = rand((m, k), torch.bfloat16, 94), rand((n, k), torch.bfloat16, 95, 0.3), rand((n,), torch.bfloat16, 96)
    parts = ops.gemm_shared_rows(w, ops.EPI_PARTIAL, a, bias=b, k_parts=k_parts)
    assert parts.shape == (k_parts, m, n) and parts.dtype == torch.float32
    exact = a.double() @ w.double().t() + b.double()
    torch.testing.assert_close(parts.double().sum(0), exact, rtol=1e-4, atol=2e-4 * math.sqrt(k))
    residual = rand((m, n), torch.float32, 97, 2.0)
    before = residual.double()
    for turn in (1, 2):
        out = ops.gemm_shared_rows(w, ops.EPI_ATOMIC, a, bias=b, k_parts=k_parts, add_into=residual)
        assert out is residual
        torch.testing.assert_close(residual.double(), before + turn * exact, rtol=1e-4, atol=turn * 2e-4 * math.sqrt(k))
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(w, ops.EPI_ATOMIC, a, k_parts=k_parts)                       # nothing to add into
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(w, ops.EPI_PARTIAL, a, k_parts=k_parts, add_into=residual)   # only the atomic form adds
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(w, ops.EPI_ATOMIC, a, k_parts=k_parts, add_into=residual[:, : n - 8])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 8), (5, 200), (40, 4864), (3, 25)])
def test_silu_mul_with_the_rows_scale(ops, dtype, shape):
    """The SiLU-gate kernel applying the 1/rms that the rows of the product before it lacked."""
    tokens, inter = shape
    hidden, parts, eps = 96, 7, 1e-5
    gate_up = rand((tokens, 2 * inter), dtype, 710, 3.0)
    sumsq = rand((tokens, parts), torch.float32, 711).abs() * 40 + 1
    factor = torch.rsqrt(sumsq.double().sum(-1, keepdim=True) / hidden + eps)
    g, u = gate_up.double()[:, :inter] * factor, gate_up.double()[:, inter:] * factor
    want = torch.nn.functional.silu(g) * u
    got = ops.silu_mul(gate_up, row_sumsq=sumsq, hidden=hidden, eps=eps)
    torch.testing.assert_close(got.double(), want, **({"rtol": 1e-2, "atol": 1e-3} if dtype == torch.bfloat16 else {"rtol": 1e-5, "atol": 1e-6}))
    plain = torch.nn.functional.silu(gate_up.double()[:, :inter]) * gate_up.double()[:, inter:]
    torch.testing.assert_close(ops.silu_mul(gate_up).double(), plain,
                               **({"rtol": 1e-2, "atol": 1e-3} if dtype == torch.bfloat16 else {"rtol": 1e-5, "atol": 1e-6}))


@pytest.mark.parametrize("shape", [(1, 128, 64), (8, 2048, 2048), (13, 200, 328), (16, 96, 1032)])
def test_norm_folded_into_the_products_around_it(ops, shape):
    """o_proj adds into the residual and leaves residual * weight; the gate/up product
    applies each row's 1 / rms to its sums: together the same as the residual product,
    the norm kernel and the plain gate/up product."""
    m, hidden, k = shape
    inter = 2 * 88
    a = rand((m, k), torch.bfloat16, 700)
    w_o, b_o = rand((hidden, k), torch.bfloat16, 701, 0.3), rand((hidden,), torch.bfloat16, 702)
    w_gu = rand((inter, hidden), torch.bfloat16, 703, 0.3)
    norm_weight = (rand((hidden,), torch.float32, 704) + 1).to(torch.bfloat16)
    eps = 1e-5
    residual = rand((m, hidden), torch.float32, 705, 2.0)
    apart = residual.clone()
    sumsq = ops.gemm_fused(w_o, ops.EPI_RESID, a, bias=b_o, residual_out=apart)
    normed = ops.rmsnorm_from_sumsq(apart, sumsq, norm_weight, eps)
    want = ops.gemm_fused(w_gu, ops.EPI_SILU, normed)
    scaled = torch.empty((m, hidden), dtype=torch.bfloat16).cuda()
    folded_sumsq = ops.gemm_fused(w_o, ops.EPI_RESID, a, bias=b_o, residual_out=residual,
                                  norm_weight=norm_weight.float().contiguous(), scaled_out=scaled)
    assert torch.equal(residual, apart) and torch.equal(folded_sumsq, sumsq)
    got = ops.gemm_fused(w_gu, ops.EPI_SILU, scaled, row_sumsq=folded_sumsq, eps=eps)
    # the same values rounded to bf16 at another point (before instead of after the division by the rms)
    exact = torch.nn.functional.silu(
        plain_qwen2.rms_norm(residual.cpu(), norm_weight.float().cpu(), eps).double() @ w_gu.double().cpu().t()[:, : inter // 2]
    ) * (plain_qwen2.rms_norm(residual.cpu(), norm_weight.float().cpu(), eps).double() @ w_gu.double().cpu().t()[:, inter // 2:])
    bound = 1e-2 * float(exact.abs().max())
    torch.testing.assert_close(got.double().cpu(), exact, rtol=2e-2, atol=bound)
    torch.testing.assert_close(want.double().cpu(), exact, rtol=2e-2, atol=bound)
    with pytest.raises(ValueError, match="scale"):
        ops.gemm_fused(w_gu, ops.EPI_BF16, scaled, row_sumsq=folded_sumsq, eps=eps)


@pytest.mark.parametrize("norm_dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_from_sumsq(ops, norm_dtype):
    residual = rand((5, 1000), torch.float32, 90, 2.0)
    weight = (rand((1000,), torch.float32, 91) + 1).to(norm_dtype)
    full = residual.pow(2).sum(-1, keepdim=True)
    sumsq = (full * torch.softmax(rand((5, 13), torch.float32, 92), dim=-1)).contiguous()
    out = ops.rmsnorm_from_sumsq(residual, sumsq, weight, 1e-5)
    want = plain_qwen2.rms_norm(residual.cpu(), weight.float().cpu(), 1e-5)
    torch.testing.assert_close(out.float().cpu(), want, **tol(torch.bfloat16))


def test_argmax_over_a_large_vocabulary(ops):
    """Two-stage greedy: chunk edges, ties across chunks (the lower index wins), a vocabulary that is no multiple of the chunk."""
    vocab = 151936 + 5
    g = torch.Generator().manual_seed(93)
    logits = torch.randn((9, vocab), generator=g).cuda()
    logits[1, vocab - 1] = 50.0
    logits[2, 0] = 50.0
    logits[3, 2047] = logits[3, 2048] = 50.0
    logits[4, 100000] = logits[4, 4096] = 50.0
    out = ops.sample(logits).tolist()
    assert out == torch.argmax(logits, dim=-1).tolist()
    assert out[1:5] == [vocab - 1, 0, 2047, 4096]


@pytest.mark.parametrize("shape", [(17, 40, 24), (64, 2560, 2048), (150, 99, 72), (300, 515, 328), (2048, 256, 2048)])
def test_gemm_library_matches_float64(ops, shape):
    """The cached interface to the vendor library: with and without bias, rows given as a strided view,
    twice (the second call takes the kept plan)."""
    m, n, k = shape
    a, w, b = rand((m, k), torch.bfloat16, 20), rand((n, k), torch.bfloat16, 21), rand((n,), torch.bfloat16, 22)
    expect = a.double() @ w.double().t()
    for _ in range(2):
        out = ops.gemm_library(a, w)
        if out is None:
            pytest.skip("the library has no algorithm for this shape")
        assert out.dtype == torch.bfloat16 and out.shape == (m, n)
        torch.testing.assert_close(out.double(), expect, rtol=1e-2, atol=1e-2 * math.sqrt(k))
        out = ops.gemm_library(a, w, b)
        torch.testing.assert_close(out.double(), expect + b.double(), rtol=1e-2, atol=1e-2 * math.sqrt(k))
        exact = ops.gemm_library(a, w, out_dtype=torch.float32)  # as for logits
        if exact is not None:
            assert exact.dtype == torch.float32
            torch.testing.assert_close(exact.double(), expect, rtol=1e-4, atol=1e-4 * math.sqrt(k))
    if k % 8 == 0:
        wide = torch.zeros((m, k + 64), dtype=torch.bfloat16).cuda()
        wide[:, :k] = a
        torch.testing.assert_close(ops.gemm_library(wide[:, :k], w, b).double(), expect + b.double(), rtol=1e-2,
                                   atol=1e-2 * math.sqrt(k))


@pytest.mark.parametrize("waves", [2, 3, 4])
@pytest.mark.parametrize("shape", [(5, 32, 128), (17, 656, 520), (37, 80, 264), (64, 2000, 2048), (70, 48, 88), (128, 130, 1160)])
def test_gemm_shared_rows_matches_float64(ops, shape, waves):
    """The form for 17 to 128 rows whose waves own columns and share the rows of A through LDS: plain with
    bias, SiLU-gate with and without rows that lack their 1/rms, and partial products of a cut K (parts that
    end inside a slice of 128, a part without any k, bias in the first part only); widths and row counts that
    fill no tile, one and two tiles a wave, rows given as a strided view."""
    m, n, k = shape
    a, w, b = rand((m, k), torch.bfloat16, 40), rand((n, k), torch.bfloat16, 41, scale=0.1), rand((n,), torch.bfloat16, 42)
    wide = torch.zeros((m, k + 24), dtype=torch.bfloat16).cuda()
    wide[:, :k] = a
    expect = a.double() @ w.double().t()
    tol = dict(rtol=1e-2, atol=1e-2 * math.sqrt(k) * 0.1)
    for tiles in (1, 2):
        out = ops.gemm_shared_rows(w, ops.EPI_BF16, a, bias=b, column_tiles=tiles, waves=waves)
        torch.testing.assert_close(out.double(), expect + b.double(), **tol)
        for parts in (1, 3, 7):
            rows = wide[:, :k] if parts == 3 else a
            out = ops.gemm_shared_rows(w, ops.EPI_PARTIAL, rows, bias=b, column_tiles=tiles, waves=waves, k_parts=parts)
            assert out.shape == (parts, m, n) and out.dtype == torch.float32
            torch.testing.assert_close(out.double().sum(0), expect + b.double(), rtol=1e-4, atol=1e-4 * math.sqrt(k))
    out = ops.gemm_shared_rows(w, ops.EPI_F32, a, bias=b, waves=waves)  # as for logits
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.double(), expect + b.double(), rtol=1e-4, atol=1e-4 * math.sqrt(k))
    gate, up = expect[:, : n // 2], expect[:, n // 2:]
    out = ops.gemm_shared_rows(w, ops.EPI_SILU, a, waves=waves)
    assert out.shape == (m, n // 2) and out.dtype == torch.bfloat16
    torch.testing.assert_close(out.double(), torch.nn.functional.silu(gate) * up, rtol=2e-2, atol=2e-2)
    # rows that lack their 1/rms: partial sums of squares of some other row vector stand for the norm's (a count
    # that is no multiple of four, one that a lane holds at once, one that needs the loop behind it)
    for sumsq_parts in (5, 8, 264):
        sumsq = torch.rand((m + 3, sumsq_parts), generator=torch.Generator().manual_seed(43)).cuda() * k / sumsq_parts
        scale = torch.rsqrt(sumsq[:m].double().sum(1, keepdim=True) / k + 1e-5)
        out = ops.gemm_shared_rows(w, ops.EPI_SILU, a, waves=waves, row_sumsq=sumsq, eps=1e-5)
        torch.testing.assert_close(out.double(), torch.nn.functional.silu(gate * scale) * (up * scale), rtol=2e-2, atol=2e-2)


def test_gemm_shared_rows_refuses_what_it_does_not_take(ops):
    a, w = rand((129, 64), torch.bfloat16, 44), rand((32, 64), torch.bfloat16, 45)
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(w, ops.EPI_BF16, a)            # more than 128 rows
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(w, ops.EPI_RESID, a[:8])       # an epilogue of the other form
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(w, ops.EPI_BF16, a[:8], k_parts=2)
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(w, ops.EPI_BF16, a[:8], waves=5)
    with pytest.raises(ValueError):
        ops.gemm_shared_rows(rand((32, 60), torch.bfloat16, 46), ops.EPI_BF16, rand((8, 60), torch.bfloat16, 47))


def test_gemm_library_with_every_algorithm_timed(ops):
    """A row count that an engine has named has every algorithm of the library timed at a shape's first
    call, and the one kept is still the product: shapes that no other test uses, so that their first call is here."""
    assert ops._tune_level(768) == 1  # (a multiple of 256 that nobody has named: the heuristic's candidates)
    with ops.library_search({768}):
        assert ops._tune_level(768) == 2 and ops._tune_level(1024) == 1 and ops._tune_level(700) == 0
        for n, k in ((1040, 520), (264, 1288)):
            a, w, b = rand((768, k), torch.bfloat16, 30), rand((n, k), torch.bfloat16, 31), rand((n,), torch.bfloat16, 32)
            expect = a.double() @ w.double().t()
            for _ in range(2):
                out = ops.gemm_library(a, w)
                if out is None:
                    pytest.skip("the library has no algorithm for this shape")
                torch.testing.assert_close(out.double(), expect, rtol=1e-2, atol=1e-2 * math.sqrt(k))
                torch.testing.assert_close(ops.gemm_library(a, w, b).double(), expect + b.double(), rtol=1e-2,
                                           atol=1e-2 * math.sqrt(k))
                exact = ops.gemm_library(a, w, out_dtype=torch.float32)
                if exact is not None:
                    torch.testing.assert_close(exact.double(), expect, rtol=1e-4, atol=1e-4 * math.sqrt(k))
    assert ops._tune_level(768) == 1  # outside the block nothing is searched
