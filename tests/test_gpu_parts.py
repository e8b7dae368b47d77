"""GPU: each part of a layer alone against the plain implementation, and a toy
mixer with state of its own that is registered, built and stepped from the test
without any change to the package."""

from __future__ import annotations

import math

import pytest
import torch

import plain_qwen2 as plain
import replay_util
from conftest import random_tokens

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


def check(got, expect, dtype):
    """float32: rounding of float32 sums.  bfloat16: every intermediate is rounded
    to 8 mantissa bits (relative 2^-9), so the error of an element scales with the
    magnitude of the tensor it was summed from, not with the element itself: the
    absolute allowance is tied to the tensor's largest value."""
    if dtype == "float32":
        torch.testing.assert_close(got, expect, rtol=1e-4, atol=2e-5)
    else:
        scale = float(expect.abs().max())
        torch.testing.assert_close(got, expect, rtol=2e-2, atol=1e-2 * max(scale, 1.0))



def harness(needs, lengths, page_size=8, dtype=torch.float32):
    """A cache with one unit per need and live requests of the given lengths (nothing committed yet)."""
    from cie_amd.cache import CacheManager
    from cie_amd.engine.device_cache import DeviceCache

    manager = CacheManager(needs, page_size, kv_tokens=512, max_running=max(4, len(lengths)), max_model_len=256)
    device_cache = DeviceCache(manager, dtype, torch.device("cuda:0"))
    for i, n in enumerate(lengths):
        manager.admit(f"r{i}")
    manager.ensure_capacity_batch({f"r{i}": n for i, n in enumerate(lengths)})
    device_cache.sync()
    return manager, device_cache


def test_device_pools_follow_what_each_need_stores():
    """Keys and values of one width share a group; a need without values has a key pool only; values of
    another width get a pool of that width (transposed, as the attention kernels read values)."""
    from cie_amd.cache import PagedKV

    needs = [PagedKV(2, 16), PagedKV(1, 24, values=False), PagedKV(2, 16), PagedKV(2, 16, value_dim=8)]
    manager, device_cache = harness(needs, [5])
    pages = 512 // 8 + 1  # (one page beyond the pool's for padded rows of captured steps)
    assert [tuple(p.shape) for p in device_cache.key_pools] == [(2, pages, 2, 8, 16), (1, pages, 1, 8, 24), (1, pages, 2, 8, 16)]
    assert device_cache.value_pools[1] is None
    assert tuple(device_cache.value_pools[0].shape) == (2, pages, 2, 16, 8)
    assert tuple(device_cache.value_pools[2].shape) == (1, pages, 2, 8, 8)
    latent = device_cache.view(1)
    assert latent.v_pool is None and tuple(latent.k_pool.shape) == (pages, 1, 8, 24)
    assert device_cache.view(2).k_pool.data_ptr() == device_cache.key_pools[0][1].data_ptr()
    stats = manager.stats()
    assert [g.reserved_bytes for g in stats.groups] == [8 * 64 * 2 * 2, 8 * 24 * 2, 8 * 48 * 2]


def batch_of(manager, portions):
    """StepBatch for portions [(request index, start, count)], built by hand."""
    from cie_amd.engine.batch import StepBatch

    positions, seq_of_token, slots, starts, q_lens, loc = [], [], [], [], [], [0]
    for s, (index, start, count) in enumerate(portions):
        positions += list(range(start, start + count))
        seq_of_token += [s] * count
        slots.append(manager.slot(f"r{index}"))
        starts.append(start)
        q_lens.append(count)
        loc.append(loc[-1] + count)
    as_dev = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")  # noqa: E731
    total = len(positions)
    return StepBatch(tokens=total, sequences=len(portions), token_ids=as_dev([0] * total), positions=as_dev(positions),
                     seq_of_token=as_dev(seq_of_token), seq_slot=as_dev(slots), seq_start=as_dev(starts),
                     seq_q_len=as_dev(q_lens), q_start_loc=as_dev(loc), logit_rows=as_dev(list(range(total))),
                     host_slots=slots, host_starts=starts, host_q_lens=q_lens)


def bound(part, prefix, dtype, seed, scale=0.2):
    from cie_amd.weights import RandomSource

    expected = part.expected_tensors(prefix)
    tensors = RandomSource(seed, std=scale).load(expected, dtype, "cuda:0")
    part.bind(tensors, prefix, torch.float32 if dtype == "float32" else torch.bfloat16, torch.device("cuda:0"))
    return {k: v.float().cpu() for k, v in tensors.items()}


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
    from cie_amd.parts.norm import RMSNorm

    norm = RMSNorm(size=200, eps=3e-5)
    weights = bound(norm, "n.", dtype, 1)
    act = norm.dtype
    residual = torch.randn((6, 200), device="cuda") * 2
    branch = torch.randn((6, 200), device="cuda").to(act)
    expect_sum = residual.cpu() + branch.float().cpu()
    out = norm.forward(residual, branch, act)
    torch.testing.assert_close(residual.cpu(), expect_sum, rtol=0, atol=0)
    check(out.float().cpu(), plain.rms_norm(expect_sum, weights["n.weight"], 3e-5), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(dtype):
    from cie_amd.parts.feed_forward import GatedMLP

    mlp = GatedMLP(hidden_size=72, intermediate_size=200)
    w = bound(mlp, "m.", dtype, 2)
    x = torch.randn((9, 72), device="cuda").to(mlp.dtype)
    expect = plain.swiglu(x.float().cpu(), w["m.gate_proj.weight"], w["m.up_proj.weight"], w["m.down_proj.weight"])
    check(mlp.forward(x).float().cpu(), expect, dtype)
    with pytest.raises(ValueError, match="silu"):
        GatedMLP(8, 8, activation="gelu")


def test_position_part_tables_and_no_position():
    from cie_amd.parts.position import NoPosition, RotaryHalf

    rotary = RotaryHalf(head_dim=48, theta=5e5, max_position=77)
    cos, sin = rotary.tables(torch.device("cuda:0"))
    ref_cos, ref_sin = plain.rope_tables(48, 77, 5e5)
    assert cos.shape == (77, 24) and cos.dtype == torch.float32
    torch.testing.assert_close(cos.cpu(), ref_cos[:, :24], rtol=0, atol=0)
    torch.testing.assert_close(sin.cpu(), ref_sin[:, :24], rtol=0, atol=0)
    assert not NoPosition().rotates


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rotary", [True, False])
def test_attention_part_whole_and_in_portions(dtype, rotary):
    """The mixer alone: one request whole, another cut into a portion and single
    tokens, in one batch with it.  Without rotation it reduces to plain masked
    attention (library routine, see tests/test_plain.py)."""
    from cie_amd.config import PartSpec
    from cie_amd.parts.attention import Attention

    hidden, heads, kv_heads, head_dim = 40, 6, 2, 16
    position = (PartSpec.of("rotary_half", head_dim=head_dim, theta=1e4, max_position=256) if rotary
                else PartSpec.of("none", head_dim=head_dim, max_position=256))
    attention = Attention(hidden, heads, kv_heads, head_dim, qkv_bias=True, out_bias=False, position=position)
    # float32 takes very peaked softmaxes (scores of order 10); in bfloat16 the rounding of q and k alone
    # moves such scores by tenths, so that case runs at a scale where the softmax is still well conditioned
    w = bound(attention, "a.", dtype, 3, scale=0.5 if dtype == "float32" else 0.3)
    lengths = [29, 21]
    manager, device_cache = harness([attention.cache_need()], lengths,
                                    dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    g = torch.Generator().manual_seed(4)
    xs = [torch.randn((n, hidden), generator=g).to(attention.dtype) for n in lengths]
    config = {"hidden_size": hidden, "num_attention_heads": heads, "head_dim": head_dim, "attention_bias": True}
    expected = []
    for x, n in zip(xs, lengths):
        if rotary:
            cos, sin = plain.rope_tables(head_dim, n, 1e4)
        else:
            cos, sin = torch.ones((n, head_dim)), torch.zeros((n, head_dim))
        expected.append(plain.attention_layer(x.float(), w, "a.", config, cos, sin, torch.arange(n)))
    view = device_cache.view(0)
    # step 1: request 0 whole, first 10 tokens of request 1
    got0 = {}
    out = attention.forward(torch.cat([xs[0], xs[1][:10]]).cuda(), batch_of(manager, [(0, 0, 29), (1, 0, 10)]), view)
    got0[0], first = out[:29], out[29:]
    manager.commit_lengths({"r0": 29, "r1": 10})
    # step 2: a 9-token portion of request 1; steps 3, 4: single tokens
    second = attention.forward(xs[1][10:19].cuda(), batch_of(manager, [(1, 10, 9)]), view)
    third = attention.forward(xs[1][19:20].cuda(), batch_of(manager, [(1, 19, 1)]), view)
    fourth = attention.forward(xs[1][20:21].cuda(), batch_of(manager, [(1, 20, 1)]), view)
    check(got0[0].float().cpu(), expected[0], dtype)
    check(torch.cat([first, second, third, fourth]).float().cpu(), expected[1], dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim,padded,rows", [(80, 96, 40), (40, 64, 5), (112, 128, 70), (24, 32, 1), (144, 256, 9)])
def test_attention_part_with_a_head_size_between_those_of_the_matrix_core_kernels(dtype, head_dim, padded, rows):
    """A head size that the matrix-core attention does not take runs as the next one it does: the cache and the
    kernels see heads padded with zeros, the tensors of the checkpoint and the results are those of the head size
    itself (the plain functions at that size), with a whole-head rotation, a portion and then single tokens, and in
    bfloat16 without a word from the generic kernel."""
    import warnings

    from cie_amd.config import PartSpec
    from cie_amd.parts.attention import Attention

    hidden, heads, kv_heads = 64, 4, 2
    position = PartSpec.of("rotary_half", head_dim=head_dim, theta=1e4, max_position=256)
    attention = Attention(hidden, heads, kv_heads, head_dim, qkv_bias=True, out_bias=False, position=position)
    assert attention.kernel_head_dim == padded and attention.cache_need().head_dim == padded
    assert attention.expected_tensors("a.")["a.q_proj.weight"].shape == (heads * head_dim, hidden)
    w = bound(attention, "a.", dtype, 7, scale=0.3)
    assert attention.w_qkv.shape == ((heads + 2 * kv_heads) * padded, hidden) and attention.w_o.shape == (hidden, heads * padded)
    total = rows + 3
    manager, device_cache = harness([attention.cache_need()], [total],
                                    dtype=torch.float32 if dtype == "float32" else torch.bfloat16, page_size=16)
    g = torch.Generator().manual_seed(8)
    x = torch.randn((total, hidden), generator=g).to(attention.dtype)
    config = {"hidden_size": hidden, "num_attention_heads": heads, "head_dim": head_dim, "attention_bias": True}
    cos, sin = plain.rope_tables(head_dim, total, 1e4)
    expected = plain.attention_layer(x.float(), w, "a.", config, cos, sin, torch.arange(total))
    view = device_cache.view(0)
    with warnings.catch_warnings():
        warnings.simplefilter("error")  # the generic kernel would say so in bfloat16
        first = attention.forward(x[:rows].cuda(), batch_of(manager, [(0, 0, rows)]), view)
        manager.commit_lengths({"r0": rows})
        rest = [attention.forward(x[i:i + 1].cuda(), batch_of(manager, [(0, i, 1)]), view) for i in range(rows, total)]
    check(torch.cat([first] + rest).float().cpu(), expected, dtype)
    # what the cache holds behind a head's own dimensions is zeros
    assert float(view.k_pool[..., head_dim:].abs().max()) == 0.0


@pytest.mark.parametrize("page_size", [8, 16])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(24, 1, 32), (40, 1, 64), (34, 2, 128), (64, 1, 32)])
def test_attention_part_with_more_than_sixteen_heads_on_a_key_head(heads, kv_heads, head_dim, page_size):
    """Groups of 17 to 64 query heads on one key head in bfloat16: a token's heads fill two or four 16-row tiles of the
    matrix-core kernels (no word from the generic kernel), as a prompt, as a portion behind context and as single
    tokens over a context that is cut into parts."""
    import warnings

    from cie_amd.config import PartSpec
    from cie_amd.parts.attention import Attention

    hidden = 64
    position = PartSpec.of("rotary_half", head_dim=head_dim, theta=1e4, max_position=512)
    attention = Attention(hidden, heads, kv_heads, head_dim, qkv_bias=True, out_bias=False, position=position)
    w = bound(attention, "a.", "bfloat16", 11, scale=0.2)
    lengths = [245, 37]
    manager, device_cache = harness([attention.cache_need()], lengths, dtype=torch.bfloat16, page_size=page_size)
    g = torch.Generator().manual_seed(12)
    xs = [torch.randn((n, hidden), generator=g).to(attention.dtype) for n in lengths]
    config = {"hidden_size": hidden, "num_attention_heads": heads, "head_dim": head_dim, "attention_bias": True}
    expected = []
    for x, n in zip(xs, lengths):
        cos, sin = plain.rope_tables(head_dim, n, 1e4)
        expected.append(plain.attention_layer(x.float(), w, "a.", config, cos, sin, torch.arange(n)))
    view = device_cache.view(0)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        # request 0: 230 tokens at once, then a portion of 8 beside the first 30 tokens of request 1
        first = attention.forward(xs[0][:230].cuda(), batch_of(manager, [(0, 0, 230)]), view)
        manager.commit_lengths({"r0": 230})
        both = attention.forward(torch.cat([xs[0][230:238], xs[1][:30]]).cuda(), batch_of(manager, [(0, 230, 8), (1, 0, 30)]), view)
        manager.commit_lengths({"r0": 238, "r1": 30})
        got0, got1 = [first, both[:8]], [both[8:]]
        # single tokens of both, one step each (request 0 over more than 192 keys: its keys are cut into parts)
        for step in range(3):
            out = attention.forward(torch.cat([xs[0][238 + step:239 + step], xs[1][30 + step:31 + step]]).cuda(),
                                    batch_of(manager, [(0, 238 + step, 1), (1, 30 + step, 1)]), view)
            manager.commit_lengths({"r0": 239 + step, "r1": 31 + step})
            got0.append(out[:1])
            got1.append(out[1:])
    check(torch.cat(got0).float().cpu(), expected[0][:241], "bfloat16")
    check(torch.cat(got1).float().cpu(), expected[1][:33], "bfloat16")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_dim,rotary_dim,rows", [(32, 16, 7), (64, 32, 1), (48, 20, 5), (128, 64, 40)])
def test_attention_part_with_a_rotation_of_the_first_dimensions_only(dtype, head_dim, rotary_dim, rows):
    """A rotary part built with ``rotary_dim < head_dim`` turns the first ``rotary_dim`` dimensions of every
    head (dimension i with i + rotary_dim / 2, angles of base ``theta`` over ``rotary_dim``) and lets the
    rest pass: the plain rotation on that slice.  With few rows, too, where the projection's own kernel
    would rotate whole heads: it must stand back."""
    import math

    from cie_amd.config import PartSpec
    from cie_amd.parts.attention import Attention
    from cie_amd.parts.position import RotaryHalf

    with pytest.raises(ValueError):
        RotaryHalf(head_dim=32, theta=1e4, max_position=8, rotary_dim=34)
    with pytest.raises(ValueError):
        RotaryHalf(head_dim=32, theta=1e4, max_position=8, rotary_dim=15)
    hidden, heads, kv_heads = 64, 4, 2
    position = PartSpec.of("rotary_half", head_dim=head_dim, theta=1e4, max_position=256, rotary_dim=rotary_dim)
    attention = Attention(hidden, heads, kv_heads, head_dim, qkv_bias=True, out_bias=False, position=position)
    w = bound(attention, "a.", dtype, 5, scale=0.3)
    assert attention.cos.shape == (256, rotary_dim // 2)
    total = rows + 3
    manager, device_cache = harness([attention.cache_need()], [total],
                                    dtype=torch.float32 if dtype == "float32" else torch.bfloat16, page_size=16)
    g = torch.Generator().manual_seed(6)
    x = torch.randn((total, hidden), generator=g).to(attention.dtype)
    # the plain parts, the rotation applied to the leading slice of every head
    cos, sin = plain.rope_tables(rotary_dim, total, 1e4)
    positions = torch.arange(total)

    def heads_of(name):
        return plain.linear(x.float(), w[f"a.{name}.weight"], w[f"a.{name}.bias"]).view(total, -1, head_dim)

    def turned(t):
        return torch.cat([plain.apply_rope(t[..., :rotary_dim], cos, sin, positions), t[..., rotary_dim:]], dim=-1)

    context = plain.causal_attention(turned(heads_of("q_proj")), turned(heads_of("k_proj")), heads_of("v_proj"),
                                     1.0 / math.sqrt(head_dim))
    expected = plain.linear(context, w["a.o_proj.weight"])
    view = device_cache.view(0)
    first = attention.forward(x[:rows].cuda(), batch_of(manager, [(0, 0, rows)]), view)
    manager.commit_lengths({"r0": rows})
    rest = [attention.forward(x[i:i + 1].cuda(), batch_of(manager, [(0, i, 1)]), view) for i in range(rows, total)]
    check(torch.cat([first] + rest).float().cpu(), expected, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_mixer_that_norms_its_heads_between_projection_and_rotation(dtype):
    """The seam between projection and rotation: a variant of the attention mixer, defined here, that
    divides every query and key head by its root mean square before the rotation overrides one method and
    reuses the rest (with the projection's own rotation switched off for it).  Expected: the plain
    functions composed with that norm, whole; the part runs a portion and then single tokens, 32-wide
    heads (which the fused projection would otherwise take)."""
    from cie_amd.config import PartSpec
    from cie_amd.parts.attention import Attention

    hidden, heads, kv_heads, head_dim, eps = 64, 4, 2, 32, 1e-5

    def normed(rows_of_heads):
        wide = rows_of_heads.float()
        return wide * torch.rsqrt(wide.pow(2).mean(-1, keepdim=True) + eps)

    class NormedHeads(Attention):
        def shape_projection(self, qkv, batch):
            rows = qkv.shape[0]
            shaped = qkv.view(rows, heads + 2 * kv_heads, head_dim)
            out = shaped.clone()
            out[:, : heads + kv_heads] = normed(shaped[:, : heads + kv_heads]).to(qkv.dtype)
            return out.view(rows, -1)

    position = PartSpec.of("rotary_half", head_dim=head_dim, theta=1e4, max_position=128)
    mixer = NormedHeads(hidden, heads, kv_heads, head_dim, qkv_bias=True, out_bias=False, position=position)
    w = bound(mixer, "a.", dtype, 8, scale=0.3)
    length = 27
    manager, device_cache = harness([mixer.cache_need()], [length],
                                    dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    x = torch.randn((length, hidden), generator=torch.Generator().manual_seed(9)).to(mixer.dtype)
    cos, sin = plain.rope_tables(head_dim, length, 1e4)
    positions = torch.arange(length)
    proj = lambda name: plain.linear(x.float(), w[f"a.{name}.weight"], w[f"a.{name}.bias"]).view(length, -1, head_dim)
    q = plain.apply_rope(normed(proj("q_proj")), cos, sin, positions)
    k = plain.apply_rope(normed(proj("k_proj")), cos, sin, positions)
    context = plain.causal_attention(q, k, proj("v_proj"), 1.0 / math.sqrt(head_dim))
    expected = plain.linear(context, w["a.o_proj.weight"])
    view = device_cache.view(0)
    first = mixer.forward(x[:12].cuda(), batch_of(manager, [(0, 0, 12)]), view)
    manager.commit_lengths({"r0": 12})
    rest = []
    for at in range(12, length):
        rest.append(mixer.forward(x[at:at + 1].cuda(), batch_of(manager, [(0, at, 1)]), view))
        manager.commit_lengths({"r0": at + 1})
    check(torch.cat([first, *rest]).float().cpu(), expected, dtype)


@pytest.mark.parametrize("part_k", [None, 32])
@pytest.mark.parametrize("rows", [13, 40, 72, 100])
@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part(dtype, rows, part_k, monkeypatch):
    """norm -> mixer -> add -> norm -> feed-forward, the add of the second branch left pending
    (as a tensor) or already done (by a product's epilogue, or by the atomic adds of a product whose K is
    cut into parts), depending on rows and dtype."""
    if part_k is not None:
        from cie_amd.parts import linear

        monkeypatch.setattr(linear, "PART_K", part_k)
        monkeypatch.setattr(linear, "PART_MIN_K", 2 * part_k)
    from cie_amd.config import Qwen2Config
    from cie_amd.parts.block import PreNormBlock

    raw = dict(model_type="qwen2", hidden_size=48, num_hidden_layers=1, num_attention_heads=3,
               num_key_value_heads=3, intermediate_size=88, vocab_size=32, rms_norm_eps=1e-5, rope_theta=1e4,
               max_position_embeddings=128)
    spec = Qwen2Config.from_hf_config(raw).model_spec().layers[0]
    block = PreNormBlock(spec)
    # (bfloat16: softmaxes that 16-bit queries and keys still resolve, as in the attention part's own test; the heads
    # of 16 run on the matrix cores, as heads of 32, where the probabilities are rounded to bfloat16 too)
    w = bound(block, "model.layers.0.", dtype, 5, scale=0.3 if dtype == "float32" else 0.2)
    manager, device_cache = harness([block.cache_need()], [rows], dtype=block.dtype)
    h = torch.randn((rows, 48), generator=torch.Generator().manual_seed(6))
    residual = h.clone().cuda()
    out_residual, pending = block.forward(residual, None, batch_of(manager, [(0, 0, rows)]), device_cache.view(0))
    p = "model.layers.0."
    cos, sin = plain.rope_tables(16, rows, 1e4)
    a = plain.rms_norm(h, w[p + "input_layernorm.weight"], 1e-5)
    mid = h + plain.attention_layer(a, w, p + "self_attn.", raw, cos, sin, torch.arange(rows))
    m = plain.rms_norm(mid, w[p + "post_attention_layernorm.weight"], 1e-5)
    branch = plain.swiglu(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    from cie_amd.parts.linear import Added, RowSumsq

    if isinstance(pending, Added):  # the last product's parts of K added their shares into the stream
        assert part_k is not None and dtype == "bfloat16"
        check(out_residual.cpu(), mid + branch, dtype)
    elif isinstance(pending, RowSumsq):  # few rows in bfloat16: the fused products added both branches themselves
        check(out_residual.cpu(), mid + branch, dtype)
        check(pending.sumsq.sum(-1).cpu(), (mid + branch).pow(2).sum(-1), dtype)
    else:
        check(out_residual.cpu(), mid, dtype)
        check(pending.float().cpu(), branch, dtype)


@pytest.mark.parametrize("rows", [1, 5, 16])
def test_block_whose_first_product_makes_the_norm_itself(rows, monkeypatch):
    """Decode rows whose stream is complete (the layer before added its branch itself): in bfloat16 the block
    hands the stream to its mixer, whose q/k/v product makes the norm of up to 16 rows itself, and no norm
    kernel runs in front of the mixer.  Everything agrees with the plain block."""
    from cie_amd.config import Qwen2Config
    from cie_amd.kernels import ops
    from cie_amd.parts.block import PreNormBlock
    from cie_amd.parts.linear import Added, RowSumsq

    raw = dict(model_type="qwen2", hidden_size=96, num_hidden_layers=1, num_attention_heads=3,
               num_key_value_heads=1, intermediate_size=88, vocab_size=32, rms_norm_eps=1e-5, rope_theta=1e4,
               max_position_embeddings=128)
    block = PreNormBlock(Qwen2Config.from_hf_config(raw).model_spec().layers[0])
    w = bound(block, "model.layers.0.", "bfloat16", 15, scale=0.2)  # (softmaxes that 16-bit keys still resolve)
    prompt = 12
    manager, device_cache = harness([block.cache_need()], [prompt + 1] * rows, dtype=block.dtype)
    g = torch.Generator().manual_seed(16)
    hs = [torch.randn((prompt + 1, 96), generator=g) * (0.5 + 0.25 * i) for i in range(rows)]
    view = device_cache.view(0)
    block.forward(torch.cat([h[:prompt] for h in hs]).cuda(), None,
                  batch_of(manager, [(i, 0, prompt) for i in range(rows)]), view)
    manager.commit_lengths({f"r{i}": prompt for i in range(rows)})
    norms = []
    real = ops.add_rmsnorm
    monkeypatch.setattr(ops, "add_rmsnorm", lambda *a, **k: (norms.append(1), real(*a, **k))[1])
    last = torch.cat([h[prompt:] for h in hs]).cuda()
    out_residual, pending = block.forward(last, Added(), batch_of(manager, [(i, prompt, 1) for i in range(rows)]), view)
    assert not norms, "a norm kernel ran although the product could make the norm"
    assert out_residual.data_ptr() == last.data_ptr()
    p = "model.layers.0."
    cos, sin = plain.rope_tables(32, prompt + 1, 1e4)
    for i, h in enumerate(hs):
        a = plain.rms_norm(h, w[p + "input_layernorm.weight"], 1e-5)
        mid = h + plain.attention_layer(a, w, p + "self_attn.", raw, cos, sin, torch.arange(prompt + 1))
        m = plain.rms_norm(mid, w[p + "post_attention_layernorm.weight"], 1e-5)
        branch = plain.swiglu(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        if isinstance(pending, (Added, RowSumsq)):
            check(out_residual[i: i + 1].cpu(), (mid + branch)[prompt:], "bfloat16")
        else:
            check(out_residual[i: i + 1].cpu(), mid[prompt:], "bfloat16")
            check(pending[i: i + 1].float().cpu(), branch[prompt:], "bfloat16")


# -- a toy mixer with state of its own -----------------------------------------------------
def register_toy():
    """A decaying running sum per request: s_t = decay * s_{t-1} + W x_t, y_t = s_t.
    Its state lives in the cache's fixed-size slots; it is defined, registered
    and wired into an architecture here, outside the package."""
    from cie_amd.cache import FixedState
    from cie_amd.config import LayerCall, LayerSpec, ModelSpec, PartSpec, Qwen2Config, register_architecture
    from cie_amd.parts import Part, register_part
    from cie_amd.weights import TensorSpec

    class RunningSum(Part):
        def __init__(self, hidden_size: int, decay: float) -> None:
            self.hidden_size, self.decay = hidden_size, decay

        def cache_need(self):
            return FixedState((self.hidden_size,), "float32")

        def expected_tensors(self, prefix):
            return {prefix + "in_proj.weight": TensorSpec((self.hidden_size, self.hidden_size))}

        def bind(self, tensors, prefix, dtype, device):
            super().bind(tensors, prefix, dtype, device)
            self.weight = tensors[prefix + "in_proj.weight"].float()

        def forward(self, x, batch, view, writes=True):
            projected = x.float() @ self.weight.t()
            out = torch.empty_like(projected)
            row = 0
            for slot, count in zip(batch.host_slots, batch.host_q_lens):
                state = view.state[slot].clone()
                for _ in range(count):
                    state = self.decay * state + projected[row]
                    out[row] = state
                    row += 1
                if writes:
                    view.state[slot] = state
            return out.to(x.dtype)

    class RunningSumOnDevice(RunningSum):
        """The same sum with every request's slot read on the device: what changes from step to step
        comes from the batch's device tensors, the loops follow the step's shape alone, so a step that holds
        it may be captured and replayed."""

        graph_safe = True

        def forward(self, x, batch, view, writes=True):
            projected = x.float() @ self.weight.t()
            slots = batch.seq_slot.long()
            state = view.state.index_select(0, slots)
            out = torch.empty_like(projected)
            row, last = 0, []
            for index, count in enumerate(batch.host_q_lens):
                current = state[index]
                for _ in range(count):
                    current = self.decay * current + projected[row]
                    out[row] = current
                    row += 1
                last.append(current)
            if writes:
                view.state.index_copy_(0, slots, torch.stack(last))
            return out.to(x.dtype)

    class TwoStates(Part):
        """A mixer with two states of different shape and type beside each other: the two inputs before
        this one (float32 [2, hidden]) and a count of the tokens seen (int32 [1]).
        y_t = W (x_t + x_{t-1} / 2 + x_{t-2} / 4) / (1 + count_t / 8)."""

        def __init__(self, hidden_size: int) -> None:
            self.hidden_size = hidden_size

        def cache_need(self):
            return (FixedState((2, self.hidden_size), "float32"), FixedState((1,), "int32"))

        def expected_tensors(self, prefix):
            return {prefix + "in_proj.weight": TensorSpec((self.hidden_size, self.hidden_size))}

        def bind(self, tensors, prefix, dtype, device):
            super().bind(tensors, prefix, dtype, device)
            self.weight = tensors[prefix + "in_proj.weight"].float()

        def forward(self, x, batch, view, writes=True):
            window, count = view
            out = torch.empty((x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
            row = 0
            for slot, tokens in zip(batch.host_slots, batch.host_q_lens):
                before, seen = window.state[slot].clone(), int(count.state[slot])
                for _ in range(tokens):
                    current = x[row].float()
                    out[row] = (self.weight @ (current + before[0] / 2 + before[1] / 4)) / (1 + seen / 8)
                    before = torch.stack([current, before[0]])
                    seen += 1
                    row += 1
                if writes:
                    window.state[slot] = before
                    count.state[slot] = seen
            return out.to(x.dtype)

    class ToyConfig(Qwen2Config):
        architecture = "ToyRunningSumForCausalLM"
        MIXER = "running_sum"

        def model_spec(self) -> ModelSpec:
            base = super().model_spec()
            attention_layer = base.layers[0]
            toy_layer = LayerSpec(
                mixer=(PartSpec.of(self.MIXER, hidden_size=self.hidden_size) if self.MIXER == "two_states"
                       else PartSpec.of(self.MIXER, hidden_size=self.hidden_size, decay=0.75)),
                feed_forward=attention_layer.feed_forward, norm1=attention_layer.norm1, norm2=attention_layer.norm2,
                names=(("norm1", "input_layernorm"), ("mixer", "toy"), ("norm2", "post_attention_layernorm"),
                       ("feed_forward", "mlp")))
            # layers: 0 toy, 1 attention; order: toy, attention, toy again (its own state unit)
            return ModelSpec(
                architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                layers=(toy_layer, attention_layer),
                order=(LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2)),
                final_norm=base.final_norm, tie_word_embeddings=True, max_position=self.max_position_embeddings)

    class OnlyStateConfig(ToyConfig):
        """Every layer the running sum: a model that caches nothing in pages."""

        architecture = "ToyOnlyStateForCausalLM"

        def model_spec(self) -> ModelSpec:
            mixed = super().model_spec()
            return ModelSpec(
                architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                layers=mixed.layers[:1], order=(LayerCall(0, 0), LayerCall(0, 1)),
                final_norm=mixed.final_norm, tie_word_embeddings=True, max_position=self.max_position_embeddings)

    class OnDeviceConfig(ToyConfig):
        architecture = "ToyRunningSumOnDeviceForCausalLM"
        MIXER = "running_sum_on_device"

    class TwoStatesConfig(ToyConfig):
        architecture = "ToyTwoStatesForCausalLM"
        MIXER = "two_states"

    register_part("mixer", "running_sum", RunningSum)
    register_part("mixer", "running_sum_on_device", RunningSumOnDevice)
    register_part("mixer", "two_states", TwoStates)
    register_architecture("ToyRunningSumOnDeviceForCausalLM", OnDeviceConfig)
    register_architecture("ToyTwoStatesForCausalLM", TwoStatesConfig)
    register_architecture("ToyRunningSumForCausalLM", ToyConfig)
    register_architecture("ToyOnlyStateForCausalLM", OnlyStateConfig)
    return ToyConfig


def toy_plain(raw, weights, tokens, order=(0, 1, 0), two_states=False):
    """Whole-sequence reference of the toy model, from the plain parts."""
    eps = raw["rms_norm_eps"]
    h = weights["model.embed_tokens.weight"][torch.tensor(tokens)]
    cos, sin = plain.rope_tables(plain.head_dim_of(raw), len(tokens), raw["rope_theta"])

    def toy(x, p):
        if two_states:
            zero = torch.zeros_like(x[:1])
            mixed = x + torch.cat([zero, x[:-1]]) / 2 + torch.cat([zero, zero, x[:-2]])[: len(x)] / 4
            return (mixed @ weights[p + "toy.in_proj.weight"].t()) / (1 + torch.arange(len(x))[:, None] / 8)
        projected = x @ weights[p + "toy.in_proj.weight"].t()
        state = torch.zeros(raw["hidden_size"])
        rows = []
        for row in projected:
            state = 0.75 * state + row
            rows.append(state)
        return torch.stack(rows)

    def mlp(x, p):
        return plain.swiglu(x, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                            weights[p + "mlp.down_proj.weight"])

    for layer in order:
        p = f"model.layers.{layer}."
        a = plain.rms_norm(h, weights[p + "input_layernorm.weight"], eps)
        if layer == 0:
            h = h + toy(a, p)
        else:
            h = h + plain.attention_layer(a, weights, p + "self_attn.", raw, cos, sin, torch.arange(len(tokens)))
        h = h + mlp(plain.rms_norm(h, weights[p + "post_attention_layernorm.weight"], eps), p)
    h = plain.rms_norm(h, weights["model.norm.weight"], eps)
    return h @ weights["model.embed_tokens.weight"].t()


def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path):
    from cie_amd.config import build_engine_config, load_config
    from cie_amd.engine import Runner, load_model
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    register_toy()
    raw = dict(architectures=["ToyRunningSumForCausalLM"], model_type="qwen2", hidden_size=32, num_hidden_layers=2,
               num_attention_heads=2, num_key_value_heads=1, intermediate_size=56, vocab_size=64,
               rms_norm_eps=1e-6, rope_theta=1e4, max_position_embeddings=128, tie_word_embeddings=True)
    write_tensors(tmp_path, raw, {})  # config.json first, so that the registry picks the toy configuration
    config = load_config(tmp_path)
    spec = config.model_spec()
    expected = expected_tensors(spec)
    assert "model.layers.0.toy.in_proj.weight" in expected and "model.layers.1.self_attn.q_proj.weight" in expected
    tensors = RandomSource(8, std=0.1).load(expected, "float32", "cpu")
    write_tensors(tmp_path, raw, tensors)
    model, _ = load_model(tmp_path, "float32")
    engine_config = build_engine_config(dtype="float32", page_size=8, kv_tokens=128, max_running=4,
                                        max_model_len=128, prefix_cache_pages=8)
    runner = Runner(model, engine_config)
    assert set(runner.cache.state_units) == {0, 2} and runner.cache.unit_group == {1: 0}
    assert runner.cache.prefix_cache_pages == 0  # state cannot be taken over page by page
    requests = {f"t{i}": random_tokens(n, 64, 70 + i) for i, n in enumerate([23, 40, 9, 31, 17])}
    reference = {rid: toy_plain(raw, tensors, tokens) for rid, tokens in requests.items()}
    for schedule in (replay_util.whole, replay_util.portions, lambda r: replay_util.mixed(r, live=3)):
        steps = schedule(requests)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        replay_util.compare(rows, reference, rtol=1e-4, atol=2e-5)
    # a slot handed to a new request starts from a cleared state (slots were reused above)
    assert runner.cache.stats().slots_used == 0


def _toy_runner(tmp_path, architecture, **options):
    from cie_amd.config import build_engine_config, load_config
    from cie_amd.engine import Runner, load_model
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    register_toy()
    raw = dict(architectures=[architecture], model_type="qwen2", hidden_size=32, num_hidden_layers=2,
               num_attention_heads=2, num_key_value_heads=1, intermediate_size=56, vocab_size=64,
               rms_norm_eps=1e-6, rope_theta=1e4, max_position_embeddings=128, tie_word_embeddings=True)
    write_tensors(tmp_path, raw, {})
    tensors = RandomSource(8, std=0.1).load(expected_tensors(load_config(tmp_path).model_spec()), "float32", "cpu")
    write_tensors(tmp_path, raw, tensors)
    model, _ = load_model(tmp_path, "float32")
    runner = Runner(model, build_engine_config(dtype="float32", page_size=8, kv_tokens=256, max_running=4,
                                               max_model_len=128, prefix_cache_pages=0, **options))
    return raw, tensors, runner


def test_a_stateful_mixer_that_reads_its_slots_on_the_device_runs_from_captured_steps(tmp_path):
    """A mixer with a state per request that declares ``graph_safe`` advances its state at every run of its
    ``forward``.  Captured steps, single tokens and portions alike, are made on rows of padding (the pad slot's
    state), so a request's state moves once per token: at the replay.  Every replay against the plain toy."""
    raw, tensors, runner = _toy_runner(tmp_path, "ToyRunningSumOnDeviceForCausalLM", graph_decode=True,
                                       graph_mixed_steps=8)
    assert runner.graphs is not None and runner.mixed_graphs is not None
    requests = {f"t{i}": random_tokens(n, 64, 70 + i) for i, n in enumerate([61, 40, 53, 31, 47])}
    reference = {rid: toy_plain(raw, tensors, tokens) for rid, tokens in requests.items()}
    for schedule in (lambda r: replay_util.fixed_portions(r, portion=8, live=3, decode_tail=12),
                     lambda r: replay_util.mixed(r, live=4, decode_tail=20, seed=3)):
        steps = schedule(requests)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        replay_util.compare(rows, reference, every_position=False, rtol=1e-4, atol=2e-5)
    assert runner.graph_replays >= 10 and runner.mixed_graph_captures >= 1 and runner.mixed_graph_replays >= 3
    assert runner.cache.stats().slots_used == 0


def test_a_mixer_with_two_states_of_different_shape(tmp_path):
    """``cache_need`` may be a tuple: the mixer is handed a tuple of views in the same order, each state has its
    own shape and type, both are cleared when a slot goes to a new request."""
    raw, tensors, runner = _toy_runner(tmp_path, "ToyTwoStatesForCausalLM", graph_decode=False)
    cache = runner.cache
    assert cache.unit_cells == [(0, 1), 2, (3, 4)] and set(cache.state_units) == {0, 1, 3, 4} and cache.unit_group == {2: 0}
    window, count = runner.device_cache.view(0)
    assert window.state.shape[1:] == (2, 32) and count.state.dtype == torch.int32
    requests = {f"t{i}": random_tokens(n, 64, 170 + i) for i, n in enumerate([23, 40, 9, 31, 17, 50])}
    reference = {rid: toy_plain(raw, tensors, tokens, two_states=True) for rid, tokens in requests.items()}
    for schedule in (replay_util.whole, replay_util.portions, lambda r: replay_util.mixed(r, live=3)):
        steps = schedule(requests)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        replay_util.compare(rows, reference, rtol=1e-4, atol=2e-5)
    assert runner.cache.stats().slots_used == 0


def test_a_model_of_fixed_states_only_runs_its_requests_side_by_side(tmp_path):
    """No unit of this model is paged: the pool has nothing to say about admission, and four requests
    run in the same steps under ``admit_within_pool``, each to the plain toy model's greedy tokens."""
    from cie_amd import Engine, GenerationConfig
    from cie_amd.config import load_config
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    register_toy()
    raw = dict(architectures=["ToyOnlyStateForCausalLM"], model_type="qwen2", hidden_size=32, num_hidden_layers=1,
               num_attention_heads=2, num_key_value_heads=1, intermediate_size=40, vocab_size=64,
               rms_norm_eps=1e-6, rope_theta=1e4, max_position_embeddings=128, tie_word_embeddings=True)
    write_tensors(tmp_path, raw, {})
    tensors = RandomSource(12, std=0.15).load(expected_tensors(load_config(tmp_path).model_spec()), "float32", "cpu")
    write_tensors(tmp_path, raw, tensors)
    engine = Engine(tmp_path, dtype="float32", page_size=8, kv_tokens=8, max_running=4, max_model_len=128,
                    token_budget=64, prefill_chunk=16, admit_within_pool=True)
    assert not engine.runner.cache.groups and set(engine.runner.cache.state_units) == {0, 1}
    prompts = [random_tokens(n, 64, 80 + n) for n in (5, 12, 21, 9)]
    results = engine.generate(prompts, GenerationConfig(max_output_tokens=6, eos_token_id=None))
    assert engine.snapshot_metrics()["runner"]["max_forward_request_count"] == 4
    for prompt, result in zip(prompts, results):
        tokens, expected = list(prompt), []
        for _ in range(6):
            expected.append(int(toy_plain(raw, tensors, tokens, order=(0, 0))[-1].argmax()))
            tokens.append(expected[-1])
        assert result.token_ids == expected
    assert engine.runner.cache.stats().slots_used == 0


# ----------------------------------------------------------------------------------------------------
# A second toy architecture, again defined here and registered from outside the package: a feed-forward
# with a router and experts, a position encoding of its own, and a windowed attention layer beside a
# full one (two cache groups with pages of their own).  It is no model of anyone's.
def register_routed_toy():
    from cie_amd.config import register_architecture
    from cie_amd.config.qwen2 import Qwen2Config
    from cie_amd.config.specs import LayerCall, LayerSpec, ModelSpec, PartSpec
    from cie_amd.parts.base import Part, register_part
    from cie_amd.parts.position import RotaryHalf
    from cie_amd.weights.tensors import TensorSpec

    class RoutedExperts(Part):
        """Top-1 of E small gated experts per token; router logits and softmax in float32; the
        chosen expert's output is scaled by its probability."""

        def __init__(self, hidden_size: int, expert_size: int, experts: int) -> None:
            self.hidden_size, self.expert_size, self.experts = hidden_size, expert_size, experts

        def expected_tensors(self, prefix):
            out = {prefix + "router.weight": TensorSpec((self.experts, self.hidden_size))}
            for e in range(self.experts):
                out[f"{prefix}experts.{e}.gate_up.weight"] = TensorSpec((2 * self.expert_size, self.hidden_size))
                out[f"{prefix}experts.{e}.down.weight"] = TensorSpec((self.hidden_size, self.expert_size))
            return out

        def bind(self, tensors, prefix, dtype, device):
            super().bind(tensors, prefix, dtype, device)
            self.router = tensors[prefix + "router.weight"].float()
            self.gate_up = [tensors[f"{prefix}experts.{e}.gate_up.weight"] for e in range(self.experts)]
            self.down = [tensors[f"{prefix}experts.{e}.down.weight"] for e in range(self.experts)]

        def forward(self, x, residual=None):
            from cie_amd.parts.linear import linear

            probabilities = torch.softmax(x.float() @ self.router.t(), dim=-1)
            weight, chosen = probabilities.max(dim=-1)
            out = torch.zeros((x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
            for e in range(self.experts):
                rows = (chosen == e).nonzero().flatten()
                if rows.numel():
                    hidden = linear(x[rows].contiguous(), self.gate_up[e], epilogue="silu")
                    out[rows] = linear(hidden, self.down[e]).float() * weight[rows, None]
            return out.to(x.dtype)

    class SlowRotary(RotaryHalf):
        """Rotary encoding whose positions advance by 1/factor per token."""

        def __init__(self, head_dim: int, theta: float, max_position: int, factor: float) -> None:
            super().__init__(head_dim=head_dim, theta=theta, max_position=max_position)
            self.factor = factor

        def tables(self, device):
            inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim))
            angles = (torch.arange(self.max_position, dtype=torch.float32) / self.factor)[:, None] * inv_freq[None, :]
            return angles.cos().to(device).contiguous(), angles.sin().to(device).contiguous()

    class RoutedToyConfig(Qwen2Config):
        architecture = "ToyRoutedWindowForCausalLM"
        WINDOW, FACTOR, EXPERTS, EXPERT_SIZE = 20, 4.0, 3, 24

        def model_spec(self) -> ModelSpec:
            base = super().model_spec()
            plain_layer = base.layers[0]
            slow = PartSpec.of("slow_rotary", head_dim=self.head_dim, theta=self.rope_theta,
                               max_position=self.max_position_embeddings, factor=self.FACTOR)
            windowed = PartSpec.of("attention", **{**dict(plain_layer.mixer.params), "window": self.WINDOW})
            slowed = PartSpec.of("attention", **{**dict(plain_layer.mixer.params), "position": slow})
            routed = PartSpec.of("routed_experts", hidden_size=self.hidden_size, expert_size=self.EXPERT_SIZE,
                                 experts=self.EXPERTS)
            first = LayerSpec(mixer=windowed, feed_forward=routed, norm1=plain_layer.norm1, norm2=plain_layer.norm2,
                              names=(("norm1", "input_layernorm"), ("mixer", "self_attn"),
                                     ("norm2", "post_attention_layernorm"), ("feed_forward", "moe")))
            second = LayerSpec(mixer=slowed, feed_forward=plain_layer.feed_forward, norm1=plain_layer.norm1,
                               norm2=plain_layer.norm2, names=plain_layer.names)
            return ModelSpec(
                architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                layers=(first, second), order=(LayerCall(0, 0), LayerCall(1, 1)),
                final_norm=base.final_norm, tie_word_embeddings=True, max_position=self.max_position_embeddings)

    register_part("feed_forward", "routed_experts", RoutedExperts)
    register_part("position", "slow_rotary", SlowRotary)
    register_architecture("ToyRoutedWindowForCausalLM", RoutedToyConfig)
    return RoutedToyConfig


def routed_toy_plain(raw, weights, tokens, config_class):
    """Whole-sequence reference of the second toy model, from the plain parts."""
    eps, d = raw["rms_norm_eps"], plain.head_dim_of(raw)
    t = len(tokens)
    h = weights["model.embed_tokens.weight"][torch.tensor(tokens)]
    positions = torch.arange(t)
    cos, sin = plain.rope_tables(d, t, raw["rope_theta"])
    inv_freq = 1.0 / (raw["rope_theta"] ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    slow_angles = (positions.float() / config_class.FACTOR)[:, None] * inv_freq[None, :]
    slow_cos, slow_sin = torch.cat([slow_angles.cos()] * 2, dim=-1), torch.cat([slow_angles.sin()] * 2, dim=-1)

    def attention(x, p, cos_t, sin_t, window):
        def proj(name):
            return plain.linear(x, weights[f"{p}{name}.weight"], weights[f"{p}{name}.bias"]).view(t, -1, d)
        q, k, v = proj("q_proj"), proj("k_proj"), proj("v_proj")
        q, k = plain.apply_rope(q, cos_t, sin_t, positions), plain.apply_rope(k, cos_t, sin_t, positions)
        context = plain.causal_attention(q, k, v, 1.0 / math.sqrt(d), past_len=0, window=window)
        return plain.linear(context, weights[p + "o_proj.weight"])

    def routed(x, p):
        probabilities = torch.softmax(x @ weights[p + "router.weight"].t(), dim=-1)
        weight, chosen = probabilities.max(dim=-1)
        out = torch.zeros_like(x)
        for row in range(t):
            e = int(chosen[row])
            gate_up = weights[f"{p}experts.{e}.gate_up.weight"]
            half = gate_up.shape[0] // 2
            out[row] = plain.swiglu(x[row:row + 1], gate_up[:half], gate_up[half:], weights[f"{p}experts.{e}.down.weight"])[0] * weight[row]
        return out

    p = "model.layers.0."
    h = h + attention(plain.rms_norm(h, weights[p + "input_layernorm.weight"], eps), p + "self_attn.", cos, sin,
                      config_class.WINDOW)
    h = h + routed(plain.rms_norm(h, weights[p + "post_attention_layernorm.weight"], eps), p + "moe.")
    p = "model.layers.1."
    h = h + attention(plain.rms_norm(h, weights[p + "input_layernorm.weight"], eps), p + "self_attn.", slow_cos[:, :d],
                      slow_sin[:, :d], None)
    h = h + plain.swiglu(plain.rms_norm(h, weights[p + "post_attention_layernorm.weight"], eps),
                         weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                         weights[p + "mlp.down_proj.weight"])
    h = plain.rms_norm(h, weights["model.norm.weight"], eps)
    return h @ weights["model.embed_tokens.weight"].t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_own_position_encoding_and_window_layer(tmp_path, dtype):
    """Registered from here: a feed-forward with a router, a position encoding of its own, and a layer
    whose attention sees a window only.  The windowed layer's cache is a group of its own: its pages
    come back as the window passes them, while the full layer keeps all of its pages."""
    from cie_amd.config import build_engine_config, load_config
    from cie_amd.engine import Runner, load_model
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    config_class = register_routed_toy()
    # bfloat16 could choose another expert than float32 where two router logits nearly tie, and everything
    # after would differ: there the toy runs a single expert (probability 1: the router changes nothing)
    config_class.EXPERTS = 3 if dtype == "float32" else 1
    raw = dict(architectures=["ToyRoutedWindowForCausalLM"], model_type="qwen2", hidden_size=64, num_hidden_layers=2,
               num_attention_heads=4, num_key_value_heads=2, head_dim=32, intermediate_size=72, vocab_size=80,
               rms_norm_eps=1e-5, rope_theta=1e4, max_position_embeddings=160, tie_word_embeddings=True)
    write_tensors(tmp_path, raw, {})
    config = load_config(tmp_path)
    expected = expected_tensors(config.model_spec())
    last_expert = config_class.EXPERTS - 1
    assert f"model.layers.0.moe.experts.{last_expert}.down.weight" in expected
    assert "model.layers.1.mlp.down_proj.weight" in expected
    tensors = RandomSource(9, std=0.15).load(expected, "float32", "cpu")
    if dtype == "bfloat16":  # the plain model runs the weights the engine holds
        tensors = {k: (v.to(torch.bfloat16).float() if v.is_floating_point() else v) for k, v in tensors.items()}
    write_tensors(tmp_path, raw, tensors)
    model, _ = load_model(tmp_path, dtype)
    engine_config = build_engine_config(dtype=dtype, page_size=8, kv_tokens=512, max_running=4, max_model_len=160,
                                        prefix_cache_pages=0, graph_decode=False)
    runner = Runner(model, engine_config)
    groups = runner.cache.groups
    assert len(groups) == 2 and {g.spec.window for g in groups} == {config_class.WINDOW, None}
    requests = {f"r{i}": random_tokens(n, 80, 90 + i) for i, n in enumerate([70, 33, 9, 120, 41])}
    reference = {rid: routed_toy_plain(raw, tensors, tokens, config_class) for rid, tokens in requests.items()}
    # bfloat16 rounds every activation to 8 bits of a row's magnitude: the absolute part of the tolerance is
    # the replay tests' 2e-2 per unit of logit magnitude (these weights are larger than theirs: logits of +-3)
    magnitude = max(1.0, max(float(r.abs().max()) for r in reference.values()))
    tolerance = dict(rtol=1e-4, atol=2e-5) if dtype == "float32" else dict(rtol=2e-2, atol=2e-2 * magnitude)
    for schedule in (replay_util.whole, replay_util.portions, lambda r: replay_util.mixed(r, live=3)):
        steps = schedule(requests)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        replay_util.compare(rows, reference, **tolerance)
        assert runner.cache.stats().pages_used == 0
    # while a long request is alive, the windowed group holds a few pages, the full group all of them
    runner.cache.admit("long")
    from cie_amd.engine.runner import StepEntry
    tokens = requests["r3"]
    for start in range(0, 120, 24):
        runner.run([StepEntry("long", tokens[start:start + 24], start, [])])
    windowed = next(g for g in groups if g.spec.window is not None)
    full = next(g for g in groups if g.spec.window is None)
    held = lambda g: sum(1 for page in g.tables["long"] if page >= 0)  # noqa: E731
    assert held(full) == 15 and held(windowed) <= -(-config_class.WINDOW // 8) + 1
    runner.cache.release("long")
    runner.cache.assert_invariants()


@pytest.mark.parametrize("seed", [201, 202, 203, 204])
def test_toy_window_layer_under_random_traces(tmp_path, seed):
    """The toy model with a windowed layer (a cache group of its own whose pages come back as the window passes),
    routed experts and its own position encoding under traces drawn at random, in float32: windows from 5 to 64
    keys against pages of 4 to 16, cuts anywhere, a pool of exactly the live requests' pages."""
    import random

    from cie_amd.config import build_engine_config, load_config
    from cie_amd.engine import Runner, load_model
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    rng = random.Random(seed)
    config_class = register_routed_toy()
    config_class.EXPERTS = 3
    config_class.WINDOW = rng.choice([5, 8, 16, 20, 33, 64])
    kv_heads = rng.choice([1, 2])
    raw = dict(architectures=["ToyRoutedWindowForCausalLM"], model_type="qwen2", hidden_size=64, num_hidden_layers=2,
               num_attention_heads=kv_heads * rng.choice([1, 2, 4]), num_key_value_heads=kv_heads,
               head_dim=rng.choice([16, 32, 64]), intermediate_size=72, vocab_size=80, rms_norm_eps=1e-5, rope_theta=1e4,
               max_position_embeddings=rng.choice([96, 160, 300]), tie_word_embeddings=True)
    try:
        write_tensors(tmp_path, raw, {})
        tensors = RandomSource(seed, std=0.15).load(expected_tensors(load_config(tmp_path).model_spec()), "float32", "cpu")
        write_tensors(tmp_path, raw, tensors)
        model, _ = load_model(tmp_path, "float32")
        page = rng.choice([4, 8, 16])
        lengths = [rng.randint(1, raw["max_position_embeddings"]) for _ in range(rng.randint(2, 5))]
        requests, steps = replay_util.random_trace(rng, lengths, raw["vocab_size"], page)
        print(f"window {config_class.WINDOW}, page {page}, lengths {lengths}, {len(steps)} steps", flush=True)
        longest_portion = max(len(entry["tokens"]) for step in steps for entry in step["entries"])
        engine_config = build_engine_config(
            dtype="float32", page_size=page, kv_tokens=replay_util.max_live_tokens(steps, page=page), max_running=4,
            max_model_len=raw["max_position_embeddings"], prefix_cache_pages=0, graph_decode=rng.random() < 0.5,
            prefill_chunk=longest_portion)
        runner = Runner(model, engine_config)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        weights = {k: v.float() for k, v in tensors.items()}
        expected = {rid: routed_toy_plain(raw, weights, requests[rid], config_class) for rid in rows}
        replay_util.compare(rows, expected, every_position=False, rtol=1e-4, atol=5e-5)
        assert runner.cache.stats().pages_used == 0
    finally:
        config_class.WINDOW = 20


def _window_case(raw, tensors, config_class, rng, length):
    """Plant one channel in the windowed layer (its slowest rotating pair): token ``ask`` scores 22 on token
    ``key`` and little on any other.  The request has keys at the very edge of the window of an asking token
    (just inside: the furthest key it may see; just outside: the nearest it may not), so that a window cut
    one key off moves that row's logits by most of the attention's share."""
    d, hidden, window = plain.head_dim_of(raw), raw["hidden_size"], config_class.WINDOW
    key, ask = raw["vocab_size"] - 1, raw["vocab_size"] - 2
    p = "model.layers.0.self_attn."
    low, high = d // 2 - 1, d - 1
    heads = raw["num_attention_heads"]
    for name, bases, column in (("k_proj", [0], 0), ("q_proj", [h * d for h in range(heads)], 1)):
        for base in bases:
            for row in (base + low, base + high):
                tensors[p + name + ".weight"][row] = 0.0
                tensors[p + name + ".bias"][row] = 0.0
            tensors[p + name + ".weight"][base + high, column] = 2.0
    embed = tensors["model.embed_tokens.weight"]
    embed[key] = 0.0
    embed[key, 0] = embed[key, 5] = 0.1
    embed[ask] *= 0.1
    embed[ask, 1] = 0.1
    tokens = [rng.randrange(raw["vocab_size"] - 2) for _ in range(length)]
    asking = []
    place = rng.randint(0, 5)
    inside = True
    while place + window < length:
        tokens[place] = key
        query = place + window - 1 if inside else place + window
        tokens[query] = ask
        asking.append((query, inside))
        inside = not inside
        place = query + rng.randint(1, 9)
    return tokens, asking


@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("page,window,head_dim", [(16, 37, 64), (64, 70, 64), (16, 100, 128), (64, 45, 128)])
def test_toy_window_layer_in_bfloat16_with_pages_of_16_and_64(tmp_path, monkeypatch, page, window, head_dim, graph):
    """The windowed layer in bfloat16 with pages that send it to the matrix-core forms of four and eight waves,
    joined decode rows and captured decode steps, while the pages that the window has passed go back to the pool
    and are handed out again (the device's block table keeps their numbers): windows that are no multiples of
    the kernels' blocks of 32 keys, a dominating key just inside the window and just outside it."""
    import random

    from cie_amd.config import build_engine_config, load_config
    from cie_amd.engine import Runner, load_model
    from cie_amd.parts import attention
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    rng = random.Random(1000 * page + window)
    config_class = register_routed_toy()
    config_class.EXPERTS, config_class.WINDOW = 1, window
    monkeypatch.setattr(attention, "EIGHT_WAVE_TILES", 0)  # heads of 128: every prompt portion in tiles of eight waves
    raw = dict(architectures=["ToyRoutedWindowForCausalLM"], model_type="qwen2", hidden_size=64, num_hidden_layers=2,
               num_attention_heads=2, num_key_value_heads=1, head_dim=head_dim, intermediate_size=72, vocab_size=80,
               rms_norm_eps=1e-5, rope_theta=1e4, max_position_embeddings=600, tie_word_embeddings=True)
    try:
        write_tensors(tmp_path, raw, {})
        tensors = RandomSource(window, std=0.15).load(expected_tensors(load_config(tmp_path).model_spec()), "float32", "cpu")
        long_tokens, asking = _window_case(raw, tensors, config_class, rng, 560)
        tensors = {k: (v.to(torch.bfloat16).float() if v.is_floating_point() else v) for k, v in tensors.items()}
        write_tensors(tmp_path, raw, tensors)
        lengths = [560, rng.randint(150, 400), rng.randint(20, 120), rng.randint(150, 300)]
        requests, steps = replay_util.random_trace(rng, lengths, raw["vocab_size"] - 2, page)
        requests["r0"][:] = long_tokens
        at: dict[str, int] = {}
        for step in steps:  # the cuts stay, the long request's tokens are the planted ones, every position is wanted
            for entry in step["entries"]:
                first = at.get(entry["id"], 0)
                entry["tokens"] = requests[entry["id"]][first: first + len(entry["tokens"])]
                entry["want"] = list(range(len(entry["tokens"])))
                at[entry["id"]] = first + len(entry["tokens"])
        longest_portion = max(len(entry["tokens"]) for step in steps for entry in step["entries"])
        model, _ = load_model(tmp_path, "bfloat16")
        runner = Runner(model, build_engine_config(
            dtype="bfloat16", page_size=page, kv_tokens=replay_util.max_live_tokens(steps, page=page), max_running=4,
            max_model_len=raw["max_position_embeddings"], prefix_cache_pages=0, graph_decode=graph,
            prefill_chunk=longest_portion))
        windowed = next(g for g in runner.cache.groups if g.spec.window is not None)
        passed, reused = set(), []  # pages the window has passed while their request lives, and those handed out again
        free, allocate = windowed.allocator.free, windowed.allocator.allocate

        def spy_free(pages, owner):
            if runner.cache.has(owner):
                passed.update(pages)
            return free(pages, owner)

        def spy_allocate(owner, count):
            pages = allocate(owner, count)
            reused.extend(page for page in pages if page in passed)
            return pages

        monkeypatch.setattr(windowed.allocator, "free", spy_free)
        monkeypatch.setattr(windowed.allocator, "allocate", spy_allocate)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        assert reused, "no page that the window had passed was handed out again"
        expected = {rid: routed_toy_plain(raw, tensors, tokens, config_class) for rid, tokens in requests.items()}
        rough = {rid: routed_toy_plain(raw, {k: v.to(torch.bfloat16) for k, v in tensors.items()}, tokens, config_class).float()
                 for rid, tokens in requests.items()}
        rms, worst, plain_rms, plain_worst = replay_util.closer_than_plain_bfloat16(rows, expected, rough)
        print(f"window {window} page {page}: rms {rms:.3e} worst {worst:.3e}, plain in bfloat16 {plain_rms:.3e} {plain_worst:.3e}",
              flush=True)
        # the yardstick: a window one key longer or shorter moves the asking rows by far more than that
        for wrong in (window + 1, window - 1):
            config_class.WINDOW = wrong
            off = routed_toy_plain(raw, tensors, long_tokens, config_class)
            moved = [float((off[q] - expected["r0"][q]).abs().max()) for q, inside in asking if inside == (wrong < window)]
            assert moved and min(moved) > 4 * 1.5 * plain_worst, (wrong, min(moved), plain_worst)
        assert runner.cache.stats().pages_used == 0
    finally:
        config_class.WINDOW, config_class.EXPERTS = 20, 3


# ----------------------------------------------------------------------------------------------------
# The run order is data: a layer may read the cache that another layer writes.  Again a toy,
# registered from here: three attention layers, the middle one without keys and values of its own.
def register_shared_cache_toy():
    from cie_amd.config import register_architecture
    from cie_amd.config.qwen2 import Qwen2Config
    from cie_amd.config.specs import LayerCall, ModelSpec

    class SharedCacheConfig(Qwen2Config):
        architecture = "ToySharedCacheForCausalLM"

        def model_spec(self) -> ModelSpec:
            base = super().model_spec()
            # layer 1 attends, with its own queries, to the keys and values that layer 0 wrote
            order = (LayerCall(0, 0), LayerCall(1, 0, writes=False), LayerCall(2, 1))
            return ModelSpec(
                architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                layers=base.layers, order=order, final_norm=base.final_norm,
                tie_word_embeddings=self.tie_word_embeddings, max_position=self.max_position_embeddings)

    register_architecture("ToySharedCacheForCausalLM", SharedCacheConfig)
    return SharedCacheConfig


def shared_cache_plain(raw, weights, tokens):
    """Whole-sequence reference from the plain parts: layer 1 uses layer 0's rotated keys and its values."""
    eps, d = raw["rms_norm_eps"], plain.head_dim_of(raw)
    t = len(tokens)
    positions = torch.arange(t)
    cos, sin = plain.rope_tables(d, t, raw["rope_theta"])
    h = weights["model.embed_tokens.weight"][torch.tensor(tokens)]
    kept = None
    for layer in range(3):
        p = f"model.layers.{layer}."
        x = plain.rms_norm(h, weights[p + "input_layernorm.weight"], eps)

        def proj(name):
            return plain.linear(x, weights[f"{p}self_attn.{name}.weight"], weights[f"{p}self_attn.{name}.bias"]).view(t, -1, d)

        q = plain.apply_rope(proj("q_proj"), cos, sin, positions)
        if layer == 1:
            k, v = kept
        else:
            k, v = plain.apply_rope(proj("k_proj"), cos, sin, positions), proj("v_proj")
        if layer == 0:
            kept = (k, v)
        context = plain.causal_attention(q, k, v, 1.0 / math.sqrt(d), past_len=0)
        h = h + plain.linear(context, weights[p + "self_attn.o_proj.weight"])
        h = h + plain.swiglu(plain.rms_norm(h, weights[p + "post_attention_layernorm.weight"], eps),
                             weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                             weights[p + "mlp.down_proj.weight"])
    h = plain.rms_norm(h, weights["model.norm.weight"], eps)
    return h @ weights["lm_head.weight"].t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_that_reads_the_cache_another_layer_writes(tmp_path, dtype):
    """Three layers on two cache units: the middle layer writes nothing and reads the first layer's pages.
    Whole, in portions and mixed with pages used again, with captured decode steps, against the plain model."""
    from cie_amd.config import build_engine_config, load_config
    from cie_amd.engine import Runner, load_model
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    register_shared_cache_toy()
    raw = dict(architectures=["ToySharedCacheForCausalLM"], model_type="qwen2", hidden_size=80, num_hidden_layers=3,
               num_attention_heads=5, num_key_value_heads=1, head_dim=32, intermediate_size=104, vocab_size=91,
               rms_norm_eps=1e-5, rope_theta=1e4, max_position_embeddings=200, tie_word_embeddings=False)
    write_tensors(tmp_path, raw, {})
    spec = load_config(tmp_path).model_spec()
    assert spec.cache_units == 2
    tensors = RandomSource(12, std=0.12).load(expected_tensors(spec), "float32", "cpu")
    # the middle layer's own key and value projections are loaded and never used: garbage there must not show
    for name in ("k_proj", "v_proj"):
        tensors[f"model.layers.1.self_attn.{name}.weight"] = tensors[f"model.layers.1.self_attn.{name}.weight"] * 50.0
    if dtype == "bfloat16":  # the plain model runs the weights the engine holds
        tensors = {k: (v.to(torch.bfloat16).float() if v.is_floating_point() else v) for k, v in tensors.items()}
    write_tensors(tmp_path, raw, tensors)
    model, _ = load_model(tmp_path, dtype)
    requests = {f"s{i}": random_tokens(n, 91, 300 + i) for i, n in enumerate([150, 37, 64, 9, 101])}
    reference = {rid: shared_cache_plain(raw, tensors, tokens) for rid, tokens in requests.items()}
    magnitude = max(1.0, max(float(r.abs().max()) for r in reference.values()))
    tolerance = dict(rtol=1e-4, atol=5e-5) if dtype == "float32" else dict(rtol=2e-2, atol=2e-2 * magnitude)
    for graphs in (False, True):
        mixed_steps = replay_util.mixed(requests, live=3)
        engine_config = build_engine_config(
            dtype=dtype, page_size=8, kv_tokens=replay_util.max_live_tokens(mixed_steps, page=8), max_running=4,
            max_model_len=200, prefix_cache_pages=0, graph_decode=graphs)
        runner = Runner(model, engine_config)
        assert len(runner.cache.groups) == 1 and sorted(runner.cache.unit_group) == [0, 1]
        for steps in (replay_util.whole(requests), replay_util.tail_one_by_one(requests, tail=32),
                      replay_util.portions(requests), mixed_steps):
            rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
            replay_util.compare(rows, reference, **tolerance)
            assert runner.cache.stats().pages_used == 0
