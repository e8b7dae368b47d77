"""CPU: the plain implementation, pinned by what fixes it beside the reference's
text: special cases that reduce to a library routine, and invariants chosen so
that a plausible mistake (a wrong sign or pairing in the rotation, a norm's
weight in the wrong place, a mask off by one, a wrong head grouping) fails."""

import math

import pytest
import torch

import plain_qwen2 as plain
from conftest import TINY_A, TINY_B, random_tokens, sharpen
from cie_amd.config import config_from_dict
from cie_amd.parts.model import expected_tensors
from cie_amd.weights import RandomSource


def test_rms_norm_is_the_library_routine():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((5, 96), generator=g) * 3
    w = torch.randn((96,), generator=g)
    expect = torch.nn.functional.rms_norm(x, (96,), w, 1e-5)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), expect, rtol=1e-6, atol=1e-6)
    ones = torch.ones(96)
    out = plain.rms_norm(x, ones, 1e-12)
    torch.testing.assert_close(out.pow(2).mean(-1), torch.ones(5), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(plain.rms_norm(x * 9, ones, 1e-12), out, rtol=1e-5, atol=1e-6)
    # eps sits inside the square root, next to the mean of squares
    tiny = torch.full((1, 4), 1e-3)
    torch.testing.assert_close(plain.rms_norm(tiny, torch.ones(4), 1.0), tiny / math.sqrt(1e-6 + 1.0))


def test_rms_norm_rounds_before_the_weight_in_16_bit():
    """reference attention.py:56-57: the normalised value is cast to the model dtype, then multiplied."""
    x = torch.tensor([[1.0, 2.0, 3.0, 4.1]], dtype=torch.bfloat16)
    w = torch.tensor([1.5, 0.3, 1.1, 0.7], dtype=torch.bfloat16)
    xf = x.float()
    normed = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    assert torch.equal(plain.rms_norm(x, w, 1e-6), w * normed)


def test_rope_is_multiplication_by_a_unit_complex_number():
    head_dim, theta = 32, 1e6
    cos, sin = plain.rope_tables(head_dim, 300, theta)
    g = torch.Generator().manual_seed(1)
    x = torch.randn((4, 3, head_dim), generator=g, dtype=torch.float64)
    positions = torch.tensor([0, 1, 77, 299])
    out = plain.apply_rope(x, cos.double(), sin.double(), positions)
    # complex form: (x[:D/2] + i x[D/2:]) * exp(i p inv_freq)
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    angle = positions[:, None].double() * inv_freq[None, :]
    z = torch.complex(x[..., : head_dim // 2], x[..., head_dim // 2:]) * torch.polar(torch.ones_like(angle), angle)[:, None, :]
    expect = torch.cat((z.real, z.imag), dim=-1)
    torch.testing.assert_close(out, expect, rtol=1e-5, atol=1e-5)  # tables are float32
    assert torch.equal(out[0], x[0]), "position 0 is the identity"
    pair_norm = lambda t: t[..., : head_dim // 2] ** 2 + t[..., head_dim // 2:] ** 2  # noqa: E731
    torch.testing.assert_close(pair_norm(out), pair_norm(x), rtol=1e-6, atol=1e-6)


def test_rope_scores_depend_on_distance_only():
    head_dim = 16
    cos, sin = plain.rope_tables(head_dim, 700, 10000.0)
    cos, sin = cos.double(), sin.double()
    g = torch.Generator().manual_seed(2)
    q = torch.randn((1, 1, head_dim), generator=g, dtype=torch.float64)
    k = torch.randn((1, 1, head_dim), generator=g, dtype=torch.float64)

    def score(m, n):
        return (plain.apply_rope(q, cos, sin, torch.tensor([m])) * plain.apply_rope(k, cos, sin, torch.tensor([n]))).sum()

    assert abs(score(10, 3) - score(510, 503)) < 2e-3
    assert abs(score(10, 3) - score(3, 10)) > 1e-2, "the rotation has a direction"
    assert abs(score(10, 3) - score(10, 4)) > 1e-3


def test_rope_table_constants_are_parameters():
    cos_a, _ = plain.rope_tables(16, 8, 10000.0)
    cos_b, _ = plain.rope_tables(16, 8, 1e6)
    assert cos_a.shape == (8, 16) and not torch.allclose(cos_a[5], cos_b[5])
    assert torch.equal(cos_a[:, :8], cos_a[:, 8:]), "the two halves carry the same angles"
    torch.testing.assert_close(cos_a[3, 1], torch.cos(torch.tensor(3.0 / 10000.0 ** (2 / 16))))


@pytest.mark.parametrize("heads,kv_heads,past", [(4, 4, 0), (4, 2, 0), (6, 1, 5), (2, 2, 9)])
def test_attention_is_library_sdpa_with_a_causal_offset_mask(heads, kv_heads, past):
    g = torch.Generator().manual_seed(3)
    tq, d = 7, 16
    tk = past + tq
    q = torch.randn((tq, heads, d), generator=g)
    k = torch.randn((tk, kv_heads, d), generator=g)
    v = torch.randn((tk, kv_heads, d), generator=g)
    scale = 1 / math.sqrt(d)
    group = heads // kv_heads
    mask = (torch.arange(tq)[:, None] + past) >= torch.arange(tk)[None, :]
    expect = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.repeat_interleave(group, 1).transpose(0, 1), v.repeat_interleave(group, 1).transpose(0, 1),
        attn_mask=mask, scale=scale).transpose(0, 1).reshape(tq, heads * d)
    torch.testing.assert_close(plain.causal_attention(q, k, v, scale, past_len=past), expect, rtol=1e-5, atol=1e-5)


def test_attention_special_cases():
    g = torch.Generator().manual_seed(4)
    d = 8
    k = torch.randn((6, 2, d), generator=g)
    v = torch.randn((6, 2, d), generator=g)
    q = torch.randn((1, 4, d), generator=g)
    # one visible key: the output is its value, whatever the query
    out = plain.causal_attention(q, k[:1], v[:1], 0.3)
    torch.testing.assert_close(out.view(4, d), v[0].repeat_interleave(2, 0))
    # zero query: the mean of the visible values; heads 0,1 read KV head 0 and heads 2,3 read KV head 1
    out = plain.causal_attention(torch.zeros((1, 4, d)), k, v, 0.3, past_len=3)
    torch.testing.assert_close(out.view(4, d), v[:4].mean(0).repeat_interleave(2, 0))
    # the window drops keys at distance >= window
    out = plain.causal_attention(torch.zeros((1, 4, d)), k, v, 0.3, past_len=5, window=2)
    torch.testing.assert_close(out.view(4, d), v[4:6].mean(0).repeat_interleave(2, 0))
    # whole = in portions (keys up to the portion's end, offset mask)
    qs = torch.randn((6, 4, d), generator=g)
    whole = plain.causal_attention(qs, k, v, 0.3)
    tail = plain.causal_attention(qs[4:], k, v, 0.3, past_len=4)
    torch.testing.assert_close(whole[4:], tail)


def test_swiglu_and_linear():
    g = torch.Generator().manual_seed(5)
    x = torch.randn((3, 12), generator=g)
    gate, up, down = (torch.randn(s, generator=g) for s in ((20, 12), (20, 12), (12, 20)))
    expect = torch.nn.functional.linear(torch.nn.functional.silu(torch.nn.functional.linear(x, gate))
                                        * torch.nn.functional.linear(x, up), down)
    torch.testing.assert_close(plain.swiglu(x, gate, up, down), expect)
    assert plain.swiglu(x, torch.zeros_like(gate), up, down).abs().max() == 0  # silu(0) = 0
    bias = torch.randn(20, generator=g)
    torch.testing.assert_close(plain.linear(x, gate, bias), torch.nn.functional.linear(x, gate, bias))
    torch.testing.assert_close(plain.linear(x, gate), plain.linear(x, gate, torch.zeros(20)))


def tiny_weights(raw, seed=0):
    expected = expected_tensors(config_from_dict(raw).model_spec())
    return {k: v.float() for k, v in sharpen(RandomSource(seed).load(expected, "bfloat16", "cpu")).items()}


def test_forward_is_causal_and_uses_the_right_head():
    for raw in (TINY_A, TINY_B):
        weights = tiny_weights(raw)
        tokens = random_tokens(24, raw["vocab_size"], 6)
        logits = plain.forward(raw, weights, tokens)
        assert logits.shape == (24, raw["vocab_size"]) and logits.dtype == torch.float32
        shorter = plain.forward(raw, weights, tokens[:10])
        torch.testing.assert_close(logits[:10], shorter, rtol=1e-5, atol=1e-6)  # later tokens change nothing earlier
        changed = plain.forward(raw, weights, [(tokens[0] + 1) % raw["vocab_size"]] + tokens[1:])
        assert (changed[-1] - logits[-1]).abs().max() > 1e-4  # the first token reaches the last position
    untied = tiny_weights(TINY_B)
    swapped = dict(untied, **{"lm_head.weight": untied["lm_head.weight"].flip(0)})
    base, flipped = plain.forward(TINY_B, untied, [1, 2, 3]), plain.forward(TINY_B, swapped, [1, 2, 3])
    torch.testing.assert_close(base.flip(1), flipped)  # the untied head is the tensor that is used
    tied = tiny_weights(TINY_A)
    final = plain.rms_norm(torch.ones(1, 64), tied["model.norm.weight"], 1e-6)
    assert plain.forward(TINY_A, tied, [5]).shape == (1, 256) and final.shape == (1, 64)


def test_queries_in_chunks_and_selected_rows_change_nothing():
    """Long sequences are attended a chunk of queries at a time, and only the wanted rows pass the head:
    the same logits as the whole square, at a chunk that divides the length and one that does not."""
    for raw in (TINY_A, TINY_B):
        weights = tiny_weights(raw)
        tokens = random_tokens(60, raw["vocab_size"], 8)
        whole = plain.forward(raw, weights, tokens)
        for chunk in (20, 7, 1):
            torch.testing.assert_close(plain.forward(raw, weights, tokens, query_chunk=chunk), whole, rtol=1e-5, atol=1e-6)
        rows = [0, 13, 59]
        torch.testing.assert_close(plain.forward(raw, weights, tokens, query_chunk=16, rows=rows), whole[rows],
                                   rtol=1e-5, atol=1e-6)


def test_forward_bias_matters_and_softmax_weights_sum_to_one():
    weights = tiny_weights(TINY_A)
    tokens = random_tokens(12, 256, 7)
    base = plain.forward(TINY_A, weights, tokens)
    no_bias = plain.forward(dict(TINY_A, attention_bias=False), weights, tokens)
    assert (base - no_bias).abs().max() > 1e-4
    zero_bias = {k: (torch.zeros_like(v) if k.endswith("proj.bias") else v) for k, v in weights.items()}
    torch.testing.assert_close(plain.forward(TINY_A, zero_bias, tokens), no_bias)
    # a sequence of one repeated token has identical values everywhere: attention returns that value at
    # every position, so every row of logits is the same (softmax weights sum to one)
    repeated = plain.forward(TINY_A, weights, [7] * 6)
    torch.testing.assert_close(repeated[1], repeated[5], rtol=1e-5, atol=1e-6)


def test_greedy_generation_is_argmax_of_the_last_row():
    weights = tiny_weights(TINY_A)
    prompt = [3, 1, 4, 1, 5]
    out = plain.generate_greedy(TINY_A, weights, prompt, 3)
    assert out[0] == int(plain.forward(TINY_A, weights, prompt)[-1].argmax())
    assert out[1] == int(plain.forward(TINY_A, weights, prompt + out[:1])[-1].argmax())


# -- the composition: what is multiplied, normalised, added and tied where --------------------------------
# The reference checks its model against a library implementation on a rented GPU
# (tests/remote_gpu_tests.py:99-119).  The model code of installed packages is no source for this
# repository, so the composition is pinned by what the reference's text implies and a library routine
# or an invariant can check: each test below fails for one plausible misreading of
# src/cloud_engine/model.py:194-228 and attention.py:129-147.
def library_forward(raw, weights, tokens):
    """The same model put together from library routines only, in another structure: torch.nn modules,
    ``scaled_dot_product_attention`` with its own default scale (1 / sqrt(head size)) and its own causal
    mask, ``rms_norm``, ``silu``, the rotation as a complex product."""
    import torch.nn.functional as F

    d = plain.head_dim_of(raw)
    heads, kv_heads = raw["num_attention_heads"], raw["num_key_value_heads"]
    t = len(tokens)
    eps = raw["rms_norm_eps"]
    bias = raw.get("attention_bias", True)
    embed = torch.nn.Embedding.from_pretrained(weights["model.embed_tokens.weight"].double())
    inv_freq = 1.0 / (raw.get("rope_theta", 10000.0) ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    turn = torch.polar(torch.ones(t, d // 2, dtype=torch.float64),
                       (torch.arange(t, dtype=torch.float32)[:, None] * inv_freq[None, :]).double())

    def module(name, with_bias=False):
        weight = weights[name + ".weight"].double()
        layer = torch.nn.Linear(weight.shape[1], weight.shape[0], bias=with_bias, dtype=torch.float64)
        layer.weight.data.copy_(weight)
        if with_bias:
            layer.bias.data.copy_(weights[name + ".bias"].double())
        return layer

    def rotate(x):  # [T, heads, D]: element i pairs with element i + D/2
        z = torch.complex(x[..., : d // 2], x[..., d // 2:]) * turn[:, None, :]
        return torch.cat((z.real, z.imag), dim=-1)

    with torch.no_grad():
        stream = embed(torch.tensor(tokens))
        for i in range(raw["num_hidden_layers"]):
            p = f"model.layers.{i}."
            x = F.rms_norm(stream, (stream.shape[-1],), weights[p + "input_layernorm.weight"].double(), eps)
            q = rotate(module(p + "self_attn.q_proj", bias)(x).view(t, heads, d)).transpose(0, 1)
            k = rotate(module(p + "self_attn.k_proj", bias)(x).view(t, kv_heads, d)).transpose(0, 1)
            v = module(p + "self_attn.v_proj", bias)(x).view(t, kv_heads, d).transpose(0, 1)
            mixed = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            stream = stream + module(p + "self_attn.o_proj")(mixed.transpose(0, 1).reshape(t, heads * d))
            x = F.rms_norm(stream, (stream.shape[-1],), weights[p + "post_attention_layernorm.weight"].double(), eps)
            gated = F.silu(module(p + "mlp.gate_proj")(x)) * module(p + "mlp.up_proj")(x)
            stream = stream + module(p + "mlp.down_proj")(gated)
        x = F.rms_norm(stream, (stream.shape[-1],), weights["model.norm.weight"].double(), eps)
        head = "model.embed_tokens" if raw.get("tie_word_embeddings", False) else "lm_head"
        return module(head)(x)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_forward_is_the_composition_of_library_routines(name):
    """Forty tokens through all three tiny configurations with randomised norms and biases and sharpened
    queries and keys: the plain forward against the library composition in float64.  Pins the score scale
    (the library's default 1 / sqrt(D)), grouped heads (``enable_gqa``: query head h reads key head
    h // group), the causal mask, bias use, the rotation's pairing and the tied or untied head."""
    from conftest import TINY

    raw = TINY[name]
    weights = tiny_weights(raw, seed=21)
    g = torch.Generator().manual_seed(5)
    for key in weights:  # norms far from one, biases far from zero: a norm or bias left out shows
        if "layernorm" in key or key == "model.norm.weight":
            weights[key] = 0.5 + torch.rand(weights[key].shape, generator=g)
        elif key.endswith(".bias"):
            weights[key] = weights[key] + 0.3 * torch.randn(weights[key].shape, generator=g)
    tokens = random_tokens(40, raw["vocab_size"], 9)
    ours = plain.forward(raw, weights, tokens)
    expect = library_forward(raw, weights, tokens)
    assert (ours.double() - expect).abs().max() <= 1e-5 * max(1.0, float(expect.abs().max()))
    # the plain forward with float64 layers comes closer still (what is left are its float32 cosine and sine
    # tables, which the reference keeps in float32 too): float32 sums are not what hides a difference
    exact = plain.forward(raw, weights, tokens, dtype=torch.float64)
    assert (exact.double() - expect).abs().max() <= 1e-6 * max(1.0, float(expect.abs().max()))


def test_the_residual_stream_passes_the_layers_unnormalised():
    """Pre-norm arrangement (src/cloud_engine/model.py:211-220: ``hidden = residual + branch(norm(hidden))``):
    with both output projections at zero every branch adds nothing, and the logits are the head of the
    final norm of the bare embedding.  A norm applied to the stream itself (post-norm) would show."""
    weights = tiny_weights(TINY_B, seed=3)
    g = torch.Generator().manual_seed(6)
    for key in weights:
        if "layernorm" in key or key == "model.norm.weight":
            weights[key] = 0.5 + torch.rand(weights[key].shape, generator=g)
        if key.endswith(("o_proj.weight", "down_proj.weight")):
            weights[key] = torch.zeros_like(weights[key])
    tokens = random_tokens(9, TINY_B["vocab_size"], 10)
    bare = weights["model.embed_tokens.weight"][torch.tensor(tokens)]
    expect = plain.rms_norm(bare, weights["model.norm.weight"], TINY_B["rms_norm_eps"]) @ weights["lm_head.weight"].t()
    torch.testing.assert_close(plain.forward(TINY_B, weights, tokens), expect, rtol=1e-5, atol=1e-6)


def test_each_branch_reads_the_normalised_stream_and_adds_to_the_raw_one():
    """With the embedding scaled by c, every branch sees the same normalised input (eps is tiny beside the
    rows' mean squares), so the stream after the layers is c x embedding + the same branch sums:
    logits(c) - logits(1) follows from the embedding alone only under the final norm; what can be
    checked exactly is one layer with the feed-forward off: stream = c e + attn(norm(e))."""
    raw = dict(TINY_A, num_hidden_layers=1, rms_norm_eps=1e-12)
    weights = tiny_weights(raw, seed=4)
    weights["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(weights["model.layers.0.mlp.down_proj.weight"])
    tokens = random_tokens(7, raw["vocab_size"], 11)
    ids = torch.tensor(tokens)
    e = weights["model.embed_tokens.weight"][ids]
    cos, sin = plain.rope_tables(16, 7, raw["rope_theta"])
    branch = plain.attention_layer(plain.rms_norm(e, weights["model.layers.0.input_layernorm.weight"], 1e-12), weights,
                                   "model.layers.0.self_attn.", raw, cos, sin, torch.arange(7))
    for c in (1.0, 3.0):
        scaled = dict(weights, **{"model.embed_tokens.weight": weights["model.embed_tokens.weight"] * c})
        # the tied head scales with the embedding: divide it out again
        got = plain.forward(raw, scaled, tokens) / c
        expect = plain.rms_norm(c * e + branch, weights["model.norm.weight"], 1e-12) @ weights["model.embed_tokens.weight"].t()
        torch.testing.assert_close(got, expect, rtol=1e-4, atol=1e-6)
