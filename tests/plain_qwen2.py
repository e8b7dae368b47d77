"""Plain, slow implementation of the Qwen2.5 dense decoder for the tests.

Whole sequences, no cache, one function per part, torch on the CPU, float32
unless told otherwise.  Written from the formulas of the reference (each
function cites where it reads them); it shares no code with ``cie_amd``: it
takes the raw ``config.json`` dictionary and a dictionary of tensors under
their checkpoint names.
"""

from __future__ import annotations

import math

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """reference src/cloud_engine/attention.py:52-57: float32 mean of squares,
    rsqrt(var + eps), cast back, times weight."""
    dtype = x.dtype
    xf = x.to(torch.float32)
    variance = xf.pow(2).mean(dim=-1, keepdim=True)
    xf = xf * torch.rsqrt(variance + eps)
    return weight * xf.to(dtype)


def rope_tables(head_dim: int, max_len: int, theta: float) -> tuple[torch.Tensor, torch.Tensor]:
    """reference src/cloud_engine/attention.py:60-67: inv_freq_j = 1/theta^(2j/D),
    angle = p * inv_freq, the D/2 angles repeated twice, cos and sin, float32."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    positions = torch.arange(max_len, dtype=torch.float32)
    angles = positions[:, None] * inv_freq[None, :]
    emb = torch.cat((angles, angles), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """reference src/cloud_engine/attention.py:70-72: (-second half, first half)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """reference src/cloud_engine/attention.py:75-85: x*cos + rotate_half(x)*sin
    with the table rows of each token's position; x is [T, heads, D]."""
    c = cos[positions][:, None, :].to(x.dtype)
    s = sin[positions][:, None, :].to(x.dtype)
    return x * c + rotate_half(x) * s


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """reference src/cloud_engine/model.py:89-137 (nn.Linear): x W^T + b, W is [out, in]."""
    out = x @ weight.t()
    return out if bias is None else out + bias


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     past_len: int = 0, window: int | None = None) -> torch.Tensor:
    """reference src/cloud_engine/attention.py:88-112 with the grouped-query
    expansion of :129-147 (query head h reads KV head h // group): scores =
    Q K^T * scale, key j allowed for query row i iff j <= past_len + i, float32
    softmax, probabilities times V, heads concatenated head-major.
    q [Tq, Hq, D]; k, v [Tk, Hkv, D].  ``window`` (not in the reference, which
    attends to all keys) additionally drops keys with j <= past_len + i - window."""
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    group = hq // hkv
    k = k.repeat_interleave(group, dim=1)
    v = v.repeat_interleave(group, dim=1)
    scores = torch.matmul(q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)) * scale  # [Hq, Tq, Tk]
    pos_q = torch.arange(tq) + past_len
    pos_k = torch.arange(tk)
    allowed = pos_q[:, None] >= pos_k[None, :]
    if window is not None:
        allowed = allowed & (pos_k[None, :] > pos_q[:, None] - window)
    scores = scores.to(torch.float32).masked_fill(~allowed[None], float("-inf"))
    probs = torch.softmax(scores, dim=-1).to(v.dtype)
    context = torch.matmul(probs, v.transpose(0, 1)).transpose(0, 1).contiguous()
    return context.reshape(tq, hq * d)


def swiglu(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """reference src/cloud_engine/model.py:99-100: down(silu(gate(x)) * up(x)), no biases."""
    return linear(torch.nn.functional.silu(linear(x, gate)) * linear(x, up), down)


def head_dim_of(config: dict) -> int:
    """reference src/cloud_engine/model.py:75: hidden_size // num_attention_heads
    (an explicit ``head_dim`` key, which the reference does not read, wins here)."""
    return int(config.get("head_dim") or config["hidden_size"] // config["num_attention_heads"])


def attention_layer(x: torch.Tensor, weights: dict, prefix: str, config: dict, cos, sin,
                    positions: torch.Tensor, query_chunk: int | None = None) -> torch.Tensor:
    """reference src/cloud_engine/model.py:132-137, 214-217: q/k/v projections
    (+ bias when ``attention_bias``, default true for qwen2, model.py:80), view as
    heads, rotate q and k, attend, o_proj without bias.  ``query_chunk``: the queries
    are attended a chunk at a time behind the keys before them (``past_len`` of
    attention.py:88-112), so that a sequence of tens of thousands of tokens needs no
    score matrix of its whole square."""
    d = head_dim_of(config)
    bias = config.get("attention_bias", True)
    t = x.shape[0]

    def proj(name: str) -> torch.Tensor:
        b = weights[f"{prefix}{name}.bias"] if bias else None
        return linear(x, weights[f"{prefix}{name}.weight"], b).view(t, -1, d)

    q, k, v = proj("q_proj"), proj("k_proj"), proj("v_proj")
    q = apply_rope(q, cos, sin, positions)
    k = apply_rope(k, cos, sin, positions)
    if query_chunk is None or t <= query_chunk:
        context = causal_attention(q, k, v, 1.0 / math.sqrt(d), past_len=0)
    else:
        context = torch.cat([
            causal_attention(q[start:start + query_chunk], k[:start + query_chunk], v[:start + query_chunk],
                             1.0 / math.sqrt(d), past_len=start)
            for start in range(0, t, query_chunk)])
    return linear(context, weights[f"{prefix}o_proj.weight"])


def forward(config: dict, weights: dict, token_ids: list[int], dtype: torch.dtype = torch.float32,
            query_chunk: int | None = None, rows: list[int] | None = None) -> torch.Tensor:
    """reference src/cloud_engine/model.py:194-228: embedding, per layer
    h += attn(norm(h)); h += mlp(norm(h)), final norm, float32 head (tied to the
    embedding when ``tie_word_embeddings``).  Returns float32 logits [T, vocab], or
    those of the positions ``rows`` only (model.py:222-225 selects rows before the head)."""
    w = {name: (t.to(dtype) if t.is_floating_point() else t) for name, t in weights.items()}
    eps = config["rms_norm_eps"]
    ids = torch.tensor(token_ids, dtype=torch.long)
    positions = torch.arange(len(token_ids))
    cos, sin = rope_tables(head_dim_of(config), max(len(token_ids), 1), config.get("rope_theta", 10000.0))
    h = w["model.embed_tokens.weight"][ids]
    for i in range(config["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = rms_norm(h, w[p + "input_layernorm.weight"], eps)
        h = h + attention_layer(a, w, p + "self_attn.", config, cos, sin, positions, query_chunk)
        m = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        h = h + swiglu(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    h = rms_norm(h, w["model.norm.weight"], eps)
    if rows is not None:
        h = h[torch.tensor(rows, dtype=torch.long)]
    head = w["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return h.to(torch.float32) @ head.to(torch.float32).t()


def greedy(logits_row: torch.Tensor) -> int:
    """reference src/cloud_engine/model.py:231-233: argmax of the float32 logits."""
    return int(torch.argmax(logits_row.to(torch.float32)).item())


def generate_greedy(config: dict, weights: dict, prompt: list[int], steps: int) -> list[int]:
    """Whole-sequence recomputation per token (the reference's naive mode)."""
    tokens = list(prompt)
    out = []
    for _ in range(steps):
        token = greedy(forward(config, weights, tokens)[-1])
        out.append(token)
        tokens.append(token)
    return out
