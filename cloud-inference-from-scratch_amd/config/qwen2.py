"""Typed configuration of the Qwen2.5 dense decoder, read from ``config.json``.

Mirrors what the reference validates in ``ModelDims.from_hf_config``
(src/cloud_engine/model.py:32-83): the same required keys, ``hidden_act`` must
be ``silu``, ``rope_scaling`` must be absent, ``attention_bias`` defaults to
true for ``model_type == "qwen2"``, ``rope_theta`` defaults to 10000.  Unlike
the reference nothing stays fixed in code: the rotary table length comes from
``max_position_embeddings`` (the reference hard-codes 32768,
src/cloud_engine/model.py:188-192) and ``head_dim`` is honoured when present.
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Any

from .specs import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

_REQUIRED = (
    "hidden_size",
    "num_hidden_layers",
    "num_attention_heads",
    "num_key_value_heads",
    "intermediate_size",
    "vocab_size",
    "rms_norm_eps",
)


@dataclass(frozen=True)
class Qwen2Config:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    head_dim: int
    rope_theta: float = 10_000.0
    attention_bias: bool = True
    tie_word_embeddings: bool = False
    eos_token_id: int | None = None
    max_position_embeddings: int = 32768
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int | None = None
    model_type: str = "qwen2"

    architecture = "Qwen2ForCausalLM"

    @classmethod
    def from_hf_config(cls, raw: dict[str, Any]) -> "Qwen2Config":
        missing = sorted(key for key in _REQUIRED if key not in raw)
        model_type = raw.get("model_type", "qwen2")
        if missing or model_type != "qwen2":
            raise ConfigError(
                f"unsupported/missing model config fields: {missing} (model_type={model_type!r})"
            )
        if raw.get("hidden_act", "silu") != "silu" or raw.get("rope_scaling"):
            raise ConfigError("only SwiGLU and unscaled RoPE model variants are supported")
        hidden = int(raw["hidden_size"])
        heads = int(raw["num_attention_heads"])
        kv_heads = int(raw["num_key_value_heads"])
        if raw.get("head_dim") is not None:
            head_dim = int(raw["head_dim"])
        else:
            if heads <= 0 or hidden % heads != 0:
                raise ConfigError("hidden_size not divisible by num_attention_heads")
            head_dim = hidden // heads
        eos = raw.get("eos_token_id")
        if isinstance(eos, (list, tuple)):
            eos = eos[0] if eos else None
        config = cls(
            hidden_size=hidden,
            num_hidden_layers=int(raw["num_hidden_layers"]),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            intermediate_size=int(raw["intermediate_size"]),
            vocab_size=int(raw["vocab_size"]),
            rms_norm_eps=float(raw["rms_norm_eps"]),
            head_dim=head_dim,
            rope_theta=float(raw.get("rope_theta", 10_000.0)),
            attention_bias=bool(raw.get("attention_bias", True)),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_id=None if eos is None else int(eos),
            max_position_embeddings=int(raw.get("max_position_embeddings", 32768)),
            hidden_act="silu",
            use_sliding_window=bool(raw.get("use_sliding_window", False)),
            sliding_window=raw.get("sliding_window"),
            max_window_layers=raw.get("max_window_layers"),
        )
        config.validate()
        return config

    def validate(self) -> None:
        for name in (
            "hidden_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "intermediate_size",
            "vocab_size",
            "head_dim",
            "max_position_embeddings",
        ):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                "num_attention_heads must be a multiple of num_key_value_heads "
                f"({self.num_attention_heads} vs {self.num_key_value_heads})"
            )
        if self.head_dim % 2 != 0:
            raise ConfigError("head_dim must be even for rotary position encoding")
        if not self.rms_norm_eps > 0:
            raise ConfigError("rms_norm_eps must be positive")
        if not self.rope_theta > 0:
            raise ConfigError("rope_theta must be positive")
        if self.use_sliding_window:
            # The reference never reads the window keys and attends to every
            # cached key in every layer (src/cloud_engine/attention.py:88-112);
            # a checkpoint that needs a window would silently differ, so refuse.
            raise ConfigError(
                "use_sliding_window=true is not run: the Qwen2.5 decoder here attends to all keys"
            )

    def to_hf_config(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architectures": [self.architecture]}
        for item in fields(self):
            out[item.name] = getattr(self, item.name)
        out["torch_dtype"] = "bfloat16"
        return out

    # -- what the engine builds from -------------------------------------
    def model_spec(self) -> ModelSpec:
        norm = PartSpec.of("rms_norm", size=self.hidden_size, eps=self.rms_norm_eps)
        position = PartSpec.of(
            "rotary_half",
            head_dim=self.head_dim,
            theta=self.rope_theta,
            max_position=self.max_position_embeddings,
        )
        mixer = PartSpec.of(
            "attention",
            hidden_size=self.hidden_size,
            num_heads=self.num_attention_heads,
            num_kv_heads=self.num_key_value_heads,
            head_dim=self.head_dim,
            qkv_bias=self.attention_bias,
            out_bias=False,
            position=position,
            window=None,
            scale=None,
        )
        feed_forward = PartSpec.of(
            "gated_mlp",
            hidden_size=self.hidden_size,
            intermediate_size=self.intermediate_size,
            activation=self.hidden_act,
        )
        layer = LayerSpec(
            mixer=mixer,
            feed_forward=feed_forward,
            norm1=norm,
            norm2=norm,
            block="pre_norm",
            names=(
                ("norm1", "input_layernorm"),
                ("mixer", "self_attn"),
                ("norm2", "post_attention_layernorm"),
                ("feed_forward", "mlp"),
            ),
        )
        count = self.num_hidden_layers
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            layers=tuple(layer for _ in range(count)),
            order=tuple(LayerCall(layer=i, cache=i, writes=True) for i in range(count)),
            final_norm=norm,
            tie_word_embeddings=self.tie_word_embeddings,
            max_position=self.max_position_embeddings,
            eos_token_id=self.eos_token_id,
        )
