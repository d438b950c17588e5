"""Model shape of the decode route (Llama-3.2-1B shape by default).

``LlamaConfig`` keeps the reference's access pattern — a class whose attributes
are read at call time and can be re-pointed at another checkpoint's shape with
``update_from_dict`` / ``update_from_hf``
(`…/A100/single_batch/decode_schedule/model_config.py:4-61`) — but the values
live in one immutable ``DecodeShape`` record so that a shape can also be passed
around explicitly (tests use reduced layer counts and vocabularies).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping


@dataclasses.dataclass(frozen=True)
class DecodeShape:
    num_hidden_layers: int = 16
    hidden_size: int = 2048
    intermediate_size: int = 8192
    head_dim: int = 64
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    vocab_size: int = 128256
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    # split-KV geometry: KV tokens are cut into blocks of this many tokens,
    # one reduction instruction merges this many query heads (= GQA ratio).
    attn_kv_block_size: int = 16
    attn_reduction_size: int = 4
    # Qwen3 op set (`…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/operations.py:52-120`):
    # opcode 1 leaves the raw QKV vector, the attention prologue applies a per-head RMSNorm to q
    # and k before RoPE; the LM head shares the embedding matrix.
    qk_norm: bool = False
    tie_word_embeddings: bool = False

    @property
    def num_heads(self) -> int:
        return self.num_attention_heads + 2 * self.num_key_value_heads

    @property
    def qkv_out_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def gqa_ratio(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def weight_bytes_per_token(self) -> int:
        """bf16 weight bytes one decode step has to stream (norm vectors included)."""
        h, f = self.hidden_size, self.intermediate_size
        per_layer = (self.qkv_out_dim * h + self.num_attention_heads * self.head_dim * h + 3 * f * h) * 2 + 2 * h * 2
        if self.qk_norm:
            per_layer += 2 * self.head_dim * 2
        return per_layer * self.num_hidden_layers + self.vocab_size * h * 2 + h * 2

    def kv_bytes_per_context_token(self) -> int:
        return self.num_hidden_layers * 2 * self.num_key_value_heads * self.head_dim * 2

    def step_bytes(self, context_len: int) -> int:
        """Algorithmic HBM bytes of one decode step attending to ``context_len`` tokens."""
        kv = self.kv_bytes_per_context_token()
        return self.weight_bytes_per_token() + kv * context_len + kv


LLAMA_3_2_1B = DecodeShape()

#: Qwen3-1.7B shape: 28 layers, 16 query / 8 KV heads of 128, per-head QK RMSNorm, tied LM head.
QWEN3_1_7B = DecodeShape(
    num_hidden_layers=28, hidden_size=2048, intermediate_size=6144, head_dim=128, num_attention_heads=16,
    num_key_value_heads=8, vocab_size=151936, rms_norm_eps=1e-6, rope_theta=1000000.0, attn_reduction_size=2,
    qk_norm=True, tie_word_embeddings=True,
)

_FIELDS = tuple(f.name for f in dataclasses.fields(DecodeShape))


class _ConfigMeta(type):
    """Class attributes of LlamaConfig resolve against the current DecodeShape."""

    def __getattr__(cls, name: str) -> Any:
        shape = type.__getattribute__(cls, "_shape")
        try:
            return getattr(shape, name)
        except AttributeError:
            raise AttributeError(f"{cls.__name__} has no attribute {name!r}") from None

    def __setattr__(cls, name: str, value: Any) -> None:
        if name in _FIELDS:
            type.__setattr__(cls, "_shape", dataclasses.replace(cls._shape, **{name: value}))
        else:
            type.__setattr__(cls, name, value)


class LlamaConfig(metaclass=_ConfigMeta):
    _shape: DecodeShape = LLAMA_3_2_1B

    @classmethod
    def shape(cls) -> DecodeShape:
        return cls._shape

    @classmethod
    def set_shape(cls, shape: DecodeShape) -> None:
        type.__setattr__(cls, "_shape", shape)

    @classmethod
    def update_from_dict(cls, config: Mapping[str, Any]) -> None:
        heads = int(config["num_attention_heads"])
        head_dim = config.get("head_dim") or int(config["hidden_size"]) // heads
        kv_heads = int(config.get("num_key_value_heads", heads))
        changes: dict[str, Any] = dict(
            num_hidden_layers=int(config["num_hidden_layers"]),
            hidden_size=int(config["hidden_size"]),
            intermediate_size=int(config["intermediate_size"]),
            head_dim=int(head_dim),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            vocab_size=int(config["vocab_size"]),
            rms_norm_eps=float(config.get("rms_norm_eps", 1e-5)),
            attn_reduction_size=heads // kv_heads,
        )
        for optional in ("rope_theta", "attn_kv_block_size", "attn_reduction_size"):
            if optional in config and config[optional] is not None:
                changes[optional] = type(getattr(cls._shape, optional))(config[optional])
        cls.set_shape(dataclasses.replace(cls._shape, **changes))

    @classmethod
    def update_from_hf(cls, config: Any) -> None:
        keys = _FIELDS + ("num_key_value_heads",)
        cls.update_from_dict({k: getattr(config, k) for k in keys if hasattr(config, k)})

    @classmethod
    def as_dict(cls) -> dict[str, Any]:
        out = dataclasses.asdict(cls._shape)
        out["num_heads"] = cls._shape.num_heads
        out["qkv_out_dim"] = cls._shape.qkv_out_dim
        return out


ModelConfig = LlamaConfig
