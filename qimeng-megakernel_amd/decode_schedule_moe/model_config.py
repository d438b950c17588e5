"""Shape and schedule constants of the MoE decode route (Qwen1.5-MoE-A2.7B by default; ``QWEN3_30B_A3B`` is
the second compiled geometry: the Qwen3 op set's attention in front of a MoE block without a shared expert).

``QwenMoeConfig`` keeps the reference's access pattern — class attributes read at call time,
``update_from_dict`` (`…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/model_config.py:8-180`)
— over one immutable ``MoeShape`` record.  Counter rows are ``opcode - 1`` (`:183-200`).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping


@dataclasses.dataclass(frozen=True)
class MoeShape:
    num_hidden_layers: int = 24
    hidden_size: int = 2048
    head_dim: int = 128
    num_attention_heads: int = 16
    num_key_value_heads: int = 16
    vocab_size: int = 151936
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1000000.0
    intermediate_size: int = 5632           # shared expert
    moe_intermediate_size: int = 1408       # one routed expert
    num_experts: int = 60
    num_experts_per_tok: int = 4
    norm_topk_prob: bool = False            # top-k weights divided by their sum (`…/fused/operations.py:405`)
    qkv_bias: bool = True
    qk_norm: bool = False                   # the Qwen3 op set's attention: raw QKV, per-head RMSNorm of q and k, RoPE
    attn_kv_block_size: int = 16
    attn_reduction_size: int = 4
    tile_n_granularity: int = 16
    num_downproj_split_k_shared: int = 4
    routed_upgate_tile: int = 16            # outputs per tile of the routed up/gate instructions (16, or 8)
    oproj_tile: int = 16                    # rows per tile of the O-projection instructions (16, or 8: one tile per queue of 256)
    qkv_tile: int = 16                      # rows per tile of the QKV instructions (16, 8, 4 or 2: whichever deals them evenly)

    @property
    def has_shared_expert(self) -> bool:
        return self.intermediate_size > 0

    @property
    def num_heads(self) -> int:
        return self.num_attention_heads + 2 * self.num_key_value_heads

    @property
    def qkv_out_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def num_hidden_blocks(self) -> int:
        return self.hidden_size // self.tile_n_granularity

    @property
    def num_moe_intermediate_blocks(self) -> int:
        return self.moe_intermediate_size // self.tile_n_granularity

    @property
    def num_oproj_blocks(self) -> int:
        return self.hidden_size // self.oproj_tile

    @property
    def num_routed_upgate_blocks(self) -> int:
        return self.moe_intermediate_size // self.routed_upgate_tile

    @property
    def split_k_granularity_shared(self) -> int:
        return self.intermediate_size // max(1, self.num_downproj_split_k_shared)

    @property
    def barrier_slots(self) -> int:
        return self.num_hidden_blocks

    def weight_bytes_per_token(self) -> int:
        """bf16 weight bytes one decode step streams: attention, router, shared expert and the
        ``num_experts_per_tok`` routed experts it selects, norms, LM head."""
        h = self.hidden_size
        attn = (self.qkv_out_dim * h + self.num_attention_heads * self.head_dim * h) * 2 + (self.qkv_out_dim * 2 if self.qkv_bias else 0)
        shared = (3 * self.intermediate_size * h * 2 + h * 2) if self.has_shared_expert else 0
        routed = self.num_experts_per_tok * 3 * self.moe_intermediate_size * h * 2
        router = self.num_experts * h * 2
        per_layer = attn + shared + routed + router + 2 * h * 2 + (2 * self.head_dim * 2 if self.qk_norm else 0)
        return per_layer * self.num_hidden_layers + self.vocab_size * h * 2 + h * 2

    def kv_bytes_per_context_token(self) -> int:
        return self.num_hidden_layers * 2 * self.num_key_value_heads * self.head_dim * 2

    def step_bytes(self, context_len: int) -> int:
        kv = self.kv_bytes_per_context_token()
        return self.weight_bytes_per_token() + kv * context_len + kv


#: Qwen1.5-MoE-A2.7B, the reference's shape.  QKV tiles of 8 rows: 768 of them, three per queue of a 256-CU device
#: (384 tiles of 16 leave half of the queues with two); `reference_scheduler` emits the reference's tiles of 16.
QWEN1_5_MOE_A2_7B = MoeShape(qkv_tile=8)

#: Qwen3-30B-A3B shape: 48 layers, 32 query / 4 KV heads of 128 (attention output 4096 wide), per-head QK RMSNorm,
#: no QKV bias, 128 experts of 768 with renormalised top-8 routing, no shared expert, untied LM head; 61 GB in bf16.
#: Routed up/gate tiles of 8 outputs: 8 x 96 = 768 tiles, three per queue of a 256-CU device; QKV tiles of 4 rows:
#: 1280 tiles, five per queue (320 tiles of 16 leave a quarter of the queues with two).
QWEN3_30B_A3B = MoeShape(
    num_hidden_layers=48, num_attention_heads=32, num_key_value_heads=4, intermediate_size=0, moe_intermediate_size=768,
    num_experts=128, num_experts_per_tok=8, norm_topk_prob=True, qkv_bias=False, qk_norm=True, attn_reduction_size=8,
    num_downproj_split_k_shared=0, routed_upgate_tile=8, oproj_tile=8, qkv_tile=4,
)

MAX_OPCODE = 14
NUM_OPCODE_ROWS = MAX_OPCODE + 1
MAX_NUM_PARTIALS = 27
A100_SM_COUNT = 108

# barriers[layer, opcode - 1, slot]
ROW_QKV_ROPE, ROW_ATTN_PARTIAL, ROW_ATTN_REDUCTION, ROW_O_PROJ, ROW_LM_HEAD = 0, 1, 2, 3, 6
ROW_ROUTER_GEMV, ROW_ROUTER_TOPK, ROW_SHARED_UPGATE, ROW_SHARED_DOWNPROJ = 7, 8, 9, 10
ROW_ROUTED_UPGATE, ROW_ROUTED_DOWNPROJ, ROW_COMBINE_COMMIT = 11, 12, 13
SLOT_ROUTER_LOGITS, SLOT_NORMED_HIDDEN = 0, 1

_FIELDS = tuple(f.name for f in dataclasses.fields(MoeShape))


class _ConfigMeta(type):
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


class QwenMoeConfig(metaclass=_ConfigMeta):
    _shape: MoeShape = QWEN1_5_MOE_A2_7B

    @classmethod
    def shape(cls) -> MoeShape:
        return cls._shape

    @classmethod
    def set_shape(cls, shape: MoeShape) -> None:
        type.__setattr__(cls, "_shape", shape)

    @classmethod
    def update_from_dict(cls, config: Mapping[str, Any]) -> None:
        heads = int(config["num_attention_heads"])
        changes: dict[str, Any] = dict(
            num_hidden_layers=int(config["num_hidden_layers"]),
            hidden_size=int(config["hidden_size"]),
            head_dim=int(config.get("head_dim") or int(config["hidden_size"]) // heads),
            num_attention_heads=heads,
            num_key_value_heads=int(config.get("num_key_value_heads", heads)),
            vocab_size=int(config["vocab_size"]),
            rms_norm_eps=float(config.get("rms_norm_eps", 1e-6)),
            intermediate_size=int(config.get("shared_expert_intermediate_size", config.get("intermediate_size", 5632))),
            moe_intermediate_size=int(config.get("moe_intermediate_size", 1408)),
            num_experts=int(config.get("num_experts", 60)),
            num_experts_per_tok=int(config.get("num_experts_per_tok", 4)),
            norm_topk_prob=bool(config.get("norm_topk_prob", False)),
        )
        if changes["intermediate_size"] == 0:    # no shared expert: nothing to split
            changes["num_downproj_split_k_shared"] = 0
        cls.set_shape(dataclasses.replace(cls._shape, **changes))


def num_partials_for(sm_count: int, shape: MoeShape) -> int:
    """Split-KV fan-out: about one wave of the device (`model_config.py:215-223`)."""
    n_kv = shape.num_key_value_heads
    return max(1, min(MAX_NUM_PARTIALS, (sm_count + n_kv - 1) // n_kv))
