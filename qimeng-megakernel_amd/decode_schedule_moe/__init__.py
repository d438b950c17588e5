"""MoE decode route at batch 1: host side (shape, tensors, instruction set, scheduler).

Mirrors the reference's ``…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule`` package
(`__init__.py:1-39`): attention and LM head as in the dense route (opcodes 1-4, 7; QKV with bias),
the dense MLP replaced by router, shared expert, routed experts and a combine step (opcodes 8-14).
``mk_kernel.get_mk`` binds ``qmk_decode_step_moe`` of the gfx950 library; there is no fallback.
"""
from .globs import Globals  # noqa: F401
from .model_config import QWEN1_5_MOE_A2_7B, MoeShape, QwenMoeConfig  # noqa: F401
