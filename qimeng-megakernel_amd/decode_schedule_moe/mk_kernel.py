"""Launcher of the MoE route's kernel (`…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/mk_kernel.py`).

The gfx950 kernel for opcodes 8-14 does not exist yet.  Nothing else stands in for it: asking for it fails.
"""
from __future__ import annotations

from typing import Any


def get_mk(mk_dir: Any = None):
    raise ImportError("the gfx950 decode kernel for the MoE opcodes (8-14) is not built; "
                      "only the dense routes (decode_schedule, decode_schedule_mb) are available")


def call_mk(globs: Any, mk: Any) -> None:
    raise ImportError("the gfx950 decode kernel for the MoE opcodes (8-14) is not built")
