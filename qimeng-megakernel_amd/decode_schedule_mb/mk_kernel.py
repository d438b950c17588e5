"""Launcher of the batch route's kernel (`…/A100/multi_batch/decode_schedule/mk_kernel.py:41-111`).

The gfx950 kernel for batch 2..16 does not exist yet.  Nothing else stands in for it: asking for
it fails.
"""
from __future__ import annotations

from typing import Any


def get_mk(mk_dir: Any = None):
    raise ImportError("the gfx950 decode kernel for batch sizes 2..16 is not built; "
                      "only the batch-1 kernel (decode_schedule.mk_kernel) is available")


def call_mk(globs: Any, mk: Any) -> None:
    raise ImportError("the gfx950 decode kernel for batch sizes 2..16 is not built")
