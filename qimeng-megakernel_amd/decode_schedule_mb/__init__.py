"""Batch 2..16 decode route: host side (instruction set, scheduler, per-row decode state, launcher).

Mirrors the reference's ``…/A100/multi_batch/decode_schedule`` package (`__init__.py:1-37`).
``mk_kernel.get_mk`` binds ``qmk_decode_step_batch`` of the gfx950 library; there is no fallback.
"""
from .globs import Globals  # noqa: F401
