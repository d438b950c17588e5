"""Batch 2..16 decode route: host side (instruction set, scheduler, per-row decode state).

Mirrors the reference's ``…/A100/multi_batch/decode_schedule`` package
(`__init__.py:1-37`).  The gfx950 kernel for this route is not built yet: ``mk_kernel.get_mk``
raises instead of falling back to anything else.
"""
from .globs import Globals  # noqa: F401
