"""MI355X single-batch decode-schedule interface.

Exports the names the reference's registry glue reads from a route package
(`qimeng_megakernel/models/LLM/registry.py:84-94, 238-262`;
`…/A100/single_batch/decode_schedule/__init__.py:6-40`): ``Globals``,
``ModelConfig``/``LlamaConfig`` eagerly, ``instructions``, ``instruction_defs``,
``scheduler`` and ``mk_kernel`` on first access.

``fused_operations``, ``layer_scheduler`` and ``python_vm`` — the reference's
CPU verification routes — are deliberately not part of this package: the
shipped path is the HIP kernel only, and their restatements live with the tests.
"""
from __future__ import annotations

import importlib

from .globs import Globals
from .model_config import DecodeShape, LlamaConfig

ModelConfig = LlamaConfig

#: Read by the reference's decode loop (`LLM/decode.py:609-611, 1383-1384`):
#: the gfx950 kernel clears its own counters when the last workgroup retires,
#: so the host must not launch a ``barriers.zero_()`` before every step.
STATIC_MEGAKERNEL = True

_LAZY = {
    "instructions": ".instructions",
    "instruction_defs": ".instructions.instruction_defs",
    "scheduler": ".instructions.scheduler",
    "mk_kernel": ".mk_kernel",
}

__all__ = ["Globals", "ModelConfig", "LlamaConfig", "DecodeShape", "STATIC_MEGAKERNEL", *_LAZY]


def __getattr__(name: str):
    target = _LAZY.get(name)
    if target is None:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    return importlib.import_module(target, __name__)
