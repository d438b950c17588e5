"""MI355X-native decode megakernel behind QiMeng-MegaKernel's ``mk`` route.

The directory name carries a hyphen, so the package is registered under the
importable name ``qimeng_megakernel_amd`` by ``__graft_entry__.load_package()``
(tests, ``bench.py`` and ``smoke()`` go through it).

Layout:
  csrc/             hand-written HIP (gfx950) megakernel + its C ABI (include/qmk.h)
  decode_schedule/  host mirror of the reference route package: Globals, LlamaConfig,
                    instruction definitions, scheduler, mk_kernel (get_mk / call_mk)
  instruction.py    instruction wire format
  synthetic.py      seeded random-init weights and Globals allocation (no checkpoint needed)
  decode.py         prefill-by-decode and the greedy step loop with the reference's timing
"""
from __future__ import annotations

from . import instruction  # noqa: F401
from .decode_schedule import Globals, LlamaConfig, DecodeShape, STATIC_MEGAKERNEL  # noqa: F401

__all__ = ["Globals", "LlamaConfig", "DecodeShape", "STATIC_MEGAKERNEL", "instruction"]
