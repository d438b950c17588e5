"""The C-ABI library: it loads, exports what include/qmk.h declares, and the ctypes mirror matches the header.

No GPU work here: only entry points that return before touching a device are called.
"""
import ctypes
import re
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from __graft_entry__ import LIBRARY, ROOT, build_library
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule_mb import mk_kernel as mk_kernel_mb
from qimeng_megakernel_amd.decode_schedule_moe import mk_kernel as mk_kernel_moe
from qimeng_megakernel_amd.decode_schedule_mb import rows_kernel as rows_kernel_mb
from qimeng_megakernel_amd.decode_schedule_moe import rows_kernel

HEADER = ROOT / "include" / "qmk.h"


@pytest.fixture(scope="module")
def lib():
    if not LIBRARY.is_file():
        build_library()
    return mk_kernel.load_library()


def test_every_declared_symbol_is_exported(lib):
    text = HEADER.read_text()
    declared = set(re.findall(r"^(?:int|uint64_t|const char\*)\s+(qmk_\w+)\s*\(", text, flags=re.M))
    assert declared == {"qmk_decode_step", "qmk_decode_step_static", "qmk_decode_step_batch", "qmk_decode_step_moe", "qmk_moe_workspace_bytes",
                        "qmk_decode_step_moe_rows", "qmk_moe_rows_workspace_bytes",
                        "qmk_decode_step_rows", "qmk_rows_workspace_bytes", "qmk_query",
                        "qmk_status_fetch", "qmk_error_string", "qmk_workspace_bytes"}
    for name in declared:
        assert hasattr(lib, name), name


@pytest.mark.parametrize("struct,mirror", [("QmkArgs", mk_kernel.QmkArgs), ("QmkBatchArgs", mk_kernel_mb.QmkBatchArgs),
                                           ("QmkMoeArgs", mk_kernel_moe.QmkMoeArgs), ("QmkMoeRowsArgs", rows_kernel.QmkMoeRowsArgs),
                                           ("QmkRowsArgs", rows_kernel_mb.QmkRowsArgs)])
def test_struct_layout_matches_header(tmp_path, struct, mirror):
    """Compile the header with gcc and compare sizeof/offsetof with the ctypes mirror."""
    fields = [name for name, _ in mirror._fields_]
    prog = tmp_path / "layout.c"
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void) {",
             f'  printf("%zu\\n", sizeof({struct}));']
    lines += [f'  printf("%zu\\n", offsetof({struct}, {f}));' for f in fields]
    lines += ["  return 0;", "}"]
    prog.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-o", str(exe), str(prog)], check=True)
    out = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    assert out[0] == ctypes.sizeof(mirror)
    assert out[1:] == [getattr(mirror, f).offset for f in fields]
    # every struct member of the header is mirrored, in order
    body = HEADER.read_text().split("typedef struct " + struct + " {")[1].split("} " + struct + ";")[0]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    members = re.findall(r"(\w+)\s*;", body)
    assert members == fields


def test_constants_match_header():
    text = HEADER.read_text()
    def define(name):
        return int(re.search(rf"#define {name} (\d+)", text).group(1))
    assert define("QMK_FLAG_KEEP_BARRIERS") == mk_kernel.QMK_FLAG_KEEP_BARRIERS
    assert define("QMK_FLAG_XCD_COUNTERS") == mk_kernel.QMK_FLAG_XCD_COUNTERS
    assert define("QMK_FLAG_TAGGED") == mk_kernel.QMK_FLAG_TAGGED
    assert define("QMK_XCD_COUNTER_ROWS") == mk_kernel.QMK_XCD_COUNTER_ROWS
    assert define("QMK_INSTRUCTION_WORDS") == 32


def test_host_side_argument_errors(lib):
    assert lib.qmk_decode_step(None) == 1                                  # QMK_ERR_NULL_ARG
    a = mk_kernel.QmkArgs()
    a.struct_size = 12
    assert lib.qmk_decode_step(ctypes.byref(a)) == 2                       # QMK_ERR_ABI
    a.struct_size = ctypes.sizeof(mk_kernel.QmkArgs)
    a.model = 99
    assert lib.qmk_decode_step(ctypes.byref(a)) == 8                       # QMK_ERR_MODEL
    a.model = 0
    assert lib.qmk_decode_step(ctypes.byref(a)) == 1                       # all tensor pointers are NULL
    assert lib.qmk_workspace_bytes(0) == 8 * (512 + 2048 + 4 * 1024 + 4096 + 1024) and lib.qmk_workspace_bytes(1) == lib.qmk_workspace_bytes(0) and lib.qmk_workspace_bytes(7) == 0
    assert lib.qmk_query(0) == 8 and lib.qmk_query(2) == 512 and lib.qmk_query(5) == 32 and lib.qmk_query(6) == 25
    assert 0 < lib.qmk_query(3) <= 160 * 1024
    assert lib.qmk_error_string(34).decode().startswith("device: counter wait")
    mk_kernel_mb.get_mk()                                                  # declares the entry point's signature
    assert lib.qmk_decode_step_batch(None) == 1
    b = mk_kernel_mb.QmkBatchArgs()
    b.struct_size = 12
    assert lib.qmk_decode_step_batch(ctypes.byref(b)) == 2
    b.struct_size = ctypes.sizeof(mk_kernel_mb.QmkBatchArgs)
    b.model = 2
    assert lib.qmk_decode_step_batch(ctypes.byref(b)) == 8                 # the MoE geometries are not compiled for this route
    for model in (0, 1):                                                   # Llama-3.2-1B, Qwen3-1.7B: all tensor pointers are NULL
        b.model = model
        assert lib.qmk_decode_step_batch(ctypes.byref(b)) == 1
    mk_kernel_moe.get_mk()
    assert lib.qmk_decode_step_moe(None) == 1
    m = mk_kernel_moe.QmkMoeArgs()
    m.struct_size = ctypes.sizeof(mk_kernel_moe.QmkMoeArgs)
    assert lib.qmk_decode_step_moe(ctypes.byref(m)) == 8                   # model 0 is not the MoE geometry
    m.model = 2
    assert lib.qmk_decode_step_moe(ctypes.byref(m)) == 1
    # the shared expert's K-slice terms, the routed experts' rows, the gate's line, the dense route's units, then the MoE route's
    # own units (router logits, one per 128-byte line; routed silu vectors; routed rows; the shared expert's gate; the top-k's
    # picks, a line per slot)
    moe_units = 8 * (512 * 16 + 8 * 1024 + 8 * 2048 + 16 + 8 * 16)
    assert lib.qmk_moe_workspace_bytes(4, 4) == 4 * 2048 * 2 + 4 * 2048 * 4 + 128 + lib.qmk_workspace_bytes(0) + moe_units
    assert lib.qmk_moe_workspace_bytes(8, 0) == 8 * 2048 * 4 + 128 + lib.qmk_workspace_bytes(0) + moe_units     # no shared expert
    assert lib.qmk_moe_workspace_bytes(9, 4) == 0
    assert lib.qmk_error_string(12345).decode() == "unknown code"
    # the dense route at 1..4 rows on the row-streaming engine: per row a set of the dense route's units and the eight
    # 128-byte lines of the row's attention count
    rows_kernel_mb.get_mk()
    per_row = lib.qmk_workspace_bytes(0) + 8 * 128
    assert [lib.qmk_rows_workspace_bytes(b) for b in (0, 1, 4, 5)] == [0, per_row, 4 * per_row, 0]
    assert lib.qmk_decode_step_rows(None) == 1
    d = rows_kernel_mb.QmkRowsArgs()
    d.struct_size = ctypes.sizeof(rows_kernel_mb.QmkRowsArgs)
    assert lib.qmk_decode_step_rows(ctypes.byref(d)) == 2                    # the nested step carries its own size
    d.step.struct_size = ctypes.sizeof(mk_kernel_mb.QmkBatchArgs)
    d.step.model = 2
    assert lib.qmk_decode_step_rows(ctypes.byref(d)) == 8
    d.step.model = 0
    assert lib.qmk_decode_step_rows(ctypes.byref(d)) == 3                    # batch_size 0
    d.step.batch_size = 4
    assert lib.qmk_decode_step_rows(ctypes.byref(d)) == 1                    # all tensor pointers are NULL
    # several requests in one launch: per row a set of the MoE route's units, in whole 128-byte lines, and the eight lines
    # of the row's attention count
    rows_kernel.get_mk()
    per_row = lib.qmk_moe_workspace_bytes(8, 0) - 8 * 2048 * 4 - 128 + 8 * 128
    assert per_row % 128 == 0 and [lib.qmk_moe_rows_workspace_bytes(b) for b in (0, 1, 4, 5)] == [0, per_row, 4 * per_row, 0]
    assert lib.qmk_decode_step_moe_rows(None) == 1
    r = rows_kernel.QmkMoeRowsArgs()
    r.struct_size = 12
    assert lib.qmk_decode_step_moe_rows(ctypes.byref(r)) == 2
    r.struct_size = ctypes.sizeof(rows_kernel.QmkMoeRowsArgs)
    assert lib.qmk_decode_step_moe_rows(ctypes.byref(r)) == 2                # the nested step carries its own size
    r.step.struct_size = ctypes.sizeof(mk_kernel_moe.QmkMoeArgs)
    r.step.model = 2
    assert lib.qmk_decode_step_moe_rows(ctypes.byref(r)) == 8                # a model with a shared expert has no rows route
    r.step.model = 3
    assert lib.qmk_decode_step_moe_rows(ctypes.byref(r)) == 3                # batch_size 0
    r.batch_size = 4
    assert lib.qmk_decode_step_moe_rows(ctypes.byref(r)) == 1                # all tensor pointers are NULL


def test_missing_library_is_an_import_error(tmp_path):
    with pytest.raises(ImportError, match="missing prebuilt kernel"):
        mk_kernel.get_mk(tmp_path)
    (tmp_path / "libqmk_hip.so").write_bytes(b"not an ELF file")
    with pytest.raises(ImportError, match="cannot load"):
        mk_kernel.load_library(tmp_path)


def test_mk_rejects_cpu_tensors_and_bad_dtypes(lib, small_model):
    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
    from qimeng_megakernel_amd.decode_schedule.model_config import LlamaConfig

    shape, w, _ = small_model
    LlamaConfig.set_shape(shape)
    g = synthetic.build_globals(w, shape, 16, "cpu")
    S.build(g)
    assert g.instructions.shape[0] == 1                                    # off-GPU: a single queue, as in the reference
    mk = mk_kernel.get_mk()
    with pytest.raises(ValueError, match="must live on the GPU"):
        mk_kernel.call_mk(g, mk)
    with pytest.raises(TypeError, match="3 scalars, got 1 positional"):
        mk(g.instructions)
    g.hidden_states = g.hidden_states.float()
    with pytest.raises((TypeError, ValueError)):
        mk_kernel.call_mk(g, mk)


def test_product_code_never_imports_the_oracle():
    """The shipped path must not route through the CPU oracle (or any CPU fallback)."""
    pkg = ROOT / "qimeng-megakernel_amd"
    for path in list(pkg.rglob("*.py")):
        text = path.read_text()
        assert "fused_oracle" not in text and "pyvm_oracle" not in text and "oracle/" not in text, path
