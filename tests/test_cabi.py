"""The C-ABI library builds into the package, loads, and exports every function the header declares."""
import ctypes
import os
import re

import scattermoe_amd._C as C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "scattermoe_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smoe_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared() == sorted(C.EXPORTED_SYMBOLS)


def test_library_exports_declared_symbols():
    lib = C.load()
    assert os.path.dirname(C.lib_path()) == os.path.join(ROOT, "scattermoe_amd")   # in-tree, not site-packages
    for name in _declared():
        assert getattr(lib, name) is not None
    assert lib.smoe_version() == 1
    assert lib.smoe_last_error() == b""


def test_argument_errors_need_no_gpu():
    lib = C.load()
    assert lib.smoe_route_workspace_bytes(4096, 8) == 0
    assert lib.smoe_route_workspace_bytes(16384, 512) == 0          # one workgroup sorts up to 16384 rows by itself
    assert lib.smoe_route_workspace_bytes(16385, 8) == 5 * 8 * 4
    assert lib.smoe_route_workspace_bytes(4097, 513) == 2 * 513 * 4
    assert lib.smoe_route(None, 0, 16, 8, None, None, None, None, 0, None) == -1          # SMOE_ERR_NULL
    assert b"NULL" in lib.smoe_last_error()
    assert lib.smoe_route(None, 0, -1, 8, None, None, None, None, 0, None) == -2          # SMOE_ERR_SHAPE
    assert lib.smoe_group(None, 0, 0, None, None, 0, 0, None, 4, 4, 1, 9, None) == -3       # SMOE_ERR_DTYPE
    one = ctypes.c_void_p(16)
    assert lib.smoe_route(one, 0, 100000, 8, one, one, one, None, 0, None) == -4          # SMOE_ERR_WORKSPACE
    assert lib.smoe_route(one, 0, 1 << 33, 8, one, one, one, one, 1 << 40, None) == -5    # SMOE_ERR_RANGE


def test_gathered_weight_gradient_rejects_what_it_cannot_gather():
    """Only the bf16 / fp16 MFMA kernel reads X through the index vector: float32 and a row count that is no
    multiple of fan_out are refused before anything is launched (so no GPU is needed to see it)."""
    lib = C.load()
    one = ctypes.c_void_p(256)
    args = lambda L, fan, dtype: (one, 64, 1, one, 64, 1, one, fan, one, 64 * 64, 1, 64, None, 0, 0, one,
                                  L, 64, 64, 2, dtype, None)
    assert lib.smoe_groupXtY_gathered(*args(128, 2, C.F32)) == C.ERR_UNSUPPORTED
    assert b"float32" in lib.smoe_last_error()
    assert lib.smoe_groupXtY_gathered(*args(127, 2, C.BF16)) == -2                          # SMOE_ERR_SHAPE
    assert b"fan_out" in lib.smoe_last_error()


def test_static_routing_reports_too_many_experts_as_range_error():
    lib = C.load()
    one = ctypes.c_void_p(256)
    assert lib.smoe_route_static(one, 0, 1 << 20, 4096, one, one, one, None) == -5          # SMOE_ERR_RANGE
    assert lib.smoe_route_static(one, 0, 1 << 22, 2048, one, one, one, None) == -4          # SMOE_ERR_WORKSPACE
