"""CPU-only: the C-ABI library loads and exports every entry point include/mi355_moe.h declares;
argument validation that needs no GPU returns the documented status codes."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    src = open(os.path.join(ROOT, "include", "mi355_moe.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", src)))


@pytest.fixture(scope="module")
def lib():
    from gfx1151_engine_amd import capi
    return capi.lib()


def test_every_declared_symbol_is_exported(lib):
    names = declared()
    assert len(names) >= 15
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_status_strings_and_version(lib):
    assert b"gfx950" in lib.moe_version()
    for code, word in [(0, b"ok"), (-1, b"unsupported"), (-2, b"invalid"), (-3, b"context")]:
        assert word in lib.moe_status_string(C.c_int(code))


def test_null_and_shape_validation_without_gpu(lib):
    # null pointers / bad shapes are rejected before anything touches the device
    assert lib.moe_q4cp_dequant_rows(None, C.c_uint64(1), C.c_uint64(32), C.c_uint64(0), C.c_uint64(1), None, None) == -2
    assert lib.moe_q4k_dequant_rows(None, C.c_uint64(1), C.c_uint64(256), None, None) == -2
    assert lib.moe_router_topk(None, None, None, 1, 8, 2, 16, None) == -2
    assert lib.moe_create(None, None) == -2
    assert lib.moe_forward(None, 0, None, 1, None, None) == -2
    assert lib.moe_routing_create(0, 8, None) == -2
    assert lib.moe_tiles(None, None, None, 8, 64, None) == -2
    assert lib.moe_gg_gemv(2, 12, None, None, None, None, None, None, None, None, 1, 256, 256, 10, 16, None) == -1
