"""The C-ABI library loads and exports every symbol include/moe_mi355.h declares
(no compute calls: this runs without a GPU)."""
import os
import re

from moe_gen_amd import _native as N

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "moe_mi355.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("moe_router", "moe_dispatch", "moe_grouped_swiglu_bf16", "moe_grouped_swiglu_w8a16",
                 "moe_combine", "moe_stage_create", "moe_stage_acquire", "moe_stage_release", "moe_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = N.lib()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in moe_mi355.h but not exported"


def test_binding_covers_header_exactly():
    assert sorted(N.SIGNATURES) == declared_functions()


def test_version_and_error_string():
    lib = N.lib()
    assert b"gfx950" in lib.moe_version()
    assert isinstance(N.last_error(), str)


def test_argument_validation_needs_no_gpu():
    """Entry points reject bad arguments on the host before touching the device."""
    import ctypes
    lib = N.lib()
    p = N.RouterParams(4, 12, 8, 2, 1, 1, 0, 0, 0, 1, 0, 0, 1e-20, 1.0)      # hidden not a multiple of 8
    rc = lib.moe_router(1, 1, None, ctypes.byref(p), 1, 1, None, None)
    assert rc == -1 and "hidden" in N.last_error()
    p = N.RouterParams(4, 16, 8, 2, 1, 1, 7, 0, 0, 1, 0, 0, 1e-20, 1.0)       # unknown scoring function
    assert lib.moe_router(1, 1, None, ctypes.byref(p), 1, 1, None, None) == -1
    assert "scoring" in N.last_error()
    assert lib.moe_combine(1, 1, None, 1, None, 4, 99, 64, 0, 1, None) == -1 and "top_k" in N.last_error()
    assert lib.moe_grouped_swiglu_bf16(1, 8, None, 1, 1, 1, 1, 8, 2, 100, 64, 1, 1, 3, None, 0, None) == -1
    assert "hidden" in N.last_error()
    assert lib.moe_dispatch(1, 4, 2, 300, 1, 1, 1, 1, None, None, 0, None, None, 0, None) == -1
