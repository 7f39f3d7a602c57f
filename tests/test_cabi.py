"""The C-ABI library loads without a GPU and exports every symbol that
include/deca_hip.h declares; the binding's table covers the same set."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "deca_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(deca_[a-z_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from deca_amd.driver.build_lib import LIB_PATH, build_library

    if not os.path.exists(LIB_PATH):
        build_library()
    return ctypes.CDLL(LIB_PATH)


def test_header_declares_entry_points():
    syms = declared_symbols()
    for name in ("deca_init", "deca_module_load", "deca_get_function", "deca_launch",
                 "deca_launch_timed", "deca_launch_between", "deca_module_unload", "deca_error_string",
                 "deca_device_info", "deca_set_max_dynamic_lds"):
        assert name in syms


def test_library_exports_every_declared_symbol(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in deca_hip.h but not exported"


def test_binding_table_matches_header():
    from deca_amd.driver.driver import C_API

    assert sorted(C_API) == declared_symbols()


def test_struct_layouts_match_header():
    from deca_amd.driver.driver import DevInfo, FuncInfo

    assert ctypes.sizeof(DevInfo) == 256 + 256 + 10 * 4 + 3 * ctypes.sizeof(ctypes.c_size_t)
    assert ctypes.sizeof(FuncInfo) == 6 * 4


def test_error_string_and_argument_checks(lib):
    lib.deca_error_string.restype = ctypes.c_char_p
    assert lib.deca_error_string(0)  # never NULL
    # null handles are rejected on the host, before any HIP call
    assert lib.deca_module_load(None, None) != 0
    assert lib.deca_get_function(None, b"deca_main", None) != 0
    assert lib.deca_launch(None, 1, 1, 1, 64, 1, 1, 0, None, None, 1) != 0


def test_missing_library_fails_loudly(tmp_path):
    from deca_amd.driver.driver import HipDriver

    with pytest.raises(RuntimeError, match="missing"):
        HipDriver(str(tmp_path / "nope.so"))
