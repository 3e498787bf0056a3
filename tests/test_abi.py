"""The C-ABI library loads on a machine without a GPU and exports every function the public headers declare
(include/boat_hip.h: the device layer; include/boat_api.h: Boat's own API).  No compute call is made here."""
import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
LIB = ROOT / "boat_amd" / "lib" / "libboat_amd.so"


def declared(header):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    names = set(re.findall(r"\b((?:bh|boat)_[a-z0-9_]+)\s*\(", text))
    # a macro in boat_api.h writes four accessor names in one line of the reference header list; they are declared one by one here
    return sorted(n for n in names if not n.endswith("_t"))


@pytest.fixture(scope="module")
def lib():
    assert LIB.exists(), f"{LIB} has not been built (python -m boat_amd.build)"
    return C.CDLL(str(LIB), mode=C.RTLD_LOCAL)


@pytest.mark.parametrize("header", ["boat_hip.h", "boat_api.h"])
def test_every_declared_symbol_is_exported(lib, header):
    names = declared(header)
    assert len(names) > 40, names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/{header} but not exported: {missing}"


def test_no_oracle_or_reference_symbols_in_the_product(lib):
    # the CPU checker must never be linked into the library under test
    for name in ("bo_matmul", "bo_adam_update", "bo_dense_backward"):
        assert not hasattr(lib, name), name


def test_error_reporting_without_a_device_call(lib):
    lib.bh_last_error.restype = C.c_char_p
    assert isinstance(lib.bh_last_error(), bytes)
    lib.boat_dtype_size.restype = C.c_size_t
    assert lib.boat_dtype_size(1) == 4          # BOAT_DTYPE_FLOAT32
