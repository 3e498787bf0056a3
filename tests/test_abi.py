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


def _reference_abi():
    import json
    return json.loads((ROOT / "tests" / "golden" / "reference_abi.json").read_text())


def test_library_exports_what_the_reference_headers_declare(lib):
    """tests/golden/reference_abi.json lists every function the REFERENCE's headers declare inside the line ranges that
    include/boat_api.h cites (written by tests/golden/make_abi_list.py from the reference tree).  Whatever the reference
    also defines must be exported here: a program that links against the reference must link against this library."""
    abi = _reference_abi()
    assert len(abi["functions"]) > 250
    missing = [f"{f['name']} ({f['header']}:{f['line']})" for f in abi["functions"] if f["defined"] and not hasattr(lib, f["name"])]
    assert not missing, f"declared and defined by the reference, not exported by libboat_amd.so: {missing}"


# Families of the reference's exports that this library does not provide, each with its reason.  Anything else the
# reference's library defines must be exported here: a new gap fails the test below instead of going unnoticed.
OUT_OF_SCOPE = {
    "boat_graph_": "the graph IR (src/graph): building, rewriting and traversing graphs is not on the training hot path; "
                   "boat_graph_create / _create_with_device / _free exist as handles a context or a model can carry",
    "boat_node_": "graph IR nodes",
    "boat_edge_": "graph IR edges",
    "boat_computation_graph_": "the graph-based autodiff prototype (src/graph); the tape of autodiff.h is what the path uses",
    "boat_lstm_layer_": "recurrent layers: not on the path, and forward-only stubs in the reference",
    "boat_gru_layer_": "recurrent layers: not on the path, and forward-only stubs in the reference",
    "boat_batchnorm2d_layer_": "batch normalisation: not on the path (the MNIST CNN and the block use none)",
}
# graph handles that do exist here although their family is out of scope
GRAPH_HANDLES = {"boat_graph_create", "boat_graph_create_with_device", "boat_graph_free"}


def test_every_reference_export_is_here_or_listed_out_of_scope(lib):
    """Every boat_* function the reference's own library defines (the `exports` list of reference_abi.json, from nm on the
    compiled reference) is exported by this library or belongs to a family listed in OUT_OF_SCOPE with its reason."""
    exports = _reference_abi()["exports"]
    assert len(exports) > 300
    unexplained = [n for n in exports if not hasattr(lib, n) and not any(n.startswith(p) for p in OUT_OF_SCOPE)]
    assert not unexplained, f"defined by the reference, neither exported here nor listed as out of scope: {unexplained}"
    assert all(hasattr(lib, n) for n in GRAPH_HANDLES)
    # the list stays honest: a family none of whose functions is missing any more should leave it
    for prefix in OUT_OF_SCOPE:
        assert any(n.startswith(prefix) and not hasattr(lib, n) for n in exports), prefix


def test_prototypes_match_the_reference_headers():
    """Same list: every function of it that include/boat_api.h declares is declared with the reference's prototype
    (return type and parameter types after removing export macros, parameter names and spacing), and every function
    the reference defines is declared."""
    import sys
    sys.path.insert(0, str(ROOT / "tests" / "golden"))
    import make_abi_list as m

    ours = {name: proto for _, name, proto in m.declarations((ROOT / "include" / "boat_api.h").read_text())}
    abi = _reference_abi()
    # the ranges recorded in the list are the ones the header cites today
    assert {h: [list(x) for x in s] for h, s in m.cited_ranges((ROOT / "include" / "boat_api.h").read_text()).items()} == abi["cited_ranges"]
    undeclared = [f["name"] for f in abi["functions"] if f["defined"] and f["name"] not in ours]
    assert not undeclared, f"defined by the reference inside the cited ranges, not declared in include/boat_api.h: {undeclared}"
    different = [(f["prototype"], ours[f["name"]]) for f in abi["functions"] if f["name"] in ours and ours[f["name"]] != f["prototype"]]
    assert not different, different


def test_no_oracle_or_reference_symbols_in_the_product(lib):
    # the CPU checker must never be linked into the library under test
    for name in ("bo_matmul", "bo_adam_update", "bo_dense_backward"):
        assert not hasattr(lib, name), name


def test_error_reporting_without_a_device_call(lib):
    lib.bh_last_error.restype = C.c_char_p
    assert isinstance(lib.bh_last_error(), bytes)
    lib.boat_dtype_size.restype = C.c_size_t
    assert lib.boat_dtype_size(1) == 4          # BOAT_DTYPE_FLOAT32
