"""CPU check of the drop-in boundary: both shared libraries load without a GPU and export every function that
include/*.h declares (and the ctypes tables used by the tests bind exactly those names).  No compute call is made."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")
LIBS = {
    "tnn_rocm.h": os.path.join(ROOT, "tnn_amd", "lib", "libtnn_rocm.so"),
    "tnn_rocm_host.h": os.path.join(ROOT, "tnn_amd", "lib", "libtnn_rocm_host.so"),
}


def declared_functions(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    text = re.sub(r"^\s*#[^\n]*", " ", text, flags=re.M)
    names = re.findall(r"\b(tnn_(?:rocm|host)_[a-z0-9_]+)\s*\(", text)
    assert names, "no declarations found in " + header
    return sorted(set(names))


def test_every_header_has_a_library():
    headers = sorted(f for f in os.listdir(INCLUDE) if f.endswith(".h"))
    assert headers == sorted(LIBS), headers


@pytest.mark.parametrize("header", sorted(LIBS))
def test_library_exports_every_declared_symbol(header):
    path = LIBS[header]
    assert os.path.exists(path), "%s is not built (python -c 'import __graft_entry__ as g; g.build()')" % path
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    missing = [n for n in declared_functions(header) if not hasattr(lib, n)]
    assert not missing, "declared in include/%s but not exported: %s" % (header, missing)


@pytest.mark.parametrize("header", sorted(LIBS))
def test_library_exports_nothing_undeclared(header):
    """the reverse direction: every tnn_rocm_* / tnn_host_* function the library exports is declared in its header"""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", LIBS[header]], capture_output=True, text=True, check=True).stdout
    exported = {l.split()[-1] for l in out.splitlines() if l.split() and l.split()[-2] in ("T", "t", "W")}
    prefix = "tnn_rocm_" if header == "tnn_rocm.h" else "tnn_host_"
    undeclared = sorted(n for n in exported if n.startswith(prefix) and n not in set(declared_functions(header)))
    assert not undeclared, undeclared


def test_ctypes_tables_match_the_headers():
    from tnn_amd import capi
    declared = set(declared_functions("tnn_rocm.h"))
    bound = set(capi.SIGNATURES) | {"tnn_rocm_last_error"}
    assert bound <= declared, sorted(bound - declared)
    assert declared <= bound, sorted(declared - bound)


def test_error_string_call_without_gpu():
    # the only entry point exercised here: it touches no device
    lib = ctypes.CDLL(LIBS["tnn_rocm.h"])
    lib.tnn_rocm_last_error.restype = ctypes.c_char_p
    assert isinstance(lib.tnn_rocm_last_error(), bytes)
