"""CPU-side checks of the drop-in boundary: the C-ABI library loads without a GPU, exports every function that
include/cnet_hip.h declares, the Python signature table covers the same set, and calls before cnet_init fail with a
status code instead of crashing.  No compute call is made here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "cnet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cnet_[a-z0-9_]+)\s*\(", text)))


def test_header_is_plain_c():
    import subprocess
    src = '#include "cnet_hip.h"\nint main(void){return (int)sizeof(cnet_device_info) == 0;}\n'
    res = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"), "-x", "c", "-",
                          "-fsyntax-only"], input=src, text=True, capture_output=True)
    assert res.returncode == 0, res.stderr


def test_library_exports_every_declared_symbol():
    from cnet_amd import capi
    lib = capi.load()
    names = declared_functions()
    assert len(names) >= 38
    for n in names:
        assert hasattr(lib, n), "libcnet_hip.so does not export %s" % n
    assert set(names) == set(capi.SIGNATURES), set(names) ^ set(capi.SIGNATURES)


def test_calls_before_init_return_a_status():
    from cnet_amd import capi
    lib = capi.load()
    if lib.cnet_stream():
        pytest.skip("library already initialised in this process")
    assert lib.cnet_sync() == -1
    p = C.c_void_p()
    assert lib.cnet_alloc(16, C.byref(p)) == -1
    assert b"cnet_init" in lib.cnet_last_error()
    assert lib.cnet_clinear_fwd(None, None, 0, None, None, 0, None, None, 0, 1, 1, 1, 0) == -1
