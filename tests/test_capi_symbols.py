"""CPU checks of the C-ABI library: it loads, exports every entry point that include/bf_hip.h declares, and
the Python binding covers exactly those entry points.  No compute call is made (no GPU here)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "bf_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bf_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_entry_point():
    from blackforge_amd import capi
    assert os.path.exists(capi.LIB_PATH), "blackforge_amd/lib/libbf_hip.so has not been built"
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 55
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in bf_hip.h but not exported: {missing}"


def test_python_binding_matches_the_header():
    from blackforge_amd import capi
    bound = set(capi.SIGNATURES) | set(capi._SPECIAL)
    assert bound == set(declared_functions())
    capi.load()


def test_error_channel_without_a_gpu():
    from blackforge_amd import capi
    lib = capi.load()
    assert lib.bf_hip_device_count(None) == capi.ERR_INVALID_ARGUMENT
    assert b"count is NULL" in lib.bf_hip_last_error()
    assert b"gfx950" in lib.bf_hip_version()
    n = ctypes.c_int(-1)
    assert lib.bf_hip_device_count(ctypes.byref(n)) == capi.OK and n.value >= 0


def test_product_never_imports_the_oracle():
    """The shipped package must not reference the CPU oracle in any form."""
    pkg = os.path.join(ROOT, "blackforge_amd")
    offenders = []
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(base, f), errors="ignore").read()
                if re.search(r"\boracle\b|bfo_|libbf_oracle|libbf_ref", text):
                    offenders.append(os.path.join(base, f))
    assert not offenders, offenders
