"""The built libraries load without a GPU and export every entry point the headers declare.

No compute call is made here.  The C headers are parsed for their function declarations;
the C++ agent header for its nixlAgent member functions; the plugin library is checked
for the two discovery symbols the reference's plugin manager resolves
(src/core/nixl_plugin_manager.cpp:46-51,94-122).
"""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
LIB = os.path.join(ROOT, "nixl_amd", "lib")

C_HEADERS = {
    "nixl_amd_hip.h": "libnixl_amd_kernels.so",
    "nixl_amd_ep.h": "libnixl_amd_kernels.so",
    "nixl_amd_capi.h": "libnixl_amd_agent.so",
}


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _declared_functions(header):
    text = _strip_comments(open(os.path.join(INC, header)).read())
    names = re.findall(r"\b(nixl_(?:amd|capi)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def _exported(lib, demangle=False):
    path = os.path.join(LIB, lib)
    if not os.path.exists(path):
        pytest.fail(f"{path} missing: run __graft_entry__.build() first")
    args = ["nm", "-D", "--defined-only"] + (["-C"] if demangle else []) + [path]
    out = subprocess.run(args, check=True, capture_output=True, text=True).stdout
    return out


@pytest.mark.parametrize("header", sorted(C_HEADERS))
def test_c_header_symbols_exported(header):
    declared = _declared_functions(header)
    assert len(declared) >= 5, declared
    lib = ctypes.CDLL(os.path.join(LIB, C_HEADERS[header]), mode=ctypes.RTLD_GLOBAL)
    missing = [n for n in declared if not hasattr(lib, n)]
    assert not missing, f"{C_HEADERS[header]} lacks {missing}"


def test_python_binding_tables_match_headers():
    """The ctypes signature tables name exactly the functions the headers declare."""
    from nixl_amd import _lib
    kernel_decl = sorted(set(_declared_functions("nixl_amd_hip.h") + _declared_functions("nixl_amd_ep.h")))
    assert kernel_decl == _lib.kernel_symbols()
    assert _declared_functions("nixl_amd_capi.h") == _lib.capi_symbols()


def test_plugin_exports_discovery_symbols():
    path = os.path.join(LIB, "plugins", "libplugin_HIP.so")
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
    assert hasattr(lib, "nixl_plugin_init") and hasattr(lib, "nixl_plugin_fini")


def test_plugin_table_without_gpu():
    """nixl_plugin_init returns the table of the reference's layout
    (src/api/cpp/backend/backend_plugin.h:33-58): api version, create, destroy, name,
    version, options, mems.  Reading it needs no GPU."""
    path = os.path.join(LIB, "plugins", "libplugin_HIP.so")
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
    lib.nixl_plugin_init.restype = ctypes.c_void_p
    table = lib.nixl_plugin_init()
    assert table
    words = (ctypes.c_void_p * 7).from_address(table)
    assert ctypes.c_int.from_address(table).value == 1  # NIXL_PLUGIN_API_VERSION
    get_name = ctypes.CFUNCTYPE(ctypes.c_char_p)(words[3])
    assert get_name() == b"HIP"
    lib.nixl_plugin_fini()


def test_agent_members_exported():
    text = _strip_comments(open(os.path.join(INC, "nixl", "nixl.h")).read())
    body = text[text.index("class nixlAgent"):]
    members = set(re.findall(r"\n\s+([a-zA-Z]\w+)\s*\(", body)) - {"nixlAgent", "operator"}
    assert {"registerMem", "prepXferDlist", "makeXferReq", "createXferReq", "postXferReq",
            "getXferStatus", "releaseXferReq", "createBackend"} <= members
    syms = _exported("libnixl_amd_agent.so", demangle=True)
    missing = [m for m in sorted(members) if f"nixlAgent::{m}(" not in syms]
    assert not missing, missing


def test_product_code_never_reaches_for_the_cpu_oracle():
    """The oracle is test infrastructure: nothing in the package imports it, no product source
    names it, and no product library links it."""
    pkg = os.path.join(ROOT, "nixl_amd")
    offenders = []
    for base, _dirs, files in os.walk(pkg):
        if "__pycache__" in base or os.path.join(pkg, "lib") in base:
            continue
        for f in files:
            if not f.endswith((".py", ".cpp", ".h", ".hip", "Makefile")):
                continue
            text = open(os.path.join(base, f), errors="replace").read()
            if re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M) or "liboracle" in text or "oracle/" in text:
                offenders.append(os.path.join(base, f))
    assert not offenders, offenders
    for lib in ("libnixl_amd_kernels.so", "libnixl_amd_agent.so", os.path.join("plugins", "libplugin_HIP.so")):
        out = subprocess.run(["readelf", "-d", os.path.join(LIB, lib)], check=True, capture_output=True, text=True).stdout
        assert "oracle" not in out.lower() and "MEMCPY" not in out, lib
