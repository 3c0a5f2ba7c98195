"""The C-ABI library loads and exports every symbol include/shv_hip.h declares.  No compute."""
import ctypes
import os
import re

import shv


def test_library_is_built_and_loads():
    assert os.path.exists(shv.pkg.lib_path()), "run python strix-halo-vulkan_amd/build.py"
    shv.pkg.load()


def test_every_declared_symbol_is_exported():
    hdr = open(os.path.join(shv.ROOT, "include", "shv_hip.h")).read()
    declared = set(re.findall(r"\b(shv_[a-z0-9_]+)\s*\(", hdr))
    assert declared, "no declarations found in the header"
    L = ctypes.CDLL(shv.pkg.lib_path())
    missing = sorted(s for s in declared if not hasattr(L, s))
    assert not missing, missing
    assert declared == set(shv.api.SYMBOLS), declared ^ set(shv.api.SYMBOLS)


def test_host_library_exports_what_its_header_declares():
    hdr = open(os.path.join(shv.ROOT, "strix-halo-vulkan_amd", "host", "shv_llm.h")).read()
    declared = set(re.findall(r"\b(shv(?:llm|gguf)_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) > 60
    L = ctypes.CDLL(shv.pkg.llm_api.lib_path())
    missing = sorted(s for s in declared if not hasattr(L, s))
    assert not missing, missing


def test_struct_sizes_fit_the_op_record():
    for t in (shv.api.GemvQ4KArgs, shv.api.DequantQ4KArgs, shv.api.QuantizeQ4KArgs,
              shv.api.FillNormalArgs, shv.api.DequantArgs, shv.api.GemvArgs):
        assert ctypes.sizeof(t) <= 248, t
    assert ctypes.sizeof(shv.api.Op) == 256


def test_errors_are_reported_not_swallowed():
    L = shv.pkg.load()
    assert L.shv_sync(None) == -1
    assert b"NULL" in L.shv_last_error()
    p = ctypes.c_void_p()
    assert L.shv_alloc(None, 16, ctypes.byref(p)) == -1
