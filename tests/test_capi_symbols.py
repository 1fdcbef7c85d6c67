"""The C-ABI library loads on a machine without a GPU and exports every symbol
include/gsampler_hip.h declares (no compute calls here)."""
import ctypes
import os
import re

from gsampler_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "gsampler_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gs_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_something():
    assert len(declared_symbols()) >= 10


def test_every_declared_symbol_is_exported_and_bound():
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} not exported by {capi.LIB_PATH}"
        assert name in capi.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(capi.SIGNATURES) == declared_symbols()


def test_host_only_entry_points():
    l = capi.lib()
    assert l.gs_abi_version() >= 1
    assert l.gs_scan_workspace_bytes(10**6) > 0
    assert l.gs_unique_workspace_bytes(10, 100, 1) >= 2 * 110 * 8
    assert l.gs_unique_workspace_bytes(-1, 0, 1) == 0


def test_argument_errors_are_reported_without_a_gpu():
    l = capi.lib()
    # negative fanout is rejected before any HIP call
    rc = l.gs_csc_col_sample_uniform_fill(None, 0, None, None, 0, -1, 0, 0, 0, 0,
                                          None, None, None, None, None, None, 0, None)
    assert rc == 1 and b"fanout" in l.gs_last_error()
    rc = l.gs_csc_col_sample_uniform_fill(None, 0, None, None, 0, 100, 0, 2, 0, 0,
                                          None, None, None, None, None, None, 0, None)
    assert rc == 1 and b"Floyd" in l.gs_last_error()
    rc = l.gs_unique_count(None, None, 0, None, None, 0, 0, None, None, None, 0, None)
    assert rc == 1
