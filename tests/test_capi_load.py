"""The C-ABI library loads and exports every symbol include/fluxmi.h declares (no compute calls)."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "fluxmi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fluxmi_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported():
    from flux_amd import capi
    lib = capi.load()
    syms = declared_symbols()
    assert len(syms) >= 10
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in fluxmi.h but not exported"
    assert set(syms) == set(capi.EXPORTS)
    assert lib.fluxmi_version() >= 100


def test_argument_errors_without_gpu():
    """Validation happens before any HIP call, so it is testable on a CPU-only host."""
    from flux_amd import capi
    lib = capi.load()
    rc = lib.fluxmi_topk_gather_reduce(None, 1, 0, None, None, 1.0, 4, 2, 64, None, None)
    assert rc == -1 and b"null pointer" in lib.fluxmi_last_error()
    ptrs = (ctypes.c_void_p * 1)(0x1000)
    rc = lib.fluxmi_topk_gather_reduce(ptrs, 9, 0, ctypes.c_void_p(0x1000), None, 1.0, 4, 2, 64, ctypes.c_void_p(0x1000), None)
    assert rc == -2 and b"ngroups" in lib.fluxmi_last_error()
    rc = lib.fluxmi_topk_gather_reduce(ptrs, 1, 0, ctypes.c_void_p(0x1000), None, 1.0, 4, 2, 60, ctypes.c_void_p(0x1000), None)
    assert rc == -2 and b"multiple of 8" in lib.fluxmi_last_error()
    rc = lib.fluxmi_quant_e4m3_rowwise(ctypes.c_void_p(0x1000), 4, 64, 32, 0.0, ctypes.c_void_p(0x1000),
                                       ctypes.c_void_p(0x1000), 0, None)
    assert rc == -2 and b"block_cols" in lib.fluxmi_last_error()
    rc = lib.fluxmi_moe_route_sort(ctypes.c_void_p(0x1000), 4, 2, 4, None, None, ctypes.c_void_p(0x1000), None, None,
                                   None, 0, None)
    assert rc == -3 and b"workspace" in lib.fluxmi_last_error()
    assert lib.fluxmi_moe_route_sort_workspace_bytes(16384, 6, 64) == (192 + 1) * 64 * 4
    args = capi.GroupedGemmArgs(dtype=7)
    rc = lib.fluxmi_grouped_gemm(ctypes.byref(args), None, 0, None)
    assert rc == -1 and b"dtype" in lib.fluxmi_last_error()
    args = capi.GroupedGemmArgs(dtype=0, nexperts=5000, max_rows=1, n=8, k=64)
    assert lib.fluxmi_grouped_gemm(ctypes.byref(args), None, 0, None) == -2
    args = capi.GroupedGemmArgs(dtype=2, nexperts=2, max_rows=1, n=8, k=64, sched_flags=16)   # fp16 is a dtype; flag 16 is not
    rc = lib.fluxmi_grouped_gemm(ctypes.byref(args), None, 0, None)
    assert rc == -1 and b"null a / b / d / splits" in lib.fluxmi_last_error()
    rc = lib.fluxmi_topk_gather_reduce(ptrs, 1, 4, ctypes.c_void_p(0x1000), None, 1.0, 4, 2, 64, ctypes.c_void_p(0x1000), None)
    assert rc == -1 and b"io_format" in lib.fluxmi_last_error()
    rc = lib.fluxmi_calib_stream(ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1000), 24, 0, None)
    assert rc == -1 and b"multiples of 16" in lib.fluxmi_last_error()
    assert lib.fluxmi_version() >= 110


def test_golden_routing_fixture_matches_oracle():
    from oracle import configs, routing
    z = np.load(os.path.join(ROOT, "tests", "golden", "routing_c1.npz"))
    assert np.array_equal(routing.splits(z["choosed"], 8), z["splits"])
    assert np.array_equal(routing.scatter_index_closed_form(z["choosed"], 8), z["scatter_index"])
    g, t = routing.gather_index(z["scatter_index"], 2)
    assert np.array_equal(g, z["gather_index"]) and np.array_equal(t, z["topk_index"])
    wl, _ = configs.make_routing("C1")
    assert np.array_equal(wl.choosed.numpy(), z["choosed"])  # the generator is still the one that wrote the fixture


def test_golden_index_hashes():
    import hashlib
    from oracle import configs
    want = json.load(open(os.path.join(ROOT, "tests", "golden", "index_hashes.json")))
    for name, h in want.items():
        wl, _ = configs.make_routing(name)
        sha = lambda a: hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
        assert wl.splits.tolist() == h["splits"]
        assert sha(wl.scatter_index) == h["scatter_index"] and sha(wl.gather_index) == h["gather_index"]
