"""The C-ABI library loads and exports every symbol include/neus2_amd.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "neus2_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(n2_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    syms = declared_symbols()
    assert "n2_grid_forward" in syms and "n2_last_error" in syms and len(syms) >= 10


def test_library_exports_every_declared_symbol():
    from neus2_amd import capi
    if not os.path.exists(capi.LIB_PATH):
        from neus2_amd.build import build_library
        build_library()
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_host_only_entry_points_work_without_gpu():
    """Object creation and the level table are pure host code."""
    import numpy as np
    from neus2_amd import capi
    L = capi.lib()
    h = ctypes.c_void_p()
    assert L.n2_grid_create(16, 2, 19, 16, ctypes.c_float(1.447), ctypes.byref(h)) == 0
    assert L.n2_grid_n_params(h) == 12599920 and L.n2_grid_output_width(h) == 32
    res = np.zeros(16, np.uint32)
    off = np.zeros(17, np.uint32)
    assert L.n2_grid_level_table(h, None, capi.ptr(res), None, capi.ptr(off)) == 0
    assert res.tolist() == [16, 24, 34, 49, 71, 102, 147, 213, 308, 445, 644, 932, 1349, 1951, 2823, 4085]
    assert int(off[-1]) == 6299960
    L.n2_grid_destroy(h)
    # error behaviour: unsupported feature count, message available
    assert L.n2_grid_create(16, 4, 19, 16, ctypes.c_float(1.447), ctypes.byref(h)) == 3
    assert b"n_features_per_level" in L.n2_last_error()
    assert L.n2_grid_create(0, 2, 19, 16, ctypes.c_float(1.447), ctypes.byref(h)) == 1


def test_level_table_matches_oracle(oracle):
    import numpy as np
    from neus2_amd import capi
    L = capi.lib()
    for cfg in [(16, 19, 16, 1.447), (14, 19, 16, 1.4472692012786865), (8, 14, 4, 2.0), (5, 4, 2, 1.5)]:
        h = ctypes.c_void_p()
        assert L.n2_grid_create(cfg[0], 2, cfg[1], cfg[2], ctypes.c_float(cfg[3]), ctypes.byref(h)) == 0
        g = oracle.Grid(*cfg)
        sc, res, ent, off = (np.zeros(cfg[0], np.float32), np.zeros(cfg[0], np.uint32), np.zeros(cfg[0], np.uint32),
                             np.zeros(cfg[0] + 1, np.uint32))
        assert L.n2_grid_level_table(h, capi.ptr(sc), capi.ptr(res), capi.ptr(ent), capi.ptr(off)) == 0
        assert np.array_equal(sc, g.scale) and np.array_equal(res, g.resolution)
        assert np.array_equal(ent, g.entries) and np.array_equal(off, g.offset)
        L.n2_grid_destroy(h)


def test_cpp_shim_host_checks():
    """The header-only C++ shim (tcnn method names over the C ABI) compiles with the host compiler and its
    host-only behaviour holds: shapes, parameter counts, matrix views, errors as std::runtime_error."""
    import subprocess
    from neus2_amd.build import build_library, build_shim_check
    build_library()
    exe = build_shim_check()
    r = subprocess.run([exe, "host"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "shim host checks ok" in r.stdout
