"""The C-ABI library loads on a machine without a GPU, exports every symbol the
header declares, and rejects bad arguments with error codes (no compute calls here)."""
import ctypes
import os
import re

import pytest

from featgraph_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "featgraph_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    return re.findall(r"^FG_API\s+[\w\s\*]+?\b(fg_\w+)\s*\(", text, flags=re.M)


def test_header_declares_the_expected_entry_points():
    names = _declared_symbols()
    assert len(names) == len(set(names)) >= 14
    for must in ("fg_spmm_plan_create", "fg_spmm_csr_f32", "fg_spmm_csr_mh_f32", "fg_sddmm_coo_f32",
                 "fg_sddmm_coo_mh_f32", "fg_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol_and_binding_matches():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_symbols()
    for name in names:
        assert hasattr(handle, name), "%s is declared in the header but not exported" % name
    assert sorted(names) == sorted(_lib.SIGNATURES)


def test_no_internal_symbols_leak():
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], stdout=subprocess.PIPE, text=True).stdout
    exported = [l.split()[-1] for l in out.splitlines() if " T " in l]
    assert sorted(exported) == sorted(_declared_symbols())


def test_version_and_error_codes_without_a_device():
    L = _lib.lib()
    assert L.fg_version() >= 100
    plan = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(-1, 0, 0, None, None, ctypes.byref(plan)) == -1
    assert b"negative" in L.fg_last_error()
    assert L.fg_spmm_plan_create(1, 1, 0, None, None, ctypes.byref(plan)) == -1      # null indptr
    assert L.fg_spmm_plan_create(1, 1, 0, None, None, None) == -1                    # null result pointer
    assert L.fg_spmm_plan_create(2 ** 31, 1, 0, 8, None, ctypes.byref(plan)) == -4   # beyond int32 indexing
    assert L.fg_spmm_csr_f32(None, None, None, None, 4, 0, None) == -1               # null plan
    assert L.fg_sddmm_coo_f32(-5, None, None, None, None, None, 4, None) == -1
    assert L.fg_sddmm_coo_f32(10, None, None, None, None, None, 4, None) == -1       # null data
    assert L.fg_sddmm_coo_mh_f32(10, 8, 8, 8, 8, 8, 0, 4, None) == -1                # H = 0
    assert L.fg_sddmm_coo_f32(0, None, None, None, None, None, 4, None) == 0         # empty edge list is legal
    L.fg_spmm_plan_destroy(None)                                                     # no-op
    with pytest.raises(_lib.FeatGraphError) as err:
        _lib.check(L.fg_sddmm_coo_f32(-1, None, None, None, None, None, 4, None))
    assert err.value.code == -1


def test_config_store_round_trip():
    assert _lib.config_get("spmm.vec") == 0
    try:
        _lib.config_set("spmm.vec", 2)
        assert _lib.config_get("spmm.vec") == 2
        _lib.config_set("spmm.pipeline", 1)
        assert _lib.config_get("spmm.pipeline") == 1
        _lib.config_set("spmm.pipeline", -1)
        assert _lib.config_get("spmm.pipeline") == -1
        with pytest.raises(_lib.FeatGraphError):
            _lib.config_set("no.such.key", 1)
    finally:
        _lib.config_set("spmm.vec", 0)
        _lib.config_set("spmm.pipeline", -1)


def test_sddmm_launch_description_is_host_only():
    buf = ctypes.create_string_buffer(512)
    assert _lib.lib().fg_sddmm_describe(1000, 8, 16, buf, len(buf)) == 0
    text = buf.value.decode()
    assert "lanes/dot=4" in text and "H=8" in text
    assert _lib.lib().fg_sddmm_describe(1000, 1, 64, buf, len(buf)) == 0
    assert "lanes/dot=16" in buf.value.decode()


def test_error_codes_of_the_later_entry_points_without_a_device():
    L = _lib.lib()
    # generalised operators: bad codes and null plans are rejected before anything touches a device
    assert L.fg_spmm_csr_general_f32(None, None, None, None, 4, 0, 0, None) == -1
    assert L.fg_sddmm_coo_general_f32(4, 8, 8, 8, 8, 8, 4, 7, None) == -1                # no such edge function
    assert L.fg_sddmm_coo_general_f32(-1, 8, 8, 8, 8, 8, 4, 1, None) == -1
    assert L.fg_sddmm_coo_general_f32(0, None, None, None, None, None, 4, 2, None) == 0  # empty edge list
    assert L.fg_sddmm_coo_general_plan_f32(None, 8, 8, 8, 4, 1, None) == -1              # no plan
    # edge softmax
    assert L.fg_edge_softmax_csr_f32(-1, None, None, None, 8, None) == -1
    assert L.fg_edge_softmax_csr_f32(4, None, None, None, 8, None) == -1                 # null data
    assert L.fg_edge_softmax_csr_f32(4, 8, 8, 8, 0, None) == -1                          # H = 0
    assert L.fg_edge_softmax_csr_f32(0, None, None, None, 8, None) == 0
    assert L.fg_sddmm_softmax_plan_f32(None, None, None, None, 8, 64, None) == -1
    # allocation-free SpMM
    assert L.fg_spmm_csr_noalloc_f32((1 << 20) + 1, 8, 0, 8, None, None, None, 8, 4, None) == -4
    assert b"1048576" in L.fg_last_error()
    assert L.fg_spmm_csr_noalloc_f32(4, 4, 0, 8, None, None, None, 8, 0, None) == -1     # F = 0
    # feature rows at a pitch
    assert L.fg_spmm_csr_pitched_f32(None, 8, 128, 8, 8, 100, None) == -1                 # no plan
    assert L.fg_pad_rows_f32(4, 100, 96, 8, 8, None) == -1                                # pitch below F
    assert L.fg_pad_rows_f32(0, 100, 128, None, None, None) == 0
    assert L.fg_sddmm_coo_plan_pitched_f32(None, 8, 8, 128, 8, 100, None) == -1            # no plan
    # gather probes
    assert L.fg_probe_gather_f32(None, 4, 64, 64, 16384, 0, None, None) == -1
    assert L.fg_probe_gather_f32(8, 4, 60, 64, 16384, 0, 8, None) == -1                  # F not a multiple of the tile
    assert L.fg_probe_gather_count(4, 48, 16384, 10) == -1
    assert L.fg_probe_gather_count(232965, 64, 16384, 114606755) >= 100_000_000
    assert L.fg_probe_gather_rows_f32(8, 4, 100, 10, 8, None) == -1
    assert L.fg_probe_gather_rows_count(512, 61948164) >= 60_000_000
    assert L.fg_probe_gather_write_rows_f32(16, 4, 512, 10, 0, 16, 4, 16, None) == -1    # a write per 0 gathers
    assert L.fg_probe_gather_write_rows_f32(16, 4, 512, 10, 24, None, 4, 16, None) == -1  # no result matrix
    g, w = ctypes.c_int64(0), ctypes.c_int64(0)
    assert L.fg_probe_gather_write_rows_count(512, 61948164, 25, ctypes.byref(g), ctypes.byref(w)) == 0
    assert g.value >= 60_000_000 and 20 <= g.value / w.value <= 30                        # about one write per 25 gathers
    assert L.fg_probe_gather_write_rows_count(100, 10, 25, ctypes.byref(g), ctypes.byref(w)) == -1
    assert L.fg_attention_csr_mh_f32(None, None, None, None, None, 8, 64, None) == -1
    assert L.fg_probe_store_rows_f32(None, 4, 512, 10, None) == -1 and L.fg_probe_store_rows_f32(16, 4, 100, 10, None) == -1
    assert L.fg_probe_gather_stream_f32(None, 16384, 10, None, 0, 0, 0, None, None) == -1            # no matrix
    assert L.fg_probe_gather_stream_f32(16, 16384, 10, 16, 1 << 20, 3 << 16, 1, 16, None) == -1      # window not a power of two
    assert L.fg_probe_gather_stream_f32(16, 16384, 10, 16, 1 << 20, 1 << 16, 4, 16, None) == -1      # no such mode
