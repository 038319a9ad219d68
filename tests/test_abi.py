"""The C-ABI library loads and exports every symbol include/dnatok_hip.h declares.
No compute calls: this runs without a GPU."""
import ctypes
import os
import re

from dnatok_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "dnatok_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dnatok_[a-z0-9_]+)\s*\(", text)))


def test_header_and_loader_agree():
    assert declared_functions() == sorted(_lib.EXPORTS)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "build with: python -m dnatok_amd.build"
    L = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(L, name), name
    L.dnatok_version.restype = ctypes.c_int
    assert L.dnatok_version() == 100


def test_argument_errors_are_reported_without_a_gpu():
    L = _lib.lib()
    rc = L.dnatok_char_table_create(None, None, 0, None)
    assert rc == -1
    assert b"null" in L.dnatok_last_error()
    rc = L.dnatok_kmer_encode_padded(None, None, None, 1, 4, 8, None, None, None, None, None, None)
    assert rc == -1
    # the entry point that pads BPE rows itself checks its arguments first as well
    rc = L.dnatok_bpe_encode_padded(None, None, None, 1, 4, 4, None, 0, None, None, 0, 8, None, None, None, None, None)
    assert rc == -1 and b"null" in L.dnatok_last_error()
    assert L.dnatok_bpe_padded_direct_max(None) == 2048
    # the per-table test switches refuse a null table
    assert L.dnatok_kmer_table_set_team_rows(None, 0) == -1 and b"null" in L.dnatok_last_error()
    assert L.dnatok_bpe_table_set_chunk_geometry(None, 256, 32) == -1
    assert L.dnatok_bpe_table_set_placement(None, 0) == -1


def test_measurement_library_is_separate():
    """bench.py's memory-only kernels live in libdnatok_diag.so (include/dnatok_diag.h), not in the
    product library."""
    from dnatok_amd import build
    assert os.path.exists(build.DIAG_LIB_PATH), "build with: python -m dnatok_amd.build"
    D = ctypes.CDLL(build.DIAG_LIB_PATH)
    D.dnatok_last_error.restype = ctypes.c_char_p
    D.dnatok_diag_copy_tiles.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    assert D.dnatok_diag_copy_tiles(None, None, 16, None) == -1 and b"null" in D.dnatok_last_error()
    assert D.dnatok_diag_kmer_shape(None, None, 1, 8, 8, None, None, None) == -1
    P = ctypes.CDLL(_lib.LIB_PATH)
    assert not hasattr(P, "dnatok_diag_copy_tiles") and not hasattr(P, "dnatok_diag_kmer_shape")


def test_phase_cycle_counters_are_a_build_of_their_own():
    """The engine's per-phase cycle counters are compiled into libdnatok_hip_phases.so only
    (-DDNATOK_BPE_PHASE_CYCLES); that library carries the whole C ABI besides."""
    from dnatok_amd import build
    assert os.path.exists(build.PHASES_LIB_PATH), "build with: python -m dnatok_amd.build"
    Q = ctypes.CDLL(build.PHASES_LIB_PATH)
    assert hasattr(Q, "dnatok_bpe_phase_cycles")
    Q.dnatok_last_error.restype = ctypes.c_char_p
    assert Q.dnatok_bpe_phase_cycles(None, 0) == -1 and b"null" in Q.dnatok_last_error()
    for name in _lib.EXPORTS:
        assert hasattr(Q, name), name
    assert not hasattr(ctypes.CDLL(_lib.LIB_PATH), "dnatok_bpe_phase_cycles")
