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
    # the entry points that pad BPE rows themselves and the measurement aids check their arguments first as well
    rc = L.dnatok_bpe_encode_padded(None, None, None, 1, 4, 4, None, 0, None, None, 0, 8, None, None, None, None, None)
    assert rc == -1 and b"null" in L.dnatok_last_error()
    rc = L.dnatok_diag_copy_tiles(None, None, 16, None)
    assert rc == -1 and b"null" in L.dnatok_last_error()
    rc = L.dnatok_diag_kmer_shape(None, None, 1, 8, 8, None, None, None)
    assert rc == -1
    assert L.dnatok_bpe_padded_direct_max() == 2048
