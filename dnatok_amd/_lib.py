"""ctypes binding of libdnatok_hip.so (the C ABI declared in include/dnatok_hip.h).

The library is the only compute path: there is no CPU or torch fallback.  If the
shared object is missing, :func:`lib` raises with the build command.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdnatok_hip.so")

# every symbol include/dnatok_hip.h declares
EXPORTS = [
    "dnatok_version", "dnatok_last_error",
    "dnatok_char_table_create", "dnatok_char_table_destroy",
    "dnatok_char_encode_padded", "dnatok_char_encode_padded_as", "dnatok_char_encode_packed",
    "dnatok_char_embed_packed",
    "dnatok_char_unpack_2bit", "dnatok_host_clean_ascii", "dnatok_host_pack_2bit", "dnatok_host_fasta_scan",
    "dnatok_kmer_table_create", "dnatok_kmer_table_destroy", "dnatok_kmer_table_set_team_rows", "dnatok_kmer_encode_padded",
    "dnatok_kmer_encode_padded_sized", "dnatok_kmer_encode_packed",
    "dnatok_bpe_table_create", "dnatok_bpe_table_destroy", "dnatok_bpe_scratch_bytes",
    "dnatok_bpe_encode", "dnatok_bpe_encode_with_chars", "dnatok_bpe_encode_padded", "dnatok_bpe_encode_padded_as", "dnatok_bpe_padded_direct_max",
    "dnatok_bpe_static_scratch_bytes", "dnatok_bpe_encode_static",
    "dnatok_bpe_table_set_chunk_geometry", "dnatok_bpe_table_set_placement", "dnatok_pack_ragged", "dnatok_pad_rows", "dnatok_pad_rows_as",
    "dnatok_normalize_bounds", "dnatok_normalize_rows",
]


class NormStep(ctypes.Structure):
    """dnatok_norm_step of include/dnatok_hip.h."""
    _fields_ = [("kind", c_int32), ("flags", c_int32), ("pattern_len", c_int32), ("content_len", c_int32),
                ("pattern", ctypes.c_uint8 * 16), ("content", ctypes.c_uint8 * 16)]

    @classmethod
    def make(cls, kind: int, flags: int = 0, pattern: bytes = b"", content: bytes = b"") -> "NormStep":
        if len(pattern) > 16 or len(content) > 16:
            raise ValueError("normalizer pattern / content longer than 16 bytes")
        st = cls(kind, flags, len(pattern), len(content))
        for i, c in enumerate(pattern):
            st.pattern[i] = c
        for i, c in enumerate(content):
            st.content[i] = c
        return st


NORM_STRIP, NORM_REPLACE, NORM_REPLACE_RUN, NORM_PREPEND, NORM_LOWERCASE = 1, 2, 3, 4, 5


_lib = None


class DnatokError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise DnatokError(
            f"{LIB_PATH} is missing: build it with `python -m dnatok_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no fallback path.")
    # torch ships its own HIP runtime (soname libamdhip64.so.7); loading it first lets the
    # library's dependency resolve to that same copy instead of a second runtime from /opt/rocm,
    # which would not see the device torch's copy already holds.
    import torch  # noqa: F401
    L = ctypes.CDLL(LIB_PATH)
    L.dnatok_version.restype = c_int
    L.dnatok_last_error.restype = c_char_p
    L.dnatok_char_table_create.argtypes = [c_void_p, c_void_p, c_int32, POINTER(c_void_p)]
    L.dnatok_char_table_destroy.argtypes = [c_void_p]
    L.dnatok_char_table_destroy.restype = None
    L.dnatok_char_encode_padded.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int,
                                            c_void_p, c_void_p, c_void_p]
    L.dnatok_char_encode_padded_as.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int,
                                               c_void_p, c_int32, c_void_p, c_void_p]
    L.dnatok_char_encode_packed.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p,
                                            c_void_p, c_void_p]
    L.dnatok_char_embed_packed.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int32,
                                           c_int64, c_void_p, c_void_p]
    L.dnatok_char_unpack_2bit.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int32, c_void_p]
    L.dnatok_host_clean_ascii.argtypes = [c_void_p, c_int64, c_int, c_int, POINTER(c_int64)]
    L.dnatok_host_pack_2bit.argtypes = [c_void_p, c_int64, c_int64, c_void_p]
    L.dnatok_host_fasta_scan.argtypes = [c_void_p, c_int64, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                         POINTER(c_int64), POINTER(c_int64)]
    L.dnatok_kmer_table_create.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_int64, c_void_p, c_int32, c_int32, POINTER(c_void_p)]
    L.dnatok_kmer_table_destroy.argtypes = [c_void_p]
    L.dnatok_kmer_table_destroy.restype = None
    L.dnatok_kmer_table_set_team_rows.argtypes = [c_void_p, c_int32]
    L.dnatok_kmer_encode_padded.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    L.dnatok_kmer_encode_padded_sized.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                  c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    L.dnatok_kmer_encode_packed.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_void_p, c_void_p]
    L.dnatok_bpe_table_create.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                          c_void_p, POINTER(c_void_p)]
    L.dnatok_bpe_table_destroy.argtypes = [c_void_p]
    L.dnatok_bpe_table_destroy.restype = None
    L.dnatok_bpe_scratch_bytes.argtypes = [c_void_p, c_int64, c_int64, c_int64]
    L.dnatok_bpe_scratch_bytes.restype = c_size_t
    L.dnatok_bpe_encode.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                    c_void_p, c_size_t, c_void_p, c_void_p, c_void_p]
    L.dnatok_bpe_encode_with_chars.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                               c_void_p, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                               c_void_p]
    L.dnatok_bpe_encode_padded.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                           c_void_p, c_size_t, c_void_p, c_void_p, c_int32, c_int64,
                                           c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    L.dnatok_bpe_encode_padded_as.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                              c_void_p, c_size_t, c_void_p, c_void_p, c_int32, c_int64, c_int,
                                              c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]
    L.dnatok_bpe_padded_direct_max.argtypes = [c_void_p]
    L.dnatok_bpe_padded_direct_max.restype = c_int64
    L.dnatok_bpe_static_scratch_bytes.restype = c_size_t
    L.dnatok_bpe_encode_static.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                           c_void_p, c_void_p, c_void_p]
    L.dnatok_bpe_table_set_chunk_geometry.argtypes = [c_void_p, c_int32, c_int32]
    L.dnatok_bpe_table_set_placement.argtypes = [c_void_p, c_int32]
    L.dnatok_pack_ragged.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_void_p]
    L.dnatok_pad_rows.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int32, c_int64,
                                  c_int64, c_void_p, c_void_p, c_void_p, c_void_p]
    L.dnatok_pad_rows_as.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int32, c_int64, c_int64,
                                     c_int64, c_int64, c_int, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]
    L.dnatok_normalize_bounds.argtypes = [c_void_p, c_int32, c_int64, c_int64, c_int64, POINTER(c_int64),
                                          POINTER(c_int64), POINTER(c_size_t)]
    L.dnatok_normalize_rows.argtypes = [c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                        c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]
    for name in EXPORTS:
        getattr(L, name)          # AttributeError here means the library is stale
    _lib = L
    return L


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().dnatok_last_error()
        raise DnatokError(f"{what} failed ({rc}): {msg.decode(errors='replace') if msg else ''}")
