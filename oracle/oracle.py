"""numpy front end of the CPU oracle (oracle/dnatok_oracle.c).

TEST INFRASTRUCTURE ONLY: the checker the HIP path is compared against.  Only
tests/, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg may
import this module; the product package never does.

Besides the ctypes bindings it restates, independently of the product code,
the two table constructions the reference does on the host:

* ``kernel_vocab_from_merges``  -- ids 0..255 are the bytes, then for every merge
  line ``a b`` the strings ``a``, ``b``, ``a+b`` get the next free id in that
  order (reference: src/gputok_bpe_backend.py:358-393 and
  src/dnatok_bpe_kernel/dnatok_bpe.cu:761-791; the two agree).
* ``kmer_tables_from_vocab``    -- the 5**k window table with A0 C1 G2 T3 N4
  digits (reference: src/dna_tokenizer.py:743-822), filled from a vocabulary
  dictionary under the grid-aligned rule: a window of k ACGT bases is one
  token, any other window is spelled out character by character.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, List, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "dnatok_oracle.c")
_LIB = os.path.join(_HERE, "libdnatok_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(_SRC):
        subprocess.check_call(["gcc", "-O2", "-std=c11", "-shared", "-fPIC", "-o", _LIB, _SRC])
    return _LIB


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.oracle_bpe_table_create.restype = ctypes.c_void_p
        _lib.oracle_kmer_encode_row.restype = ctypes.c_int64
        _lib.oracle_bpe_encode_row.restype = ctypes.c_int64
        _lib.oracle_bpe_encode_row_naive.restype = ctypes.c_int64
    return _lib


def _p(a: np.ndarray):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


# ---------------------------------------------------------------- char

def char_encode_padded(lut, data: np.ndarray, offsets: np.ndarray, t_out: int, pad_id: int,
                       start_lut=None, pad_left: bool = False) -> Tuple[np.ndarray, np.ndarray]:
    lut = _i32(lut)
    start = _i32(start_lut) if start_lut is not None else None
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    b = offsets.size - 1
    ids = np.empty((b, t_out), dtype=np.int32)
    mask = np.empty((b, t_out), dtype=np.uint8)
    lib().oracle_char_encode_padded(_p(lut), _p(start), ctypes.c_int32(pad_id), _p(data),
                                    _p(offsets), ctypes.c_int64(b), ctypes.c_int64(t_out),
                                    ctypes.c_int(int(pad_left)), _p(ids), _p(mask))
    return ids, mask


def char_encode_packed(lut, data: np.ndarray) -> np.ndarray:
    lut = _i32(lut)
    ids = np.empty(data.size, dtype=np.int32)
    lib().oracle_char_encode_packed(_p(lut), _p(data), ctypes.c_int64(data.size), _p(ids))
    return ids


def clean_ascii(data: np.ndarray, upper_case: bool, invalid_to_n: bool) -> np.ndarray:
    """Upper-case a-z, then bytes outside ACGTN (ACGTNacgtn without upper-casing) -> 'N'
    (reference: src/dna_tokenizer.py:2637-2649).  Pinned by hand-written cases in
    tests/test_oracle.py."""
    arr = np.array(data, dtype=np.uint8, copy=True)
    if upper_case:
        lower = (arr >= ord("a")) & (arr <= ord("z"))
        arr[lower] -= 32
    if invalid_to_n:
        valid = np.frombuffer(b"ACGTN" if upper_case else b"ACGTNacgtn", dtype=np.uint8)
        arr[~np.isin(arr, valid)] = ord("N")
    return arr


def pack_2bit(ascii_rows: np.ndarray) -> np.ndarray:
    """uint8 [B, T] ASCII -> uint8 [B, ceil(T/4)], byte = c0 | c1<<2 | c2<<4 | c3<<6 with
    A C G T (either case) = 0 1 2 3, everything else 0, rows filled up with code 0
    (reference: src/dna_tokenizer.py:3129-3141, 3195-3209).  Pinned by known bytes
    ("ACGT" -> 0xE4, "TTTT" -> 0xFF, "CA" -> 0x01) and by the round trip through
    ``unpack_2bit_ids`` in tests/test_oracle.py."""
    code = np.zeros(256, dtype=np.uint8)
    for j, ch in enumerate("ACGT"):
        code[ord(ch)] = j
        code[ord(ch.lower())] = j
    b, t = ascii_rows.shape
    tp = (t + 3) // 4
    codes = np.zeros((b, tp * 4), dtype=np.uint8)
    codes[:, :t] = code[ascii_rows]
    c = codes.reshape(b, tp, 4)
    return (c[..., 0] | (c[..., 1] << 2) | (c[..., 2] << 4) | (c[..., 3] << 6)).astype(np.uint8)


def unpack_2bit_ids(lut, packed: np.ndarray, t_true: int, start_lut=None) -> np.ndarray:
    """Packed uint8 [B, ceil(T/4)] -> int64 ids [B, T]: lut["ACGT"[code]], column 0 from the
    start table (reference: src/dna_tokenizer.py:3232-3275)."""
    lut = np.asarray(lut)
    acgt = np.frombuffer(b"ACGT", dtype=np.uint8)
    b, tp = packed.shape
    codes = np.stack([(packed >> s) & 3 for s in (0, 2, 4, 6)], axis=2).reshape(b, tp * 4)[:, :t_true]
    ids = lut[acgt[codes]].astype(np.int64)
    if start_lut is not None and t_true > 0:
        ids[:, 0] = np.asarray(start_lut)[acgt[codes[:, 0]]]
    return ids


# --------------------------------------------------------------- k-mer

def base5_digits(fold_case: bool = False) -> np.ndarray:
    d = np.full(256, -1, dtype=np.int8)
    for i, c in enumerate("ACGTN"):
        d[ord(c)] = i
        if fold_case:
            d[ord(c.lower())] = i
    return d


class KmerTables:
    def __init__(self, k, digit, kmer_lut, exp_off, exp_len, exp_flat, single, missing_id):
        self.k = k
        self.digit = np.ascontiguousarray(digit, dtype=np.int8)
        self.kmer_lut = _i32(kmer_lut)
        self.exp_off = _i32(exp_off)
        self.exp_len = _i32(exp_len)
        self.exp_flat = _i32(exp_flat)
        self.single = _i32(single)
        self.missing_id = int(missing_id)


def kmer_tables_from_vocab(vocab: Dict[str, int], k: int, unk_id: int) -> KmerTables:
    n = 5 ** k
    kmer_lut = np.full(n, -1, dtype=np.int32)
    exp_off = np.zeros(n, dtype=np.int32)
    exp_len = np.zeros(n, dtype=np.int32)
    flat: List[int] = []
    single = np.full(256, unk_id, dtype=np.int32)
    for c in range(256):
        single[c] = vocab.get(chr(c), unk_id)
    alphabet = "ACGTN"
    for code in range(n):
        digits = []
        c = code
        for _ in range(k):
            digits.append(c % 5)
            c //= 5
        s = "".join(alphabet[d] for d in reversed(digits))
        if "N" not in s:
            kmer_lut[code] = vocab.get(s, unk_id)
        else:
            exp_off[code] = len(flat)
            exp_len[code] = k
            flat.extend(vocab.get(ch, unk_id) for ch in s)
    return KmerTables(k, base5_digits(), kmer_lut, exp_off, exp_len,
                      np.asarray(flat, dtype=np.int32), single, unk_id)


def kmer_encode(t: KmerTables, data: np.ndarray, offsets: np.ndarray
                ) -> Tuple[List[np.ndarray], np.ndarray]:
    """Per-row token arrays and per-row status bits (1 = byte outside ACGTN, 2 = no entry)."""
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    rows, status = [], np.zeros(offsets.size - 1, dtype=np.int32)
    for b in range(offsets.size - 1):
        row = np.ascontiguousarray(data[offsets[b]:offsets[b + 1]])
        out = np.empty(max(1, row.size), dtype=np.int32)
        st = ctypes.c_int32(0)
        n = lib().oracle_kmer_encode_row(
            ctypes.c_int(t.k), _p(t.digit), _p(t.kmer_lut), _p(t.exp_off), _p(t.exp_len),
            _p(t.exp_flat), _p(t.single), ctypes.c_int32(t.missing_id), _p(row),
            ctypes.c_int64(row.size), _p(out), ctypes.c_int64(out.size), ctypes.byref(st))
        rows.append(out[:n].copy())
        status[b] = st.value
    return rows, status


def kmer_encode_batch(t: KmerTables, data: np.ndarray, offsets: np.ndarray, t_cap: int,
                      pad_id: int) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Whole batch in one C call: padded ids [B, t_cap], mask, lengths."""
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    b = offsets.size - 1
    ids = np.empty((b, t_cap), dtype=np.int32)
    mask = np.empty((b, t_cap), dtype=np.uint8)
    lengths = np.empty(b, dtype=np.int32)
    lib().oracle_kmer_encode_batch(
        ctypes.c_int(t.k), _p(t.digit), _p(t.kmer_lut), _p(t.exp_off), _p(t.exp_len),
        _p(t.exp_flat), _p(t.single), ctypes.c_int32(t.missing_id), ctypes.c_int32(pad_id),
        _p(data), _p(offsets), ctypes.c_int64(b), ctypes.c_int64(t_cap), _p(ids), _p(mask),
        _p(lengths))
    return ids, mask, lengths


def pad_rows(rows: Sequence[np.ndarray], pad_id: int, t_out: int | None = None, *, pad_left: bool = False,
             min_width: int = 0, pad_multiple: int = 1, dtype=np.int32) -> Tuple[np.ndarray, np.ndarray]:
    """Pad to the longest row (or t_out): ids [B,T], mask uint8 [B,T].  Right padding:
    mask[b,j] = j < len_b (reference: src/gputok_bpe_backend.py:593-600).  pad_left, min_width
    (token_len) and pad_multiple as DNATok pads rows: a row's tokens end at the last column, the
    width is at least min_width and a multiple of pad_multiple (src/dna_tokenizer.py:1878-1894
    _pad_id_list, 2150-2236 encode_batch_with_padding); a row longer than the width keeps its
    first tokens."""
    t = max((r.size for r in rows), default=0) if t_out is None else t_out
    t = max(t, int(min_width))
    if pad_multiple > 1 and t % pad_multiple:
        t += pad_multiple - t % pad_multiple
    ids = np.full((len(rows), t), pad_id, dtype=dtype)
    mask = np.zeros((len(rows), t), dtype=np.uint8)
    for b, r in enumerate(rows):
        n = min(t, r.size)
        if pad_left:
            ids[b, t - n:] = r[:n]
            mask[b, t - n:] = 1
        else:
            ids[b, :n] = r[:n]
            mask[b, :n] = 1
    return ids, mask


# ----------------------------------------------------------------- BPE

def merges_from_tokenizer_json(cfg: dict) -> List[Tuple[str, str]]:
    out = []
    for m in cfg["model"]["merges"]:
        if isinstance(m, str):
            a, b = m.split(" ")
        else:
            a, b = m
        out.append((a, b))
    return out


def kernel_vocab_from_merges(merges: Sequence[Tuple[str, str]]
                             ) -> Tuple[List[str], np.ndarray, np.ndarray, np.ndarray]:
    """Kernel-space vocabulary and the (a, b, new) id triples in rank order."""
    vocab = [chr(b) for b in range(256)]
    index = {s: i for i, s in enumerate(vocab)}

    def add(s: str) -> int:
        i = index.get(s)
        if i is None:
            i = len(vocab)
            vocab.append(s)
            index[s] = i
        return i

    a_ids, b_ids, n_ids = [], [], []
    for a, b in merges:
        ia, ib = add(a), add(b)
        a_ids.append(ia)
        b_ids.append(ib)
        n_ids.append(add(a + b))
    return vocab, _i32(a_ids), _i32(b_ids), _i32(n_ids)


class BpeOracle:
    """Merge table in kernel id space plus the kernel-id -> HF-id map."""

    def __init__(self, merges: Sequence[Tuple[str, str]], hf_vocab: Dict[str, int] | None = None,
                 unk_id: int = 0):
        self.vocab, self.pair_a, self.pair_b, self.new_id = kernel_vocab_from_merges(merges)
        self.byte_to_id = np.arange(256, dtype=np.int32)
        self._t = ctypes.c_void_p(lib().oracle_bpe_table_create(
            _p(self.pair_a), _p(self.pair_b), _p(self.new_id), ctypes.c_int32(len(merges))))
        self.remap = None
        if hf_vocab is not None:
            self.remap = np.array([hf_vocab.get(s, unk_id) for s in self.vocab], dtype=np.int32)

    def __del__(self):
        try:
            lib().oracle_bpe_table_destroy(self._t)
        except Exception:
            pass

    def encode_row(self, row: np.ndarray, naive: bool = False, remap: bool = True) -> np.ndarray:
        row = np.ascontiguousarray(row, dtype=np.uint8)
        out = np.empty(max(1, row.size), dtype=np.int32)
        fn = lib().oracle_bpe_encode_row_naive if naive else lib().oracle_bpe_encode_row
        n = fn(self._t, _p(self.byte_to_id), _p(row), ctypes.c_int64(row.size), _p(out))
        out = out[:n]
        if remap and self.remap is not None:
            out = self.remap[out]
        return out.copy()

    def encode_batch(self, data: np.ndarray, offsets: np.ndarray, remap: bool = True
                     ) -> List[np.ndarray]:
        offsets = np.ascontiguousarray(offsets, dtype=np.int64)
        data = np.ascontiguousarray(data, dtype=np.uint8)
        b = offsets.size - 1
        tmp = np.empty(max(1, data.size), dtype=np.int32)
        lengths = np.empty(b, dtype=np.int32)
        lib().oracle_bpe_encode_batch(self._t, _p(self.byte_to_id), _p(data), _p(offsets),
                                      ctypes.c_int64(b), _p(tmp), _p(lengths))
        rows = []
        for i in range(b):
            r = tmp[offsets[i]:offsets[i] + lengths[i]]
            if remap and self.remap is not None:
                r = self.remap[r]
            rows.append(r.copy())
        return rows


def bpe_oracle_from_tokenizer_json(cfg: dict) -> BpeOracle:
    model = cfg["model"]
    unk = model.get("unk_token")
    vocab = model["vocab"]
    return BpeOracle(merges_from_tokenizer_json(cfg), vocab,
                     vocab.get(unk, 0) if unk is not None else 0)
