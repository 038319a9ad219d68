"""Host-side k-mer tables in the layout of the reference's ``DNATok._build_kmer_lut``
(src/dna_tokenizer.py:743-822): a 5**k window table over the digits A0 C1 G2 T3 N4
holding a single token id or -1, and for -1 entries an (offset, length) into a
flat list of the window's own tokens."""
from __future__ import annotations

from typing import Callable, Dict, List, Optional, Sequence

import numpy as np

ALPHABET = "ACGTN"


def digit_table(fold_case: bool = False) -> np.ndarray:
    d = np.full(256, -1, dtype=np.int8)
    for i, ch in enumerate(ALPHABET):
        d[ord(ch)] = i
        if fold_case:
            d[ord(ch.lower())] = i
    return d


def window_string(code: int, k: int) -> str:
    chars = []
    for _ in range(k):
        chars.append(ALPHABET[code % 5])
        code //= 5
    return "".join(reversed(chars))


class KmerTables:
    def __init__(self, k: int):
        self.k = k
        n = 5 ** k
        self.digit = digit_table()
        self.kmer_lut = np.full(n, -1, dtype=np.int32)
        self.exp_off = np.zeros(n, dtype=np.int32)
        self.exp_len = np.zeros(n, dtype=np.int32)
        self.exp_flat = np.zeros(0, dtype=np.int32)
        self.single = np.zeros(256, dtype=np.int32)


def tables_from_tokenize(tokenize_batch: Callable[[List[str]], Sequence[Sequence[int]]], k: int,
                         unk_id: int, batch: int = 4096) -> KmerTables:
    """Probe a tokenizer with every window over ACGTN (batches of 4096, as the reference does):
    one token -> kmer_lut, several -> expansion list, none -> stays -1 without expansion."""
    t = KmerTables(k)
    n = 5 ** k
    flat: List[int] = []
    for s0 in range(0, n, batch):
        codes = list(range(s0, min(n, s0 + batch)))
        outs = tokenize_batch([window_string(c, k) for c in codes])
        for c, ids in zip(codes, outs):
            ids = list(ids)
            if len(ids) == 1:
                t.kmer_lut[c] = ids[0]
            elif len(ids) > 1:
                t.exp_off[c] = len(flat)
                t.exp_len[c] = len(ids)
                flat.extend(int(x) for x in ids)
    t.exp_flat = np.asarray(flat, dtype=np.int32)
    singles = tokenize_batch([chr(b) if 32 <= b < 127 else "N" for b in range(256)])
    for b in range(256):
        ids = list(singles[b])
        t.single[b] = ids[0] if (len(ids) == 1 and 32 <= b < 127) else unk_id
    return t


def tables_from_vocab(vocab: Dict[str, int], k: int, unk_id: int) -> KmerTables:
    """Grid-aligned tables straight from a vocabulary: a window of k ACGT bases is its own
    token, any other window is spelled character by character."""
    def tok(batch: List[str]):
        out = []
        for s in batch:
            if len(s) == k and all(ch in "ACGT" for ch in s):
                out.append([vocab.get(s, unk_id)])
            else:
                out.append([vocab.get(ch, unk_id) for ch in s])
        return out
    return tables_from_tokenize(tok, k, unk_id)
