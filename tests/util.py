"""Shared helpers of the test suite: golden fixtures, oracle tables, HF tokenizers."""
from __future__ import annotations

import json
import os
from functools import lru_cache

import numpy as np

from tests.support import hf_tokenizers as hf
from tests.support import workloads as wl
from oracle import oracle as O

from tests.golden.check import GOLDEN_DIR, check_against_golden, golden, sha_of_rows  # noqa: F401


@lru_cache(maxsize=None)
def tokenizer_json(which: str) -> dict:
    with open(hf.bpe_tokenizer_path(which)) as fh:
        return json.load(fh)


@lru_cache(maxsize=None)
def bpe_oracle(which: str):
    return O.bpe_oracle_from_tokenizer_json(tokenizer_json(which))


@lru_cache(maxsize=None)
def kmer_oracle_tables():
    return O.kmer_tables_from_vocab(hf.kmer_vocab(6), 6, 0)


def char_lut(fold_case: bool = False) -> np.ndarray:
    """NTv3 rule: A T C G N keep their ids, everything else is <unk> (id 0)."""
    vocab = hf.char_vocab()
    lut = np.zeros(256, dtype=np.int32)
    for ch in "ACGTN":
        lut[ord(ch)] = vocab[ch]
        if fold_case:
            lut[ord(ch.lower())] = vocab[ch]
    return lut


def small_cases():
    from tests.golden.make_golden import SMALL_CASES
    return SMALL_CASES


def batch_from_strings(strings) -> wl.Batch:
    lens = np.array([len(s) for s in strings], dtype=np.int64)
    off = np.zeros(len(strings) + 1, dtype=np.int64)
    np.cumsum(lens, out=off[1:])
    data = np.frombuffer("".join(strings).encode("ascii"), dtype=np.uint8).copy()
    return wl.Batch(data, off)


def split_small(name: str):
    g = golden()
    lens = g[f"small_{name}_lengths"]
    ids = g[f"small_{name}_ids"]
    out, p = [], 0
    for n in lens:
        out.append(ids[p:p + n])
        p += n
    return out
