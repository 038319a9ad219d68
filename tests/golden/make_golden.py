"""Writes the golden fixtures under tests/golden/ with the Hugging Face `tokenizers` library.

    python tests/golden/make_golden.py train     # bpe4096_tokenizer.json, bpe32000_tokenizer.json
    python tests/golden/make_golden.py vectors   # golden_vectors.npz

`train` runs BpeTrainer on the seeded synthetic corpora (about 2 min and 6 min on 8 cores).
`vectors` encodes the five seeded benchmark inputs with the HF tokenizers
(add_special_tokens=False) and stores, per configuration and tokenizer: the per-row token
counts, a SHA-256 over all ids (int32 little endian, rows back to back), and the ids of the
first row (first 2048).  It also stores a few small hand-sized cases in full.  The inputs
are regenerated from their seeds by tests.support.workloads, so only outputs are stored.
"""
from __future__ import annotations

import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from tests.support import hf_tokenizers as hf   # noqa: E402
from tests.support import workloads as wl       # noqa: E402

SMALL_CASES = [
    "", "A", "N", "ACGT", "AAAAAAAAAAAAAAAAAAAAAAAAAAAAAAAAA", "ACACACACACACACACACACACACAC",
    "ACGTNNNNACGTACGTACGTAACCGGTTN", "TTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTTT",
    "GATTACAGATTACAGATTACAGATTACAGATTACAGATTACAGATTACA", "CGCGCGCGCGCGCGCGCGCGCGCGCGCGCGCGCGCGCGCG",
    "ACGTXACGTacgtACGT", "NACGTACGTACGTACGTACGTACGTACGTACGTACGTACGTACGTAC",
]


def train() -> None:
    for which in ("4096", "32000"):
        corp = wl.bpe_corpus(which)
        buf, line = corp.tobytes(), corp.shape[1]
        lines = (buf[i * line:(i + 1) * line].decode() for i in range(corp.shape[0]))
        tk = hf.train_bpe_tokenizer(lines, int(which), corp.shape[0])
        tk.save(hf.bpe_tokenizer_path(which), pretty=False)
        print(which, "vocab", tk.get_vocab_size(), flush=True)


def summarise(name: str, rows, out: dict) -> None:
    lengths = np.array([len(r) for r in rows], dtype=np.int32)
    flat = np.concatenate([np.asarray(r, dtype=np.int32) for r in rows]) if rows else np.zeros(0, np.int32)
    out[name + "_lengths"] = lengths
    out[name + "_sha256"] = np.frombuffer(hashlib.sha256(flat.astype("<i4").tobytes()).digest(), dtype=np.uint8)
    out[name + "_row0"] = np.asarray(rows[0][:2048], dtype=np.int32) if rows else np.zeros(0, np.int32)


def encode(tk, strings):
    return [e.ids for e in tk.encode_batch(strings, add_special_tokens=False)]


def vectors() -> None:
    out: dict = {}
    tk_char, tk_kmer = hf.build_char_tokenizer(), hf.build_kmer_tokenizer(6)
    tk4k, tk32k = hf.load_bpe_tokenizer("4096"), hf.load_bpe_tokenizer("32000")
    summarise("C1_char", encode(tk_char, wl.config1_char().strings()), out)
    summarise("C2_kmer", encode(tk_kmer, wl.config2_kmer().strings()), out)
    summarise("C3_bpe4096", encode(tk4k, wl.config3_bpe4096().strings()), out)
    summarise("C4_bpe32000", encode(tk32k, wl.config4_bpe32000().strings()), out)
    c5 = wl.config5_ragged().strings()
    summarise("C5_char", encode(tk_char, c5), out)
    summarise("C5_bpe4096", encode(tk4k, c5), out)
    for name, tk in (("char", tk_char), ("kmer", tk_kmer), ("bpe4096", tk4k), ("bpe32000", tk32k)):
        rows = encode(tk, SMALL_CASES)
        out[f"small_{name}_lengths"] = np.array([len(r) for r in rows], dtype=np.int32)
        out[f"small_{name}_ids"] = np.concatenate([np.asarray(r, dtype=np.int32) for r in rows])
    np.savez_compressed(os.path.join(HERE, "golden_vectors.npz"), **out)
    for k, v in out.items():
        if k.endswith("_lengths"):
            print(k, v.size, int(v.sum()))


if __name__ == "__main__":
    {"train": train, "vectors": vectors}[sys.argv[1]]()
