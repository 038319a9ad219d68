"""Host-side BPE tables: merge list -> kernel id space -> arrays for dnatok_bpe_table_create.

Kernel id space (the one the reference's kernel and its Python glue agree on,
src/dnatok_bpe_kernel/dnatok_bpe.cu:761-791 and src/gputok_bpe_backend.py:358-393):
ids 0..255 are the byte symbols; then, walking the merge list in rank order,
``a``, ``b`` and ``a + b`` each take the next free id the first time they are seen.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Sequence, Tuple

import numpy as np


def parse_merges_txt(path: str) -> List[Tuple[str, str]]:
    """GPT-2 style merges file: the first line is always skipped, blank and '#'
    lines are skipped, every other line is a whitespace-separated pair
    (reference: src/dnatok_bpe_kernel/dnatok_bpe.cu:769-790)."""
    pairs: List[Tuple[str, str]] = []
    with open(path, "r", encoding="utf-8") as fh:
        lines = fh.read().split("\n")
    if not lines or (len(lines) == 1 and lines[0] == ""):
        raise ValueError(f"empty merges file: {path}")
    for line in lines[1:]:
        if not line or line[0] == "#":
            continue
        parts = line.split()
        if len(parts) >= 2:
            pairs.append((parts[0], parts[1]))
    return pairs


def split_merges(merges: Iterable) -> List[Tuple[str, str]]:
    """tokenizer.json stores merges as "a b" strings or [a, b] lists
    (reference: src/gputok_bpe_backend.py:251-262)."""
    out: List[Tuple[str, str]] = []
    for m in merges:
        if isinstance(m, str):
            parts = m.split()
            if len(parts) != 2:
                continue
            out.append((parts[0], parts[1]))
        elif isinstance(m, (list, tuple)) and len(m) == 2:
            out.append((str(m[0]), str(m[1])))
        else:
            raise ValueError(f"Unrecognised merge entry: {m!r}")
    return out


class KernelVocab:
    """Kernel-space vocabulary plus the (a, b, new) triples of every merge rule."""

    def __init__(self, merges: Sequence[Tuple[str, str]]):
        self.id_to_token: List[str] = [chr(b) for b in range(256)]
        self.token_to_id: Dict[str, int] = {t: i for i, t in enumerate(self.id_to_token)}
        n = len(merges)
        self.pair_a = np.empty(n, dtype=np.int32)
        self.pair_b = np.empty(n, dtype=np.int32)
        self.new_id = np.empty(n, dtype=np.int32)
        for rank, (a, b) in enumerate(merges):
            self.pair_a[rank] = self._intern(a)
            self.pair_b[rank] = self._intern(b)
            self.new_id[rank] = self._intern(a + b)

    def _intern(self, tok: str) -> int:
        idx = self.token_to_id.get(tok)
        if idx is None:
            idx = len(self.id_to_token)
            self.id_to_token.append(tok)
            self.token_to_id[tok] = idx
        return idx

    def __len__(self) -> int:
        return len(self.id_to_token)

    def remap_to(self, hf_vocab: Dict[str, int], unk_id: int) -> np.ndarray:
        """kernel id -> HF id; tokens the HF vocabulary lacks map to unk_id
        (reference: src/gputok_bpe_backend.py:451-466)."""
        out = np.full(len(self.id_to_token), int(unk_id), dtype=np.int32)
        for kid, tok in enumerate(self.id_to_token):
            hid = hf_vocab.get(tok)
            if isinstance(hid, int):
                out[kid] = hid
        return out
