"""Loads tests/golden/golden_vectors.npz and compares per-row id arrays against it.
Pure data comparison: imports neither the oracle nor the product."""
from __future__ import annotations

import hashlib
import os
from functools import lru_cache

import numpy as np

GOLDEN_DIR = os.path.dirname(os.path.abspath(__file__))


@lru_cache(maxsize=None)
def golden():
    return dict(np.load(os.path.join(GOLDEN_DIR, "golden_vectors.npz"), allow_pickle=False))


def sha_of_rows(rows) -> np.ndarray:
    flat = np.concatenate([np.asarray(r, dtype=np.int32) for r in rows]) if len(rows) else np.zeros(0, np.int32)
    return np.frombuffer(hashlib.sha256(flat.astype("<i4").tobytes()).digest(), dtype=np.uint8)


def check_against_golden(name: str, rows) -> None:
    g = golden()
    lengths = np.array([len(r) for r in rows], dtype=np.int32)
    np.testing.assert_array_equal(lengths, g[name + "_lengths"], err_msg=name + " lengths")
    np.testing.assert_array_equal(np.asarray(rows[0][:2048], dtype=np.int32), g[name + "_row0"],
                                  err_msg=name + " row 0")
    np.testing.assert_array_equal(sha_of_rows(rows), g[name + "_sha256"], err_msg=name + " sha256")
