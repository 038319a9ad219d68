"""Seeded synthetic DNA workloads for the five benchmark configurations.

Every generator draws from ``numpy.random.Generator(PCG64(seed))`` only, so the
same seed gives the same bytes on every machine.  All sequences are returned as
uint8 ASCII (``A C G T N``) in one flat buffer plus an int64 ``offsets[B+1]``
array -- the layout the encode kernels consume.

Workloads
---------
C1  char      64 x 8192 bp, i.i.d. uniform ACGT, each base -> N with p = 0.001
C2  6-mer     256 x 6000 bp, uniform ACGT, N in runs of 1..50 bp (~0.5 % of bases)
C3  BPE-4096  1024 x 1024 bp from an order-2 Markov chain with 41 % GC
C4  BPE-32000 32 x 100 kbp from an order-3 Markov chain, 10 % of bases inside
              tandem repeats (homopolymers 5-40 bp, 2-6 bp units x 5-30 copies)
C5  ragged    4096 sequences, lognormal lengths (median 2 kbp, clipped to
              100..131072 bp, ~12 Mbp), 0.2 % N, bases from the C3 chain

The composition (A/T 0.295, C/G 0.205) follows the "human GC41" weights of the
reference's workload generator (benchmarks/run_realistic_benchmark.py:88).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Tuple

import numpy as np

BASES = np.frombuffer(b"ACGT", dtype=np.uint8)
N_BYTE = ord("N")
BASE_COMPOSITION = np.array([0.295, 0.205, 0.205, 0.295])  # A C G T

SEEDS = {"C1": 1001, "C2": 1002, "C3": 1003, "C4": 1004, "C5": 1005,
         "corpus4096": 2003, "corpus32000": 2004,
         "chain2": 3002, "chain3": 3003}


@dataclass
class Batch:
    """A ragged batch: ``data[offsets[b]:offsets[b+1]]`` is sequence ``b``."""
    data: np.ndarray      # uint8 [total]
    offsets: np.ndarray   # int64 [B+1]

    @property
    def n_seqs(self) -> int:
        return int(self.offsets.size - 1)

    @property
    def total(self) -> int:
        return int(self.offsets[-1])

    def row(self, b: int) -> np.ndarray:
        return self.data[self.offsets[b]:self.offsets[b + 1]]

    def strings(self) -> List[str]:
        buf = self.data.tobytes()
        o = self.offsets
        return [buf[o[b]:o[b + 1]].decode("ascii") for b in range(self.n_seqs)]

    def lengths(self) -> np.ndarray:
        return np.diff(self.offsets)


def _dense(arr2d: np.ndarray) -> Batch:
    b, t = arr2d.shape
    return Batch(np.ascontiguousarray(arr2d).reshape(-1),
                 np.arange(b + 1, dtype=np.int64) * t)


# --------------------------------------------------------------------------
# Markov chains
# --------------------------------------------------------------------------

def markov_cdf(order: int, seed: int, concentration: float = 24.0) -> np.ndarray:
    """Cumulative transition table ``cdf[4**order, 4]`` of a seeded chain.

    Each context row is a Dirichlet draw centred on BASE_COMPOSITION, so the
    stationary GC content stays close to 41 %.
    """
    rng = np.random.Generator(np.random.PCG64(seed))
    p = rng.dirichlet(BASE_COMPOSITION * concentration, size=4 ** order)
    cdf = np.cumsum(p, axis=1)
    cdf[:, -1] = 1.0
    return cdf


def markov_matrix(rng: np.random.Generator, cdf: np.ndarray, n_rows: int,
                  length: int) -> np.ndarray:
    """Equal-length chain realisations as a dense code matrix [n_rows, length] (0..3)."""
    n_ctx = cdf.shape[0]
    ctx = rng.integers(0, n_ctx, size=n_rows)
    out = np.empty((length, n_rows), dtype=np.uint8)
    block = 256
    for t0 in range(0, length, block):
        t1 = min(length, t0 + block)
        u = rng.random((t1 - t0, n_rows))
        for t in range(t0, t1):
            row_cdf = cdf[ctx]
            nxt = (u[t - t0, :, None] > row_cdf[:, :3]).sum(axis=1).astype(np.int64)
            out[t] = nxt
            ctx = (ctx * 4 + nxt) % n_ctx
    return np.ascontiguousarray(out.T)


def place_tandem_repeats(rng: np.random.Generator, codes: np.ndarray,
                         fraction: float = 0.10) -> np.ndarray:
    """Overwrite ~``fraction`` of each row with tandem repeats, in place.

    Half of the events are homopolymers of 5..40 bp, half are microsatellites
    (unit 2..6 bp, 5..30 copies).  Mean event length is about 46 bp.
    """
    n_rows, length = codes.shape
    mean_len = 0.5 * 22.5 + 0.5 * (4.0 * 17.5)
    n_events = rng.poisson(fraction * length / mean_len, size=n_rows)
    for r in range(n_rows):
        for _ in range(int(n_events[r])):
            if rng.random() < 0.5:
                unit = rng.integers(0, 4, size=1)
                total = int(rng.integers(5, 41))
            else:
                unit = rng.integers(0, 4, size=int(rng.integers(2, 7)))
                total = int(unit.size * rng.integers(5, 31))
            total = min(total, length)
            start = int(rng.integers(0, length - total + 1))
            reps = -(-total // unit.size)
            codes[r, start:start + total] = np.tile(unit, reps)[:total]
    return codes


# --------------------------------------------------------------------------
# The five configurations
# --------------------------------------------------------------------------

def config1_char(n_rows: int = 64, length: int = 8192, seed: int = SEEDS["C1"],
                 n_rate: float = 0.001) -> Batch:
    rng = np.random.Generator(np.random.PCG64(seed))
    arr = BASES[rng.integers(0, 4, size=(n_rows, length), dtype=np.uint8)]
    arr[rng.random((n_rows, length)) < n_rate] = N_BYTE
    return _dense(arr)


def config2_kmer(n_rows: int = 256, length: int = 6000, seed: int = SEEDS["C2"],
                 n_fraction: float = 0.005) -> Batch:
    rng = np.random.Generator(np.random.PCG64(seed))
    arr = BASES[rng.integers(0, 4, size=(n_rows, length), dtype=np.uint8)]
    # run starts are Bernoulli with rate n_fraction / mean_run (mean run = 25.5 bp)
    starts = rng.random((n_rows, length)) < (n_fraction / 25.5)
    rr, cc = np.nonzero(starts)
    run = rng.integers(1, 51, size=rr.size)
    for r, c, ln in zip(rr.tolist(), cc.tolist(), run.tolist()):
        arr[r, c:c + ln] = N_BYTE
    return _dense(arr)


def bpe_corpus(which: str, n_bases: int | None = None, line: int = 1024) -> np.ndarray:
    """Training corpus as a dense ASCII matrix [n_lines, line].

    ``which`` = "4096": 50 Mbp of the order-2 chain; "32000": 200 Mbp of the
    order-3 chain with 10 % tandem repeats.
    """
    if which == "4096":
        n_bases = n_bases or 50_000_000
        rng = np.random.Generator(np.random.PCG64(SEEDS["corpus4096"]))
        cdf = markov_cdf(2, SEEDS["chain2"])
        codes = markov_matrix(rng, cdf, n_bases // line, line)
    elif which == "32000":
        n_bases = n_bases or 200_000_000
        rng = np.random.Generator(np.random.PCG64(SEEDS["corpus32000"]))
        cdf = markov_cdf(3, SEEDS["chain3"])
        codes = markov_matrix(rng, cdf, n_bases // line, line)
        place_tandem_repeats(rng, codes, 0.10)
    else:
        raise ValueError(which)
    return BASES[codes]


def config3_bpe4096(n_rows: int = 1024, length: int = 1024, seed: int = SEEDS["C3"]) -> Batch:
    rng = np.random.Generator(np.random.PCG64(seed))
    cdf = markov_cdf(2, SEEDS["chain2"])
    return _dense(BASES[markov_matrix(rng, cdf, n_rows, length)])


def config4_bpe32000(n_rows: int = 32, length: int = 100_000, seed: int = SEEDS["C4"]) -> Batch:
    rng = np.random.Generator(np.random.PCG64(seed))
    cdf = markov_cdf(3, SEEDS["chain3"])
    codes = markov_matrix(rng, cdf, n_rows, length)
    place_tandem_repeats(rng, codes, 0.10)
    return _dense(BASES[codes])


def config5_lengths(n_seqs: int = 4096, seed: int = SEEDS["C5"]) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    ln = np.rint(rng.lognormal(np.log(2000.0), 0.87, size=n_seqs)).astype(np.int64)
    return np.clip(ln, 100, 131072)


def config5_ragged(n_seqs: int = 4096, seed: int = SEEDS["C5"], n_rate: float = 0.002) -> Batch:
    lengths = config5_lengths(n_seqs, seed)
    offsets = np.zeros(n_seqs + 1, dtype=np.int64)
    np.cumsum(lengths, out=offsets[1:])
    total = int(offsets[-1])
    rng = np.random.Generator(np.random.PCG64(seed + 7919))
    cdf = markov_cdf(2, SEEDS["chain2"])
    # one pool of chain output (2048 parallel realisations laid end to end), cut into reads
    lanes = 2048
    pool = markov_matrix(rng, cdf, lanes, -(-total // lanes)).reshape(-1)[:total]
    data = BASES[pool]
    data[rng.random(total) < n_rate] = N_BYTE
    return Batch(data, offsets)


def describe(batch: Batch) -> dict:
    """Composition summary recorded next to every measurement."""
    import hashlib
    d = batch.data
    counts = np.bincount(d, minlength=256)
    acgt = counts[ord("A")] + counts[ord("C")] + counts[ord("G")] + counts[ord("T")]
    ln = batch.lengths()
    return {
        "n_seqs": batch.n_seqs, "total_bp": batch.total,
        "gc": float((counts[ord("C")] + counts[ord("G")]) / max(1, acgt)),
        "n_frac": float(counts[N_BYTE] / max(1, d.size)),
        "len_min": int(ln.min()) if ln.size else 0, "len_max": int(ln.max()) if ln.size else 0,
        "sha256": hashlib.sha256(d.tobytes() + batch.offsets.tobytes()).hexdigest(),
    }


def get(name: str) -> Batch:
    return {"C1": config1_char, "C2": config2_kmer, "C3": config3_bpe4096,
            "C4": config4_bpe32000, "C5": config5_ragged}[name]()
