"""Times the Hugging Face `tokenizers` CPU tokenizer on one benchmark configuration.

Run as its own process (rayon sizes its thread pool once per process):

    RAYON_NUM_THREADS=N TOKENIZERS_PARALLELISM=true python -m tests.support.hf_baseline --config C2

Prints one JSON line: Mbp/s = input bases / median wall time / 1e6, the definition the
reference's CLI bench uses (src/dnatok_cli.py:272,299-301).  bytes -> str conversion
happens before the clock starts.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import time


def tokenizer_for(config: str):
    from . import hf_tokenizers as hf
    if config in ("C1", "C5char"):
        return hf.build_char_tokenizer()
    if config == "C2":
        return hf.build_kmer_tokenizer(6)
    if config in ("C3", "C5"):
        return hf.load_bpe_tokenizer("4096")
    if config == "C4":
        return hf.load_bpe_tokenizer("32000")
    raise ValueError(config)


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", required=True)
    ap.add_argument("--reps", type=int, default=3)
    ap.add_argument("--max-bases", type=int, default=0, help="truncate the batch to this many bases")
    ap.add_argument("--budget", type=float, default=20.0, help="seconds; stop repeating beyond it")
    a = ap.parse_args()
    from . import workloads as wl
    batch = wl.get("C5" if a.config == "C5char" else a.config)
    strings = batch.strings()
    if a.max_bases:
        keep, total = [], 0
        for s in strings:
            if total + len(s) > a.max_bases and keep:
                break
            keep.append(s)
            total += len(s)
        strings = keep
    n_bases = sum(len(s) for s in strings)
    tk = tokenizer_for(a.config)
    t_start = time.perf_counter()
    tk.encode_batch(strings[:max(1, len(strings) // 8)], add_special_tokens=False)   # warm-up
    times = []
    for _ in range(a.reps):
        t0 = time.perf_counter()
        tk.encode_batch(strings, add_special_tokens=False)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_start > a.budget:
            break
    med = statistics.median(times)
    print(json.dumps({"config": a.config, "mbp_per_s": n_bases / med / 1e6, "bases": n_bases,
                      "n_seqs": len(strings), "reps": len(times), "median_s": med,
                      "threads": os.environ.get("RAYON_NUM_THREADS", "default")}))


if __name__ == "__main__":
    main()
