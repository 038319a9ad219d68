"""``python -m dnatok_amd.dnatok_cli``: info / encode / validate / bench from a shell.

The four commands of the reference's command line (src/dnatok_cli.py:162-307) with the same
options and the same output fields (plus ``encode --fasta FILE``).  ``--model`` names a tokenizer that can be had without a
network: a directory or ``tokenizer.json`` on disk (loaded with ``tokenizers.Tokenizer.from_file``
and, for directories, ``transformers.AutoTokenizer`` when that works offline), or one of the
built-in synthetic tokenizers of the benchmark configurations:

    char      single nucleotides, NTv3 vocabulary order     (kernel: char)
    ntv3      the NTv3 compat tokenizer class                (kernel: char)
    evo2      byte-level ids, id = ord(c)                    (kernel: char)
    kmer6     non-overlapping 6-mers, grid-aligned fallback  (kernel: k-mer)

A BPE tokenizer is named by the path of its ``tokenizer.json`` (kernel: BPE engine).

All encoding runs on the GPU through libdnatok_hip.so; the reference tokenizer it is compared
with runs on the host.
"""
from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time
from typing import Any, List, Optional, Tuple

BUILTIN = ("char", "ntv3", "evo2", "kmer6")


class _TokenizerCall:
    """``tokenizers.Tokenizer`` behind the call style DNATok probes (``tok(texts, ...)``)."""

    def __init__(self, tk, pad_id: int = 0, padding_side: str = "right"):
        self.backend_tokenizer = tk
        self._tk = tk
        self.pad_token_id = pad_id
        self.padding_side = padding_side
        self.vocab_size = tk.get_vocab_size()

    def get_vocab(self):
        return self._tk.get_vocab()

    def to_str(self):
        return self._tk.to_str()

    def __call__(self, texts, add_special_tokens=False, **_):
        single = isinstance(texts, str)
        rows = [e.ids for e in self._tk.encode_batch([texts] if single else list(texts),
                                                     add_special_tokens=add_special_tokens)]
        return {"input_ids": rows[0] if single else rows}


def _load_tokenizer(model: str):
    from . import builtin_tokenizers as hf, dnatok_compat
    if model == "char":
        return _TokenizerCall(hf.build_char_tokenizer(), pad_id=hf.char_vocab()["<pad>"])
    if model == "ntv3":
        return dnatok_compat.NTv3Tokenizer()
    if model == "evo2":
        return dnatok_compat.Evo2ByteTokenizer()
    if model == "kmer6":
        return _TokenizerCall(hf.build_kmer_tokenizer(6), pad_id=hf.kmer_vocab(6)["<pad>"])
    path = model
    if os.path.isdir(path):
        try:
            os.environ.setdefault("HF_HUB_OFFLINE", "1")
            from transformers import AutoTokenizer
            return AutoTokenizer.from_pretrained(path, local_files_only=True)
        except Exception:
            path = os.path.join(path, "tokenizer.json")
    if os.path.isfile(path):
        from tokenizers import Tokenizer
        tk = Tokenizer.from_file(path)
        pad = tk.padding["pad_id"] if tk.padding else (tk.token_to_id("[PAD]") or tk.token_to_id("<pad>") or 0)
        return _TokenizerCall(tk, pad_id=int(pad))
    raise SystemExit(f"--model {model!r}: not a built-in name ({', '.join(BUILTIN)}) and not a path on disk")


def _build_dnatok(model: str, device: str):
    import torch
    from .dna_tokenizer import DNATok
    tok = _load_tokenizer(model)

    class _Embedder:
        def __init__(self, t):
            self.tokenizer = t
            size = getattr(t, "vocab_size", 0)
            size = int(size) if isinstance(size, int) and size else len(t.get_vocab())
            self.embed_table = torch.nn.Embedding(size + 4, 16).to(device)

        def embed_tokens(self, ids):
            return self.embed_table(ids)

    dn = DNATok(_Embedder(tok), normalize_case=False, handle_invalid_chars=False)
    dn.discover()
    return tok, dn


def _detect_path(dn) -> str:
    if getattr(dn, "kmer_k", None) is not None:
        return f"kmer-{dn.kmer_k}"
    if getattr(dn, "bpe_backend", None) is not None:
        return "gpu-bpe-kernel"
    if getattr(dn, "ascii_lut", None) is not None and dn.use_ids_path:
        return "ascii-lut"
    return "hf-fallback"


def _default_device() -> str:
    import torch
    return "cuda" if torch.cuda.is_available() else "cpu"


def _emit(payload: Any, as_json: bool) -> None:
    if as_json:
        json.dump(payload, sys.stdout, indent=2)
        print()
    elif isinstance(payload, dict):
        width = max(map(len, payload)) if payload else 0
        for k, v in payload.items():
            print(f"  {k:<{width}}  {v}")
    else:
        print(payload)


def _strip_pad(row: List[int], pad: int, side: str) -> List[int]:
    if side == "left":
        j = 0
        while j < len(row) and row[j] == pad:
            j += 1
        return row[j:]
    j = len(row)
    while j > 0 and row[j - 1] == pad:
        j -= 1
    return row[:j]


def _hf_ids(tok, seqs: List[str]) -> List[List[int]]:
    out = tok(seqs, add_special_tokens=False, padding=False, truncation=False, return_tensors=None)
    rows = out["input_ids"]
    return [r.tolist() if hasattr(r, "tolist") else list(r) for r in rows]


def cmd_info(args) -> int:
    device = args.device or _default_device()
    tok, dn = _build_dnatok(args.model, device)
    size = getattr(tok, "vocab_size", 0)
    _emit({
        "model": args.model,
        "tokenizer_class": type(tok).__name__,
        "vocab_size": int(size) if isinstance(size, int) and size else len(tok.get_vocab()),
        "selected_path": _detect_path(dn),
        "device": device,
        "kmer_k": dn.kmer_k,
        "has_ascii_lut": dn.ascii_lut is not None,
        "has_gpu_bpe_backend": dn.bpe_backend is not None,
        "has_cached_lmm": dn.lmm_bpe is not None,
        "padding_side": dn.padding_side,
        "id_pad": int(dn.id_pad),
    }, args.json)
    return 0


def cmd_encode(args) -> int:
    device = args.device or _default_device()
    _, dn = _build_dnatok(args.model, device)
    if args.fasta:
        # every record of a FASTA file (not in the reference's command line, which takes --seq only)
        ids, mask, names = dn.encode_fasta_device(args.fasta, device=device)
        counts = mask.sum(dim=1).tolist()
        _emit({
            "model": args.model,
            "fasta": args.fasta,
            "n_records": len(names),
            "n_tokens_total": int(sum(counts)),
            "records": [{"name": n, "n_tokens": int(c)} for n, c in zip(names, counts)][: None if args.json else 8],
            "selected_path": _detect_path(dn),
        }, args.json)
        return 0
    if not args.seq:
        raise SystemExit("encode: give --seq or --fasta")
    ids = _strip_pad(dn.encode_batch_to_ids([args.seq])[0].tolist(), int(dn.id_pad), dn.padding_side)
    _emit({
        "model": args.model,
        "sequence": args.seq[:80] + ("..." if len(args.seq) > 80 else ""),
        "sequence_length_bp": len(args.seq),
        "n_tokens": len(ids),
        "token_ids": ids if args.json else ids[:32] + (["..."] if len(ids) > 32 else []),
        "selected_path": _detect_path(dn),
    }, args.json)
    return 0


def cmd_validate(args) -> int:
    """Bit identity with the tokenizer itself on n random ACGT sequences of one length."""
    device = args.device or _default_device()
    tok, dn = _build_dnatok(args.model, device)
    rng = random.Random(args.seed)
    seqs = ["".join(rng.choices("ACGT", k=args.window)) for _ in range(args.n)]
    ours = dn.encode_batch_to_ids(seqs).cpu().tolist()
    theirs = _hf_ids(tok, seqs)
    pad = int(dn.id_pad)
    n_match, first = 0, None
    for i, s in enumerate(seqs):
        row = _strip_pad(ours[i], pad, dn.padding_side)
        if row == list(theirs[i]):
            n_match += 1
        elif first is None:
            first = {"i": i, "seq_head": s[:40], "dnatok_head": row[:8], "hf_head": list(theirs[i])[:8]}
    _emit({
        "model": args.model,
        "n_sequences": args.n,
        "n_match": n_match,
        "n_mismatch": args.n - n_match,
        "match_rate": n_match / max(args.n, 1),
        "selected_path": _detect_path(dn),
        "first_mismatch": first,
    }, args.json)
    return 0 if n_match == args.n else 1


def cmd_bench(args) -> int:
    """Strings in, ids out, chunk by chunk: this backend beside the tokenizer on the host."""
    device = args.device or _default_device()
    os.environ["RAYON_NUM_THREADS"] = str(args.hf_threads)
    os.environ["TOKENIZERS_PARALLELISM"] = "true" if args.hf_threads > 1 else "false"
    tok, dn = _build_dnatok(args.model, device)
    rng = random.Random(args.seed)
    seqs = ["".join(rng.choices("ACGT", k=args.window)) for _ in range(args.n)]
    bp_total = sum(map(len, seqs))
    tok(seqs[:min(args.chunk, args.n)], add_special_tokens=False)
    dn.encode_batch_to_ids(seqs[:min(args.chunk, args.n)])
    t0 = time.perf_counter()
    for i in range(0, args.n, args.chunk):
        tok(seqs[i:i + args.chunk], add_special_tokens=False)
    t_hf = time.perf_counter() - t0
    import torch
    if device == "cuda":
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(0, args.n, args.chunk):
        dn.encode_batch_to_ids(seqs[i:i + args.chunk])
    if device == "cuda":
        torch.cuda.synchronize()
    t_dn = time.perf_counter() - t0
    _emit({
        "model": args.model,
        "n_sequences": args.n,
        "window_bp": args.window,
        "chunk": args.chunk,
        "total_bp": bp_total,
        "hf_threads": args.hf_threads,
        "hf_time_s": round(t_hf, 4),
        "hf_mbp_per_s": round(bp_total / t_hf / 1e6, 2),
        "dnatok_time_s": round(t_dn, 4),
        "dnatok_mbp_per_s": round(bp_total / t_dn / 1e6, 2),
        "speedup_dnatok_vs_hf": round(t_hf / t_dn, 2),
        "selected_path": _detect_path(dn),
        "device": device,
    }, args.json)
    return 0


def cmd_demo(args) -> int:
    """info, encode of a sample, bit identity on 50 short sequences, a small benchmark: the
    reference's end-to-end run (src/dnatok_cli.py:310-348) over a model this build can load."""
    print("=" * 70)
    print(f"dnatok demo: model={args.model}")
    print("=" * 70)
    args.json = False
    print("\n[1/4] tokenizer info")
    cmd_info(args)
    print("\n[2/4] encode a sample sequence")
    args.seq, args.fasta = args.sample or "ACGT" * 15, None
    cmd_encode(args)
    print("\n[3/4] bit identity with the tokenizer (n=50, random ACGT sequences, 256 bp)")
    args.n, args.window, args.seed = 50, 256, 42
    rc = cmd_validate(args)
    if rc != 0:
        print("  bit identity FAILED: see first_mismatch above")
        return rc
    print("  bit identity holds")
    print("\n[4/4] small benchmark (n=100, 1024 bp, 32 per call, 4 host threads)")
    args.n, args.window, args.chunk, args.hf_threads, args.seed = 100, 1024, 32, 4, 11
    return cmd_bench(args)


# What --model accepts.  The reference's registry (src/dnatok_cli.py:55-76) names models on the
# Hugging Face hub; nothing is downloaded here, so the registry names what is built in and what a
# local path may be.
MODEL_REGISTRY = {
    "char": ("char", "built in", "single-nucleotide ids A C G T N + specials (vocab 11): byte table kernel"),
    "ntv3": ("ntv3", "built in", "NTv3 single-nucleotide vocabulary (dnatok_compat.NTv3Tokenizer): byte table kernel"),
    "evo2": ("evo2", "built in", "Evo2 byte tokenizer, id = byte (dnatok_compat.Evo2ByteTokenizer): byte table kernel"),
    "kmer6": ("kmer6", "built in", "non-overlapping 6-mers, windows with N spelled per character (vocab 4101): k-mer kernel"),
    "bpe": ("<path>/tokenizer.json", "local file", "Hugging Face BPE tokenizer (DNABERT-2, GENA-LM, METAGENE-1 style files): "
            "BPE engine when GPUTokBPEBackend.is_supported accepts it, else the tokenizer itself"),
}


def cmd_list_models(args) -> int:
    rows = [{"family": fam, "model": model, "source": source, "notes": notes}
            for fam, (model, source, notes) in MODEL_REGISTRY.items()]
    if args.json:
        json.dump(rows, sys.stdout, indent=2)
        print()
        return 0
    widths = {k: max(len(k), max(len(str(r[k])) for r in rows)) for k in rows[0]}
    print("  " + "  ".join(k.ljust(widths[k]) for k in rows[0]))
    print("  " + "  ".join("-" * widths[k] for k in rows[0]))
    for r in rows:
        print("  " + "  ".join(str(r[k]).ljust(widths[k]) for k in rows[0]))
    return 0


def main(argv: Optional[list] = None) -> int:
    ap = argparse.ArgumentParser(prog="dnatok", description="DNA tokenization on the MI355X backend")
    sub = ap.add_subparsers(dest="cmd", required=True)

    def common(p):
        p.add_argument("--model", required=True, help="built-in name (%s) or a tokenizer path" % ", ".join(BUILTIN))
        p.add_argument("--device", default=None, help="cuda (default when a GPU is present)")
        p.add_argument("--json", action="store_true", help="emit machine-readable JSON")

    p = sub.add_parser("info", help="tokenizer family and the kernel it is routed to")
    common(p)
    p.set_defaults(fn=cmd_info)
    p = sub.add_parser("encode", help="encode one sequence")
    common(p)
    p.add_argument("--seq", default=None, help="DNA sequence (ACGT[N])")
    p.add_argument("--fasta", default=None, help="encode every record of this FASTA file instead")
    p.set_defaults(fn=cmd_encode)
    p = sub.add_parser("validate", help="bit identity with the tokenizer on random sequences")
    common(p)
    p.add_argument("--n", type=int, default=500)
    p.add_argument("--window", type=int, default=1024)
    p.add_argument("--seed", type=int, default=42)
    p.set_defaults(fn=cmd_validate)
    p = sub.add_parser("bench", help="strings -> ids throughput beside the host tokenizer")
    common(p)
    p.add_argument("--n", type=int, default=1000)
    p.add_argument("--window", type=int, default=4096)
    p.add_argument("--chunk", type=int, default=32)
    p.add_argument("--hf-threads", type=int, default=8)
    p.add_argument("--seed", type=int, default=11)
    p.set_defaults(fn=cmd_bench)
    p = sub.add_parser("demo", help="info + encode + validate + a small bench, end to end")
    common(p)
    p.add_argument("--sample", default=None, help="sample sequence for the encode step")
    p.set_defaults(fn=cmd_demo)
    p = sub.add_parser("list-models", help="what --model accepts")
    p.add_argument("--json", action="store_true")
    p.set_defaults(fn=cmd_list_models)
    args = ap.parse_args(argv)
    return int(args.fn(args))


if __name__ == "__main__":
    raise SystemExit(main())
