"""Hugging Face ``tokenizers`` objects for the five benchmark configurations: the ground truth
("bit-exact vs HF") and the CPU baseline that is timed next to the GPU path.  Test and benchmark
infrastructure; nothing here is on the encode path.

* char, 6-mer -- the tokenizers the CLI offers by name (dnatok_amd.builtin_tokenizers).
* BPE         -- ``models.BPE`` trained with ``BpeTrainer`` on the seeded synthetic corpora; the
                 trained ``tokenizer.json`` files are kept under tests/golden/.
"""
from __future__ import annotations

import os
from typing import Iterable, List

from dnatok_amd.builtin_tokenizers import (KMER_SPECIALS, NTV3_VOCAB, build_char_tokenizer,  # noqa: F401
                                           build_kmer_tokenizer, char_vocab, kmer_vocab)

BPE_SPECIALS: List[str] = ["[UNK]", "[CLS]", "[SEP]", "[PAD]", "[MASK]"]


def train_bpe_tokenizer(lines: Iterable[str], vocab_size: int, n_lines: int | None = None):
    """``BpeTrainer`` run as the benchmark configurations state it: no normaliser,
    no pre-tokenizer (each line is one word), ACGTN as the initial alphabet."""
    from tokenizers import Tokenizer, models, trainers
    tk = Tokenizer(models.BPE(unk_token="[UNK]"))
    trainer = trainers.BpeTrainer(vocab_size=vocab_size, special_tokens=BPE_SPECIALS,
                                  initial_alphabet=list("ACGTN"), show_progress=False)
    tk.train_from_iterator(lines, trainer=trainer, length=n_lines)
    return tk


def golden_dir() -> str:
    here = os.path.dirname(os.path.abspath(__file__))
    return os.path.join(os.path.dirname(here), "golden")


def load_bpe_tokenizer(which: str):
    """Load the committed ``tokenizer.json`` for vocab "4096" or "32000"."""
    from tokenizers import Tokenizer
    return Tokenizer.from_file(bpe_tokenizer_path(which))


def bpe_tokenizer_path(which: str) -> str:
    return os.path.join(golden_dir(), f"bpe{which}_tokenizer.json")
