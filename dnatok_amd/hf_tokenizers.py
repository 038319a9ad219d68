"""Hugging Face ``tokenizers`` objects for the five benchmark configurations.

These are the ground truth ("bit-exact vs HF") and the CPU baseline that is
timed next to the GPU path.  Nothing here is on the encode path itself.

* char   -- ``WordLevel`` over the NTv3 vocabulary order
            (reference: src/dnatok_compat.py:144) with one token per character.
* 6-mer  -- ``WordLevel`` over 5 specials + 4096 six-mers + the single
            characters ``A C G T N``; a two-stage ``Split`` makes the windows
            grid-aligned: a window holding anything but ACGT, and the trailing
            remainder, come out as single characters.
* BPE    -- ``models.BPE`` trained with ``BpeTrainer`` on the seeded synthetic
            corpora; the trained ``tokenizer.json`` files are kept under
            tests/golden/.
"""
from __future__ import annotations

import itertools
import os
from typing import Dict, Iterable, List

NTV3_VOCAB: List[str] = ["<unk>", "<pad>", "<mask>", "<cls>", "<eos>", "<bos>",
                         "A", "T", "C", "G", "N"]
KMER_SPECIALS: List[str] = ["<unk>", "<pad>", "<mask>", "<cls>", "<eos>"]
BPE_SPECIALS: List[str] = ["[UNK]", "[CLS]", "[SEP]", "[PAD]", "[MASK]"]


def char_vocab() -> Dict[str, int]:
    return {t: i for i, t in enumerate(NTV3_VOCAB)}


def kmer_vocab(k: int = 6) -> Dict[str, int]:
    """specials, then all 4**k k-mers in A<C<G<T lexicographic order, then A C G T N."""
    vocab = {t: i for i, t in enumerate(KMER_SPECIALS)}
    for km in itertools.product("ACGT", repeat=k):
        vocab["".join(km)] = len(vocab)
    for c in "ACGTN":
        vocab[c] = len(vocab)
    return vocab


def build_char_tokenizer():
    from tokenizers import Regex, Tokenizer, models, pre_tokenizers
    tk = Tokenizer(models.WordLevel(char_vocab(), unk_token="<unk>"))
    tk.pre_tokenizer = pre_tokenizers.Split(Regex("."), "isolated")
    return tk


def build_kmer_tokenizer(k: int = 6):
    from tokenizers import Regex, Tokenizer, models, pre_tokenizers
    tk = Tokenizer(models.WordLevel(kmer_vocab(k), unk_token="<unk>"))
    tk.pre_tokenizer = pre_tokenizers.Sequence([
        pre_tokenizers.Split(Regex(".{%d}" % k), "isolated"),
        pre_tokenizers.Split(Regex("[ACGT]{%d}|." % k), "isolated"),
    ])
    return tk


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
    return os.path.join(os.path.dirname(here), "tests", "golden")


def load_bpe_tokenizer(which: str):
    """Load the committed ``tokenizer.json`` for vocab "4096" or "32000"."""
    from tokenizers import Tokenizer
    return Tokenizer.from_file(bpe_tokenizer_path(which))


def bpe_tokenizer_path(which: str) -> str:
    return os.path.join(golden_dir(), f"bpe{which}_tokenizer.json")
