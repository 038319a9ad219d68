"""The tokenizers the CLI offers by name, built in memory with the Hugging Face ``tokenizers``
library (the reference's CLI resolves hub model names instead, src/dnatok_cli.py:55-102; this
backend has no network path).

* char   -- ``WordLevel`` over the NTv3 vocabulary order
            (reference: src/dnatok_compat.py:144) with one token per character.
* k-mer  -- ``WordLevel`` over 5 specials + 4**k k-mers + the single characters
            ``A C G T N``; a two-stage ``Split`` makes the windows grid-aligned: a window
            holding anything but ACGT, and the trailing remainder, come out as single
            characters.
"""
from __future__ import annotations

import itertools
from typing import Dict, List

NTV3_VOCAB: List[str] = ["<unk>", "<pad>", "<mask>", "<cls>", "<eos>", "<bos>",
                         "A", "T", "C", "G", "N"]
KMER_SPECIALS: List[str] = ["<unk>", "<pad>", "<mask>", "<cls>", "<eos>"]


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
