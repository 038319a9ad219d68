"""Tokenizer classes the reference's compat shim provides, as plain Python objects.

The reference's ``dnatok_compat`` (src/dnatok_compat.py) registers NTv3 / Evo2 tokenizer
classes with ``transformers`` and patches its hub, Triton and Blackwell handling at import
time.  The patches are specific to NVIDIA software stacks and to network loading and are not
carried over.  What the encode path needs from that module are the vocabulary definitions,
kept here behind the same class names and the usual tokenizer call surface
(``__call__``, ``encode``, ``get_vocab``, ``vocab_size``, ``pad_token_id``, ``unk_token_id``).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, List, Optional, Sequence, Union

import torch

NTV3_DEFAULT_VOCAB: List[str] = ["<unk>", "<pad>", "<mask>", "<cls>", "<eos>", "<bos>",
                                 "A", "T", "C", "G", "N"]


class _SimpleTokenizer:
    """Shared call surface: ``tok(texts, add_special_tokens=False, padding=False,
    return_tensors=None)`` -> {"input_ids": ...}."""

    pad_token_id: int = 0
    unk_token_id: int = 0
    padding_side: str = "right"

    def _encode_one(self, text: str) -> List[int]:
        raise NotImplementedError

    def encode(self, text: Union[str, Sequence[str]], add_special_tokens: bool = False, **_: Any):
        if isinstance(text, str):
            return self._encode_one(text)
        return [self._encode_one(t) for t in text]

    def __call__(self, texts: Union[str, Sequence[str]], add_special_tokens: bool = False,
                 padding: Union[bool, str] = False, truncation: bool = False,
                 max_length: Optional[int] = None, return_tensors: Optional[str] = None, **_: Any):
        single = isinstance(texts, str)
        rows = [self._encode_one(t) for t in ([texts] if single else texts)]
        if truncation and max_length:
            rows = [r[:max_length] for r in rows]
        if padding or return_tensors == "pt":
            width = max((len(r) for r in rows), default=0)
            if padding == "max_length" and max_length:
                width = max_length
            pad = self.pad_token_id
            if self.padding_side == "left":
                rows = [[pad] * (width - len(r)) + r for r in rows]
            else:
                rows = [r + [pad] * (width - len(r)) for r in rows]
        if return_tensors == "pt":
            return {"input_ids": torch.tensor(rows, dtype=torch.long)}
        return {"input_ids": rows[0] if single and not padding else rows}


class NTv3Tokenizer(_SimpleTokenizer):
    """Single-nucleotide tokenizer of NTv3: upper-cases its input, anything outside
    A T C G N is ``<unk>`` (reference: src/dnatok_compat.py:135-166)."""

    def __init__(self, vocab_file: Optional[str] = None, unk_token: str = "<unk>",
                 pad_token: str = "<pad>", mask_token: str = "<mask>", **_: Any) -> None:
        if vocab_file and os.path.isfile(vocab_file):
            with open(vocab_file, "r", encoding="utf-8") as fh:
                loaded = json.load(fh)
            if isinstance(loaded, dict):
                self._token_to_id = {str(k): int(v) for k, v in loaded.items()}
            else:
                self._token_to_id = {str(t): i for i, t in enumerate(loaded)}
        else:
            self._token_to_id = {t: i for i, t in enumerate(NTV3_DEFAULT_VOCAB)}
        self._id_to_token = {v: k for k, v in self._token_to_id.items()}
        self.unk_token, self.pad_token, self.mask_token = unk_token, pad_token, mask_token
        self.unk_token_id = self._token_to_id.get(unk_token, 0)
        self.pad_token_id = self._token_to_id.get(pad_token, 1)
        self._std = {"A", "T", "C", "G", "N"}

    def get_vocab(self) -> Dict[str, int]:
        return dict(self._token_to_id)

    @property
    def vocab_size(self) -> int:
        return len(self._token_to_id)

    def _encode_one(self, text: str) -> List[int]:
        unk = self.unk_token_id
        return [self._token_to_id.get(c.upper(), unk) if c.upper() in self._std else unk for c in text]

    def save_vocabulary(self, save_dir: str, prefix: Optional[str] = None):
        """Writes ``[prefix-]vocab.json`` (token -> id), which the constructor reads back
        (reference: src/dnatok_compat.py:152-156)."""
        os.makedirs(save_dir, exist_ok=True)
        path = os.path.join(save_dir, (f"{prefix}-" if prefix else "") + "vocab.json")
        with open(path, "w", encoding="utf-8") as fh:
            json.dump(self._token_to_id, fh, indent=2)
        return (path,)


class Evo2ByteTokenizer(_SimpleTokenizer):
    """Byte-level tokenizer of Evo2: id = ord(c) (reference: src/dnatok_compat.py:181-218)."""

    def __init__(self, vocab_size: int = 512, **_: Any) -> None:
        self._vocab_size = int(vocab_size)
        self.unk_token_id = 0
        self.pad_token_id = 1

    @property
    def vocab_size(self) -> int:
        return self._vocab_size

    def get_vocab(self) -> Dict[str, int]:
        return {chr(i): i for i in range(self._vocab_size)}

    def _encode_one(self, text: str) -> List[int]:
        return [ord(c) if ord(c) < self._vocab_size else self.unk_token_id for c in text]

    def save_vocabulary(self, save_dir: str, prefix: Optional[str] = None):
        """Writes ``[prefix-]evo2_vocab.json`` holding the vocabulary size, all there is to this
        tokenizer (reference: src/dnatok_compat.py:213-218)."""
        os.makedirs(save_dir, exist_ok=True)
        path = os.path.join(save_dir, (f"{prefix}-" if prefix else "") + "evo2_vocab.json")
        with open(path, "w", encoding="utf-8") as fh:
            json.dump({"vocab_size": self._vocab_size}, fh)
        return (path,)


class CharTokenizer(_SimpleTokenizer):
    """HyenaDNA-style fallback: {A:7, C:8, G:9, T:10, N:11}, upper-cased, unknown -> N
    (reference: src/dnatok_compat.py:220-238)."""

    def __init__(self, vocab: Optional[Dict[str, int]] = None) -> None:
        self.vocab = vocab or {"A": 7, "C": 8, "G": 9, "T": 10, "N": 11}
        self.unk_token_id = self.vocab.get("N", 11)
        self.pad_token_id = 0
        self.model_max_length = 32768

    def get_vocab(self) -> Dict[str, int]:
        return dict(self.vocab)

    @property
    def vocab_size(self) -> int:
        return max(self.vocab.values()) + 1

    def _encode_one(self, text: str) -> List[int]:
        return [self.vocab.get(c.upper(), self.unk_token_id) for c in text]
