"""``DnatokBpeKernel``: the reference's kernel wrapper interface over the MI355X BPE engine.

Mirrors ``dnatok_bpe_kernel.DnatokBpeKernel`` of the reference
(src/dnatok_bpe_kernel/__init__.py:81-136) and the pybind class behind it
(src/dnatok_bpe_kernel/dnatok_bpe.cu:1042-1055): built from a merges.txt file, it
tokenizes strings into the kernel's own id space (0..255 = bytes, then merge
results in first-seen order) and returns device tensors.  Translation to the
tokenizer's ids is the caller's remap table, as in ``GPUTokBPEBackend``.
"""
from __future__ import annotations

from typing import Optional, Dict, List, Optional, Sequence, Tuple

import torch

from . import bpe_vocab, encoders

# one instance per (merges_path, max_iters), as the reference caches them (__init__.py:46,96-102)
_INSTANCES: Dict[Tuple[str, int], "_Impl"] = {}


class _Impl:
    def __init__(self, merges_path: str):
        self.vocab = bpe_vocab.KernelVocab(bpe_vocab.parse_merges_txt(merges_path))
        self.encoder = encoders.BpeEncoder(self.vocab.pair_a, self.vocab.pair_b, self.vocab.new_id,
                                           len(self.vocab))
        # persistent, grow-only workspace; tokenize_batch returns views into it
        self.tok: Optional[torch.Tensor] = None
        self.lengths: Optional[torch.Tensor] = None
        self.ids: Optional[torch.Tensor] = None
        self.mask_unused = None
        self.max_len: Optional[torch.Tensor] = None


class DnatokBpeKernel:
    """Build-on-first-use wrapper around the BPE merge engine.

    ``max_iters`` is accepted for interface compatibility; the engine always runs to
    completion (the reference stores the value and never reads it,
    src/dnatok_bpe_kernel/dnatok_bpe.cu:807,1017).
    """

    def __init__(self, merges_path: str, max_iters: int = 1024) -> None:
        key = (str(merges_path), int(max_iters))
        impl = _INSTANCES.get(key)
        if impl is None:
            impl = _Impl(str(merges_path))
            _INSTANCES[key] = impl
        self._impl = impl

    def vocab_size(self) -> int:
        return len(self._impl.vocab)

    def id_to_token(self, idx: int) -> str:
        idx = int(idx)
        if idx < 0 or idx >= len(self._impl.vocab):
            raise IndexError("id out of range")
        return self._impl.vocab.id_to_token[idx]

    def tokenize_device(self, data: torch.Tensor, offsets: torch.Tensor, max_len: int, *,
                        lengths: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """Device-resident entry: uint8 bytes + int64 offsets -> (tok_tmp, lengths); row b's
        tokens are tok_tmp[offsets[b] : offsets[b] + lengths[b]].  ``lengths`` (int32 [B] on the
        device) may be given by the caller."""
        return self._impl.encoder.encode(data, offsets, max_len, lengths=lengths)

    def tokenize_padded_device(self, data: torch.Tensor, offsets: torch.Tensor, max_len: int, stride: int,
                               pad_id: int, *, remap: Optional[torch.Tensor] = None, out=None,
                               pad_left: bool = False):
        """Device-resident entry with the padding done by the engine: (ids [B, stride] of the type
        of ``out``'s ids (int32 without ``out``), mask uint8 [B, stride], lengths int32 [B], longest
        int32 [1]); see ``BpeEncoder.encode_padded``."""
        return self._impl.encoder.encode_padded(data, offsets, max_len, stride, pad_id, remap=remap, out=out,
                                                pad_left=pad_left)

    def tokenize_batch(self, texts: Sequence[str], *, clone: bool = False
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Encode a batch of strings.

        Returns ``ids`` int32 cuda [B, T_max] (T_max = longest input in bytes, at least 1),
        zero-filled beyond each row's length, and ``lengths`` int32 cuda [B]
        (-1 = row longer than supported, -2 = the engine gave up; neither happens for
        inputs below 2^31 bytes).  Unless ``clone=True`` both are views into a workspace
        that the next call on this instance overwrites.
        """
        impl = self._impl
        texts = list(texts)
        b = len(texts)
        if b == 0:
            return (torch.empty((0, 0), dtype=torch.int32, device="cuda"),
                    torch.empty((0,), dtype=torch.int32, device="cuda"))
        data, offsets, lens = encoders.bytes_from_strings(texts, "cuda", encoding="utf-8")
        t_max = max(int(lens.max()), 1)
        total = int(data.numel())
        if impl.tok is None or impl.tok.numel() < max(total, 1):
            impl.tok = torch.empty(max(total, 1), dtype=torch.int32, device="cuda")
        if impl.lengths is None or impl.lengths.numel() < b:
            impl.lengths = torch.empty(b, dtype=torch.int32, device="cuda")
            impl.max_len = torch.empty(1, dtype=torch.int32, device="cuda")
        if impl.ids is None or impl.ids.numel() < b * t_max:
            impl.ids = torch.empty(b * t_max, dtype=torch.int32, device="cuda")
        lengths = impl.lengths[:b]
        impl.encoder.encode(data, offsets, t_max, tok_tmp=impl.tok, lengths=lengths)
        ids = impl.ids[:b * t_max].view(b, t_max)
        encoders.pad_rows(impl.tok, offsets, lengths, 0, t_max, fill_to=t_max, want_mask=False,
                          out=(ids, None, impl.max_len))
        if clone:
            return ids.clone(), lengths.clone()
        return ids, lengths
