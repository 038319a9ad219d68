"""``DNATok``: the reference's drop-in wrapper API over the MI355X encode kernels.

Same constructor, ``discover()`` and ``encode_*`` surface as the reference's
``dna_tokenizer.DNATok`` (src/dna_tokenizer.py:85-133, 864-1110, 2049-2338, 2594-3110).
``discover()`` probes the embedder's tokenizer with short strings and selects one of
three paths; all three run on the GPU through libdnatok_hip.so:

* single-nucleotide tokenizers -> 256-entry byte table  (char kernel)
* non-overlapping k-mer tokenizers (2 <= k <= 6) -> 5**k window table with per-window
  expansion lists (k-mer kernel)
* BPE tokenizers -> ``GPUTokBPEBackend`` (merge engine + packer)

There is no numpy / torch fallback for the encode itself; a missing library raises.
Rows the tables cannot express (a k-mer window with no known tokenization) are
re-tokenized by the tokenizer object itself, as the reference does
(src/dna_tokenizer.py:1955-2047).
"""
from __future__ import annotations

import inspect
import logging
import os
from typing import Any, Iterator, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import encoders, kmer_tables

_DNA_UPPER = "ACGTN"


def _smallest_dtype(max_id: int) -> torch.dtype:
    if max_id <= 255:
        return torch.uint8
    if max_id <= 32_767:
        return torch.int16
    if max_id <= 2_147_483_647:
        return torch.int32
    return torch.int64


class DNATok:
    DEFAULT_IDS_MAX_TOKENS_PER_CALL = 1_048_576

    def __init__(self, embedder: object, ids_max_tokens_per_call: int = DEFAULT_IDS_MAX_TOKENS_PER_CALL,
                 logger: Optional[logging.Logger] = None, *,
                 prefer_int32_h2d: bool = True, overlap_h2d_compute: bool = True,
                 force_fp32_outputs: bool = True, strict_lut_check: bool = True,
                 normalize_case: bool = False, handle_invalid_chars: bool = False,
                 require_valid_chars: bool = False, allow_incomplete_kmer_lut: bool = False,
                 padding_side: str = "left", pack_2bit_h2d: bool = False, use_uint8_ids: bool = False,
                 use_cuda_graph: bool = False, use_fused_kernel: bool = False) -> None:
        self.embedder = embedder
        self.log = logger or logging.getLogger("DNATok")
        if not self.log.handlers:
            h = logging.StreamHandler()
            h.setFormatter(logging.Formatter("[%(name)s] %(message)s"))
            self.log.addHandler(h)
            level = os.environ.get("DNATOK_LOG_LEVEL", "WARNING").upper()
            self.log.setLevel(getattr(logging, level, logging.WARNING))
        if padding_side not in ("left", "right"):
            raise ValueError("padding_side must be 'left' or 'right'")
        self.ids_max_tokens_per_call = int(ids_max_tokens_per_call)
        self.prefer_int32_h2d = bool(prefer_int32_h2d)
        self.overlap_h2d_compute = bool(overlap_h2d_compute)
        self.force_fp32_outputs = bool(force_fp32_outputs)
        self.strict_lut_check = bool(strict_lut_check)
        self.normalize_case = bool(normalize_case)
        self.handle_invalid_chars = bool(handle_invalid_chars)
        self.require_valid_chars = bool(require_valid_chars)
        env_allow = os.environ.get("DNATOK_ALLOW_INCOMPLETE_KMER_LUT")
        self.allow_incomplete_kmer_lut = (env_allow.strip().lower() in ("1", "true", "yes", "y")
                                          if env_allow is not None else bool(allow_incomplete_kmer_lut))
        self.padding_side = padding_side
        # accepted for interface compatibility; the device kernels make them moot
        self.pack_2bit_h2d, self.use_uint8_ids = bool(pack_2bit_h2d), bool(use_uint8_ids)
        self.use_cuda_graph, self.use_fused_kernel = bool(use_cuda_graph), bool(use_fused_kernel)
        self._reset()

    # ------------------------------------------------------------------ state

    def _reset(self) -> None:
        self.use_ids_path = False
        self.ascii_lut: Optional[np.ndarray] = None         # int64 [256]
        self.ascii_start_lut: Optional[np.ndarray] = None
        self.id_pad = 0
        self.id_N = 0
        self.id_unk: Optional[int] = None
        self.invalid_char_id: Optional[int] = None
        self.token_len: Optional[int] = None
        self.vocab_size = 0
        self.kmer_k: Optional[int] = None
        self.kmer_lut: Optional[np.ndarray] = None
        self.kmer_single_char_lut: Optional[np.ndarray] = None
        self.bpe_backend: Optional[Any] = None
        self.lmm_bpe: Optional[Any] = None
        self._char_enc: Optional[encoders.CharEncoder] = None
        self._kmer_enc: Optional[encoders.KmerEncoder] = None
        self._kmer_tables: Optional[kmer_tables.KmerTables] = None
        self._staging_bytes_cpu: Optional[torch.Tensor] = None
        self._packed_2bit_cpu: Optional[torch.Tensor] = None
        self._dev_ping: Optional[torch.Tensor] = None
        self._dev_pong: Optional[torch.Tensor] = None
        self._graph = None
        self._graph_shape: Optional[Tuple[int, int]] = None
        self._graph_static_in: Optional[torch.Tensor] = None
        self._graph_static_out: Optional[torch.Tensor] = None

    def free_buffers(self) -> None:
        self._staging_bytes_cpu = None
        self._packed_2bit_cpu = None
        self._dev_ping = None
        self._dev_pong = None
        self._graph = None
        self._graph_static_in = None
        self._graph_static_out = None

    # ------------------------------------------------------------- tokenizer access

    def _tok_ids(self, texts: Sequence[str]) -> List[List[int]]:
        """Token ids of each text, no special tokens, through whatever call style the
        tokenizer object offers."""
        tok = self.embedder.tokenizer
        texts = list(texts)
        try:
            out = tok(texts, add_special_tokens=False)
            ids = out["input_ids"] if isinstance(out, dict) or hasattr(out, "__getitem__") else out.input_ids
            if torch.is_tensor(ids):
                ids = ids.tolist()
            return [list(map(int, r)) for r in ids]
        except TypeError:
            pass
        if hasattr(tok, "encode_batch"):
            return [list(e.ids) for e in tok.encode_batch(texts, add_special_tokens=False)]
        return [list(map(int, tok.encode(t))) for t in texts]

    def _tokenize_batch_cpu(self, seqs: Sequence[str], dtype: torch.dtype = torch.long,
                            pin: bool = False) -> torch.Tensor:
        """The tokenizer itself, padded like the fast paths pad (reference: 1591-1777)."""
        rows = self._tok_ids(seqs)
        width = max((len(r) for r in rows), default=0)
        if self.token_len is not None and self.token_len > width:
            width = int(self.token_len)
        out = torch.full((len(rows), width), int(self.id_pad), dtype=dtype)
        for i, r in enumerate(rows):
            if r:
                cur = torch.as_tensor(r, dtype=dtype)
                if self.padding_side == "left":
                    out[i, width - len(r):] = cur
                else:
                    out[i, :len(r)] = cur
        return out.pin_memory() if pin and torch.cuda.is_available() else out

    # ---------------------------------------------------------------- discovery

    def discover(self) -> None:
        self._reset()
        emb = self.embedder
        if not callable(getattr(emb, "embed_tokens", None)):
            self.log.info("embedder has no embed_tokens(); ids path disabled")
            return
        tok = getattr(emb, "tokenizer", None)
        self.id_pad = self._first_int((emb, "pad_id"), (emb, "pad_token_id"), (tok, "pad_token_id"), default=0)
        self.id_unk = self._first_int((tok, "unk_token_id"), (emb, "unk_id"), default=None)
        side = getattr(tok, "padding_side", None)
        if side in ("left", "right"):
            self.padding_side = side
        if tok is None:
            # fixed map when no tokenizer is attached (reference: 907-932)
            lut = np.zeros(256, dtype=np.int64)
            for ch, v in zip("ACGTN", (1, 2, 3, 4, 0)):
                lut[ord(ch)] = v
                lut[ord(ch.lower())] = v
            self._install_char(lut, None, id_n=0, vocab_size=5)
            return
        self.vocab_size = self._discover_vocab_size(tok)
        # a probe can be fooled (a BPE vocabulary may split homopolymers evenly); a table that
        # does not reproduce the tokenizer on random input is dropped and the next path is tried
        k = self._probe_kmer()
        if k is not None:
            try:
                self._install_kmer(k)
                return
            except RuntimeError as e:
                self.log.info("k-mer probe (k=%d) rejected: %s", k, e)
                keep = (self.id_pad, self.id_unk, self.padding_side, self.vocab_size)
                self._reset()
                self.id_pad, self.id_unk, self.padding_side, self.vocab_size = keep
        try:
            if self._probe_char():
                return
        except RuntimeError as e:
            self.log.info("single-nucleotide probe rejected: %s", e)
            keep = (self.id_pad, self.id_unk, self.padding_side, self.vocab_size)
            self._reset()
            self.id_pad, self.id_unk, self.padding_side, self.vocab_size = keep
        from .gputok_bpe_backend import GPUTokBPEBackend
        if GPUTokBPEBackend.is_supported(tok):
            self.bpe_backend = GPUTokBPEBackend(tok, engine="dnatok")
            self.id_pad = self.bpe_backend.pad_id
            self.use_ids_path = True
            return
        self.log.warning("tokenizer is neither single-nucleotide, k-mer nor a supported BPE; ids path disabled")

    @staticmethod
    def _first_int(*candidates, default):
        for obj, name in candidates:
            v = getattr(obj, name, None) if obj is not None else None
            if isinstance(v, (int, np.integer)) and not isinstance(v, bool):
                return int(v)
        return default

    def _discover_vocab_size(self, tok) -> int:
        for name in ("vocab_size",):
            v = getattr(tok, name, None)
            if isinstance(v, (int, np.integer)):
                return int(v)
        for name in ("get_vocab_size",):
            f = getattr(tok, name, None)
            if callable(f):
                try:
                    return int(f())
                except Exception:
                    pass
        try:
            return int(len(tok))
        except Exception:
            pass
        gv = getattr(tok, "get_vocab", None)
        if callable(gv):
            try:
                return int(max(gv().values())) + 1
            except Exception:
                pass
        return 0

    def _probe_kmer(self) -> Optional[int]:
        """k = 24 / tokens("A" * 24), accepted when it divides, 2 <= k <= 6, and the other
        homopolymers and a mixed probe give the same count (reference: 655-741)."""
        try:
            n = len(self._tok_ids(["A" * 24])[0])
            if n == 0 or 24 % n != 0:
                return None
            k = 24 // n
            if not 2 <= k <= 6:
                return None
            probes = ["C" * 24, "G" * 24, "T" * 24, ("ACGT" * 6)]
            if any(len(r) != n for r in self._tok_ids(probes)):
                return None
            rng = np.random.default_rng(1)
            mixed = ["".join(rng.choice(list("ACGT"), size=m * k)) for m in (1, 2, 3, 5, 8)]
            if [len(r) for r in self._tok_ids(mixed)] != [1, 2, 3, 5, 8]:
                return None
            return k
        except Exception:
            return None

    def _install_kmer(self, k: int) -> None:
        unk = self.id_unk if self.id_unk is not None else self.id_pad
        t = kmer_tables.tables_from_tokenize(self._tok_ids, k, int(unk))
        t.digit = kmer_tables.digit_table(fold_case=self.normalize_case)
        if self.normalize_case:
            for ch in _DNA_UPPER:
                t.single[ord(ch.lower())] = t.single[ord(ch)]
        n_missing = int(((t.kmer_lut < 0) & (t.exp_len == 0)).sum())
        if n_missing and not self.allow_incomplete_kmer_lut:
            self.log.info("%d of %d windows have no tokenization of their own; such rows are "
                          "re-tokenized by the tokenizer", n_missing, t.kmer_lut.size)
        self._kmer_tables = t
        self.kmer_k = k
        self.kmer_lut = t.kmer_lut.astype(np.int64)
        self.kmer_single_char_lut = t.single.astype(np.int64)
        self.id_N = int(t.single[ord("N")])
        missing = int(unk)
        self._kmer_enc = encoders.KmerEncoder(k, t.digit, t.kmer_lut, t.single, int(self.id_pad), missing,
                                              t.exp_off, t.exp_len, t.exp_flat)
        if self.vocab_size <= 0:
            self.vocab_size = int(max(t.kmer_lut.max(), t.single.max())) + 1
        self.use_ids_path = True
        self._self_check()            # always: a mis-probed k must not survive

    def _probe_char(self) -> bool:
        """One token per character on fixed probes, then a byte table from probing every
        printable byte (reference: 447-653, 1139-1218)."""
        probes = ["ACGTACGT", "NNNNACGT", "TTTTGGGG", "CAGTNACG"]
        try:
            if any(len(r) != 8 for r in self._tok_ids(probes)):
                return False
            chars = [chr(b) if 32 < b < 127 else "N" for b in range(256)]
            singles = self._tok_ids(chars)
        except Exception:
            return False
        id_n_row = singles[ord("N")]
        if len(id_n_row) != 1:
            return False
        id_n = int(id_n_row[0])
        fallback = self.id_unk if self.id_unk is not None else id_n
        lut = np.full(256, int(fallback), dtype=np.int64)
        for b in range(256):
            if 32 < b < 127 and len(singles[b]) == 1:
                lut[b] = int(singles[b][0])
        # a separate first-position table only if the tokenizer treats position 0 differently
        start = None
        try:
            firsts = self._tok_ids([c + "A" for c in _DNA_UPPER])
            if all(len(r) == 2 for r in firsts) and any(int(r[0]) != lut[ord(c)] for r, c in zip(firsts, _DNA_UPPER)):
                start = lut.copy()
                for r, c in zip(firsts, _DNA_UPPER):
                    start[ord(c)] = int(r[0])
        except Exception:
            start = None
        self._install_char(lut, start, id_n=id_n, vocab_size=self.vocab_size or int(lut.max()) + 1)
        if self.strict_lut_check:
            self._self_check()
        return True

    def _install_char(self, lut: np.ndarray, start: Optional[np.ndarray], *, id_n: int, vocab_size: int) -> None:
        lut = lut.copy()
        self.id_N = int(id_n)
        if self.normalize_case:
            for ch in _DNA_UPPER:
                lut[ord(ch.lower())] = lut[ord(ch)]
                if start is not None:
                    start[ord(ch.lower())] = start[ord(ch)]
        if self.handle_invalid_chars:
            valid = set(map(ord, _DNA_UPPER)) | set(map(ord, _DNA_UPPER.lower()))
            inv = self.invalid_char_id if self.invalid_char_id is not None else self.id_N
            for b in range(256):
                if b not in valid:
                    lut[b] = inv
                    if start is not None:
                        start[b] = inv
        self.ascii_lut = lut
        self.ascii_start_lut = start
        self.vocab_size = int(vocab_size)
        self._char_enc = encoders.CharEncoder(lut.astype(np.int32), int(self.id_pad),
                                              None if start is None else start.astype(np.int32))
        self.use_ids_path = True

    def _self_check(self) -> None:
        """32 random ACGTN strings must encode exactly as the tokenizer does
        (reference: 1220-1273)."""
        if not torch.cuda.is_available():
            return
        rng = np.random.default_rng(0)
        k = self.kmer_k or 1
        seqs = ["".join(rng.choice(list(_DNA_UPPER), size=8 * k)) for _ in range(32)]
        got = self.encode_batch_to_ids(seqs)
        want = self._tokenize_batch_cpu(seqs)
        if got.shape != want.shape or not torch.equal(got.cpu(), want):
            raise RuntimeError("DNATok.discover(): table encode disagrees with the tokenizer")
        if k > 1:
            # A trailing remainder of fewer than k characters is spelled with the single-character
            # table; a tokenizer that does something else with it (drops it, one <unk> for all of it)
            # gets such rows back from the tokenizer itself.
            self._kmer_tail_ok = True
            tails = ["".join(rng.choice(list(_DNA_UPPER), size=m)) for m in (8 * k + 1, 3 * k + k - 1, 2 * k + 1)]
            got = self.encode_batch_to_ids(tails)
            want = self._tokenize_batch_cpu(tails)
            if got.shape != want.shape or not torch.equal(got.cpu(), want):
                self._kmer_tail_ok = False
                self.log.info("trailing characters are not tokenized one by one; rows whose length is "
                              "no multiple of %d go to the tokenizer", k)

    # ------------------------------------------------------------------- encode

    def _require_ready(self) -> None:
        if not self.use_ids_path:
            raise RuntimeError("DNATok.discover() must be called before encoding.")

    def encode_batch_device(self, seqs: Sequence[str], device="cuda") -> Tuple[torch.Tensor, torch.Tensor]:
        """Device-resident encode: (ids int32 [B, T], mask uint8 [B, T]) on the GPU, every row
        padded on ``padding_side`` to the longest row, or to ``token_len`` when that is larger
        (reference: _pad_id_list, src/dna_tokenizer.py:1878-1894)."""
        return self._encode_rows_device(seqs, device, dtype=torch.int32,
                                        min_width=int(self.token_len or 0), pad_multiple=1)

    def _encode_rows_device(self, seqs: Sequence[str], device, *, dtype: torch.dtype, min_width: int,
                            pad_multiple: int, host_ids: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
        """``host_ids``: the caller wants the ids on the host; where the layout allows it they are
        copied down inside the call, under its one wait, and left in ``_staged_host_ids`` (a view
        of the tokenizer's pinned buffer, valid until the next call)."""
        self._require_ready()
        if not seqs:
            raise ValueError("No sequences provided for encoding.")
        left = self.padding_side == "left"
        self._staged_host_ids = None
        if self.bpe_backend is not None:
            return self._encode_bpe_rows(list(seqs), device, dtype=dtype, min_width=min_width,
                                         pad_multiple=pad_multiple, host_ids=host_ids)
        data, offsets, lens = encoders.bytes_from_strings(seqs, device)
        if self._kmer_enc is not None:
            return self._encode_kmer_device(seqs, data, offsets, lens, dtype=dtype, min_width=min_width,
                                            pad_multiple=pad_multiple, host_ids=host_ids)
        width = max(int(lens.max()), int(min_width))
        if pad_multiple > 1 and width % pad_multiple:
            width += pad_multiple - width % pad_multiple
        return self._char_enc.encode_padded(data, offsets, width, pad_left=left, dtype=dtype)

    def _encode_bpe_rows(self, seqs: List[str], device, *, dtype: torch.dtype, min_width: int,
                         pad_multiple: int, host_ids: bool) -> Tuple[torch.Tensor, torch.Tensor]:
        """BPE rows with the reference's fallback chain (src/dna_tokenizer.py:2066-2100: any failure
        of the backend ends at the tokenizer itself, with a warning).  Finer than the reference
        where the backend says which rows it cannot reproduce (``UnsupportedRows``: white space
        under a pre-tokenizer, a character outside the vocabulary without unk_token): those rows
        alone get the tokenizer's ids, the others stay on the GPU, as the k-mer path splices its
        rows.  The reference's middle link (CachedLMM, approximate) is not part of this build."""
        from .gputok_bpe_backend import UnsupportedRows
        try:
            return self._bpe_rows_on_gpu(seqs, device, dtype=dtype, min_width=min_width,
                                         pad_multiple=pad_multiple, host_ids=host_ids)
        except UnsupportedRows as e:
            self._staged_host_ids = None
            bad = e.rows
            self.log.warning("BPE backend: %d of %d rows go to the tokenizer (%s)", len(bad), len(seqs), e)
            fixed = self._tok_ids([seqs[i] for i in bad])
            is_bad = set(bad)
            keep = [i for i in range(len(seqs)) if i not in is_bad]
            if not keep:
                return self._tokenizer_rows_device(seqs, device, dtype=dtype, min_width=min_width,
                                                   pad_multiple=pad_multiple)
            try:
                good_ids, good_mask = self._bpe_rows_on_gpu([seqs[i] for i in keep], device, dtype=dtype,
                                                            min_width=min_width, pad_multiple=pad_multiple,
                                                            host_ids=False)
            except Exception as e2:
                self.log.warning("BPE backend failed (%s); falling back to the tokenizer.", e2)
                return self._tokenizer_rows_device(seqs, device, dtype=dtype, min_width=min_width,
                                                   pad_multiple=pad_multiple)
            # the clean rows at their places in a batch of the full height, then the others spliced in
            n, w = len(seqs), good_ids.shape[1]
            ids = torch.full((n, w), int(self.id_pad), dtype=good_ids.dtype, device=good_ids.device)
            mask = torch.zeros((n, w), dtype=torch.uint8, device=good_ids.device)
            at = torch.as_tensor(keep, dtype=torch.int64, device=good_ids.device)
            ids[at] = good_ids
            mask[at] = good_mask
            return self._splice_tokenizer_rows(ids, mask, bad, fixed, pad_multiple=pad_multiple)
        except Exception as e:
            self._staged_host_ids = None
            self.log.warning("BPE backend failed (%s); falling back to the tokenizer.", e)
            return self._tokenizer_rows_device(seqs, device, dtype=dtype, min_width=min_width,
                                               pad_multiple=pad_multiple)

    def _bpe_rows_on_gpu(self, seqs: List[str], device, *, dtype: torch.dtype, min_width: int,
                         pad_multiple: int, host_ids: bool) -> Tuple[torch.Tensor, torch.Tensor]:
        # the engine pads the rows itself while it writes them out: side, width and id type are final
        left = self.padding_side == "left"
        staged = []

        def stage(ids):
            if host_ids:
                nbytes = ids.numel() * ids.element_size()
                host = self._pinned(nbytes)[:nbytes].view(ids.dtype).view(ids.shape)
                host.copy_(ids, non_blocking=True)
                staged[:] = [host]

        ids, mask = self.bpe_backend.padded_device(seqs, device=device, min_width=min_width,
                                                   pad_multiple=pad_multiple, stage_ids=stage,
                                                   pad_left=left, dtype=dtype)
        if staged and staged[0].shape[1] == ids.stride(0):      # (not those of a first, too narrow, try)
            cap, width = staged[0].shape[1], ids.shape[1]
            self._staged_host_ids = staged[0][:, cap - width:] if left else staged[0][:, :width]
        return ids, mask

    def _pad_bpe_runs(self, tok, offsets, lengths, t_cap: int, *, dtype, min_width: int, pad_multiple: int,
                      host_ids: bool = False, stats_behind_lengths: bool = False):
        """The engine's token runs -> padded rows: remap, padding side, least width, multiple and
        id type in one launch; one host read for the shape (and the smallest length: a negative
        one is a failed row)."""
        be = self.bpe_backend
        worst = max(int(t_cap), int(min_width), 1)
        if pad_multiple > 1 and worst % pad_multiple:
            worst += pad_multiple - worst % pad_multiple
        # In a stream of batches the rows are laid out only as far apart as the recent batches were
        # wide (encoders.WidthGuess, plus a margin): a token run is several times shorter than its row of bytes.  A
        # batch that needs more room than that is padded again with room for the worst case.
        if not hasattr(self, "_bpe_widths"):
            self._bpe_widths = encoders.WidthGuess()
        guess = self._bpe_widths.next()
        cap = worst
        if guess:
            cap = max(guess + (-guess) % 128, int(min_width))
            if pad_multiple > 1 and cap % pad_multiple:
                cap += pad_multiple - cap % pad_multiple
            cap = min(cap, worst)
        n = lengths.numel()
        # lengths and the padding's two statistics in one allocation: one copy brings them down
        # (with stats_behind_lengths the caller got the lengths as the head of an allocation of n + 2)
        meta = torch.as_strided(lengths, (n + 2,), (1,)) if stats_behind_lengths else None
        while True:
            ids, mask, stats = encoders.pad_rows_as(tok, offsets, lengths, int(be.pad_id), cap, min_width=min_width,
                                                    pad_multiple=pad_multiple, pad_left=(self.padding_side == "left"),
                                                    dtype=dtype, remap=be._remap_on(tok.device),
                                                    stats=None if meta is None else meta[n:])
            staged = None
            if host_ids and cap < worst:
                nbytes = n * cap * ids.element_size()
                staged = self._pinned(nbytes)[:nbytes].view(ids.dtype).view(n, cap)
                staged.copy_(ids, non_blocking=True)
            if meta is not None:
                meta_h = meta.cpu().numpy()                                  # (the one wait)
                longest, width, shortest = int(meta_h[n]), int(meta_h[n + 1]), int(meta_h[:n].min())
            else:
                longest, width, shortest = torch.cat((stats, lengths.min()[None])).tolist()
            if shortest < 0:
                raise RuntimeError("BPE engine reported a failed row (negative length)")
            if longest < cap or cap >= worst:            # (the packer reports lengths cut to the stride)
                break
            cap = worst                                  # a row may have been cut: once more, with room for all
        self._bpe_widths.update(longest)
        self._staged_host_ids = staged[:, :width] if staged is not None else None
        return ids[:, :width], mask[:, :width]

    def encode_fasta_device(self, source, device="cuda"):
        """FASTA file (path) or FASTA text (bytes) -> (ids int32 [B, T], mask uint8 [B, T], names),
        one row per record, on the GPU.  The text is scanned once on the host
        (``encoders.fasta_to_bytes``: no Python string per record), the sequences cross the bus as
        bytes, and the same kernels run as for ``encode_batch_device``.  Not in the reference,
        whose callers read their files into Python strings first (src/dna_tokenizer.py:2594-2651)."""
        self._require_ready()
        host, off_h, names = encoders.fasta_to_bytes(source, upper_case=bool(self.normalize_case))
        if not names:
            raise ValueError("No sequences provided for encoding.")
        lens = (off_h[1:] - off_h[:-1]).numpy()
        data, offsets = host.to(device, non_blocking=True), off_h.to(device)
        min_width = int(self.token_len or 0)

        class _Rows:                                     # strings of single rows, made only when asked for
            def __getitem__(self, i):
                return bytes(host[int(off_h[i]):int(off_h[i + 1])].numpy()).decode("ascii", errors="replace")

            def __len__(self):
                return len(names)

        rows = _Rows()
        if self.bpe_backend is not None:
            be = self.bpe_backend
            if getattr(be, "_normalize", None) is not None or getattr(be, "_input_guard", None) is not None:
                ids, mask = self.encode_batch_device([rows[i] for i in range(len(names))], device=device)
                return ids, mask, names
            t_cap = max(int(lens.max()), 1)
            try:
                tok, lengths = be._dnatok.tokenize_device(data, offsets, t_cap)
                ids, mask = self._pad_bpe_runs(tok, offsets, lengths, t_cap, dtype=torch.int32,
                                               min_width=min_width, pad_multiple=1)
            except Exception as e:
                self.log.warning("BPE backend failed (%s); falling back to the tokenizer.", e)
                ids, mask = self._tokenizer_rows_device([rows[i] for i in range(len(names))], device,
                                                        dtype=torch.int32, min_width=min_width, pad_multiple=1)
            return ids, mask, names
        if self._kmer_enc is not None:
            ids, mask = self._encode_kmer_device(rows, data, offsets, lens, dtype=torch.int32, min_width=min_width,
                                                 pad_multiple=1)
            return ids, mask, names
        width = max(int(lens.max()), min_width)
        ids, mask = self._char_enc.encode_padded(data, offsets, width, pad_left=(self.padding_side == "left"))
        return ids, mask, names

    def _pinned(self, nbytes: int) -> torch.Tensor:
        """The tokenizer's pinned host buffer for results on their way down (grown as needed; its
        content is copied out before the call that filled it returns)."""
        buf = getattr(self, "_pinned_buf", None)
        if buf is None or buf.numel() < nbytes:
            size = 1 << 20
            while size < nbytes:
                size *= 2
            buf = self._pinned_buf = torch.empty(size, dtype=torch.uint8, pin_memory=True)
        return buf

    def _encode_kmer_device(self, seqs, data, offsets, lens, *, dtype=torch.int32, min_width: int = 0,
                            pad_multiple: int = 1, host_ids: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
        """k-mer rows on the device.  Right padding to the longest row with int32 ids comes straight
        out of the encoder; any other layout (left padding, a least width, a multiple, a narrower id
        type) is one more launch of the packer over the encoder's rows.  Rows the tables cannot
        express (a window without tokens of its own, more tokens than the row's room, a foreign byte
        when those are not accepted, a row shorter than one window, which the reference hands to the
        tokenizer as well, src/dna_tokenizer.py:1389-1398) get the tokenizer's own answer."""
        k = int(self.kmer_k)
        left = self.padding_side == "left"
        n = len(lens)
        longest_in = int(lens.max())
        # room per row: every window may expand to the longest expansion of the table
        grow = max(int(self._kmer_tables.exp_len.max(initial=0)), 1)
        t_cap = (longest_in // k) * grow + k
        # a stride of whole 128-byte lines keeps every row of ids and of the mask on line boundaries
        t_cap += (-t_cap) % 128
        plain = (not left) and dtype == torch.int32 and pad_multiple <= 1
        # The width of the recent batches (encoders.WidthGuess, plus a margin) is a good guess of this
        # one's in a stream of batches: rows are padded that far while they are written, and the rows are laid out
        # that far apart (whole 128-byte lines), which makes the output nearly dense in memory
        # instead of a fifth of a worst-case buffer.  A batch that turns out wider than the guess
        # fills the stride to the last cell; it is then encoded again with room for the worst case.
        if not hasattr(self, "_kmer_widths"):
            self._kmer_widths = encoders.WidthGuess()
        guess = self._kmer_widths.next() if plain else 0
        worst = t_cap
        if guess:
            t_cap = min(worst, guess + (-guess) % 128)
        # lengths, status and the longest row share one allocation: one copy brings them to the host
        meta = torch.empty(2 * n + 1, dtype=torch.int32, device=data.device)

        def run(cap: int, guess: int):
            out = (torch.empty((n, cap), dtype=torch.int32, device=data.device),
                   torch.empty((n, cap), dtype=torch.uint8, device=data.device), meta[:n], meta[n:2 * n], meta[2 * n:])
            return self._kmer_enc.encode_padded(data, offsets, cap, fill_to=0, width_guess=guess, out=out)

        ids, mask, lengths, status, longest = run(t_cap, guess)
        staged = None
        if host_ids and plain and guess:
            # the ids start their way down before the width is known (the rows lie only the guess
            # apart, so little more than the answer is copied); the wait below covers both copies
            staged = self._pinned(n * t_cap * 4)[:n * t_cap * 4].view(torch.int32).view(n, t_cap)
            staged.copy_(ids, non_blocking=True)
        meta_h = meta.cpu().numpy()                      # (the one wait of the call)
        if plain:
            width = int(meta_h[2 * n])                   # the output shape
            if width >= t_cap and t_cap < worst:
                t_cap = worst
                staged = None
                ids, mask, lengths, status, longest = run(t_cap, 0)
                meta_h = meta.cpu().numpy()
                width = int(meta_h[2 * n])
            self._kmer_widths.update(width)
            plain = width >= min_width
        if not plain:
            cap = max(t_cap, int(min_width))
            if pad_multiple > 1 and cap % pad_multiple:
                cap += pad_multiple - cap % pad_multiple
            row_at = torch.arange(n, dtype=torch.int64, device=ids.device) * t_cap
            ids, mask, stats = encoders.pad_rows_as(ids.view(-1), row_at, lengths, int(self.id_pad), cap,
                                                    min_width=min_width, pad_multiple=pad_multiple, pad_left=left,
                                                    dtype=dtype)
            width = int(stats[1].item())
        ids, mask = ids[:, :width], mask[:, :width]
        self._staged_host_ids = staged[:, :width] if staged is not None and plain else None
        bad = meta_h[n:2 * n]
        need = (bad & (2 | 4)) != 0
        if self.require_valid_chars or not self.handle_invalid_chars:
            need |= (bad & 1) != 0
        need |= np.asarray(lens) < k
        if not getattr(self, "_kmer_tail_ok", True):
            need |= (np.asarray(lens) % k) != 0
        if need.any() and not self.allow_incomplete_kmer_lut:
            self._staged_host_ids = None
            rows = np.nonzero(need)[0].tolist()
            ids, mask = self._splice_tokenizer_rows(ids, mask, rows, self._tok_ids([seqs[i] for i in rows]),
                                                    pad_multiple=pad_multiple)
        return ids, mask

    def _splice_tokenizer_rows(self, ids: torch.Tensor, mask: torch.Tensor, rows: List[int],
                               fixed: List[List[int]], *, pad_multiple: int = 1):
        """Rows ``rows`` of a padded batch on the device get the tokenizer's own ids ``fixed``; the
        batch grows (on ``padding_side``) when one of them is longer than it is wide."""
        left = self.padding_side == "left"
        n, width = ids.shape
        new_w = max(width, max((len(r) for r in fixed), default=0))
        if pad_multiple > 1 and new_w % pad_multiple:
            new_w += pad_multiple - new_w % pad_multiple
        if new_w > width:
            extra = new_w - width
            pad_i = torch.full((n, extra), int(self.id_pad), dtype=ids.dtype, device=ids.device)
            pad_m = torch.zeros((n, extra), dtype=torch.uint8, device=ids.device)
            ids = torch.cat([pad_i, ids], dim=1) if left else torch.cat([ids, pad_i], dim=1)
            mask = torch.cat([pad_m, mask], dim=1) if left else torch.cat([mask, pad_m], dim=1)
        else:
            ids, mask = ids.clone(), mask.clone()
        for i, r in zip(rows, fixed):
            ids[i] = int(self.id_pad)
            mask[i] = 0
            if r:
                cur = torch.as_tensor(r, dtype=ids.dtype, device=ids.device)
                if left:
                    ids[i, new_w - len(r):] = cur
                    mask[i, new_w - len(r):] = 1
                else:
                    ids[i, :len(r)] = cur
                    mask[i, :len(r)] = 1
        return ids, mask

    def _tokenizer_rows_device(self, seqs: Sequence[str], device, *, dtype: torch.dtype, min_width: int,
                               pad_multiple: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """The whole batch through the tokenizer itself, laid out as the device paths lay it out
        (padding side, least width, multiple, id type): where a fast path ends when it cannot serve
        a batch (reference: _tokenize_batch_cpu, src/dna_tokenizer.py:1591-1777, 2100)."""
        fixed = self._tok_ids(seqs)
        width = max(max((len(r) for r in fixed), default=0), int(min_width))
        if pad_multiple > 1 and width % pad_multiple:
            width += pad_multiple - width % pad_multiple
        ids = torch.full((len(fixed), width), int(self.id_pad), dtype=dtype)
        mask = torch.zeros((len(fixed), width), dtype=torch.uint8)
        left = self.padding_side == "left"
        for i, r in enumerate(fixed):
            if r:
                cur = torch.as_tensor(r, dtype=dtype)
                if left:
                    ids[i, width - len(r):] = cur
                    mask[i, width - len(r):] = 1
                else:
                    ids[i, :len(r)] = cur
                    mask[i, :len(r)] = 1
        return ids.to(device), mask.to(device)

    def encode_batch_to_ids(self, seqs: List[str]) -> torch.Tensor:
        """CPU pinned int64 [B, T] (reference: 2049-2148)."""
        single = self.bpe_backend is None and self._kmer_enc is None
        ids, _ = self._encode_rows_device(seqs, "cuda", dtype=torch.int64 if single else torch.int32,
                                          min_width=int(self.token_len or 0), pad_multiple=1, host_ids=True)
        out = torch.empty(ids.shape, dtype=torch.int64, pin_memory=True)
        staged = self._staged_host_ids
        # k-mer and BPE ids came down inside the call (int32 -> int64 on the host); the character
        # tables write int64 themselves and are copied as they are
        out.copy_(staged if staged is not None else ids)
        return out

    def encode_batch_to_ids_staging(self, seqs: List[str], *, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        ids = self.encode_batch_to_ids(seqs)
        want = dtype or (torch.int32 if self.prefer_int32_h2d else torch.int64)
        return ids.to(want).pin_memory() if want != ids.dtype else ids

    def encode_batch_with_padding(self, seqs: List[str], max_tokens: int, pad_to_max: bool = False,
                                  pad_multiple: int = 16) -> Tuple[torch.Tensor, torch.Tensor]:
        """Truncate to max_tokens, pad to a multiple of pad_multiple tokens, smallest integer
        dtype that holds the vocabulary (reference: 2150-2236).  Returned on the GPU."""
        self._require_ready()
        if not seqs:
            raise ValueError("Empty batch")
        k = int(self.kmer_k) if self.kmer_k else 1
        max_chars = int(max_tokens) * k
        seqs = [s[:max_chars] for s in seqs]
        max_id = max(int(self.vocab_size) - 1, int(self.id_pad))
        narrow = _smallest_dtype(max_id)
        if self._char_enc is not None and self._kmer_enc is None and self.bpe_backend is None:
            # single-nucleotide tables: one kernel writes the final width, padding side and dtype
            data, offsets, lens = encoders.bytes_from_strings(seqs, "cuda")
            target = int(lens.max())
            if pad_to_max:
                target = max(target, int(max_tokens))
            if pad_multiple > 1 and target % pad_multiple:
                target += pad_multiple - target % pad_multiple
            return self._char_enc.encode_padded(data, offsets, target, pad_left=(self.padding_side == "left"),
                                                dtype=narrow)
        # k-mer and BPE: side, width and id type come out of the packer's launch
        return self._encode_rows_device(seqs, "cuda", dtype=narrow,
                                        min_width=int(max_tokens) if pad_to_max else 0,
                                        pad_multiple=int(pad_multiple))

    # ------------------------------------------------------------------ bytes path

    def encode_batch_to_ascii_bytes(self, seqs: List[str]) -> torch.Tensor:
        """Equal-length strings -> persistent pinned uint8 [B, T]; with ``normalize_case`` the
        bytes are upper-cased, with ``handle_invalid_chars`` (and no separate invalid id) bytes
        outside ACGTN become N (reference: 2594-2651).  One join, one native pass."""
        if not seqs:
            raise ValueError("No sequences provided for encoding.")
        t = len(seqs[0])
        if any(len(s) != t for s in seqs):
            raise ValueError("All sequences in a batch must have equal length.")
        buf = "".join(seqs).encode("ascii", errors="replace")
        need = len(seqs) * t
        if self._staging_bytes_cpu is None or self._staging_bytes_cpu.numel() < need:
            self._staging_bytes_cpu = torch.empty(max(need, 1), dtype=torch.uint8,
                                                  pin_memory=torch.cuda.is_available())
        out = self._staging_bytes_cpu[:need].view(len(seqs), t)
        out.copy_(torch.frombuffer(bytearray(buf), dtype=torch.uint8).view(len(seqs), t))
        to_n = self.handle_invalid_chars and (self.invalid_char_id is None or self.invalid_char_id == self.id_N)
        if self.normalize_case or to_n:
            encoders.clean_ascii_host(out, upper_case=self.normalize_case, invalid_to_n=to_n)
        return out

    def encode_batch_to_packed_2bit(self, seqs: List[str]) -> Tuple[torch.Tensor, int]:
        """Equal-length strings -> (pinned uint8 [B, ceil(T/4)], T): four bases per byte, first
        base in the low bits, A C G T = 0 1 2 3; N and every other byte travel as code 0
        (reference: 3143-3210).  A quarter of the bytes path's PCIe payload."""
        if not seqs:
            raise ValueError("No sequences provided.")
        ascii_rows = self.encode_batch_to_ascii_bytes(seqs)
        b, t = ascii_rows.shape
        tp = (t + 3) // 4
        if self._packed_2bit_cpu is None or tuple(self._packed_2bit_cpu.shape) != (b, tp):
            self._packed_2bit_cpu = torch.empty((b, tp), dtype=torch.uint8, pin_memory=torch.cuda.is_available())
        encoders.pack_2bit_host(ascii_rows, out=self._packed_2bit_cpu)
        return self._packed_2bit_cpu, t

    def _unpack_2bit(self, packed_cpu: torch.Tensor, t_true: int, device, dtype: torch.dtype) -> torch.Tensor:
        self._require_ready()
        if self._char_enc is None or self._kmer_enc is not None or self.bpe_backend is not None:
            raise RuntimeError("the 2-bit path serves single-nucleotide table tokenizers")
        if packed_cpu.dim() != 2 or packed_cpu.dtype != torch.uint8:
            raise TypeError("packed must be a uint8 [B, ceil(T/4)] tensor")
        packed = packed_cpu.to(device, non_blocking=True).contiguous()
        return self._char_enc.unpack_2bit(packed, int(t_true), dtype=dtype)

    def _unpack_2bit_to_ids_cuda(self, packed_cpu: torch.Tensor, T_true: int, device="cuda") -> torch.Tensor:
        """H2D of the packed bytes, then unpack + table lookup in one kernel -> int64 [B, T]
        (reference: 3212-3275)."""
        return self._unpack_2bit(packed_cpu, T_true, device, torch.int64)

    def _unpack_2bit_to_ids_cuda_u8(self, packed_cpu: torch.Tensor, T_true: int, device="cuda") -> torch.Tensor:
        """Same for vocabularies of at most 256 ids; the result is int64 like the reference's
        (3278-3330), written by the kernel directly."""
        if not self._ascii_lut_fits_uint8():
            raise RuntimeError("uint8 IDs path requires vocab <= 256.")
        return self._unpack_2bit(packed_cpu, T_true, device, torch.int64)

    def _ascii_lut_fits_uint8(self) -> bool:
        if self.ascii_lut is None:
            return False
        return int(np.max(self.ascii_lut, initial=0)) <= 255 and int(self.id_pad) <= 255

    def ids_from_ascii_bytes_cuda(self, u8_cpu: torch.Tensor, device="cuda") -> torch.Tensor:
        """uint8 [B, T] on the host -> int64 ids on the GPU (reference: 2653-2723, 2826-2940)."""
        self._require_ready()
        if self.bpe_backend is not None:
            raise RuntimeError("the bytes path serves table tokenizers; BPE goes through encode_batch_device")
        b, t = u8_cpu.shape
        data = u8_cpu.to(device, non_blocking=True).reshape(-1)
        offsets = torch.arange(b + 1, dtype=torch.int64, device=device) * t
        if self._kmer_enc is not None:
            t_cap = t + 4 + (-(t + 4)) % 128
            ids, mask, lengths, status, longest = self._kmer_enc.encode_padded(data, offsets, t_cap, fill_to=0)
            if bool((status & 7).any().item()):
                raise RuntimeError("k-mer bytes path: a row needs the tokenizer's own answer")
            return ids[:, :int(longest.item())].to(torch.int64)
        ids, _ = self._char_enc.encode_packed(data, row_len=t)
        return ids.view(b, t).to(torch.int64)

    def fused_tokenize_gather(self, ascii_bytes: torch.Tensor, embed_weight: torch.Tensor,
                              device="cuda") -> torch.Tensor:
        """``embed_weight[ascii_lut[ascii_bytes]]`` in one kernel: uint8 [B, T] (host or device)
        and a [V, D] device weight -> [B, T, D] of the weight's dtype; the id tensor is never
        written (reference: _fused_tokenize_gather, 3465-3532, a Triton kernel there).
        Single-nucleotide tokenizers only."""
        self._require_ready()
        if self._char_enc is None or self._kmer_enc is not None or self.bpe_backend is not None:
            raise RuntimeError("the fused kernel serves single-nucleotide table tokenizers")
        b, t = ascii_bytes.shape
        data = ascii_bytes.to(device, non_blocking=True).reshape(-1)
        weight = embed_weight if embed_weight.is_contiguous() else embed_weight.contiguous()
        # like the reference's kernel, this is weight[ascii_lut[bytes]]: the separate table for a
        # row's first character is not applied here
        out = self._char_enc.embed_packed(data, weight, row_len=0)
        return out.view(b, t, weight.shape[1])

    _fused_tokenize_gather = fused_tokenize_gather

    # ------------------------------------------------------------------ HIP graph

    def _record_cuda_graph(self, seqs_template: List[str], device="cuda", emb_batch: int = 0) -> None:
        """Capture the bytes -> ids kernel for one fixed [B, T] shape in a HIP graph: static
        uint8 input and int64 output buffers, one kernel node (the ids are written as int64 by
        the kernel, there is no cast node).  Replays take new bytes through
        ``_replay_cuda_graph`` (reference: 3382-3427).  Single-nucleotide tokenizers."""
        self._require_ready()
        if not torch.cuda.is_available():
            raise RuntimeError("HIP graphs need a GPU.")
        if self._char_enc is None or self._kmer_enc is not None or self.bpe_backend is not None:
            raise RuntimeError("the graph path serves single-nucleotide table tokenizers")
        dev = torch.device(device)
        ascii_cpu = self.encode_batch_to_ascii_bytes(seqs_template)
        b, t = int(ascii_cpu.shape[0]), int(ascii_cpu.shape[1])
        self._graph_shape = (b, t)
        self._graph_static_in = torch.empty((b, t), dtype=torch.uint8, device=dev)
        self._graph_static_out = torch.empty((b, t), dtype=torch.long, device=dev)
        self._graph_offsets = torch.arange(b + 1, dtype=torch.int64, device=dev) * t
        self._graph_static_in.copy_(ascii_cpu, non_blocking=True)
        side = torch.cuda.Stream(device=dev)                       # default priority
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):                              # warm-up outside the capture
            self._char_enc.encode_padded(self._graph_static_in.view(-1), self._graph_offsets, t, want_mask=False,
                                         dtype=torch.int64, ids=self._graph_static_out)
        torch.cuda.current_stream(dev).wait_stream(side)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._char_enc.encode_padded(self._graph_static_in.view(-1), self._graph_offsets, t, want_mask=False,
                                         dtype=torch.int64, ids=self._graph_static_out)

    def _replay_cuda_graph(self, ascii_cpu: torch.Tensor) -> torch.Tensor:
        """Copy new bytes into the graph's input buffer and replay it; returns the graph's
        output buffer, which the next replay overwrites (reference: 3429-3451)."""
        if getattr(self, "_graph", None) is None:
            raise RuntimeError("CUDA graph not recorded.")
        if tuple(ascii_cpu.shape) != self._graph_shape:
            raise ValueError(f"Graph shape mismatch: recorded {self._graph_shape}, got {tuple(ascii_cpu.shape)}")
        self._graph_static_in.copy_(ascii_cpu, non_blocking=True)
        self._graph.replay()
        return self._graph_static_out

    # ------------------------------------------------------------------ embedding

    def _embed_call(self, ids_dev: torch.Tensor) -> torch.Tensor:
        kwargs = {}
        try:
            if "rc_invariant" in inspect.signature(self.embedder.embed_tokens).parameters:
                kwargs["rc_invariant"] = False
        except (TypeError, ValueError):
            pass
        with torch.amp.autocast(device_type="cuda", dtype=torch.float16, enabled=ids_dev.is_cuda):
            out = self.embedder.embed_tokens(ids_dev, **kwargs)
        return out.float() if self.force_fp32_outputs and out.is_floating_point() else out

    def _ids_micro_bs_for_T(self, t: int, emb_batch: int) -> int:
        """Rows per embed call: emb_batch, capped so that a call holds at most
        ids_max_tokens_per_call tokens (reference: 2322-2339)."""
        cap = max(1, int(self.ids_max_tokens_per_call) // max(1, int(t)))
        return max(1, min(int(emb_batch), cap))

    def iter_embed_tokens_in_slices(self, ids: torch.Tensor, emb_batch: int, device) -> Iterator[torch.Tensor]:
        """One slice after the other on the current stream (reference: 2377-2452)."""
        dev = torch.device(device)
        if ids.dim() != 2 or ids.shape[0] == 0:
            return
        step = self._ids_micro_bs_for_T(int(ids.shape[1]), emb_batch)
        for s in range(0, ids.shape[0], step):
            chunk = ids[s:s + step].to(dev, dtype=torch.long, non_blocking=True)
            yield self._embed_call(chunk)

    def iter_embed_tokens_pipelined(self, ids_cpu: torch.Tensor, emb_batch: int, device="cuda", *,
                                    use_int32_h2d: Optional[bool] = None) -> Iterator[torch.Tensor]:
        """Two device buffers and a copy stream: the H2D copy of slice i+1 (int32 over the bus
        when ``use_int32_h2d``, widened on the device) runs while ``embed_tokens`` works on
        slice i (reference: 2454-2591).  A slice's buffer is handed out again only after the
        compute stream has passed the embed call that read it."""
        dev = torch.device(device)
        if dev.type != "cuda" or not torch.cuda.is_available() or ids_cpu.is_cuda:
            yield from self.iter_embed_tokens_in_slices(ids_cpu, emb_batch, device)
            return
        if ids_cpu.dim() != 2:
            raise ValueError("ids must be [B, T]")
        b, t = int(ids_cpu.shape[0]), int(ids_cpu.shape[1])
        if b == 0:
            return
        if use_int32_h2d is None:
            use_int32_h2d = self.prefer_int32_h2d
        wire = torch.int32 if use_int32_h2d else torch.int64
        src = ids_cpu if ids_cpu.dtype == wire else ids_cpu.to(wire)
        if not src.is_pinned():
            src = src.pin_memory()
        step = self._ids_micro_bs_for_T(t, emb_batch)
        if (self._dev_ping is None or self._dev_ping.device != dev or self._dev_ping.dtype != wire
                or self._dev_ping.shape[0] < step or self._dev_ping.shape[1] != t):
            self._dev_ping = torch.empty((step, t), dtype=wire, device=dev)
            self._dev_pong = torch.empty((step, t), dtype=wire, device=dev)
        bufs = (self._dev_ping, self._dev_pong)
        compute = torch.cuda.current_stream(dev)
        copy_stream = torch.cuda.Stream(device=dev)                 # default priority
        copied = (torch.cuda.Event(), torch.cuda.Event())
        consumed = (torch.cuda.Event(), torch.cuda.Event())
        starts = list(range(0, b, step))

        def schedule(i: int) -> None:
            lo = starts[i]
            hi = min(b, lo + step)
            which = i & 1
            with torch.cuda.stream(copy_stream):
                if i >= 2:
                    copy_stream.wait_event(consumed[which])         # the embed call that read it
                else:
                    copy_stream.wait_stream(compute)                # whatever used the buffers before
                bufs[which][:hi - lo].copy_(src[lo:hi], non_blocking=True)
                copied[which].record(copy_stream)

        schedule(0)
        if len(starts) > 1:
            schedule(1)
        for i, lo in enumerate(starts):
            hi = min(b, lo + step)
            which = i & 1
            compute.wait_event(copied[which])
            buf = bufs[which][:hi - lo]
            ids_dev = buf.to(torch.long)
            if ids_dev.data_ptr() != buf.data_ptr():                # widened copy: the buffer is free after it
                consumed[which].record(compute)
                if i + 2 < len(starts):
                    schedule(i + 2)
                out = self._embed_call(ids_dev)
            else:                                                   # embed_tokens reads the buffer itself
                out = self._embed_call(ids_dev)
                consumed[which].record(compute)
                if i + 2 < len(starts):
                    schedule(i + 2)
            yield out
        compute.wait_stream(copy_stream)

    def embed_from_strings(self, seqs: List[str], emb_batch: int, device, *, path: str = "ids"
                           ) -> Iterator[torch.Tensor]:
        """Tokenize on the GPU, then feed ``embedder.embed_tokens`` in slices of emb_batch rows
        on ``device`` (reference: 2962-3110).  ``path`` = "ids" | "bytes" select the same
        kernels; "bytes" falls back to "ids" when a row needs the tokenizer's own answer."""
        self._require_ready()
        if path == "bytes" and self.bpe_backend is None and len({len(s) for s in seqs}) == 1:
            try:
                ids = self.ids_from_ascii_bytes_cuda(self.encode_batch_to_ascii_bytes(seqs))
                if self.token_len is not None and self.token_len > ids.shape[1]:
                    raise RuntimeError("needs padding")
                yield from self.iter_embed_tokens_in_slices(ids, emb_batch, device)
                return
            except RuntimeError:
                pass
        ids, _ = self.encode_batch_device(seqs)
        yield from self.iter_embed_tokens_in_slices(ids, emb_batch, device)
