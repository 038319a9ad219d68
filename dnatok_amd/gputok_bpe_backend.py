"""``GPUTokBPEBackend``: HF-compatible BPE encode on the MI355X engine.

Same surface as the reference's ``gputok_bpe_backend`` module
(src/gputok_bpe_backend.py): the constructor takes a Hugging Face tokenizer,
reads its ``tokenizer.json``, compiles the normalizer, materialises merges.txt
and builds the kernel-id -> HF-id remap; ``encode_batch`` returns
``(input_ids int64 [B, L], attention_mask uint8 [B, L])`` on the device, padded
with the tokenizer's pad id to the longest row, with ids identical to
``hf_tokenizer(seqs, add_special_tokens=False)``.

What differs from the reference underneath: remap, padding and mask are fused
into one packer kernel, nothing is routed to the CPU tokenizer by length (the
engine has no length pathology), and negative per-row lengths raise instead of
silently becoming all-pad rows.
"""
from __future__ import annotations

import hashlib
import json
import os
import re as _re
from pathlib import Path
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib, bpe_vocab, encoders


# ------------------------------------------------------------------ tokenizer.json

def _read_tokenizer_json(hf_tokenizer: Any) -> Optional[Dict[str, Any]]:
    """tokenizer.json of an HF tokenizer: a local path in ``name_or_path`` / ``vocab_file``,
    else the in-memory spec of a ``tokenizers`` object (``to_str``), directly or through
    ``backend_tokenizer`` (reference: src/gputok_bpe_backend.py:132-176; the hub-cache
    lookup is left out: there is no network path in this backend)."""
    for attr in ("name_or_path", "vocab_file"):
        base = getattr(hf_tokenizer, attr, None)
        if isinstance(base, str) and base:
            for cand in (os.path.join(base, "tokenizer.json"), base):
                if os.path.isfile(cand) and cand.endswith("tokenizer.json"):
                    with open(cand) as fh:
                        return json.load(fh)
    for obj in (getattr(hf_tokenizer, "backend_tokenizer", None), hf_tokenizer):
        to_str = getattr(obj, "to_str", None)
        if callable(to_str):
            try:
                return json.loads(to_str())
            except Exception:
                continue
    return None


def _compile_normalizer_step(step: Dict[str, Any]) -> Optional[Callable[[str], str]]:
    """One HF normalizer step as a str -> str callable, or None when it cannot be reproduced
    (reference: src/gputok_bpe_backend.py:179-236)."""
    if not isinstance(step, dict):
        return None
    kind = step.get("type")
    if kind == "Strip":
        left = bool(step.get("strip_left", True))
        right = bool(step.get("strip_right", True))
        if left and right:
            return lambda s: s.strip()
        if left:
            return lambda s: s.lstrip()
        if right:
            return lambda s: s.rstrip()
        return lambda s: s
    if kind == "Replace":
        pattern = step.get("pattern")
        content = str(step.get("content", ""))
        if isinstance(pattern, dict) and "String" in pattern:
            literal = pattern["String"]
            return lambda s: s.replace(literal, content)
        if isinstance(pattern, dict) and "Regex" in pattern:
            rx = _re.compile(pattern["Regex"])
            return lambda s: rx.sub(content, s)
        return None
    if kind == "Prepend":
        prefix = str(step.get("prepend", ""))
        return lambda s: prefix + s
    if kind == "Lowercase":
        return lambda s: s.lower()
    if kind in (None, "NFC", "NFKC", "NFD", "NFKD", "StripAccents"):
        return lambda s: s            # identity on ASCII DNA
    if kind == "Sequence":
        parts = [_compile_normalizer_step(sub) for sub in step.get("normalizers", [])]
        if any(p is None for p in parts):
            return None

        def run(s: str) -> str:
            for p in parts:
                s = p(s)
            return s
        return run
    return None


def _compile_normalizer(cfg: Dict[str, Any]) -> Optional[Callable[[str], str]]:
    norm = cfg.get("normalizer")
    if norm is None:
        return None
    fn = _compile_normalizer_step(norm)
    if fn is None:
        raise ValueError(f"Unsupported normalizer config: {norm.get('type')!r}")
    return fn


_PLAIN = _re.compile(r"[A-Za-z0-9_ \-]")
_RUN_RX = _re.compile(r"^(\\?.)(?:\{(\d+),\}|\+)$", _re.S)


def _has_border(p: bytes) -> bool:
    return any(p[:k] == p[len(p) - k:] for k in range(1, len(p)))


def _device_steps_of(step: Dict[str, Any]) -> Optional[List[_lib.NormStep]]:
    """One HF normalizer step as device steps (C ABI: dnatok_norm_step), or None when the
    device pass cannot express it: a regex other than ``^``, ``c{n,}``, ``c+`` or a plain
    literal, a literal that overlaps itself or is empty, anything longer than 16 bytes.  The
    device steps act on the UTF-8 bytes of ASCII rows exactly as the callables of
    ``_compile_normalizer_step`` act on the strings."""
    if not isinstance(step, dict):
        return None
    kind = step.get("type")
    try:
        if kind == "Strip":
            flags = (1 if step.get("strip_left", True) else 0) | (2 if step.get("strip_right", True) else 0)
            return [_lib.NormStep.make(_lib.NORM_STRIP, flags)] if flags else []
        if kind == "Replace":
            pattern = step.get("pattern")
            content = str(step.get("content", "")).encode("utf-8")
            if isinstance(pattern, dict) and "String" in pattern:
                lit = str(pattern["String"]).encode("utf-8")
                if not lit or _has_border(lit) or not lit.isascii():
                    return None
                return [_lib.NormStep.make(_lib.NORM_REPLACE, 0, lit, content)]
            if isinstance(pattern, dict) and "Regex" in pattern:
                rx = str(pattern["Regex"])
                if b"\\" in content:                      # group references / escapes in the replacement
                    return None
                if rx == "^":
                    return [_lib.NormStep.make(_lib.NORM_PREPEND, 0, b"", content)]
                m = _RUN_RX.match(rx)
                if m:
                    ch = m.group(1)
                    if len(ch) == 2:                        # escaped: only punctuation escapes are literal
                        ch = ch[1] if not ch[1].isalnum() else ""
                    elif not _PLAIN.fullmatch(ch):
                        ch = ""
                    n = int(m.group(2)) if m.group(2) is not None else 1
                    if len(ch) == 1 and ch.isascii() and 1 <= n <= 64:
                        return [_lib.NormStep.make(_lib.NORM_REPLACE_RUN, n, ch.encode(), content)]
                    return None
                if rx and all(_PLAIN.fullmatch(c) for c in rx) and not _has_border(rx.encode()):
                    return [_lib.NormStep.make(_lib.NORM_REPLACE, 0, rx.encode(), content)]
            return None
        if kind == "Prepend":
            return [_lib.NormStep.make(_lib.NORM_PREPEND, 0, b"", str(step.get("prepend", "")).encode("utf-8"))]
        if kind == "Lowercase":
            return [_lib.NormStep.make(_lib.NORM_LOWERCASE)]
        if kind in (None, "NFC", "NFKC", "NFD", "NFKD", "StripAccents"):
            return []
        if kind == "Sequence":
            out: List[_lib.NormStep] = []
            for sub in step.get("normalizers", []):
                part = _device_steps_of(sub)
                if part is None:
                    return None
                out.extend(part)
            return out
    except ValueError:                                      # longer than the step record holds
        return None
    return None


def _compile_device_normalizer(cfg: Dict[str, Any]) -> Optional["encoders.RowNormalizer"]:
    """The tokenizer's normalizer as a device program, or None (no normalizer, or one the
    device pass cannot express: the host callables are used then)."""
    norm = cfg.get("normalizer")
    if norm is None:
        return None
    steps = _device_steps_of(norm)
    if steps is None:
        return None
    return encoders.RowNormalizer(steps)


def _extract_merges(cfg: Dict[str, Any]) -> List[str]:
    """Merges as ``"a b"`` strings in rank order (reference: 251-262)."""
    out: List[str] = []
    for m in cfg.get("model", {}).get("merges", []):
        if isinstance(m, str):
            out.append(m)
        elif isinstance(m, (list, tuple)) and len(m) == 2:
            out.append(f"{m[0]} {m[1]}")
        else:
            raise ValueError(f"Unrecognised merge entry: {m!r}")
    return out


_SPLIT_WHITESPACE_REGEX = {r"\s+", r"\s", " +", " ", r"\n", r"\n+", r"[ \t\n]+", r"[\s]+"}


def _pre_tokenizer_reason(pre: Any, model: Dict[str, Any]) -> Optional[str]:
    """None when the pre-tokenizer leaves a row without white space in one piece (or in pieces the
    merges never join anyway), else why not."""
    if pre is None:
        return None
    kind = pre.get("type") if isinstance(pre, dict) else None
    if kind in (None, "WhitespaceSplit"):
        return None
    if kind == "Whitespace":
        # \w+|[^\w\s]+ also cuts between word characters and punctuation: the same as no cut only
        # when no merge rule spans such a border
        for m in model.get("merges", []):
            a, b = (m.split() + ["", ""])[:2] if isinstance(m, str) else (str(m[0]), str(m[1]))
            word = [bool(_re.match(r"\w", c)) for c in a + b]
            if any(x != word[0] for x in word):
                return "pre_tokenizer='Whitespace' with a merge rule across a word / punctuation border"
        return None
    if kind == "Split":
        pattern = pre.get("pattern") or {}
        if pre.get("invert", False):
            return "pre_tokenizer='Split' with invert"
        if "String" in pattern and pattern["String"] and pattern["String"].isspace():
            return None
        if pattern.get("Regex") in _SPLIT_WHITESPACE_REGEX:
            return None
        return f"pre_tokenizer='Split' on {pattern!r} (only white-space patterns are reproduced)"
    return f"pre_tokenizer={kind!r}"


def _supported_tokenizer(cfg: Optional[Dict[str, Any]]) -> Tuple[bool, str]:
    """(ok, reason): a BPE model whose ids this engine reproduces bit for bit.  Refused: another
    model type; a pre-tokenizer that can cut a row without white space; a normalizer that is not
    reproduced; and the BPE options that change the ids -- dropout, byte_fallback, ignore_merges,
    fuse_unk, a continuing_subword_prefix or end_of_word_suffix.  (The reference's gate looks at
    model type, pre-tokenizer type and normalizer only, src/gputok_bpe_backend.py:265-295, and
    encodes such a tokenizer as if the options were off.)"""
    if cfg is None:
        return False, "tokenizer.json not found"
    model = cfg.get("model") or {}
    if model.get("type") != "BPE":
        return False, f"model.type={model.get('type')!r} (only BPE supported)"
    if model.get("dropout"):
        return False, f"model.dropout={model.get('dropout')!r} (merges are skipped at random)"
    for flag in ("byte_fallback", "ignore_merges", "fuse_unk"):
        if model.get(flag):
            return False, f"model.{flag}=true changes the ids"
    for affix in ("continuing_subword_prefix", "end_of_word_suffix"):
        if model.get(affix):
            return False, f"model.{affix}={model.get(affix)!r} changes the symbols"
    reason = _pre_tokenizer_reason(cfg.get("pre_tokenizer"), model)
    if reason is not None:
        return False, reason
    norm = cfg.get("normalizer")
    if norm is not None and _compile_normalizer_step(norm) is None:
        return False, f"unsupported normalizer={norm.get('type')!r}"
    return True, "ok"


def _cache_dir() -> Path:
    p = Path(os.environ.get("DNATOK_GPUTOK_CACHE", str(Path.home() / ".cache" / "dnatok-gputok")))
    p.mkdir(parents=True, exist_ok=True)
    return p


def _merges_cache_path(merges: Sequence[str]) -> Path:
    h = hashlib.sha256()
    for m in merges:
        h.update(m.encode("utf-8"))
        h.update(b"\n")
    return _cache_dir() / f"merges_{h.hexdigest()[:16]}.txt"


def _reconstruct_gputok_vocab(merges: Sequence[str]) -> List[str]:
    """Kernel id -> token string (reference: 358-393)."""
    return list(bpe_vocab.KernelVocab(bpe_vocab.split_merges(merges)).id_to_token)


# ------------------------------------------------------------------------- backend

class UnsupportedRows(ValueError):
    """Rows of a batch that the tokenizer cuts or drops characters from (white space with a
    pre-tokenizer, a character outside the vocabulary without unk_token), which the engine does
    not reproduce.  ``rows`` holds their indices in the batch, in rising order: a caller that
    owns the tokenizer (DNATok) encodes those rows with it and the others on the GPU."""

    def __init__(self, rows: List[int], message: str) -> None:
        super().__init__(message)
        self.rows = list(rows)


class GPUTokBPEBackend:
    """HF-compatible GPU BPE encoder (reference: src/gputok_bpe_backend.py:396-679)."""

    def __init__(self, hf_tokenizer: Any, *, engine: str = "dnatok") -> None:
        if engine not in ("gputok", "dnatok"):
            raise ValueError(f"engine must be 'gputok' or 'dnatok', got {engine!r}")
        if engine == "gputok":
            raise RuntimeError("engine='gputok' is the reference's third-party comparison kernel; "
                               "this backend ships the 'dnatok' engine only")
        self.tokenizer = hf_tokenizer
        self.engine = engine
        self.normalize_on_device = True
        cfg = _read_tokenizer_json(hf_tokenizer)
        ok, reason = _supported_tokenizer(cfg)
        if not ok:
            raise RuntimeError(f"GPUTokBPEBackend cannot accelerate this tokenizer: {reason}")
        self._normalize = _compile_normalizer(cfg)
        # the same steps as a device program, used for all-ASCII batches; None: host callables
        self._normalize_device = _compile_device_normalizer(cfg) if self._normalize is not None else None
        # What the engine cannot reproduce depends on the input for two kinds of tokenizer: with a
        # pre-tokenizer, white space inside a row cuts it into words (and is dropped); without an
        # unk_token, characters outside the vocabulary are dropped.  Such input raises UnsupportedRows
        # (a ValueError naming the rows; DNATok catches it and gives those rows to the tokenizer
        # itself, the reference's fallback of src/dna_tokenizer.py:2066-2100 row by row).
        self._input_guard: Optional[_re.Pattern] = None
        guard = []
        if cfg.get("pre_tokenizer") is not None:
            guard.append(r"\s")
        if (cfg.get("model") or {}).get("unk_token") is None:
            singles = "".join(_re.escape(t) for t in (cfg.get("model") or {}).get("vocab", {}) if len(t) == 1)
            guard.append(f"[^{singles}]" if singles else ".")
        if guard:
            self._input_guard = _re.compile("|".join(guard), _re.S)
        self._merges: List[str] = _extract_merges(cfg)
        if not self._merges:
            raise RuntimeError("Tokenizer has no merges; nothing to accelerate.")
        path = _merges_cache_path(self._merges)
        if not path.exists():
            with open(path, "w") as fh:
                fh.write("#version: 0.2\n")
                for m in self._merges:
                    fh.write(m + "\n")
        self._merges_path = str(path)

        from .dnatok_bpe_kernel import DnatokBpeKernel
        self._dnatok = DnatokBpeKernel(self._merges_path, max_iters=1024)

        model = cfg.get("model", {})
        get_vocab = getattr(hf_tokenizer, "get_vocab", None)
        hf_vocab = get_vocab() if callable(get_vocab) else dict(model.get("vocab", {}))
        unk_id = getattr(hf_tokenizer, "unk_token_id", None)
        if unk_id is None:
            unk_tok = model.get("unk_token")
            unk_id = hf_vocab.get(unk_tok, 0) if unk_tok is not None else 0
        self.unk_id = int(unk_id or 0)
        pad_id = getattr(hf_tokenizer, "pad_token_id", None)
        if pad_id is None:
            pad = (cfg.get("padding") or {})
            pad_id = pad.get("pad_id", hf_vocab.get("[PAD]", hf_vocab.get("<pad>", 0)))
        self.pad_id = int(pad_id or 0)
        kvocab = self._dnatok._impl.vocab
        remap = kvocab.remap_to(hf_vocab, self.unk_id)
        self._n_unmapped = int(sum(1 for t in kvocab.id_to_token if t not in hf_vocab))
        self._remap_cpu = torch.from_numpy(remap.astype("int64"))          # int64 [V_kernel]
        self._remap_i32 = torch.from_numpy(remap)                          # int32, what the packer reads
        self._remap_cuda: Optional[torch.Tensor] = None
        self._widths = encoders.WidthGuess()           # how wide the recent batches came out (padded_device)
        size = getattr(hf_tokenizer, "vocab_size", None)
        if callable(size):
            size = None
        if size is None:
            gvs = getattr(hf_tokenizer, "get_vocab_size", None)
            size = gvs() if callable(gvs) else len(hf_vocab)
        self.vocab_size = int(size or len(hf_vocab))

    @staticmethod
    def is_supported(hf_tokenizer: Any) -> bool:
        try:
            ok, _ = _supported_tokenizer(_read_tokenizer_json(hf_tokenizer))
            return ok
        except Exception:
            return False

    # -------------------------------------------------------------- device-resident path

    def _remap_on(self, dev: torch.device) -> torch.Tensor:
        if self._remap_cuda is None or self._remap_cuda.device != dev:
            self._remap_cuda = self._remap_i32.to(dev)
        return self._remap_cuda

    def encode_device(self, data: torch.Tensor, offsets: torch.Tensor, max_len: int, *,
                      packed: bool = False):
        """Bytes already on the device (uint8 [total] + int64 offsets [B+1]).

        padded (default): ``(ids int32 [B, max_len], mask uint8 [B, max_len], lengths int32 [B],
        longest int32 [1])`` -- rows are padded to the longest row found on the device, view
        ``ids[:, :longest]``.  packed: ``(ids int32 [cap], out_offsets int64 [B+1], mask)``.
        No host synchronisation either way.
        """
        tok, lengths = self._dnatok.tokenize_device(data, offsets, max_len)
        remap = self._remap_on(data.device)
        if packed:
            return encoders.pack_ragged(tok, offsets, lengths, remap=remap)
        ids, mask, longest = encoders.pad_rows(tok, offsets, lengths, self.pad_id, max(int(max_len), 1),
                                               fill_to=0, remap=remap)
        return ids, mask, lengths, longest

    # ------------------------------------------------------------------- reference API

    def bytes_device(self, seqs: List[str], *, device: object = "cuda"):
        """Strings -> what the engine reads: ``(data uint8, offsets int64 [B+1], t_cap)`` on the
        device, normalizer applied (on the device where its steps allow), t_cap a host-known bound
        of the row lengths in bytes."""
        if not seqs:
            raise ValueError("No sequences provided.")
        dev = torch.device(device) if not isinstance(device, torch.device) else device
        if dev.type != "cuda":
            raise RuntimeError("GPUTokBPEBackend.encode_batch runs on the GPU only (device='cuda')")
        if self._input_guard is not None:
            if self._normalize is not None:
                seqs = [self._normalize(s) for s in seqs]
            hit = self._input_guard.search("".join(seqs))
            if hit is not None:
                rows = [i for i, s in enumerate(seqs) if self._input_guard.search(s) is not None]
                raise UnsupportedRows(rows, f"character {hit.group(0)!r} (row {rows[0]}; {len(rows)} of "
                                      f"{len(seqs)} rows) is cut or dropped by this tokenizer (pre-tokenizer / "
                                      "no unk_token); not reproduced by the GPU engine")
        if self._normalize is None or self._input_guard is not None:
            data, offsets, lens = encoders.bytes_from_strings(seqs, dev, encoding="utf-8")
            t_cap = int(lens.max())
        elif self._normalize_device is not None and self.normalize_on_device and "".join(seqs).isascii():
            # raw bytes up, normalizer steps as compaction passes on the device; the sizes after
            # them stay on the device, the engine is sized by their upper bounds
            data, offsets, lens = encoders.bytes_from_strings(seqs, dev, encoding="utf-8")
            data, offsets, _, t_cap = self._normalize_device.apply(data, offsets, int(lens.sum()), int(lens.max()))
        else:
            norm = [self._normalize(s) for s in seqs]
            data, offsets, lens = encoders.bytes_from_strings(norm, dev, encoding="utf-8")
            t_cap = int(lens.max())
        return data, offsets, max(t_cap, 1)

    def tokens_device(self, seqs: List[str], *, device: object = "cuda", meta_tail: int = 0):
        """Strings -> the engine's token runs on the device: ``(tok_tmp int32, offsets int64 [B+1],
        lengths int32 [B], t_cap)`` with row b's kernel-space tokens at
        ``tok_tmp[offsets[b] : offsets[b] + lengths[b]]`` and t_cap a host-known bound of the row
        lengths.  DNATok pads these runs its own way where the engine's own padding does not fit (padding
        on the left, narrow id types).  With
        ``meta_tail`` > 0 the lengths are the head of an int32 allocation with that many more
        entries behind them (for the padding's statistics: one copy then brings both to the host)."""
        data, offsets, t_cap = self.bytes_device(seqs, device=device)
        n = offsets.numel() - 1
        lengths = torch.empty(n + int(meta_tail), dtype=torch.int32, device=data.device)[:n] if meta_tail else None
        tok, lengths = self._dnatok.tokenize_device(data, offsets, t_cap, lengths=lengths)
        return tok, offsets, lengths, t_cap

    def padded_device(self, seqs: List[str], *, device: object = "cuda", min_width: int = 0,
                      pad_multiple: int = 1, stage_ids=None, pad_left: bool = False,
                      dtype: torch.dtype = torch.int32) -> Tuple[torch.Tensor, torch.Tensor]:
        """Strings -> ``(ids [B, T] of dtype, mask uint8 [B, T])`` on the device, tokenizer ids, padded
        with ``pad_id`` (on the right, or with ``pad_left`` on the left) to the longest row (at least
        ``min_width``, a multiple of ``pad_multiple``): one engine launch writes the padded rows in
        their final type and on their final side (``dnatok_bpe_encode_padded_as``),
        one copy brings the lengths to the host.  The rows are laid out only as
        far apart as the recent batches of this backend were wide (``encoders.WidthGuess``); a batch
        that needs more room is encoded again with room for the worst case (a token per byte).
        ``stage_ids``: a callable ``(ids) -> None`` run before the wait when the layout was not the
        worst-case one (DNATok copies the ids to pinned memory there)."""
        data, offsets, t_cap = self.bytes_device(seqs, device=device)
        dev = data.device
        n = offsets.numel() - 1

        def rounded(w: int) -> int:
            return w + (-w) % pad_multiple if pad_multiple > 1 else w

        worst = rounded(max(int(t_cap), int(min_width), 1))
        guess = self._widths.next()
        cap = min(rounded(max(guess + (-guess) % 32, int(min_width))), worst) if guess else worst
        lengths = torch.empty(n, dtype=torch.int32, device=dev)
        while True:
            # (no longest row from the device: the lengths come down anyway, and the launch ends earlier without it)
            out = (torch.empty((n, cap), dtype=dtype, device=dev),
                   torch.empty((n, cap), dtype=torch.uint8, device=dev), lengths, None)
            ids, mask, _, _ = self._dnatok.tokenize_padded_device(data, offsets, t_cap, cap, int(self.pad_id),
                                                                  remap=self._remap_on(dev), out=out, pad_left=pad_left)
            if stage_ids is not None and cap < worst:
                stage_ids(ids)
            lengths_h = lengths.cpu().numpy()                            # (the one wait)
            longest, shortest = int(lengths_h.max()), int(lengths_h.min())
            if shortest < 0:
                raise RuntimeError("BPE engine reported a failed row (negative length)")
            if longest <= cap:
                break
            cap = worst                                  # a row was cut: once more, with room for all
        self._widths.update(longest)
        width = min(rounded(max(longest, int(min_width))), cap)
        if pad_left:                                     # (the rows' tokens end at the stride's last cell)
            return ids[:, cap - width:], mask[:, cap - width:]
        return ids[:, :width], mask[:, :width]

    def encode_batch(self, seqs: List[str], *, device: object = "cuda"
                     ) -> Tuple[torch.Tensor, torch.Tensor]:
        """(ids int64 [B, L] padded with the tokenizer's pad id, mask uint8 [B, L]), as the reference
        returns them (src/gputok_bpe_backend.py:489, 581-600); the engine writes int64 itself."""
        ids, mask = self.padded_device(seqs, device=device, dtype=torch.long)
        return ids, mask

    def encode_batch_ids_only(self, seqs: List[str], *, device: object = "cuda") -> torch.Tensor:
        ids, _ = self.encode_batch(seqs, device=device)
        return ids
