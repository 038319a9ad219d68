"""Device-side encoders: thin torch-tensor wrappers over the C ABI.

torch is used for device memory and the current stream only; every encode is a
call into libdnatok_hip.so on ``torch.cuda.current_stream()``.  Inputs are
device uint8 buffers plus int64 row offsets (the layout
``workloads.Batch`` / ``bytes_from_strings`` produce); outputs are int32 ids
and uint8 masks that stay on the device.
"""
from __future__ import annotations

import ctypes
import threading
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    # torch's current stream as the raw handle the C ABI takes (the Stream object of
    # torch.cuda.current_stream() costs ten times as much to build, on every call)
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _np_ptr(a: Optional[np.ndarray]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if a is None else a.ctypes.data)


def _require_cuda(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if not t.is_cuda or t.dtype != dtype or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous {dtype} tensor on the GPU")


try:                                    # the C packer is host code; without it the strings are joined in Python
    from . import _hostpack
except ImportError:                     # pragma: no cover
    _hostpack = None


class _PinnedStage(threading.local):
    """Per thread: a pinned host buffer the packer writes into, and the event that says when the
    last copy out of it has finished."""
    buf: Optional[torch.Tensor] = None
    event = None


_stage = _PinnedStage()


def _pack_to_device(seqs: Sequence[str], device, utf8: bool):
    """Strings -> pinned buffer (offsets, then bytes, written by the C packer) -> one copy to the
    device.  Returns (data, offsets, host_lengths) as views of one device allocation."""
    st = _stage
    if st.event is not None:
        st.event.synchronize()                   # the previous batch has left the buffer
    if st.buf is None:
        st.buf = torch.empty(1 << 20, dtype=torch.uint8, pin_memory=True)
    r = _hostpack.pack_strings(seqs, st.buf.data_ptr(), st.buf.numel(), int(utf8))
    if isinstance(r, int):                       # too small: -r bytes are needed
        size = 1 << 20
        while size < -r:
            size *= 2
        st.buf = torch.empty(size, dtype=torch.uint8, pin_memory=True)
        r = _hostpack.pack_strings(seqs, st.buf.data_ptr(), st.buf.numel(), int(utf8))
    n, total, _, bytes_at = r
    used = bytes_at + total
    dev = torch.empty(used, dtype=torch.uint8, device=device)
    dev.copy_(st.buf[:used], non_blocking=True)
    if st.event is None:
        st.event = torch.cuda.Event()
    st.event.record()
    lens = np.diff(st.buf[:8 * (n + 1)].view(torch.int64).numpy())
    return dev[bytes_at:used], dev[:8 * (n + 1)].view(torch.int64), lens


def bytes_from_strings(seqs: Sequence[str], device="cuda", encoding: str = "ascii"
                       ) -> Tuple[torch.Tensor, torch.Tensor, np.ndarray]:
    """Concatenate strings into one device uint8 buffer + device int64 offsets.

    Returns (data, offsets, host_lengths).  The rows' bytes and their offsets are written into a
    pinned buffer by one pass in C and cross the bus in one copy
    (reference: DNATokBPE::tokenize_batch, src/dnatok_bpe_kernel/dnatok_bpe.cu:872-887).
    ``encoding`` = "ascii": one byte per character, non-ASCII characters become ``?`` (what the
    table paths of the reference do, src/dna_tokenizer.py:1793); "utf-8": the bytes the
    reference's BPE kernel sees, since its binding receives ``std::string``.
    """
    if _hostpack is not None and torch.device(device).type == "cuda":
        return _pack_to_device(seqs, device, encoding == "utf-8")
    joined = "".join(seqs)
    if encoding == "utf-8" and not joined.isascii():
        parts = [s.encode("utf-8") for s in seqs]
        lens = np.fromiter((len(p) for p in parts), dtype=np.int64, count=len(parts))
        buf = b"".join(parts)
    else:
        lens = np.fromiter((len(s) for s in seqs), dtype=np.int64, count=len(seqs))
        buf = joined.encode("ascii", errors="replace")
    offsets = np.zeros(len(seqs) + 1, dtype=np.int64)
    np.cumsum(lens, out=offsets[1:])
    host = torch.frombuffer(bytearray(buf), dtype=torch.uint8) if buf else torch.empty(0, dtype=torch.uint8)
    data = host.to(device)
    return data, torch.from_numpy(offsets).to(device), lens


def clean_ascii_host(buf: torch.Tensor, *, upper_case: bool, invalid_to_n: bool) -> int:
    """In place on a contiguous host uint8 tensor: a-z -> A-Z, then bytes outside ACGTN -> 'N'
    (one pass; reference: DNATok._encode_ascii_bytes_impl, src/dna_tokenizer.py:2637-2649).
    Returns how many bytes were replaced."""
    if buf.is_cuda or buf.dtype != torch.uint8 or not buf.is_contiguous():
        raise ValueError("buf must be a contiguous uint8 tensor on the host")
    n = ctypes.c_int64(0)
    _lib.check(_lib.lib().dnatok_host_clean_ascii(ctypes.c_void_p(buf.data_ptr()), buf.numel(), int(upper_case),
                                                  int(invalid_to_n), ctypes.byref(n)),
               "dnatok_host_clean_ascii")
    return int(n.value)


def pack_2bit_host(ascii_rows: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Host uint8 [B, T] ASCII -> host uint8 [B, ceil(T/4)], four bases per byte, first base in
    the low bits, A C G T = 0 1 2 3, anything else 0 (reference:
    DNATok.encode_batch_to_packed_2bit, src/dna_tokenizer.py:3143-3210)."""
    if ascii_rows.is_cuda or ascii_rows.dtype != torch.uint8 or ascii_rows.dim() != 2 or not ascii_rows.is_contiguous():
        raise ValueError("ascii_rows must be a contiguous uint8 [B, T] tensor on the host")
    b, t = ascii_rows.shape
    tp = (t + 3) // 4
    if out is None:
        out = torch.empty((b, tp), dtype=torch.uint8, pin_memory=torch.cuda.is_available())
    if tuple(out.shape) != (b, tp) or out.is_cuda or out.dtype != torch.uint8 or not out.is_contiguous():
        raise ValueError("out must be a contiguous uint8 [B, ceil(T/4)] tensor on the host")
    _lib.check(_lib.lib().dnatok_host_pack_2bit(ctypes.c_void_p(ascii_rows.data_ptr()), b, t,
                                                ctypes.c_void_p(out.data_ptr())),
               "dnatok_host_pack_2bit")
    return out


def fasta_to_bytes(source, device=None, *, upper_case: bool = False):
    """FASTA text -> (data uint8 [total], offsets int64 [n + 1], names) in the layout the encoders take.

    ``source``: a path, or the text itself as bytes / bytearray / memoryview / a host uint8 array.
    A path is memory-mapped, so the file is read once, by the scan.  The sequences land in pinned
    host memory when a GPU is present and are copied to ``device`` (default: stay on the host).
    ``names`` is a list of the header lines (without '>'); bases in front of the first header
    form a record named "" (C ABI: dnatok_host_fasta_scan)."""
    if isinstance(source, (str, bytes, bytearray, memoryview, np.ndarray)) and not isinstance(source, str):
        text = np.frombuffer(source, dtype=np.uint8) if not isinstance(source, np.ndarray) else source
    else:
        import os
        text = np.memmap(os.fspath(source), dtype=np.uint8, mode="r") if os.path.getsize(os.fspath(source)) else \
            np.empty(0, dtype=np.uint8)
    text = np.ascontiguousarray(text, dtype=np.uint8)
    n_rec, n_bases = ctypes.c_int64(0), ctypes.c_int64(0)
    L = _lib.lib()
    ptr = ctypes.c_void_p(text.ctypes.data) if text.size else None
    _lib.check(L.dnatok_host_fasta_scan(ptr, text.size, int(upper_case), None, 0, None, None, 0,
                                        ctypes.byref(n_rec), ctypes.byref(n_bases)), "dnatok_host_fasta_scan")
    n, total = int(n_rec.value), int(n_bases.value)
    room = torch.empty(max(total, 1), dtype=torch.uint8, pin_memory=torch.cuda.is_available())
    offsets = np.zeros(n + 1, dtype=np.int64)
    spans = np.zeros((max(n, 1), 2), dtype=np.int64)
    _lib.check(L.dnatok_host_fasta_scan(ptr, text.size, int(upper_case), ctypes.c_void_p(room.data_ptr()), total,
                                        ctypes.c_void_p(offsets.ctypes.data), ctypes.c_void_p(spans.ctypes.data), n,
                                        ctypes.byref(n_rec), ctypes.byref(n_bases)), "dnatok_host_fasta_scan")
    host = room[:total]
    names = [bytes(text[lo:hi]).decode("utf-8", errors="replace") for lo, hi in spans[:n]]
    off_t = torch.from_numpy(offsets)
    if device is not None:
        host, off_t = host.to(device, non_blocking=True), off_t.to(device)
    return host, off_t, names


class RowNormalizer:
    """A tokenizer normalizer as a device program over ragged rows of bytes
    (C ABI: dnatok_normalize_rows).  ``steps`` are ``_lib.NormStep`` records."""

    def __init__(self, steps):
        self.steps = list(steps)
        self._arr = (_lib.NormStep * max(len(self.steps), 1))(*self.steps)
        self._scratch: Optional[torch.Tensor] = None
        rc = _lib.lib().dnatok_normalize_bounds(self._arr, len(self.steps), 0, 0, 0, None, None, None)
        _lib.check(rc, "dnatok_normalize_bounds")

    def bounds(self, n_rows: int, total: int, max_len: int) -> Tuple[int, int, int]:
        """(total bytes, longest row, scratch bytes): upper bounds after the steps."""
        t, m, sc = ctypes.c_int64(0), ctypes.c_int64(0), ctypes.c_size_t(0)
        _lib.check(_lib.lib().dnatok_normalize_bounds(self._arr, len(self.steps), int(n_rows), int(total),
                                                      int(max_len), ctypes.byref(t), ctypes.byref(m),
                                                      ctypes.byref(sc)), "dnatok_normalize_bounds")
        return int(t.value), int(m.value), int(sc.value)

    def apply(self, data: torch.Tensor, offsets: torch.Tensor, total: int, max_len: int
              ) -> Tuple[torch.Tensor, torch.Tensor, int, int]:
        """(bytes, offsets, total bound, longest-row bound) of the normalized rows; the real
        sizes stay on the device (``offsets[-1]``)."""
        _require_cuda(data, torch.uint8, "data")
        _require_cuda(offsets, torch.int64, "offsets")
        n_rows = offsets.numel() - 1
        out_total, out_max, need = self.bounds(n_rows, total, max_len)
        if self._scratch is None or self._scratch.numel() < need or self._scratch.device != data.device:
            self._scratch = torch.empty(max(need, 1), dtype=torch.uint8, device=data.device)   # grow-only
        out = torch.empty(max(out_total, 1), dtype=torch.uint8, device=data.device)
        out_offsets = torch.empty(n_rows + 1, dtype=torch.int64, device=data.device)
        _lib.check(_lib.lib().dnatok_normalize_rows(self._arr, len(self.steps), _ptr(data), _ptr(offsets), n_rows,
                                                    int(total), int(max_len), _ptr(out), out.numel(),
                                                    _ptr(out_offsets), _ptr(self._scratch),
                                                    self._scratch.numel(), _stream()),
                   "dnatok_normalize_rows")
        return out, out_offsets, out_total, out_max


class CharEncoder:
    """ids = table[byte] with padding and mask (C ABI: dnatok_char_*)."""

    def __init__(self, lut, pad_id: int, start_lut=None):
        self.lut = np.ascontiguousarray(lut, dtype=np.int32)
        if self.lut.shape != (256,):
            raise ValueError("lut must have 256 entries")
        self.start_lut = None if start_lut is None else np.ascontiguousarray(start_lut, dtype=np.int32)
        self.pad_id = int(pad_id)
        h = ctypes.c_void_p()
        _lib.check(_lib.lib().dnatok_char_table_create(_np_ptr(self.lut), _np_ptr(self.start_lut),
                                                       self.pad_id, ctypes.byref(h)),
                   "dnatok_char_table_create")
        self._h = h

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            try:
                _lib.lib().dnatok_char_table_destroy(h)
            except Exception:
                pass

    def encode_padded(self, data: torch.Tensor, offsets: torch.Tensor, t_out: int, *,
                      pad_left: bool = False, want_mask: bool = True, dtype: torch.dtype = torch.int32,
                      ids: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None):
        """Ragged rows -> ids [B, t_out] of ``dtype`` (uint8, int16, int32 or int64) and mask
        uint8 [B, t_out], padded with the pad id on the right, or on the left with ``pad_left``."""
        _require_cuda(data, torch.uint8, "data")
        _require_cuda(offsets, torch.int64, "offsets")
        if dtype not in (torch.uint8, torch.int16, torch.int32, torch.int64):
            raise ValueError("dtype must be uint8, int16, int32 or int64")
        n_rows = offsets.numel() - 1
        if ids is None:
            ids = torch.empty((n_rows, t_out), dtype=dtype, device=data.device)
        else:
            _require_cuda(ids, dtype, "ids")
        if want_mask and mask is None:
            mask = torch.empty((n_rows, t_out), dtype=torch.uint8, device=data.device)
        _lib.check(_lib.lib().dnatok_char_encode_padded_as(self._h, _ptr(data), _ptr(offsets), n_rows,
                                                           int(t_out), int(pad_left), _ptr(ids),
                                                           ids.element_size(),
                                                           _ptr(mask if want_mask else None), _stream()),
                   "dnatok_char_encode_padded")
        return ids, (mask if want_mask else None)

    def encode_packed(self, data: torch.Tensor, *, row_len: int = 0, want_mask: bool = False,
                      ids: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None):
        _require_cuda(data, torch.uint8, "data")
        total = data.numel()
        if ids is None:
            ids = torch.empty(total, dtype=torch.int32, device=data.device)
        if want_mask and mask is None:
            mask = torch.empty(total, dtype=torch.uint8, device=data.device)
        _lib.check(_lib.lib().dnatok_char_encode_packed(self._h, _ptr(data), total, int(row_len),
                                                        _ptr(ids), _ptr(mask if want_mask else None),
                                                        _stream()),
                   "dnatok_char_encode_packed")
        return ids, (mask if want_mask else None)


    def embed_packed(self, data: torch.Tensor, weight: torch.Tensor, *, row_len: int = 0,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """out[i, :] = weight[lut[data[i]], :] in one kernel (no id tensor).  ``weight`` is a
        contiguous [V, D] device tensor of any dtype whose rows are a multiple of 16 bytes."""
        _require_cuda(data, torch.uint8, "data")
        if not (weight.is_cuda and weight.dim() == 2 and weight.is_contiguous()):
            raise ValueError("weight must be a contiguous [V, D] device tensor")
        total = data.numel()
        row_bytes = weight.shape[1] * weight.element_size()
        if out is None:
            out = torch.empty((total, weight.shape[1]), dtype=weight.dtype, device=data.device)
        _lib.check(_lib.lib().dnatok_char_embed_packed(self._h, _ptr(data), total, int(row_len), _ptr(weight),
                                                       int(weight.shape[0]), int(row_bytes), _ptr(out),
                                                       _stream()),
                   "dnatok_char_embed_packed")
        return out


    def unpack_2bit(self, packed: torch.Tensor, row_len: int, *, dtype: torch.dtype = torch.int32,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Device uint8 [B, ceil(row_len/4)] of 2-bit codes -> ids [B, row_len] of ``dtype``
        (uint8, int32 or int64): ids = lut["ACGT"[code]], column 0 from the start table."""
        _require_cuda(packed, torch.uint8, "packed")
        if packed.dim() != 2 or packed.shape[1] != (int(row_len) + 3) // 4:
            raise ValueError("packed must be [B, ceil(row_len / 4)]")
        if dtype not in (torch.uint8, torch.int32, torch.int64):
            raise ValueError("dtype must be uint8, int32 or int64")
        b = packed.shape[0]
        if out is None:
            out = torch.empty((b, int(row_len)), dtype=dtype, device=packed.device)
        elif tuple(out.shape) != (b, int(row_len)):
            raise ValueError("out must be [B, row_len]")
        else:
            _require_cuda(out, dtype, "out")
        _lib.check(_lib.lib().dnatok_char_unpack_2bit(self._h, _ptr(packed), b, int(row_len), _ptr(out),
                                                      out.element_size(), _stream()),
                   "dnatok_char_unpack_2bit")
        return out


def width_guess_after(previous_width: int) -> int:
    """The ``width_guess`` to pass for the next batch of a stream whose last batch came out
    ``previous_width`` tokens wide.  A guess above the true width costs the few extra pad cells
    (written next to the row's own cells); a guess below it costs a second visit to every row, so
    the guess carries a margin: 1/64 of the width, at least 8 tokens, up to a whole 128-byte line of
    ids."""
    w = int(previous_width)
    if w <= 0:
        return 0
    w += max(8, w >> 6)
    return w + (-w) % 32


class WidthGuess:
    """The width guess of a stream of batches.  The widest row of a batch of a few hundred
    sequences moves by a tenth from one batch to the next (6-mers of 256 x 6000 bp with runs of N:
    1100 .. 1265 tokens), so the guess is not taken from the previous batch alone but from the
    largest of the recent widths, which fades by 1/256 per batch: on that stream (1023 batches)
    the stride derived from the previous width plus the margin was too small for one batch in seven
    (a second encode with the worst-case stride each time), the one from the fading peak for two
    batches in a thousand, with rows 130 instead of 105 cells further apart than they had to be."""

    def __init__(self):
        self.peak = 0

    def __bool__(self) -> bool:
        return self.peak > 0

    def update(self, width: int) -> None:
        """A batch came out ``width`` tokens wide."""
        self.peak = max(int(width), self.peak - max(1, self.peak >> 8))

    def next(self) -> int:
        """The ``width_guess`` for the next batch (0: none yet)."""
        return width_guess_after(self.peak)


class KmerEncoder:
    """Grid-aligned k-mer windows with per-window fallback (C ABI: dnatok_kmer_*)."""

    def __init__(self, k: int, digit, kmer_lut, single, pad_id: int, missing_id: int,
                 exp_off=None, exp_len=None, exp_flat=None):
        self.k = int(k)
        self.digit = np.ascontiguousarray(digit, dtype=np.int8)
        self.kmer_lut = np.ascontiguousarray(kmer_lut, dtype=np.int32)
        self.single = np.ascontiguousarray(single, dtype=np.int32)
        if self.kmer_lut.size != 5 ** self.k:
            raise ValueError("kmer_lut must have 5**k entries")
        self.pad_id = int(pad_id)
        self.exp_off = None if exp_off is None else np.ascontiguousarray(exp_off, dtype=np.int32)
        self.exp_len = None if exp_len is None else np.ascontiguousarray(exp_len, dtype=np.int32)
        self.exp_flat = None if exp_flat is None else np.ascontiguousarray(exp_flat, dtype=np.int32)
        n_flat = 0 if self.exp_flat is None else int(self.exp_flat.size)
        h = ctypes.c_void_p()
        _lib.check(_lib.lib().dnatok_kmer_table_create(
            self.k, _np_ptr(self.digit), _np_ptr(self.kmer_lut), _np_ptr(self.exp_off),
            _np_ptr(self.exp_len), _np_ptr(self.exp_flat), n_flat, _np_ptr(self.single),
            self.pad_id, int(missing_id), ctypes.byref(h)), "dnatok_kmer_table_create")
        self._h = h

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            try:
                _lib.lib().dnatok_kmer_table_destroy(h)
            except Exception:
                pass

    def set_team_rows(self, max_rows: int) -> None:
        """Test and measurement hook (``dnatok_kmer_table_set_team_rows``): batches of up to
        ``max_rows`` rows get a workgroup per row, larger ones a wave per row; -1 = automatic."""
        _lib.check(_lib.lib().dnatok_kmer_table_set_team_rows(self._h, int(max_rows)), "dnatok_kmer_table_set_team_rows")

    def encode_padded(self, data: torch.Tensor, offsets: torch.Tensor, t_cap: int, *,
                      fill_to: int = 0, width_guess: int = 0, want_mask: bool = True, out=None):
        """Returns (ids[B, t_cap], mask, lengths[B], status[B], max_len[1]); with fill_to = 0 the
        rows are padded to the device-side maximum, view ``ids[:, :max_len]``.  ``width_guess``
        (only with fill_to = 0) is the caller's guess of that maximum, e.g. the width of the
        previous batch of a stream: rows are padded that far while they are written."""
        _require_cuda(data, torch.uint8, "data")
        _require_cuda(offsets, torch.int64, "offsets")
        n_rows = offsets.numel() - 1
        dev = data.device
        if out is None:
            ids = torch.empty((n_rows, t_cap), dtype=torch.int32, device=dev)
            mask = torch.empty((n_rows, t_cap), dtype=torch.uint8, device=dev) if want_mask else None
            lengths = torch.empty(n_rows, dtype=torch.int32, device=dev)
            status = torch.empty(n_rows, dtype=torch.int32, device=dev)
            max_len = torch.empty(1, dtype=torch.int32, device=dev)
        else:
            ids, mask, lengths, status, max_len = out
        # (the batch's size tells the call how long its rows are on average: a batch of mostly short
        # rows with some long ones is split between two kernels, row by row on the device)
        _lib.check(_lib.lib().dnatok_kmer_encode_padded_sized(
            self._h, _ptr(data), _ptr(offsets), n_rows, int(data.numel()), int(t_cap),
            int(fill_to) if fill_to > 0 else -min(int(width_guess), int(t_cap)), _ptr(ids),
            _ptr(mask), _ptr(lengths), _ptr(status), _ptr(max_len), _stream()),
            "dnatok_kmer_encode_padded_sized")
        return ids, mask, lengths, status, max_len

    def encode_packed(self, data: torch.Tensor, offsets: torch.Tensor, *, want_mask: bool = False, out=None):
        """Packed layout: ``(ids int32 [total], out_offsets int64 [B + 1], mask uint8 [total] or None,
        lengths int32 [B], status int32 [B])``; row b's tokens are ``ids[out_offsets[b] :
        out_offsets[b + 1]]``, nothing is padded.  ``ids`` and ``mask`` have room for one cell per
        input byte; ``out`` = (ids, out_offsets, mask, lengths, status) reuses caller buffers."""
        _require_cuda(data, torch.uint8, "data")
        _require_cuda(offsets, torch.int64, "offsets")
        n_rows = offsets.numel() - 1
        total = int(data.numel())
        dev = data.device
        if out is None:
            ids = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
            out_offsets = torch.empty(n_rows + 1, dtype=torch.int64, device=dev)
            mask = torch.empty(max(total, 1), dtype=torch.uint8, device=dev) if want_mask else None
            lengths = torch.empty(n_rows, dtype=torch.int32, device=dev)
            status = torch.empty(n_rows, dtype=torch.int32, device=dev)
        else:
            ids, out_offsets, mask, lengths, status = out
        _lib.check(_lib.lib().dnatok_kmer_encode_packed(
            self._h, _ptr(data), _ptr(offsets), n_rows, total, _ptr(ids), _ptr(out_offsets),
            _ptr(mask) if mask is not None else None, _ptr(lengths), _ptr(status), _stream()),
            "dnatok_kmer_encode_packed")
        return ids, out_offsets, mask, lengths, status


class BpeEncoder:
    """BPE merge engine + packer (C ABI: dnatok_bpe_*, dnatok_pack_ragged, dnatok_pad_rows)."""

    def __init__(self, pair_a, pair_b, new_id, n_symbols: int, byte_to_id=None, out_remap=None):
        self.pair_a = np.ascontiguousarray(pair_a, dtype=np.int32)
        self.pair_b = np.ascontiguousarray(pair_b, dtype=np.int32)
        self.new_id = np.ascontiguousarray(new_id, dtype=np.int32)
        self.n_symbols = int(n_symbols)
        self.byte_to_id = (np.arange(256, dtype=np.int32) if byte_to_id is None
                           else np.ascontiguousarray(byte_to_id, dtype=np.int32))
        self.out_remap = None if out_remap is None else np.ascontiguousarray(out_remap, dtype=np.int32)
        h = ctypes.c_void_p()
        _lib.check(_lib.lib().dnatok_bpe_table_create(
            _np_ptr(self.byte_to_id), _np_ptr(self.pair_a), _np_ptr(self.pair_b),
            _np_ptr(self.new_id), int(self.pair_a.size), self.n_symbols, _np_ptr(self.out_remap),
            ctypes.byref(h)), "dnatok_bpe_table_create")
        self._h = h
        self._scratch: Optional[torch.Tensor] = None

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            try:
                _lib.lib().dnatok_bpe_table_destroy(h)
            except Exception:
                pass

    def _get_scratch(self, n_rows: int, max_len: int, total: int, device) -> torch.Tensor:
        need = int(_lib.lib().dnatok_bpe_scratch_bytes(self._h, n_rows, max_len, total))
        if self._scratch is None or self._scratch.numel() < need or self._scratch.device != device:
            self._scratch = torch.empty(need, dtype=torch.uint8, device=device)   # grow-only
        return self._scratch

    def encode(self, data: torch.Tensor, offsets: torch.Tensor, max_len: int, *,
               tok_tmp: Optional[torch.Tensor] = None, lengths: Optional[torch.Tensor] = None):
        """Row b's tokens land in tok_tmp[offsets[b] : offsets[b] + lengths[b]]."""
        _require_cuda(data, torch.uint8, "data")
        _require_cuda(offsets, torch.int64, "offsets")
        n_rows = offsets.numel() - 1
        total = data.numel()
        if tok_tmp is None:
            tok_tmp = torch.empty(max(total, 1), dtype=torch.int32, device=data.device)
        if lengths is None:
            lengths = torch.empty(n_rows, dtype=torch.int32, device=data.device)
        scratch = self._get_scratch(n_rows, int(max_len), total, data.device)
        _lib.check(_lib.lib().dnatok_bpe_encode(self._h, _ptr(data), _ptr(offsets), n_rows,
                                                int(max_len), total, _ptr(scratch), scratch.numel(),
                                                _ptr(tok_tmp), _ptr(lengths), _stream()),
                   "dnatok_bpe_encode")
        return tok_tmp, lengths

    def encode_padded(self, data: torch.Tensor, offsets: torch.Tensor, max_len: int, stride: int, pad_id: int, *,
                      remap: Optional[torch.Tensor] = None, want_mask: bool = True, want_longest: bool = True,
                      out=None, tok_tmp: Optional[torch.Tensor] = None, pad_left: bool = False,
                      dtype: torch.dtype = torch.int32):
        """Engine and padding in one pass: ``ids[B, stride]`` of ``dtype`` (uint8, int16, int32 or
        int64; through ``remap``, ``pad_id`` behind a row's tokens -- with ``pad_left`` before them,
        the tokens ending at the row's last cell), ``mask[B, stride]`` uint8, ``lengths[B]`` (full token counts) and
        ``longest[1]`` (their maximum; None with ``want_longest=False`` or in ``out``: the caller takes it
        from the lengths), all on the device.  A row with more tokens than ``stride``
        keeps its first ``stride``: compare ``longest`` with it.  ``out`` = (ids, mask, lengths,
        longest) reuses caller buffers.  Rows above ``padded_direct_max()`` bytes go through a token
        buffer (``tok_tmp``, allocated here when not given)."""
        _require_cuda(data, torch.uint8, "data")
        _require_cuda(offsets, torch.int64, "offsets")
        n_rows = offsets.numel() - 1
        total = data.numel()
        dev = data.device
        stride = int(stride)
        if out is None:
            ids = torch.empty((n_rows, stride), dtype=dtype, device=dev)
            mask = torch.empty((n_rows, stride), dtype=torch.uint8, device=dev) if want_mask else None
            lengths = torch.empty(n_rows, dtype=torch.int32, device=dev)
            longest = torch.empty(1, dtype=torch.int32, device=dev) if want_longest else None
        else:
            ids, mask, lengths, longest = out
            if ids.shape != (n_rows, stride) or not ids.is_contiguous():
                raise ValueError("ids must be a contiguous [n_rows, stride] tensor")
        if ids.dtype not in (torch.uint8, torch.int16, torch.int32, torch.int64):
            raise ValueError("ids must be uint8, int16, int32 or int64")
        if int(max_len) > self.padded_direct_max() and tok_tmp is None:
            tok_tmp = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
        scratch = self._get_scratch(n_rows, int(max_len), total, dev)
        _lib.check(_lib.lib().dnatok_bpe_encode_padded_as(
            self._h, _ptr(data), _ptr(offsets), n_rows, int(max_len), total, _ptr(scratch), scratch.numel(),
            _ptr(tok_tmp) if tok_tmp is not None else None, _ptr(remap) if remap is not None else None,
            int(pad_id), stride, 1 if pad_left else 0, _ptr(ids), ids.element_size(),
            _ptr(mask) if mask is not None else None, _ptr(lengths), _ptr(longest),
            _stream()), "dnatok_bpe_encode_padded_as")
        return ids, mask, lengths, longest

    def padded_direct_max(self) -> int:
        """Longest row (bytes) that ``encode_padded`` writes without a token buffer."""
        return int(_lib.lib().dnatok_bpe_padded_direct_max(self._h))

    def set_chunk_geometry(self, core: int, overlap: int) -> None:
        """Test hook (``dnatok_bpe_table_set_chunk_geometry``): this encoder's calls cut long rows
        into chunks of ``core`` bytes extended by ``overlap`` on both sides; (0, 0) = shipped."""
        _lib.check(_lib.lib().dnatok_bpe_table_set_chunk_geometry(self._h, int(core), int(overlap)),
                   "dnatok_bpe_table_set_chunk_geometry")

    def set_table_placement(self, mode: int) -> None:
        """Measurement hook (``dnatok_bpe_table_set_placement``): 0 = merge table in global memory
        (default), 1 / 2 = its compact form in LDS where the batch allows."""
        _lib.check(_lib.lib().dnatok_bpe_table_set_placement(self._h, int(mode)), "dnatok_bpe_table_set_placement")

    def encode_with_chars(self, data: torch.Tensor, offsets: torch.Tensor, max_len: int, char_lut: torch.Tensor, *,
                          tok_tmp: Optional[torch.Tensor] = None, lengths: Optional[torch.Tensor] = None,
                          char_ids: Optional[torch.Tensor] = None, char_mask: Optional[torch.Tensor] = None,
                          want_char_mask: bool = True):
        """``encode`` plus the single-character ids of the same bytes from the same pass over them:
        ``char_ids[i] = char_lut[data[i]]`` (``char_lut``: device int32[256], e.g.
        ``CharEncoder.lut_device``), ``char_mask[i] = 1``.  Returns (tok_tmp, lengths, char_ids, char_mask)."""
        _require_cuda(data, torch.uint8, "data")
        _require_cuda(offsets, torch.int64, "offsets")
        _require_cuda(char_lut, torch.int32, "char_lut")
        if char_lut.numel() != 256:
            raise ValueError("char_lut must hold 256 ids")
        n_rows = offsets.numel() - 1
        total = data.numel()
        if tok_tmp is None:
            tok_tmp = torch.empty(max(total, 1), dtype=torch.int32, device=data.device)
        if lengths is None:
            lengths = torch.empty(n_rows, dtype=torch.int32, device=data.device)
        if char_ids is None:
            char_ids = torch.empty(max(total, 1), dtype=torch.int32, device=data.device)
        if char_mask is None and want_char_mask:
            char_mask = torch.empty(max(total, 1), dtype=torch.uint8, device=data.device)
        scratch = self._get_scratch(n_rows, int(max_len), total, data.device)
        _lib.check(_lib.lib().dnatok_bpe_encode_with_chars(
            self._h, _ptr(data), _ptr(offsets), n_rows, int(max_len), total, _ptr(scratch), scratch.numel(),
            _ptr(tok_tmp), _ptr(lengths), _ptr(char_lut), _ptr(char_ids),
            _ptr(char_mask) if char_mask is not None else None, _stream()), "dnatok_bpe_encode_with_chars")
        return tok_tmp, lengths, char_ids, char_mask


def pack_ragged(tok_tmp: torch.Tensor, in_offsets: torch.Tensor, lengths: torch.Tensor, *,
                remap: Optional[torch.Tensor] = None, want_mask: bool = True, out=None):
    """Packed ids (capacity = tok_tmp.numel()), int64 offsets[B+1], mask; all on the device.
    ``out`` = (ids_out, out_offsets, mask) reuses caller buffers."""
    n_rows = lengths.numel()
    dev = tok_tmp.device
    if out is not None:
        ids_out, out_offsets, mask = out
    else:
        ids_out = torch.empty(tok_tmp.numel(), dtype=torch.int32, device=dev)
        out_offsets = torch.empty(n_rows + 1, dtype=torch.int64, device=dev)
        mask = torch.empty(tok_tmp.numel(), dtype=torch.uint8, device=dev) if want_mask else None
    _lib.check(_lib.lib().dnatok_pack_ragged(_ptr(tok_tmp), _ptr(in_offsets), _ptr(lengths), n_rows,
                                             _ptr(remap), _ptr(ids_out), _ptr(out_offsets),
                                             _ptr(mask), _stream()), "dnatok_pack_ragged")
    return ids_out, out_offsets, mask


def pad_rows(tok_tmp: torch.Tensor, in_offsets: torch.Tensor, lengths: torch.Tensor, pad_id: int,
             t_cap: int, *, fill_to: int = 0, remap: Optional[torch.Tensor] = None,
             want_mask: bool = True, out=None):
    """Padded ids[B, t_cap] + mask + max_len[1]; with fill_to = 0 view ``ids[:, :max_len]``.
    ``out`` = (ids, mask, max_len) reuses caller buffers."""
    n_rows = lengths.numel()
    dev = tok_tmp.device
    if out is not None:
        ids, mask, max_len = out
    else:
        ids = torch.empty((n_rows, t_cap), dtype=torch.int32, device=dev)
        mask = torch.empty((n_rows, t_cap), dtype=torch.uint8, device=dev) if want_mask else None
        max_len = torch.empty(1, dtype=torch.int32, device=dev)
    _lib.check(_lib.lib().dnatok_pad_rows(_ptr(tok_tmp), _ptr(in_offsets), _ptr(lengths), n_rows,
                                          _ptr(remap), int(pad_id), int(t_cap), int(fill_to),
                                          _ptr(ids), _ptr(mask), _ptr(max_len), _stream()),
               "dnatok_pad_rows")
    return ids, mask, max_len


def pad_rows_as(tok_tmp: torch.Tensor, in_offsets: torch.Tensor, lengths: torch.Tensor, pad_id: int,
                t_cap: int, *, fill_to: int = 0, min_width: int = 0, pad_multiple: int = 1,
                pad_left: bool = False, dtype: torch.dtype = torch.int32,
                remap: Optional[torch.Tensor] = None, want_mask: bool = True,
                stats: Optional[torch.Tensor] = None):
    """The padded layout with the choices of DNATok's padding: side, a least width (``token_len``),
    a multiple, the id type.  Returns (ids[B, t_cap] of ``dtype``, mask, stats int32[2] =
    {longest row, width}); view ``ids[:, :width]`` (C ABI: dnatok_pad_rows_as).  ``stats`` may be
    given (two int32 on the device, e.g. next to the lengths, so that one copy brings both down)."""
    if dtype not in (torch.uint8, torch.int16, torch.int32, torch.int64):
        raise ValueError("dtype must be uint8, int16, int32 or int64")
    n_rows = lengths.numel()
    dev = tok_tmp.device
    ids = torch.empty((n_rows, t_cap), dtype=dtype, device=dev)
    mask = torch.empty((n_rows, t_cap), dtype=torch.uint8, device=dev) if want_mask else None
    if stats is None:
        stats = torch.empty(2, dtype=torch.int32, device=dev)
    _lib.check(_lib.lib().dnatok_pad_rows_as(
        _ptr(tok_tmp), _ptr(in_offsets), _ptr(lengths), n_rows, _ptr(remap), int(pad_id), int(t_cap),
        int(fill_to), min(int(min_width), int(t_cap)), int(pad_multiple), int(bool(pad_left)), _ptr(ids),
        ids.element_size(), _ptr(mask), ctypes.c_void_p(stats.data_ptr()),
        ctypes.c_void_p(stats.data_ptr() + 4), _stream()), "dnatok_pad_rows_as")
    return ids, mask, stats
