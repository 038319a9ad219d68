#!/usr/bin/env python3
"""Encode-throughput benchmark of the MI355X DNA tokenization backend.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2] [--no-extras] [--no-cpu]

A step is one pass of the encode path over one batch of seeded synthetic input that is
already resident in HBM.  The headline workload (default C2, the non-overlapping 6-mer
tokenizer) is timed in its sustained form: many distinct 256 x 6000 bp batches laid out
back to back and encoded by one call, because a single 1.5 Mbp batch (2.8 MB of traffic)
is launch-bound and says nothing about the HBM roofline; the per-call latency of the
exact configurations is reported under "per_call".  One JSON line is printed.
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

BPE_BOUND_NOTE = ("BPE merges are a chain of dependent rounds, not a stream: the HBM fraction is reported because the "
                  "metric asks for it, but the bound of a row is rounds x dependent reads per round x read latency, "
                  "spread over the teams that fit the chip at once")


# ------------------------------------------------------------------------------ inputs

def many_batches_uniform(n_rows: int, length: int, seed: int, n_rate: float = 0.0,
                         n_run_fraction: float = 0.0) -> np.ndarray:
    """Fast generator for the sustained runs: same distributions as workloads.config1_char /
    config2_kmer, vectorised for hundreds of Mbp."""
    rng = np.random.Generator(np.random.PCG64(seed))
    total = n_rows * length
    codes = rng.integers(0, 4, size=total, dtype=np.uint8)
    arr = np.frombuffer(b"ACGT", dtype=np.uint8)[codes]
    del codes
    if n_rate > 0:
        n = rng.binomial(total, n_rate)
        arr[rng.integers(0, total, size=n)] = ord("N")
    if n_run_fraction > 0:
        n = rng.binomial(total, n_run_fraction / 25.5)
        starts = rng.integers(0, total, size=n)
        runs = rng.integers(1, 51, size=n)
        for s, r in zip(starts.tolist(), runs.tolist()):
            e = min(s + r, (s // length + 1) * length)       # runs do not cross rows
            arr[s:e] = ord("N")
    return arr


class Workload:
    name = ""
    dtype = "u8"

    def step(self):
        raise NotImplementedError


def host_threads() -> int:
    """Threads for the CPU legs: the share of the host this job owns, not the machine's core count."""
    n = os.cpu_count() or 1
    for var in ("OMP_NUM_THREADS", "MAX_JOBS"):
        v = os.environ.get(var, "")
        if v.isdigit() and int(v) > 0:
            return min(n, int(v))
    return n


def hf_live_rows(tokenizer, host: np.ndarray, offsets) -> list:
    """Token ids of the rows host[offsets[i]:offsets[i+1]] from the Hugging Face tokenizer itself,
    in this process: the checker for rows that have no committed golden vector."""
    raw = host.tobytes()
    strings = [raw[int(offsets[i]):int(offsets[i + 1])].decode("ascii") for i in range(len(offsets) - 1)]
    return [np.asarray(e.ids, dtype=np.int32) for e in tokenizer.encode_batch(strings, add_special_tokens=False)]


def same_rows(got: list, want: list, what: str) -> None:
    assert len(got) == len(want), what
    for i, (g, w) in enumerate(zip(got, want)):
        assert g.shape == w.shape and np.array_equal(g, w), f"{what}: row {i} differs from Hugging Face tokenizers"


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda")


class CharDense(Workload):
    """C1: 64 x 8192 bp char tokenizer; ids int32 + mask uint8, dense [B, T]."""

    def __init__(self, n_batches: int):
        from dnatok_amd import encoders
        from tests.support import hf_tokenizers as hf, workloads as wl
        vocab = hf.char_vocab()
        lut = np.zeros(256, dtype=np.int32)
        for ch in "ACGTN":
            lut[ord(ch)] = vocab[ch]
        self.lut = lut
        self.enc = encoders.CharEncoder(lut, pad_id=vocab["<pad>"])
        first = wl.config1_char()
        parts = [first.data]
        if n_batches > 1:
            parts.append(many_batches_uniform(64 * (n_batches - 1), 8192, 7001, n_rate=0.001))
        host = np.concatenate(parts)
        self.host = host
        self.data = _dev(host)
        import torch
        self.ids = torch.empty(host.size, dtype=torch.int32, device="cuda")
        self.mask = torch.empty(host.size, dtype=torch.uint8, device="cuda")
        self.bases = host.size
        self.algorithmic_bytes = 6 * host.size
        self.kernel = "char_packed_kernel"
        self.name = f"C1 char vocab-11, 64x8192 bp batches, {n_batches} distinct batch(es) per call"

    def step(self):
        self.enc.encode_packed(self.data, row_len=8192, want_mask=True, ids=self.ids, mask=self.mask)

    def check(self):
        import torch
        from tests.golden import check as util
        self.step()
        torch.cuda.synchronize()
        ids = self.ids[:64 * 8192].cpu().numpy().reshape(64, 8192)
        util.check_against_golden("C1_char", list(ids))
        # every id of every batch: the table lookup, done by torch
        lut = torch.from_numpy(self.lut).to("cuda")
        step = 1 << 26
        for lo in range(0, self.data.numel(), step):
            assert torch.equal(self.ids[lo:lo + step], lut[self.data[lo:lo + step].long()])
        assert bool((self.mask == 1).all())

    def oracle_port(self, budget_s: float):
        from oracle import oracle as O
        n = min(self.host.size, 64 * 8192 * 64)
        sample = self.host[:n]
        off = np.arange(n // 8192 + 1, dtype=np.int64) * 8192
        reps, t0 = 0, time.perf_counter()
        while True:
            O.char_encode_padded(self.lut, sample, off, 8192, 1)
            reps += 1
            if time.perf_counter() - t0 > budget_s:
                break
        dt = time.perf_counter() - t0
        return n * reps / dt / 1e6, f"{n // (64 * 8192)} batches of 64x8192 bp, {reps} passes"


class KmerPadded(Workload):
    """C2: 256 x 6000 bp 6-mer tokenizer; padded int32 ids + uint8 mask + lengths.

    The output buffers hold 6016 cells per row: room for the worst case (every base of a
    6000 bp row spelled on its own), rounded up to whole 128-byte lines for ids and mask.

    A stream of batches: two different data sets take turns, and the width guess a call gets is
    derived from the width of the call before it, which ran on the other data set.  ``guess``
    selects the policy: "previous" (the library's: previous width plus a margin), "stale"
    (the previous width as it is, which is too small every other call) or "none"."""

    def __init__(self, n_batches: int, t_cap: int = 0, guess: str = "previous"):
        from dnatok_amd import encoders, kmer_tables
        from tests.support import hf_tokenizers as hf, workloads as wl
        import torch
        vocab = hf.kmer_vocab(6)
        self.vocab = vocab
        t = kmer_tables.tables_from_vocab(vocab, 6, vocab["<unk>"])
        self.enc = encoders.KmerEncoder(6, t.digit, t.kmer_lut, t.single, vocab["<pad>"], vocab["<unk>"],
                                        t.exp_off, t.exp_len, t.exp_flat)
        self.n_rows = 256 * n_batches
        self.guess = guess
        self.off = _dev(np.arange(self.n_rows + 1, dtype=np.int64) * 6000)
        self.hosts, self.sets = [], []
        for which in (0, 1):
            parts = [wl.config2_kmer().data if which == 0 else wl.config2_kmer(seed=wl.SEEDS["C2"] + 500).data]
            if n_batches > 1:
                parts.append(many_batches_uniform(256 * (n_batches - 1), 6000, 7002 + 10 * which, n_run_fraction=0.005))
            host = np.concatenate(parts)
            self.hosts.append(host)
            self.sets.append(_dev(host))
        dev = "cuda"
        # the widths of the two data sets, from a first pass with room for the worst case
        self.t_cap = 6016
        scratch = tuple(torch.empty(shape, dtype=dt, device=dev) for shape, dt in (
            ((self.n_rows, 6016), torch.int32), ((self.n_rows, 6016), torch.uint8), ((self.n_rows,), torch.int32),
            ((self.n_rows,), torch.int32), ((1,), torch.int32)))
        self.widths = []
        for which in (0, 1):
            self.out = scratch
            self.run(which, 0)
            torch.cuda.synchronize()
            t_max = int(scratch[4].item())
            assert t_max == int(scratch[2].max().item())
            self.widths.append(t_max)
        del scratch
        self.out = None
        torch.cuda.empty_cache()
        # The stride of the rows: as the library does it in a stream of batches, the guess of the
        # width rounded up to whole 128-byte lines (a batch wider than that would come out cut
        # and be encoded again with the worst-case stride; check() sees that none is).  Without
        # a usable guess the rows lie the worst case apart.
        if not t_cap:
            t_cap = 6016
            if guess in ("previous", "fixed"):
                g = max(encoders.width_guess_after(wd) for wd in self.widths)
                t_cap = g + (-g) % 128
        self.t_cap = t_cap
        self.out = (torch.empty((self.n_rows, t_cap), dtype=torch.int32, device=dev),
                    torch.empty((self.n_rows, t_cap), dtype=torch.uint8, device=dev),
                    torch.empty(self.n_rows, dtype=torch.int32, device=dev),
                    torch.empty(self.n_rows, dtype=torch.int32, device=dev),
                    torch.empty(1, dtype=torch.int32, device=dev) if guess != "fixed" else None)
        self.bases = self.hosts[0].size
        self.kernel = "kmer_rows_kernel"
        how = {"previous": "width of the previous call, which ran on different data, plus the library's margin, passed as the guess",
               "stale": "width of the previous call, which ran on different data, passed as the guess as it is",
               "none": "no width guess", "fixed": ""}[guess]
        self.name = (f"C2 non-overlapping 6-mer vocab-4106, 256x6000 bp batches, {n_batches} distinct batch(es) "
                     f"per call, two data sets taking turns, " +
                     (f"pad to longest row ({how})" if guess != "fixed" else
                      f"padded to a fixed width of {t_cap} cells (the reference's token_len; no longest row to find)") +
                     f", rows {t_cap} cells apart" +
                     ("; the stride comes from an untimed set-up pass over both data sets, so no timed call outgrows it "
                      "(a stream whose widths drift re-encodes about 2 batches in 1000 with the worst-case stride: "
                      "encoders.WidthGuess)" if guess == "previous" and t_cap < 6016 else ""))
        # 1 B/base read; int32 id + uint8 mask for every cell of [rows, T_max] (the fixed width: of
        # [rows, t_cap]); int32 length per row; the mean over the two data sets, which take turns
        cells = self.n_rows * sum(self.widths) // 2 if guess != "fixed" else self.n_rows * t_cap
        self.algorithmic_bytes = self.bases + 5 * cells + 4 * self.n_rows
        self.turn = 0

    def run(self, which: int, width_guess: int):
        self.enc.encode_padded(self.sets[which], self.off, self.t_cap, fill_to=self.t_cap if self.guess == "fixed" else 0,
                               width_guess=width_guess, out=self.out)
        self.last = which

    def step(self):
        from dnatok_amd import encoders
        previous = self.widths[self.turn ^ 1]
        guess = {"previous": encoders.width_guess_after(previous), "stale": previous, "none": 0, "fixed": 0}[self.guess]
        self.run(self.turn, guess)
        self.turn ^= 1

    def check(self):
        """First batch of data set 0 against the committed golden vectors, last batch of data set 1
        against the Hugging Face tokenizer run here, and every row's padding and mask."""
        import torch
        from tests.golden import check as util
        from tests.support import hf_tokenizers as hf
        ids, mask, lengths, status, max_len = self.out
        pad = self.vocab["<pad>"]
        for which in (0, 1):
            self.turn = which
            self.step()
            torch.cuda.synchronize()
            ln = lengths.cpu().numpy()
            m = int(max_len.item()) if max_len is not None else self.t_cap
            assert self.widths[which] == int(ln.max()) and (max_len is None or m == self.widths[which])
            assert int(status.abs().sum().item()) == 0
            if which == 0:
                util.check_against_golden("C2_kmer", [ids[r, :ln[r]].cpu().numpy() for r in range(256)])
            else:
                first = self.n_rows - 256
                want = hf_live_rows(hf.build_kmer_tokenizer(6), self.hosts[1][first * 6000:],
                                    np.arange(257, dtype=np.int64) * 6000)
                same_rows([ids[first + r, :ln[first + r]].cpu().numpy() for r in range(256)], want, "C2 last batch")
            col = torch.arange(m, device="cuda")[None, :]
            inside = col < lengths[:, None]
            assert bool((mask[:, :m].bool() == inside).all())
            assert bool((ids[:, :m][~inside] == pad).all())
            # a window is one token, or six when it holds an N
            host = self.hosts[which].reshape(self.n_rows, 1000, 6)
            n_windows = (host == ord("N")).any(axis=2).sum(axis=1)
            assert np.array_equal(ln, 1000 + 5 * n_windows)
        self.turn = 0

    def oracle_port(self, budget_s: float):
        from oracle import oracle as O
        ot = O.kmer_tables_from_vocab(self.vocab, 6, self.vocab["<unk>"])
        rows = min(self.n_rows, 256 * 16)
        sample = self.hosts[0][:rows * 6000]
        off = np.arange(rows + 1, dtype=np.int64) * 6000
        reps, t0 = 0, time.perf_counter()
        while True:
            O.kmer_encode_batch(ot, sample, off, self.widths[0], self.vocab["<pad>"])
            reps += 1
            if time.perf_counter() - t0 > budget_s:
                break
        dt = time.perf_counter() - t0
        return rows * 6000 * reps / dt / 1e6, f"{rows // 256} batches of 256x6000 bp, {reps} passes"


class BpePadded(Workload):
    """C3 / C4: BPE encode, remap, pad to the longest row, mask.  Rows that the engine takes whole
    (C3) are padded by the engine itself while it writes them out (dnatok_bpe_encode_padded), the
    rows as far apart as the stream's width guess says (encoders.WidthGuess, fed by the set-up
    call); rows that are cut into chunks (C4) are assembled first and padded by a launch of its own."""

    def __init__(self, which: str, n_batches: int):
        from dnatok_amd import bpe_vocab, encoders
        from tests.support import hf_tokenizers as hf, workloads as wl
        import torch
        with open(hf.bpe_tokenizer_path(which)) as fh:
            cfg = json.load(fh)
        self.cfg = cfg
        self.which = which
        kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
        vocab = cfg["model"]["vocab"]
        self.pad_id = vocab["[PAD]"]
        self.enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv),
                                       out_remap=kv.remap_to(vocab, vocab["[UNK]"]))
        if which == "4096":
            rows, length, golden, seed0 = 1024, 1024, "C3_bpe4096", wl.SEEDS["C3"]
            mk = wl.config3_bpe4096
        else:
            rows, length, golden, seed0 = 32, 100_000, "C4_bpe32000", wl.SEEDS["C4"]
            mk = wl.config4_bpe32000
        self.golden = golden
        self.rows_per_batch, self.length = rows, length
        parts = [mk().data] + [mk(rows, length, seed=seed0 + 100 + i).data for i in range(n_batches - 1)]
        host = np.concatenate(parts)
        self.host = host
        self.n_rows = rows * n_batches
        self.data = _dev(host)
        self.off = _dev(np.arange(self.n_rows + 1, dtype=np.int64) * length)
        self.tok = torch.empty(host.size, dtype=torch.int32, device="cuda")
        self.lengths = torch.empty(self.n_rows, dtype=torch.int32, device="cuda")
        self.t_cap = length
        self.pad_out = (torch.empty((self.n_rows, length), dtype=torch.int32, device="cuda"),
                        torch.empty((self.n_rows, length), dtype=torch.uint8, device="cuda"),
                        torch.empty(1, dtype=torch.int32, device="cuda"))
        self.bases = host.size
        self.kernel = "bpe_lds_kernel" if length <= 4096 else "bpe_long_kernel"
        self.name = (f"{'C3' if which == '4096' else 'C4'} BPE vocab-{which}, {rows}x{length} bp batches, "
                     f"{n_batches} distinct batch(es) per call, pad to longest row")
        self.one_pass = False
        self.step()
        torch.cuda.synchronize()
        t_max = int(self.max_len.item())
        self.t_max = t_max
        if length <= self.enc.padded_direct_max():
            widths = encoders.WidthGuess()
            widths.update(t_max)
            self.stride = min(widths.next(), length)
            self.pad_out = (torch.empty((self.n_rows, self.stride), dtype=torch.int32, device="cuda"),
                            torch.empty((self.n_rows, self.stride), dtype=torch.uint8, device="cuda"),
                            self.lengths, torch.empty(1, dtype=torch.int32, device="cuda"))
            self.one_pass = True
            self.name += f" (one pass, rows {self.stride} cells apart)"
        self.algorithmic_bytes = host.size + 5 * self.n_rows * t_max + 4 * self.n_rows

    def step(self):
        from dnatok_amd import encoders
        if self.one_pass:
            self.ids, self.mask, _, self.max_len = self.enc.encode_padded(
                self.data, self.off, self.length, self.stride, self.pad_id, out=self.pad_out)
            return
        self.enc.encode(self.data, self.off, self.length, tok_tmp=self.tok, lengths=self.lengths)
        self.ids, self.mask, self.max_len = encoders.pad_rows(self.tok, self.off, self.lengths, self.pad_id,
                                                              self.t_cap, fill_to=0, out=self.pad_out)

    def check(self):
        """First batch against the committed golden vectors; with more than one batch per call, rows
        of the last batch against the Hugging Face tokenizer run here."""
        import torch
        from tests.golden import check as util
        from tests.support import hf_tokenizers as hf
        self.step()
        torch.cuda.synchronize()
        ln = self.lengths.cpu().numpy()
        rows = [self.ids[r, :ln[r]].cpu().numpy() for r in range(self.rows_per_batch)]
        util.check_against_golden(self.golden, rows)
        assert (ln > 0).all() and int(self.max_len.item()) == int(ln.max())
        assert not self.one_pass or int(ln.max()) <= self.stride, "a row was cut by the stride"
        if self.n_rows > self.rows_per_batch:
            n_live = min(self.rows_per_batch, 256)
            first = self.n_rows - n_live
            want = hf_live_rows(hf.load_bpe_tokenizer(self.which), self.host[first * self.length:],
                                np.arange(n_live + 1, dtype=np.int64) * self.length)
            same_rows([self.ids[first + r, :ln[first + r]].cpu().numpy() for r in range(n_live)], want,
                      f"BPE vocab-{self.which} last batch")
        m = int(ln.max())
        col = torch.arange(m, device="cuda")[None, :]
        inside = col < self.lengths[:, None]
        assert bool((self.mask[:, :m].bool() == inside).all())
        assert bool((self.ids[:, :m][~inside] == self.pad_id).all())

    def oracle_port(self, budget_s: float):
        from oracle import oracle as O
        bo = O.bpe_oracle_from_tokenizer_json(self.cfg)
        rows = min(self.n_rows, self.rows_per_batch)
        sample = self.host[:rows * self.length]
        off = np.arange(rows + 1, dtype=np.int64) * self.length
        reps, t0 = 0, time.perf_counter()
        while True:
            bo.encode_batch(sample, off)
            reps += 1
            if time.perf_counter() - t0 > budget_s:
                break
        dt = time.perf_counter() - t0
        return rows * self.length * reps / dt / 1e6, f"1 batch of {rows}x{self.length} bp, {reps} passes"


class RaggedBoth(Workload):
    """C5: 4096 ragged sequences through the vocab-4096 BPE and the char tokenizer in one
    pass over the same device buffer; packed ids + offsets + masks stay on the device."""

    def __init__(self, n_batches: int = 1):
        from dnatok_amd import bpe_vocab, encoders
        from tests.support import hf_tokenizers as hf, workloads as wl
        import torch
        with open(hf.bpe_tokenizer_path("4096")) as fh:
            cfg = json.load(fh)
        self.cfg = cfg
        kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
        vocab = cfg["model"]["vocab"]
        self.bpe = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv),
                                       out_remap=kv.remap_to(vocab, vocab["[UNK]"]))
        cv = hf.char_vocab()
        lut = np.zeros(256, dtype=np.int32)
        for ch in "ACGTN":
            lut[ord(ch)] = cv[ch]
        self.lut = lut
        self.char = encoders.CharEncoder(lut, pad_id=cv["<pad>"])
        self.lut_dev = _dev(lut)
        self.one_pass = True          # False: the char tokenizer as a launch of its own after the BPE engine
        first = wl.config5_ragged()
        self.first = first
        batches = [first] + [wl.config5_ragged(seed=wl.SEEDS["C5"] + 100 + i) for i in range(n_batches - 1)]
        self.host = np.concatenate([b.data for b in batches])
        lens = np.concatenate([b.lengths() for b in batches])
        self.offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        self.n_seqs = lens.size
        total = int(self.offsets[-1])
        self.data, self.off = _dev(self.host), _dev(self.offsets)
        self.max_len = int(lens.max())
        self.tok = torch.empty(total, dtype=torch.int32, device="cuda")
        self.lengths = torch.empty(self.n_seqs, dtype=torch.int32, device="cuda")
        self.pack_out = (torch.empty(total, dtype=torch.int32, device="cuda"),
                         torch.empty(self.n_seqs + 1, dtype=torch.int64, device="cuda"),
                         torch.empty(total, dtype=torch.uint8, device="cuda"))
        self.cids = torch.empty(total, dtype=torch.int32, device="cuda")
        self.cmask = torch.empty(total, dtype=torch.uint8, device="cuda")
        self.bases = total
        self.kernel = "bpe_lds_kernel"
        self.name = (f"C5 ragged, {n_batches} x 4096 sequences ({total / 1e6:.1f} Mbp) per call: BPE vocab-4096 + char in one pass over the bytes, "
                     f"packed ids/offsets/masks")
        self.step()
        torch.cuda.synchronize()
        n_tok = int(self.out_off[-1].item())
        # input once; char: 4+1 B/base; BPE: 4+1 B/token; two offset arrays
        self.algorithmic_bytes = total + 5 * total + 5 * n_tok + 2 * 8 * (self.n_seqs + 1)

    def step(self):
        from dnatok_amd import encoders
        if self.one_pass:
            # BPE tokens and single-character ids from one pass over the bytes
            self.bpe.encode_with_chars(self.data, self.off, self.max_len, self.lut_dev, tok_tmp=self.tok,
                                       lengths=self.lengths, char_ids=self.cids, char_mask=self.cmask)
        else:
            self.bpe.encode(self.data, self.off, self.max_len, tok_tmp=self.tok, lengths=self.lengths)
        self.pids, self.out_off, self.pmask = encoders.pack_ragged(self.tok, self.off, self.lengths,
                                                                   out=self.pack_out)
        if not self.one_pass:
            self.char.encode_packed(self.data, want_mask=True, ids=self.cids, mask=self.cmask)

    def check(self):
        """The first 4096 sequences against the committed golden vectors; with more batches per call,
        the last 512 sequences against the Hugging Face tokenizers run here."""
        import torch
        from tests.golden import check as util
        from tests.support import hf_tokenizers as hf
        self.step()
        torch.cuda.synchronize()
        b = self.first
        oo, flat = self.out_off.cpu().numpy(), self.pids.cpu().numpy()
        util.check_against_golden("C5_bpe4096", [flat[oo[i]:oo[i + 1]] for i in range(b.n_seqs)])
        cf = self.cids.cpu().numpy()
        util.check_against_golden("C5_char", [cf[b.offsets[i]:b.offsets[i + 1]] for i in range(b.n_seqs)])
        assert bool((self.pmask[:int(oo[-1])] == 1).all()) and bool((self.cmask == 1).all())
        if self.n_seqs > b.n_seqs:
            lo = self.n_seqs - 512
            base = int(self.offsets[lo])
            rel = self.offsets[lo:] - base
            want = hf_live_rows(hf.load_bpe_tokenizer("4096"), self.host[base:], rel)
            same_rows([flat[oo[i]:oo[i + 1]] for i in range(lo, self.n_seqs)], want, "C5 BPE last sequences")
            want = hf_live_rows(hf.build_char_tokenizer(), self.host[base:], rel)
            same_rows([cf[self.offsets[i]:self.offsets[i + 1]] for i in range(lo, self.n_seqs)], want,
                      "C5 char last sequences")

    def oracle_port(self, budget_s: float):
        from oracle import oracle as O
        bo = O.bpe_oracle_from_tokenizer_json(self.cfg)
        b = self.first
        rows = 1024
        data, off = b.data[:b.offsets[rows]], b.offsets[:rows + 1]
        reps, t0 = 0, time.perf_counter()
        while True:
            bo.encode_batch(data, off)
            O.char_encode_packed(self.lut, data)
            reps += 1
            if time.perf_counter() - t0 > budget_s:
                break
        dt = time.perf_counter() - t0
        return int(off[-1]) * reps / dt / 1e6, f"first {rows} sequences ({int(off[-1])} bp), {reps} passes"


def make_workload(config: str, sustained: bool, guess: str = "previous") -> Workload:
    if config == "C1":
        return CharDense(340 if sustained else 1)
    if config == "C2":
        return KmerPadded(256 if sustained else 1, guess=guess)
    if config == "C3":
        return BpePadded("4096", 16 if sustained else 1)
    if config == "C4":
        return BpePadded("32000", 8 if sustained else 1)
    if config == "C5":
        return RaggedBoth(8 if sustained else 1)
    raise SystemExit(f"unknown config {config}")


# ------------------------------------------------------------------------------ timing

def time_steps(w: Workload, steps: int, warmup: int):
    import torch
    for _ in range(warmup):
        w.step()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        w.step()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    dev_ms = start.elapsed_time(end) / steps
    return wall_ms, dev_ms


def step_spread(w: Workload, steps: int = 100) -> dict:
    """Device time of single steps (an event between every two of them): median, p5 and p95 in
    microseconds.  A pass of its own after the timed region, which is bracketed as a whole (the
    event between two steps costs each of them a microsecond or two)."""
    import torch
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    for _ in range(10):
        w.step()
    torch.cuda.synchronize()
    marks[0].record()
    for i in range(steps):
        w.step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    us = np.array([marks[i].elapsed_time(marks[i + 1]) * 1e3 for i in range(steps)])
    return {"n": steps, "median_us": float(np.median(us)), "p5_us": float(np.percentile(us, 5)),
            "p95_us": float(np.percentile(us, 95)), "min_us": float(us.min()), "max_us": float(us.max())}


def hf_cpu(config: str, threads: int, max_bases: int) -> dict | None:
    env = dict(os.environ, RAYON_NUM_THREADS=str(threads), TOKENIZERS_PARALLELISM="true")
    cmd = [sys.executable, "-m", "tests.support.hf_baseline", "--config", config, "--budget", "12"]
    if max_bases:
        cmd += ["--max-bases", str(max_bases)]
    try:
        out = subprocess.run(cmd, env=env, cwd=ROOT, capture_output=True, text=True, timeout=240)
        line = [l for l in out.stdout.splitlines() if l.startswith("{")][-1]
        return json.loads(line)
    except Exception as e:          # tokenizers missing or too slow: report that, invent nothing
        return {"error": f"{type(e).__name__}: {e}"}


def memory_only_extra(w, dev_ms: float) -> dict:
    """What this machine gives the 6-mer workload's loads and stores when nothing is computed
    (dnatok_diag_kmer_shape: the same rows, steps, strides and padding, no arithmetic), and its
    fastest plain copy (dnatok_diag_copy_tiles), beside the encoder's own step."""
    import ctypes
    import torch
    from dnatok_amd import build as _build
    # the measurement kernels are a library of their own (include/dnatok_diag.h), not part of the product
    L = ctypes.CDLL(_build.DIAG_LIB_PATH)
    L.dnatok_last_error.restype = ctypes.c_char_p
    L.dnatok_diag_copy_tiles.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    L.dnatok_diag_kmer_shape.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]

    def ok(rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed ({rc}): {L.dnatok_last_error().decode(errors='replace')}")

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    ids = torch.empty((w.n_rows, w.t_cap), dtype=torch.int32, device="cuda")
    mask = torch.empty((w.n_rows, w.t_cap), dtype=torch.uint8, device="cuda")
    fill = sum(w.widths) // 2

    def timed(fn, n):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    shape_ms = timed(lambda: ok(L.dnatok_diag_kmer_shape(ptr(w.sets[0]), ptr(w.off), w.n_rows, w.t_cap, fill,
                                                                 ptr(ids), ptr(mask), stream), "dnatok_diag_kmer_shape"), 100)
    del ids, mask
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    copy_ms = timed(lambda: ok(L.dnatok_diag_copy_tiles(ptr(src), ptr(dst), n, stream), "dnatok_diag_copy_tiles"), 30)
    same = bool(torch.equal(src, dst))
    del src, dst
    by = w.algorithmic_bytes
    return {"kmer_shape": {"what": "the workload's loads and stores without the arithmetic: same rows, 1536-byte steps, "
                                   f"row stride {w.t_cap} cells, padded to {fill} cells",
                           "device_ms_per_step": shape_ms, "GB/s": by / (shape_ms * 1e-3) / 1e9,
                           "hbm_frac": by / (shape_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                           "encoder_rate_over_this": shape_ms / dev_ms},
            "copy_tiles_1GiB": {"what": "device-to-device copy of 1 GiB in contiguous 16 KB tiles per workgroup "
                                        "(1 GiB read + 1 GiB written)", "device_ms": copy_ms,
                                "GB/s": 2 * n / (copy_ms * 1e-3) / 1e9, "hbm_frac": 2 * n / (copy_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                "copied_exactly": same}}


def fused_embed_extra():
    """Fused byte -> id -> embedding row kernel on one C1 batch (64 x 8192 bases), bf16 rows of 512:
    1 byte read and 1 KiB written per base; checked against the two-step torch form."""
    import torch
    from dnatok_amd import encoders
    from tests.support import hf_tokenizers as hf, workloads as wl
    vocab = hf.char_vocab()
    lut = np.zeros(256, dtype=np.int32)
    for ch in "ACGTN":
        lut[ord(ch)] = vocab[ch]
    enc = encoders.CharEncoder(lut, 1)
    data = _dev(wl.config1_char().data)
    weight = torch.randn((len(vocab), 512), device="cuda").to(torch.bfloat16)
    out = torch.empty((data.numel(), 512), dtype=torch.bfloat16, device="cuda")
    enc.embed_packed(data, weight, out=out)
    ids, _ = enc.encode_packed(data)
    assert torch.equal(out.view(torch.int16), weight[ids.long()].view(torch.int16)), "fused embedding gather differs"

    class W:
        def step(self):
            enc.embed_packed(data, weight, out=out)
    wm, dm = time_steps(W(), 20, 3)
    by = data.numel() * (1 + 1024)
    return {"workload": "C1 batch 64x8192 bases -> bf16 [B, T, 512]", "ms_per_call": wm, "device_ms_per_call": dm,
            "mbp_per_s": data.numel() / (wm * 1e-3) / 1e6, "algorithmic_bytes": by,
            "hbm_frac": by / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS, "kernel": "char_embed_kernel"}


def unpack_2bit_extra():
    """2-bit packed bases -> int32 ids, sustained form: 340 distinct C1 batches (178 Mbp) packed on
    the host by the library, one launch; 0.25 byte read and 4 bytes written per base; checked
    against the byte path's ids wherever the text is ACGT (N travels as A)."""
    import torch
    from dnatok_amd import encoders
    from tests.support import hf_tokenizers as hf
    vocab = hf.char_vocab()
    lut = np.zeros(256, dtype=np.int32)
    for ch in "ACGTN":
        lut[ord(ch)] = vocab[ch]
    enc = encoders.CharEncoder(lut, 1)
    n_rows = 64 * 340
    host = many_batches_uniform(n_rows, 8192, 7001, n_rate=0.001).reshape(n_rows, 8192)
    t0 = time.perf_counter()
    packed_h = encoders.pack_2bit_host(torch.from_numpy(host))
    pack_s = time.perf_counter() - t0
    packed = packed_h.to("cuda")
    ids = torch.empty((n_rows, 8192), dtype=torch.int32, device="cuda")
    enc.unpack_2bit(packed, 8192, out=ids)
    want = lut[host[-64:]].copy()
    want[host[-64:] == ord("N")] = lut[ord("A")]
    assert np.array_equal(ids[-64:].cpu().numpy(), want), "2-bit unpack differs"

    class W:
        def step(self):
            enc.unpack_2bit(packed, 8192, out=ids)
    wm, dm = time_steps(W(), 10, 2)
    by = host.size * 4 + host.size // 4
    return {"workload": "340 C1 batches (64x8192 bases each), 2-bit packed -> int32 ids", "ms_per_call": wm,
            "device_ms_per_call": dm, "mbp_per_s": host.size / (wm * 1e-3) / 1e6, "algorithmic_bytes": by,
            "hbm_frac": by / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS, "kernel": "char_unpack2bit_kernel",
            "host_pack_mbp_per_s_1_core": host.size / pack_s / 1e6}


def device_normalizer_extra():
    """Normalizer steps on the device over the C5 batch (4096 ragged rows, ~12 Mbp): strip,
    N{10,} -> "-", prepend "_", lowercase (four steps, fused into one compaction pass), beside the
    same steps as Python callables string by string on one host core; results compared row by row."""
    import torch
    from dnatok_amd import encoders
    from tests.support import workloads as wl
    from dnatok_amd.gputok_bpe_backend import _compile_normalizer_step, _device_steps_of
    spec = {"type": "Sequence", "normalizers": [
        {"type": "Strip", "strip_left": True, "strip_right": True},
        {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "-"},
        {"type": "Prepend", "prepend": "_"},
        {"type": "Lowercase"}]}
    b = wl.config5_ragged()
    data, offsets = _dev(b.data), _dev(b.offsets)
    norm = encoders.RowNormalizer(_device_steps_of(spec))
    total, longest = int(b.offsets[-1]), int(np.diff(b.offsets).max())
    out, out_off, _, _ = norm.apply(data, offsets, total, longest)
    host_fn = _compile_normalizer_step(spec)
    raw = b.data.tobytes()
    rows = [raw[b.offsets[i]:b.offsets[i + 1]].decode("ascii") for i in range(b.n_seqs)]
    t0 = time.perf_counter()
    want = [host_fn(r) for r in rows]
    host_s = time.perf_counter() - t0
    got_off = out_off.cpu().numpy()
    got = out.cpu().numpy().tobytes()
    assert all(got[got_off[i]:got_off[i + 1]].decode("ascii") == want[i] for i in range(b.n_seqs)), \
        "device normalizer differs from the host callables"

    class W:
        def step(self):
            norm.apply(data, offsets, total, longest)
    wm, dm = time_steps(W(), 20, 3)
    by = 3 * total                                                 # one pass: every byte read by count and emit, written once
    return {"workload": "C5 batch, 4096 ragged rows: strip + N{10,} -> '-' + prepend + lowercase", "steps": 4,
            "passes": 1,
            "ms_per_call": wm, "device_ms_per_call": dm, "mbp_per_s": total / (wm * 1e-3) / 1e6,
            "algorithmic_bytes": by, "hbm_frac": by / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "host_python_mbp_per_s_1_core": total / host_s / 1e6,
            "kernels": "norm_rows_kernel + norm_count_kernel + norm_emit_kernel"}


def pathological_extra():
    """BPE on rows made of long runs of equal pairs (a homopolymer, tandem repeats), beside random rows
    of the same size: a run makes every pair's rank equal to its neighbour's, the case in which a
    candidate's walk along its left chain would be as long as the run.  Every row is checked against
    the Hugging Face tokenizer run here."""
    import random
    import torch
    from dnatok_amd import bpe_vocab, encoders
    from tests.support import hf_tokenizers as hf
    rng = random.Random(3)
    rnd = lambda n: "".join(rng.choices("ACGT", k=n))
    out = {}
    for which in ("4096", "32000"):
        with open(hf.bpe_tokenizer_path(which)) as fh:
            cfg = json.load(fh)
        kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
        vocab = cfg["model"]["vocab"]
        enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv), out_remap=kv.remap_to(vocab, vocab["[UNK]"]))
        tk = hf.load_bpe_tokenizer(which)
        rows = {}
        for name, text in (("random_2kb", rnd(2048)), ("poly_a_2kb", "A" * 2048), ("ac_repeat_2kb", "AC" * 1024),
                           ("random_100kb", rnd(100_000)), ("poly_a_100kb", "A" * 100_000),
                           ("aaat_repeat_100kb", "AAAT" * 25_000)):
            host = np.frombuffer(text.encode("ascii"), dtype=np.uint8)
            data, off = _dev(host), _dev(np.array([0, host.size], dtype=np.int64))
            tok = torch.empty(host.size, dtype=torch.int32, device="cuda")
            lengths = torch.empty(1, dtype=torch.int32, device="cuda")
            enc.encode(data, off, host.size, tok_tmp=tok, lengths=lengths)
            torch.cuda.synchronize()
            got = tok[:int(lengths.item())].cpu().numpy()
            same_rows([got], hf_live_rows(tk, host, [0, host.size]), f"BPE vocab-{which} {name}")

            class W:
                def step(self):
                    enc.encode(data, off, host.size, tok_tmp=tok, lengths=lengths)
            _, dm = time_steps(W(), 10, 2)
            rows[name] = {"device_us_per_call": dm * 1e3}
        rows["poly_a_2kb_over_random_2kb"] = rows["poly_a_2kb"]["device_us_per_call"] / rows["random_2kb"]["device_us_per_call"]
        out[f"vocab_{which}"] = rows
    return out


def short_reads_extra():
    """BPE (vocabulary 4096) on batches of short reads, 100 to 300 bp each, padded by the engine: the
    shape of a sequencing run rather than of the five configurations.  Rows this short go to teams
    of one wave and are handed out through several work counters; the last 512 rows of every batch
    are checked against the Hugging Face tokenizer run here."""
    import torch
    from dnatok_amd import bpe_vocab, encoders
    from tests.support import hf_tokenizers as hf
    with open(hf.bpe_tokenizer_path("4096")) as fh:
        cfg = json.load(fh)
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    vocab = cfg["model"]["vocab"]
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv), out_remap=kv.remap_to(vocab, vocab["[UNK]"]))
    tk = hf.load_bpe_tokenizer("4096")
    rng = np.random.Generator(np.random.PCG64(1006))
    out = {}
    for n_rows in (4096, 20_000, 100_000):
        lens = rng.integers(100, 301, n_rows)
        off_h = np.zeros(n_rows + 1, dtype=np.int64)
        off_h[1:] = np.cumsum(lens)
        host = rng.choice(np.frombuffer(b"ACGT", dtype=np.uint8), int(off_h[-1]), p=[.295, .205, .205, .295])
        data, off = _dev(host), _dev(off_h)
        stride = 128
        buf = (torch.empty((n_rows, stride), dtype=torch.int32, device="cuda"),
               torch.empty((n_rows, stride), dtype=torch.uint8, device="cuda"),
               torch.empty(n_rows, dtype=torch.int32, device="cuda"), torch.empty(1, dtype=torch.int32, device="cuda"))

        class W:
            def step(self):
                enc.encode_padded(data, off, 300, stride, vocab["[PAD]"], out=buf)
        W().step()
        torch.cuda.synchronize()
        ln = buf[2].cpu().numpy()
        assert int(buf[3].item()) == int(ln.max()) <= stride
        first = n_rows - 512
        want = hf_live_rows(tk, host[off_h[first]:], off_h[first:] - off_h[first])
        same_rows([buf[0][first + r, :ln[first + r]].cpu().numpy() for r in range(512)], want, f"short reads, {n_rows} rows")
        _, dm = time_steps(W(), 50, 10)
        out[f"{n_rows}_rows"] = {"bases": int(off_h[-1]), "device_us_per_call": dm * 1e3,
                                 "mbp_per_s": float(off_h[-1]) / (dm * 1e-3) / 1e6}
        if n_rows == 100_000:
            out["6mer_100000_rows"] = short_reads_kmer(host, off_h, data, off)
    return out


def short_reads_kmer(host, off_h, data, off) -> dict:
    """The same reads through the 6-mer encoder (rows 128 cells apart, padded to the longest),
    the last 512 rows checked against the Hugging Face tokenizer run here."""
    import torch
    from dnatok_amd import encoders, kmer_tables
    from tests.support import hf_tokenizers as hf
    vocab = hf.kmer_vocab(6)
    t = kmer_tables.tables_from_vocab(vocab, 6, vocab["<unk>"])
    enc = encoders.KmerEncoder(6, t.digit, t.kmer_lut, t.single, vocab["<pad>"], vocab["<unk>"],
                               t.exp_off, t.exp_len, t.exp_flat)
    n_rows = off_h.size - 1
    buf = (torch.empty((n_rows, 128), dtype=torch.int32, device="cuda"), torch.empty((n_rows, 128), dtype=torch.uint8, device="cuda"),
           torch.empty(n_rows, dtype=torch.int32, device="cuda"), torch.empty(n_rows, dtype=torch.int32, device="cuda"),
           torch.empty(1, dtype=torch.int32, device="cuda"))

    class W:
        def step(self):
            enc.encode_padded(data, off, 128, fill_to=0, width_guess=64, out=buf)
    W().step()
    torch.cuda.synchronize()
    ln = buf[2].cpu().numpy()
    width = int(buf[4].item())
    assert width == int(ln.max()) and int(buf[3].abs().sum().item()) == 0
    first = n_rows - 512
    want = hf_live_rows(hf.build_kmer_tokenizer(6), host[off_h[first]:], off_h[first:] - off_h[first])
    same_rows([buf[0][first + r, :ln[first + r]].cpu().numpy() for r in range(512)], want, "short reads, 6-mer")
    _, dm = time_steps(W(), 50, 10)
    by = int(off_h[-1]) + 5 * n_rows * width + 4 * n_rows
    out = {"bases": int(off_h[-1]), "device_us_per_call": dm * 1e3, "mbp_per_s": float(off_h[-1]) / (dm * 1e-3) / 1e6,
           "hbm_frac": by / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS}

    def packed(d, o, o_h, h, what):
        """The packed layout (tokens back to back, no padding): 1 B read twice per base, 4 B per
        token, 8 B of offsets and 4 B of length per row."""
        n = o_h.size - 1
        pbuf = (torch.empty(int(o_h[-1]), dtype=torch.int32, device="cuda"), torch.empty(n + 1, dtype=torch.int64, device="cuda"),
                None, torch.empty(n, dtype=torch.int32, device="cuda"), torch.empty(n, dtype=torch.int32, device="cuda"))

        class P:
            def step(self):
                enc.encode_packed(d, o, out=pbuf)
        P().step()
        torch.cuda.synchronize()
        oo = pbuf[1].cpu().numpy()
        flat = pbuf[0].cpu().numpy()
        rows = np.concatenate([np.arange(n - 256, n), np.argsort(o_h[1:] - o_h[:-1])[-8:]])
        want = hf_live_rows(hf.build_kmer_tokenizer(6), np.concatenate([h[o_h[r]:o_h[r + 1]] for r in rows]),
                            np.concatenate([[0], np.cumsum([o_h[r + 1] - o_h[r] for r in rows])]))
        same_rows([flat[oo[r]:oo[r + 1]] for r in rows], want, what)
        _, pm = time_steps(P(), 50, 10)
        pby = 2 * int(o_h[-1]) + 4 * int(oo[-1]) + 12 * n
        return {"tokens": int(oo[-1]), "device_us_per_call": pm * 1e3, "mbp_per_s": float(o_h[-1]) / (pm * 1e-3) / 1e6,
                "hbm_frac": pby / (pm * 1e-3) / 1e9 / HBM_PEAK_GBS}

    out["packed"] = packed(data, off, off_h, host, "short reads, 6-mer, packed")
    # the same reads with 50 rows of 2-20 kbp among them: every row gets its kernel by its own length
    rng = np.random.Generator(np.random.PCG64(1007))
    where = np.sort(rng.choice(n_rows, 50, replace=False))
    parts, lens2, prev = [], [], 0
    for at in where:
        parts.append(host[off_h[prev]:off_h[at]])
        lens2.extend((off_h[prev + 1:at + 1] - off_h[prev:at]).tolist())
        n_long = int(rng.integers(2000, 20001))
        parts.append(rng.choice(np.frombuffer(b"ACGT", dtype=np.uint8), n_long))
        lens2.append(n_long)
        prev = at
    parts.append(host[off_h[prev]:])
    lens2.extend((off_h[prev + 1:] - off_h[prev:-1]).tolist())
    host2 = np.concatenate(parts)
    off2_h = np.zeros(len(lens2) + 1, dtype=np.int64)
    off2_h[1:] = np.cumsum(lens2)
    data2, off2 = _dev(host2), _dev(off2_h)
    n2 = off2_h.size - 1
    cap2 = int(max(lens2)) // 6 + 6
    cap2 += (-cap2) % 128
    buf2 = (torch.empty((n2, cap2), dtype=torch.int32, device="cuda"), torch.empty((n2, cap2), dtype=torch.uint8, device="cuda"),
            torch.empty(n2, dtype=torch.int32, device="cuda"), torch.empty(n2, dtype=torch.int32, device="cuda"),
            torch.empty(1, dtype=torch.int32, device="cuda"))
    mixed = {"rows": n2, "bases": int(off2_h[-1]), "rows_apart": cap2}
    for name, team_rows in (("by_row_class", -1), ("a_wave_per_row", 0)):
        enc.set_team_rows(team_rows)

        class M:
            def step(self):
                enc.encode_padded(data2, off2, cap2, fill_to=0, width_guess=0, out=buf2)
        M().step()
        torch.cuda.synchronize()
        ln2 = buf2[2].cpu().numpy()
        rows = np.concatenate([np.arange(n2 - 128, n2), np.argsort(lens2)[-8:]])
        want = hf_live_rows(hf.build_kmer_tokenizer(6), np.concatenate([host2[off2_h[r]:off2_h[r + 1]] for r in rows]),
                            np.concatenate([[0], np.cumsum([lens2[r] for r in rows])]))
        same_rows([buf2[0][r, :ln2[r]].cpu().numpy() for r in rows], want, f"mixed rows, 6-mer, {name}")
        _, mm = time_steps(M(), 30, 5)
        mixed[name + "_us_per_call"] = mm * 1e3
    enc.set_team_rows(-1)
    mixed["packed"] = packed(data2, off2, off2_h, host2, "mixed rows, 6-mer, packed")
    out["with_50_rows_of_2_to_20_kbp"] = mixed
    return out


def kmer_rows_with_n_extra():
    """The 6-mer encoder on 65,536 rows of 6000 bp that differ only in where they hold N: none, one
    per row (anywhere / at the start: every later step of the row is then written shifted), 32
    windows of N at the start (160 extra cells: later steps fall on whole lines again) and the
    workload's 0.5 % in runs of 1-50.  Every data set is checked against the Hugging Face tokenizer
    run here on a sample of rows; the stride and the guess follow the library's policy for a stream
    of batches."""
    import torch
    from dnatok_amd import encoders, kmer_tables
    from tests.support import hf_tokenizers as hf
    n_rows, length = 65536, 6000
    vocab = hf.kmer_vocab(6)
    t = kmer_tables.tables_from_vocab(vocab, 6, vocab["<unk>"])
    enc = encoders.KmerEncoder(6, t.digit, t.kmer_lut, t.single, vocab["<pad>"], vocab["<unk>"],
                               t.exp_off, t.exp_len, t.exp_flat)
    tk = hf.build_kmer_tokenizer(6)
    off = _dev(np.arange(n_rows + 1, dtype=np.int64) * length)
    rng = np.random.default_rng(5)

    def free():
        return many_batches_uniform(n_rows, length, 7002)

    def one_anywhere():
        a = free().reshape(n_rows, length)
        a[np.arange(n_rows), rng.integers(0, length, n_rows)] = ord("N")
        return a.reshape(-1)

    def at_start(n_windows):
        a = free().reshape(n_rows, length)
        a[:, :max(1, 6 * n_windows)] = ord("N")
        return a.reshape(-1)

    out = {}
    for name, make in (("no_n", free), ("one_n_per_row_anywhere", one_anywhere),
                       ("one_n_at_row_start", lambda: at_start(0)), ("32_n_windows_at_row_start", lambda: at_start(32)),
                       ("workload_runs_of_n", lambda: many_batches_uniform(n_rows, length, 7002, n_run_fraction=0.005))):
        host = make()
        data = _dev(host)
        r = enc.encode_padded(data, off, 6016, fill_to=0)
        torch.cuda.synchronize()
        width = int(r[4].item())
        del r
        guess = encoders.width_guess_after(width)
        t_cap = guess + (-guess) % 128
        buf = (torch.empty((n_rows, t_cap), dtype=torch.int32, device="cuda"),
               torch.empty((n_rows, t_cap), dtype=torch.uint8, device="cuda"),
               torch.empty(n_rows, dtype=torch.int32, device="cuda"), torch.empty(n_rows, dtype=torch.int32, device="cuda"),
               torch.empty(1, dtype=torch.int32, device="cuda"))

        class W:
            def step(self):
                enc.encode_padded(data, off, t_cap, fill_to=0, width_guess=guess, out=buf)
        W().step()
        torch.cuda.synchronize()
        assert int(buf[4].item()) == width
        rows = np.concatenate([np.arange(64), rng.integers(0, n_rows, 64)])
        want = hf_live_rows(tk, np.concatenate([host[r * length:(r + 1) * length] for r in rows]),
                            np.arange(rows.size + 1, dtype=np.int64) * length)
        ids, ln = buf[0].cpu().numpy(), buf[2].cpu().numpy()
        same_rows([ids[r, :ln[r]] for r in rows], want, f"6-mer rows, {name}")
        _, dm = time_steps(W(), 10, 3)
        by = n_rows * length + 5 * n_rows * width + 4 * n_rows
        out[name] = {"t_max": width, "rows_apart": t_cap, "device_us_per_call": dm * 1e3,
                     "hbm_frac": by / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS}
        del data, buf
        torch.cuda.empty_cache()
    return out


def strings_in_extra():
    """What a caller of DNATok sees: Python strings in, int64 ids back on the host
    (`DNATok.encode_batch_to_ids`), on the workload of the reference's own CLI example
    (docs/CLI.md:104-115: 1000 sequences of 4096 bp) at 32 and at 256 sequences per call, for the
    single-nucleotide, the 6-mer and the BPE-4096 tokenizer.  Every call's ids are compared with the
    Hugging Face tokenizer's (an untimed pass); the tokenizer itself is timed beside it on this
    host's threads.  Includes the bus both ways and all of the Python around the kernels."""
    import random
    import torch
    from dnatok_amd import dnatok_cli
    from tests.support import hf_tokenizers as hf
    rng = random.Random(42)
    seqs = ["".join(rng.choices("ACGT", k=4096)) for _ in range(1000)]
    bases = sum(map(len, seqs))
    out = {"workload": "1000 sequences x 4096 bp of random ACGT, strings in, int64 ids on the host out",
           "host_threads": host_threads()}
    for name, model in (("char", "char"), ("kmer6", "kmer6"), ("bpe4096", hf.bpe_tokenizer_path("4096"))):
        tok, dn = dnatok_cli._build_dnatok(model, "cuda")
        row = {"path": dnatok_cli._detect_path(dn)}
        for chunk in (32, 256):
            for i in range(0, len(seqs), chunk):                       # untimed: warm-up and the check
                got = dn.encode_batch_to_ids(seqs[i:i + chunk])
                want = tok(seqs[i:i + chunk], add_special_tokens=False)["input_ids"]
                for r, w_ in zip(got.tolist(), want):
                    assert r[:len(w_)] == list(w_) and all(x == dn.id_pad for x in r[len(w_):]), (name, chunk, i)
            best = None
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(0, len(seqs), chunk):
                    dn.encode_batch_to_ids(seqs[i:i + chunk])
                torch.cuda.synchronize()
                dt = time.perf_counter() - t0
                best = dt if best is None or dt < best else best
            t0 = time.perf_counter()
            for i in range(0, len(seqs), chunk):
                tok(seqs[i:i + chunk], add_special_tokens=False)
            t_hf = time.perf_counter() - t0
            row[f"{chunk}_per_call"] = {"mbp_per_s": bases / best / 1e6, "ms_per_call": best / ((len(seqs) + chunk - 1) // chunk) * 1e3,
                                        "hf_tokenizers_mbp_per_s": bases / t_hf / 1e6}
        out[name] = row
        del dn, tok
        torch.cuda.empty_cache()
    return out


PHASE_NAMES = ["initial_pairs", "round_minimum", "collect_candidates", "decide", "late_walks_or_scan", "apply",
               "re_rank", "refresh", "output"]


def bpe_phase_cycles_extra():
    """Where the teams of the BPE engine spend their cycles, phase by phase, on the three BPE
    configurations: from the build of the library with the phase clocks compiled in
    (libdnatok_hip_phases.so, which this process loads in place of the product library: run with
    --only-extra bpe_phase_cycles, nothing else in the line is then the product's).  The shares are
    what thread 0 of each team saw, barriers counted with the phase they end."""
    import ctypes
    import torch
    from dnatok_amd import _lib
    L = _lib.lib()
    if not hasattr(L, "dnatok_bpe_phase_cycles"):
        raise RuntimeError("the loaded library has no phase clocks (python -m dnatok_amd.build makes libdnatok_hip_phases.so)")
    cells = (ctypes.c_ulonglong * 16)()
    out = {}
    for cfg, sustained in (("C3", False), ("C3", True), ("C4", False), ("C5", False)):
        w = make_workload(cfg, sustained)
        w.check()
        _lib.check(L.dnatok_bpe_phase_cycles(cells, 1), "dnatok_bpe_phase_cycles")
        _, dm = time_steps(w, 20, 0)
        _lib.check(L.dnatok_bpe_phase_cycles(cells, 1), "dnatok_bpe_phase_cycles")
        total = float(sum(cells[:9])) or 1.0
        items, positions = int(cells[15]) or 1, int(cells[14]) or 1
        out[cfg + ("_sustained" if sustained else "_per_call")] = {
            "workload": w.name, "device_ms_per_call_instrumented": dm,
            "share": {n: round(cells[q] / total, 4) for q, n in enumerate(PHASE_NAMES)},
            "cycles_per_position": round(total / positions, 2), "rounds_per_item": round(cells[12] / items, 2),
            "merges_per_item": round(cells[13] / items, 1), "positions_per_item": round(positions / items, 1)}
        del w
        torch.cuda.empty_cache()
    return out


def merge_table_placement_extra():
    """The BPE merge table of the 4096 vocabulary in global memory (L2; the default) against its compact
    48 KB form kept in LDS by every workgroup (`dnatok_bpe_table_set_placement`), on batches of 1 KB rows:
    512 rows (one per workgroup resident with the table in LDS) and the C3 batch of 1024 rows (two rounds
    of workgroups with the table in LDS).  Tokens compared between the placements and, for C3, with the
    golden vectors."""
    import torch
    from dnatok_amd import _lib, bpe_vocab, encoders
    from tests.golden import check as util
    from tests.support import hf_tokenizers as hf, workloads as wl
    with open(hf.bpe_tokenizer_path("4096")) as fh:
        cfg = json.load(fh)
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    vocab = cfg["model"]["vocab"]
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv), out_remap=kv.remap_to(vocab, vocab["[UNK]"]))
    place = enc.set_table_placement
    out = {}
    try:
        for rows in (512, 1024):
            b = wl.config3_bpe4096() if rows == 1024 else wl.config3_bpe4096(rows, 1024, seed=wl.SEEDS["C3"] + 7)
            data, off = _dev(b.data), _dev(b.offsets)
            tok = torch.empty(b.total, dtype=torch.int32, device="cuda")
            lengths = torch.empty(rows, dtype=torch.int32, device="cuda")
            seen = {}
            for name, mode in (("global_memory", 0), ("lds", 2)):
                place(mode)
                enc.encode(data, off, 1024, tok_tmp=tok, lengths=lengths)
                torch.cuda.synchronize()
                ln = lengths.cpu().numpy()
                flat = tok.cpu().numpy()
                seen[name] = [flat[b.offsets[i]:b.offsets[i] + ln[i]].copy() for i in range(rows)]

                class W:
                    def step(self):
                        enc.encode(data, off, 1024, tok_tmp=tok, lengths=lengths)
                _, dm = time_steps(W(), 20, 3)
                out[f"{rows}_rows_{name}_us"] = dm * 1e3
            same_rows(seen["lds"], seen["global_memory"], f"merge table placement, {rows} rows")
            if rows == 1024:
                util.check_against_golden("C3_bpe4096", seen["lds"])
    finally:
        place(0)
    return out


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400,
                    help="timed steps (the default runs the headline for 70 ms: the first tens of steps after an idle\n"
                         "period run 2-3 %% slower than the hundreds after them)")
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--config", default="C2", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--per-call", action="store_true", help="time one exact batch instead of the sustained form")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--only-extra", default="", choices=["", "merge_table_placement", "pathological", "kmer_rows_with_n", "strings_in",
                                                         "short_reads", "bpe_phase_cycles"],
                    help="run only this extra after the headline (for profiling it)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, the known-size kernel that the "
                         "FETCH_SIZE / WRITE_SIZE counters are scaled by when profiling")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this backend and this benchmark are single-GPU (rows are independent: several "
              "GPUs would each take a share of the rows, with no exchange). Run with --gpus 1.", file=sys.stderr)
        raise SystemExit(2)
    if args.only_extra == "bpe_phase_cycles":
        # the build with the phase clocks in place of the product library, for this whole process
        from dnatok_amd import _lib, build as _build
        _lib.LIB_PATH = _build.PHASES_LIB_PATH

    import torch
    from dnatok_amd import _lib
    _lib.lib()                                   # fail loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    w = make_workload(args.config, sustained=not args.per_call)
    w.check()                                    # bit-exact: golden vectors + Hugging Face tokenizers run here
    # The pass that times single steps runs first: check() keeps the host busy for seconds with the
    # GPU idle, and the first milliseconds after an idle period run 2-3 % slower than the steady
    # rate.  The timed region proper is then exactly --steps steps after --warmup warm-up steps;
    # `protocols` below also holds the same steps after an idle second and 400 steps after 50.
    spread = step_spread(w)
    wall_ms, dev_ms = time_steps(w, args.steps, args.warmup)
    value = w.bases / (wall_ms * 1e-3) / 1e6
    achieved = w.algorithmic_bytes / (dev_ms * 1e-3) / 1e9

    result = {
        "metric": "encode Mbp/s on 1 MI355X (bit-exact vs HF) + % of HBM BW roofline",
        "value": value, "unit": "Mbp/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": w.name, "bases_per_step": int(w.bases),
                   "algorithmic_bytes_per_step": int(w.algorithmic_bytes)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None, "kernel": w.kernel,
                     "device_ms_per_step": dev_ms,
                     "timed": "HIP events on the launch stream around the timed steps; a step is the kernel named "
                              "here plus the small launches of the same call"},
        "bit_exact": "golden vectors written by Hugging Face tokenizers + rows of the last batch against "
                     "Hugging Face tokenizers run in this process",
    }
    if args.config in ("C3", "C4", "C5"):
        result["roofline"]["note"] = BPE_BOUND_NOTE
    result["step_spread"] = spread
    frac_of = lambda ms: w.algorithmic_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
    protocols = {"as_run": {"steps": args.steps, "warmup": args.warmup, "before": "the step-spread pass (110 steps)",
                            "device_ms_per_step": dev_ms, "hbm_frac": frac_of(dev_ms)}}
    if not args.per_call:
        _, long_ms = time_steps(w, 400, 50)
        protocols["steady"] = {"steps": 400, "warmup": 50, "device_ms_per_step": long_ms, "hbm_frac": frac_of(long_ms)}
        torch.cuda.synchronize()
        time.sleep(1.0)
        _, cold_ms = time_steps(w, args.steps, args.warmup)
        protocols["after_idle"] = {"steps": args.steps, "warmup": args.warmup, "before": "one second with the GPU idle",
                                   "device_ms_per_step": cold_ms, "hbm_frac": frac_of(cold_ms)}
    result["roofline"]["protocols"] = protocols

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.config == "C2" and not args.per_call and (args.calibrate_copy or not args.no_extras):
        result["memory_only"] = memory_only_extra(w, dev_ms)

    # HBM bytes per launch come from rocprofv3 counter runs of this same command, which cannot run
    # inside it; the committed summary says when and how they were taken
    traffic_file = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(traffic_file):
        with open(traffic_file) as fh:
            known = json.load(fh).get(f"{args.config}:{'per_call' if args.per_call else 'sustained'}")
        if known and known.get("bases_per_step") == int(w.bases) and known.get("kernel") == w.kernel:
            result["roofline"]["traffic"] = known["hbm_bytes_per_launch"]
            result["roofline"]["traffic_source"] = known["source"]

    threads = host_threads()
    if not args.no_cpu:
        cap = {"C1": 0, "C2": 0, "C3": 0, "C4": 400_000, "C5": 1_500_000}[args.config]
        hf_all, hf_one = hf_cpu(args.config, threads, cap), hf_cpu(args.config, 1, cap)
        if "mbp_per_s" in hf_all:
            result["cpu_baseline"] = {
                "value": hf_all["mbp_per_s"], "unit": "Mbp/s", "cores": threads, "kind": "reference",
                "sample": (f"Hugging Face tokenizers encode_batch (the reference's CPU path) in this run, own process, "
                           f"{threads} threads: {hf_all['n_seqs']} sequences, {hf_all['bases']} bases, median of "
                           f"{hf_all['reps']} passes"),
                "one_thread": hf_one.get("mbp_per_s")}
        else:
            result["cpu_baseline"] = {"value": None, "unit": "Mbp/s", "cores": threads, "kind": "reference",
                                      "sample": hf_all.get("error", "no result")}
        v, sample = w.oracle_port(8.0)
        result["oracle_port_cpu"] = {"value": v, "unit": "Mbp/s", "cores": 1, "kind": "port",
                                     "sample": sample + " (C restatement used by the tests, one thread)"}

    if args.only_extra:
        result[args.only_extra] = {"merge_table_placement": merge_table_placement_extra,
                                   "pathological": pathological_extra,
                                   "kmer_rows_with_n": kmer_rows_with_n_extra,
                                   "short_reads": short_reads_extra, "strings_in": strings_in_extra,
                                   "bpe_phase_cycles": bpe_phase_cycles_extra}[args.only_extra]()
    elif not args.no_extras:
        per_call = {}
        for cfg in ["C1", "C2", "C3", "C4", "C5"]:
            ww = make_workload(cfg, sustained=False)
            ww.check()
            # 200 calls: a call of 10 us is otherwise timed by the host's first, slow launches
            wm, dm = time_steps(ww, 200, 20)
            per_call[cfg] = {"workload": ww.name, "ms_per_call": wm, "device_ms_per_call": dm,
                             "mbp_per_s": ww.bases / (wm * 1e-3) / 1e6,
                             "hbm_frac": ww.algorithmic_bytes / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS}
            del ww
            torch.cuda.empty_cache()
        result["per_call"] = per_call
        sustained = {}
        for cfg in ["C1", "C2", "C3", "C4", "C5"]:
            if cfg == args.config and not args.per_call:
                continue
            ww = make_workload(cfg, sustained=True)
            ww.check()
            wm, dm = time_steps(ww, 50, 10)
            sustained[cfg] = {"workload": ww.name, "ms_per_step": wm, "device_ms_per_step": dm,
                              "mbp_per_s": ww.bases / (wm * 1e-3) / 1e6,
                              "hbm_frac": ww.algorithmic_bytes / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS}
            del ww
            torch.cuda.empty_cache()
        result["sustained"] = sustained
        if args.config == "C2" and not args.per_call:
            # the same workload under the other width-guess policies, and padded to a fixed width instead
            other = {}
            for guess in ("stale", "none", "fixed"):
                ww = make_workload("C2", sustained=True, guess=guess)
                ww.check()
                wm, dm = time_steps(ww, args.steps, args.warmup)
                other[guess] = {"workload": ww.name, "ms_per_step": wm, "device_ms_per_step": dm,
                                "mbp_per_s": ww.bases / (wm * 1e-3) / 1e6,
                                "hbm_frac": ww.algorithmic_bytes / (dm * 1e-3) / 1e9 / HBM_PEAK_GBS}
                del ww
                torch.cuda.empty_cache()
            result["width_guess_policies"] = other
        if not args.no_cpu:
            # every other configuration next to the HF CPU tokenizer of the same run (bounded samples)
            hf_rows = {}
            for cfg, cap in (("C1", 0), ("C2", 0), ("C3", 0), ("C4", 400_000), ("C5", 1_500_000)):
                if cfg == args.config:
                    continue
                hf_rows[cfg] = {"threads_1": hf_cpu(cfg, 1, cap), f"threads_{threads}": hf_cpu(cfg, threads, cap)}
            result["hf_tokenizers_cpu_other_configs"] = hf_rows
        result["fused_embedding_gather"] = fused_embed_extra()
        result["unpack_2bit"] = unpack_2bit_extra()
        result["device_normalizer"] = device_normalizer_extra()
        result["pathological"] = pathological_extra()
        result["short_reads"] = short_reads_extra()
        result["merge_table_placement"] = merge_table_placement_extra()
        result["strings_in"] = strings_in_extra()

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
