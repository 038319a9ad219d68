"""Parity of the HIP path (through the C ABI) with the CPU oracle and the golden vectors.
Bit-exact: everything here is integer / index work."""
import random

import numpy as np
import pytest
import torch

from dnatok_amd import bpe_vocab, encoders, kmer_tables
from tests.support import hf_tokenizers as hf
from tests.support import workloads as wl
from oracle import oracle as O
from tests import util

pytestmark = pytest.mark.gpu
DEV = "cuda"


def to_dev(b: wl.Batch):
    return torch.from_numpy(b.data).to(DEV), torch.from_numpy(b.offsets).to(DEV)


def say(msg):
    print(msg, flush=True)


# ------------------------------------------------------------------ char

@pytest.fixture(scope="module")
def char_enc():
    return encoders.CharEncoder(util.char_lut(), pad_id=1)


def test_char_c1_dense(char_enc):
    say("char C1 64x8192 packed/dense")
    b = wl.config1_char()
    data, off = to_dev(b)
    ids, mask = char_enc.encode_packed(data, row_len=8192, want_mask=True)
    torch.cuda.synchronize()
    rows = list(ids.cpu().numpy().reshape(64, 8192))
    util.check_against_golden("C1_char", rows)
    assert bool((mask == 1).all())
    ids2, mask2 = char_enc.encode_padded(data, off, 8192)
    torch.cuda.synchronize()
    assert torch.equal(ids2.reshape(-1), ids) and bool((mask2 == 1).all())


@pytest.mark.parametrize("t_out,pad_left", [(0, False), (37, False), (64, False), (1031, True), (4100, False), (50, True)])
def test_char_ragged_padded(t_out, pad_left):
    say(f"char ragged padded t_out={t_out} left={pad_left}")
    rng = np.random.default_rng(t_out + 1)
    lens = rng.integers(0, 3000, size=97)
    lens[:4] = [0, 1, 3, 4099]
    strings = ["".join(rng.choice(list("ACGTNacgtX"), size=n)) for n in lens]
    b = util.batch_from_strings(strings)
    lut = util.char_lut(fold_case=True)
    start = lut + 50
    for st in (None, start):
        enc = encoders.CharEncoder(lut, pad_id=1, start_lut=st)
        data, off = to_dev(b)
        ids, mask = enc.encode_padded(data, off, t_out, pad_left=pad_left)
        torch.cuda.synchronize()
        eids, emask = O.char_encode_padded(lut, b.data, b.offsets, t_out, 1, start_lut=st, pad_left=pad_left)
        np.testing.assert_array_equal(ids.cpu().numpy(), eids)
        np.testing.assert_array_equal(mask.cpu().numpy(), emask)


@pytest.mark.parametrize("total", [0, 1, 5, 4095, 4096, 4097, 123457])
def test_char_packed_sizes(char_enc, total):
    say(f"char packed total={total}")
    rng = np.random.default_rng(total)
    data_h = rng.integers(0, 256, size=total, dtype=np.uint8)
    data = torch.from_numpy(data_h).to(DEV)
    ids, mask = char_enc.encode_packed(data, want_mask=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(ids.cpu().numpy(), O.char_encode_packed(util.char_lut(), data_h))
    assert bool((mask == 1).all())


def test_char_packed_start_table():
    lut = util.char_lut()
    enc = encoders.CharEncoder(lut, pad_id=1, start_lut=lut + 7)
    for row_len in (1, 2, 3, 5, 512, 4096):
        say(f"char packed start table row_len={row_len}")
        b = wl.config1_char(9, row_len, seed=row_len)
        data, off = to_dev(b)
        ids, _ = enc.encode_packed(data, row_len=row_len)
        torch.cuda.synchronize()
        eids, _ = O.char_encode_padded(lut, b.data, b.offsets, row_len, 1, start_lut=lut + 7)
        np.testing.assert_array_equal(ids.cpu().numpy().reshape(9, row_len), eids)


@pytest.mark.parametrize("dtype,dim", [(torch.bfloat16, 512), (torch.float32, 36), (torch.float16, 8)])
def test_char_fused_embedding_gather(dtype, dim):
    """out[i, :] = weight[lut[byte[i]], :], compared with the two-step torch form; also with a
    first-column table, an id without a row (zeros) and a byte count that is no multiple of 64."""
    say(f"char fused embed {dtype} D={dim}")
    lut = util.char_lut()
    rng = np.random.default_rng(dim)
    weight = torch.from_numpy(rng.standard_normal((int(lut.max()) + 1, dim)).astype(np.float32)).to(DEV).to(dtype)
    for start, n_vocab_cut in ((None, 0), (lut + 0, 0), (None, 2)):
        enc = encoders.CharEncoder(lut, pad_id=1, start_lut=start)
        b = wl.config1_char(5, 1000 + 37, seed=dim)
        data, _ = to_dev(b)
        w = weight[:weight.shape[0] - n_vocab_cut].contiguous()
        out = enc.embed_packed(data, w, row_len=1037)
        torch.cuda.synchronize()
        ids = torch.from_numpy(O.char_encode_packed(lut, b.data)).to(DEV).long()
        ok = ids < w.shape[0]
        ref = torch.zeros((ids.numel(), dim), dtype=dtype, device=DEV)
        ref[ok] = w[ids[ok]]
        assert torch.equal(out.view(torch.uint8), ref.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
def test_char_padded_in_every_id_width(dtype):
    """Ragged rows padded on either side, ids written as uint8 / int16 / int32 / int64: widths
    that are and are not a multiple of 4 (one store of four ids, or id by id), a first-column table,
    an id that needs more than 8 bits (cut to the width, like a cast)."""
    lut = util.char_lut().copy()
    lut[ord("G")] = 300                                               # does not fit uint8
    rng = np.random.default_rng(2)
    for start in (None, lut + 5):
        enc = encoders.CharEncoder(lut, pad_id=1, start_lut=start)
        for t_out in (1, 7, 64, 1001, 4100):
            lens = rng.integers(0, t_out + 40, size=33)
            lens[0], lens[1] = 0, t_out
            rows = [rng.choice(np.frombuffer(b"ACGTN", dtype=np.uint8), size=int(n)) for n in lens]
            offsets = np.zeros(len(rows) + 1, dtype=np.int64)
            offsets[1:] = np.cumsum(lens)
            data = np.concatenate(rows) if offsets[-1] else np.zeros(0, dtype=np.uint8)
            d_data, d_off = torch.from_numpy(data).to(DEV), torch.from_numpy(offsets).to(DEV)
            for pad_left in (False, True):
                say(f"char padded {dtype} t_out={t_out} left={pad_left} start={start is not None}")
                ids, mask = enc.encode_padded(d_data, d_off, t_out, pad_left=pad_left, dtype=dtype)
                torch.cuda.synchronize()
                eids, emask = O.char_encode_padded(lut, data, offsets, t_out, 1, start_lut=start, pad_left=pad_left)
                want = torch.from_numpy(eids).to(dtype)                # the cast an int32 result would get
                assert ids.dtype == dtype and torch.equal(ids.cpu(), want)
                np.testing.assert_array_equal(mask.cpu().numpy(), emask)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int32, torch.int64])
def test_char_unpack_2bit(dtype):
    """2-bit packed rows -> ids of three widths, rows of every length mod 4 (the flat and the
    row-by-row kernel), with and without a first-column table; packed by the host function of
    the library, checked against the oracle's unpack of the oracle's packing."""
    lut = util.char_lut()
    rng = np.random.default_rng(11)
    alphabet = np.frombuffer(b"ACGTNacgt", dtype=np.uint8)
    for start in (None, lut + 3):
        enc = encoders.CharEncoder(lut, pad_id=1, start_lut=start)
        for b, t in ((3, 1), (5, 7), (4, 64), (7, 1001), (2, 8190), (64, 8192), (300, 516)):
            say(f"char unpack 2bit {dtype} B={b} T={t} start={start is not None}")
            rows = rng.choice(alphabet, size=(b, t))
            packed = encoders.pack_2bit_host(torch.from_numpy(rows))
            np.testing.assert_array_equal(packed.numpy(), O.pack_2bit(rows))
            out = torch.full((b * t + 8,), 77, dtype=dtype, device=DEV)       # guard cells behind the rows
            ids = enc.unpack_2bit(packed.to(DEV), t, dtype=dtype, out=out[:b * t].view(b, t))
            torch.cuda.synchronize()
            want = O.unpack_2bit_ids(lut, packed.numpy(), t, start_lut=start)
            np.testing.assert_array_equal(ids.cpu().numpy().astype(np.int64), want)
            assert bool((out[b * t:] == 77).all())


def test_char_c5_packed(char_enc):
    say("char C5 packed")
    b = wl.config5_ragged()
    data, off = to_dev(b)
    ids, _ = char_enc.encode_packed(data)
    torch.cuda.synchronize()
    flat = ids.cpu().numpy()
    util.check_against_golden("C5_char", [flat[b.offsets[i]:b.offsets[i + 1]] for i in range(b.n_seqs)])


# ----------------------------------------------------------------- k-mer

@pytest.fixture
def kmer_kernel_choice(request, monkeypatch):
    """Which k-mer kernel the test's batches get: a wave per row (forced for all batches) or the
    automatic choice, which gives the batches of these tests a workgroup per row.  The switch
    belongs to the table object, so every encoder is set before each of its calls."""
    rows = 0 if request.param == "rows_by_wave" else -1
    plain = encoders.KmerEncoder.encode_padded

    def encode_padded(self, *args, **kwargs):
        self.set_team_rows(rows)
        try:
            return plain(self, *args, **kwargs)
        finally:
            self.set_team_rows(-1)

    monkeypatch.setattr(encoders.KmerEncoder, "encode_padded", encode_padded)
    yield request.param


both_kmer_kernels = pytest.mark.parametrize("kmer_kernel_choice", ["rows_by_wave", "rows_by_workgroup"], indirect=True)


@pytest.fixture(scope="module")
def kmer_enc():
    t = kmer_tables.tables_from_vocab(hf.kmer_vocab(6), 6, 0)
    return encoders.KmerEncoder(6, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=0,
                                exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)


def rows_from_padded(ids, lengths):
    ids, lengths = ids.cpu().numpy(), lengths.cpu().numpy()
    return [ids[r, :lengths[r]] for r in range(ids.shape[0])]


@both_kmer_kernels
def test_kmer_c2(kmer_enc, kmer_kernel_choice):
    say("kmer C2 256x6000")
    b = wl.config2_kmer()
    data, off = to_dev(b)
    ids, mask, lengths, status, max_len = kmer_enc.encode_padded(data, off, 6000)
    torch.cuda.synchronize()
    rows = rows_from_padded(ids, lengths)
    util.check_against_golden("C2_kmer", rows)
    m = int(max_len.item())
    assert m == int(lengths.max().item())
    eids, emask = O.pad_rows(rows, 1, m)
    np.testing.assert_array_equal(ids[:, :m].cpu().numpy(), eids)
    np.testing.assert_array_equal(mask[:, :m].cpu().numpy(), emask)
    assert int(status.abs().sum().item()) == 0


@both_kmer_kernels
@pytest.mark.parametrize("k", [2, 3, 4, 5, 6, 7, 8])
def test_kmer_ragged_all_k(k, kmer_kernel_choice):
    say(f"kmer ragged k={k}")
    vocab = hf.kmer_vocab(k)
    t = kmer_tables.tables_from_vocab(vocab, k, 0)
    enc = encoders.KmerEncoder(k, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=0,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    ot = O.kmer_tables_from_vocab(vocab, k, 0)
    rng = np.random.default_rng(k)
    lens = rng.integers(0, 9000, size=61)
    lens[:6] = [0, 1, k - 1, k, k + 1, 5000 * k + 3]
    strings = ["".join(rng.choice(list("ACGTN"), p=[.24, .24, .24, .24, .04], size=n)) for n in lens]
    strings[7] = "N" * 3000
    strings[8] = "ACGTx" * 300
    b = util.batch_from_strings(strings)
    data, off = to_dev(b)
    t_cap = int(max(len(s) for s in strings)) + 3
    t_cap += (-t_cap) % 4
    for fill_to, cap in ((0, t_cap), (t_cap, t_cap), (0, 1000), (0, 1001)):
        ids, mask, lengths, status, max_len = enc.encode_padded(data, off, cap, fill_to=fill_to)
        torch.cuda.synchronize()
        erows, estatus = O.kmer_encode(ot, b.data, b.offsets)
        np.testing.assert_array_equal(lengths.cpu().numpy(), [r.size for r in erows])
        st = status.cpu().numpy()
        np.testing.assert_array_equal(st & 3, estatus)
        np.testing.assert_array_equal((st & 4) != 0, np.array([r.size > cap for r in erows]))
        width = fill_to if fill_to else min(cap, max(r.size for r in erows))
        assert int(max_len.item()) == min(cap, max(r.size for r in erows))
        eids, emask = O.pad_rows(erows, 1, width)
        np.testing.assert_array_equal(ids[:, :width].cpu().numpy(), eids)
        np.testing.assert_array_equal(mask[:, :width].cpu().numpy(), emask)


@both_kmer_kernels
@pytest.mark.parametrize("k", [3, 6, 8])
def test_kmer_steps_with_more_tokens_than_the_staging_area(kmer_kernel_choice, k):
    """Long stretches of N (every window of a step spelled out: up to k times 256 tokens where a
    wave stages 512) between plain stretches of every length, so that such a step is entered and
    left at every alignment, follows and precedes staged and plain steps, ends a row, and is cut
    by the row stride."""
    say(f"kmer steps beyond the staging area k={k}")
    vocab = hf.kmer_vocab(k)
    t = kmer_tables.tables_from_vocab(vocab, k, 0)
    enc = encoders.KmerEncoder(k, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=0,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    ot = O.kmer_tables_from_vocab(vocab, k, 0)
    rng = np.random.default_rng(100 + k)
    strings = []
    for r in range(96):
        parts = []
        for _ in range(rng.integers(1, 6)):
            parts.append("".join(rng.choice(list("ACGT"), size=rng.integers(0, 2500))))
            parts.append("N" * int(rng.integers(1, 4000)))
            if rng.random() < 0.3:
                parts.append("".join(rng.choice(list("ACGTN"), p=[.2, .2, .2, .2, .2], size=rng.integers(0, 900))))
        if r % 3 == 0:
            parts.append("".join(rng.choice(list("ACGT"), size=rng.integers(0, 2000))))
        strings.append("".join(parts))
    strings[5] = "N" * 20000
    strings[6] = "ACGT" * 100 + "N" * (256 * k * 3) + "ACGT" * 700
    b = util.batch_from_strings(strings)
    data, off = to_dev(b)
    erows, estatus = O.kmer_encode(ot, b.data, b.offsets)
    longest = max(r.size for r in erows)
    for cap in (longest + 5, longest // 2 + 3, 2048):
        ids, mask, lengths, status, max_len = enc.encode_padded(data, off, cap, fill_to=0)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(lengths.cpu().numpy(), [r.size for r in erows])
        st = status.cpu().numpy()
        np.testing.assert_array_equal(st & 3, estatus)
        np.testing.assert_array_equal((st & 4) != 0, np.array([r.size > cap for r in erows]))
        width = min(cap, longest)
        assert int(max_len.item()) == width
        eids, emask = O.pad_rows(erows, 1, width)
        np.testing.assert_array_equal(ids[:, :width].cpu().numpy(), eids)
        np.testing.assert_array_equal(mask[:, :width].cpu().numpy(), emask)


@pytest.mark.parametrize("k", [3, 6, 8])
def test_kmer_mostly_short_rows_with_some_long_ones(k):
    """Rows are given their kernel by their own length: in a batch of thousands of short reads with
    some rows of 2-20 kbp among them the reads get sixteen lanes each and the long rows a wave each,
    two launches over the one output (the reference groups rows by length,
    src/dna_tokenizer.py:1476-1531).  Padded (to a fixed width, to the longest with and without a
    guess) and packed, against the oracle; the packed form also for a table the 16-lane kernel does
    not serve and for batches of long rows only."""
    say(f"kmer mixed row lengths k={k}")
    vocab = hf.kmer_vocab(k)
    t = kmer_tables.tables_from_vocab(vocab, k, 0)
    enc = encoders.KmerEncoder(k, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=0,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    ot = O.kmer_tables_from_vocab(vocab, k, 0)
    rng = np.random.default_rng(60 + k)
    n_short = 6000
    lens = rng.integers(0, 301, size=n_short)
    strings = ["".join(rng.choice(list("ACGTN"), p=[.245, .245, .245, .245, .02], size=n)) for n in lens]
    for at in rng.choice(n_short, size=40, replace=False):              # the long rows, anywhere in the batch
        strings[at] = "".join(rng.choice(list("ACGTN"), p=[.248, .248, .248, .248, .008], size=int(rng.integers(2000, 20001))))
    strings[17] = "ACGTx" * 700
    strings[18] = "N" * (384 * k)                                       # exactly at the border between the classes
    strings[19] = "A" * (384 * k + 1)
    b = util.batch_from_strings(strings)
    data, off = to_dev(b)
    erows, estatus = O.kmer_encode(ot, b.data, b.offsets)
    longest = max(r.size for r in erows)
    cap = longest + (-longest) % 128
    for fill_to, guess in ((0, 0), (cap, 0), (0, longest + 3), (0, 64)):
        ids, mask, lengths, status, max_len = enc.encode_padded(data, off, cap, fill_to=fill_to, width_guess=guess)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(lengths.cpu().numpy(), [r.size for r in erows])
        np.testing.assert_array_equal(status.cpu().numpy() & 7, estatus)
        width = fill_to if fill_to else longest
        if not fill_to:
            assert int(max_len.item()) == longest
        eids, emask = O.pad_rows(erows, 1, width)
        np.testing.assert_array_equal(ids[:, :width].cpu().numpy(), eids)
        np.testing.assert_array_equal(mask[:, :width].cpu().numpy(), emask)

    def check_packed(e, bb, rows_want, status_want):
        d, o = to_dev(bb)
        for want_mask in (True, False):
            ids, out_off, mask, lengths, status = e.encode_packed(d, o, want_mask=want_mask)
            torch.cuda.synchronize()
            oo = out_off.cpu().numpy()
            np.testing.assert_array_equal(lengths.cpu().numpy(), [r.size for r in rows_want])
            np.testing.assert_array_equal(oo, np.concatenate([[0], np.cumsum([r.size for r in rows_want])]))
            np.testing.assert_array_equal(status.cpu().numpy() & 7, status_want)
            flat = ids.cpu().numpy()
            np.testing.assert_array_equal(flat[:oo[-1]], np.concatenate(rows_want) if oo[-1] else np.zeros(0, np.int32))
            if want_mask:
                assert bool((mask[:oo[-1]] == 1).all())

    check_packed(enc, b, erows, estatus)
    long_only = [s_ for s_ in strings if len(s_) > 384 * k][:20] + ["", "ACG"]
    bl = util.batch_from_strings(long_only)
    check_packed(enc, bl, *O.kmer_encode(ot, bl.data, bl.offsets))
    # a digit table that is not the plain one: a wave per row for every row, also when packed
    digit = t.digit.copy()
    digit[ord("U")] = digit[ord("T")]
    single = t.single.copy()
    single[ord("U")] = single[ord("T")]
    enc2 = encoders.KmerEncoder(k, digit, t.kmer_lut, single, pad_id=1, missing_id=0,
                                exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    sub = strings[:300] + [strings[int(i)] for i in np.argsort([-len(s_) for s_ in strings])[:5]]
    bs = util.batch_from_strings(sub)
    check_packed(enc2, bs, *O.kmer_encode(ot, bs.data, bs.offsets))


@both_kmer_kernels
def test_kmer_pad_to_longest_with_width_guess(kmer_kernel_choice):
    """fill_to = 0 with a guess of the longest row: a guess below, at or above the true width
    gives the same ids / mask / lengths / max_len inside [:, :max_len]."""
    say("kmer width guess")
    k = 6
    vocab = hf.kmer_vocab(k)
    t = kmer_tables.tables_from_vocab(vocab, k, 0)
    enc = encoders.KmerEncoder(k, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=0,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    b = wl.config2_kmer(64, 3000, seed=77, n_fraction=0.02)
    data, off = to_dev(b)
    ref = enc.encode_padded(data, off, 3008, fill_to=0)
    torch.cuda.synchronize()
    width = int(ref[4].item())
    erows, _ = O.kmer_encode(O.kmer_tables_from_vocab(vocab, k, 0), b.data, b.offsets)
    eids, emask = O.pad_rows(erows, 1, width)
    np.testing.assert_array_equal(ref[0][:, :width].cpu().numpy(), eids)
    for guess in (1, width - 37, width, width + 5, 3008, 10 ** 9):
        got = enc.encode_padded(data, off, 3008, fill_to=0, width_guess=guess)
        torch.cuda.synchronize()
        assert int(got[4].item()) == width
        np.testing.assert_array_equal(got[0][:, :width].cpu().numpy(), eids)
        np.testing.assert_array_equal(got[1][:, :width].cpu().numpy(), emask)
        np.testing.assert_array_equal(got[2].cpu().numpy(), ref[2].cpu().numpy())
        np.testing.assert_array_equal(got[3].cpu().numpy(), ref[3].cpu().numpy())


@both_kmer_kernels
def test_kmer_pad_to_longest_with_row_stride_cut_to_the_guess(kmer_enc, kmer_kernel_choice):
    """Rows only a little further apart than the guessed width (the layout a stream of batches
    uses): the workgroup-per-row kernel then pads to the stride and reports the maximum itself,
    with no padding launch.  Guesses below, at and above the true width, strides that cut rows
    off, eager calls and calls with a wide stride in between (they share the running maximum's
    slot), and a captured call replayed over changing input."""
    say("kmer tight stride")
    n, length = 48, 3000
    batches = [wl.config2_kmer(n, length, seed=s, n_fraction=f) for s, f in ((91, 0.02), (92, 0.0), (93, 0.06))]
    want = []
    for b in batches:
        data, off = to_dev(b)
        r = kmer_enc.encode_padded(data, off, 3008, fill_to=0)
        torch.cuda.synchronize()
        want.append((int(r[4].item()), r[0].cpu().numpy(), r[1].cpu().numpy(), r[2].cpu().numpy()))
    for rnd in range(2):
        for b, (width, ids, mask, lengths) in zip(batches, want):
            data, off = to_dev(b)
            for guess, t_cap in ((width - 40, width + 24), (width, width), (width + 3, width + 131), (width + 3, width + 259),
                                 (width - 100, width - 36), (8, 200)):
                got = kmer_enc.encode_padded(data, off, t_cap, fill_to=0, width_guess=guess)
                torch.cuda.synchronize()
                w = min(width, t_cap)
                assert int(got[4].item()) == w, (guess, t_cap)
                np.testing.assert_array_equal(got[0][:, :w].cpu().numpy(), ids[:, :w])
                np.testing.assert_array_equal(got[1][:, :w].cpu().numpy(), mask[:, :w])
                np.testing.assert_array_equal(got[2].cpu().numpy(), lengths)
                np.testing.assert_array_equal((got[3].cpu().numpy() & 4) != 0, lengths > t_cap)
    # every shape of the tree the maximum is gathered on: 1 .. 1024 rows, the longest row anywhere
    for n_rows in (1, 2, 3, 4, 5, 7, 16, 17, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025):
        rng = np.random.default_rng(n_rows)
        lens = rng.integers(0, 240, size=n_rows)
        lens[rng.integers(0, n_rows)] = 300 + n_rows % 7
        b = util.batch_from_strings(["".join(rng.choice(list("ACGTN"), p=[.245, .245, .245, .245, .02], size=m)) for m in lens])
        data, off = to_dev(b)
        ref = kmer_enc.encode_padded(data, off, 320, fill_to=0)
        torch.cuda.synchronize()
        width = int(ref[4].item())
        assert width == int(ref[2].max().item())
        for rep in range(2):
            got = kmer_enc.encode_padded(data, off, width + 8, fill_to=0, width_guess=width - 3 + 5 * rep)
            torch.cuda.synchronize()
            assert int(got[4].item()) == width, n_rows
            np.testing.assert_array_equal(got[0][:, :width].cpu().numpy(), ref[0][:, :width].cpu().numpy())
            np.testing.assert_array_equal(got[1][:, :width].cpu().numpy(), ref[1][:, :width].cpu().numpy())
            np.testing.assert_array_equal(got[2].cpu().numpy(), ref[2].cpu().numpy())
    # a captured call with a tight stride, replayed over the three batches
    t_cap, guess = max(w[0] for w in want) + 16, max(w[0] for w in want) - 8
    data = torch.zeros(n * length, dtype=torch.uint8, device=DEV)
    off = torch.arange(n + 1, dtype=torch.int64, device=DEV) * length
    out = (torch.empty((n, t_cap), dtype=torch.int32, device=DEV), torch.empty((n, t_cap), dtype=torch.uint8, device=DEV),
           torch.empty(n, dtype=torch.int32, device=DEV), torch.empty(n, dtype=torch.int32, device=DEV),
           torch.empty(1, dtype=torch.int32, device=DEV))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        kmer_enc.encode_padded(data, off, t_cap, fill_to=0, width_guess=guess, out=out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        kmer_enc.encode_padded(data, off, t_cap, fill_to=0, width_guess=guess, out=out)
    for i in (0, 1, 2, 1, 0, 2):
        data.copy_(torch.from_numpy(batches[i].data))
        graph.replay()
        torch.cuda.synchronize()
        width, ids, mask, lengths = want[i]
        assert int(out[4].item()) == width
        np.testing.assert_array_equal(out[0][:, :width].cpu().numpy(), ids[:, :width])
        np.testing.assert_array_equal(out[1][:, :width].cpu().numpy(), mask[:, :width])
        np.testing.assert_array_equal(out[2].cpu().numpy(), lengths)


@both_kmer_kernels
@pytest.mark.parametrize("k", [2, 3, 4, 5, 7, 8])
def test_kmer_row_stride_cut_to_the_guess_for_every_k(kmer_kernel_choice, k):
    """The one-launch form of pad-to-longest (rows as far apart as the guess) for the other window
    lengths, with and without a mask, with strides that are no multiple of four cells: the same
    ids, mask, lengths and longest row as the call with room for the worst case."""
    say(f"kmer tight stride k={k}")
    vocab = hf.kmer_vocab(k)
    t = kmer_tables.tables_from_vocab(vocab, k, 0)
    enc = encoders.KmerEncoder(k, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=0,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    rng = np.random.default_rng(200 + k)
    for n_rows in (3, 70, 1300):
        lens = rng.integers(0, 900, size=n_rows)
        b = util.batch_from_strings(["".join(rng.choice(list("ACGTN"), p=[.24, .24, .24, .24, .04], size=m)) for m in lens])
        data, off = to_dev(b)
        ref = enc.encode_padded(data, off, 904, fill_to=0)
        torch.cuda.synchronize()
        width = int(ref[4].item())
        assert width == int(ref[2].max().item())
        for t_cap, guess, want_mask in ((width + 1, width - 5, True), (width + 30, width + 2, False), (width + 255, width, True)):
            got = enc.encode_padded(data, off, t_cap, fill_to=0, width_guess=guess, want_mask=want_mask)
            torch.cuda.synchronize()
            assert int(got[4].item()) == width, (n_rows, t_cap)
            np.testing.assert_array_equal(got[0][:, :width].cpu().numpy(), ref[0][:, :width].cpu().numpy())
            if want_mask:
                np.testing.assert_array_equal(got[1][:, :width].cpu().numpy(), ref[1][:, :width].cpu().numpy())
            np.testing.assert_array_equal(got[2].cpu().numpy(), ref[2].cpu().numpy())
            np.testing.assert_array_equal(got[3].cpu().numpy(), ref[3].cpu().numpy())


@both_kmer_kernels
def test_kmer_pad_to_longest_replayed_from_a_graph(kmer_enc, kmer_kernel_choice):
    """A captured pad-to-longest call, replayed over changing input: every replay reports the
    longest row of its own input (first a batch with long rows, then shorter ones, then long
    again), and matches the eager call."""
    say("kmer graph replay")
    n, length = 32, 2400
    batches = [wl.config2_kmer(n, length, seed=5, n_fraction=0.05),
               wl.config2_kmer(n, length, seed=6, n_fraction=0.0),
               wl.config2_kmer(n, length, seed=7, n_fraction=0.01),
               wl.config2_kmer(n, length, seed=8, n_fraction=0.08)]
    data = torch.zeros(n * length, dtype=torch.uint8, device=DEV)
    off = torch.arange(n + 1, dtype=torch.int64, device=DEV) * length
    t_cap = 2432
    out = (torch.empty((n, t_cap), dtype=torch.int32, device=DEV), torch.empty((n, t_cap), dtype=torch.uint8, device=DEV),
           torch.empty(n, dtype=torch.int32, device=DEV), torch.empty(n, dtype=torch.int32, device=DEV),
           torch.empty(1, dtype=torch.int32, device=DEV))
    data.copy_(torch.from_numpy(batches[0].data))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        kmer_enc.encode_padded(data, off, t_cap, fill_to=0, out=out)        # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        kmer_enc.encode_padded(data, off, t_cap, fill_to=0, out=out)
    widths = []
    for b in batches + batches[:2]:
        data.copy_(torch.from_numpy(b.data))
        graph.replay()
        torch.cuda.synchronize()
        width = int(out[4].item())
        widths.append(width)
        got_ids, got_mask = out[0][:, :width].cpu().numpy(), out[1][:, :width].cpu().numpy()
        eager = kmer_enc.encode_padded(data, off, t_cap, fill_to=0)
        torch.cuda.synchronize()
        assert int(eager[4].item()) == width == int(out[2].max().item())
        np.testing.assert_array_equal(got_ids, eager[0][:, :width].cpu().numpy())
        np.testing.assert_array_equal(got_mask, eager[1][:, :width].cpu().numpy())
    assert widths[1] == length // 6 and widths[0] > widths[1] and widths[3] > widths[2] > widths[1]


@both_kmer_kernels
def test_kmer_pad_to_longest_calls_on_many_streams_do_not_share_a_maximum(kmer_enc, kmer_kernel_choice):
    """Pad-to-longest calls queued on several streams at once, nothing synchronised in between:
    every call reports the longest row of its own batch.  70 streams is more than the table keeps
    running maxima for, so the last ones take the path that clears the caller's max_len instead."""
    say("kmer pad-to-longest on many streams")
    n, length, t_cap = 256, 6000, 6016
    batches = [wl.config2_kmer(n, length, seed=40 + i, n_fraction=f) for i, f in enumerate((0.0, 0.05, 0.01, 0.1))]
    dev = [to_dev(b) for b in batches]
    want = []
    for data, off in dev:
        r = kmer_enc.encode_padded(data, off, t_cap, fill_to=0)
        torch.cuda.synchronize()
        want.append((int(r[4].item()), r[0].cpu().numpy(), r[2].cpu().numpy()))
    assert len({w[0] for w in want}) == len(want)
    streams = [torch.cuda.Stream() for _ in range(70)]
    torch.cuda.synchronize()
    got = []
    for rnd in range(2):
        for i, st in enumerate(streams):
            which = (i + rnd) % len(dev)
            with torch.cuda.stream(st):
                got.append((which, kmer_enc.encode_padded(dev[which][0], dev[which][1], t_cap, fill_to=0,
                                                          width_guess=length // 6 if i % 3 else 0)))
    torch.cuda.synchronize()
    for which, r in got:
        width, ids, lengths = want[which]
        assert int(r[4].item()) == width
        np.testing.assert_array_equal(r[2].cpu().numpy(), lengths)
        np.testing.assert_array_equal(r[0][:, :width].cpu().numpy(), ids[:, :width])


@both_kmer_kernels
def test_kmer_general_tables_not_spelled(kmer_kernel_choice):
    """Tables whose N windows are not spelled character by character: N windows that have an
    id of their own, expansions of other lengths, and windows with nothing at all."""
    say("kmer general (non-spelled) tables")
    k = 4
    vocab = hf.kmer_vocab(k)

    def tok(batch):
        out = []
        for s in batch:
            if len(s) == k and "N" not in s:
                out.append([vocab[s]])
            elif len(s) == k and s.count("N") == 1:
                out.append([2])                                   # one token for the whole window
            elif len(s) == k and s.count("N") == 2:
                out.append([vocab[c] for c in s if c != "N"] + [3])   # 3 tokens
            elif len(s) == k and s.count("N") == 3:
                out.append([])                                    # nothing known
            else:
                out.append([vocab.get(c, 0) for c in s])
        return out
    t = kmer_tables.tables_from_tokenize(tok, k, 0)
    enc = encoders.KmerEncoder(k, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=4,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    ot = O.KmerTables(k, t.digit, t.kmer_lut, t.exp_off, t.exp_len, t.exp_flat, t.single, 4)
    rng = np.random.default_rng(5)
    strings = ["".join(rng.choice(list("ACGTN"), p=[.2, .2, .2, .2, .2], size=n))
               for n in rng.integers(0, 5000, size=40)]
    b = util.batch_from_strings(strings)
    data, off = to_dev(b)
    ids, mask, lengths, status, max_len = enc.encode_padded(data, off, 5000)
    torch.cuda.synchronize()
    erows, estatus = O.kmer_encode(ot, b.data, b.offsets)
    np.testing.assert_array_equal(lengths.cpu().numpy(), [r.size for r in erows])
    np.testing.assert_array_equal(status.cpu().numpy() & 3, estatus)
    m = int(max_len.item())
    eids, emask = O.pad_rows(erows, 1, m)
    np.testing.assert_array_equal(ids[:, :m].cpu().numpy(), eids)
    np.testing.assert_array_equal(mask[:, :m].cpu().numpy(), emask)


@both_kmer_kernels
@pytest.mark.parametrize("k", [3, 6, 8])
@pytest.mark.parametrize("form", ["both_cases", "u_reads_as_t"])
def test_kmer_digit_tables_of_other_forms(kmer_kernel_choice, k, form):
    """The kernel that takes a row per wave finds the digits of the plain table (A C G T N in
    upper case, or in both cases) by arithmetic on the bytes and those of any other table in the
    table itself: a table that folds the case (lower-case rows, rows of mixed case, bytes that
    differ from a base in one bit only), and one with a sixth letter, against the oracle's walk
    through the same tables."""
    say(f"kmer digit table {form} k={k}")
    vocab = hf.kmer_vocab(k)
    t = kmer_tables.tables_from_vocab(vocab, k, 0)
    digit = kmer_tables.digit_table(fold_case=(form == "both_cases"))
    if form == "u_reads_as_t":
        digit[ord("U")] = 3
    single = t.single.copy()
    for ch in "acgtnU":
        single[ord(ch)] = single[ord(ch.upper() if ch != "U" else "T")]
    enc = encoders.KmerEncoder(k, digit, t.kmer_lut, single, pad_id=1, missing_id=0,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    ot = O.KmerTables(k, digit, t.kmer_lut, t.exp_off, t.exp_len, t.exp_flat, single, 0)
    rng = np.random.default_rng(100 + k)
    letters = list("ACGTNacgtnU")
    strings = ["".join(rng.choice(letters, p=[.2, .2, .2, .2, .02, .04, .04, .04, .04, .01, .01], size=n))
               for n in rng.integers(0, 7000, size=40)]
    strings += ["acgt" * 1500, "ACGTU" * 900, "".join(chr(ord(c) ^ b) for c, b in zip("ACGTN" * 600, [1, 2, 4, 8, 16, 32, 64] * 429)),
                "ACGT" * 700 + "a!c{g`t@" * 50 + "ACGT" * 700]
    b = util.batch_from_strings(strings)
    data, off = to_dev(b)
    t_cap = max(len(s) for s in strings) + 4
    t_cap += (-t_cap) % 4
    ids, mask, lengths, status, max_len = enc.encode_padded(data, off, t_cap)
    torch.cuda.synchronize()
    erows, estatus = O.kmer_encode(ot, b.data, b.offsets)
    np.testing.assert_array_equal(lengths.cpu().numpy(), [r.size for r in erows])
    np.testing.assert_array_equal(status.cpu().numpy() & 3, estatus)
    m = int(max_len.item())
    assert m == max(r.size for r in erows)
    eids, emask = O.pad_rows(erows, 1, m)
    np.testing.assert_array_equal(ids[:, :m].cpu().numpy(), eids)
    np.testing.assert_array_equal(mask[:, :m].cpu().numpy(), emask)


@pytest.mark.parametrize("k", [2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("fold", [False, True])
def test_kmer_short_rows_sixteen_lanes_each(k, fold):
    """Row strides of at most 384 cells send a batch to the kernel that gives a row sixteen lanes:
    reads of a few hundred bases with N, lower case (a table that folds the case, and one that does
    not), foreign bytes, every tail length, empty rows, rows of more than one step of 64 windows and
    rows cut by the stride; padded to a fixed width, to the longest row with a guess (one launch), and
    to the longest row without one (a padding launch follows), all against the oracle."""
    say(f"kmer short rows k={k} fold={fold}")
    vocab = hf.kmer_vocab(k)
    t = kmer_tables.tables_from_vocab(vocab, k, 0)
    digit = kmer_tables.digit_table(fold_case=fold)
    single = t.single.copy()
    for ch in "acgtn":
        single[ord(ch)] = single[ord(ch.upper())] if fold else 0
    enc = encoders.KmerEncoder(k, digit, t.kmer_lut, single, pad_id=1, missing_id=0,
                               exp_off=t.exp_off, exp_len=t.exp_len, exp_flat=t.exp_flat)
    ot = O.KmerTables(k, digit, t.kmer_lut, t.exp_off, t.exp_len, t.exp_flat, single, 0)
    rng = np.random.default_rng(40 + k)
    letters = list("ACGTNacgtx")
    p = [.22, .22, .22, .22, .03, .02, .02, .02, .02, .01]
    strings = ["".join(rng.choice(letters, p=p, size=n)) for n in rng.integers(0, 64 * k + 40, size=3000)]
    strings[:8] = ["", "A", "ACGT"[:k - 1], "ACGTACGT"[:k], "N" * (3 * k + 1), "ACGT" * 400, "x" * 50, "ACGTN" * 90]
    strings += ["".join(rng.choice(list("ACGT"), size=n)) for n in rng.integers(100, 301, size=2000)]
    b = util.batch_from_strings(strings)
    data, off = to_dev(b)
    erows, estatus = O.kmer_encode(ot, b.data, b.offsets)
    elen = np.array([r.size for r in erows])
    for cap in (64, 128, 384):
        for fill_to, guess in ((cap, 0), (0, cap - 7), (0, 0)):
            ids, mask, lengths, status, max_len = enc.encode_padded(data, off, cap, fill_to=fill_to, width_guess=guess)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(lengths.cpu().numpy(), elen)
            st = status.cpu().numpy()
            np.testing.assert_array_equal(st & 3, estatus)
            np.testing.assert_array_equal((st & 4) != 0, elen > cap)
            width = fill_to if fill_to else min(cap, int(elen.max()))
            assert int(max_len.item()) == min(cap, int(elen.max()))
            eids, emask = O.pad_rows(erows, 1, width)
            np.testing.assert_array_equal(ids[:, :width].cpu().numpy(), eids)
            np.testing.assert_array_equal(mask[:, :width].cpu().numpy(), emask)
    ids, mask, lengths, status, max_len = enc.encode_padded(data, off, 128, fill_to=128, want_mask=False)
    torch.cuda.synchronize()
    assert mask is None
    np.testing.assert_array_equal(ids.cpu().numpy(), O.pad_rows(erows, 1, 128)[0])


@both_kmer_kernels
def test_kmer_missing_windows_without_expansion(kmer_kernel_choice):
    say("kmer missing windows")
    t = kmer_tables.tables_from_vocab(hf.kmer_vocab(4), 4, 0)
    enc = encoders.KmerEncoder(4, t.digit, t.kmer_lut, t.single, pad_id=1, missing_id=3)
    b = util.batch_from_strings(["ACGTACNTACGTAC", "ACGTACGT"])
    data, off = to_dev(b)
    ids, mask, lengths, status, _ = enc.encode_padded(data, off, 16)
    torch.cuda.synchronize()
    assert lengths.tolist() == [3 + 2, 2]
    assert status.tolist() == [2, 0]
    assert ids[0, 1].item() == 3


# ------------------------------------------------------------------- BPE

@pytest.fixture(scope="module", params=["4096", "32000"])
def bpe(request):
    which = request.param
    cfg = util.tokenizer_json(which)
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    remap = kv.remap_to(cfg["model"]["vocab"], cfg["model"]["vocab"]["[UNK]"])
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv), out_remap=remap)
    return which, enc, util.bpe_oracle(which)


def bpe_rows(enc, b: wl.Batch):
    data, off = to_dev(b)
    max_len = int(b.lengths().max()) if b.n_seqs else 0
    tok, lengths = enc.encode(data, off, max_len)
    torch.cuda.synchronize()
    tok, lengths = tok.cpu().numpy(), lengths.cpu().numpy()
    return [tok[b.offsets[i]:b.offsets[i] + lengths[i]] for i in range(b.n_seqs)]


def test_bpe_small_and_edge_cases(bpe):
    which, enc, bo = bpe
    say(f"bpe{which} small cases")
    cases = util.small_cases()
    rows = bpe_rows(enc, util.batch_from_strings(cases))
    for s, r, g in zip(cases, rows, util.split_small("bpe" + which)):
        np.testing.assert_array_equal(r, g, err_msg=repr(s))


def test_bpe_random_lengths_and_homopolymers(bpe):
    which, enc, bo = bpe
    say(f"bpe{which} random lengths / homopolymers")
    random.seed(0)
    seqs = ["".join(random.choices("ACGT", k=random.choice([4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048])))
            for _ in range(256)]
    seqs += [c * n for c in "ACGTN" for n in (32, 64, 128, 256, 512, 1024, 4096)]
    seqs += ["AC" * 700, "ACG" * 500, "AAAT" * 300 + "A" * 100, "N" * 10 + "ACGT" * 100 + "NN"]
    b = util.batch_from_strings(seqs)
    rows = bpe_rows(enc, b)
    ref = bo.encode_batch(b.data, b.offsets)
    for s, r, e in zip(seqs, rows, ref):
        np.testing.assert_array_equal(r, e, err_msg=s[:40])


def test_bpe_c3_golden():
    say("bpe4096 C3 1024x1024")
    cfg = util.tokenizer_json("4096")
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv),
                              out_remap=kv.remap_to(cfg["model"]["vocab"], 0))
    util.check_against_golden("C3_bpe4096", bpe_rows(enc, wl.config3_bpe4096()))


def test_bpe_long_rows(bpe):
    which, enc, bo = bpe
    say(f"bpe{which} long rows (global-state path)")
    b = wl.config4_bpe32000(3, 20_000, seed=77)
    rows = bpe_rows(enc, b)
    for r, e in zip(rows, bo.encode_batch(b.data, b.offsets)):
        np.testing.assert_array_equal(r, e)
    # mixed short and long rows in one batch, with N
    strings = wl.config5_ragged(40, seed=9).strings() + ["A" * 9000, "ACGT" * 3000 + "N" + "TG" * 2000]
    b2 = util.batch_from_strings(strings)
    for r, e in zip(bpe_rows(enc, b2), bo.encode_batch(b2.data, b2.offsets)):
        np.testing.assert_array_equal(r, e)


BPE_LENGTH_MIXES = [
    [(1.0, 1, 300)],
    [(0.1, 0, 0), (0.5, 1, 40), (0.4, 100, 520)],
    [(1.0, 900, 1100)],
    [(0.6, 1, 600), (0.3, 600, 2100), (0.1, 2100, 9000)],
    [(0.5, 2040, 2060), (0.5, 1, 30)],
    [(0.9, 1, 3000), (0.1, 20000, 40000)],
]


@pytest.mark.parametrize("mix", range(len(BPE_LENGTH_MIXES)))
def test_bpe_random_batches_in_buffers_that_start_anywhere(bpe, mix):
    """Rows of mixed lengths (every form of the engine in one batch or another) made of corpus
    pieces, random bases, short tandem repeats and stretches with N, in a device buffer that starts
    1-7 bytes off an 8-byte boundary: the engine brings a row in by aligned 8-byte words, and the
    words at a row's two ends take a path of their own.  Token runs, the single-character ids of
    the same pass and the rows padded by the engine, against the oracle."""
    which, enc, bo = bpe
    rng = np.random.default_rng(4200 + mix)
    kinds = BPE_LENGTH_MIXES[mix]
    n_rows = [300, 400, 120, 150, 160, 24][mix]
    lens = np.array([int(rng.integers(kinds[j][1], kinds[j][2] + 1))
                     for j in rng.choice(len(kinds), size=n_rows, p=[k[0] for k in kinds])], dtype=np.int64)
    total = int(lens.sum())
    corpus = wl.bpe_corpus("4096", 1 << 18).reshape(-1)
    letters = np.frombuffer(b"ACGT", dtype=np.uint8)
    data = np.empty(total, dtype=np.uint8)
    pos = 0
    while pos < total:
        n = int(min(total - pos, rng.integers(1, 4000)))
        kind = int(rng.integers(0, 4))
        if kind == 0:
            at = int(rng.integers(0, corpus.size - n))
            data[pos:pos + n] = corpus[at:at + n]
        elif kind == 1:
            data[pos:pos + n] = letters[rng.integers(0, 4, n)]
        elif kind == 2:
            data[pos:pos + n] = np.resize(letters[rng.integers(0, 4, int(rng.integers(1, 7)))], n)
        else:
            piece = letters[rng.integers(0, 4, n)]
            piece[rng.random(n) < 0.01] = ord("N")
            data[pos:pos + n] = piece
        pos += n
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    shift = 1 + mix % 7
    say(f"bpe{which} random batch {mix}: {n_rows} rows, {total} bytes, buffer {shift} bytes off")
    buf = torch.empty(total + 16, dtype=torch.uint8, device="cuda")
    assert buf.data_ptr() % 8 == 0
    d = buf[shift:shift + total]
    d.copy_(torch.from_numpy(data))
    o = torch.from_numpy(off).cuda()
    max_len = int(lens.max())
    want = bo.encode_batch(data, off)
    lut = np.zeros(256, dtype=np.int32)
    for i, ch in enumerate("ACGTN"):
        lut[ord(ch)] = 5 + i
    tok, lengths, cids, cmask = enc.encode_with_chars(d, o, max_len, torch.from_numpy(lut).cuda())
    tok2, lengths2 = enc.encode(d, o, max_len)
    torch.cuda.synchronize()
    assert torch.equal(lengths, lengths2)
    lh = lengths.cpu().numpy()
    for t in (tok.cpu().numpy(), tok2.cpu().numpy()):
        for i in range(n_rows):
            np.testing.assert_array_equal(t[off[i]:off[i] + lh[i]], want[i], err_msg=f"row {i}")
    np.testing.assert_array_equal(cids.cpu().numpy()[:total], lut[data])
    assert bool((cmask[:total] == 1).all())
    longest = max(1, int(lh.max()))
    for pad_left in (False, True):
        stride = longest + 5
        ids, mask, pl, plong = enc.encode_padded(d, o, max_len, stride, -3, pad_left=pad_left, dtype=torch.int64)
        torch.cuda.synchronize()
        assert int(plong.item()) == int(lh.max()) and torch.equal(pl, lengths)
        ih, mh = ids.cpu().numpy(), mask.cpu().numpy()
        for i in range(n_rows):
            n = int(lh[i])
            row = np.full(stride, -3, dtype=np.int64)
            m = np.zeros(stride, dtype=np.uint8)
            if pad_left:
                row[stride - n:] = want[i]; m[stride - n:] = 1
            else:
                row[:n] = want[i]; m[:n] = 1
            np.testing.assert_array_equal(ih[i], row, err_msg=f"row {i} pad_left={pad_left}")
            np.testing.assert_array_equal(mh[i], m, err_msg=f"mask of row {i} pad_left={pad_left}")


def test_bpe_with_single_character_ids_from_the_same_pass(bpe):
    """dnatok_bpe_encode_with_chars: the tokens are those of dnatok_bpe_encode and the character ids
    are lut[byte] for every byte, on every route a row can take: short rows one per team, more rows
    than teams (the work list), rows cut into chunks (each chunk writes the characters of its
    core), rows redone by the whole-row kernel, empty rows, a mask or none; buffers start at odd
    addresses so that no store may assume more than its 4-byte alignment."""
    which, enc, bo = bpe
    say(f"bpe{which} + single-character ids in one pass")
    lut = np.zeros(256, dtype=np.int32)
    for i, ch in enumerate("ACGTN"):
        lut[ord(ch)] = 7 + i
    lut_dev = torch.from_numpy(lut).to(DEV)
    rng = random.Random(41)
    rnd = lambda n: "".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 4], k=n))
    batches = [
        [rnd(n) for n in (0, 1, 7, 8, 9, 63, 1000, 1024, 0, 333)],
        [rnd(rng.randint(0, 900)) for _ in range(3000)],
        wl.config5_ragged(300, seed=12).strings() + ["", rnd(5000), "A" * 30000, rnd(100_001), "ACGTC" * 4000],
    ]
    for seqs in batches:
        b = util.batch_from_strings(seqs)
        data, off = to_dev(b)
        max_len = int(b.lengths().max())
        total = int(b.data.size)
        for shift, want_mask in ((0, True), (3, False), (5, True)):
            # the same bytes at another alignment: outputs that start `shift` elements into their allocation
            d2 = torch.empty(total + 16, dtype=torch.uint8, device=DEV)[shift:shift + total].copy_(data)
            cids = torch.full((total + 16,), -1, dtype=torch.int32, device=DEV)[shift:shift + max(total, 1)]
            cmask = torch.zeros(total + 16, dtype=torch.uint8, device=DEV)[shift:shift + max(total, 1)] if want_mask else None
            tok, lengths, cids, cmask = enc.encode_with_chars(d2, off, max_len, lut_dev, char_ids=cids, char_mask=cmask,
                                                              want_char_mask=want_mask)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(cids[:total].cpu().numpy(), lut[b.data])
            if want_mask:
                assert bool((cmask[:total] == 1).all())
            tok, lengths = tok.cpu().numpy(), lengths.cpu().numpy()
            ref = bo.encode_batch(b.data, b.offsets)
            for i, e in enumerate(ref):
                np.testing.assert_array_equal(tok[b.offsets[i]:b.offsets[i] + lengths[i]], e, err_msg=f"row {i}")


def check_padded(enc, bo, seqs, stride, *, remap_h=None, want_mask=True, want_longest=True, pad_id=-7, out=None,
                 ref=None):
    b = util.batch_from_strings(seqs)
    data, off = to_dev(b)
    max_len = int(b.lengths().max()) if b.n_seqs else 0
    remap = None if remap_h is None else torch.from_numpy(remap_h).to(DEV)
    ids, mask, lengths, longest = enc.encode_padded(data, off, max_len, stride, pad_id, remap=remap,
                                                    want_mask=want_mask, want_longest=want_longest, out=out)
    torch.cuda.synchronize()
    ids_h, len_h = ids.cpu().numpy(), lengths.cpu().numpy()
    mask_h = mask.cpu().numpy() if mask is not None else None
    ref = bo.encode_batch(b.data, b.offsets) if ref is None else ref
    want_longest = max((len(e) for e in ref), default=0)
    assert longest is None or int(longest.item()) == want_longest
    for i, e in enumerate(ref):
        e = np.asarray(e, dtype=np.int64)
        if remap_h is not None:
            e = remap_h[e]
        assert len_h[i] == len(e), f"row {i}"
        kept = min(len(e), stride)
        np.testing.assert_array_equal(ids_h[i, :kept], e[:kept], err_msg=f"row {i}")
        assert (ids_h[i, kept:] == pad_id).all(), f"row {i}: padding"
        if mask_h is not None:
            assert (mask_h[i, :kept] == 1).all() and (mask_h[i, kept:] == 0).all(), f"row {i}: mask"
    return ref


def test_bpe_padded_in_one_pass(bpe):
    """dnatok_bpe_encode_padded: ids, mask, lengths and the longest row as dnatok_bpe_encode followed by
    dnatok_pad_rows give them, on every route: one row per team, more rows than teams (the work
    list), every LDS capacity, rows cut by a stride that is too small, empty rows and an empty
    batch, a second id map or none, a mask or none, and batches with rows long enough to be cut into
    chunks (assembled in the token buffer first)."""
    which, enc, bo = bpe
    say(f"bpe{which} padded in one pass")
    rng = random.Random(5)
    rnd = lambda n: "".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 4], k=n))
    remap_h = np.random.default_rng(3).permutation(70000).astype(np.int32)
    short = [rnd(n) for n in (0, 1, 7, 8, 9, 63, 1000, 1024, 0, 333)]
    ref = check_padded(enc, bo, short, 512)
    check_padded(enc, bo, short, 512, remap_h=remap_h, want_mask=False, ref=ref)
    check_padded(enc, bo, short, 100, ref=ref)                     # rows cut by the stride
    check_padded(enc, bo, short, 100, want_longest=False, ref=ref)  # the caller takes the longest row from the lengths
    check_padded(enc, bo, short, 1, remap_h=remap_h, ref=ref)
    check_padded(enc, bo, ["", "", ""], 16)
    none = enc.encode_padded(torch.empty(0, dtype=torch.uint8, device=DEV), torch.zeros(1, dtype=torch.int64, device=DEV),
                             0, 8, 0)
    torch.cuda.synchronize()
    assert none[0].shape == (0, 8) and int(none[3].item()) == 0
    for cap_len in (1300, 1536, 2048):                             # the other LDS capacities
        check_padded(enc, bo, [rnd(cap_len), rnd(5), "", rnd(cap_len - 7)], 640, remap_h=remap_h)
    many = [rnd(rng.randint(0, 700)) for _ in range(5000)]          # more rows than teams
    ref = check_padded(enc, bo, many, 256, remap_h=remap_h)
    check_padded(enc, bo, many, 120, ref=ref)
    check_padded(enc, bo, many, 256, want_longest=False, ref=ref)
    # several calls in a row on one stream share the tree that carries the longest row; a smaller batch after a larger one
    check_padded(enc, bo, many[:1500], 256, ref=ref[:1500])
    check_padded(enc, bo, many[:3], 256, ref=ref[:3])
    # rows that are cut into chunks, or redone by the whole-row kernel: through the token buffer
    long_rows = wl.config5_ragged(40, seed=12).strings() + ["", rnd(5000), "A" * 9000, rnd(20_001)]
    ref = check_padded(enc, bo, long_rows, 6000, remap_h=remap_h)
    check_padded(enc, bo, long_rows, 300, ref=ref)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("pad_left", [False, True])
def test_bpe_padded_in_every_layout(bpe, dtype, pad_left):
    """dnatok_bpe_encode_padded_as: the engine's launch writes the final tensor -- any id width, the
    padding on either side -- for rows it takes whole (every team shape, one row per team and a work
    list) and, through the token buffer, for rows that are cut into chunks.  Expected: the oracle's
    rows padded by the oracle's pad_rows with the same options (a row with more tokens than the
    stride keeps its first ones on either side)."""
    which, enc, bo = bpe
    say(f"bpe{which} padded as {dtype} left={pad_left}")
    rng = random.Random(17)
    rnd = lambda n: "".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 4], k=n))
    top = {torch.uint8: 200, torch.int16: 30000, torch.int32: 70000, torch.int64: 70000}[dtype]
    remap_h = np.random.default_rng(4).integers(0, top, size=70000).astype(np.int32)
    np_dtype = {torch.uint8: np.uint8, torch.int16: np.int16, torch.int32: np.int32, torch.int64: np.int64}[dtype]
    pad_id = 7
    batches = [([rnd(n) for n in (0, 1, 7, 8, 9, 63, 300, 511, 0, 333)], (160, 5)),              # one-wave teams
               ([rnd(n) for n in (1000, 1024, 0, 3, 700)], (300, 64)),                             # 256-thread teams
               ([rnd(rng.randint(0, 700)) for _ in range(3000)], (256, 100)),                      # more rows than teams
               ([rnd(rng.randint(20, 300)) for _ in range(1500)] + [rnd(900), rnd(640)], (256,)),  # split between two launches
               (wl.config5_ragged(30, seed=13).strings() + ["", rnd(5000), "A" * 9000], (4000, 250))]  # through the token buffer
    for seqs, strides in batches:
        b = util.batch_from_strings(seqs)
        data, off = to_dev(b)
        max_len = int(b.lengths().max())
        rows = [remap_h[np.asarray(e, dtype=np.int64)] for e in bo.encode_batch(b.data, b.offsets)]
        for stride in strides:
            ids, mask, lengths, longest = enc.encode_padded(data, off, max_len, stride, pad_id,
                                                            remap=torch.from_numpy(remap_h).to(DEV), pad_left=pad_left,
                                                            dtype=dtype)
            torch.cuda.synchronize()
            assert ids.dtype == dtype and tuple(ids.shape) == (len(seqs), stride)
            want_ids, want_mask = O.pad_rows(rows, pad_id, stride, pad_left=pad_left, dtype=np_dtype)
            np.testing.assert_array_equal(lengths.cpu().numpy(), [len(r) for r in rows])
            assert int(longest.item()) == max(len(r) for r in rows)
            np.testing.assert_array_equal(ids.cpu().numpy(), want_ids, err_msg=f"{len(seqs)} rows, stride {stride}")
            np.testing.assert_array_equal(mask.cpu().numpy(), want_mask, err_msg=f"{len(seqs)} rows, stride {stride}")


def test_bpe_padded_on_two_streams_and_in_a_graph(bpe):
    """Every stream has its own tree; replays of a captured call give the eager result each time,
    with eager calls (which use the same tree) in between."""
    which, enc, bo = bpe
    say(f"bpe{which} padded: streams and graph")
    rng = random.Random(9)
    rnd = lambda n: "".join(rng.choices("ACGT", k=n))
    seqs_a = [rnd(rng.randint(1, 1000)) for _ in range(700)]
    seqs_b = [rnd(rng.randint(1, 500)) for _ in range(2500)]
    s2 = torch.cuda.Stream()
    ref_a = check_padded(enc, bo, seqs_a, 300)
    with torch.cuda.stream(s2):
        ref_b = check_padded(enc, bo, seqs_b, 160)
    b = util.batch_from_strings(seqs_a)
    data, off = to_dev(b)
    max_len = int(b.lengths().max())
    out = (torch.empty((len(seqs_a), 300), dtype=torch.int32, device=DEV),
           torch.empty((len(seqs_a), 300), dtype=torch.uint8, device=DEV),
           torch.empty(len(seqs_a), dtype=torch.int32, device=DEV), torch.empty(1, dtype=torch.int32, device=DEV))
    eager = [t.clone() for t in enc.encode_padded(data, off, max_len, 300, 0, out=out)]
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        enc.encode_padded(data, off, max_len, 300, 0, out=out)       # the side stream's first call, outside the capture
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=side):
            enc.encode_padded(data, off, max_len, 300, 0, out=out)
    for _ in range(3):
        for t in out:
            t.fill_(-1 if t.dtype != torch.uint8 else 7)
        g.replay()
        torch.cuda.synchronize()
        for got, want in zip(out, eager):
            assert torch.equal(got, want)
        check_padded(enc, bo, seqs_b[:900], 160, ref=ref_b[:900])


def test_bpe_more_rows_of_about_one_length_than_teams(bpe):
    """A batch of more rows than resident teams whose rows are about equally long is dealt in the
    rows' given order, without the sorted work list: tokens as the oracle's, through the plain call
    and through the one that pads."""
    which, enc, bo = bpe
    say(f"bpe{which} rows of one length, dealt in order")
    rng = random.Random(23)
    seqs = ["".join(rng.choices("ACGT", k=rng.randint(290, 300))) for _ in range(4000)]
    b = util.batch_from_strings(seqs)
    ref = bo.encode_batch(b.data, b.offsets)
    for r, e in zip(bpe_rows(enc, b), ref):
        np.testing.assert_array_equal(r, e)
    check_padded(enc, bo, seqs, 128, ref=ref)


@pytest.mark.parametrize("longest", [250, 380, 500])
def test_bpe_many_short_rows_a_wave_each(bpe, longest):
    """Batches whose rows are at most 256 / 384 / 512 bytes long go to teams of one wave (four rows to a
    workgroup), more rows than teams through several work counters: every row as the oracle has it,
    through the plain call, the one that pads, and the one that also writes the single-character ids;
    a few rows only, empty rows, rows of one length (dealt in order) and ragged ones."""
    which, enc, bo = bpe
    say(f"bpe{which} short rows, longest {longest}")
    rng = random.Random(1000 + longest)
    rnd = lambda n: "".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 4], k=n))
    lut = np.arange(256, dtype=np.int32) + 3
    lut_dev = torch.from_numpy(lut).to(DEV)
    batches = [[rnd(rng.randint(0, longest)) for _ in range(9000)],       # so many that they are dealt unsorted
               [rnd(rng.randint(0, longest)) for _ in range(7500)],       # more than teams: the sorted work list
               [rnd(rng.randint(longest - 8, longest)) for _ in range(7000)],
               [rnd(longest), "", rnd(1), rnd(longest - 1), ""],
               [rnd(rng.randint(1, longest)) for _ in range(300)]]
    for seqs in batches:
        b = util.batch_from_strings(seqs)
        ref = bo.encode_batch(b.data, b.offsets)
        for r, e in zip(bpe_rows(enc, b), ref):
            np.testing.assert_array_equal(r, e)
        check_padded(enc, bo, seqs, 160, ref=ref)
        data, off = to_dev(b)
        tok, lengths, cids, _ = enc.encode_with_chars(data, off, int(b.lengths().max()), lut_dev, want_char_mask=False)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(cids[:b.data.size].cpu().numpy(), lut[b.data])
        tok, lengths = tok.cpu().numpy(), lengths.cpu().numpy()
        for i, e in enumerate(ref):
            np.testing.assert_array_equal(tok[b.offsets[i]:b.offsets[i] + lengths[i]], e, err_msg=f"row {i}")


@pytest.mark.parametrize("long_ones", ["up to 1 KB", "up to 2 KB", "cut into chunks"])
def test_bpe_mostly_short_rows_with_some_long_ones(bpe, long_ones):
    """A batch of mostly short rows with a few long ones among them is split between two launches (the
    shortest class of the work list to teams of one wave, the rest to 256-thread teams): every row as
    the oracle has it, through the plain call, the one that pads (whose longest row then comes from
    the lengths) and the one that also writes the single-character ids."""
    which, enc, bo = bpe
    say(f"bpe{which} mostly short rows, long ones {long_ones}")
    rng = random.Random(77)
    rnd = lambda n: "".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 4], k=n))
    seqs = [rnd(rng.randint(0, 320)) for _ in range(6000)]
    extra = {"up to 1 KB": [rnd(rng.randint(513, 1000)) for _ in range(40)],
             "up to 2 KB": [rnd(rng.randint(400, 2048)) for _ in range(60)],
             "cut into chunks": [rnd(rng.randint(400, 2048)) for _ in range(30)] + [rnd(5000), rnd(20_001), "A" * 7000]}[long_ones]
    for e in extra:
        seqs.insert(rng.randint(0, len(seqs)), e)
    b = util.batch_from_strings(seqs)
    ref = bo.encode_batch(b.data, b.offsets)
    for r, e in zip(bpe_rows(enc, b), ref):
        np.testing.assert_array_equal(r, e)
    check_padded(enc, bo, seqs, 520 if long_ones != "cut into chunks" else 6000, ref=ref)
    check_padded(enc, bo, seqs, 96, want_longest=False, ref=ref)
    lut = np.arange(256, dtype=np.int32) + 3
    data, off = to_dev(b)
    tok, lengths, cids, _ = enc.encode_with_chars(data, off, int(b.lengths().max()), torch.from_numpy(lut).to(DEV),
                                                  want_char_mask=False)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(cids[:b.data.size].cpu().numpy(), lut[b.data])
    tok, lengths = tok.cpu().numpy(), lengths.cpu().numpy()
    for i, e in enumerate(ref):
        np.testing.assert_array_equal(tok[b.offsets[i]:b.offsets[i] + lengths[i]], e, err_msg=f"row {i}")


def test_bpe_work_list_of_many_rows_built_tile_by_tile(bpe):
    """Above 8,192 rows the work list is built by two launches with a workgroup per tile of 4,096
    rows (sums, then placement) instead of by one workgroup: 21,000 ragged rows of all classes,
    long rows that are cut into chunks (one of them a homopolymer), empty rows, a last tile that is
    not full."""
    which, enc, bo = bpe
    say(f"bpe{which} work list of 21,000 rows")
    rng = random.Random(91)
    rnd = lambda n: "".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 4], k=n))
    seqs = [rnd(rng.choice([0, 1, 40, 200, 300, 520, 700, 1030, 1500, 2048])) for _ in range(21_000)]
    for e in [rnd(2049), rnd(5000), rnd(20_001), "A" * 7000, rnd(3000)] + [rnd(rng.randint(2049, 9000)) for _ in range(25)]:
        seqs.insert(rng.randint(0, len(seqs)), e)
    b = util.batch_from_strings(seqs)
    ref = bo.encode_batch(b.data, b.offsets)
    for i, (r, e) in enumerate(zip(bpe_rows(enc, b), ref)):
        np.testing.assert_array_equal(r, e, err_msg=f"row {i} of {len(seqs[i])} bytes")


def test_bpe_rows_without_a_seam_fall_back_to_the_whole_row_kernel(bpe):
    """Tandem repeats far longer than the chunk overlap: neighbouring chunk runs can stay out
    of phase, no seam is accepted, and the row is redone by the whole-row kernel."""
    which, enc, bo = bpe
    say(f"bpe{which} seam fallback")
    seqs = ["A" * 30000, "ACGTC" * 5000, "AC" * 4000 + "ACGTTGCA" * 2500,
            wl.config4_bpe32000(1, 9000, seed=3).strings()[0]]
    b = util.batch_from_strings(seqs)
    for s, r, e in zip(seqs, bpe_rows(enc, b), bo.encode_batch(b.data, b.offsets)):
        np.testing.assert_array_equal(r, e, err_msg=s[:20])


def test_bpe_long_runs_of_equal_pairs(bpe):
    """Rows in which every pair has the rank of its neighbour for thousands of positions (a
    homopolymer, a tandem repeat after its first merges): the left chain of a candidate would be
    as long as the run, so such rounds decide by a scan over the positions instead of walking.
    100 kbp rows go through chunks, seams and, where no seam is accepted, the whole-row kernel."""
    which, enc, bo = bpe
    say(f"bpe{which} long runs of equal pairs")
    rng = random.Random(17)
    rnd = lambda n: "".join(rng.choices("ACGT", k=n))
    seqs = ["A" * 100_000, "AC" * 50_000, "AAAT" * 25_000,
            rnd(3000) + "A" * 2000 + rnd(3000),                   # a 2 kbp run inside random sequence
            rnd(500) + "T" * 700 + rnd(100) + "GA" * 400 + rnd(200),
            "A" * 25, "A" * 26, "C" * 49, "AC" * 25, "A" * 23 + "C" + "A" * 30, "G" * 2047, "G" * 2048]
    b = util.batch_from_strings(seqs)
    for s, r, e in zip(seqs, bpe_rows(enc, b), bo.encode_batch(b.data, b.offsets)):
        np.testing.assert_array_equal(r, e, err_msg=f"{s[:24]}... ({len(s)} bp)")


@pytest.mark.parametrize("core,overlap", [(256, 32), (512, 96), (300, 35), (700, 160)])
def test_bpe_small_chunks_many_seams_and_fallbacks(bpe, core, overlap):
    """The chunk / seam / gather / whole-row-fallback machinery with chunks far smaller than the
    shipped ones: a few thousand ragged, random and tandem-repeat rows per vocabulary go through tens
    of thousands of seams, many of which find no position and send their row to the whole-row
    kernel.  Every row is compared with the oracle.  (300, 35): a chunk of 370 symbols is no whole
    number of 16-byte loads, which takes the gather's general form instead of the one that holds
    a whole chunk per wave; (700, 160): a shared stretch of more than 256 positions, which takes the
    seam search that walks from token start to token start instead of the one on ballots.)"""
    which, enc, bo = bpe
    say(f"bpe{which} chunks of {core} + 2 x {overlap}")
    ext = core + 2 * overlap
    enc.set_chunk_geometry(core, overlap)
    try:
        rng = random.Random(int(which) + core)
        n_rows = n_chunked = n_failed = 0
        for trial in range(5):
            strings = wl.config5_ragged(300, seed=100 + trial).strings()
            strings += ["".join(rng.choice("ACGT") for _ in range(rng.randint(1, 6000))) for _ in range(100)]
            strings += [rng.choice(["A", "AC", "ACG", "AATT", "ACGTC"]) * rng.randint(1, 900) +
                        "".join(rng.choice("ACGTN") for _ in range(rng.randint(0, 3000))) for _ in range(30)]
            rng.shuffle(strings)
            b = util.batch_from_strings(strings)
            rows = bpe_rows(enc, b)
            # the plan's counters sit at the start of the scratch buffer: [1] chunk items, [3] rows redone whole
            counts = enc._scratch[:16].view(torch.int32).cpu().numpy()
            assert counts[1] > 0
            n_failed += int(counts[3])
            n_chunked += int((b.lengths() > ext).sum())
            n_rows += b.n_seqs
            for i, (r, e) in enumerate(zip(rows, bo.encode_batch(b.data, b.offsets))):
                np.testing.assert_array_equal(r, e, err_msg=f"trial {trial} row {i} len {len(strings[i])}")
        say(f"  {n_rows} rows, {n_chunked} chunked, {n_failed} redone by the whole-row kernel")
        assert n_rows >= 2000 and 0 < n_failed < n_chunked       # seams accepted and seams refused
    finally:
        enc.set_chunk_geometry(0, 0)


def test_bpe_compact_table_in_lds_gives_the_same_tokens():
    """The 4096 vocabulary has a compact form that workgroups keep in LDS for batches of short rows
    that leave the room (not the default: it measured slower).  Same tokens as with the table in
    global memory and as the oracle: a batch small enough for one row per resident workgroup, and the C3
    batch with the compact form forced."""
    from dnatok_amd import _lib
    say("bpe4096 compact table in LDS")
    cfg = util.tokenizer_json("4096")
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv), out_remap=kv.remap_to(cfg["model"]["vocab"], 0))
    bo = util.bpe_oracle("4096")
    rng = random.Random(5)
    seqs = ["".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 1], k=rng.choice([1, 2, 7, 64, 500, 1000, 1023, 1024])))
            for _ in range(300)] + ["A" * 1024, "AC" * 512, ""]
    small = util.batch_from_strings(seqs)
    want = [np.asarray(r) for r in bo.encode_batch(small.data, small.offsets)]
    # many mostly short rows with some of 600-1000 bytes among them: the batch is split between two
    # launches that share a work list, which the compact form (one launch, no list) must stay out of
    rng2 = random.Random(6)
    split_seqs = ["".join(rng2.choice("ACGT") for _ in range(rng2.randint(20, 300))) for _ in range(1500)]
    for at in range(0, 1500, 60):
        split_seqs[at] = "".join(rng2.choice("ACGT") for _ in range(rng2.randint(600, 1000)))
    split = util.batch_from_strings(split_seqs)
    want_split = [np.asarray(r) for r in bo.encode_batch(split.data, split.offsets)]
    try:
        for mode in (0, 1, 2):
            enc.set_table_placement(mode)
            for s, r, e in zip(seqs, bpe_rows(enc, small), want):
                np.testing.assert_array_equal(r, e, err_msg=f"mode {mode}: {s[:20]}")
            util.check_against_golden("C3_bpe4096", bpe_rows(enc, wl.config3_bpe4096()))
            for i, (r, e) in enumerate(zip(bpe_rows(enc, split), want_split)):
                np.testing.assert_array_equal(r, e, err_msg=f"mode {mode}: split batch row {i}")
        with pytest.raises(_lib.DnatokError):
            enc.set_table_placement(3)
    finally:
        enc.set_table_placement(0)


def test_bpe_c4_golden():
    say("bpe32000 C4 32x100k")
    cfg = util.tokenizer_json("32000")
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv),
                              out_remap=kv.remap_to(cfg["model"]["vocab"], 0))
    util.check_against_golden("C4_bpe32000", bpe_rows(enc, wl.config4_bpe32000()))


def test_bpe_nonmonotone_random_tables():
    """Random small merge tables, including ones where two rules give the same string."""
    say("bpe random tables")
    rng = random.Random(11)
    for trial in range(40):
        alpha = "ACGT"[:rng.choice([2, 3, 4])]
        toks, merges, seen, strings = list(alpha), [], set(), set(alpha)
        for _ in range(rng.randint(1, 50)):
            a, b2 = rng.choice(toks), rng.choice(toks)
            if (a, b2) in seen or len(a + b2) > 10:
                continue
            seen.add((a, b2))
            merges.append((a, b2))
            if a + b2 not in strings:
                strings.add(a + b2)
                toks.append(a + b2)
        kv = bpe_vocab.KernelVocab(merges)
        enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
        bo = O.BpeOracle(merges)
        seqs = ["".join(rng.choice(alpha) for _ in range(rng.randint(1, 300))) for _ in range(30)]
        seqs += [rng.choice(alpha) * rng.randint(1, 200) for _ in range(6)]
        b = util.batch_from_strings(seqs)
        for s, r, e in zip(seqs, bpe_rows(enc, b), bo.encode_batch(b.data, b.offsets, remap=False)):
            np.testing.assert_array_equal(r, e, err_msg=f"trial {trial} {s} {merges}")


@pytest.mark.parametrize("letters, ruled", [(12, 12), (9, 6), (8, 8), (20, 3)])
def test_bpe_tables_over_larger_alphabets(letters, ruled):
    """The first pair of a position comes from a table by byte class when at most 8 bytes take part in
    rules between single bytes, and from the general table otherwise; bytes that take part in no such
    rule have no class.  Alphabets of `letters` bytes of which `ruled` occur in rules between single
    bytes: more than 8 (no class table), exactly 8, and fewer with classless bytes among the input;
    rows up to 5,000 bytes, so that whole rows, chunks and one-wave teams all meet them."""
    say(f"bpe alphabets: {letters} letters, {ruled} in rules between single bytes")
    rng = random.Random(100 * letters + ruled)
    alpha = "ACGTNRYKMSWBDHVacgt"[:letters] if letters <= 19 else "ACGTNRYKMSWBDHVacgtn"
    for trial in range(6):
        base = list(alpha[:ruled])
        toks, merges, seen = list(base), [], set()
        while len(merges) < rng.randint(20, 120):
            a, b2 = rng.choice(toks), rng.choice(toks)
            if (a, b2) in seen or len(a + b2) > 8:
                continue
            seen.add((a, b2))
            merges.append((a, b2))
            if a + b2 not in toks:
                toks.append(a + b2)
        # rules of a longer token with a letter that pairs with no single byte: the letter has a symbol, no class
        for c in alpha[ruled:]:
            long_toks = [t for t in toks if len(t) > 1]
            if long_toks:
                t = rng.choice(long_toks)
                if (t, c) not in seen and len(t + c) <= 9:
                    seen.add((t, c))
                    merges.append((t, c))
        # monotone: a rule's product is only used by later rules (rows may then be cut into chunks)
        kv = bpe_vocab.KernelVocab(merges)
        enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
        bo = O.BpeOracle(merges)
        seqs = ["".join(rng.choice(alpha) for _ in range(rng.choice([1, 2, 63, 200, 400, 900, 1024, 1500, 2048, 3000, 5000])))
                for _ in range(40)]
        seqs += ["".join(rng.choice(alpha[:max(ruled, 1)]) for _ in range(700)), alpha * 30]
        b = util.batch_from_strings(seqs)
        for s2, r, e in zip(seqs, bpe_rows(enc, b), bo.encode_batch(b.data, b.offsets, remap=False)):
            np.testing.assert_array_equal(r, e, err_msg=f"trial {trial} {s2[:40]}")
        short = util.batch_from_strings([q[:300] for q in seqs] * 40)          # teams of one wave
        for s2, r, e in zip(seqs * 40, bpe_rows(enc, short), bo.encode_batch(short.data, short.offsets, remap=False)):
            np.testing.assert_array_equal(r, e, err_msg=f"short, trial {trial} {s2[:40]}")


def test_bpe_nonmonotone_tables_with_rows_above_the_lds_capacity():
    """Tables with two rules for one string are not chunked: rows above 2048 bytes go to the whole-row
    kernel (state in global memory), including its rounds that merge a single pair."""
    say("bpe non-monotone tables, long rows")
    rng = random.Random(29)
    n_nonmonotone = 0
    for trial in range(6):
        # "ACG" is made by two rules, and used (rank 3) before the second of them (rank 4)
        merges = [("A", "C"), ("C", "G"), ("AC", "G"), ("ACG", "T"), ("A", "CG")]
        toks, seen = list("ACGT") + ["AC", "CG", "ACG", "ACGT"], set(merges)
        for _ in range(rng.randint(20, 80)):
            a, b2 = rng.choice(toks), rng.choice(toks)
            if (a, b2) in seen or len(a + b2) > 10:
                continue
            seen.add((a, b2))
            merges.append((a, b2))
            if a + b2 not in toks:
                toks.append(a + b2)
        strings = [a + b2 for a, b2 in merges]
        n_nonmonotone += len(set(strings)) < len(strings)
        kv = bpe_vocab.KernelVocab(merges)
        enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
        bo = O.BpeOracle(merges)
        seqs = ["".join(rng.choice("ACGT") for _ in range(n)) for n in (2049, 3000, 5000, 700, 1)]
        seqs.append("AC" * 1500 + "".join(rng.choice("ACGT") for _ in range(500)))
        b = util.batch_from_strings(seqs)
        for s, r, e in zip(seqs, bpe_rows(enc, b), bo.encode_batch(b.data, b.offsets, remap=False)):
            np.testing.assert_array_equal(r, e, err_msg=f"trial {trial} len {len(s)} {merges}")
        # the same rows with the single-character ids asked for: rows left to the whole-row kernel get theirs too
        data, off = to_dev(b)
        lut = (np.arange(256, dtype=np.int32) * 3 + 1)
        tok, lengths, cids, cmask = enc.encode_with_chars(data, off, int(b.lengths().max()), torch.from_numpy(lut).to(DEV))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(cids.cpu().numpy(), lut[b.data])
        assert bool((cmask == 1).all())
        tok, lengths = tok.cpu().numpy(), lengths.cpu().numpy()
        for i, e in enumerate(bo.encode_batch(b.data, b.offsets, remap=False)):
            np.testing.assert_array_equal(tok[b.offsets[i]:b.offsets[i] + lengths[i]], e)
    assert n_nonmonotone == 6


def test_bpe_encode_and_pad_replayed_from_a_graph(bpe):
    """The engine (work list, chunked rows, seams, gather) and the padder captured once and replayed
    over changing bytes of the same shape: every replay matches the oracle, i.e. nothing a call
    leaves behind in the scratch buffer (counters, lists, flags) leaks into the next."""
    which, enc, bo = bpe
    say(f"bpe{which} graph replay")
    lens = [5000, 300, 2048, 2049, 1, 9000, 700, 1500]
    off_h = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    total, n = int(off_h[-1]), len(lens)

    def batch(seed):
        rng = np.random.default_rng(seed)
        d = np.frombuffer(b"ACGT", dtype=np.uint8)[rng.integers(0, 4, size=total)].copy()
        if seed % 2:                                  # a tandem repeat across a chunk border of row 0
            d[1500:2300] = np.frombuffer(b"AC" * 400, dtype=np.uint8)
        return d

    data = torch.from_numpy(batch(0)).to(DEV)
    off = torch.from_numpy(off_h).to(DEV)
    t_cap = max(lens)
    tok_tmp = torch.empty(total, dtype=torch.int32, device=DEV)
    lengths = torch.empty(n, dtype=torch.int32, device=DEV)
    out = (torch.empty((n, t_cap), dtype=torch.int32, device=DEV), torch.empty((n, t_cap), dtype=torch.uint8, device=DEV),
           torch.empty(1, dtype=torch.int32, device=DEV))

    def call():
        enc.encode(data, off, t_cap, tok_tmp=tok_tmp, lengths=lengths)
        encoders.pad_rows(tok_tmp, off, lengths, 0, t_cap, fill_to=0, out=out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()                                        # warm-up outside the capture (scratch, attributes)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for seed in (1, 2, 3, 1):
        host = batch(seed)
        data.copy_(torch.from_numpy(host))
        graph.replay()
        torch.cuda.synchronize()
        ref = bo.encode_batch(host, off_h)
        width = int(out[2].item())
        assert width == max(len(r) for r in ref)
        ids, mask, ln = out[0].cpu().numpy(), out[1].cpu().numpy(), lengths.cpu().numpy()
        for i, r in enumerate(ref):
            assert ln[i] == len(r)
            np.testing.assert_array_equal(ids[i, :len(r)], r, err_msg=f"seed {seed} row {i}")
            assert (ids[i, len(r):width] == 0).all() and mask[i, :len(r)].all() and not mask[i, len(r):width].any()


def test_bpe_repeated_pair_takes_its_last_entry():
    """A pair listed twice counts with its later rank, as in the HF library (the oracle's rule is
    pinned against the library by tests/test_oracle.py); known case first, then random lists."""
    say("bpe tables with repeated pairs")
    from tests.test_oracle import random_merge_list
    known = [("A", "C"), ("C", "G"), ("A", "C")]
    kv = bpe_vocab.KernelVocab(known)
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
    (row,) = bpe_rows(enc, util.batch_from_strings(["ACG"]))
    assert [kv.id_to_token[i] for i in row] == ["A", "CG"]
    rng = random.Random(5)
    for trial in range(25):
        merges = random_merge_list(rng, rng.randint(3, 40), duplicates=rng.randint(1, 6))
        kv = bpe_vocab.KernelVocab(merges)
        enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
        bo = O.BpeOracle(merges)
        seqs = ["".join(rng.choice("ACGT") for _ in range(rng.randint(1, 400))) for _ in range(30)]
        seqs.append("".join(rng.choice("ACGT") for _ in range(5000)))        # chunked or whole-row path
        b = util.batch_from_strings(seqs)
        for sq, r, e in zip(seqs, bpe_rows(enc, b), bo.encode_batch(b.data, b.offsets, remap=False)):
            np.testing.assert_array_equal(r, e, err_msg=f"trial {trial} {sq[:60]} {merges}")


def test_bpe_table_near_the_size_limit():
    """60,000 rules (the 16-bit state allows 65,534): the hashed rule table at its largest."""
    say("bpe table with 60,000 rules")
    rng = random.Random(23)
    short, merges, seen = list("ACGT"), [], set()          # tokens of at most 7 letters
    while len(merges) < 60000:
        a, b2 = rng.choice(short), rng.choice(short)
        if (a, b2) in seen:
            continue
        seen.add((a, b2))
        merges.append((a, b2))
        if len(a + b2) <= 7:
            short.append(a + b2)
    kv = bpe_vocab.KernelVocab(merges)
    assert len(kv) <= 65535
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
    bo = O.BpeOracle(merges)
    seqs = ["".join(rng.choice("ACGT") for _ in range(rng.randint(1, 1500))) for _ in range(96)]
    b = util.batch_from_strings(seqs)
    for s, r, e in zip(seqs, bpe_rows(enc, b), bo.encode_batch(b.data, b.offsets, remap=False)):
        np.testing.assert_array_equal(r, e, err_msg=s[:40])


# ---------------------------------------------------------------- packer

def test_c5_ragged_bpe_and_char_packed(char_enc):
    say("C5 ragged: BPE-4096 + char, packed on device")
    cfg = util.tokenizer_json("4096")
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))        # kernel ids out
    remap = torch.from_numpy(kv.remap_to(cfg["model"]["vocab"], 0)).to(DEV)
    b = wl.config5_ragged()
    data, off = to_dev(b)
    tok, lengths = enc.encode(data, off, int(b.lengths().max()))
    ids, out_off, mask = encoders.pack_ragged(tok, off, lengths, remap=remap)
    cids, _ = char_enc.encode_packed(data)
    torch.cuda.synchronize()
    oo = out_off.cpu().numpy()
    flat = ids.cpu().numpy()
    rows = [flat[oo[i]:oo[i + 1]] for i in range(b.n_seqs)]
    util.check_against_golden("C5_bpe4096", rows)
    assert bool((mask[:oo[-1]] == 1).all())
    cf = cids.cpu().numpy()
    util.check_against_golden("C5_char", [cf[b.offsets[i]:b.offsets[i + 1]] for i in range(b.n_seqs)])


def test_pad_rows_matches_reference_semantics():
    say("pad_rows")
    cfg = util.tokenizer_json("4096")
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
    remap_h = kv.remap_to(cfg["model"]["vocab"], 0)
    remap = torch.from_numpy(remap_h).to(DEV)
    b = wl.config5_ragged(50, seed=3)
    data, off = to_dev(b)
    tok, lengths = enc.encode(data, off, int(b.lengths().max()))
    erows = util.bpe_oracle("4096").encode_batch(b.data, b.offsets)
    cap = max(r.size for r in erows) + 5
    for fill_to in (0, cap):
        ids, mask, max_len = encoders.pad_rows(tok, off, lengths, 3, cap, fill_to=fill_to, remap=remap)
        torch.cuda.synchronize()
        width = fill_to or int(max_len.item())
        assert int(max_len.item()) == max(r.size for r in erows)
        eids, emask = O.pad_rows(erows, 3, width)
        np.testing.assert_array_equal(ids[:, :width].cpu().numpy(), eids)
        np.testing.assert_array_equal(mask[:, :width].cpu().numpy(), emask)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("pad_left", [False, True])
def test_pad_rows_side_width_multiple_and_id_type(dtype, pad_left):
    """dnatok_pad_rows_as against the oracle's padding rules (pinned by hand-written cases): ragged token
    runs, empty rows, a least width above and below the longest row, multiples, a fixed width that cuts
    rows, and both the small-batch and the large-batch form of the kernel."""
    say(f"pad_rows_as {dtype} left={pad_left}")
    rng = np.random.default_rng(17)
    hi = 200 if dtype == torch.uint8 else 30000
    np_dtype = {torch.uint8: np.uint8, torch.int16: np.int16, torch.int32: np.int32, torch.int64: np.int64}[dtype]
    for n_rows in (1, 37, 2500):
        lens = rng.integers(0, 300, size=n_rows)
        lens[0] = 0
        rows = [rng.integers(0, hi, size=n, dtype=np.int32) for n in lens]
        room = lens + rng.integers(0, 5, size=n_rows)               # runs lie apart in the source buffer
        off_h = np.concatenate([[0], np.cumsum(room)]).astype(np.int64)
        flat = np.full(int(off_h[-1]) + 1, -1, dtype=np.int32)
        for r, o in zip(rows, off_h):
            flat[o:o + r.size] = r
        remap_h = rng.permutation(hi).astype(np.int32)
        tok, off = torch.from_numpy(flat).to(DEV), torch.from_numpy(off_h).to(DEV)
        lengths = torch.from_numpy(lens.astype(np.int32)).to(DEV)
        remap = torch.from_numpy(remap_h).to(DEV)
        longest = int(lens.max())
        for fill_to, min_width, mult in ((0, 0, 1), (0, longest + 13, 1), (0, 5, 16), (0, 0, 64), (longest // 2 + 1, 0, 1),
                                         (longest + 7, 0, 8)):
            t_cap = max(longest, fill_to, min_width) + 70
            ids, mask, stats = encoders.pad_rows_as(tok, off, lengths, 3, t_cap, fill_to=fill_to, min_width=min_width,
                                                    pad_multiple=mult, pad_left=pad_left, dtype=dtype, remap=remap)
            torch.cuda.synchronize()
            got_longest, width = stats.cpu().tolist()
            assert got_longest == longest
            want_rows = [remap_h[r] for r in rows]
            e_ids, e_mask = O.pad_rows(want_rows, 3, fill_to if fill_to else None, pad_left=pad_left, min_width=min_width,
                                       pad_multiple=mult, dtype=np_dtype)
            if fill_to and not pad_left:
                # right padding writes a row longer than the fixed width in full; compare the width's columns
                e_ids, e_mask = e_ids[:, :width], e_mask[:, :width]
            assert width == e_ids.shape[1], (n_rows, fill_to, min_width, mult, width, e_ids.shape)
            np.testing.assert_array_equal(ids[:, :width].cpu().numpy(), e_ids)
            np.testing.assert_array_equal(mask[:, :width].cpu().numpy(), e_mask)
