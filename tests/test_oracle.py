"""Pins the CPU oracle: against the committed golden vectors (written by the Hugging Face
`tokenizers` library), against the live HF library when it is importable, against closed
forms, and heap form vs. the textbook O(n^2) form of BPE."""
import random

import numpy as np
import pytest

from tests.support import hf_tokenizers as hf
from tests.support import workloads as wl
from oracle import oracle as O
from tests import util


def hf_rows(tk, strings):
    return [np.asarray(e.ids, dtype=np.int32) for e in tk.encode_batch(strings, add_special_tokens=False)]


# ------------------------------------------------------------------ char

def test_char_closed_form_and_golden():
    b = wl.config1_char()
    lut = util.char_lut()
    ids, mask = O.char_encode_padded(lut, b.data, b.offsets, 8192, pad_id=1)
    # closed form: ids = lut[byte]
    np.testing.assert_array_equal(ids, lut[b.data].reshape(64, 8192))
    assert mask.all()
    util.check_against_golden("C1_char", list(ids))
    np.testing.assert_array_equal(O.char_encode_packed(lut, b.data), ids.reshape(-1))


def test_char_ragged_padding_sides_and_start_table():
    strings = ["ACGT", "", "NNA", "ACGTACGTAC"]
    b = util.batch_from_strings(strings)
    lut = util.char_lut()
    start = lut + 100
    ids, mask = O.char_encode_padded(lut, b.data, b.offsets, 6, pad_id=1, start_lut=start)
    exp = np.full((4, 6), 1, np.int32)
    expm = np.zeros((4, 6), np.uint8)
    for r, s in enumerate(strings):
        row = [lut[ord(c)] for c in s][:6]
        if row:
            row[0] += 100
        exp[r, :len(row)] = row
        expm[r, :len(row)] = 1
    np.testing.assert_array_equal(ids, exp)
    np.testing.assert_array_equal(mask, expm)
    ids_l, mask_l = O.char_encode_padded(lut, b.data, b.offsets, 6, pad_id=1, pad_left=True)
    for r, s in enumerate(strings):
        n = min(len(s), 6)
        np.testing.assert_array_equal(ids_l[r, 6 - n:], [lut[ord(c)] for c in s[:n]])
        assert (ids_l[r, :6 - n] == 1).all() and mask_l[r].sum() == n


def test_char_matches_hf_live():
    tk = hf.build_char_tokenizer()
    b = wl.config1_char(8, 1000, seed=5)
    rows = hf_rows(tk, b.strings())
    ids, _ = O.char_encode_padded(util.char_lut(), b.data, b.offsets, 1000, pad_id=1)
    for r in range(8):
        np.testing.assert_array_equal(ids[r], rows[r])


# ----------------------------------------------------------------- k-mer

def test_kmer_golden_and_brute_force():
    t = util.kmer_oracle_tables()
    b = wl.config2_kmer()
    rows, status = O.kmer_encode(t, b.data, b.offsets)
    assert (status == 0).all()
    util.check_against_golden("C2_kmer", rows)
    # brute force over every ACGT 6-mer: id = 5 + base-4 value
    vocab = hf.kmer_vocab(6)
    import itertools
    allk = ["".join(p) for p in itertools.product("ACGT", repeat=6)]
    bb = util.batch_from_strings(["".join(allk)])
    got, _ = O.kmer_encode(t, bb.data, bb.offsets)
    np.testing.assert_array_equal(got[0], np.arange(5, 5 + 4096))
    assert [vocab[k] for k in allk] == list(range(5, 5 + 4096))


def test_kmer_small_cases_and_hf_live():
    t = util.kmer_oracle_tables()
    cases = [c for c in util.small_cases()]
    b = util.batch_from_strings([c.upper().replace("X", "N") for c in cases])
    rows, _ = O.kmer_encode(t, b.data, b.offsets)
    tk = hf.build_kmer_tokenizer(6)
    ref = hf_rows(tk, b.strings())
    for r, e in zip(rows, ref):
        np.testing.assert_array_equal(r, e)
    # golden small cases were written from the raw strings; compare those without lower case / X
    gold = util.split_small("kmer")
    for c, g, r in zip(cases, gold, rows):
        if c == c.upper() and "X" not in c:
            np.testing.assert_array_equal(r, g)


def test_kmer_status_bits():
    t = util.kmer_oracle_tables()
    b = util.batch_from_strings(["ACGTAxACGTAC"])
    rows, status = O.kmer_encode(t, b.data, b.offsets)
    assert status[0] == 1                      # byte outside the alphabet, encoded as N
    assert rows[0].size == 6 + 1


def test_kmer_encode_batch_equals_rows_plus_padding():
    """The one-call batch form (the benchmark's CPU leg) against the per-row form + pad_rows, on
    the C2 golden batch, on ragged rows, and with a stride that cuts the longest rows."""
    t = util.kmer_oracle_tables()
    b = wl.config2_kmer()
    rows, _ = O.kmer_encode(t, b.data, b.offsets)
    t_max = max(r.size for r in rows)
    ids, mask, lengths = O.kmer_encode_batch(t, b.data, b.offsets, t_max, pad_id=1)
    util.check_against_golden("C2_kmer", [ids[r, :lengths[r]] for r in range(len(rows))])
    e_ids, e_mask = O.pad_rows(rows, 1, t_max)
    np.testing.assert_array_equal(ids, e_ids)
    np.testing.assert_array_equal(mask, e_mask)
    np.testing.assert_array_equal(lengths, [r.size for r in rows])
    strings = ["", "A", "ACGTAC", "ACGTACN", "NNNNNNNNNNNNACGTACGTAC", "ACGTAC" * 40 + "NACG", "ACGTA"]
    rb = util.batch_from_strings(strings)
    rrows, _ = O.kmer_encode(t, rb.data, rb.offsets)
    for t_cap in (max(r.size for r in rrows), 9, 1):
        ids, mask, lengths = O.kmer_encode_batch(t, rb.data, rb.offsets, t_cap, pad_id=7)
        e_ids, e_mask = O.pad_rows(rrows, 7, t_cap)
        np.testing.assert_array_equal(ids, e_ids)
        np.testing.assert_array_equal(mask, e_mask)
        np.testing.assert_array_equal(lengths, [r.size for r in rrows])     # the full count, also when cut
    # hand-written expectation: "ACGTACN" = one window + the tail character N
    v = hf.kmer_vocab(6)
    ids, mask, lengths = O.kmer_encode_batch(t, rb.data, rb.offsets, 4, pad_id=7)
    np.testing.assert_array_equal(ids[3], [v["ACGTAC"], v["N"], 7, 7])
    np.testing.assert_array_equal(mask[3], [1, 1, 0, 0])


def test_pad_rows_sides_width_and_multiple_by_hand():
    """The padding rules of DNATok (side, token_len as a least width, a multiple) on cases written
    out by hand."""
    rows = [np.array([5, 6, 7], np.int32), np.array([], np.int32), np.array([9], np.int32)]
    ids, mask = O.pad_rows(rows, 0)
    np.testing.assert_array_equal(ids, [[5, 6, 7], [0, 0, 0], [9, 0, 0]])
    np.testing.assert_array_equal(mask, [[1, 1, 1], [0, 0, 0], [1, 0, 0]])
    ids, mask = O.pad_rows(rows, 0, pad_left=True)
    np.testing.assert_array_equal(ids, [[5, 6, 7], [0, 0, 0], [0, 0, 9]])
    np.testing.assert_array_equal(mask, [[1, 1, 1], [0, 0, 0], [0, 0, 1]])
    ids, mask = O.pad_rows(rows, 2, pad_left=True, min_width=5)
    np.testing.assert_array_equal(ids, [[2, 2, 5, 6, 7], [2, 2, 2, 2, 2], [2, 2, 2, 2, 9]])
    np.testing.assert_array_equal(mask, [[0, 0, 1, 1, 1], [0, 0, 0, 0, 0], [0, 0, 0, 0, 1]])
    ids, mask = O.pad_rows(rows, 1, min_width=2, pad_multiple=4, dtype=np.uint8)
    assert ids.dtype == np.uint8
    np.testing.assert_array_equal(ids, [[5, 6, 7, 1], [1, 1, 1, 1], [9, 1, 1, 1]])
    ids, mask = O.pad_rows(rows, 1, 2, pad_left=True)             # a fixed width below the longest row
    np.testing.assert_array_equal(ids, [[5, 6], [1, 1], [1, 9]])
    np.testing.assert_array_equal(mask, [[1, 1], [0, 0], [0, 1]])


# ------------------------------------------------------------------- BPE

@pytest.mark.parametrize("which,name,maker", [
    ("4096", "C3_bpe4096", wl.config3_bpe4096),
    ("32000", "C4_bpe32000", wl.config4_bpe32000),
])
def test_bpe_golden(which, name, maker):
    bo = util.bpe_oracle(which)
    b = maker()
    util.check_against_golden(name, bo.encode_batch(b.data, b.offsets))


def test_c5_golden_char_and_bpe():
    b = wl.config5_ragged()
    lut = util.char_lut()
    flat = O.char_encode_packed(lut, b.data)
    util.check_against_golden("C5_char", [flat[b.offsets[i]:b.offsets[i + 1]] for i in range(b.n_seqs)])
    util.check_against_golden("C5_bpe4096", util.bpe_oracle("4096").encode_batch(b.data, b.offsets))


@pytest.mark.parametrize("which", ["4096", "32000"])
def test_bpe_small_cases_golden(which):
    bo = util.bpe_oracle(which)
    for s, g in zip(util.small_cases(), util.split_small("bpe" + which)):
        row = np.frombuffer(s.encode(), dtype=np.uint8)
        np.testing.assert_array_equal(bo.encode_row(row), g, err_msg=repr(s))
        np.testing.assert_array_equal(bo.encode_row(row, naive=True), g, err_msg=repr(s))


@pytest.mark.parametrize("which", ["4096", "32000"])
def test_bpe_invariants_and_hf_live(which):
    """Replay of the reference's random generator (tests/test_gputok_bpe_backend.py:100-105):
    random.seed(0), lengths from a fixed menu; plus homopolymers 32..1024 (293-308)."""
    bo = util.bpe_oracle(which)
    tk = hf.load_bpe_tokenizer(which)
    random.seed(0)
    seqs = ["".join(random.choices("ACGT", k=random.choice([4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048])))
            for _ in range(64)]
    seqs += [c * n for c in "ACGT" for n in (32, 64, 128, 256, 512, 1024)]
    b = util.batch_from_strings(seqs)
    rows = bo.encode_batch(b.data, b.offsets)
    ref = hf_rows(tk, seqs)
    id_to_tok = {v: k for k, v in util.tokenizer_json(which)["model"]["vocab"].items()}
    merges = set(O.merges_from_tokenizer_json(util.tokenizer_json(which)))
    for s, r, e in zip(seqs, rows, ref):
        np.testing.assert_array_equal(r, e)
        toks = [id_to_tok[int(i)] for i in r]
        assert "".join(toks) == s                                  # decode round trip
        assert not any((a, b2) in merges for a, b2 in zip(toks, toks[1:]))   # nothing left to merge


def random_merge_list(rng, n_rules, duplicates=0, max_len=6):
    """A random merge list over ACGT; `duplicates` pairs are listed a second time further down."""
    toks, merges, seen, strings = list("ACGT"), [], set(), set("ACGT")
    while len(merges) < n_rules:
        a, b2 = rng.choice(toks), rng.choice(toks)
        if (a, b2) in seen or len(a + b2) > max_len:
            continue
        seen.add((a, b2))
        merges.append((a, b2))
        if a + b2 not in strings:
            strings.add(a + b2)
            toks.append(a + b2)
    for _ in range(duplicates):
        i = rng.randrange(len(merges))
        merges.insert(rng.randint(i + 1, len(merges)), merges[i])
    return merges


def hf_bpe_from_merges(merges):
    from tokenizers import Tokenizer, models
    vocab = {"[UNK]": 0}
    for t in list("ACGTN") + [x for a, b2 in merges for x in (a, b2, a + b2)]:
        vocab.setdefault(t, len(vocab))
    return Tokenizer(models.BPE(vocab=vocab, merges=list(merges), unk_token="[UNK]")), vocab


def test_bpe_repeated_pair_takes_its_last_entry_as_hf_does():
    """HF collects the merges into a map in list order: a pair listed again further down takes
    the later rank.  Known case first, then random lists with repeats against the live library."""
    tk, vocab = hf_bpe_from_merges([("A", "C"), ("C", "G"), ("A", "C")])
    assert tk.encode("ACG").tokens == ["A", "CG"]
    bo = O.BpeOracle([("A", "C"), ("C", "G"), ("A", "C")], vocab, 0)
    np.testing.assert_array_equal(bo.encode_row(np.frombuffer(b"ACG", np.uint8)), [vocab["A"], vocab["CG"]])
    rng = random.Random(31)
    for trial in range(40):
        merges = random_merge_list(rng, rng.randint(3, 30), duplicates=rng.randint(1, 5))
        tk, vocab = hf_bpe_from_merges(merges)
        bo = O.BpeOracle(merges, vocab, 0)
        seqs = ["".join(rng.choice("ACGT") for _ in range(rng.randint(1, 120))) for _ in range(20)]
        for sq, e in zip(seqs, hf_rows(tk, seqs)):
            row = np.frombuffer(sq.encode(), np.uint8)
            np.testing.assert_array_equal(bo.encode_row(row), e, err_msg=f"trial {trial} {sq}")
            np.testing.assert_array_equal(bo.encode_row(row, naive=True), e, err_msg=f"trial {trial} {sq}")


def test_bpe_heap_equals_naive_on_random_tables():
    rng = random.Random(7)
    for trial in range(300):
        alpha = "ACGT"[:rng.choice([2, 3, 4])]
        toks, merges, seen, strings = list(alpha), [], set(), set(alpha)
        for _ in range(rng.randint(1, 40)):
            a, b2 = rng.choice(toks), rng.choice(toks)
            if (a, b2) in seen or len(a + b2) > 10:
                continue
            seen.add((a, b2))
            merges.append((a, b2))
            if a + b2 not in strings:
                strings.add(a + b2)
                toks.append(a + b2)
        bo = O.BpeOracle(merges)
        for _ in range(4):
            s = "".join(rng.choice(alpha) for _ in range(rng.randint(1, 80)))
            row = np.frombuffer(s.encode(), dtype=np.uint8)
            np.testing.assert_array_equal(bo.encode_row(row, remap=False),
                                          bo.encode_row(row, naive=True, remap=False))


def test_kernel_vocab_first_seen_order():
    vocab, a, b2, n = O.kernel_vocab_from_merges([("A", "C"), ("AC", "G"), ("G", "T"), ("A", "CG")])
    assert vocab[256:] == ["AC", "ACG", "GT", "CG"]       # 'CG' is interned before 'A'+'CG' reuses 'ACG'
    assert a.tolist() == [65, 256, 71, 65] and b2.tolist() == [67, 71, 84, 259]
    assert n.tolist() == [256, 257, 258, 257]


# ------------------------------------------------------------------ 2-bit ingest

def test_pack_2bit_known_bytes_and_round_trip():
    as_rows = lambda s: np.frombuffer(s.encode(), dtype=np.uint8).reshape(1, -1)
    assert O.pack_2bit(as_rows("ACGT")).tolist() == [[0xE4]]            # 0 | 1<<2 | 2<<4 | 3<<6
    assert O.pack_2bit(as_rows("TTTT")).tolist() == [[0xFF]]
    assert O.pack_2bit(as_rows("CA")).tolist() == [[0x01]]              # filled up with code 0
    assert O.pack_2bit(as_rows("acgtN")).tolist() == [[0xE4, 0x00]]     # case folded, N travels as A
    assert O.pack_2bit(as_rows("AAAAG")).tolist() == [[0x00, 0x02]]
    # every packed byte spells its four bases back, first base in the low bits
    lut = np.arange(256, dtype=np.int64)                                # id = ASCII code
    every = np.arange(256, dtype=np.uint8).reshape(1, 256)
    ids = O.unpack_2bit_ids(lut, every, 1024)[0].reshape(256, 4)
    for b in (0, 1, 0x1B, 0xE4, 0xFF):
        want = ["ACGT"[(b >> (2 * j)) & 3] for j in range(4)]
        assert [chr(x) for x in ids[b]] == want
    # round trip on ACGT text of every length mod 4; N reads back as A
    rng = np.random.default_rng(5)
    for t in (1, 2, 3, 4, 5, 63, 64, 257):
        rows = rng.choice(np.frombuffer(b"ACGT", dtype=np.uint8), size=(7, t))
        assert np.array_equal(O.unpack_2bit_ids(lut, O.pack_2bit(rows), t), rows)
    start = lut + 1000
    got = O.unpack_2bit_ids(lut, O.pack_2bit(as_rows("GATN")), 4, start_lut=start)
    assert got.tolist() == [[ord("G") + 1000, ord("A"), ord("T"), ord("A")]]


def test_clean_ascii_cases():
    raw = np.frombuffer(b"acgtnACGTNxX-?rR", dtype=np.uint8)
    assert O.clean_ascii(raw, False, False).tobytes() == b"acgtnACGTNxX-?rR"
    assert O.clean_ascii(raw, True, False).tobytes() == b"ACGTNACGTNXX-?RR"
    assert O.clean_ascii(raw, False, True).tobytes() == b"acgtnACGTNNNNNNN"
    assert O.clean_ascii(raw, True, True).tobytes() == b"ACGTNACGTNNNNNNN"
