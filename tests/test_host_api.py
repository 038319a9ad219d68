"""Host-side logic of the drop-in API that needs no GPU: normalizer compiler truth tables
(the reference's own CPU unit tests, tests/test_gputok_bpe_backend.py:319-425), tokenizer.json
handling, and the compat tokenizer classes."""
import json

import numpy as np
import pytest

from dnatok_amd import dnatok_compat
from tests.support import hf_tokenizers as hf
from dnatok_amd.gputok_bpe_backend import (GPUTokBPEBackend, _compile_normalizer, _compile_normalizer_step, _extract_merges,
                                           _read_tokenizer_json, _reconstruct_gputok_vocab,
                                           _supported_tokenizer)


def test_normalizer_strip():
    fn = _compile_normalizer_step({"type": "Strip", "strip_left": True, "strip_right": True})
    assert fn("  ACGT  ") == "ACGT" and fn("ACGT") == "ACGT"
    assert _compile_normalizer_step({"type": "Strip", "strip_left": True, "strip_right": False})("  ACGT  ") == "ACGT  "
    assert _compile_normalizer_step({"type": "Strip", "strip_left": False, "strip_right": True})("  ACGT  ") == "  ACGT"


def test_normalizer_replace_string_and_regex():
    fn = _compile_normalizer_step({"type": "Replace", "pattern": {"String": "N"}, "content": "-"})
    assert fn("ACGTNNACGT") == "ACGT--ACGT"
    rx = _compile_normalizer_step({"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "-"})
    assert rx("ACGT" + "N" * 9 + "ACGT") == "ACGT" + "N" * 9 + "ACGT"
    assert rx("ACGT" + "N" * 10 + "ACGT") == "ACGT-ACGT"


def test_normalizer_prepend_lowercase_identity():
    assert _compile_normalizer_step({"type": "Prepend", "prepend": "_"})("ACGT") == "_ACGT"
    assert _compile_normalizer_step({"type": "Prepend", "prepend": "_"})("") == "_"
    assert _compile_normalizer_step({"type": "Lowercase"})("ACGTACGT") == "acgtacgt"
    for typ in ("NFC", "NFKC", "NFD", "NFKD", "StripAccents"):
        assert _compile_normalizer_step({"type": typ})("ACGT") == "ACGT"


def test_normalizer_sequence_and_rejections():
    fn = _compile_normalizer_step({"type": "Sequence", "normalizers": [
        {"type": "Strip", "strip_left": True, "strip_right": True},
        {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "-"}]})
    assert fn("   " + "N" * 12 + "ACGT  ") == "-ACGT"
    for typ in ("BertNormalizer", "Nmt", "Precompiled", "SomeNewThingHFAdds"):
        assert _compile_normalizer_step({"type": typ}) is None
    assert _compile_normalizer_step({"type": "Sequence", "normalizers": [
        {"type": "Strip"}, {"type": "BertNormalizer"}]}) is None
    ok, reason = _supported_tokenizer({"model": {"type": "BPE", "merges": ["A A"]},
                                       "pre_tokenizer": {"type": "Whitespace"},
                                       "normalizer": {"type": "BertNormalizer"}})
    assert not ok and "normalizer" in reason.lower()
    assert _compile_normalizer({"normalizer": None}) is None


def test_supported_tokenizer_gate():
    assert _supported_tokenizer(None) == (False, "tokenizer.json not found")
    assert not _supported_tokenizer({"model": {"type": "WordLevel"}})[0]
    assert not _supported_tokenizer({"model": {"type": "BPE"}, "pre_tokenizer": {"type": "ByteLevel"}})[0]
    assert _supported_tokenizer({"model": {"type": "BPE"}, "pre_tokenizer": None})[0]


def test_gate_refuses_bpe_options_that_change_the_ids():
    """Live HF tokenizers built with each BPE option: the option changes what the library returns
    (so a backend that ignores it would be wrong), and the gate refuses the tokenizer."""
    from tokenizers import Tokenizer, models, pre_tokenizers
    vocab = {"[UNK]": 0, "A": 1, "C": 2, "G": 3, "T": 4, "AC": 5, "ACG": 6, "##C": 7, "##G": 8, "T</w>": 9,
             "<0x4E>": 10, "ACGT": 11, "GT": 12}
    merges = [("A", "C"), ("AC", "G"), ("G", "T")]
    plain = Tokenizer(models.BPE(vocab=vocab, merges=merges, unk_token="[UNK]"))
    assert plain.encode("ACGT").ids == [6, 4] and plain.encode("ANNC").ids == [1, 0, 0, 2]
    assert _supported_tokenizer(json.loads(plain.to_str())) == (True, "ok")
    variants = {
        "dropout": (dict(dropout=0.5), None),
        "fuse_unk": (dict(fuse_unk=True), ("ANNC", [1, 0, 2])),
        "byte_fallback": (dict(byte_fallback=True), ("ANC", [1, 10, 2])),
        "ignore_merges": (dict(ignore_merges=True), ("ACGT", [11])),
        "continuing_subword_prefix": (dict(continuing_subword_prefix="##", merges=[("A", "##C")]), ("AG", [1, 8])),
        "end_of_word_suffix": (dict(end_of_word_suffix="</w>"), ("AT", [1, 9])),
    }
    for name, (kwargs, known) in variants.items():
        tk = Tokenizer(models.BPE(vocab=vocab, unk_token="[UNK]", **dict(dict(merges=merges), **kwargs)))
        if known is not None:
            text, ids = known
            assert tk.encode(text).ids == ids and plain.encode(text).ids != ids, name
        ok, reason = _supported_tokenizer(json.loads(tk.to_str()))
        assert not ok and name in reason, (name, reason)
        assert not GPUTokBPEBackend.is_supported(tk)
    # pre-tokenizers: white-space cuts are fine (rows hold none), other cuts are not
    for pre, want in ((pre_tokenizers.WhitespaceSplit(), True), (pre_tokenizers.Whitespace(), True),
                      (pre_tokenizers.Split(" ", "removed"), True), (pre_tokenizers.Split("C", "isolated"), False),
                      (pre_tokenizers.ByteLevel(), False), (pre_tokenizers.Digits(), False)):
        tk = Tokenizer(models.BPE(vocab=vocab, merges=merges, unk_token="[UNK]"))
        tk.pre_tokenizer = pre
        assert _supported_tokenizer(json.loads(tk.to_str()))[0] is want, pre
    # "Whitespace" also cuts between letters and punctuation: refused when a merge spans such a border
    v2 = dict(vocab, **{"-": 13, "A-": 14})
    tk = Tokenizer(models.BPE(vocab=v2, merges=merges + [("A", "-")], unk_token="[UNK]"))
    tk.pre_tokenizer = pre_tokenizers.Whitespace()
    assert tk.encode("A-C").ids == [1, 13, 2]                   # the library does not apply A + -
    ok, reason = _supported_tokenizer(json.loads(tk.to_str()))
    assert not ok and "border" in reason


def test_tokenizer_json_from_live_object_and_merges():
    tk = hf.load_bpe_tokenizer("4096")
    cfg = _read_tokenizer_json(tk)
    assert cfg["model"]["type"] == "BPE"
    merges = _extract_merges(cfg)
    assert len(merges) == len(cfg["model"]["merges"]) and all(len(m.split(" ")) == 2 for m in merges)
    assert _extract_merges({"model": {"merges": [["A", "C"], "AC G"]}}) == ["A C", "AC G"]
    vocab = _reconstruct_gputok_vocab(["A C", "AC G", "G T", "A CG"])
    assert vocab[:256] == [chr(b) for b in range(256)] and vocab[256:] == ["AC", "ACG", "GT", "CG"]


def test_compat_tokenizers():
    nt = dnatok_compat.NTv3Tokenizer()
    assert nt.vocab_size == 11 and nt.pad_token_id == 1 and nt.unk_token_id == 0
    assert nt.encode("ATCGNxa") == [6, 7, 8, 9, 10, 0, 6]
    out = nt(["AC", "ACGT"], padding=True, return_tensors="pt")["input_ids"]
    assert out.tolist() == [[6, 8, 1, 1], [6, 8, 9, 7]]
    evo = dnatok_compat.Evo2ByteTokenizer()
    assert evo.encode("ACGT") == [65, 67, 71, 84] and evo.vocab_size == 512
    ch = dnatok_compat.CharTokenizer()
    assert ch.encode("acgtnX") == [7, 8, 9, 10, 11, 11] and ch.pad_token_id == 0
    # the HF WordLevel tokenizer of the benchmark and NTv3Tokenizer agree on upper-case DNA
    tk = hf.build_char_tokenizer()
    s = "ACGTNNACGTTTGACN"
    assert tk.encode(s, add_special_tokens=False).ids == nt.encode(s)


# ------------------------------------------------------------------ host ingest (C ABI, CPU code)

def test_compat_tokenizers_save_their_vocabulary(tmp_path):
    """save_vocabulary as the reference's classes have it (src/dnatok_compat.py:152-156, 213-218):
    the NTv3 file is read back by the constructor, the Evo2 file holds the vocabulary size."""
    t = dnatok_compat.NTv3Tokenizer()
    (path,) = t.save_vocabulary(str(tmp_path), "x")
    assert path.endswith("x-vocab.json")
    again = dnatok_compat.NTv3Tokenizer(vocab_file=path)
    assert again.get_vocab() == t.get_vocab() and again.encode("ACGTNacgtx") == t.encode("ACGTNacgtx")
    (path,) = dnatok_compat.Evo2ByteTokenizer(300).save_vocabulary(str(tmp_path))
    assert path.endswith("evo2_vocab.json") and json.load(open(path)) == {"vocab_size": 300}


def test_host_clean_ascii_matches_oracle():
    import torch
    from dnatok_amd import encoders
    from oracle import oracle as O
    rng = np.random.default_rng(3)
    raw = rng.integers(0, 256, size=10_000, dtype=np.uint8)
    raw[::3] = rng.choice(np.frombuffer(b"ACGTNacgtn", dtype=np.uint8), size=raw[::3].size)
    for upper in (False, True):
        for to_n in (False, True):
            buf = torch.from_numpy(raw.copy())
            n = encoders.clean_ascii_host(buf, upper_case=upper, invalid_to_n=to_n)
            want = O.clean_ascii(raw, upper, to_n)
            assert np.array_equal(buf.numpy(), want)
            if to_n:
                up = O.clean_ascii(raw, upper, False)
                assert n == int((up != want).sum())
    assert encoders.clean_ascii_host(torch.empty(0, dtype=torch.uint8), upper_case=True, invalid_to_n=True) == 0


def test_host_pack_2bit_matches_oracle():
    import torch
    from dnatok_amd import encoders
    from oracle import oracle as O
    rng = np.random.default_rng(4)
    for b, t in ((1, 1), (3, 4), (5, 7), (2, 64), (9, 1001), (64, 8192)):
        rows = rng.choice(np.frombuffer(b"ACGTNacgtnX", dtype=np.uint8), size=(b, t))
        got = encoders.pack_2bit_host(torch.from_numpy(rows)).numpy()
        assert got.shape == (b, (t + 3) // 4)
        assert np.array_equal(got, O.pack_2bit(rows))
    assert encoders.pack_2bit_host(torch.from_numpy(np.frombuffer(b"ACGT", dtype=np.uint8).reshape(1, 4).copy())
                                   ).numpy().tolist() == [[0xE4]]
    with pytest.raises(ValueError):
        encoders.pack_2bit_host(torch.zeros(4, dtype=torch.uint8))


# ------------------------------------------------------------------ device normalizer: host-side compile

def test_device_normalizer_compile_and_validation():
    import ctypes
    from dnatok_amd import _lib
    from dnatok_amd.gputok_bpe_backend import _device_steps_of
    kinds = lambda step: [(s.kind, s.flags, bytes(s.pattern[:s.pattern_len]), bytes(s.content[:s.content_len]))
                          for s in _device_steps_of(step)]
    assert kinds({"type": "Strip", "strip_left": True, "strip_right": False}) == [(_lib.NORM_STRIP, 1, b"", b"")]
    assert kinds({"type": "Strip", "strip_left": False, "strip_right": False}) == []
    assert kinds({"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "-"}) == \
        [(_lib.NORM_REPLACE_RUN, 10, b"N", b"-")]
    assert kinds({"type": "Replace", "pattern": {"Regex": "N+"}, "content": ""}) == [(_lib.NORM_REPLACE_RUN, 1, b"N", b"")]
    assert kinds({"type": "Replace", "pattern": {"Regex": "\\-{2,}"}, "content": "-"}) == \
        [(_lib.NORM_REPLACE_RUN, 2, b"-", b"-")]
    assert kinds({"type": "Replace", "pattern": {"Regex": "^"}, "content": "_"}) == [(_lib.NORM_PREPEND, 0, b"", b"_")]
    assert kinds({"type": "Replace", "pattern": {"String": "AC"}, "content": "x"}) == [(_lib.NORM_REPLACE, 0, b"AC", b"x")]
    assert kinds({"type": "Prepend", "prepend": "\u2581"}) == [(_lib.NORM_PREPEND, 0, b"", "\u2581".encode())]
    assert kinds({"type": "Sequence", "normalizers": [{"type": "NFKC"}, {"type": "Lowercase"}]}) == \
        [(_lib.NORM_LOWERCASE, 0, b"", b"")]
    for not_on_device in (
            {"type": "Replace", "pattern": {"Regex": "[NX]{2,}"}, "content": "N"},      # a character class
            {"type": "Replace", "pattern": {"Regex": ".{3,}"}, "content": "N"},         # any character
            {"type": "Replace", "pattern": {"Regex": "\\d+"}, "content": "N"},          # a class escape
            {"type": "Replace", "pattern": {"Regex": "(N)\\1"}, "content": "N"},
            {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "\\g<0>"},   # group reference
            {"type": "Replace", "pattern": {"Regex": "N{100,}"}, "content": "N"},       # longer than the window
            {"type": "Replace", "pattern": {"String": "AA"}, "content": "x"},           # overlaps itself
            {"type": "Replace", "pattern": {"String": "ATA"}, "content": "x"},
            {"type": "Replace", "pattern": {"String": ""}, "content": "x"},
            {"type": "Replace", "pattern": {"String": "ACGTACGTACGTACGTA"[:17] + "C"}, "content": "x"},
            {"type": "Prepend", "prepend": "x" * 17},
            {"type": "BertNormalizer"}):
        assert _device_steps_of(not_on_device) is None, not_on_device
    # the library validates the records itself as well
    L = _lib.lib()
    bad = (_lib.NormStep * 1)(_lib.NormStep.make(_lib.NORM_REPLACE, 0, b"AA", b"x"))
    assert L.dnatok_normalize_bounds(bad, 1, 1, 10, 10, None, None, None) == -1
    assert b"overlaps itself" in L.dnatok_last_error()
    run = (_lib.NormStep * 2)(_lib.NormStep.make(_lib.NORM_REPLACE_RUN, 3, b"N", b"0123456789"),
                              _lib.NormStep.make(_lib.NORM_PREPEND, 0, b"", b"__"))
    t, m, sc = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_size_t()
    assert L.dnatok_normalize_bounds(run, 2, 4, 100, 30, ctypes.byref(t), ctypes.byref(m), ctypes.byref(sc)) == 0
    assert (t.value, m.value) == (33 * 10 + 1 + 8, 100 + 2) and sc.value >= 2 * t.value


def test_fasta_scan_layout_names_and_edge_cases(tmp_path):
    """Records end to end + offsets; CR LF, blanks inside lines, ';' lines, an empty record, bases in
    front of the first header, no line feed at the end."""
    from dnatok_amd import encoders
    text = b"; comment\nACG T\n>chr1 first\nACGT\nacgtn\r\n\n>empty\n>chr2\nTT\tTT\nGG"
    data, off, names = encoders.fasta_to_bytes(text)
    assert bytes(data.numpy()) == b"ACGTACGTacgtnTTTTGG"
    assert off.tolist() == [0, 4, 13, 13, 19]
    assert names == ["", "chr1 first", "empty", "chr2"]
    data, off, _ = encoders.fasta_to_bytes(text, upper_case=True)
    assert bytes(data.numpy()) == b"ACGTACGTACGTNTTTTGG"
    # from a file, against a plain Python reading of the same text
    rng = np.random.default_rng(4)
    seqs = ["".join(rng.choice(list("ACGTN"), size=int(n))) for n in rng.integers(0, 500, size=40)]
    path = tmp_path / "reads.fa"
    with open(path, "w") as fh:
        for i, s in enumerate(seqs):
            fh.write(f">read{i} len={len(s)}\n")
            for j in range(0, len(s), 60):
                fh.write(s[j:j + 60] + "\n")
    data, off, names = encoders.fasta_to_bytes(str(path))
    assert names == [f"read{i} len={len(s)}" for i, s in enumerate(seqs)]
    assert off.tolist() == np.concatenate([[0], np.cumsum([len(s) for s in seqs])]).tolist()
    assert bytes(data.numpy()).decode() == "".join(seqs)
    empty = encoders.fasta_to_bytes(b"")
    assert empty[0].numel() == 0 and empty[1].tolist() == [0] and empty[2] == []


def test_fasta_scan_rejects_too_small_outputs():
    import ctypes
    from dnatok_amd import _lib
    L = _lib.lib()
    text = np.frombuffer(b">a\nACGT\n>b\nAC\n", dtype=np.uint8)
    seq = np.zeros(16, dtype=np.uint8)
    off = np.zeros(4, dtype=np.int64)
    n_rec, n_bases = ctypes.c_int64(0), ctypes.c_int64(0)
    args = (ctypes.c_void_p(text.ctypes.data), text.size, 0, ctypes.c_void_p(seq.ctypes.data))
    rc = L.dnatok_host_fasta_scan(*args, 16, ctypes.c_void_p(off.ctypes.data), None, 1,
                                  ctypes.byref(n_rec), ctypes.byref(n_bases))
    assert rc == -3 and b"records" in L.dnatok_last_error()
    rc = L.dnatok_host_fasta_scan(*args, 5, ctypes.c_void_p(off.ctypes.data), None, 2,
                                  ctypes.byref(n_rec), ctypes.byref(n_bases))
    assert rc == -3 and b"bases" in L.dnatok_last_error()
    rc = L.dnatok_host_fasta_scan(*args, 6, ctypes.c_void_p(off.ctypes.data), None, 2,
                                  ctypes.byref(n_rec), ctypes.byref(n_bases))
    assert rc == 0 and (n_rec.value, n_bases.value) == (2, 6) and off[:3].tolist() == [0, 4, 6]


def test_hostpack_writes_offsets_and_bytes_as_the_python_path_does():
    """The C packer against plain Python: offsets, bytes, the two encodings, the size it asks for."""
    import torch
    from dnatok_amd import _hostpack
    rows = ["ACGT", "", "h\u00e9llo\u4e16", "N" * 300, "acgt"]
    for utf8 in (0, 1):
        want = [r.encode("utf-8") if utf8 else r.encode("ascii", errors="replace") for r in rows]
        buf = torch.zeros(4096, dtype=torch.uint8)
        n, total, longest, at = _hostpack.pack_strings(rows, buf.data_ptr(), buf.numel(), utf8)
        assert (n, total, longest) == (len(rows), sum(map(len, want)), max(map(len, want))) and at % 256 == 0
        offsets = buf[:8 * (n + 1)].view(torch.int64).tolist()
        assert offsets == [sum(map(len, want[:i])) for i in range(n + 1)]
        assert bytes(buf[at:at + total].numpy()) == b"".join(want)
        assert _hostpack.pack_strings(rows, buf.data_ptr(), at + total - 1, utf8) == -(at + total)
        assert _hostpack.pack_strings(tuple(rows), buf.data_ptr(), buf.numel(), utf8)[1] == total
    assert _hostpack.pack_strings([], buf.data_ptr(), buf.numel(), 0) == (0, 0, 0, 256)
    with pytest.raises(TypeError):
        _hostpack.pack_strings(["A", b"C"], buf.data_ptr(), buf.numel(), 0)


def test_width_guess_of_a_stream_follows_the_recent_peak():
    """encoders.WidthGuess: the guess of the next batch's width comes from the largest of the recent
    widths (fading by 1/256 per batch), not from the last batch alone.  On widths that wander as
    those of small 6-mer batches do (1100 .. 1265 tokens) the row stride derived from it (whole
    128-byte lines) is then almost never too small, which the previous width plus its margin is for
    one batch in seven; it still comes down when the stream turns narrower."""
    from dnatok_amd import encoders
    rng = np.random.default_rng(3)
    # widest row of a batch: a base level with an occasional long run of N
    widths = 1100 + (rng.gamma(1.2, 28, size=4000)).astype(np.int64).clip(0, 165)
    stride = lambda g: g + (-g) % 128
    wg, short_peak, short_prev = encoders.WidthGuess(), 0, 0
    assert not wg and wg.next() == 0
    for i, w in enumerate(widths[:-1]):
        wg.update(int(w))
        assert wg and wg.next() >= int(w) + 8 and wg.next() % 32 == 0
        short_peak += int(widths[i + 1]) >= stride(wg.next())
        short_prev += int(widths[i + 1]) >= stride(encoders.width_guess_after(int(w)))
    assert short_peak * 8 < short_prev and short_peak < 0.015 * widths.size
    # a stream that turns narrower: the guess follows within a few hundred batches
    for _ in range(450):
        wg.update(300)
    assert wg.next() <= 352
