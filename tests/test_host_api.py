"""Host-side logic of the drop-in API that needs no GPU: normalizer compiler truth tables
(the reference's own CPU unit tests, tests/test_gputok_bpe_backend.py:319-425), tokenizer.json
handling, and the compat tokenizer classes."""
import numpy as np
import pytest

from dnatok_amd import dnatok_compat, hf_tokenizers as hf
from dnatok_amd.gputok_bpe_backend import (_compile_normalizer, _compile_normalizer_step, _extract_merges,
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
