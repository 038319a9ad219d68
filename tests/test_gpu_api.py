"""The drop-in Python surface on a GPU: DNATok / GPUTokBPEBackend / DnatokBpeKernel against the
tokenizers they wrap.  The fake tokenizers follow the reference's own test doubles
(tests/test_benchmark_correctness.py:22-57, tests/test_ids_path_equivalence.py:310-345,
tests/test_kmer_bytes_fallback.py:8-59)."""
import random

import numpy as np
import pytest
import torch

from dnatok_amd import dnatok_compat
from tests.support import hf_tokenizers as hf
from dnatok_amd.dna_tokenizer import DNATok
from dnatok_amd.dnatok_bpe_kernel import DnatokBpeKernel
from dnatok_amd.gputok_bpe_backend import GPUTokBPEBackend
from tests import util

pytestmark = pytest.mark.gpu


class SimpleCharTokenizer(dnatok_compat._SimpleTokenizer):
    def __init__(self):
        self.pad_token_id = 0
        self.padding_side = "left"
        self.vocab = {"<pad>": 0, "A": 1, "C": 2, "G": 3, "T": 4, "N": 5}
        for k, v in list(self.vocab.items()):
            if len(k) == 1:
                self.vocab[k.lower()] = v

    def _encode_one(self, text):
        return [self.vocab.get(ch, self.vocab["N"]) for ch in text]


class MockKmerTokenizer(dnatok_compat._SimpleTokenizer):
    """Non-overlapping k-mers over ACGT; a window holding anything else is spelled out."""

    def __init__(self, k=4):
        self.k, self.pad_token_id, self.unk_token_id, self.padding_side = k, 0, 1, "right"
        import itertools
        self.vocab = {"".join(p): i + 10 for i, p in enumerate(itertools.product("ACGT", repeat=k))}
        self.single = {c: 2 + i for i, c in enumerate("ACGTN")}

    def __len__(self):
        return 10 + 4 ** self.k

    def _encode_one(self, text):
        out = []
        for i in range(0, len(text), self.k):
            w = text[i:i + self.k]
            if len(w) == self.k and w in self.vocab:
                out.append(self.vocab[w])
            else:
                out.extend(self.single.get(c, self.unk_token_id) for c in w)
        return out


class FakeKmerTokenizer(dnatok_compat._SimpleTokenizer):
    """k = 3; a window holding N gives two tokens (97, 98), so its table entry stays -1."""

    def __init__(self, k=3):
        self.k, self.pad_token_id, self.padding_side, self._ids = k, 0, "right", {}

    def __len__(self):
        return 256

    def _encode_one(self, text):
        ids = []
        for i in range(0, len(text), self.k):
            chunk = text[i:i + self.k]
            if len(chunk) < self.k:
                continue
            if "N" in chunk:
                ids.extend([97, 98])
            else:
                ids.append(self._ids.setdefault(chunk, len(self._ids) + 1))
        return ids


class RecordingEmbedder(torch.nn.Module):
    def __init__(self, tokenizer, vocab=8192):
        super().__init__()
        self.tokenizer = tokenizer
        self.pad_id = tokenizer.pad_token_id if tokenizer is not None else 0
        self._embed = torch.nn.Embedding(vocab, 4)
        self.last_ids = None

    def embed_tokens(self, input_ids, rc_invariant=False):
        self.last_ids = input_ids.detach().clone()
        return self._embed(input_ids)


def random_seqs(b, t, alphabet="ACGTN", seed=0):
    random.seed(seed)
    return ["".join(random.choice(alphabet) for _ in range(t)) for _ in range(b)]


def test_char_discover_and_encode_matches_tokenizer():
    tok = SimpleCharTokenizer()
    helper = DNATok(RecordingEmbedder(tok))
    helper.discover()
    assert helper.use_ids_path and helper.kmer_k is None and helper.bpe_backend is None
    assert helper.id_pad == 0 and helper.id_N == 5 and helper.padding_side == "left"
    seqs = random_seqs(100, 64, seed=42)
    want = tok(seqs, padding=True, return_tensors="pt")["input_ids"]
    got = helper.encode_batch_to_ids(seqs)
    assert got.dtype == torch.int64 and got.is_pinned() and torch.equal(got, want)
    for base in "ACGTN":
        assert bool((helper.encode_batch_to_ids([base * 16]) == tok.vocab[base]).all())
    with pytest.raises(ValueError, match="No sequences"):
        helper.encode_batch_to_ids([])
    # ragged input is padded on the tokenizer's side
    ragged = ["ACGT", "ACGTACGTAC", "N"]
    assert torch.equal(helper.encode_batch_to_ids(ragged), tok(ragged, padding=True, return_tensors="pt")["input_ids"])


def test_char_case_and_invalid_handling():
    tok = SimpleCharTokenizer()
    h = DNATok(RecordingEmbedder(tok), normalize_case=True)
    h.discover()
    ids = h.encode_batch_to_ids(["AcGt", "acgt", "ACGT"])
    assert torch.equal(ids[0], ids[1]) and torch.equal(ids[0], ids[2])
    h2 = DNATok(RecordingEmbedder(tok), handle_invalid_chars=True)
    h2.discover()
    assert torch.equal(h2.encode_batch_to_ids(["ACXGT", "AC$GT"]), h2.encode_batch_to_ids(["ACNGT", "ACNGT"]))


def test_no_tokenizer_uses_fixed_map():
    h = DNATok(RecordingEmbedder(None))
    h.discover()
    assert h.encode_batch_to_ids(["ACGTN"]).tolist() == [[1, 2, 3, 4, 0]]


def test_ids_and_bytes_paths_feed_the_same_ids():
    tok = SimpleCharTokenizer()
    emb = RecordingEmbedder(tok)
    h = DNATok(emb)
    h.discover()
    seqs = random_seqs(4, 16)
    out_ids = list(h.embed_from_strings(seqs, emb_batch=4, device="cpu", path="ids"))
    a = emb.last_ids.clone()
    out_bytes = list(h.embed_from_strings(seqs, emb_batch=4, device="cpu", path="bytes"))
    assert torch.equal(a, emb.last_ids)
    assert torch.equal(a, tok(seqs, padding=True, return_tensors="pt")["input_ids"])
    assert all(torch.equal(x, y) for x, y in zip(out_ids, out_bytes))


@pytest.mark.parametrize("side", ["left", "right"])
def test_char_encode_batch_with_padding_follows_the_reference_form(side):
    """Single-nucleotide tokenizers: truncate to max_tokens, pad with N to the longest (or to
    max_tokens), round up to pad_multiple, overwrite the padding with the pad id, narrow the ids
    (the steps of the reference, src/dna_tokenizer.py:2150-2236, done here with numpy)."""
    tok = SimpleCharTokenizer()
    tok.padding_side = side
    h = DNATok(RecordingEmbedder(tok))
    h.discover()
    assert h.padding_side == side
    seqs = random_seqs(1, 50, seed=1) + random_seqs(1, 3, seed=2) + random_seqs(1, 37, seed=3) + ["A"]
    for max_tokens, pad_to_max, mult in ((40, False, 16), (100, True, 16), (100, False, 1), (37, False, 8), (64, True, 1)):
        ids, mask = h.encode_batch_with_padding(seqs, max_tokens, pad_to_max=pad_to_max, pad_multiple=mult)
        cut = [s[:max_tokens] for s in seqs]
        target = max(len(s) for s in cut)
        if pad_to_max:
            target = max(target, max_tokens)
        if mult > 1 and target % mult:
            target += mult - target % mult
        want = np.full((len(cut), target), tok.pad_token_id, dtype=np.int64)
        want_mask = np.zeros((len(cut), target), dtype=np.uint8)
        for i, sq in enumerate(cut):
            row = [tok.vocab[c] for c in sq]
            if side == "left":
                want[i, target - len(row):] = row
                want_mask[i, target - len(row):] = 1
            else:
                want[i, :len(row)] = row
                want_mask[i, :len(row)] = 1
        assert ids.dtype == torch.uint8 and mask.dtype == torch.uint8 and ids.is_cuda
        np.testing.assert_array_equal(ids.cpu().numpy().astype(np.int64), want)
        np.testing.assert_array_equal(mask.cpu().numpy(), want_mask)
    with pytest.raises(ValueError, match="Empty batch"):
        h.encode_batch_with_padding([], 10)


def test_two_bit_path_feeds_the_same_ids_as_the_bytes_path():
    tok = SimpleCharTokenizer()
    h = DNATok(RecordingEmbedder(tok), normalize_case=True, handle_invalid_chars=True)
    h.discover()
    for t in (64, 67):
        seqs = random_seqs(9, t, alphabet="ACGTacgt", seed=t)
        packed, t_true = h.encode_batch_to_packed_2bit(seqs)
        assert t_true == t and tuple(packed.shape) == (9, (t + 3) // 4) and packed.dtype == torch.uint8
        ids = h._unpack_2bit_to_ids_cuda(packed, t_true, "cuda")
        assert ids.dtype == torch.int64 and ids.is_cuda
        assert torch.equal(ids, h.ids_from_ascii_bytes_cuda(h.encode_batch_to_ascii_bytes(seqs)))
        assert torch.equal(ids.cpu(), tok(seqs, padding=True, return_tensors="pt")["input_ids"])
        assert torch.equal(ids, h._unpack_2bit_to_ids_cuda_u8(packed, t_true, "cuda"))
    # N and every other byte travel as code 0 and come back as A
    packed, t_true = h.encode_batch_to_packed_2bit(["ANxT"])
    assert h._unpack_2bit_to_ids_cuda(packed, t_true, "cuda").tolist() == [[1, 1, 1, 4]]
    # the staging bytes are cleaned the way the reference cleans them
    assert bytes(h.encode_batch_to_ascii_bytes(["acgtnx-R"]).numpy().tobytes()) == b"ACGTNNNN"


def test_fused_tokenize_gather_equals_lookup_then_embedding():
    tok = SimpleCharTokenizer()
    emb = RecordingEmbedder(tok).to("cuda")
    h = DNATok(emb)
    h.discover()
    seqs = random_seqs(6, 333, seed=8)
    weight = torch.randn((8, 64), device="cuda").to(torch.bfloat16)
    staged = h.encode_batch_to_ascii_bytes(seqs)
    out = h._fused_tokenize_gather(staged, weight, "cuda")
    ids = h.ids_from_ascii_bytes_cuda(staged)
    assert out.shape == (6, 333, 64) and out.dtype == torch.bfloat16
    assert torch.equal(out.view(torch.int16), weight[ids].view(torch.int16))


def test_recorded_graph_replays_with_new_bytes():
    """The bytes -> ids kernel captured in a HIP graph: several replays with different inputs,
    eager encodes and synchronisations in between, every replay checked against the eager ids."""
    tok = SimpleCharTokenizer()
    h = DNATok(RecordingEmbedder(tok))
    h.discover()
    with pytest.raises(RuntimeError, match="not recorded"):
        h._replay_cuda_graph(torch.zeros((2, 2), dtype=torch.uint8))
    h._record_cuda_graph(random_seqs(12, 200, seed=1), device="cuda", emb_batch=4)
    for seed in (2, 3, 4, 5):
        seqs = random_seqs(12, 200, seed=seed)
        want = tok(seqs, padding=True, return_tensors="pt")["input_ids"]
        staged = h.encode_batch_to_ascii_bytes(seqs)
        got = h._replay_cuda_graph(staged)
        assert got.dtype == torch.int64 and got.is_cuda
        assert torch.equal(got.cpu(), want)
        h.encode_batch_to_ids(random_seqs(3, 50, seed=seed + 10))     # eager work between the replays
        torch.cuda.synchronize()
    with pytest.raises(ValueError, match="shape mismatch"):
        h._replay_cuda_graph(torch.zeros((12, 100), dtype=torch.uint8))


@pytest.mark.parametrize("use_i32", [True, False])
def test_pipelined_streamer_equals_slices(use_i32):
    tok = SimpleCharTokenizer()
    emb = RecordingEmbedder(tok).to("cuda")
    h = DNATok(emb, ids_max_tokens_per_call=3 * 128, force_fp32_outputs=True)
    h.discover()
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 6, (23, 128), generator=g, dtype=torch.int64)        # 8 slices of <= 3 rows
    seen = []
    orig = emb.embed_tokens
    emb.embed_tokens = lambda input_ids, rc_invariant=False: (seen.append(input_ids.clone()), orig(input_ids))[1]
    for _ in range(2):                                                       # the second pass reuses the buffers
        seen.clear()
        outs = list(h.iter_embed_tokens_pipelined(ids, emb_batch=8, device="cuda", use_int32_h2d=use_i32))
        torch.cuda.synchronize()
        assert [o.shape[0] for o in outs] == [3] * 7 + [2]
        assert torch.equal(torch.cat(seen).cpu(), ids)
        ref = list(h.iter_embed_tokens_in_slices(ids, emb_batch=8, device="cuda"))
        assert all(torch.equal(a, b) for a, b in zip(outs, ref)) and len(outs) == len(ref)
    assert list(h.iter_embed_tokens_pipelined(ids[:0], 8, "cuda")) == []


def test_kmer_discover_and_encode():
    tok = MockKmerTokenizer(4)
    h = DNATok(RecordingEmbedder(tok))
    h.discover()
    assert h.kmer_k == 4 and h.use_ids_path
    seqs = random_seqs(64, 130, alphabet="ACGTACGTACGTN", seed=3)     # tail of 2, some N windows
    want = tok(seqs, padding=True, return_tensors="pt")["input_ids"]
    assert torch.equal(h.encode_batch_to_ids(seqs), want)
    ids, mask = h.encode_batch_with_padding(seqs, max_tokens=20, pad_multiple=16)
    assert ids.shape[1] % 16 == 0 and ids.dtype == torch.int16 and mask.dtype == torch.uint8
    short = tok([s[:80] for s in seqs], padding=True, return_tensors="pt")["input_ids"]
    assert torch.equal(ids[:, :short.shape[1]].cpu().long(), short)
    assert bool((ids[:, short.shape[1]:] == 0).all()) and bool((mask[:, short.shape[1]:] == 0).all())


def test_kmer_stream_of_batches_with_a_much_wider_one_in_between():
    """In a stream of batches the rows are laid out only as far apart as the previous batch was
    wide (plus a margin); a batch that needs more room than that is encoded again with room for
    the worst case, and every batch equals the tokenizer's own answer."""
    tok = MockKmerTokenizer(4)
    h = DNATok(RecordingEmbedder(tok))
    h.discover()
    narrow = random_seqs(48, 2000, alphabet="ACGT", seed=11)
    few_n = random_seqs(48, 2000, alphabet="ACGT" * 30 + "N", seed=12)
    wide = random_seqs(48, 2000, alphabet="ACGTN", seed=13)            # most windows are spelled
    for seqs in (narrow, few_n, narrow, wide, wide, narrow, few_n):
        want = tok(seqs, padding=True, return_tensors="pt")["input_ids"]
        ids, mask = h.encode_batch_device(seqs)
        assert torch.equal(ids.cpu().long(), want)
        assert torch.equal(mask.cpu().bool(), want != tok.pad_token_id)
        assert torch.equal(h.encode_batch_to_ids(seqs), want)


def test_kmer_stream_of_batches_of_short_reads():
    """Batches of reads of 100-300 bases: from the second batch on the rows lie a guess apart (at most
    384 cells), which sends them to the k-mer kernel for short rows; every batch as the tokenizer
    has it, a row with a foreign byte (which goes back to the tokenizer) included."""
    tok = MockKmerTokenizer(4)
    h = DNATok(RecordingEmbedder(tok))
    h.discover()
    assert h.kmer_k == 4
    rng = random.Random(12)
    for batch in range(5):
        seqs = ["".join(rng.choices("ACGTN", weights=[24, 24, 24, 24, 4], k=rng.randint(100, 300))) for _ in range(3000)]
        if batch == 3:
            seqs[7] = seqs[7][:50] + "x" + seqs[7][51:]
        want = tok(seqs, padding=True, return_tensors="pt")["input_ids"]
        assert torch.equal(h.encode_batch_to_ids(seqs), want), batch


def test_kmer_multi_token_windows_follow_the_tokenizer():
    tok = FakeKmerTokenizer(3)
    emb = RecordingEmbedder(tok, 256)
    h = DNATok(emb)
    h.discover()
    assert h.kmer_k == 3
    seqs = ["AAANNN", "ACGTAC", "NNNACG"]
    want = h._tokenize_batch_cpu(seqs)
    list(h.embed_from_strings(seqs, emb_batch=2, device="cpu", path="bytes"))
    assert torch.equal(h.encode_batch_to_ids(seqs), want)


@pytest.mark.parametrize("which", ["4096", "32000"])
def test_bpe_backend_matches_hf(which):
    tk = hf.load_bpe_tokenizer(which)
    assert GPUTokBPEBackend.is_supported(tk)
    be = GPUTokBPEBackend(tk, engine="dnatok")
    assert be.pad_id == 3 and be.unk_id == 0 and be.vocab_size == int(which)
    random.seed(0)
    seqs = ["".join(random.choices("ACGT", k=random.choice([4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048])))
            for _ in range(256)]
    seqs[3] = "ACGTNNNNNNACGTacgtXACGT"          # N, lower case and a byte outside the vocabulary
    ids, mask = be.encode_batch(seqs, device="cuda")
    assert ids.dtype == torch.int64 and mask.dtype == torch.uint8 and ids.is_cuda
    ref = [e.ids for e in tk.encode_batch(seqs, add_special_tokens=False)]
    assert ids.shape[1] == max(len(r) for r in ref)
    ids_h, mask_h = ids.cpu(), mask.cpu()
    for i, r in enumerate(ref):
        assert ids_h[i, :len(r)].tolist() == r
        assert bool((ids_h[i, len(r):] == be.pad_id).all())
        assert int(mask_h[i].sum()) == len(r) and bool(mask_h[i, :len(r)].all())
    # determinism and B = 1
    ids2, _ = be.encode_batch(seqs, device="cuda")
    assert torch.equal(ids, ids2)
    one, m1 = be.encode_batch([seqs[7]], device="cuda")
    assert one[0].tolist() == ref[7] and bool(m1.all())
    with pytest.raises(ValueError):
        be.encode_batch([], device="cuda")
    with pytest.raises(RuntimeError):
        GPUTokBPEBackend(tk, engine="gputok")


def test_bpe_backend_with_normalizer():
    import json
    from tokenizers import Tokenizer
    cfg = dict(util.tokenizer_json("4096"))
    cfg["normalizer"] = {"type": "Sequence", "normalizers": [
        {"type": "Strip", "strip_left": True, "strip_right": True},
        {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "N"}]}
    tk = Tokenizer.from_str(json.dumps(cfg))
    be = GPUTokBPEBackend(tk)
    seqs = ["  ACGTACGTTTGA  ", "ACGT" + "N" * 14 + "GGCATTA", "ACGTNNNACGT"]
    ids, mask = be.encode_batch(seqs)
    for i, e in enumerate(tk.encode_batch(seqs, add_special_tokens=False)):
        assert ids[i, :len(e.ids)].tolist() == e.ids and int(mask[i].sum()) == len(e.ids)


def test_bpe_backend_guards_input_it_cannot_reproduce():
    """Without an unk_token the library drops characters outside the vocabulary; with a
    pre-tokenizer it cuts rows at white space.  Rows without such characters are identical, rows
    with them raise UnsupportedRows, a ValueError that names them (DNATok catches it and takes those rows
    to the tokenizer itself: test_dnatok_bpe_rows_the_engine_cannot_reproduce_go_to_the_tokenizer)."""
    import json
    from tokenizers import Tokenizer
    cfg = json.loads(json.dumps(util.tokenizer_json("4096")))
    cfg["model"]["unk_token"] = None
    tk = Tokenizer.from_str(json.dumps(cfg))
    assert [e.ids for e in tk.encode_batch(["ACXGT"])] == [e.ids for e in tk.encode_batch(["ACGT"])]
    be = GPUTokBPEBackend(tk)
    seqs = random_seqs(12, 500, alphabet="ACGTN", seed=3)
    ids, mask = be.encode_batch(seqs)
    for i, e in enumerate(tk.encode_batch(seqs, add_special_tokens=False)):
        assert ids[i, :len(e.ids)].tolist() == e.ids and int(mask[i].sum()) == len(e.ids)
    with pytest.raises(ValueError) as caught:
        be.encode_batch(seqs[:3] + ["ACXGT"] + seqs[3:] + ["xx"])
    assert caught.value.rows == [3, len(seqs) + 1]
    cfg = json.loads(json.dumps(util.tokenizer_json("4096")))
    cfg["pre_tokenizer"] = {"type": "Whitespace"}
    tk = Tokenizer.from_str(json.dumps(cfg))
    be = GPUTokBPEBackend(tk)
    ids, mask = be.encode_batch(seqs)
    for i, e in enumerate(tk.encode_batch(seqs, add_special_tokens=False)):
        assert ids[i, :len(e.ids)].tolist() == e.ids and int(mask[i].sum()) == len(e.ids)
    with pytest.raises(ValueError):
        be.encode_batch(["ACGT ACGT"])


def _rows_to_device(rows):
    from dnatok_amd import encoders
    return encoders.bytes_from_strings(rows, "cuda", encoding="utf-8")


def _rows_from_device(data, offsets):
    off = offsets.cpu().numpy()
    raw = data.cpu().numpy().tobytes()
    return [raw[off[i]:off[i + 1]].decode("utf-8") for i in range(len(off) - 1)]


NORMALIZER_CASES = [
    {"type": "Strip", "strip_left": True, "strip_right": True},
    {"type": "Strip", "strip_left": True, "strip_right": False},
    {"type": "Strip", "strip_left": False, "strip_right": True},
    {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "-"},
    {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": ""},
    {"type": "Replace", "pattern": {"Regex": "N+"}, "content": "<run-of-N>"},
    {"type": "Replace", "pattern": {"Regex": "N{3,}"}, "content": "0123456789abcdef"},
    {"type": "Replace", "pattern": {"String": "N"}, "content": "nn"},
    {"type": "Replace", "pattern": {"String": "ACG"}, "content": "x"},
    {"type": "Replace", "pattern": {"String": "GT"}, "content": "[gt-pair]"},
    {"type": "Replace", "pattern": {"Regex": "^"}, "content": "_"},
    {"type": "Prepend", "prepend": "\u2581"},
    {"type": "Lowercase"},
    {"type": "Sequence", "normalizers": [
        {"type": "Strip", "strip_left": True, "strip_right": True},
        {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "-"},
        {"type": "Prepend", "prepend": "_"},
        {"type": "NFC"},
        {"type": "Lowercase"}]},
    {"type": "Sequence", "normalizers": [
        {"type": "Lowercase"},
        {"type": "Replace", "pattern": {"String": "acgt"}, "content": "ACGTACGT"},
        {"type": "Replace", "pattern": {"Regex": "n{2,}"}, "content": "N"},
        {"type": "Replace", "pattern": {"String": "TA"}, "content": ""}]},
]


@pytest.mark.parametrize("case", range(len(NORMALIZER_CASES)))
def test_device_normalizer_equals_the_host_callables(case):
    """Every normalizer step the device pass expresses, on rows built to hit its edges: empty
    rows (also first and last), rows of nothing but whitespace or N, runs of 9 / 10 / 11 N at row
    starts and ends, runs and matches that straddle the 16-position lane spans and the
    4096-position tiles; expected values from the str -> str callables (the reference's form)."""
    from dnatok_amd.gputok_bpe_backend import _compile_normalizer_step, _device_steps_of
    from dnatok_amd import encoders
    step = NORMALIZER_CASES[case]
    host = _compile_normalizer_step(step)
    steps = _device_steps_of(step)
    assert host is not None and steps is not None
    rng = random.Random(case)
    rows = ["", "N" * 9, "N" * 10, "N" * 11, "  \t ", " ", "ACGT", "  ACGTN" + "N" * 12 + "ACG \n", "",
            "N" * 10 + "A" + "N" * 9 + "C" + "N" * 30, "GTGTGT", "ACGACGAC", "TTACGTTTA", "NNN", "N", "G", "T" + "N" * 4095,
            "N" * 5000, "\x1c\x1fAC\x0b\x0c", ""]
    for n in (15, 16, 17, 31, 33, 4090, 4096, 4100, 9000):
        body = "".join(rng.choice("ACGTN") for _ in range(n))
        rows.append(body)
        rows.append("A" * (n - 5) + "N" * 12 + body[:7])          # a run across the n-th position
        rows.append("C" * (n - 2) + "ACGT" + "GT" * 3)            # matches across it
    rng.shuffle(rows)
    rows = [""] + rows + [""]
    data, offsets, lens = _rows_to_device(rows)
    norm = encoders.RowNormalizer(steps)
    out, out_off, total_bound, longest_bound = norm.apply(data, offsets, int(lens.sum()), int(lens.max()))
    torch.cuda.synchronize()
    want = [host(r) for r in rows]
    got = _rows_from_device(out, out_off)
    assert got == want
    want_bytes = [len(w.encode("utf-8")) for w in want]
    assert sum(want_bytes) <= total_bound and max(want_bytes) <= longest_bound
    # the input is left as it was
    assert _rows_from_device(data, offsets) == rows
    # no rows at all, and one empty row
    for few in ([], [""]):
        d2, o2, l2 = _rows_to_device(few)
        out2, off2, _, _ = norm.apply(d2, o2, 0, 0)
        assert _rows_from_device(out2, off2) == [host(r) for r in few]


def test_device_normalizer_on_a_batch_above_8192_tiles():
    """36 Mbases in 4000 rows: more than 8192 tiles of 4096 positions, where the tile sizes are
    scanned by a launch of their own and two passes alternate between the scratch buffers."""
    from dnatok_amd import encoders
    from dnatok_amd.gputok_bpe_backend import _compile_normalizer_step, _device_steps_of
    rng = np.random.default_rng(3)
    n_rows = 4000
    lens = rng.integers(100, 18_000, size=n_rows)
    data = np.frombuffer(b"ACGTN", dtype=np.uint8)[rng.integers(0, 5, size=int(lens.sum()))].copy()
    for at in rng.integers(0, data.size - 100, size=15_000):
        data[at:at + rng.integers(1, 40)] = ord("N")
    off = np.zeros(n_rows + 1, dtype=np.int64)
    off[1:] = np.cumsum(lens)
    assert data.size // 4096 > 8192
    spec = {"type": "Sequence", "normalizers": [
        {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "-"},
        {"type": "Prepend", "prepend": "_"}, {"type": "Lowercase"},
        {"type": "Replace", "pattern": {"String": "acg"}, "content": "ACGT"}]}
    host = _compile_normalizer_step(spec)
    norm = encoders.RowNormalizer(_device_steps_of(spec))
    out, out_off, bound, _ = norm.apply(torch.from_numpy(data).cuda(), torch.from_numpy(off).cuda(),
                                        int(off[-1]), int(lens.max()))
    torch.cuda.synchronize()
    oo, raw = out_off.cpu().numpy(), out.cpu().numpy()
    assert oo[-1] <= bound
    for i in range(n_rows):
        want = host(data[off[i]:off[i + 1]].tobytes().decode()).encode()
        assert raw[oo[i]:oo[i + 1]].tobytes() == want, i


def test_bpe_backend_normalizes_on_the_device_like_on_the_host():
    import json
    from tokenizers import Tokenizer
    cfg = dict(util.tokenizer_json("4096"))
    cfg["normalizer"] = {"type": "Sequence", "normalizers": [
        {"type": "Strip", "strip_left": True, "strip_right": True},
        {"type": "Replace", "pattern": {"Regex": "N{10,}"}, "content": "N"}]}
    tk = Tokenizer.from_str(json.dumps(cfg))
    be = GPUTokBPEBackend(tk)
    assert be._normalize_device is not None and be.normalize_on_device
    random.seed(3)
    seqs = []
    for _ in range(200):
        n = random.choice([0, 1, 5, 64, 500, 3000, 9000])
        body = "".join(random.choice("ACGT") for _ in range(n))
        if n > 40 and random.random() < 0.7:
            at = random.randrange(n - 30)
            body = body[:at] + "N" * random.choice([3, 9, 10, 11, 25]) + body[at + 25:]
        seqs.append(random.choice(["", " ", "  "]) + body + random.choice(["", "\n", " "]))
    ids, mask = be.encode_batch(seqs)
    be.normalize_on_device = False
    ids_h, mask_h = be.encode_batch(seqs)
    assert torch.equal(ids, ids_h) and torch.equal(mask, mask_h)
    for i, e in enumerate(tk.encode_batch(seqs, add_special_tokens=False)):
        assert ids[i, :len(e.ids)].tolist() == e.ids and int(mask[i].sum()) == len(e.ids)
    # a regex the device pass does not express keeps the host callables
    cfg["normalizer"] = {"type": "Replace", "pattern": {"Regex": "[NX]{2,}"}, "content": "N"}
    be2 = GPUTokBPEBackend(Tokenizer.from_str(json.dumps(cfg)))
    assert be2._normalize_device is None and be2._normalize is not None


def test_dnatok_routes_bpe_tokenizers_to_the_backend():
    tk = hf.load_bpe_tokenizer("4096")

    class Wrapped:                       # the attributes DNATok reads from an HF tokenizer
        pad_token_id, unk_token_id, padding_side = 3, 0, "right"
        backend_tokenizer = tk

        def __call__(self, texts, add_special_tokens=False, **kw):
            return {"input_ids": [e.ids for e in tk.encode_batch(list(texts), add_special_tokens=False)]}

        def get_vocab(self):
            return tk.get_vocab()

    h = DNATok(RecordingEmbedder(Wrapped()))
    h.discover()
    assert h.bpe_backend is not None and h.kmer_k is None and h.ascii_lut is None
    seqs = random_seqs(20, 300, alphabet="ACGT", seed=5) + ["ACGTACGTACGT"]
    got = h.encode_batch_to_ids(seqs)
    ref = [e.ids for e in tk.encode_batch(seqs, add_special_tokens=False)]
    for i, r in enumerate(ref):
        assert got[i, :len(r)].tolist() == r and bool((got[i, len(r):] == 3).all())


def _bpe_wrapped(side):
    tk = hf.load_bpe_tokenizer("4096")

    class Wrapped:                       # the attributes DNATok reads from an HF tokenizer
        pad_token_id, unk_token_id, padding_side = 3, 0, side
        backend_tokenizer = tk

        def __call__(self, texts, add_special_tokens=False, **kw):
            return {"input_ids": [e.ids for e in tk.encode_batch(list(texts), add_special_tokens=False)]}

        def get_vocab(self):
            return tk.get_vocab()

    return Wrapped()


def _bpe_wrapped_from(cfg, side):
    import json
    from tokenizers import Tokenizer
    tk = Tokenizer.from_str(json.dumps(cfg))

    class Wrapped:
        pad_token_id, padding_side = 3, side
        unk_token_id = 0 if cfg["model"].get("unk_token") is not None else None
        backend_tokenizer = tk

        def __call__(self, texts, add_special_tokens=False, **kw):
            return {"input_ids": [e.ids for e in tk.encode_batch(list(texts), add_special_tokens=False)]}

        def get_vocab(self):
            return tk.get_vocab()

    return Wrapped()


@pytest.mark.parametrize("side", ["left", "right"])
@pytest.mark.parametrize("kind", ["whitespace", "no_unk"])
def test_dnatok_bpe_rows_the_engine_cannot_reproduce_go_to_the_tokenizer(kind, side, caplog):
    """The reference's DNATok never raises on a BPE batch: whatever its backend cannot do ends at
    the tokenizer itself (src/dna_tokenizer.py:2066-2100).  Here the backend names the rows it cannot
    reproduce (white space under a pre-tokenizer, which cuts the row into words; a character outside
    the vocabulary without unk_token, which is dropped); those rows get the tokenizer's ids, the
    others stay on the GPU.  Expected in every case: the tokenizer's own rows, padded in plain
    Python on the tokenizer's side."""
    import json
    import logging
    cfg = json.loads(json.dumps(util.tokenizer_json("4096")))
    if kind == "whitespace":
        cfg["pre_tokenizer"] = {"type": "Whitespace"}
        odd = ["ACGT ACGTTTGA", "A C G T", " ACGTAC", "ACGTACGTAGCTAGCTAGCATCGATCGATCGACTAGCTAGCTAC\nACGT" * 30]
    else:
        cfg["model"]["unk_token"] = None
        odd = ["ACXGT", "xxxx", "ACGTACGTAGCTAGCTAGCATCGATCGATCGACTAGCTAGCTAC" * 30 + "acgt", "ACGTNNNNRY"]
    tok = _bpe_wrapped_from(cfg, side)
    h = DNATok(RecordingEmbedder(tok, vocab=8192), padding_side=side)
    h.discover()
    assert h.bpe_backend is not None and h.bpe_backend._input_guard is not None
    clean = random_seqs(9, 300, alphabet="ACGT", seed=31) + ["ACGTACGTACGT", "A"]
    mixed = clean[:4] + odd[:2] + clean[4:] + odd[2:]
    for seqs, n_odd in ((clean, 0), (mixed, len(odd)), (odd, len(odd)), ([odd[0]], 1), (clean, 0)):
        caplog.clear()
        with caplog.at_level(logging.WARNING, logger=h.log.name):
            want = h._tokenize_batch_cpu(seqs)
            got = h.encode_batch_to_ids(seqs)
            assert got.dtype == torch.int64 and got.shape == want.shape and torch.equal(got, want), (kind, side)
            ids, mask = h.encode_batch_device(seqs)
            assert ids.is_cuda and ids.dtype == torch.int32 and torch.equal(ids.cpu().long(), want)
            lens = torch.tensor([len(r) for r in h._tok_ids(seqs)])
            col = torch.arange(want.shape[1])[None, :]
            inside = (col >= want.shape[1] - lens[:, None]) if side == "left" else (col < lens[:, None])
            assert torch.equal(mask.cpu().bool(), inside)
            ids8, mask8 = h.encode_batch_with_padding(seqs, 10_000, pad_to_max=False, pad_multiple=8)
            assert ids8.shape[1] % 8 == 0 and ids8.shape[1] - want.shape[1] in range(8)
            for i, n in enumerate(lens.tolist()):
                sl = slice(ids8.shape[1] - n, ids8.shape[1]) if side == "left" else slice(0, n)
                assert ids8[i, sl].cpu().long().tolist() == h._tok_ids([seqs[i]])[0] and int(mask8[i].sum()) == n
        warned = [r for r in caplog.records if "tokenizer" in r.getMessage()]
        assert bool(warned) == bool(n_odd), (kind, side, n_odd, [r.getMessage() for r in caplog.records])


@pytest.mark.parametrize("side", ["left", "right"])
def test_dnatok_bpe_backend_failure_falls_back_to_the_tokenizer(side, monkeypatch, caplog):
    """Fault injection as in the reference's tests/test_bytes_path_fallback.py:56-75: the backend's
    entry points raise, and DNATok answers with the tokenizer's own rows and a warning."""
    import logging
    tok = _bpe_wrapped(side)
    h = DNATok(RecordingEmbedder(tok, vocab=8192), padding_side=side)
    h.discover()
    seqs = random_seqs(7, 200, alphabet="ACGT", seed=41) + ["ACGT"]
    want = h._tokenize_batch_cpu(seqs)
    assert torch.equal(h.encode_batch_to_ids(seqs), want)

    def boom(*args, **kwargs):
        raise RuntimeError("forced failure")

    monkeypatch.setattr(h.bpe_backend, "padded_device", boom)
    monkeypatch.setattr(h.bpe_backend, "tokens_device", boom)
    with caplog.at_level(logging.WARNING, logger=h.log.name):
        got = h.encode_batch_to_ids(seqs)
        ids, mask = h.encode_batch_device(seqs)
    assert torch.equal(got, want) and torch.equal(ids.cpu().long(), want)
    assert torch.equal(mask.cpu().bool(), want != 3)
    assert any("forced failure" in r.getMessage() for r in caplog.records)
    # a failed row (negative length from the engine) ends the same way
    monkeypatch.undo()

    def failed_row(*args, **kwargs):
        raise RuntimeError("BPE engine reported a failed row (negative length)")

    monkeypatch.setattr(h, "_pad_bpe_runs", failed_row)
    monkeypatch.setattr(h.bpe_backend, "padded_device", failed_row)
    assert torch.equal(h.encode_batch_to_ids(seqs), want)


@pytest.mark.parametrize("side", ["left", "right"])
def test_bpe_stream_of_batches_with_longer_rows_in_between(side):
    """As for the k-mer rows: in a stream of batches BPE rows are laid out only as far apart as the
    previous batch was wide; a batch with longer token rows than that is padded again with room for
    the worst case.  Ids on the host and on the device equal the tokenizer's own rows."""
    tok = _bpe_wrapped(side)
    h = DNATok(RecordingEmbedder(tok, vocab=8192), padding_side=side)
    h.discover()
    short = random_seqs(24, 600, alphabet="ACGT", seed=21)
    long_ = random_seqs(24, 5000, alphabet="ACGT", seed=22)
    ragged = [s[:n] for s, n in zip(random_seqs(24, 3000, alphabet="ACGT", seed=23), range(1, 3000, 120))]
    for seqs in (short, short, long_, short, ragged, long_, long_, short):
        want = h._tokenize_batch_cpu(seqs)
        got = h.encode_batch_to_ids(seqs)
        assert got.dtype == torch.int64 and got.shape == want.shape and torch.equal(got, want)
        ids, mask = h.encode_batch_device(seqs)
        assert torch.equal(ids.cpu().long(), want)
        assert torch.equal(mask.cpu().bool(), want != 3)


@pytest.mark.parametrize("side", ["left", "right"])
@pytest.mark.parametrize("family", ["kmer", "bpe"])
def test_ragged_rows_follow_padding_side_and_token_len(family, side):
    """Ragged batches through a k-mer and a BPE tokenizer: every row padded on the tokenizer's side to
    the longest row or to token_len, as the reference pads token rows (_pad_id_list,
    src/dna_tokenizer.py:1878-1894; BPE rows 2063-2078).  Expected: the tokenizer's own rows, padded in
    plain Python."""
    if family == "kmer":
        tok = MockKmerTokenizer(k=4)
        tok.padding_side = side
        alphabet = "ACGTN"
    else:
        tok, alphabet = _bpe_wrapped(side), "ACGT"
    h = DNATok(RecordingEmbedder(tok, vocab=8192), padding_side=side)
    h.discover()
    assert h.padding_side == side
    assert (h.kmer_k == 4) if family == "kmer" else (h.bpe_backend is not None)
    random.seed(3)
    seqs = ["".join(random.choice(alphabet) for _ in range(n)) for n in (40, 7, 400, 1, 123, 4, 399, 64)]
    rows = h._tok_ids(seqs)
    for token_len in (None, max(len(r) for r in rows) + 9, 3):
        h.token_len = token_len
        got = h.encode_batch_to_ids(seqs)
        want = h._tokenize_batch_cpu(seqs)
        assert got.shape == want.shape and torch.equal(got, want), (family, side, token_len)
        ids, mask = h.encode_batch_device(seqs)
        assert ids.dtype == torch.int32 and torch.equal(ids.cpu().long(), want)
        lens = torch.tensor([len(r) for r in rows])
        assert torch.equal(mask.cpu().sum(1).long(), lens)
        col = torch.arange(want.shape[1])[None, :]
        inside = (col >= want.shape[1] - lens[:, None]) if side == "left" else (col < lens[:, None])
        assert torch.equal(mask.cpu().bool(), inside)
    h.token_len = None
    # encode_batch_with_padding: cut to max_tokens, a multiple of pad_multiple, the narrowest id type
    k = 4 if family == "kmer" else 1
    for max_tokens, to_max, mult in ((50, False, 16), (50, True, 8), (500, True, 1)):
        ids, mask = h.encode_batch_with_padding(seqs, max_tokens, pad_to_max=to_max, pad_multiple=mult)
        cut = h._tok_ids([q[:max_tokens * k] for q in seqs])
        width = max(len(r) for r in cut)
        if to_max:
            width = max(width, max_tokens)
        if mult > 1 and width % mult:
            width += mult - width % mult
        assert tuple(ids.shape) == (len(seqs), width) and ids.dtype in (torch.uint8, torch.int16)
        for i, r in enumerate(cut):
            row, m = ids[i].cpu().long(), mask[i].cpu()
            sl = slice(width - len(r), width) if side == "left" else slice(0, len(r))
            assert row[sl].tolist() == r and int(m.sum()) == len(r) and bool(m[sl].all())
            assert int((row != h.id_pad).sum()) <= len(r)


def _write_fasta(path, seqs, width=70):
    with open(path, "w") as fh:
        for i, s in enumerate(seqs):
            fh.write(f">rec{i}\n")
            for j in range(0, len(s), width):
                fh.write(s[j:j + width] + "\n")


def test_fasta_file_encodes_like_the_same_strings(tmp_path):
    """File -> ids through the host scan, for each of the three kernel families."""
    rng = random.Random(8)
    seqs = ["".join(rng.choice("ACGTACGTN") for _ in range(rng.randint(1, 700))) for _ in range(50)]
    path = tmp_path / "reads.fa"
    _write_fasta(path, seqs)
    names = [f"rec{i}" for i in range(len(seqs))]

    h = DNATok(RecordingEmbedder(SimpleCharTokenizer()))
    h.discover()
    ids, mask, got_names = h.encode_fasta_device(str(path))
    want_ids, want_mask = h.encode_batch_device(seqs)
    assert got_names == names and torch.equal(ids, want_ids) and torch.equal(mask, want_mask)

    hk = DNATok(RecordingEmbedder(MockKmerTokenizer(4)))
    hk.discover()
    ids, mask, _ = hk.encode_fasta_device(str(path))
    want_ids, want_mask = hk.encode_batch_device(seqs)
    assert torch.equal(ids, want_ids) and torch.equal(mask, want_mask)

    tk = hf.load_bpe_tokenizer("4096")

    class Wrapped:
        pad_token_id, unk_token_id, padding_side = 3, 0, "right"
        backend_tokenizer = tk

        def __call__(self, texts, add_special_tokens=False, **kw):
            return {"input_ids": [e.ids for e in tk.encode_batch(list(texts), add_special_tokens=False)]}

        def get_vocab(self):
            return tk.get_vocab()

    hb = DNATok(RecordingEmbedder(Wrapped()))
    hb.discover()
    ids, mask, _ = hb.encode_fasta_device(path.read_bytes())
    for i, e in enumerate(tk.encode_batch(seqs, add_special_tokens=False)):
        assert ids[i, :len(e.ids)].tolist() == e.ids and int(mask[i].sum()) == len(e.ids)
    with pytest.raises(ValueError, match="No sequences"):
        h.encode_fasta_device(b"")


def test_bpe_kernel_wrapper_contract(tmp_path):
    cfg = util.tokenizer_json("4096")
    p = tmp_path / "merges.txt"
    p.write_text("#version: 0.2\n" + "\n".join(m if isinstance(m, str) else " ".join(m) for m in cfg["model"]["merges"]) + "\n")
    k = DnatokBpeKernel(str(p))
    bo = util.bpe_oracle("4096")
    assert k.vocab_size() == len(bo.vocab) and k.id_to_token(65) == "A" and k.id_to_token(300) == bo.vocab[300]
    with pytest.raises(IndexError):
        k.id_to_token(10 ** 6)
    seqs = random_seqs(9, 200, alphabet="ACGT", seed=1) + ["A", "ACGTACGTAC" * 90]
    ids, lens = k.tokenize_batch(seqs)
    assert ids.dtype == torch.int32 and ids.shape == (11, 900) and lens.dtype == torch.int32
    ids_h, lens_h = ids.cpu().numpy(), lens.cpu().numpy()
    for i, s in enumerate(seqs):
        want = bo.encode_row(np.frombuffer(s.encode(), dtype=np.uint8), remap=False)
        assert lens_h[i] == want.size and np.array_equal(ids_h[i, :want.size], want)
        assert (ids_h[i, want.size:] == 0).all()                 # zero-filled tail
    # views into a workspace: the next call overwrites them unless clone=True
    kept, kept_l = k.tokenize_batch(seqs, clone=True)
    view, _ = k.tokenize_batch(seqs)
    k.tokenize_batch(["T" * 900] * 11)
    torch.cuda.synchronize()
    assert torch.equal(kept.cpu(), torch.from_numpy(ids_h)) and not torch.equal(view.cpu(), kept.cpu())
    e_ids, e_len = k.tokenize_batch([])
    assert e_ids.shape == (0, 0) and e_len.shape == (0,)


@pytest.mark.parametrize("model,path", [("char", "ascii-lut"), ("ntv3", "ascii-lut"), ("evo2", "ascii-lut"),
                                        ("kmer6", "kmer-6"), ("bpe4096", "gpu-bpe-kernel")])
def test_cli_info_encode_validate(model, path, capsys, tmp_path):
    import json
    from dnatok_amd import dnatok_cli
    if model == "bpe4096":                       # a BPE tokenizer is named by the path of its tokenizer.json
        model = hf.bpe_tokenizer_path("4096")
    fa = tmp_path / "two.fa"
    fa.write_text(">first\nACGTACGTTTGACCA\n>second\nACGT\nTTGA\n")
    assert dnatok_cli.main(["encode", "--model", model, "--fasta", str(fa), "--json"]) == 0
    rec = json.loads(capsys.readouterr().out)
    assert rec["n_records"] == 2 and [r["name"] for r in rec["records"]] == ["first", "second"]
    assert rec["n_tokens_total"] == sum(r["n_tokens"] for r in rec["records"]) > 0
    assert dnatok_cli.main(["info", "--model", model, "--json"]) == 0
    info = json.loads(capsys.readouterr().out)
    assert info["selected_path"] == path and info["device"] == "cuda"
    assert dnatok_cli.main(["encode", "--model", model, "--seq", "ACGTACGTTTGACCA", "--json"]) == 0
    enc = json.loads(capsys.readouterr().out)
    assert enc["sequence_length_bp"] == 15 and enc["n_tokens"] == len(enc["token_ids"]) > 0
    assert dnatok_cli.main(["validate", "--model", model, "--n", "40", "--window", "600", "--json"]) == 0
    val = json.loads(capsys.readouterr().out)
    assert val["n_match"] == 40 and val["n_mismatch"] == 0 and val["first_mismatch"] is None
    assert dnatok_cli.main(["bench", "--model", model, "--n", "64", "--window", "512", "--chunk", "32",
                            "--hf-threads", "2", "--json"]) == 0
    b = json.loads(capsys.readouterr().out)
    assert b["total_bp"] == 64 * 512 and b["dnatok_mbp_per_s"] > 0


def test_cli_demo_and_list_models(capsys):
    """`demo` runs info, encode, validate and a small bench in a row and returns their verdict;
    `list-models` prints what --model accepts."""
    import json
    from dnatok_amd import dnatok_cli
    assert dnatok_cli.main(["demo", "--model", "kmer6", "--sample", "ACGTNNACGTACGT"]) == 0
    out = capsys.readouterr().out
    assert "[4/4]" in out and "bit identity holds" in out and "kmer-6" in out
    assert dnatok_cli.main(["list-models", "--json"]) == 0
    rows = json.loads(capsys.readouterr().out)
    assert {"char", "kmer6", "bpe"} <= {r["family"] for r in rows}
