"""The BPE fallback chain of DNATok on the host alone (no GPU): a stand-in backend that keeps the
contract of GPUTokBPEBackend.padded_device (padded tokenizer ids of the rows it is given, or
UnsupportedRows naming the rows it cannot take, or any other failure) behind DNATok._encode_bpe_rows.
What comes out must be the tokenizer's own rows in DNATok's layout, whatever mix of rows the backend
refused (reference: src/dna_tokenizer.py:2066-2100, tests/test_bytes_path_fallback.py:56-75)."""
import logging

import pytest
import torch

from dnatok_amd import DNATok
from dnatok_amd.gputok_bpe_backend import UnsupportedRows


class WordTokenizer:
    """Ids by letter pairs, enough of a tokenizer for DNATok._tok_ids: 'ACGT' -> [id(AC), id(GT)];
    white space splits words and is dropped (what a whitespace pre-tokenizer does)."""
    pad_token_id = 0

    def __call__(self, texts, add_special_tokens=False):
        out = []
        for t in texts:
            ids = []
            for word in t.split():
                ids += [1 + (ord(word[i]) * 7 + (ord(word[i + 1]) if i + 1 < len(word) else 0)) % 997
                        for i in range(0, len(word), 2)]
            out.append(ids)
        return {"input_ids": out}


class Embedder(torch.nn.Module):
    def __init__(self, tokenizer):
        super().__init__()
        self.tokenizer = tokenizer
        self.pad_id = 0


class StandInBackend:
    """Takes rows without white space; the others it names.  `fail` makes every call raise."""

    def __init__(self, tok, fail=None):
        self.tok, self.fail, self.calls = tok, fail, []

    def padded_device(self, seqs, *, device="cpu", min_width=0, pad_multiple=1, stage_ids=None, pad_left=False,
                      dtype=torch.int32):
        self.calls.append(list(seqs))
        if self.fail is not None:
            raise self.fail
        bad = [i for i, s in enumerate(seqs) if " " in s]
        if bad:
            raise UnsupportedRows(bad, f"white space in rows {bad}")
        rows = self.tok(seqs)["input_ids"]
        width = max(max((len(r) for r in rows), default=0), int(min_width), 1)
        if pad_multiple > 1 and width % pad_multiple:
            width += pad_multiple - width % pad_multiple
        ids = torch.zeros((len(rows), width), dtype=dtype)
        mask = torch.zeros((len(rows), width), dtype=torch.uint8)
        for i, r in enumerate(rows):
            if r:
                at = slice(width - len(r), width) if pad_left else slice(0, len(r))
                ids[i, at] = torch.as_tensor(r, dtype=dtype)
                mask[i, at] = 1
        return ids, mask


def _helper(side, backend_fail=None):
    tok = WordTokenizer()
    h = DNATok(Embedder(tok), padding_side=side)
    h.id_pad = 0
    h.bpe_backend = StandInBackend(tok, fail=backend_fail)
    return tok, h


def _expected(tok, seqs, side, dtype, min_width=0, pad_multiple=1):
    rows = tok(seqs)["input_ids"]
    width = max(max(len(r) for r in rows), min_width)
    if pad_multiple > 1 and width % pad_multiple:
        width += pad_multiple - width % pad_multiple
    ids = torch.zeros((len(rows), width), dtype=dtype)
    mask = torch.zeros((len(rows), width), dtype=torch.uint8)
    for i, r in enumerate(rows):
        if r:
            at = slice(width - len(r), width) if side == "left" else slice(0, len(r))
            ids[i, at] = torch.as_tensor(r, dtype=dtype)
            mask[i, at] = 1
    return ids, mask


CLEAN = ["ACGTACGTAC", "AC", "ACGTTTGACCATG", "", "GGGTTT"]


@pytest.mark.parametrize("side", ["left", "right"])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.int16])
@pytest.mark.parametrize("bad_rows", [
    {},                                                             # nothing refused: the backend's rows as they are
    {1: "AC GT"},                                                   # one short row refused
    {0: "ACGT ACGTACGTACGTACGTACGTACGT TTGA"},                      # a refused row wider than every row that stayed
    {0: "A C", 2: "ACG TT", 4: " "},                                # several, one of them all white space
    {0: "A C", 1: "C G", 2: "G T", 3: "T A", 4: "A A"},             # every row refused: the whole batch to the tokenizer
])
def test_rows_the_backend_names_are_spliced_from_the_tokenizer(side, dtype, bad_rows):
    tok, h = _helper(side)
    seqs = [bad_rows.get(i, s) for i, s in enumerate(CLEAN)]
    for min_width, pad_multiple in ((0, 1), (0, 8), (20, 1)):
        ids, mask = h._encode_bpe_rows(seqs, "cpu", dtype=dtype, min_width=min_width, pad_multiple=pad_multiple,
                                       host_ids=False)
        want_ids, want_mask = _expected(tok, seqs, side, dtype, min_width, pad_multiple)
        assert ids.dtype == dtype and mask.dtype == torch.uint8
        # the layouts agree up to all-padding columns on the padding side (a batch of clean rows
        # padded to a multiple stays that wide when a shorter refused row is spliced in)
        w = want_ids.shape[1]
        assert ids.shape[1] >= w
        if side == "left":
            assert torch.equal(ids[:, ids.shape[1] - w:], want_ids) and torch.equal(mask[:, ids.shape[1] - w:], want_mask)
            assert int(mask[:, :ids.shape[1] - w].sum()) == 0
        else:
            assert torch.equal(ids[:, :w], want_ids) and torch.equal(mask[:, :w], want_mask)
            assert int(mask[:, w:].sum()) == 0
    if bad_rows and len(bad_rows) < len(CLEAN):
        assert h.bpe_backend.calls[1] == [s for i, s in enumerate(seqs) if i not in bad_rows]    # the rest stayed with the backend


@pytest.mark.parametrize("side", ["left", "right"])
def test_any_other_backend_failure_sends_the_batch_to_the_tokenizer(side, caplog):
    tok, h = _helper(side, backend_fail=RuntimeError("engine gave up on row 3"))
    seqs = ["ACGTAC", "ACG T", "TTTT"]
    with caplog.at_level(logging.WARNING, logger=h.log.name):
        h.log.propagate = True
        ids, mask = h._encode_bpe_rows(seqs, "cpu", dtype=torch.int64, min_width=0, pad_multiple=1, host_ids=False)
    want_ids, want_mask = _expected(tok, seqs, side, torch.int64)
    assert torch.equal(ids, want_ids) and torch.equal(mask, want_mask)
    assert any("falling back to the tokenizer" in r.getMessage() for r in caplog.records)


def test_a_failure_on_the_clean_rows_after_a_refusal_still_ends_at_the_tokenizer():
    tok, h = _helper("right")
    first = {"done": False}
    inner = h.bpe_backend.padded_device

    def flaky(seqs, **kw):
        if first["done"]:
            raise RuntimeError("scratch too small")
        first["done"] = True
        return inner(seqs, **kw)

    h.bpe_backend.padded_device = flaky
    seqs = ["ACGT", "AC GT", "TTGA"]
    ids, mask = h._encode_bpe_rows(seqs, "cpu", dtype=torch.int32, min_width=0, pad_multiple=1, host_ids=False)
    want_ids, want_mask = _expected(tok, seqs, "right", torch.int32)
    assert torch.equal(ids, want_ids) and torch.equal(mask, want_mask)
