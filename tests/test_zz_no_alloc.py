"""dnatok_bpe_encode_static, the entry point that allocates nothing (its work space is an array
inside the library's device image), against dnatok_bpe_encode on the same input: two calls in a
row through the C ABI, the second with a smaller batch, so that what the first call left in the
shared array must not leak into the second.  Collected last on purpose."""
import ctypes

import numpy as np
import pytest
import torch

from dnatok_amd import _lib, bpe_vocab, encoders
from tests import util
from tests.support import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _encode_both(enc, batch):
    L = _lib.lib()
    data = torch.from_numpy(batch.data).to(DEV)
    off = torch.from_numpy(batch.offsets).to(DEV)
    n, total, max_len = batch.n_seqs, int(batch.total), int(batch.lengths().max())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want_tok, want_len = enc.encode(data, off, max_len)                       # dnatok_bpe_encode
    tok = torch.full((max(total, 1),), -7, dtype=torch.int32, device=DEV)
    lengths = torch.full((n,), -7, dtype=torch.int32, device=DEV)
    print(f"dnatok_bpe_encode_static rows={n} total={total} max_len={max_len}", flush=True)
    _lib.check(L.dnatok_bpe_encode_static(enc._h, _ptr(data), _ptr(off), n, max_len, total, _ptr(tok),
                                          _ptr(lengths), stream), "dnatok_bpe_encode_static")
    torch.cuda.synchronize()
    want_len_h, len_h = want_len.cpu().numpy(), lengths.cpu().numpy()
    np.testing.assert_array_equal(len_h, want_len_h)
    want_h, tok_h = want_tok.cpu().numpy(), tok.cpu().numpy()
    for i in range(n):
        lo = int(batch.offsets[i])
        np.testing.assert_array_equal(tok_h[lo:lo + len_h[i]], want_h[lo:lo + len_h[i]], err_msg=f"row {i}")
    return [tok_h[int(batch.offsets[i]):int(batch.offsets[i]) + len_h[i]] for i in range(n)]


@pytest.mark.parametrize("which", ["4096", "32000"])
def test_static_entry_point_equals_the_one_with_caller_scratch(which):
    cfg = util.tokenizer_json(which)
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    remap = kv.remap_to(cfg["model"]["vocab"], cfg["model"]["vocab"]["[UNK]"])
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv), out_remap=remap)
    bo = util.bpe_oracle(which)
    # first call: ragged rows, chunked long rows, and rows that no seam joins (whole-row fallback)
    first = wl.config5_ragged(300, seed=41).strings() + ["A" * 30000, "ACGTC" * 3000, "ACGT"]
    big = util.batch_from_strings(first)
    rows = _encode_both(enc, big)
    for r, e in zip(rows, bo.encode_batch(big.data, big.offsets)):
        np.testing.assert_array_equal(r, e)
    # second call, smaller, straight after: fewer rows, fewer chunks, one fallback row
    second = wl.config5_ragged(40, seed=42).strings() + ["AC" * 5000, "", "N"]
    small = util.batch_from_strings(second)
    rows = _encode_both(enc, small)
    for r, e in zip(rows, bo.encode_batch(small.data, small.offsets)):
        np.testing.assert_array_equal(r, e)
    # third: short rows only (no work list at all)
    tiny = wl.config3_bpe4096(64, 1024, seed=5)
    _encode_both(enc, tiny)


def test_static_entry_point_refuses_what_its_buffer_cannot_hold():
    L = _lib.lib()
    cap = int(L.dnatok_bpe_static_scratch_bytes())
    assert cap == 32 << 20
    cfg = util.tokenizer_json("4096")
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv))
    # sizes alone decide (nothing is launched): 64 Mbases of 100 kb rows need far more chunk space
    n, length = 640, 100_000
    assert int(L.dnatok_bpe_scratch_bytes(enc._h, n, length, n * length)) > cap
    off = torch.arange(n + 1, dtype=torch.int64, device=DEV) * length
    data = torch.full((n * length,), ord("A"), dtype=torch.uint8, device=DEV)      # real sizes all the same
    tok = torch.empty(n * length, dtype=torch.int32, device=DEV)
    lengths = torch.empty(n, dtype=torch.int32, device=DEV)
    rc = L.dnatok_bpe_encode_static(enc._h, _ptr(data), _ptr(off), n, length, n * length, _ptr(tok), _ptr(lengths),
                                    None)
    torch.cuda.synchronize()
    assert rc == -3 and b"built-in buffer" in L.dnatok_last_error()


def test_static_entry_point_replayed_from_a_graph():
    """The callers this entry point is for capture it into a HIP graph.  After one eager call of
    the same shape class (the first call of a kernel form sets its attributes and asks the runtime
    how many workgroups fit, which a capture does not allow), the call is captured and replayed
    with other input in the same buffers; every replay must give what an eager call gives, with
    eager calls of another shape (they share the one work buffer) between the replays."""
    L = _lib.lib()
    cfg = util.tokenizer_json("4096")
    kv = bpe_vocab.KernelVocab(bpe_vocab.split_merges(cfg["model"]["merges"]))
    remap = kv.remap_to(cfg["model"]["vocab"], cfg["model"]["vocab"]["[UNK]"])
    enc = encoders.BpeEncoder(kv.pair_a, kv.pair_b, kv.new_id, len(kv), out_remap=remap)
    bo = util.bpe_oracle("4096")
    n, length = 96, 3000                                           # rows cut into chunks: work list, seams, gather
    batches = [wl.config3_bpe4096(n, length, seed=70 + i) for i in range(3)]
    data = torch.empty(n * length, dtype=torch.uint8, device=DEV)
    off = torch.from_numpy(batches[0].offsets).to(DEV)
    tok = torch.empty(n * length, dtype=torch.int32, device=DEV)
    lengths = torch.empty(n, dtype=torch.int32, device=DEV)
    side = torch.cuda.Stream()

    def call():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        _lib.check(L.dnatok_bpe_encode_static(enc._h, _ptr(data), _ptr(off), n, length, n * length, _ptr(tok),
                                              _ptr(lengths), stream), "dnatok_bpe_encode_static")

    data.copy_(torch.from_numpy(batches[0].data))
    print(f"dnatok_bpe_encode_static in a graph rows={n} length={length}", flush=True)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        call()                                                     # the eager call of this shape, on the capture's stream
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=side):
            call()
    other = util.batch_from_strings(wl.config5_ragged(50, seed=9).strings())
    for b in batches:
        data.copy_(torch.from_numpy(b.data))
        tok.fill_(-1)
        lengths.fill_(-1)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        ln, flat = lengths.cpu().numpy(), tok.cpu().numpy()
        for i, e in enumerate(bo.encode_batch(b.data, b.offsets)):
            np.testing.assert_array_equal(flat[i * length:i * length + ln[i]], np.asarray(e), err_msg=f"replayed row {i}")
        _encode_both(enc, other)                                   # eager work on the shared buffer in between
