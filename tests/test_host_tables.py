"""Host-side table builders of the product against the oracle's independent restatement."""
import numpy as np

from dnatok_amd import bpe_vocab, kmer_tables
from tests.support import hf_tokenizers as hf
from oracle import oracle as O
from tests import util


def test_kernel_vocab_matches_oracle():
    for which in ("4096", "32000"):
        cfg = util.tokenizer_json(which)
        merges = bpe_vocab.split_merges(cfg["model"]["merges"])
        kv = bpe_vocab.KernelVocab(merges)
        vocab, a, b, n = O.kernel_vocab_from_merges(O.merges_from_tokenizer_json(cfg))
        assert kv.id_to_token == vocab
        np.testing.assert_array_equal(kv.pair_a, a)
        np.testing.assert_array_equal(kv.pair_b, b)
        np.testing.assert_array_equal(kv.new_id, n)
        remap = kv.remap_to(cfg["model"]["vocab"], 0)
        np.testing.assert_array_equal(remap, util.bpe_oracle(which).remap)


def test_merges_txt_parsing(tmp_path):
    p = tmp_path / "merges.txt"
    p.write_text("#version: 0.2\nA C\n\n# comment\nAC G\nbroken\nG T extra\n")
    assert bpe_vocab.parse_merges_txt(str(p)) == [("A", "C"), ("AC", "G"), ("G", "T")]
    # the first line is skipped even when it is a merge (reference behaviour)
    p.write_text("A C\nAC G\n")
    assert bpe_vocab.parse_merges_txt(str(p)) == [("AC", "G")]


def test_kmer_tables_match_oracle():
    vocab = hf.kmer_vocab(6)
    t = kmer_tables.tables_from_vocab(vocab, 6, 0)
    o = util.kmer_oracle_tables()
    np.testing.assert_array_equal(t.kmer_lut, o.kmer_lut)
    np.testing.assert_array_equal(t.exp_len, o.exp_len)
    # same expansions, possibly at other offsets
    for c in np.nonzero(t.exp_len)[0][:500]:
        np.testing.assert_array_equal(t.exp_flat[t.exp_off[c]:t.exp_off[c] + t.exp_len[c]],
                                      o.exp_flat[o.exp_off[c]:o.exp_off[c] + o.exp_len[c]])
    for ch in "ACGTN":
        assert t.single[ord(ch)] == o.single[ord(ch)]


def test_kmer_tables_from_live_hf_tokenizer():
    tk = hf.build_kmer_tokenizer(3)

    def tok(batch):
        return [e.ids for e in tk.encode_batch(batch, add_special_tokens=False)]
    t = kmer_tables.tables_from_tokenize(tok, 3, 0)
    ref = kmer_tables.tables_from_vocab(hf.kmer_vocab(3), 3, 0)
    np.testing.assert_array_equal(t.kmer_lut, ref.kmer_lut)
    np.testing.assert_array_equal(t.exp_len, ref.exp_len)
    np.testing.assert_array_equal(t.exp_flat, ref.exp_flat)
    assert (t.kmer_lut >= 0).sum() == 64 and (t.exp_len == 3).sum() == 125 - 64
