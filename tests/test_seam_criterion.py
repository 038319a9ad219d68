"""CPU check of the rule the BPE engine uses to join independently merged chunks of a long
row: a seam is accepted where two neighbouring chunk runs both have a token boundary and agree
on the token ending there and on the token starting there.  Whatever the chunk size and overlap,
an accepted set of seams must reproduce the tokenization of the whole row (a missing seam only
means the row is redone whole).  Tested with the oracle on random rule tables and on the
trained vocabularies."""
import random

import numpy as np

from tests.support import workloads as wl
from oracle import oracle as O
from tests import util


def tokens_with_pos(bo, row, lens):
    ids = bo.encode_row(row, remap=False)
    pos, p = np.zeros(len(ids), dtype=np.int64), 0
    for i, t in enumerate(ids):
        pos[i] = p
        p += lens[t]
    assert p == len(row)
    return ids, pos


def chunked_encode(bo, row, lens, core, overlap):
    """Returns the assembled token list, or None when some overlap holds no seam."""
    n = len(row)
    if n <= core + 2 * overlap:
        return bo.encode_row(row, remap=False).tolist()
    nc = -(-n // core)
    runs = []
    for k in range(nc):
        e0, e1 = max(0, k * core - overlap), min(n, (k + 1) * core + overlap)
        ids, pos = tokens_with_pos(bo, row[e0:e1], lens)
        start_to_tok = {int(p) + e0: int(t) for p, t in zip(pos, ids)}
        runs.append((e0, start_to_tok, sorted(start_to_tok)))
    seams = [0]
    for k in range(nc - 1):
        _, sa, pa = runs[k]
        eb0, sb, _ = runs[k + 1]
        found = None
        for i, j in zip(pa, pa[1:]):
            if i >= eb0 and sb.get(i) == sa[i] and sb.get(j) == sa[j]:
                found = j
                break
        if found is None:
            return None
        seams.append(found)
    seams.append(n)
    out = []
    for k in range(nc):
        _, s, ps = runs[k]
        out.extend(s[p] for p in ps if seams[k] <= p < seams[k + 1])
    return out


def test_seams_on_random_tables():
    accepted = 0
    for trial in range(400):
        rng = random.Random(trial)
        alpha = "ACGT"[:rng.choice([2, 3, 4])]
        toks, merges, seen, strings = list(alpha), [], set(), set(alpha)
        for _ in range(rng.randint(3, 60)):
            a, b = rng.choice(toks), rng.choice(toks)
            if (a, b) in seen or len(a + b) > 8 or (a + b) in strings:
                continue            # every product is new: rules only use earlier products
            seen.add((a, b)); merges.append((a, b)); strings.add(a + b); toks.append(a + b)
        bo = O.BpeOracle(merges)
        lens = np.array([len(s) for s in bo.vocab])
        for rep in range(3):
            n = rng.randint(40, 300)
            if rep == 0:
                s = "".join(rng.choice(alpha) for _ in range(n))
            else:
                unit = "".join(rng.choice(alpha) for _ in range(rng.randint(1, 5)))
                s = ("".join(rng.choice(alpha) for _ in range(n // 3)) + (unit * n)[:n // 3] +
                     "".join(rng.choice(alpha) for _ in range(n // 3)))
            row = np.frombuffer(s.encode(), dtype=np.uint8)
            got = chunked_encode(bo, row, lens, rng.choice([16, 24, 40]), rng.choice([4, 8, 12]))
            if got is not None:
                accepted += 1
                assert got == bo.encode_row(row, remap=False).tolist(), (trial, s, merges)
    assert accepted > 600


def test_seams_on_trained_vocabularies():
    for which, batch in (("4096", wl.config5_ragged(120, seed=11)), ("32000", wl.config4_bpe32000(2, 30000, seed=5))):
        bo = util.bpe_oracle(which)
        lens = np.array([len(s) for s in bo.vocab])
        n_long = 0
        for r in range(batch.n_seqs):
            row = batch.row(r)
            if len(row) <= 2048:
                continue
            n_long += 1
            got = chunked_encode(bo, row, lens, 1536, 256)       # the engine's chunk geometry
            assert got is not None and got == bo.encode_row(row, remap=False).tolist()
        assert n_long >= 2
