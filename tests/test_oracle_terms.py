"""Pins of the masks given by terms: the oracle's restatement (oracle.mask_from_terms) against numpy's triangles,
a loop over single entries, and the tile totals the reference's mask semantics fix for known masks; the product's
host-side helpers (MaskTerm.encode / transposed, materialize_mask_terms) against the oracle."""
import numpy as np
import pytest
import torch

import oracle
from sparseattention_amd import MaskTerm, block_term, causal_term, materialize_mask_terms

BACK, AHEAD, QR, KR, DOC = 1, 2, 4, 8, 16


def test_causal_and_windows_are_numpy_triangles():
    S = 97
    causal = oracle.mask_from_terms([[AHEAD, 0, 0, 1, 0, 0, 0, 0]], 1, S, S)[0]
    assert np.array_equal(causal, np.tril(np.ones((S, S), bool)))
    for w in (1, 5, 64, 200):
        got = oracle.mask_from_terms([[BACK | AHEAD, 0, w, 1, 0, 0, 0, 0]], 1, S, S)[0]
        assert np.array_equal(got, np.tril(np.ones((S, S), bool)) & ~np.tril(np.ones((S, S), bool), -w)), w
    # two-sided window: |q - k| < 3
    got = oracle.mask_from_terms([[BACK | AHEAD, 0, 3, 3, 0, 0, 0, 0]], 1, S, S)[0]
    i = np.arange(S)
    assert np.array_equal(got, np.abs(i[:, None] - i[None, :]) < 3)
    # Sq != Sk: offset Sk - Sq lets the last query see every key and the first one Sk - Sq + 1 keys
    Sq, Sk = 40, 100
    got = oracle.mask_from_terms([[AHEAD, Sk - Sq, 0, 1, 0, 0, 0, 0]], 1, Sq, Sk)[0]
    assert got[-1].all() and got[0].sum() == Sk - Sq + 1
    assert np.array_equal(got, np.tril(np.ones((Sq, Sk), bool), Sk - Sq))


def test_entry_by_entry_loop_with_documents_ranges_and_several_terms():
    rng = np.random.default_rng(3)
    B, Sq, Sk = 2, 23, 31
    doc_q = np.sort(rng.integers(0, 4, size=(B, Sq)), axis=1).astype(np.int32)
    doc_k = np.sort(rng.integers(0, 4, size=(B, Sk)), axis=1).astype(np.int32)
    terms = [[AHEAD | DOC, 3, 0, 1, 0, 0, 0, 0], [QR | KR, 0, 0, 0, 2, 9, 20, 31], [BACK | KR, -2, 4, 0, 0, 0, 0, 6]]
    got = oracle.mask_from_terms(terms, B, Sq, Sk, doc_q, doc_k)
    for b in range(B):
        for q in range(Sq):
            for k in range(Sk):
                t0 = (k - (q + 3) < 1) and doc_q[b, q] == doc_k[b, k]
                t1 = 2 <= q < 9 and 20 <= k < 31
                t2 = ((q - 2) - k < 4) and 0 <= k < 6
                assert got[b, q, k] == (t0 or t1 or t2), (b, q, k)
    # a strip of rows is the same rows of the whole
    assert np.array_equal(oracle.mask_from_terms(terms, B, Sq, Sk, doc_q, doc_k, q_rows=(5, 17)), got[:, 5:17])


def test_tile_totals_of_the_composed_long_context_mask():
    # (k <= q and q - k < 1024) or (q < 2048 and k < 2048) at S = 32768, tiles 128 x 32: 7744 FULL and 1920 PARTIAL
    # tiles, counted from the geometry of the band and the square when the workloads were laid down
    S, BQ, BK = 32768, 128, 32
    terms = [[BACK | AHEAD, 0, 1024, 1, 0, 0, 0, 0], [QR | KR, 0, 0, 0, 0, 2048, 0, 2048]]
    full = part = 0
    for i in range(S // BQ):
        strip = oracle.mask_from_terms(terms, 1, S, S, q_rows=(i * BQ, (i + 1) * BQ))
        md = oracle.classify_numpy(strip[None], BQ, BK)
        full += int(md.unmasked_lens.sum())
        part += int(md.masked_lens.sum())
    assert (full, part) == (7744, 1920)


def test_encode_and_transposed_against_the_oracle():
    rng = np.random.default_rng(11)
    B, Sq, Sk = 2, 48, 80
    doc_q = np.sort(rng.integers(0, 5, size=(B, Sq)), axis=1).astype(np.int32)
    doc_k = np.sort(rng.integers(0, 5, size=(B, Sk)), axis=1).astype(np.int32)
    terms = [causal_term(window=20, offset=Sk - Sq, same_doc=True), block_term((0, 10), (60, 80)),
             MaskTerm(back=7, ahead=3, offset=5), block_term(k_range=(0, 2)), MaskTerm(ahead=-4, q_range=(30, 48))]
    assert causal_term().encode() == [AHEAD, 0, 0, 1, 0, 0, 0, 0]
    assert causal_term(window=9, offset=2, same_doc=True).encode() == [BACK | AHEAD | DOC, 2, 9, 1, 0, 0, 0, 0]
    assert block_term((1, 2), (3, 4)).encode() == [QR | KR, 0, 0, 0, 1, 2, 3, 4]
    enc = [t.encode() for t in terms]
    want = oracle.mask_from_terms(enc, B, Sq, Sk, doc_q, doc_k)
    got = materialize_mask_terms(terms, B, Sq, Sk, torch.from_numpy(doc_q), torch.from_numpy(doc_k))
    assert got.shape == (B, 1, Sq, Sk) and np.array_equal(got[:, 0].numpy(), want)
    # keys as rows: transposed terms with the documents swapped give the transposed mask
    enc_t = [t.transposed().encode() for t in terms]
    assert np.array_equal(oracle.mask_from_terms(enc_t, B, Sk, Sq, doc_k, doc_q), want.transpose(0, 2, 1))
    assert all(t.transposed().transposed() == t for t in terms)
    # without documents the mask has one plane
    assert materialize_mask_terms([causal_term()], 3, 8, 8).shape == (1, 1, 8, 8)
    with pytest.raises(ValueError):
        materialize_mask_terms([causal_term(same_doc=True)], 1, 8, 8)
