"""Masks given by terms (compute_mask_terms): the same lists and packed PARTIAL tiles, bit for bit, as the tensor path
gives for the materialised mask and as the oracle gives; forward and backward without any mask tensor."""
import numpy as np
import pytest
import torch

import oracle
from sparseattention_amd import (MaskTerm, _native, block_term, causal_term, compute_backward_metadata,
                                 compute_backward_metadata_terms, compute_mask_kernel, compute_mask_terms,
                                 materialize_mask_terms, sparse_attention, sparse_attention_backward, workloads as W)

pytestmark = pytest.mark.gpu


def docs(B, S, seed, device, lo=40, hi=300):
    g = torch.Generator().manual_seed(seed)
    out = torch.zeros(B, S, dtype=torch.int32)
    for b in range(B):
        pos, d = 0, 0
        while pos < S:
            n = int(torch.randint(lo, hi, (1,), generator=g))
            out[b, pos:pos + n] = d
            pos, d = pos + n, d + 1
    return out.to(device)


def same_metadata(got, want, BQ, BK, packed=True):
    assert torch.equal(got.unmasked_lens, want.unmasked_lens) and torch.equal(got.masked_lens, want.masked_lens)
    nK = got.unmasked_kv_ids.shape[-1]
    pos = torch.arange(nK, device=got.unmasked_lens.device)
    vf = pos < want.unmasked_lens[..., None]
    vp = pos < want.masked_lens[..., None]
    assert torch.equal(got.unmasked_kv_ids[vf], want.unmasked_kv_ids[vf])
    assert torch.equal(got.masked_kv_ids[vp], want.masked_kv_ids[vp])
    if packed:
        assert got.packed_masks.shape == want.packed_masks.shape
        assert torch.equal(got.packed_masks[vp], want.packed_masks[vp])


CASES = {
    "causal": lambda Sq, Sk: [causal_term(offset=Sk - Sq)],
    "window": lambda Sq, Sk: [causal_term(window=100, offset=Sk - Sq)],
    "window+prefix": lambda Sq, Sk: [causal_term(window=70), block_term((0, 96), (0, 96)), block_term(k_range=(0, 4))],
    "two-sided": lambda Sq, Sk: [MaskTerm(back=33, ahead=17, offset=5)],
    "documents": lambda Sq, Sk: [causal_term(offset=Sk - Sq, same_doc=True)],
    "documents+global": lambda Sq, Sk: [MaskTerm(same_doc=True), block_term(k_range=(0, 16)), block_term(q_range=(Sq - 8, Sq))],
}


@pytest.mark.parametrize("BQ,BK", [(128, 32), (64, 16), (128, 64), (256, 128), (32, 256), (16, 16)])
@pytest.mark.parametrize("case", list(CASES))
def test_lists_and_packed_tiles_match_the_tensor_path_and_the_oracle(gpu, case, BQ, BK):
    B, H, Sq, Sk = 2, 3, 512, 768
    terms = CASES[case](Sq, Sk)
    dq, dk = docs(B, Sq, 1, gpu), docs(B, Sk, 2, gpu)
    # the documents of the queries are those of the last Sq keys, so that causal + same_doc leaves every row a key
    dq = dk[:, Sk - Sq:].contiguous()
    uses_docs = any(t.same_doc for t in terms)
    md = compute_mask_terms(terms, B, H, Sq, Sk, BQ, BK, dq if uses_docs else None, dk if uses_docs else None, device=gpu)
    assert md.unmasked_kv_ids.shape == (B, H, Sq // BQ, Sk // BK) and md.unmasked_kv_ids.stride(1) == 0
    assert (md.unmasked_kv_ids.stride(0) == 0) == (not uses_docs)
    mask = materialize_mask_terms(terms, B, Sq, Sk, dq if uses_docs else None, dk if uses_docs else None, device=gpu)
    want = compute_mask_kernel(mask.expand(B, H, Sq, Sk), BQ, BK, pack_partial=True)
    same_metadata(md, want, BQ, BK)
    # and the oracle, from the encoded terms
    m_or = oracle.mask_from_terms([t.encode() for t in terms], B, Sq, Sk, dq.cpu().numpy(), dk.cpu().numpy())
    assert np.array_equal(m_or, mask.expand(B, 1, Sq, Sk)[:, 0].cpu().numpy())
    o_md = oracle.classify(np.ascontiguousarray(m_or[:, None]), BQ, BK)
    assert np.array_equal(md.unmasked_lens[:, 0].cpu().numpy(), o_md.unmasked_lens[:, 0])
    assert np.array_equal(md.masked_lens[:, 0].cpu().numpy(), o_md.masked_lens[:, 0])
    o_pk = oracle.pack_partial(np.ascontiguousarray(m_or[:, None]), BQ, BK, o_md)
    vp = np.arange(Sk // BK) < o_md.masked_lens[..., None]
    assert np.array_equal(md.packed_masks[:, :1].cpu().numpy()[vp], o_pk[vp])
    assert int(md.masked_lens.sum()) > 0
    # lists only
    md2 = compute_mask_terms(terms, B, H, Sq, Sk, BQ, BK, dq if uses_docs else None, dk if uses_docs else None,
                             device=gpu, pack_partial=False)
    assert md2.packed_masks is None
    same_metadata(md2, want, BQ, BK, packed=False)


def test_composed_long_context_mask_without_the_tensor(gpu):
    # (k <= q and q - k < 1024) or (q < 2048 and k < 2048) at S = 32768: a 1 GiB bool tensor that is never built
    S = 32768
    md = compute_mask_terms([causal_term(window=1024), block_term((0, 2048), (0, 2048))], 1, 32, S, S, 128, 32, device=gpu)
    assert (int(md.unmasked_lens[0, 0].sum()), int(md.masked_lens[0, 0].sum())) == (7744, 1920)
    q, k, v = W.qkv(1, 2, S, 128, torch.bfloat16, seed=3, device=gpu)
    md2 = compute_mask_terms([causal_term(window=1024), block_term((0, 2048), (0, 2048))], 1, 2, S, S, 128, 32, device=gpu)
    o = sparse_attention(q, k, v, None, 128, 32, mask_metadata=md2)
    # a strip of rows against the dense formula in fp32
    rows = slice(S - 256, S)
    strip = materialize_mask_terms([causal_term(window=1024, offset=S - 256)], 1, 256, S, device=gpu)
    want = torch.nn.functional.scaled_dot_product_attention(q[:, :, rows].float(), k.float(), v.float(), attn_mask=strip)
    assert float((o[:, :, rows].float() - want).abs().max()) <= 2e-2
    rows = slice(0, 256)
    strip = materialize_mask_terms([block_term(k_range=(0, 2048))], 1, 256, S, device=gpu)
    want = torch.nn.functional.scaled_dot_product_attention(q[:, :, rows].float(), k.float(), v.float(), attn_mask=strip)
    assert float((o[:, :, rows].float() - want).abs().max()) <= 2e-2


@pytest.mark.parametrize("D", [64, 128])
def test_forward_and_backward_without_a_mask_tensor(gpu, D):
    B, H, Sq, Sk = 2, 2, 384, 640
    q, _, _ = W.qkv(B, H, Sq, D, torch.bfloat16, seed=11, device=gpu)
    _, k, v = W.qkv(B, H, Sk, D, torch.bfloat16, seed=12, device=gpu)
    do = torch.randn(B, H, Sq, D, generator=torch.Generator().manual_seed(13)).to(gpu, torch.bfloat16)
    dk_ = docs(B, Sk, 5, gpu)
    dq_ = dk_[:, Sk - Sq:].contiguous()
    terms = [causal_term(window=200, offset=Sk - Sq, same_doc=True), block_term(k_range=(0, 8))]
    mask = materialize_mask_terms(terms, B, Sq, Sk, dq_, dk_, device=gpu).expand(B, H, Sq, Sk)
    for BQ, BK, sch in ((128, 32, None), (64, 64, "pairs"), (128, 128, None)):
        md = compute_mask_terms(terms, B, H, Sq, Sk, BQ, BK, dq_, dk_, schedule=sch)
        o, lse = sparse_attention(q, k, v, None, BQ, BK, mask_metadata=md, return_lse=True)
        o_t, lse_t = sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=compute_mask_kernel(mask, BQ, BK, schedule=sch),
                                      return_lse=True)
        assert torch.equal(o, o_t) and torch.equal(lse, lse_t)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    assert float((o.float() - want).abs().max()) <= 2e-2
    bmd = compute_backward_metadata_terms(terms, B, H, Sq, Sk, dq_, dk_)
    got = sparse_attention_backward(do, q, k, v, o, lse, None, bmd)
    ref = sparse_attention_backward(do, q, k, v, o, lse, mask, compute_backward_metadata(mask))
    assert all(torch.equal(a, b) for a, b in zip(got, ref))
    with pytest.raises(ValueError):
        sparse_attention(q, k, v, None, 128, 32)
    with pytest.raises(ValueError):
        sparse_attention(q, k, v, None, 128, 32, mask_metadata=compute_mask_terms(terms, B, H, Sq, Sk, 128, 32, dq_, dk_, pack_partial=False))


def test_argument_errors(gpu):
    lib = _native.load()
    with pytest.raises(ValueError):
        compute_mask_terms([], 1, 1, 128, 128, 128, 32, device=gpu)
    with pytest.raises(ValueError):
        compute_mask_terms([causal_term()] * 9, 1, 1, 128, 128, 128, 32, device=gpu)
    with pytest.raises(ValueError):
        compute_mask_terms([causal_term(same_doc=True)], 1, 1, 128, 128, 128, 32, device=gpu)
    with pytest.raises(AssertionError):
        compute_mask_terms([causal_term()], 1, 1, 100, 128, 128, 32, device=gpu)
    with pytest.raises(ValueError):
        compute_mask_terms([causal_term(same_doc=True)], 1, 1, 128, 128, 128, 32,
                           torch.zeros(128, dtype=torch.int64, device=gpu), torch.zeros(128, dtype=torch.int32, device=gpu))
    assert lib.sa_mask_terms_workspace_bytes(2, 256, 512, 128, 32) == 2 * 2 * 16
    assert lib.sa_mask_terms_workspace_bytes(0, 256, 512, 128, 32) == 0
    with pytest.raises(_native.SparseAttnError):  # BLOCK_K below 16
        compute_mask_terms([causal_term()], 1, 1, 128, 128, 128, 8, device=gpu)


@pytest.mark.parametrize("seed", range(48))
def test_seeded_random_terms(gpu, seed):
    # random flags and values (negative and huge offsets, ranges past the extents, empty ranges, unsorted documents),
    # random tilings and lengths: the decisions taken from the first and last row of a tile must agree with the
    # entry-by-entry tensor path everywhere
    g = torch.Generator().manual_seed(1000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    BQ, BK = [(128, 32), (64, 16), (32, 64), (16, 128), (256, 32), (128, 256)][seed % 6]
    B, H = ri(1, 4), ri(1, 3)
    Sq, Sk = BQ * ri(1, 5), max(BK, 64) * ri(1, 6)
    n_docs = ri(1, 6)
    if seed % 3 == 0:  # contiguous documents of random lengths
        dk = torch.sort(torch.randint(0, n_docs, (B, Sk), generator=g), dim=1).values.int()
        dq = torch.sort(torch.randint(0, n_docs, (B, Sq), generator=g), dim=1).values.int()
    elif seed % 3 == 1:  # blocks of 32 positions with arbitrary document numbers
        dk = torch.randint(0, n_docs, (B, (Sk + 31) // 32), generator=g).repeat_interleave(32, 1)[:, :Sk].int()
        dq = torch.randint(0, n_docs, (B, (Sq + 31) // 32), generator=g).repeat_interleave(32, 1)[:, :Sq].int()
    else:  # one layout for the whole batch
        dk = torch.sort(torch.randint(0, n_docs, (1, Sk), generator=g), dim=1).values.int()
        dq = torch.sort(torch.randint(0, n_docs, (1, Sq), generator=g), dim=1).values.int()
    dq, dk = dq.to(gpu), dk.to(gpu)
    big = [2 ** 31 - 1, -2 ** 31, 2 ** 30, -2 ** 30 - 5]
    val = lambda span: big[ri(0, 4)] if ri(0, 12) == 0 else ri(-span, span + 1)
    terms = []
    for _ in range(ri(1, 5)):
        rng = lambda S: tuple(sorted((ri(-20, S + 20), ri(-20, S + 20)))) if ri(0, 3) else (ri(0, S), ri(0, S))
        terms.append(MaskTerm(back=val(Sk) if ri(0, 2) else None, ahead=val(Sk // 2) if ri(0, 2) else None,
                              offset=val(Sk) if ri(0, 2) else 0, q_range=rng(Sq) if ri(0, 3) == 0 else None,
                              k_range=rng(Sk) if ri(0, 3) == 0 else None, same_doc=ri(0, 3) == 0))
    md = compute_mask_terms(terms, B, H, Sq, Sk, BQ, BK, dq, dk)
    mask = materialize_mask_terms(terms, B, Sq, Sk, dq, dk, device=gpu)
    want = compute_mask_kernel(mask.expand(B, H, Sq, Sk), BQ, BK, pack_partial=True)
    same_metadata(md, want, BQ, BK)
    m_or = oracle.mask_from_terms([t.encode() for t in terms], B, Sq, Sk, dq.cpu().numpy(), dk.cpu().numpy())
    assert np.array_equal(m_or, mask.expand(B, 1, Sq, Sk)[:, 0].cpu().numpy())
