"""select_block_sizes: the chosen tiles minimise the priced work, and the metadata returned is the one
compute_mask_* gives for them.  CPU cases use compute_mask_slow underneath; the GPU case the HIP kernels."""
import pytest
import torch

from sparseattention_amd import compute_mask_slow, select_block_sizes
from sparseattention_amd.mask_utils import RELATIVE_COST_PER_ENTRY
from sparseattention_amd import workloads as W


def brute_cost(mask, BQ, BK, partial_cost):
    m = mask[0, 0]
    t = m.reshape(m.shape[0] // BQ, BQ, m.shape[1] // BK, BK).sum((1, 3))
    full = int((t == BQ * BK).sum())
    part = int(((t > 0) & (t < BQ * BK)).sum())
    return full, part, (full + partial_cost * part) * BQ * BK * RELATIVE_COST_PER_ENTRY.get(BQ, 1.0)


def test_block_aligned_mask_prefers_matching_tiles():
    # 128x128 blocks, every block either all set or all clear: 128-row tiles see no partial tile at any BK
    g = torch.Generator().manual_seed(3)
    blocks = torch.rand(8, 8, generator=g) < 0.5
    mask = blocks.repeat_interleave(128, 0).repeat_interleave(128, 1)[None, None]
    BQ, BK, md, report = select_block_sizes(mask)
    assert BQ == 128
    for bq, bk, full, part, cost in report:
        f, p, c = brute_cost(mask, bq, bk, 1.25)
        assert (full, part) == (f, p) and abs(cost - c) < 1e-6
    assert min(r[4] for r in report) == [r[4] for r in report if (r[0], r[1]) == (BQ, BK)][0]
    want = compute_mask_slow(mask, BQ, BK)
    assert torch.equal(md.unmasked_lens, want.unmasked_lens) and torch.equal(md.masked_lens, want.masked_lens)


def test_fine_grained_mask_prefers_small_tiles():
    # a band of width 48 around the diagonal: large tiles are almost all partial and execute far more entries
    S = 1024
    i = torch.arange(S)
    mask = ((i[:, None] - i[None, :]).abs() < 48)[None, None]
    BQ, BK, md, report = select_block_sizes(mask, candidates=((128, 128), (64, 32), (32, 32)), partial_cost=1.0)
    costs = {(r[0], r[1]): r[4] for r in report}
    assert (BQ, BK) == min(costs, key=costs.get)
    assert (BQ, BK) != (128, 128)


def test_candidates_that_do_not_divide_are_skipped():
    mask = torch.ones(1, 1, 96, 96, dtype=torch.bool)
    BQ, BK, md, report = select_block_sizes(mask, candidates=((128, 32), (64, 32), (32, 32), (96, 16)))
    assert [(r[0], r[1]) for r in report] == [(32, 32), (96, 16)]
    with pytest.raises(ValueError):
        select_block_sizes(mask, candidates=((128, 32),))


@pytest.mark.gpu
def test_gpu_selection_matches_cpu(gpu):
    S = 2048
    mask = W.document_mask(S, seed=5, device=gpu, lo=100, hi=600)[None, None]
    got = select_block_sizes(mask)
    want = select_block_sizes(mask.cpu())
    assert got[:2] == want[:2]
    assert [r[:4] for r in got[3]] == [r[:4] for r in want[3]]
    assert torch.equal(got[2].unmasked_lens.cpu(), want[2].unmasked_lens)
