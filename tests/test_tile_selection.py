"""select_block_sizes: the chosen tiles minimise the priced work, and the metadata returned is the one
compute_mask_* gives for them.  CPU cases use compute_mask_slow underneath; the GPU case the HIP kernels."""
import pytest
import torch

from sparseattention_amd import compute_mask_slow, select_block_sizes
from sparseattention_amd.mask_utils import entry_cost
from sparseattention_amd import workloads as W


def brute_cost(mask, BQ, BK, partial_cost):
    m = mask[0, 0]
    t = m.reshape(m.shape[0] // BQ, BQ, m.shape[1] // BK, BK).sum((1, 3))
    full = int((t == BQ * BK).sum())
    part = int(((t > 0) & (t < BQ * BK)).sum())
    return full, part, (full + partial_cost * part) * BQ * BK * entry_cost(BQ, BK)


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


# Kernel times of every tile candidate on two masks (ms; B=2 H=32 D=128 bf16 on MI355X), as the `tile_selection` leg of
# bench.py printed them: what the cost table of select_block_sizes was fitted to.  The clock is consulted there, not in
# this suite: a timing comparison inside the parity tests fails on a busy or power-limited device for reasons that are
# not parity.
RECORDED_KERNEL_MS = {
    "causal S=4096": {(128, 32): 0.2619, (128, 64): 0.2576, (128, 128): 0.2565, (64, 32): 0.3982, (64, 64): 0.3896,
                      (256, 32): 0.2922, (256, 64): 0.2853},
    "random blocks p=0.75 S=4096": {(128, 32): 0.183, (128, 64): 0.1764, (128, 128): 0.1813, (64, 32): 0.2615,
                                    (64, 64): 0.2525, (256, 32): 0.3274, (256, 64): 0.3137},
}


@pytest.mark.parametrize("kind", sorted(RECORDED_KERNEL_MS))
def test_pick_is_close_to_the_fastest_candidate_recorded(kind):
    # The cost model against recorded measurements: its pick is within 5 % of the fastest candidate, and it ranks the
    # 128-row candidates ahead of the 64- and 256-row ones as the measurements do.
    S = 4096
    mask = (W.causal_mask(S) if kind.startswith("causal") else W.random_block_mask(S, 128, 0.75, seed=75))[None, None]
    bq, bk, _, report = select_block_sizes(mask)
    times = RECORDED_KERNEL_MS[kind]
    assert {(r[0], r[1]) for r in report} == set(times)
    assert times[(bq, bk)] <= 1.05 * min(times.values())
    cost = {(r[0], r[1]): r[4] for r in report}
    for c128 in [c for c in times if c[0] == 128]:
        for other in [c for c in times if c[0] != 128]:
            assert (cost[c128] < cost[other]) == (times[c128] < times[other])


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["causal", "fine documents"])
def test_picked_tiles_run_and_match_sdpa(gpu, kind):
    # what select_block_sizes returns (tile sizes + metadata) goes straight into the forward
    import torch.nn.functional as F

    from sparseattention_amd import sparse_attention

    B, H, S, D = 1, 2, 2048, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=0, device=gpu)
    m = W.causal_mask(S, gpu) if kind == "causal" else W.document_mask(S, seed=2, device=gpu, lo=40, hi=300)
    me = m[None, None].expand(B, H, S, S)
    bq, bk, md, _ = select_block_sizes(me)
    o = sparse_attention(q, k, v, me, bq, bk, mask_metadata=md)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=m)
    assert (o.float() - want).abs().max() <= 2e-2


def _shifted_blocks(S, block, shift):
    """Block-diagonal mask whose blocks of `block` rows start `shift` rows after a multiple of `block`."""
    i = torch.arange(S)
    g = (i + block - shift) // block
    return (g[:, None] == g[None, :])[None, None]


def test_grid_origin_removes_partial_tiles_cpu():
    from sparseattention_amd import select_tiling

    mask = _shifted_blocks(1024, 128, 32)
    t = select_tiling(mask, candidates=((128, 32), (128, 64)), offsets=((0, 0), (96, 0), (96, 32), (32, 32)))
    assert (t.BLOCK_Q, t.q_offset) == (128, 96) and t.k_offset % 32 == 0
    costs = {r[:4]: r for r in t.report}
    # at the origin every block straddles two rows of tiles; with the grid moved by 96 rows none does
    assert costs[(128, 32, 0, 0)][5] > 0 and costs[(128, 32, 96, 0)][4] > 0
    assert costs[(128, 32, 96, 0)][6] < costs[(128, 32, 0, 0)][6]
    assert t.padded_mask.shape[-2:] == (1024 + 96 + 32, 1024)
    assert not t.padded_mask[0, 0, :96].any() and torch.equal(t.padded_mask[0, 0, 96:96 + 1024, :1024], mask[0, 0])
    # offsets that do not fit a candidate are skipped, and (0, 0) alone is select_block_sizes
    t0 = select_tiling(mask, candidates=((128, 32), (64, 64)))
    bq, bk, md, _ = select_block_sizes(mask, candidates=((128, 32), (64, 64)))
    assert (t0.BLOCK_Q, t0.BLOCK_K, t0.q_offset, t0.k_offset) == (bq, bk, 0, 0)
    assert torch.equal(t0.metadata.unmasked_lens, md.unmasked_lens)


@pytest.mark.gpu
def test_forward_on_a_moved_grid(gpu):
    import torch.nn.functional as F

    from sparseattention_amd import select_tiling, sparse_attention, sparse_attention_tiled

    B, H, S, D = 1, 2, 1024, 64
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=3, device=gpu)
    mask = _shifted_blocks(S, 128, 32).to(gpu).expand(B, H, S, S)
    t = select_tiling(mask, candidates=((128, 32), (128, 64)), offsets=((0, 0), (96, 0), (96, 32), (32, 32)))
    assert (t.q_offset, t.k_offset % 32) == (96, 0)
    o, lse = sparse_attention_tiled(q, k, v, t, return_lse=True)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    assert o.shape == q.shape and (o.float() - want).abs().max() <= 2e-2
    plain = sparse_attention(q, k, v, mask, 128, 32)
    assert (o.float() - plain.float()).abs().max() <= 2e-2
    s = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) / D ** 0.5
    assert (lse - torch.logsumexp(s.masked_fill(~mask, float("-inf")), -1)).abs().max() <= 6e-3
    # a tiling without offsets is sparse_attention itself
    t0 = select_tiling(mask, candidates=((128, 32),))
    assert torch.equal(sparse_attention_tiled(q, k, v, t0), plain)
