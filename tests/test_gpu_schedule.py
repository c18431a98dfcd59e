"""Persistent workgroups: the schedule holds every Q tile exactly once with its counts, and the forward that
follows it gives the same bits as the forward that launches one workgroup per Q tile."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from sparseattention_amd import MaskMetadata, _native, compute_mask_kernel, sparse_attention, workloads as W

pytestmark = pytest.mark.gpu


def check_schedule(md, B, H, nQ):
    s = md.schedule.cpu().numpy()
    G, R1, four = s.shape
    assert four == 4 and G % 8 == 0
    fl = md.unmasked_lens.cpu().numpy()
    pl = md.masked_lens.cpu().numpy()
    seen = np.zeros((B, H, nQ), np.int32)
    loads = []
    for g in range(G):
        n = s[g, 0, 0]
        assert 0 <= n <= R1 - 1
        load = 0
        for e in s[g, 1:1 + n]:
            b, h, qt = int(e[0]) >> 16, int(e[0]) & 0xffff, int(e[1])
            assert 0 <= b < B and 0 <= h < H and 0 <= qt < nQ
            seen[b, h, qt] += 1
            assert e[2] == fl[b, h, qt] and e[3] == pl[b, h, qt]
            load += int(e[2]) + int(e[3])
        loads.append(load)
    assert (seen == 1).all(), "every Q tile must be scheduled exactly once"
    return np.array(loads), s


def without(md, packed=True, schedule="persistent"):
    return MaskMetadata(md.unmasked_kv_ids, md.unmasked_lens, md.masked_kv_ids, md.masked_lens,
                        md.packed_masks if packed else None, md.schedule if schedule else None)


def test_schedule_covers_every_tile_and_balances_causal(gpu):
    B, H, S = 8, 32, 4096
    me = W.causal_mask(S, gpu)[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, 32, schedule="persistent")
    assert md.schedule is not None and md.schedule.dtype == torch.int32
    loads, s = check_schedule(md, B, H, S // 128)
    # causal: tile qt has 4qt+4 entries; pairing heavy with light tiles keeps every workgroup within one tile
    assert loads.max() - loads.min() <= 132, (loads.min(), loads.max())
    # workgroups 8j + x stay inside the x-th eighth of the planes
    for g in (0, 1, 7, 8, 509):
        n = s[g, 0, 0]
        bh = (s[g, 1:1 + n, 0] >> 16) * H + (s[g, 1:1 + n, 0] & 0xffff)
        assert bh.min() >= (g % 8) * 32 and bh.max() < (g % 8 + 1) * 32


@pytest.mark.parametrize("mode", ["persistent", "pairs"])
@pytest.mark.parametrize("B,H,S,BQ,BK", [(1, 1, 256, 128, 32), (1, 3, 1024, 64, 16), (3, 5, 1024, 32, 64),
                                          (2, 7, 2048, 128, 128), (1, 2, 8192, 128, 32), (1, 1, 384, 128, 32)])
def test_schedule_odd_shapes(gpu, B, H, S, BQ, BK, mode):
    mask = W.random_block_mask(S, 64, 0.6, seed=S + BQ, device=gpu, batch=B)
    md = compute_mask_kernel(mask.expand(B, H, S, S), BQ, BK, schedule=mode)
    check_schedule(md, B, H, S // BQ)
    if mode == "pairs":
        assert md.schedule.shape[1] == 3 and int(md.schedule[:, 0, 0].max()) <= 2


def test_pairs_carry_equal_loads_under_a_causal_mask(gpu):
    B, H, S = 2, 3, 4096
    me = W.causal_mask(S, gpu)[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, 32, schedule="pairs")
    loads, s = check_schedule(md, B, H, S // 128)
    used = loads[s[:, 0, 0] == 2]
    assert used.min() == used.max() == 132  # (4 qt + 4) + (4 (31 - qt) + 4)


def test_no_schedule_for_unsupported_tiles(gpu):
    S = 512
    me = W.causal_mask(S, gpu)[None, None]
    assert compute_mask_kernel(me, 128, 32).schedule is None  # opt-in
    with pytest.raises(ValueError):
        compute_mask_kernel(me, 256, 32, schedule="persistent")
    with pytest.raises(ValueError):
        compute_mask_kernel(me, 128, 8, schedule="persistent", pack_partial=False)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("BQ", [32, 64, 128])
@pytest.mark.parametrize("BK", [16, 32, 64, 128])
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("mode", ["persistent", "pairs"])
def test_scheduled_forward_equals_per_tile_forward(gpu, D, BQ, BK, packed, mode):
    B, H, S = 2, 3, 1024
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=BQ + BK + D, device=gpu)
    mask = W.random_block_mask(S, 32, 0.5, seed=BQ * BK + 2, device=gpu, partial_fraction=0.3, batch=B)
    # a few Q tiles without any entry: their rows must come out as zeros
    mask[0, 0, :BQ] = False
    mask[1, 0, S - 2 * BQ:S - BQ] = False
    me = mask.expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, BK, schedule=mode)
    assert md.schedule is not None
    a = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=without(md, packed, schedule=False))
    b = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=without(md, packed, schedule="persistent"))
    torch.cuda.synchronize()
    assert not torch.isnan(b).any()
    assert torch.equal(a, b), f"max diff {(a.float() - b.float()).abs().max()}"
    assert (b[0, :, :BQ] == 0).all()


def test_persistent_forward_many_tiles_per_workgroup(gpu):
    # 8192 Q tiles on 512 workgroups: 16 tiles each, causal, against torch's causal attention and the oracle plane 0
    B, H, S, D = 8, 32, 4096, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=21, device=gpu)
    me = W.causal_mask(S, gpu)[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, 32, schedule="persistent")
    o = sparse_attention(q, k, v, me, 128, 32, mask_metadata=md)
    o2 = sparse_attention(q, k, v, me, 128, 32, mask_metadata=without(md, True, False))
    assert torch.equal(o, o2)
    o3 = sparse_attention(q, k, v, me, 128, 32, mask_metadata=compute_mask_kernel(me, 128, 32, schedule="pairs"))
    assert torch.equal(o, o3)
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert (o.float() - ref.float()).abs().max() <= 2e-2


def test_persistent_forward_single_chunk_tiles_and_fp16(gpu):
    # lists of one or two entries: every tile is shorter than the look-ahead of the chunk pipeline
    B, H, S, D = 2, 4, 2048, 128
    q, k, v = W.qkv(B, H, S, D, torch.float16, seed=4, device=gpu)
    i = torch.arange(S, device=gpu)
    mask = (i[:, None] // 64 == i[None, :] // 64) & (i[None, :] <= i[:, None])  # 64-wide causal blocks on the diagonal
    me = mask[None, None].expand(B, H, S, S)
    for BQ, BK, mode in ((64, 64, "persistent"), (128, 32, "pairs"), (32, 16, "persistent"), (64, 128, "pairs")):
        md = compute_mask_kernel(me, BQ, BK, schedule=mode)
        a = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md)
        b = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=without(md, True, False))
        assert torch.equal(a, b), (BQ, BK)
        ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
        assert (a.float() - ref).abs().max() <= 2e-3, (BQ, BK)


def test_schedule_size_mismatch_falls_back(gpu):
    S = 512
    q, k, v = W.qkv(1, 2, S, 128, torch.bfloat16, seed=1, device=gpu)
    me = W.causal_mask(S, gpu)[None, None].expand(1, 2, S, S)
    md = compute_mask_kernel(me, 128, 32, schedule="persistent")
    wrong = without(md)
    wrong.schedule = md.schedule[:, :-1].contiguous() if md.schedule.shape[1] > 2 else torch.zeros(8, dtype=torch.int32, device=gpu)
    a = sparse_attention(q, k, v, me, 128, 32, mask_metadata=wrong)  # wrong size: one workgroup per tile
    b = sparse_attention(q, k, v, me, 128, 32, mask_metadata=md)
    assert torch.equal(a, b)
