"""Bit-packed PARTIAL tiles on the GPU: sa_mask_pack_partial against the oracle, bit for bit, and the forward fed
from the packed bits against the forward fed from the bool mask, which must agree bit for bit as well."""
import numpy as np
import pytest
import torch

import oracle
from sparseattention_amd import MaskMetadata, _native, compute_mask_kernel, sparse_attention, workloads as W

pytestmark = pytest.mark.gpu


def check_packed(mask, BQ, BK):
    md = compute_mask_kernel(mask, BQ, BK, pack_partial=True)
    torch.cuda.synchronize()
    m = mask.cpu().numpy()
    meta = oracle.classify(m, BQ, BK)
    want = oracle.pack_partial(m, BQ, BK, meta)
    got = md.packed_masks.cpu().numpy()
    assert got.shape == want.shape and got.dtype == np.uint8
    pos = np.arange(want.shape[3]) < meta.masked_lens[..., None]
    assert pos.any()
    assert np.array_equal(got[pos], want[pos])
    return md


@pytest.mark.parametrize("BQ,BK", [(128, 32), (32, 16), (64, 64), (256, 128), (128, 8), (48, 24), (16, 1024)])
def test_pack_matches_oracle_tile_shapes(gpu, BQ, BK):
    S = 3072 if BK == 1024 or BQ == 48 else 1024
    mask = W.random_block_mask(S, 64, 0.4, seed=BQ + BK, device=gpu, partial_fraction=0.3)[None, None]
    check_packed(mask, BQ, BK)


def test_pack_planes_strides_and_odd_bytes(gpu):
    g = torch.Generator().manual_seed(3)
    raw = torch.randint(0, 256, (2, 3, 256, 320), generator=g, dtype=torch.uint8)
    raw[torch.rand(raw.shape, generator=g) < 0.7] = 0
    mask = raw.to(gpu).view(torch.bool)  # bytes other than 0/1 behind a bool view
    md = check_packed(mask, 64, 32)
    assert md.packed_masks.stride(0) != 0 and md.packed_masks.stride(1) != 0
    # head-broadcast, per-batch planes
    mb = mask[:, :1].expand(2, 3, 256, 320)
    md = check_packed(mb, 64, 32)
    assert md.packed_masks.stride(1) == 0 and md.packed_masks.stride(0) != 0
    # key stride != 1 and a misaligned base take the byte-wise loads
    mt = mask.transpose(2, 3).contiguous().transpose(2, 3)
    assert mt.stride(3) != 1
    check_packed(mt, 64, 32)
    check_packed(mask[..., 1:, 8:], 51, 8)


def test_pack_untouched_slots_and_default(gpu):
    S = 512
    mask = W.causal_mask(S, gpu)[None, None].expand(2, 2, S, S)
    lib = _native.load()
    md = compute_mask_kernel(mask, 128, 32, pack_partial=False)
    assert md.packed_masks is None
    assert compute_mask_kernel(mask, 128, 32).packed_masks is not None      # default: BLOCK_K % 8 == 0
    assert compute_mask_kernel(mask, 128, 4).packed_masks is None
    packed = torch.full((1, 1, 4, 16, 512), 0x5A, dtype=torch.uint8, device=gpu)
    S_ = _native.strides
    rc = lib.sa_mask_pack_partial(mask.data_ptr(), S_(mask.stride()), 2, 2, S, S, 128, 32,
                                  md.masked_kv_ids.data_ptr(), S_(md.masked_kv_ids.stride()),
                                  md.masked_lens.data_ptr(), S_(md.masked_lens.stride()),
                                  packed.data_ptr(), S_((0, 0)), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert (packed[0, 0, :, 4:] == 0x5A).all() and not (packed[0, 0, :, :4] == 0x5A).all()
    words = packed[0, 0].cpu().numpy().view("<u4")
    assert int(words[2, 1, 40]) == (1 << 9) - 1  # Q tile 2, slot 1 (keys 288..319), row 40 = query 296: 9 keys


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("BQ", [32, 64, 128, 256])
@pytest.mark.parametrize("BK", [16, 32, 64, 128])
def test_forward_packed_equals_forward_from_mask(gpu, D, BQ, BK):
    B, H, S = 2, 2, 1024
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=BQ + BK + D, device=gpu)
    mask = W.random_block_mask(S, 32, 0.5, seed=BQ * BK + 1, device=gpu, partial_fraction=0.3, batch=B)
    me = mask.expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, BK, pack_partial=True)
    plain = MaskMetadata(md.unmasked_kv_ids, md.unmasked_lens, md.masked_kv_ids, md.masked_lens)
    o_mask = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=plain)
    o_pack = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md)
    # the packed route must not read the bool mask: hand it a mask of the right shape with the wrong content
    o_blind = sparse_attention(q, k, v, torch.zeros_like(me), BQ, BK, mask_metadata=md)
    torch.cuda.synchronize()
    assert not torch.isnan(o_pack).any()
    assert torch.equal(o_mask, o_pack), f"max diff {(o_mask.float() - o_pack.float()).abs().max()}"
    assert torch.equal(o_pack, o_blind)


def test_forward_packed_fp16_and_odd_list_lengths(gpu):
    # fp16, and Q tiles whose lists end in a half-filled chunk (causal at 128x32 never does; this mask does)
    B, H, S, D = 1, 3, 1024, 128
    q, k, v = W.qkv(B, H, S, D, torch.float16, seed=5, device=gpu)
    i = torch.arange(S, device=gpu)
    mask = ((i[:, None] - i[None, :]).abs() < 40) | (i[None, :] < 32)
    me = mask[None, None].expand(B, H, S, S)
    for BQ, BK in ((128, 32), (64, 16), (128, 16)):
        md = compute_mask_kernel(me, BQ, BK, pack_partial=True)
        assert ((md.unmasked_lens + md.masked_lens) % (64 // BK) != 0).any()
        plain = MaskMetadata(md.unmasked_kv_ids, md.unmasked_lens, md.masked_kv_ids, md.masked_lens)
        a = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=plain)
        b = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md)
        assert torch.equal(a, b)
        ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
        assert (b.float() - ref).abs().max() <= 2e-3


def test_forward_packed_headline_shape_causal(gpu):
    B, H, S, D = 2, 4, 4096, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=9, device=gpu)
    me = W.causal_mask(S, gpu)[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, 32)
    assert md.packed_masks is not None and md.packed_masks.stride(0) == 0
    plain = MaskMetadata(md.unmasked_kv_ids, md.unmasked_lens, md.masked_kv_ids, md.masked_lens)
    a = sparse_attention(q, k, v, me, 128, 32, mask_metadata=plain)
    b = sparse_attention(q, k, v, me, 128, 32, mask_metadata=md)
    assert torch.equal(a, b)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert (b.float() - ref.float()).abs().max() <= 2e-2


def test_packed_argument_errors(gpu):
    S = 256
    mask = W.causal_mask(S, gpu)[None, None]
    md = compute_mask_kernel(mask, 64, 32)
    q, k, v = W.qkv(1, 1, S, 64, torch.bfloat16, seed=0, device=gpu)
    bad = MaskMetadata(md.unmasked_kv_ids, md.unmasked_lens, md.masked_kv_ids, md.masked_lens, md.packed_masks[..., :128])
    with pytest.raises(ValueError):
        sparse_attention(q, k, v, mask, 64, 32, mask_metadata=bad)
    with pytest.raises(ValueError):
        compute_mask_kernel(mask, 64, 4, pack_partial=True)
