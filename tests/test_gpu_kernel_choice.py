"""The forward's other kernel forms (sa_sparse_attention_fwd_kernel): SA_FWD_KERNEL_SHORT_LISTS (three workgroups per
compute unit, 32 keys per step) and SA_FWD_KERNEL_ROTATED_BY(G) (FULL entries walked from a start that depends on the
Q tile), against the same checkers as the default kernel: the C oracle and fp32 masked SDPA (test_attn.py:40), max-abs
<= 2e-2 on bf16/fp16 inputs; and against the default kernel within twice that."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from sparseattention_amd import (_native, causal_term, compute_mask_kernel, compute_mask_terms, sparse_attention,
                                 with_list_stats, workloads as W)

pytestmark = pytest.mark.gpu
TOL = 2e-2


def sdpa32(q, k, v, mask):
    out = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    return torch.nan_to_num(out, nan=0.0)  # rows that attend to nothing: 0 here, NaN there


def oracle_out(q, k, v, mask, BQ, BK):
    B, H, Sq, _ = q.shape
    m = mask.expand(B, H, Sq, k.shape[2]).cpu().numpy()
    return torch.from_numpy(oracle.forward(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), m,
                                           BQ, BK, p_round=1))


@pytest.mark.parametrize("BK", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_tile_widths_against_oracle_and_sdpa(gpu, BK, dtype):
    B, H, S, D = 2, 2, 1024, 128
    q, k, v = W.qkv(B, H, S, D, dtype, seed=BK, device=gpu)
    mask = W.random_block_mask(S, 32, 0.5, seed=BK + 1, device=gpu, partial_fraction=0.25)
    md = compute_mask_kernel(mask[None, None].expand(B, H, S, S), 128, BK, list_stats=True)
    assert md.list_stats is not None and md.list_stats[1] <= S // BK
    o = sparse_attention(q, k, v, mask, 128, BK, md, kernel="short")
    torch.cuda.synchronize()
    assert o.shape == q.shape and o.dtype == q.dtype and not torch.isnan(o).any()
    err = (o.float().cpu() - oracle_out(q, k, v, mask, 128, BK)).abs()
    assert err.max() <= TOL and err.mean() <= 1e-3, f"vs oracle: max {err.max()}, mean {err.mean()}"
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
    assert (o.float() - sparse_attention(q, k, v, mask, 128, BK, md, kernel="default").float()).abs().max() <= 2 * TOL


@pytest.mark.parametrize("kind", ["causal", "dense", "window", "documents", "one chunk", "empty tiles and dead rows"])
@pytest.mark.parametrize("BK", [16, 32, 64])
def test_mask_families(gpu, kind, BK):
    # lists of every length from 0 to the row of tiles (at BK = 16 and S = 4096: the 256 entries the kernel holds),
    # odd lengths (a last chunk with a missing entry at BK = 16), Q tiles with FULL entries only and PARTIAL only
    B, H, D = 1, 2, 128
    S = 4096 if kind in ("causal", "dense") and BK == 16 else 1024
    i = torch.arange(S, device=gpu)
    if kind == "causal":
        mask = W.causal_mask(S, gpu)
    elif kind == "dense":
        mask = torch.ones(S, S, dtype=torch.bool, device=gpu)
    elif kind == "window":
        mask = ((i[:, None] - i[None, :]).abs() < 40) | (i[None, :] < 48)
    elif kind == "documents":
        mask = W.document_mask(S, seed=3, device=gpu, lo=30, hi=300)
    elif kind == "one chunk":
        mask = (i[:, None] // 128 == i[None, :] // 128) & (i[None, :] % 128 < 16)
    else:
        mask = W.random_block_mask(S, 128, 0.8, seed=5, device=gpu, partial_fraction=0.3)
        mask[256:384] = False       # a Q tile with nothing to do
        mask[700] = False           # a dead row inside a live tile
        mask[5, :] = False
        mask[5, 900] = True         # a row whose only key comes late
    md = compute_mask_kernel(mask[None, None].expand(B, H, S, S), 128, BK, list_stats=True)
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=BK + len(kind), device=gpu)
    o, lse = sparse_attention(q, k, v, mask, 128, BK, md, kernel="short", return_lse=True)
    torch.cuda.synchronize()
    assert not torch.isnan(o).any()
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
    dead = ~mask.any(-1)
    assert (o[:, :, dead] == 0).all() and torch.isneginf(lse[:, :, dead]).all()
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double()) / math.sqrt(D)
    want_lse = torch.logsumexp(s.masked_fill(~mask, float("-inf")), -1)
    assert (lse.double()[:, :, ~dead] - want_lse[:, :, ~dead]).abs().max() <= 6e-3
    # o does not depend on whether the lse is asked for
    assert torch.equal(o, sparse_attention(q, k, v, mask, 128, BK, md, kernel="short"))


def test_storage_orders_planes_and_formula_masks(gpu):
    B, H, S, D, BK = 2, 4, 1024, 128, 32
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn(3, B, S, H, D, generator=g).to(gpu, torch.bfloat16)  # [B,S,H,D] storage
    q, k, v = (t.permute(0, 2, 1, 3) for t in qkv)
    mask = W.random_block_mask(S, 64, 0.6, seed=12, device=gpu, batch=B, partial_fraction=0.2)  # per-batch planes
    me = mask.expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, BK, list_stats=True)
    o = sparse_attention(q, k, v, me, 128, BK, md, kernel="short")
    assert o.stride() == q.stride()
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
    # per-head planes as well
    mh = (torch.rand(B, H, S, S, generator=g) < 0.3).to(gpu)
    mdh = compute_mask_kernel(mh, 128, BK, list_stats=True)
    assert (sparse_attention(q, k, v, mh, 128, BK, mdh, kernel="short").float() - sdpa32(q, k, v, mh)).abs().max() <= TOL
    # no mask tensor at all: lists and packed tiles from the formula
    mdt = with_list_stats(compute_mask_terms([causal_term()], B, H, S, S, 128, BK, device=gpu))
    oc = sparse_attention(q, k, v, None, 128, BK, mdt, kernel="short")
    assert (oc.float() - sdpa32(q, k, v, W.causal_mask(S, gpu))).abs().max() <= TOL


def test_selection_and_refusals(gpu):
    B, H, S, D = 1, 2, 2048, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=1, device=gpu)
    sparse_mask = W.random_block_mask(S, 128, 0.9, seed=2, device=gpu)[None, None].expand(B, H, S, S)
    dense_mask = torch.ones(B, H, S, S, dtype=torch.bool, device=gpu)
    md_s = compute_mask_kernel(sparse_mask, 128, 32, list_stats=True)
    md_d = compute_mask_kernel(dense_mask, 128, 32, list_stats=True)
    assert md_d.list_stats == (64.0, 64) and 0 < md_s.list_stats[0] < 24
    # "auto" follows the statistics: the sparse mask runs the short-list kernel, the dense one the default kernel
    assert torch.equal(sparse_attention(q, k, v, sparse_mask, 128, 32, md_s), sparse_attention(q, k, v, sparse_mask, 128, 32, md_s, kernel="short"))
    assert torch.equal(sparse_attention(q, k, v, dense_mask, 128, 32, md_d), sparse_attention(q, k, v, dense_mask, 128, 32, md_d, kernel="default"))
    # without statistics nothing changes: the default kernel, and "short" is refused
    plain = compute_mask_kernel(sparse_mask, 128, 32)
    assert plain.list_stats is None
    assert torch.equal(sparse_attention(q, k, v, sparse_mask, 128, 32, plain), sparse_attention(q, k, v, sparse_mask, 128, 32, md_s, kernel="default"))
    with pytest.raises(ValueError, match="short"):
        sparse_attention(q, k, v, sparse_mask, 128, 32, plain, kernel="short")
    with pytest.raises(ValueError, match="short"):
        sparse_attention(q, k, v, sparse_mask, 64, 32, compute_mask_kernel(sparse_mask, 64, 32, list_stats=True), kernel="short")
    # a list longer than the kernel holds: the wrapper does not select it
    long = compute_mask_kernel(torch.ones(1, 1, 128, 16384, dtype=torch.bool, device=gpu), 128, 32, list_stats=True)
    assert long.list_stats == (512.0, 512)
    with pytest.raises(ValueError, match="short"):
        sparse_attention(q[:, :1, :128], torch.zeros(1, 1, 16384, D, device=gpu, dtype=q.dtype),
                         torch.zeros(1, 1, 16384, D, device=gpu, dtype=q.dtype), None, 128, 32, long, kernel="short")
    # the C entry point refuses what the kernel does not have
    lib = _native.load()
    st = _native.strides
    md = md_s
    o = torch.empty_like(q)

    def raw(packed, D_, BQ, kernel):
        return lib.sa_sparse_attention_fwd_kernel(
            q.data_ptr(), st(q.stride()), k.data_ptr(), st(k.stride()), v.data_ptr(), st(v.stride()), o.data_ptr(), st(o.stride()),
            sparse_mask.data_ptr(), st(sparse_mask.stride()), md.unmasked_kv_ids.data_ptr(), st(md.unmasked_kv_ids.stride()),
            md.unmasked_lens.data_ptr(), st(md.unmasked_lens.stride()), md.masked_kv_ids.data_ptr(), st(md.masked_kv_ids.stride()),
            md.masked_lens.data_ptr(), st(md.masked_lens.stride()), packed.data_ptr() if packed is not None else None,
            st(packed.stride()[:2]) if packed is not None else None, None, None, B, H, S, S, D_, BQ, 32, 0,
            D ** -0.5 / math.log(2), kernel, torch.cuda.current_stream().cuda_stream)

    assert raw(None, D, 128, 1) == _native.SA_ERR_UNSUPPORTED
    assert raw(md.packed_masks, D, 64, 1) == _native.SA_ERR_UNSUPPORTED
    assert raw(md.packed_masks, D, 128, 7) == _native.SA_ERR_INVALID_ARGUMENT
    assert raw(md.packed_masks, D, 128, 1) == 0
    torch.cuda.synchronize()
    assert torch.equal(o, sparse_attention(q, k, v, sparse_mask, 128, 32, md_s, kernel="short"))
    # kernel 0 through the same entry point is the default kernel
    assert raw(md.packed_masks, D, 128, 0) == 0
    torch.cuda.synchronize()
    assert torch.equal(o, sparse_attention(q, k, v, sparse_mask, 128, 32, md_s, kernel="default"))


def test_lists_cut_at_the_cap_stay_inside_their_tensors(gpu):
    # straight through the C ABI with counts above the 256 entries the kernel holds: it reads the first 256 entries
    # (FULL ones first) and nothing else, so the result is attention over those tiles
    B, H, S, D, BK = 1, 1, 8192, 128, 16
    nK = S // BK
    q, k, v = W.qkv(B, H, 128, D, torch.bfloat16, seed=9, device=gpu, Sk=S)
    mask = torch.ones(1, 1, 128, S, dtype=torch.bool, device=gpu)
    md = compute_mask_kernel(mask, 128, BK)
    lib = _native.load()
    st = _native.strides
    o = torch.full_like(q, float("nan"))
    rc = lib.sa_sparse_attention_fwd_kernel(
        q.data_ptr(), st(q.stride()), k.data_ptr(), st(k.stride()), v.data_ptr(), st(v.stride()), o.data_ptr(), st(o.stride()),
        None, None, md.unmasked_kv_ids.data_ptr(), st(md.unmasked_kv_ids.stride()),
        md.unmasked_lens.data_ptr(), st(md.unmasked_lens.stride()), md.masked_kv_ids.data_ptr(), st(md.masked_kv_ids.stride()),
        md.masked_lens.data_ptr(), st(md.masked_lens.stride()), md.packed_masks.data_ptr(), st(md.packed_masks.stride()[:2]),
        None, None, B, H, 128, S, D, 128, BK, 0, D ** -0.5 / math.log(2), 1, torch.cuda.current_stream().cuda_stream)
    _native.check(rc)
    torch.cuda.synchronize()
    assert nK == 512
    cut = mask.clone()
    cut[..., 256 * BK:] = False
    assert (o.float() - sdpa32(q, k, v, cut)).abs().max() <= TOL


@pytest.mark.parametrize("BQ,BK,D", [(128, 32, 128), (128, 16, 128), (128, 64, 128), (128, 128, 64), (64, 32, 64), (256, 32, 128)])
@pytest.mark.parametrize("group", [2, 8, 16, 64])
def test_rotated_walk_of_the_full_entries(gpu, BQ, BK, D, group):
    # a causal window (lists that slide), a prefix block and a dense stripe; bool mask and packed tiles; bf16
    B, H, S = 1, 3, 2048
    i = torch.arange(S, device=gpu)
    mask = ((i[:, None] >= i[None, :]) & (i[:, None] - i[None, :] < 700)) | (i[None, :] < 200) | (i[:, None] >= 1800)
    me = mask[None, None].expand(B, H, S, S)
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=group + BK, device=gpu)
    want = sdpa32(q, k, v, mask)
    for pack in (True, False):
        md = compute_mask_kernel(me, BQ, BK, pack_partial=pack)
        md.list_rotation = group
        o, lse = sparse_attention(q, k, v, me, BQ, BK, md, return_lse=True)
        torch.cuda.synchronize()
        assert (o.float() - want).abs().max() <= TOL
        assert torch.equal(o, sparse_attention(q, k, v, me, BQ, BK, md, kernel="rotated"))
        o_def, lse_def = sparse_attention(q, k, v, me, BQ, BK, md, kernel="default", return_lse=True)
        assert (o.float() - o_def.float()).abs().max() <= TOL and (lse - lse_def).abs().max() <= 6e-3
    # the rotation permutes FULL entries only: a mask without FULL tiles gives the default kernel's bits
    band = (i[:, None] - i[None, :]).abs() < 8
    mdb = compute_mask_kernel(band[None, None].expand(B, H, S, S), BQ, BK)
    assert int(mdb.unmasked_lens.sum()) == 0
    ob = sparse_attention(q, k, v, band, BQ, BK, mdb, kernel="default")
    mdb.list_rotation = group
    assert torch.equal(ob, sparse_attention(q, k, v, band, BQ, BK, mdb))


def test_rotation_hint_and_its_refusals(gpu):
    S = 4096
    i = torch.arange(S, device=gpu)
    window = ((i[:, None] >= i[None, :]) & (i[:, None] - i[None, :] < 1024))[None, None]
    assert compute_mask_kernel(window, 128, 32, list_stats=True).list_rotation == 16
    assert compute_mask_kernel(W.composed_mask(4 * S, device=gpu)[None, None], 128, 32, list_stats=True).list_rotation == 16
    assert compute_mask_kernel(W.causal_mask(S, gpu)[None, None], 128, 32, list_stats=True).list_rotation == 0
    assert compute_mask_kernel(W.document_mask(S, seed=0, device=gpu, lo=200, hi=900)[None, None], 128, 32, list_stats=True).list_rotation == 0
    assert compute_mask_kernel(W.random_block_mask(S, 128, 0.5, seed=1, device=gpu)[None, None], 128, 32, list_stats=True).list_rotation == 0
    assert compute_mask_kernel(window, 128, 32).list_rotation == 0  # nothing is read back unless asked for
    lib = _native.load()
    st = _native.strides
    B, H, D = 1, 1, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=3, device=gpu)
    md = compute_mask_kernel(window, 128, 32)
    o = torch.empty_like(q)

    def raw(kernel, dtype=0):
        return lib.sa_sparse_attention_fwd_kernel(
            q.data_ptr(), st(q.stride()), k.data_ptr(), st(k.stride()), v.data_ptr(), st(v.stride()), o.data_ptr(), st(o.stride()),
            window.data_ptr(), st(window.stride()), md.unmasked_kv_ids.data_ptr(), st(md.unmasked_kv_ids.stride()),
            md.unmasked_lens.data_ptr(), st(md.unmasked_lens.stride()), md.masked_kv_ids.data_ptr(), st(md.masked_kv_ids.stride()),
            md.masked_lens.data_ptr(), st(md.masked_lens.stride()), None, None, None, None, B, H, S, S, D, 128, 32, dtype,
            D ** -0.5 / math.log(2), kernel, torch.cuda.current_stream().cuda_stream)

    for bad in (_native.SA_FWD_KERNEL_ROTATED, _native.SA_FWD_KERNEL_ROTATED | (3 << 8), _native.SA_FWD_KERNEL_ROTATED | (128 << 8),
                _native.SA_FWD_KERNEL_DEFAULT | (8 << 8)):
        assert raw(bad) == _native.SA_ERR_INVALID_ARGUMENT
    assert raw(_native.SA_FWD_KERNEL_ROTATED | (8 << 8)) == 0
    torch.cuda.synchronize()
    assert raw(_native.SA_FWD_KERNEL_ROTATED | (8 << 8), dtype=_native.SA_DTYPE_FP32) == _native.SA_ERR_UNSUPPORTED
    assert (o.float() - sdpa32(q, k, v, window[0, 0])).abs().max() <= TOL
    # the Python wrapper refuses the request where no kernel can honour it, as it does for "short"
    with pytest.raises(ValueError, match="rotated"):
        sparse_attention(q.float(), k.float(), v.float(), window, 128, 32, md, kernel="rotated")
    with pytest.raises(ValueError, match="rotated"):
        sparse_attention(q, k, v, window, 128, 32, compute_mask_kernel(window, 128, 32, schedule="pairs"), kernel="rotated")
    with pytest.raises(ValueError, match="kernel must be"):
        sparse_attention(q, k, v, window, 128, 32, md, kernel="fast")
