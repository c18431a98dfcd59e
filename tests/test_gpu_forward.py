"""Parity of the HIP block-sparse forward (sa_sparse_attention_fwd through the Python binding).

Tolerance: max-abs <= 2e-2 for bf16/fp16 inputs against masked attention evaluated in fp32 on the
same (already rounded) inputs - the oracle on small shapes, torch's masked SDPA (the reference's own
checker, test_attn.py:40) on all shapes."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import golden_io
import oracle
from sparseattention_amd import MaskMetadata, _native, compute_mask_kernel, sparse_attention, workloads as W

pytestmark = pytest.mark.gpu

TOL = 2e-2


def sdpa32(q, k, v, mask):
    return F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)


def oracle_out(q, k, v, mask, BQ, BK, p_round):
    B, H, Sq, _ = q.shape
    Sk = k.shape[2]
    m = mask.expand(B, H, Sq, Sk).cpu().numpy()
    return torch.from_numpy(oracle.forward(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), m,
                                           BQ, BK, p_round=p_round))


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("BQ", [32, 64, 128, 256])
@pytest.mark.parametrize("BK", [16, 32, 64, 128, 256])
def test_tile_shapes_against_oracle_and_sdpa(gpu, D, BQ, BK):
    B, H, S = 2, 2, 512
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=BQ + BK + D, device=gpu)
    mask = W.random_block_mask(S, 32, 0.5, seed=BQ * BK, device=gpu)
    o = sparse_attention(q, k, v, mask, BQ, BK)
    torch.cuda.synchronize()
    assert o.shape == q.shape and o.dtype == q.dtype and not torch.isnan(o).any()
    want = oracle_out(q, k, v, mask, BQ, BK, p_round=1)
    err = (o.float().cpu() - want).abs()
    assert err.max() <= TOL and err.mean() <= 1e-3, f"vs oracle: max {err.max()}, mean {err.mean()}"
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reference_style_check_bf16_sdpa(gpu, dtype):
    # the reference's own comparison: SDPA in the input dtype, atol 1e-2 / rtol 1e-4 (test_attn.py:40,51);
    # here held to the stated max-abs bound
    B, H, S, D = 2, 4, 1024, 128
    q, k, v = W.qkv(B, H, S, D, dtype, seed=11, device=gpu)
    mask = W.random_block_mask(S, 128, 0.5, seed=12, device=gpu, batch=B)
    me = mask.expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, 32)
    o = sparse_attention(q, k, v, me, 128, 32, mask_metadata=md)
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    assert (o.float() - ref.float()).abs().max() <= TOL
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= (TOL if dtype == torch.bfloat16 else 2e-3)


def test_all_true_mask_is_dense_attention(gpu):
    B, H, S, D = 1, 4, 1024, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=1, device=gpu)
    ones = torch.ones(S, S, dtype=torch.bool, device=gpu)
    o = sparse_attention(q, k, v, ones, 128, 32)
    dense = F.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert (o.float() - dense).abs().max() <= TOL


def test_one_hot_rows_copy_value_rows_exactly(gpu):
    B, H, S, D = 1, 2, 512, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=2, device=gpu)
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(5)).to(gpu)
    mask = torch.zeros(S, S, dtype=torch.bool, device=gpu)
    mask[torch.arange(S, device=gpu), perm] = True
    for BQ, BK in ((128, 32), (64, 64), (32, 16)):
        o = sparse_attention(q, k, v, mask, BQ, BK)
        assert torch.equal(o, v[:, :, perm]), f"tiles {BQ}x{BK}"


def test_identical_keys_give_uniform_average(gpu):
    B, H, S, D = 1, 1, 512, 64
    q, _, v = W.qkv(B, H, S, D, torch.bfloat16, seed=4, device=gpu)
    k = torch.full((B, H, S, D), 0.25, dtype=torch.bfloat16, device=gpu)
    mask = W.random_block_mask(S, 16, 0.5, seed=8, device=gpu)
    o = sparse_attention(q, k, v, mask, 128, 32)
    m = mask.double()
    want = (m @ v[0, 0].double()) / m.sum(-1, keepdim=True)
    assert (o[0, 0].double() - want).abs().max() <= TOL


def test_rows_masked_in_first_partial_tile_stay_finite(gpu):
    # document boundary inside a Q tile, no full tile before it (the reference's open hazard, :53)
    B, H, S, D = 1, 2, 256, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=6, device=gpu)
    doc = torch.tensor([0] * 40 + [1] * 100 + [2] * 116, device=gpu)
    idx = torch.arange(S, device=gpu)
    mask = (doc[:, None] == doc[None, :]) & (idx[None, :] <= idx[:, None])
    md = compute_mask_kernel(mask[None, None].expand(B, H, S, S), 128, 32)
    assert int(md.unmasked_lens[0, 0, 0]) == 0
    o = sparse_attention(q, k, v, mask, 128, 32)
    assert torch.isfinite(o).all()
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL


def test_rows_and_tiles_without_any_key_give_zero(gpu):
    B, H, S, D = 1, 1, 256, 64
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=7, device=gpu)
    mask = torch.ones(S, S, dtype=torch.bool, device=gpu)
    mask[5] = False
    mask[128:] = False
    o = sparse_attention(q, k, v, mask, 128, 32)
    assert (o[0, 0, 5] == 0).all() and (o[0, 0, 128:] == 0).all()
    live = [r for r in range(128) if r != 5]
    want = F.scaled_dot_product_attention(q[:, :, live].float(), k.float(), v.float())
    assert (o[0, 0, live].float() - want[0, 0]).abs().max() <= TOL


def test_metadata_given_or_computed_and_list_order(gpu):
    B, H, S, D = 2, 2, 512, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=8, device=gpu)
    mask = W.random_block_mask(S, 32, 0.3, seed=1, device=gpu)[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(mask, 128, 32)
    a = sparse_attention(q, k, v, mask, 128, 32, mask_metadata=md)
    b = sparse_attention(q, k, v, mask, 128, 32)
    assert torch.equal(a, b)
    # materialised (contiguous) metadata: same result
    mdc = MaskMetadata(*(t.contiguous() for t in (md.unmasked_kv_ids, md.unmasked_lens, md.masked_kv_ids, md.masked_lens)))
    assert torch.equal(a, sparse_attention(q, k, v, mask, 128, 32, mask_metadata=mdc))
    # reversed lists: another accumulation order, same mathematics
    rev_f, rev_p = mdc.unmasked_kv_ids.clone(), mdc.masked_kv_ids.clone()
    for ids, lens in ((rev_f, mdc.unmasked_lens), (rev_p, mdc.masked_lens)):
        for bb in range(B):
            for hh in range(H):
                for i in range(S // 128):
                    n = int(lens[bb, hh, i])
                    ids[bb, hh, i, :n] = ids[bb, hh, i, :n].flip(0)
    c = sparse_attention(q, k, v, mask, 128, 32, mask_metadata=MaskMetadata(rev_f, mdc.unmasked_lens, rev_p, mdc.masked_lens))
    assert (a.float() - c.float()).abs().max() <= TOL


def test_layouts_strides_and_cross_attention(gpu):
    B, H, Sq, Sk, D = 2, 4, 256, 768, 128
    g = torch.Generator(device=gpu).manual_seed(3)
    # [B,S,H,D] storage viewed as [B,H,S,D]: head stride D, sequence stride H*D
    q = torch.randn(B, Sq, H, D, generator=g, device=gpu).to(torch.bfloat16).transpose(1, 2)
    k = torch.randn(B, Sk, H, D, generator=g, device=gpu).to(torch.bfloat16).transpose(1, 2)
    v = torch.randn(B, Sk, H, D, generator=g, device=gpu).to(torch.bfloat16).transpose(1, 2)
    mask = (torch.rand(B, 1, Sq, Sk, generator=g, device=gpu) < 0.7)
    mask[:, :, :, :64] = True
    mask[:, :, 128:, 256:512] = False
    o = sparse_attention(q, k, v, mask, 64, 64)
    assert o.shape == q.shape and o.stride() == q.stride()
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
    # mask with a non-unit key stride (byte loads in the partial pass)
    mt = mask.transpose(-1, -2).contiguous().transpose(-1, -2)
    assert mt.stride(-1) != 1
    assert torch.equal(o, sparse_attention(q, k, v, mt, 64, 64))
    # a last dimension that is not contiguous is copied by the wrapper
    q2 = torch.randn(B, H, D, Sq, generator=g, device=gpu).to(torch.bfloat16).transpose(-1, -2)
    o2 = sparse_attention(q2, k, v, mask, 64, 64)
    assert (o2.float() - sdpa32(q2, k, v, mask)).abs().max() <= TOL
    # one K/V head for all query heads, as a view with head stride 0: no copy is made, same bits as from copies
    k1, v1 = k[:, :1].expand(B, H, Sk, D), v[:, :1].expand(B, H, Sk, D)
    assert k1.stride(1) == 0
    o3 = sparse_attention(q, k1, v1, mask, 64, 64)
    assert torch.equal(o3, sparse_attention(q, k1.contiguous(), v1.contiguous(), mask, 64, 64))
    assert (o3.float() - sdpa32(q, k1, v1, mask)).abs().max() <= TOL
    qd = q[:, :, :8]
    od = sparse_attention(qd, k1, v1, mask[:, :, :8], 8, 64)  # the few-rows kernels
    assert (od.float() - sdpa32(qd, k1, v1, mask[:, :, :8])).abs().max() <= TOL


def test_wrapper_errors(gpu):
    q = torch.zeros(1, 1, 128, 128, device=gpu)
    m = torch.ones(128, 128, dtype=torch.bool, device=gpu)
    with pytest.raises(TypeError):
        sparse_attention(q.double(), q.double(), q.double(), m, 128, 32)  # bf16, fp16 and fp32 only
    with pytest.raises(TypeError):
        sparse_attention(q, q.bfloat16(), q, m, 128, 32)  # one element type for all three
    qb = torch.zeros(1, 1, 128, 512, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(_native.SparseAttnError, match="head dim"):
        sparse_attention(qb, qb, qb, m, 128, 32)
    qb = torch.zeros(1, 1, 128, 128, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(AssertionError):
        sparse_attention(qb, qb, qb, m, 128, 48)
    # tiles the kernels do not have are refused at the C ABI and need a mask tensor in the wrapper
    md = compute_mask_kernel(m[None, None], 16, 32)
    with pytest.raises(ValueError, match="without a mask tensor"):
        sparse_attention(qb, qb, qb, None, 16, 32, mask_metadata=md)


@pytest.mark.parametrize("Sq,D,BQ,BK", [(256, 128, 16, 32), (256, 128, 16, 8), (1024, 64, 512, 4), (256, 256, 32, 32),
                                         (256, 256, 256, 64), (16, 128, 8, 16), (24, 64, 24, 8), (96, 128, 48, 32)])
def test_tile_sizes_the_kernels_do_not_have(gpu, Sq, D, BQ, BK):
    """Any tile sizes that divide the mask work, as in the reference: the wrapper classifies the mask again at sizes the
    kernels tile by, once per metadata object and mask."""
    from sparseattention_amd.sparse_attn_kernel import kernel_tiles
    B, H, Sk = 2, 2, 512
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=Sq + BQ, device=gpu, Sk=Sk)
    mask = (torch.rand(B, 1, Sq, Sk, generator=torch.Generator().manual_seed(BK)) < 0.6).to(gpu)
    mask[..., :Sq // 2, Sk // 2:] = False
    mask[..., 0] = True
    tiles = kernel_tiles(Sq, Sk, D, BQ, BK)
    assert tiles is not None and tiles != (BQ, BK) and Sq % tiles[0] == 0 and Sk % tiles[1] == 0
    want = sdpa32(q, k, v, mask)
    o = sparse_attention(q, k, v, mask, BQ, BK)
    assert (o.float() - want).abs().max() <= TOL
    assert torch.equal(o, sparse_attention(q, k, v, mask, *tiles))
    # with the caller's metadata at its own tile sizes: classified again once, then reused
    md = compute_mask_kernel(mask.expand(B, H, Sq, Sk), BQ, BK)
    assert torch.equal(o, sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=md))
    again = md._retiled
    assert torch.equal(o, sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=md)) and md._retiled is again
    mask[..., 1] = ~mask[..., 1]  # the mask changed in place: classified anew
    o2 = sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=md)
    assert md._retiled is not again
    assert (o2.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL


@pytest.mark.parametrize("Sq,D,BQ,BK", [(48, 128, 16, 16), (80, 64, 16, 32), (40, 128, 8, 8), (33, 32, 33, 64)])
def test_row_counts_no_kernel_tile_divides(gpu, Sq, D, BQ, BK):
    """More than 32 query rows, not a multiple of 32: the wrapper pads q and the mask with rows that attend to nothing."""
    B, H, Sk = 2, 2, 256
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=Sq, device=gpu, Sk=Sk)
    for mask in ((torch.rand(Sq, Sk, generator=torch.Generator().manual_seed(BQ)) < 0.5).to(gpu),
                 (torch.rand(B, 1, 1, Sk, generator=torch.Generator().manual_seed(BK)) < 0.5).to(gpu)):
        mask[..., 0] = True
        o, lse = sparse_attention(q, k, v, mask, BQ, BK, return_lse=True)
        assert o.shape == q.shape and lse.shape == (B, H, Sq)
        assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
        assert torch.equal(o, sparse_attention(q, k, v, mask, BQ, BK))


@pytest.mark.parametrize("name", golden_io.names())
def test_golden_outputs(gpu, name):
    g = golden_io.load(name)
    q, k, v = g.q.to(gpu), g.k.to(gpu), g.v.to(gpu)
    m = torch.from_numpy(g.mask).to(gpu)
    o = sparse_attention(q, k, v, m, g.BQ, g.BK)
    assert (o.float().cpu() - torch.from_numpy(g.out)).abs().max() <= TOL


def planes_vs_sdpa(o, q, k, v, mask, planes, rows=2048):
    """Compare chosen (b,h) planes with fp32 masked SDPA, evaluated in row slabs to bound memory."""
    worst = 0.0
    S = q.shape[2]
    for b, h in planes:
        mb = mask[b if mask.shape[0] > 1 else 0, h if mask.shape[1] > 1 else 0]
        for r0 in range(0, S, rows):
            ref = F.scaled_dot_product_attention(q[b, h, r0:r0 + rows].float()[None, None], k[b, h].float()[None, None],
                                                 v[b, h].float()[None, None], attn_mask=mb[r0:r0 + rows])
            worst = max(worst, (o[b, h, r0:r0 + rows].float() - ref[0, 0]).abs().max().item())
    return worst


def mass_per_key_block(q, k, mask, BQ, BK):
    """V whose row kv is the one-hot of kv's key block (D blocks): the output is then the attention mass
    each query puts on every block - zero exactly where the mask allows no key, rows summing to one."""
    B, H, S, D = q.shape
    blk = torch.arange(S, device=q.device) // (S // D)
    v = F.one_hot(blk, D).to(q.dtype)[None, None].expand(B, H, S, D).contiguous()
    o = sparse_attention(q, k, v, mask, BQ, BK).float()
    allowed = mask.reshape(*mask.shape[:-1], D, S // D).any(-1)  # mask: the un-expanded [1,1,S,S] tensor
    return o, allowed


def test_causal_config_full_size(gpu):
    B, H, S, D = 8, 32, 4096, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=0, device=gpu)
    mask = W.causal_mask(S, gpu)[None, None]
    me = mask.expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, 32)
    o = sparse_attention(q, k, v, me, 128, 32, mask_metadata=md)
    assert torch.isfinite(o).all()
    assert planes_vs_sdpa(o, q, k, v, mask, [(0, 0), (3, 17), (7, 31)]) <= TOL
    # against torch's own causal flash path on every plane
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert (o.float() - ref.float()).abs().max() <= TOL
    mass, allowed = mass_per_key_block(q, k, mask, 128, 32)
    assert (mass[~allowed.expand_as(mass)] == 0).all()
    assert (mass.sum(-1) - 1).abs().max() <= TOL


@pytest.mark.parametrize("p", [0.25, 0.5, 0.75, 0.9])
def test_random_block_config_full_size(gpu, p):
    B, H, S, D = 8, 32, 4096, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=1, device=gpu)
    mask = W.random_block_mask(S, 128, p, seed=int(p * 100), device=gpu)[None, None]
    me = mask.expand(B, H, S, S)
    o = sparse_attention(q, k, v, me, 128, 32)
    assert torch.isfinite(o).all()
    assert planes_vs_sdpa(o, q, k, v, mask, [(0, 0), (5, 9), (7, 31)]) <= TOL
    mass, allowed = mass_per_key_block(q, k, mask, 128, 32)
    assert (mass[~allowed.expand_as(mass)] == 0).all()
    assert (mass.sum(-1) - 1).abs().max() <= TOL


def test_document_config_full_size(gpu):
    B, H, S, D = 4, 32, 16384, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=2, device=gpu)
    mask = W.document_mask(S, seed=0, device=gpu)[None, None]
    me = mask.expand(B, H, S, S)
    o = sparse_attention(q, k, v, me, 128, 32)
    assert torch.isfinite(o).all()
    assert planes_vs_sdpa(o, q, k, v, mask, [(0, 0), (3, 31)]) <= TOL
    mass, allowed = mass_per_key_block(q, k, mask, 128, 32)
    assert (mass[~allowed.expand_as(mass)] == 0).all()
    assert (mass.sum(-1) - 1).abs().max() <= TOL


def test_composed_config_full_size(gpu):
    B, H, S, D = 1, 32, 32768, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=3, device=gpu)
    mask = W.composed_mask(S, device=gpu)[None, None]
    me = mask.expand(B, H, S, S)
    o = sparse_attention(q, k, v, me, 128, 32)
    assert torch.isfinite(o).all()
    assert planes_vs_sdpa(o, q, k, v, mask, [(0, 0), (0, 31)]) <= TOL
    mass, allowed = mass_per_key_block(q, k, mask, 128, 32)
    assert (mass[~allowed.expand_as(mass)] == 0).all()
    assert (mass.sum(-1) - 1).abs().max() <= TOL


def test_runs_on_a_side_stream(gpu):
    B, H, S, D = 1, 2, 512, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=5, device=gpu)
    mask = W.causal_mask(S, gpu)
    want = sparse_attention(q, k, v, mask, 128, 32)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        got = sparse_attention(q, k, v, mask, 128, 32)
    s.synchronize()
    assert torch.equal(got, want)


def test_calls_from_several_host_threads(gpu):
    # four host threads, each with a stream of its own and shapes of its own (so each is the first to raise the LDS
    # limit of some kernel variant), forward with preprocessing, lse and errors in between: the results equal the
    # ones computed one after the other, and an error message stays with the thread that caused it
    import threading

    cases = [(1, 2, 256, 64, 64, 32), (2, 1, 512, 128, 128, 64), (1, 3, 384, 128, 128, 16), (2, 2, 256, 64, 32, 128)]
    inputs = []
    for i, (B, H, S, D, BQ, BK) in enumerate(cases):
        q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=40 + i, device=gpu)
        mask = W.random_block_mask(S, 32, 0.5, seed=50 + i, device=gpu)
        inputs.append((q, k, v, mask, BQ, BK))
    want = [sparse_attention(*inp, return_lse=True) for inp in inputs]
    torch.cuda.synchronize()
    got, errors = [None] * len(cases), []

    def work(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for _ in range(5):
                    got[i] = sparse_attention(*inputs[i], return_lse=True)
                    q, k, v, mask, BQ, BK = inputs[i]
                    try:
                        wide = 264 + 8 * i  # beyond every kernel, and different in every thread
                        sparse_attention(*(t.repeat(1, 1, 1, 5)[..., :wide] for t in (q, k, v)), mask, BQ, BK)
                        errors.append(f"thread {i}: head dim {wide} was accepted")
                    except _native.SparseAttnError as e:
                        if f"head dim {wide}" not in str(e):
                            errors.append(f"thread {i}: foreign message {e}")
            s.synchronize()
        except Exception as e:  # noqa: BLE001 - reported by the assertion below
            errors.append(f"thread {i}: {type(e).__name__} {e}")

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for (o, lse), (o_w, lse_w) in zip(got, want):
        assert torch.equal(o, o_w) and torch.equal(lse, lse_w)


@pytest.mark.parametrize("route", ["plain", "packed+pairs", "persistent"])
@pytest.mark.parametrize("BQ,BK", [(128, 32), (64, 64), (256, 16)])
def test_lse_output(gpu, route, BQ, BK):
    B, H, S, D = 2, 2, 1024, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=41, device=gpu)
    mask = W.random_block_mask(S, 32, 0.5, seed=42, device=gpu, batch=B).clone()
    mask[1, :, 77] = False  # a row that attends to nothing
    me = mask.expand(B, H, S, S)
    if route == "plain":
        md = compute_mask_kernel(me, BQ, BK, pack_partial=False)
    elif BQ == 256:
        pytest.skip("no scheduled forward for BLOCK_Q = 256")
    else:
        md = compute_mask_kernel(me, BQ, BK, schedule="pairs" if route == "packed+pairs" else "persistent")
    o, lse = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md, return_lse=True)
    assert torch.equal(o, sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md))
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double()) / math.sqrt(D)
    want = torch.logsumexp(s.masked_fill(~me, -math.inf), dim=-1)
    assert lse.shape == (B, H, S) and lse.dtype == torch.float32
    assert (lse[1, :, 77] == -math.inf).all()
    live = torch.isfinite(want)
    assert torch.equal(live, torch.isfinite(lse))
    # the row sum adds up P as rounded to bf16 (8 significant bits) for the P.V product: a sum that one term
    # dominates is off by up to 2^-8 of itself
    assert (lse[live].double() - want[live]).abs().max() <= 6e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("BQ", [64, 128])
@pytest.mark.parametrize("BK", [16, 32, 64, 256])
def test_head_dim_256(gpu, BQ, BK, dtype):
    # one workgroup per CU with the whole register file; bool-mask reads, packed tiles, lse, a schedule that is ignored
    B, H, Sq, Sk, D = 2, 2, 384, 768, 256
    q, _, _ = W.qkv(B, H, Sq, D, dtype, seed=BQ + BK, device=gpu)
    _, k, v = W.qkv(B, H, Sk, D, dtype, seed=BQ * BK, device=gpu)
    coarse = torch.rand(B, 1, Sq // 32, Sk // 32, generator=torch.Generator().manual_seed(BK)) < 0.5
    fine = torch.rand(B, 1, Sq, Sk, generator=torch.Generator().manual_seed(BQ)) < 0.7
    mask = (coarse.repeat_interleave(32, 2).repeat_interleave(32, 3) & fine).to(gpu)
    mask[..., :16] = True
    me = mask.expand(B, H, Sq, Sk)
    o = sparse_attention(q, k, v, me, BQ, BK, compute_mask_kernel(me, BQ, BK, pack_partial=False))
    want = oracle_out(q, k, v, mask, BQ, BK, p_round=1 if dtype == torch.bfloat16 else 2)
    err = (o.float().cpu() - want).abs()
    assert err.max() <= TOL and err.mean() <= 1e-3, f"vs oracle: max {err.max()}, mean {err.mean()}"
    ref = sdpa32(q, k, v, mask)
    assert (o.float() - ref).abs().max() <= TOL
    sched = "pairs" if BK <= 64 else None
    o2, lse = sparse_attention(q, k, v, None, BQ, BK, compute_mask_kernel(me, BQ, BK, pack_partial=True, schedule=sched),
                               return_lse=True)
    assert torch.equal(o, o2)
    s = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) / math.sqrt(D)
    want_lse = torch.logsumexp(s.masked_fill(~me, float("-inf")), dim=-1)
    assert (lse - want_lse).abs().max() <= 6e-3


def test_head_dim_256_limits_and_long_rows(gpu):
    qb = torch.zeros(1, 1, 256, 256, dtype=torch.bfloat16, device=gpu)
    m = torch.ones(256, 256, dtype=torch.bool, device=gpu)
    lib = _native.load()
    md = compute_mask_kernel(m[None, None], 32, 32, pack_partial=False)
    S = _native.strides
    me = m[None, None]
    rc = lib.sa_sparse_attention_fwd(
        qb.data_ptr(), S(qb.stride()), qb.data_ptr(), S(qb.stride()), qb.data_ptr(), S(qb.stride()),
        torch.empty_like(qb).data_ptr(), S(qb.stride()), me.data_ptr(), S(me.stride()),
        md.unmasked_kv_ids.data_ptr(), S(md.unmasked_kv_ids.stride()), md.unmasked_lens.data_ptr(),
        S(md.unmasked_lens.stride()), md.masked_kv_ids.data_ptr(), S(md.masked_kv_ids.stride()),
        md.masked_lens.data_ptr(), S(md.masked_lens.stride()), 1, 1, 256, 256, 256, 32, 32, 0, 0.09, None)
    assert rc == _native.SA_ERR_UNSUPPORTED and "head dim 256" in lib.sa_last_error().decode()
    # causal, 4096 keys: long lists, every plane against fp32 SDPA
    B, H, S, D = 1, 4, 4096, 256
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=77, device=gpu)
    mask = W.causal_mask(S, gpu)
    o = sparse_attention(q, k, v, mask, 128, 32)
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL


@pytest.mark.parametrize("BK", [16, 32, 64])
def test_lists_longer_than_the_lds_copy(gpu, BK):
    # more list entries per Q tile than the kernel keeps in LDS (2048): the entries are then read from global memory
    # chunk by chunk; FULL and PARTIAL entries, an odd count, with and without packed tiles
    B, H, Sq, D = 1, 2, 128, 64
    Sk = BK * 2048 + 5 * BK * (64 // BK if BK < 64 else 1) + BK * 3
    Sk = (Sk + 63) // 64 * 64
    q, _, _ = W.qkv(B, H, Sq, D, torch.bfloat16, seed=61, device=gpu)
    _, k, v = W.qkv(B, H, Sk, D, torch.bfloat16, seed=62, device=gpu)
    mask = torch.ones(Sq, Sk, dtype=torch.bool, device=gpu)
    mask[:, 1000:1000 + 3 * BK] = torch.rand(Sq, 3 * BK, generator=torch.Generator().manual_seed(63)).to(gpu) < 0.5
    mask[:, 5000:5000 + BK] = False
    me = mask[None, None].expand(B, H, Sq, Sk)
    want = sdpa32(q, k, v, mask)
    for pack in (False, True):
        md = compute_mask_kernel(me, 128, BK, pack_partial=pack)
        assert int(md.unmasked_lens[0, 0, 0] + md.masked_lens[0, 0, 0]) > 2048
        o = sparse_attention(q, k, v, me, 128, BK, mask_metadata=md)
        assert (o.float() - want).abs().max() <= TOL
