"""float32 q, k, v through the forward: the reference's kernel takes the element type of its inputs
(sparse_attn_kernel.py:98-101, :145), so the CPU-plumbing configuration (B1 H4 S512 D64 fp32) runs on the GPU as it is.
Checked against fp32 masked SDPA on the CPU and against the C oracle with P kept in fp32, both to 1e-5 max-abs."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from sparseattention_amd import (_native, causal_term, compute_mask_kernel, compute_mask_terms, sparse_attention,
                                 workloads as W)

pytestmark = pytest.mark.gpu
TOL32 = 1e-5


def sdpa_cpu(q, k, v, mask):
    out = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), attn_mask=mask)
    return torch.nan_to_num(out, nan=0.0).float()  # rows that attend to nothing: 0 here, NaN there


@pytest.mark.parametrize("BQ,BK", [(32, 32), (128, 32), (64, 16), (16, 8), (256, 64), (8, 128)])
def test_cpu_plumbing_workload_in_float32(gpu, BQ, BK):
    B, H, S, D = 1, 4, 512, 64
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=0)
    mask = W.random_block_mask(S, 32, 0.5, seed=0)
    want = sdpa_cpu(q, k, v, mask)
    me = mask.to(gpu)[None, None].expand(B, H, S, S)
    o = sparse_attention(q.to(gpu), k.to(gpu), v.to(gpu), me, BQ, BK)
    assert o.dtype == torch.float32 and o.shape == q.shape
    assert (o.cpu() - want).abs().max() <= TOL32
    ref = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy()[None, None], BQ, BK, p_round=0)
    assert np.abs(o.cpu().numpy() - ref).max() <= TOL32


@pytest.mark.parametrize("D,BQ,BK", [(128, 128, 32), (256, 128, 64), (256, 64, 32), (80, 64, 32), (128, 1, 32)])
def test_head_dims_and_lse(gpu, D, BQ, BK):
    B, H, Sq, Sk = 2, 3, 256, 384
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, H, Sq, D, generator=g)
    k = torch.randn(B, H, Sk, D, generator=g)
    v = torch.randn(B, H, Sk, D, generator=g)
    mask = torch.rand(B, 1, Sq, Sk, generator=g) < 0.4
    mask[:, :, 7] = False  # a row that attends to nothing
    mask[:, :, 64:128, :128] = True  # FULL tiles
    mask[:, :, :, 256:] &= torch.rand(1, 1, 1, 128, generator=g) < 0.5
    me = mask.expand(B, H, Sq, Sk)
    want = sdpa_cpu(q, k, v, me)
    o, lse = sparse_attention(q.to(gpu), k.to(gpu), v.to(gpu), me.to(gpu), BQ, BK, return_lse=True)
    assert (o.cpu() - want).abs().max() <= TOL32
    assert torch.equal(o[:, :, 7].cpu(), torch.zeros(B, H, D))
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double()) / math.sqrt(D)
    want_lse = torch.logsumexp(s.masked_fill(~me, float("-inf")), -1)
    got = lse.cpu().double()
    assert torch.isneginf(got[:, :, 7]).all()
    live = ~torch.isneginf(want_lse)
    assert (got[live] - want_lse[live]).abs().max() <= 1e-5


def test_strided_inputs_precomputed_metadata_and_formula_masks(gpu):
    B, H, S, D, BQ, BK = 2, 4, 512, 64, 64, 32
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn(3, B, S, H, D, generator=g).to(gpu)  # [B,S,H,D] storage
    q, k, v = (t.permute(0, 2, 1, 3) for t in qkv)
    mask = W.causal_mask(S, gpu)[None, None].expand(B, H, S, S)
    want = sdpa_cpu(q.cpu(), k.cpu(), v.cpu(), mask.cpu())
    md = compute_mask_kernel(mask, BQ, BK)
    o = sparse_attention(q, k, v, mask, BQ, BK, md)
    assert o.stride() == q.stride() and (o.cpu() - want).abs().max() <= TOL32
    # the same from packed tiles alone (no mask tensor), and from the bool mask alone (no packed tiles)
    mdt = compute_mask_terms([causal_term()], B, H, S, S, BQ, BK, device=gpu)
    assert torch.equal(sparse_attention(q, k, v, None, BQ, BK, mdt), o)
    assert torch.equal(sparse_attention(q, k, v, mask, BQ, BK, compute_mask_kernel(mask, BQ, BK, pack_partial=False)), o)
    # against the 16-bit kernels on the same numbers: within their tolerance
    ob = sparse_attention(q.bfloat16(), k.bfloat16(), v.bfloat16(), mask, BQ, BK, md)
    assert (ob.float() - o).abs().max() <= 2e-2


def test_c_abi_limits_of_float32(gpu):
    lib = _native.load()
    B, H, S, D = 1, 1, 512, 256
    q = torch.zeros(B, H, S, D, device=gpu)
    mask = torch.ones(B, H, S, S, dtype=torch.bool, device=gpu)
    with pytest.raises(_native.SparseAttnError, match="BLOCK_Q"):
        md = compute_mask_kernel(mask, 256, 32, pack_partial=False)
        st = _native.strides
        rc = lib.sa_sparse_attention_fwd(
            q.data_ptr(), st(q.stride()), q.data_ptr(), st(q.stride()), q.data_ptr(), st(q.stride()), q.data_ptr(), st(q.stride()),
            mask.data_ptr(), st(mask.stride()), md.unmasked_kv_ids.data_ptr(), st(md.unmasked_kv_ids.stride()),
            md.unmasked_lens.data_ptr(), st(md.unmasked_lens.stride()), md.masked_kv_ids.data_ptr(), st(md.masked_kv_ids.stride()),
            md.masked_lens.data_ptr(), st(md.masked_lens.stride()), B, H, S, S, D, 256, 32, _native.SA_DTYPE_FP32, 0.09, None)
        _native.check(rc)
    # the wrapper runs the same request on tiles the kernel has
    o = sparse_attention(q, q, q, mask, 256, 32)
    assert torch.equal(o, torch.zeros_like(q))


@pytest.mark.parametrize("D,BQ,BK", [(64, 48, 24), (64, 64, 40), (128, 32, 96), (128, 256, 32), (64, 8, 24)])
def test_tile_widths_that_are_no_power_of_two_and_the_widest_tile(gpu, D, BQ, BK):
    # BLOCK_K not a multiple of 32 ends every tile in a partial 32-key step; both mask sources; D = 128 at 256-row tiles
    B, H, S = 1, 2, 960 if BK in (24, 40, 96) else 512
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=BQ + BK)
    mask = W.random_block_mask(S, 16, 0.5, seed=BK, partial_fraction=0.3)
    want = sdpa_cpu(q, k, v, mask)
    me = mask.to(gpu)[None, None].expand(B, H, S, S)
    lib = _native.load()
    st = _native.strides
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    md_all = compute_mask_kernel(me, BQ, BK, pack_partial=BK % 8 == 0)
    for packed in ([None, md_all.packed_masks] if BK % 8 == 0 else [None]):
        o = torch.full_like(qg, float("nan"))
        rc = lib.sa_sparse_attention_fwd_ex(
            qg.data_ptr(), st(qg.stride()), kg.data_ptr(), st(kg.stride()), vg.data_ptr(), st(vg.stride()), o.data_ptr(),
            st(o.stride()), me.data_ptr(), st(me.stride()),
            md_all.unmasked_kv_ids.data_ptr(), st(md_all.unmasked_kv_ids.stride()), md_all.unmasked_lens.data_ptr(),
            st(md_all.unmasked_lens.stride()), md_all.masked_kv_ids.data_ptr(), st(md_all.masked_kv_ids.stride()),
            md_all.masked_lens.data_ptr(), st(md_all.masked_lens.stride()),
            packed.data_ptr() if packed is not None else None, st(packed.stride()[:2]) if packed is not None else None,
            None, 0, 0, B, H, S, S, D, BQ, BK, _native.SA_DTYPE_FP32, D ** -0.5 / math.log(2),
            torch.cuda.current_stream().cuda_stream)
        _native.check(rc)
        torch.cuda.synchronize()
        assert (o.cpu() - want).abs().max() <= TOL32, f"packed={packed is not None}"
        ref = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy()[None, None], BQ, BK, p_round=0)
        assert np.abs(o.cpu().numpy() - ref).max() <= TOL32


@pytest.mark.parametrize("D,BQ,BK", [(128, 128, 64), (128, 128, 128), (64, 32, 64), (64, 64, 256), (128, 64, 16), (64, 128, 16),
                                     (128, 128, 32), (64, 32, 32)])
def test_sizes_of_the_matrix_unit_kernel(gpu, D, BQ, BK):
    # the float32 forward runs these sizes on v_mfma_f32_32x32x2_f32: every tile width class (16, 32, wider), every
    # workgroup size, both mask sources, per-batch masks, a dead row, lists with FULL and PARTIAL entries, the lse
    B, H, Sq, Sk = 2, 2, 512, 1024
    g = torch.Generator().manual_seed(D + BQ + BK)
    q = torch.randn(B, H, Sq, D, generator=g)
    k = torch.randn(B, H, Sk, D, generator=g)
    v = torch.randn(B, H, Sk, D, generator=g)
    mask = torch.rand(B, 1, Sq, Sk, generator=g) < 0.3
    mask[:, :, 9] = False
    mask[:, :, 128:256, :512] = True
    mask[:, :, 256:, 768:] = False
    me = mask.expand(B, H, Sq, Sk)
    want = sdpa_cpu(q, k, v, me)
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double()) / math.sqrt(D)
    want_lse = torch.logsumexp(s.masked_fill(~me, float("-inf")), -1)
    qg, kg, vg, mg = q.to(gpu), k.to(gpu), v.to(gpu), me.to(gpu)
    for pack in (True, False):
        md = compute_mask_kernel(mg, BQ, BK, pack_partial=pack)
        o, lse = sparse_attention(qg, kg, vg, mg, BQ, BK, md, return_lse=True)
        torch.cuda.synchronize()
        assert (o.cpu() - want).abs().max() <= TOL32, f"pack={pack}"
        assert torch.equal(o[:, :, 9].cpu(), torch.zeros(B, H, D))
        live = ~torch.isneginf(want_lse)
        assert torch.isneginf(lse.cpu()[~live]).all() and (lse.cpu().double()[live] - want_lse[live]).abs().max() <= 1e-5
