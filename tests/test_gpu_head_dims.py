"""Head dims without a kernel of their own (16, 32, 80, 96, 192 ...): the wrappers pad q, k, v with zero columns up to
the next size the kernels have, keep the softmax scale of the given D and cut the result back.  Forward, few-rows path
and backward against fp32 masked SDPA and autograd on the same rounded inputs."""
import pytest
import torch
import torch.nn.functional as F

from sparseattention_amd import (compute_backward_metadata, sparse_attention, sparse_attention_backward,
                                 sparse_attention_decode, sparse_attention_trainable, workloads as W)

pytestmark = pytest.mark.gpu

TOL = 2e-2


def some_mask(Sq, Sk, gpu, seed):
    m = (torch.rand(Sq, Sk, generator=torch.Generator().manual_seed(seed)) < 0.5).to(gpu)
    m[: Sq // 2, Sk // 2:] = False  # empty tiles
    m[Sq // 2:, : Sk // 4] = True   # full tiles
    m[:, 0] = True
    return m


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [16, 32, 40, 80, 96, 192])
def test_forward(gpu, D, dtype):
    B, H, Sq, Sk = 2, 3, 256, 384
    q, k, v = W.qkv(B, H, Sq, D, dtype, seed=D, device=gpu, Sk=Sk)
    mask = some_mask(Sq, Sk, gpu, D)
    o, lse = sparse_attention(q, k, v, mask, 128, 32, return_lse=True)
    assert o.shape == q.shape and o.dtype == dtype and o.is_contiguous()
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    assert (o.float() - want).abs().max() <= TOL
    s = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) / D ** 0.5
    assert (lse - torch.logsumexp(s.masked_fill(~mask, float("-inf")), dim=-1)).abs().max() <= 2e-2


@pytest.mark.parametrize("D,Sq,BQ", [(192, 256, 32), (256, 256, 256), (192, 8, 8), (256, 24, 8), (160, 48, 16)])
def test_wide_heads_with_tiles_and_rows_they_have_no_kernel_for(gpu, D, Sq, BQ):
    B, H, Sk = 1, 2, 256
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=D + Sq, device=gpu, Sk=Sk)
    mask = some_mask(Sq, Sk, gpu, D)
    o = sparse_attention(q, k, v, mask, BQ, 32)
    assert o.shape == q.shape
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    assert (o.float() - want).abs().max() <= TOL


@pytest.mark.parametrize("D,Sq", [(32, 1), (96, 16), (80, 32)])
def test_few_rows(gpu, D, Sq):
    B, H, Sk = 2, 2, 2048
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=D, device=gpu, Sk=Sk)
    mask = some_mask(Sq, Sk, gpu, D) if Sq > 1 else torch.ones(1, Sk, dtype=torch.bool, device=gpu)
    o = sparse_attention_decode(q, k, v, mask, 64)
    assert o.shape == q.shape
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    assert (o.float() - want).abs().max() <= TOL


@pytest.mark.parametrize("D", [32, 96])
def test_backward(gpu, D):
    B, H, S = 1, 2, 256
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=D, device=gpu)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(5)).to(gpu, torch.bfloat16)
    mask = some_mask(S, S, gpu, D)
    me = mask[None, None].expand(B, H, S, S)
    o, lse = sparse_attention(q, k, v, me, 128, 32, return_lse=True)
    got = sparse_attention_backward(do, q, k, v, o, lse, None, compute_backward_metadata(me))
    q32, k32, v32 = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(q32, k32, v32, attn_mask=mask).backward(do.float())
    for g_, w, name in zip(got, (q32.grad, k32.grad, v32.grad), ("dq", "dk", "dv")):
        assert g_.shape == w.shape
        assert float((g_.float() - w).abs().max()) / max(1.0, float(w.abs().max())) <= TOL, name
    # and through autograd
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    sparse_attention_trainable(qa, ka, va, me, 128, 32).backward(do)
    for g_, a in zip(got, (qa.grad, ka.grad, va.grad)):
        assert torch.equal(g_, a)


@pytest.mark.parametrize("Sq,Sk,D", [(192, 320, 128), (96, 96, 64), (48, 208, 32)])
def test_backward_sizes_not_multiples_of_128(gpu, Sq, Sk, D):
    """The backward tiles by 128 rows both ways; other sizes are padded with rows that attend to nothing."""
    B, H = 2, 2
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=Sq, device=gpu, Sk=Sk)
    do = torch.randn(B, H, Sq, D, generator=torch.Generator().manual_seed(6)).to(gpu, torch.bfloat16)
    mask = some_mask(Sq, Sk, gpu, Sk)
    me = mask[None, None].expand(B, H, Sq, Sk)
    q32, k32, v32 = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(q32, k32, v32, attn_mask=mask).backward(do.float())
    want = (q32.grad, k32.grad, v32.grad)
    BK = 16
    for bmd in (None, compute_backward_metadata(me), compute_backward_metadata(me, pack_partial=False)):
        qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
        sparse_attention_trainable(qa, ka, va, me, 16, BK, bwd_metadata=bmd).backward(do)
        for g_, w, name in zip((qa.grad, ka.grad, va.grad), want, ("dq", "dk", "dv")):
            assert g_.shape == w.shape
            assert float((g_.float() - w).abs().max()) / max(1.0, float(w.abs().max())) <= TOL, name
