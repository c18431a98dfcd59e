"""Scores that spread over hundreds of exp2 units: the running reference value of the online softmax has to move again
and again (and the accumulators have to be rescaled), which N(0,1) inputs never ask for.  Forward, decode and backward
against fp32 masked SDPA and autograd on the same rounded inputs."""
import math

import pytest
import torch
import torch.nn.functional as F

from sparseattention_amd import (compute_backward_metadata, sparse_attention, sparse_attention_backward,
                                 sparse_attention_decode, workloads as W)

pytestmark = pytest.mark.gpu

TOL = 2e-2


def growing_scores(B, H, Sq, Sk, D, dtype, device, per_key, seed, noise=0.5):
    """q, k, v whose scores q.k/sqrt(D) grow by about `per_key` (natural units) from one key to the next, plus noise."""
    g = torch.Generator().manual_seed(seed)
    e = torch.randn(B, H, 1, D, generator=g)
    e = e / e.norm(dim=-1, keepdim=True)
    qn = torch.randn(B, H, Sq, D, generator=g) * 0.1
    kn = torch.randn(B, H, Sk, D, generator=g) * noise
    amp = math.sqrt(D) ** 0.5 * 4.0
    q = amp * e + qn
    ramp = torch.arange(Sk, dtype=torch.float32)[None, None, :, None] * (per_key * math.sqrt(D) / amp)
    k = ramp * e + kn
    v = torch.randn(B, H, Sk, D, generator=g)
    return q.to(device, dtype), k.to(device, dtype), v.to(device, dtype)


@pytest.mark.parametrize("per_key", [0.05, 0.3, -0.3])
@pytest.mark.parametrize("BQ,BK,D", [(128, 32, 128), (64, 64, 64), (256, 16, 128), (128, 128, 256)])
def test_forward(gpu, BQ, BK, D, per_key):
    B, H, S = 1, 2, 1024
    q, k, v = growing_scores(B, H, S, S, D, torch.bfloat16, gpu, per_key, seed=BQ + BK)
    for mask in (W.causal_mask(S, gpu), torch.ones(S, S, dtype=torch.bool, device=gpu),
                 W.random_block_mask(S, 32, 0.5, seed=7, device=gpu)):
        o, lse = sparse_attention(q, k, v, mask, BQ, BK, return_lse=True)
        want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
        assert not torch.isnan(o).any()
        assert (o.float() - want).abs().max() <= TOL
        # The kernel multiplies the queries by scale/ln 2 and rounds them to the input dtype again, so that the matrix
        # unit delivers exp2 arguments: against scores of those rounded queries the lse is tight; against the scores
        # of the given queries it is off by up to 2^-9 of the score's size (one more rounding of every query element).
        qs = (q.float() * torch.tensor(1.0 / math.sqrt(D) / math.log(2.0), dtype=torch.float32)).to(q.dtype)
        s2 = torch.einsum("bhqd,bhkd->bhqk", qs.float(), k.float()) * math.log(2.0)
        want_lse = torch.logsumexp(s2.masked_fill(~mask, float("-inf")), dim=-1)
        assert (lse - want_lse).abs().max() <= 6e-3
        s = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) / math.sqrt(D)
        exact_lse = torch.logsumexp(s.masked_fill(~mask, float("-inf")), dim=-1)
        assert (lse - exact_lse).abs().max() <= 6e-3 + 2.0 ** -9 * float(s.abs().max())


@pytest.mark.parametrize("per_key", [0.3, -0.3])
@pytest.mark.parametrize("Sq,D", [(1, 128), (16, 64), (32, 128)])
def test_decode(gpu, Sq, D, per_key):
    B, H, Sk, BK = 2, 2, 4096, 64
    q, k, v = growing_scores(B, H, Sq, Sk, D, torch.bfloat16, gpu, per_key, seed=Sq)
    mask = torch.rand(Sq, Sk, generator=torch.Generator().manual_seed(3)).to(gpu) < 0.8
    mask[:, 0] = True
    me = mask[None, None].expand(B, H, Sq, Sk)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    for splits in (1, 4, 0):
        o = sparse_attention_decode(q, k, v, me, BK, num_splits=splits)
        assert (o.float() - want).abs().max() <= TOL


@pytest.mark.parametrize("per_key", [0.05, -0.05])
@pytest.mark.parametrize("D", [64, 128])
def test_backward(gpu, D, per_key):
    B, H, S = 1, 2, 512
    q, k, v = growing_scores(B, H, S, S, D, torch.bfloat16, gpu, per_key, seed=D, noise=1.0)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(5)).to(gpu, torch.bfloat16)
    mask = W.causal_mask(S, gpu) if per_key > 0 else torch.ones(S, S, dtype=torch.bool, device=gpu)
    me = mask[None, None].expand(B, H, S, S)
    o, lse = sparse_attention(q, k, v, me, 128, 32, return_lse=True)
    got = sparse_attention_backward(do, q, k, v, o, lse, None, compute_backward_metadata(me))
    q32, k32, v32 = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(q32, k32, v32, attn_mask=mask).backward(do.float())
    for g_, w, name in zip(got, (q32.grad, k32.grad, v32.grad), ("dq", "dk", "dv")):
        assert not torch.isnan(g_).any()
        scale = max(1.0, float(w.abs().max()))
        assert float((g_.float() - w).abs().max()) / scale <= TOL, name
