"""Merge of attention results over disjoint key ranges (sa_merge_attention_parts): the exchange a key-axis sharding
ends with.  Checked against the unsplit forward and fp32 masked SDPA, tolerance 2e-2 max-abs as for the forward."""
import math

import pytest
import torch
import torch.nn.functional as F

from sparseattention_amd import (merge_attention_parts, sparse_attention, sparse_attention_kv_split, workloads as W)

pytestmark = pytest.mark.gpu

TOL = 2e-2


@pytest.mark.parametrize("splits", [1, 2, 4, 8])
@pytest.mark.parametrize("D", [64, 128])
def test_kv_split_equals_the_unsplit_forward(gpu, splits, D):
    B, H, Sq, Sk = 2, 3, 256, 2048
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=51, device=gpu, Sk=Sk)
    mask = (torch.rand(B, 1, Sq, Sk, generator=torch.Generator().manual_seed(52)) < 0.3).to(gpu)
    coarse = (torch.rand(B, 1, Sq // 64, Sk // 64, generator=torch.Generator().manual_seed(53)) < 0.5).to(gpu)
    mask = mask & coarse.repeat_interleave(64, -2).repeat_interleave(64, -1)
    mask[1, :, 7] = False          # a row without any key
    mask[0, :, :, Sk // 2:] = False  # a batch element whose keys all lie in the first half
    mask[0, :, :, 0] = True
    o, lse = sparse_attention_kv_split(q, k, v, mask, 64, 32, splits, return_lse=True)
    whole, lse_whole = sparse_attention(q, k, v, mask, 64, 32, return_lse=True)
    assert not torch.isnan(o).any() and (o[1, :, 7] == 0).all() and (lse[1, :, 7] == -math.inf).all()
    if splits == 1:
        assert torch.equal(o, whole)
    assert (o.float() - whole.float()).abs().max() <= TOL
    live = torch.isfinite(lse_whole)
    assert torch.equal(live, torch.isfinite(lse)) and (lse[live] - lse_whole[live]).abs().max() <= 1e-2
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    ref = torch.nan_to_num(ref, nan=0.0)
    assert (o.float() - ref).abs().max() <= TOL


def test_merge_of_given_parts_fp16_and_strided(gpu):
    n, B, H, Sq, D = 3, 2, 2, 64, 128
    g = torch.Generator().manual_seed(54)
    o_parts = torch.randn(n, B, Sq, H, D, generator=g).to(gpu, torch.float16).transpose(2, 3)  # [n,B,H,Sq,D] view
    lse_parts = torch.randn(n, B, H, Sq, generator=g).to(gpu) * 3
    lse_parts[0, 0, 0, :5] = -math.inf
    o, lse = merge_attention_parts(o_parts, lse_parts, return_lse=True)
    w = torch.softmax(lse_parts.double(), 0)
    want = (w[..., None] * o_parts.double()).sum(0)
    assert (o.double() - want).abs().max() <= 2e-3
    assert (lse.double() - torch.logsumexp(lse_parts.double(), 0)).abs().max() <= 1e-5
