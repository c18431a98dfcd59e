"""Seeded random sweep over shapes, tile sizes, mask families and storage layouts for the three paths (forward,
decode, backward), each case against fp32 masked SDPA (and its autograd) on the same bf16 inputs.  Tolerance as in
the dedicated test files: 2e-2 max-abs for outputs, 2e-2 of the gradient's own scale for gradients."""
import math
import random

import pytest
import torch
import torch.nn.functional as F

from sparseattention_amd import (compute_mask_kernel, sparse_attention, sparse_attention_backward,
                                 sparse_attention_decode, workloads as W)

pytestmark = pytest.mark.gpu

TOL = 2e-2


def random_mask(rng, B, H, Sq, Sk, device):
    """One of: block-random, banded + random far columns, per-row random prefix, dense with holes.  Shape
    [b,h,Sq,Sk] with b in {1,B}, h in {1,H}; every row keeps at least one key."""
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    b = rng.choice((1, B))
    h = rng.choice((1, H))
    kind = rng.randrange(4)
    if kind == 0:
        blk = rng.choice((16, 32, 64))
        coarse = torch.rand(b, h, -(-Sq // blk), -(-Sk // blk), generator=g) < rng.uniform(0.2, 0.8)
        m = coarse.repeat_interleave(blk, -2).repeat_interleave(blk, -1)[..., :Sq, :Sk]
        m = m ^ (torch.rand(b, h, Sq, Sk, generator=g) < 0.02)
    elif kind == 1:
        q = torch.arange(Sq)[:, None] * (Sk / Sq)
        kk = torch.arange(Sk)[None, :]
        band = (kk <= q) & (q - kk < rng.choice((64, 200, 513)))
        far = torch.rand(b, h, 1, Sk, generator=g) < 0.1
        m = band[None, None] | far
    elif kind == 2:
        lens = torch.randint(1, Sk + 1, (b, h, Sq, 1), generator=g)
        m = torch.arange(Sk)[None, None, None, :] < lens
    else:
        m = torch.rand(b, h, Sq, Sk, generator=g) < 0.97
    m = m.clone()
    m[..., 0] = True
    return m.to(device)


def tensors(rng, B, H, Sq, Sk, D, device, n=3):
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    seq_major = rng.random() < 0.3  # [B,S,H,D] storage seen as [B,H,S,D]
    out = []
    for i, S in enumerate((Sq, Sk, Sk, Sq)[:n]):
        if seq_major:
            out.append(torch.randn(B, S, H, D, generator=g).to(device, torch.bfloat16).transpose(1, 2))
        else:
            out.append(torch.randn(B, H, S, D, generator=g).to(device, torch.bfloat16))
    return out


def sdpa32(q, k, v, mask):
    return F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)


@pytest.mark.parametrize("seed", range(24))
def test_forward(gpu, seed):
    rng = random.Random(1000 + seed)
    B, H, D = rng.choice((1, 2, 3)), rng.choice((1, 2, 5)), rng.choice((64, 128))
    BQ, BK = rng.choice((32, 64, 128, 256)), rng.choice((16, 32, 64, 128))
    Sq, Sk = BQ * rng.randint(1, 1024 // BQ), BK * rng.randint(1, 1024 // BK)
    q, k, v = tensors(rng, B, H, Sq, Sk, D, gpu)
    mask = random_mask(rng, B, H, Sq, Sk, gpu)
    me = mask.expand(B, H, Sq, Sk)
    sched = rng.choice((None, None, "pairs", "persistent")) if BQ != 256 else None
    md = compute_mask_kernel(me, BQ, BK, pack_partial=rng.random() < 0.5 if BK % 8 == 0 else False, schedule=sched)
    o, lse = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md, return_lse=True)
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL, (B, H, Sq, Sk, D, BQ, BK, sched)
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double()) / math.sqrt(D)
    # P is summed as rounded to bf16 (8 significant bits): up to 2^-8 of the sum
    assert (lse.double() - torch.logsumexp(s.masked_fill(~me, -math.inf), -1)).abs().max() <= 6e-3


@pytest.mark.parametrize("seed", range(16))
def test_decode(gpu, seed):
    rng = random.Random(2000 + seed)
    B, H, D = rng.choice((1, 2, 4)), rng.choice((1, 3, 8)), rng.choice((64, 128))
    Sq, BK = rng.randint(1, 32), rng.choice((32, 64, 128, 512))
    Sk = BK * rng.randint(1, 4096 // BK)
    q, k, v = tensors(rng, B, H, Sq, Sk, D, gpu)
    mask = random_mask(rng, B, H, Sq, Sk, gpu)
    o = sparse_attention_decode(q, k, v, mask, BK, num_splits=rng.choice((0, 0, 1, 3, 9)))
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL, (B, H, Sq, Sk, D, BK)


@pytest.mark.parametrize("seed", range(16))
def test_backward(gpu, seed):
    rng = random.Random(3000 + seed)
    B, H, D = rng.choice((1, 2)), rng.choice((1, 2, 3)), rng.choice((64, 128))
    Sq, Sk = 128 * rng.randint(1, 6), 128 * rng.randint(1, 6)
    q, k, v, do = tensors(rng, B, H, Sq, Sk, D, gpu, n=4)
    mask = random_mask(rng, B, H, Sq, Sk, gpu)
    me = mask.expand(B, H, Sq, Sk)
    BQ = rng.choice((32, 64, 128))
    o, lse = sparse_attention(q, k, v, me, BQ, 32, return_lse=True)
    got = sparse_attention_backward(do, q, k, v, o, lse, me)
    q32, k32, v32 = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(q32, k32, v32, attn_mask=mask).backward(do.float())
    for g, w, name in zip(got, (q32.grad, k32.grad, v32.grad), ("dq", "dk", "dv")):
        err = float((g.float() - w).abs().max()) / max(1.0, float(w.abs().max()))
        assert err <= TOL, (name, err, B, H, Sq, Sk, D)
