"""Parity of the backward pass (sa_sparse_attention_bwd through the Python binding).

The reference has no backward; the checkers are the dense fp64 derivative of the oracle package (pinned against
autograd and finite differences in tests/test_oracle_backward.py) on small shapes and torch autograd through
fp32 masked SDPA on the same bf16 inputs on all shapes.  Tolerance: gradients of bf16 inputs within 2e-2 max-abs
of the fp32 reference relative to the gradient's own scale (max-abs of the reference, at least 1)."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from sparseattention_amd import (compute_backward_metadata, compute_mask_kernel, sparse_attention,
                                 sparse_attention_backward, sparse_attention_trainable, workloads as W)

pytestmark = pytest.mark.gpu

TOL = 2e-2


def sdpa_grads(q, k, v, mask, do):
    q32, k32, v32 = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    o = F.scaled_dot_product_attention(q32, k32, v32, attn_mask=mask)
    o.backward(do.float())
    return q32.grad, k32.grad, v32.grad


def check(got, want, what):
    for g, w, name in zip(got, want, ("dq", "dk", "dv")):
        assert not torch.isnan(g).any(), f"{what}: {name} has NaN"
        scale = max(1.0, float(w.abs().max()))
        err = float((g.float() - w.float().to(g.device)).abs().max()) / scale
        assert err <= TOL, f"{what}: {name} off by {err:.3e} of its scale {scale:.2f}"


def live_mask(S, block, p, seed, device, batch=None):
    m = W.random_block_mask(S, block, p, seed=seed, device=device, batch=batch)
    return m


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("S,block,p", [(256, 32, 0.3), (512, 64, 0.5), (512, 32, 0.7)])
def test_against_oracle_and_autograd(gpu, S, block, p, D):
    B, H = 1, 2
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=S + block, device=gpu)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(7)).to(gpu, torch.bfloat16)
    mask = live_mask(S, block, p, seed=S, device=gpu)
    o, lse = sparse_attention(q, k, v, mask, 128, 32, return_lse=True)
    got = sparse_attention_backward(do, q, k, v, o, lse, mask)
    torch.cuda.synchronize()
    want = oracle.backward_dense_fp64(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                      mask.cpu().numpy(), do.float().cpu().numpy())
    check(got, [torch.from_numpy(w) for w in want], "vs oracle")
    check(got, sdpa_grads(q, k, v, mask, do), "vs autograd")


@pytest.mark.parametrize("D", [64, 128])
def test_causal_dense_and_cross_shapes(gpu, D):
    B, H = 2, 2
    for Sq, Sk, kind in ((512, 512, "causal"), (256, 512, "dense"), (512, 256, "random")):
        q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=Sq + Sk, device=gpu, Sk=Sk)
        do = torch.randn(B, H, Sq, D, generator=torch.Generator().manual_seed(8)).to(gpu, torch.bfloat16)
        if kind == "causal":
            mask = W.causal_mask(Sq, gpu)
        elif kind == "dense":
            mask = torch.ones(Sq, Sk, dtype=torch.bool, device=gpu)
        else:
            mask = (torch.rand(B, 1, Sq, Sk, generator=torch.Generator().manual_seed(9)) < 0.5).to(gpu)
            mask[..., 0] = True
        me = mask.expand(B, H, Sq, Sk)
        o, lse = sparse_attention(q, k, v, me, 128, 64, return_lse=True)
        got = sparse_attention_backward(do, q, k, v, o, lse, me)
        check(got, sdpa_grads(q, k, v, mask, do), kind)


def test_dead_rows_and_empty_tiles(gpu):
    B, H, S, D = 1, 1, 512, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=3, device=gpu)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(4)).to(gpu, torch.bfloat16)
    mask = live_mask(S, 64, 0.5, seed=5, device=gpu).clone()
    mask[100] = False        # a query that attends to nothing
    mask[:, 128:256] = False  # keys nobody attends to: dk = dv = 0 there
    mask[0, 0] = True
    o, lse = sparse_attention(q, k, v, mask, 128, 32, return_lse=True)
    dq, dk, dv = sparse_attention_backward(do, q, k, v, o, lse, mask)
    assert (dq[0, 0, 100] == 0).all() and (dk[0, 0, 128:256] == 0).all() and (dv[0, 0, 128:256] == 0).all()
    want = oracle.backward_dense_fp64(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                      mask.cpu().numpy(), do.float().cpu().numpy())
    check((dq, dk, dv), [torch.from_numpy(w) for w in want], "dead rows")


def test_autograd_function_and_metadata_reuse(gpu):
    B, H, S, D = 1, 2, 256, 128
    q, k, v = (t.requires_grad_(True) for t in W.qkv(B, H, S, D, torch.bfloat16, seed=11, device=gpu))
    mask = W.causal_mask(S, gpu)
    me = mask[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, 128, 32)
    bmd = compute_backward_metadata(me)
    o = sparse_attention_trainable(q, k, v, me, 128, 32, md, bmd)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(12)).to(gpu, torch.bfloat16)
    o.backward(do)
    check((q.grad, k.grad, v.grad), sdpa_grads(q.detach(), k.detach(), v.detach(), mask, do), "autograd function")


@pytest.mark.parametrize("D", [64, 128])
def test_fp16(gpu, D):
    B, H, S = 1, 2, 256
    q, k, v = W.qkv(B, H, S, D, torch.float16, seed=13, device=gpu)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(14)).to(gpu, torch.float16)
    mask = live_mask(S, 32, 0.4, seed=15, device=gpu)
    o, lse = sparse_attention(q, k, v, mask, 64, 32, return_lse=True)
    got = sparse_attention_backward(do, q, k, v, o, lse, mask)
    for g, w in zip(got, sdpa_grads(q, k, v, mask, do)):
        assert float((g.float() - w).abs().max()) / max(1.0, float(w.abs().max())) <= 4e-3


def test_strided_storage_batch_masks_and_errors(gpu):
    # [B,S,H,D] storage seen as [B,H,S,D]; one mask per batch element, broadcast over heads
    B, H, S, D = 2, 3, 256, 128
    g = torch.Generator().manual_seed(21)
    q, k, v, do = (torch.randn(B, S, H, D, generator=g).to(gpu, torch.bfloat16).transpose(1, 2) for _ in range(4))
    mask = live_mask(S, 32, 0.5, seed=22, device=gpu, batch=B)
    me = mask.expand(B, H, S, S)
    o, lse = sparse_attention(q, k, v, me, 128, 32, return_lse=True)
    got = sparse_attention_backward(do, q, k, v, o, lse, me)
    assert got[0].stride() == q.stride()
    check(got, sdpa_grads(q, k, v, mask, do), "strided")
    bmd = compute_backward_metadata(me)
    assert bmd.by_key.unmasked_kv_ids.shape == (B, H, S // 128, S // 64) and bmd.by_key.unmasked_kv_ids.stride(1) == 0
    again = sparse_attention_backward(do, q, k, v, o, lse, me, bmd)
    assert all(torch.equal(a, b) for a, b in zip(got, again))
    # lengths that are not multiples of 128 have no backward kernel: the wrapper pads (more in test_gpu_head_dims.py)
    qs, ks, vs = W.qkv(1, 1, 192, 128, torch.bfloat16, seed=24, device=gpu)
    ms = torch.ones(192, 192, dtype=torch.bool, device=gpu)
    os_, lses = sparse_attention(qs, ks, vs, ms, 64, 32, return_lse=True)
    got = sparse_attention_backward(os_, qs, ks, vs, os_, lses, ms)
    check(got, sdpa_grads(qs, ks, vs, ms, os_), "padded to 256")


def test_full_size_causal_planes_against_autograd(gpu):
    B, H, S, D = 8, 32, 4096, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=31, device=gpu)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(32)).to(gpu, torch.bfloat16)
    mask = W.causal_mask(S, gpu)
    me = mask[None, None].expand(B, H, S, S)
    o, lse = sparse_attention(q, k, v, me, 128, 32, return_lse=True)
    dq, dk, dv = sparse_attention_backward(do, q, k, v, o, lse, me)
    assert not (torch.isnan(dq).any() or torch.isnan(dk).any() or torch.isnan(dv).any())
    for b, h in ((0, 0), (5, 13), (7, 31)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        check((dq[sl], dk[sl], dv[sl]), sdpa_grads(q[sl], k[sl], v[sl], mask, do[sl]), f"plane {b},{h}")
    # every plane: dv is a P-weighted sum of dO rows, so column sums of dv equal those of dO (P rows sum to one)
    assert (dv.float().sum(2) - do.float().sum(2)).abs().max() <= 0.5


def test_transposed_mask_copy_changes_nothing(gpu):
    B, H, S, D = 2, 2, 512, 128
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=41, device=gpu)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(42)).to(gpu, torch.bfloat16)
    mask = (torch.rand(B, 1, S, S, generator=torch.Generator().manual_seed(43)) < 0.5).to(gpu)
    me = mask.expand(B, H, S, S)
    o, lse = sparse_attention(q, k, v, me, 128, 32, return_lse=True)
    bmd = compute_backward_metadata(me, pack_partial=False)
    assert bmd.by_query.packed_masks is None and bmd.by_key.packed_masks is None
    assert bmd.transposed_mask.shape == (B, H, S, S) and bmd.transposed_mask.stride(1) == 0
    with_copy = sparse_attention_backward(do, q, k, v, o, lse, me, bmd)
    bmd.transposed_mask = None
    without = sparse_attention_backward(do, q, k, v, o, lse, me, bmd)
    assert all(torch.equal(a, b) for a, b in zip(with_copy, without))
    check(with_copy, sdpa_grads(q, k, v, mask, do), "every tile partial")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_packed_partial_tiles_replace_both_masks(gpu, D, dtype):
    # the same gradients, bit for bit, from the packed PARTIAL tiles as from the bool mask and its transposed copy;
    # with packed tiles in both lists no mask is passed at all
    B, H, Sq, Sk = 2, 3, 384, 640
    q, _, _ = W.qkv(B, H, Sq, D, dtype, seed=51, device=gpu)
    _, k, v = W.qkv(B, H, Sk, D, dtype, seed=52, device=gpu)
    do = torch.randn(B, H, Sq, D, generator=torch.Generator().manual_seed(53)).to(gpu, dtype)
    g = torch.Generator().manual_seed(54)
    # squares of 128 in turn full, ragged and empty, so both tilings (128 x 64 each way) see all three kinds; the
    # ragged ones mix random entries with empty blocks of 32; one mask per batch element
    i, j = torch.arange(Sq // 128)[:, None], torch.arange(Sk // 128)[None, :]
    kind = ((i + 2 * j) % 3).repeat_interleave(128, 0).repeat_interleave(128, 1)
    fine = torch.rand(B, 1, Sq, Sk, generator=g) < 0.6
    holes = (torch.rand(B, 1, Sq // 32, Sk // 32, generator=g) < 0.3).repeat_interleave(32, 2).repeat_interleave(32, 3)
    mask = ((kind == 0) | ((kind == 1) & fine & ~holes)).to(gpu)
    mask[..., 0] = True
    me = mask.expand(B, H, Sq, Sk)
    o, lse = sparse_attention(q, k, v, me, 128, 32, return_lse=True)
    plain = compute_backward_metadata(me, pack_partial=False)
    packed = compute_backward_metadata(me)
    assert packed.transposed_mask is None
    assert packed.by_query.packed_masks.shape == (B, H, Sq // 128, Sk // 64, 1024)
    assert packed.by_key.packed_masks.shape == (B, H, Sk // 128, Sq // 64, 1024)
    assert packed.by_key.packed_masks.stride(1) == 0
    assert int(packed.by_query.masked_lens.sum()) > 0 and int(packed.by_query.unmasked_lens.sum()) > 0
    want = sparse_attention_backward(do, q, k, v, o, lse, me, plain)
    got = sparse_attention_backward(do, q, k, v, o, lse, None, packed)
    assert all(torch.equal(a, b) for a, b in zip(got, want))
    # one orientation packed, the other from the mask
    packed.by_key.packed_masks = None
    mixed = sparse_attention_backward(do, q, k, v, o, lse, me, packed)
    assert all(torch.equal(a, b) for a, b in zip(mixed, want))
    with pytest.raises(ValueError):
        sparse_attention_backward(do, q, k, v, o, lse, None, packed)
    if dtype == torch.bfloat16:
        check(got, sdpa_grads(q, k, v, mask, do), "packed tiles")
