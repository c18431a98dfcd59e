"""Pins the oracle's two-pass forward (oracle_forward, following sparse_attn_kernel.py:28-63,
:103-146) against routines and exact answers that are not the oracle: torch's masked SDPA (the
reference's own checker, test_attn.py:40), a dense fp64 softmax, and special cases."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from sparseattention_amd import workloads as W


def sdpa(q, k, v, mask):
    return F.scaled_dot_product_attention(q, k, v, attn_mask=mask)


def test_cpu_plumbing_config_vs_sdpa_fp32():
    # B=1 H=4 S=512 D=64 fp32, 32x32 random blocks, p=0.5, 10 % partial, diagonal True: max-abs <= 1e-5
    B, H, S, D = 1, 4, 512, 64
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=0)
    mask = W.random_block_mask(S, 32, 0.5, seed=0)
    ref = sdpa(q, k, v, mask).numpy()
    for BQ, BK in ((32, 32), (128, 32), (32, 128), (64, 64)):
        out = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy()[None, None], BQ, BK)
        err = np.abs(out - ref).max()
        assert err <= 1e-5, f"tiles {BQ}x{BK}: max-abs {err}"


def test_vs_dense_fp64():
    B, H, S, D = 2, 2, 256, 32
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=3)
    mask = W.random_block_mask(S, 32, 0.6, seed=9, batch=B)
    want = oracle.forward_dense_fp64(q.numpy(), k.numpy(), v.numpy(), mask.numpy())
    got = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy(), 64, 32)
    assert np.abs(got - want).max() <= 2e-6
    # and the fp64 routine itself agrees with SDPA
    assert np.abs(want - sdpa(q.double(), k.double(), v.double(), mask).numpy()).max() <= 1e-12


def test_all_true_mask_equals_dense_attention():
    B, H, S, D = 1, 2, 128, 64
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=1)
    ones = torch.ones(S, S, dtype=torch.bool)
    got = oracle.forward(q.numpy(), k.numpy(), v.numpy(), ones.numpy()[None, None], 32, 32)
    want = F.scaled_dot_product_attention(q, k, v).numpy()
    assert np.abs(got - want).max() <= 1e-5


def test_one_hot_rows_copy_value_rows_exactly():
    # each query attends to exactly one key -> softmax weight is exactly 1 -> o[r] == v[c] bit for bit
    B, H, S, D = 1, 1, 128, 16
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=2)
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(5))
    mask = torch.zeros(S, S, dtype=torch.bool)
    mask[torch.arange(S), perm] = True
    got = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy()[None, None], 32, 16)
    assert np.array_equal(got[0, 0], v.numpy()[0, 0, perm.numpy()])


def test_identical_keys_give_uniform_average_of_allowed_values():
    B, H, S, D = 1, 1, 128, 32
    q, _, v = W.qkv(B, H, S, D, torch.float32, seed=4)
    k = torch.ones(B, H, S, D) * 0.25
    mask = W.random_block_mask(S, 16, 0.5, seed=8)
    got = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy()[None, None], 32, 32)
    m = mask.double()
    want = (m @ v[0, 0].double()) / m.sum(-1, keepdim=True)
    assert np.abs(got[0, 0] - want.numpy()).max() <= 1e-5


def test_rows_masked_in_first_partial_tile_stay_finite():
    # The hazard the reference leaves open (sparse_attn_kernel.py:53): a Q tile with no full tile
    # whose first partial tile has rows with no attended key.  Document boundary inside a Q tile.
    B, H, S, D = 1, 2, 256, 32
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=6)
    doc = torch.tensor([0] * 40 + [1] * 100 + [2] * 116)
    idx = torch.arange(S)
    mask = (doc[:, None] == doc[None, :]) & (idx[None, :] <= idx[:, None])
    meta = oracle.classify(mask.numpy()[None, None], 128, 32)
    assert meta.unmasked_lens[0, 0, 0] == 0  # the hazard is actually exercised
    got = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy()[None, None], 128, 32, meta=None)
    assert np.isfinite(got).all()
    assert np.abs(got - sdpa(q, k, v, mask).numpy()).max() <= 1e-5


def test_rows_without_any_key_give_zero():
    B, H, S, D = 1, 1, 64, 16
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=7)
    mask = torch.ones(S, S, dtype=torch.bool)
    mask[5] = False   # one dead row inside an otherwise attended tile
    mask[32:] = False  # a whole Q tile with empty lists
    got = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask.numpy()[None, None], 32, 32)
    assert np.all(got[0, 0, 5] == 0) and np.all(got[0, 0, 32:] == 0)
    live = [r for r in range(32) if r != 5]
    want = F.scaled_dot_product_attention(q[:, :, live], k, v).numpy()
    assert np.abs(got[0, 0, live] - want[0, 0]).max() <= 1e-5


def test_explicit_metadata_and_list_order():
    B, H, S, D = 1, 2, 128, 32
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=8)
    mask = W.random_block_mask(S, 32, 0.3, seed=1).numpy()[None, None]
    mask = np.broadcast_to(mask, (B, H, S, S))
    meta = oracle.classify(mask, 32, 32)
    a = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask, 32, 32, meta=meta)
    b = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask, 32, 32)
    assert np.array_equal(a, b)
    # reversing the valid part of each list only reorders the accumulation: same result up to rounding
    rev = oracle.OracleMetadata(meta.unmasked_kv_ids.copy(), meta.unmasked_lens, meta.masked_kv_ids.copy(), meta.masked_lens)
    for ids, lens in ((rev.unmasked_kv_ids, rev.unmasked_lens), (rev.masked_kv_ids, rev.masked_lens)):
        for h in range(H):
            for i in range(S // 32):
                n = lens[0, h, i]
                ids[0, h, i, :n] = ids[0, h, i, :n][::-1]
    c = oracle.forward(q.numpy(), k.numpy(), v.numpy(), mask, 32, 32, meta=rev)
    assert np.abs(a - c).max() <= 1e-5 and not np.array_equal(meta.unmasked_kv_ids, rev.unmasked_kv_ids)


def test_bf16_rounding_of_p():
    # with P rounded to bf16 before P.V (what the kernels do for bf16 inputs) the result stays within
    # the bf16 tolerance of SDPA and differs from the unrounded run
    B, H, S, D = 1, 2, 256, 64
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=9)
    mask = W.causal_mask(S)
    qf, kf, vf = (t.float().numpy() for t in (q, k, v))
    exact = oracle.forward(qf, kf, vf, mask.numpy()[None, None], 128, 32, p_round=0)
    rounded = oracle.forward(qf, kf, vf, mask.numpy()[None, None], 128, 32, p_round=1)
    ref = sdpa(q.float(), k.float(), v.float(), mask).numpy()
    assert np.abs(exact - ref).max() <= 1e-5
    assert 0 < np.abs(rounded - ref).max() <= 2e-2


def test_fp16_and_bf16_rounding_helpers():
    # the helpers that round P must agree with torch's casts (round to nearest even), incl. subnormals,
    # ties and the fp16 overflow threshold
    g = torch.Generator().manual_seed(0)
    vals = torch.cat([
        torch.linspace(0, 1, 4097), torch.rand(2000, generator=g) * 2.0 ** -14, torch.rand(2000, generator=g) * 2.0 ** -24,
        torch.tensor([2.0 ** -20, 3e-5, 6.1e-5, 0.333333, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -11,
                      1.0 + 3 * 2.0 ** -11, 65504.0, 65519.9, 65520.0, 1e30]),
    ])
    vals = torch.cat([vals, -vals])
    want_bf16 = vals.to(torch.bfloat16).float().tolist()
    want_fp16 = vals.to(torch.float16).float().tolist()
    for x, wb, wh in zip(vals.tolist(), want_bf16, want_fp16):
        assert oracle.round_bf16(x) == wb, x
        assert oracle.round_fp16(x) == wh, x
