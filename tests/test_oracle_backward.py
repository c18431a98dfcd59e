"""Pins the oracle's dense fp64 backward (oracle.backward_dense_fp64) against routines that are not the oracle:
torch autograd through masked SDPA in float64, finite differences, and special cases with closed forms."""
import numpy as np
import torch
import torch.nn.functional as F

import oracle
from sparseattention_amd import workloads as W


def autograd_grads(q, k, v, mask, do):
    q, k, v = (t.double().clone().requires_grad_(True) for t in (q, k, v))
    o = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    o.backward(do.double())
    return q.grad.numpy(), k.grad.numpy(), v.grad.numpy()


def test_vs_autograd_through_sdpa_fp64():
    B, H, S, D = 2, 2, 192, 32
    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=1)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(2))
    mask = W.random_block_mask(S, 32, 0.5, seed=3, batch=B)
    got = oracle.backward_dense_fp64(q.numpy(), k.numpy(), v.numpy(), mask.numpy(), do.numpy())
    want = autograd_grads(q, k, v, mask, do)
    for g, w, name in zip(got, want, ("dq", "dk", "dv")):
        assert np.abs(g - w).max() <= 1e-12, name


def test_cross_attention_shapes_and_finite_differences():
    B, H, Sq, Sk, D = 1, 1, 5, 7, 4
    g = torch.Generator().manual_seed(4)
    q, k, v, do = (torch.randn(B, H, n, D, generator=g, dtype=torch.float64) for n in (Sq, Sk, Sk, Sq))
    mask = torch.rand(Sq, Sk, generator=g) < 0.6
    mask[:, 0] = True
    dq, dk, dv = oracle.backward_dense_fp64(q.numpy(), k.numpy(), v.numpy(), mask.numpy(), do.numpy())

    def loss(qq, kk, vv):
        return float((oracle.forward_dense_fp64(qq, kk, vv, mask.numpy()) * do.numpy()).sum())

    eps = 1e-6
    base = [q.numpy(), k.numpy(), v.numpy()]
    for which, grad in enumerate((dq, dk, dv)):
        for idx in ((0, 0, 1, 2), (0, 0, 3, 0), (0, 0, 4, 3)):
            hi, lo = list(base), list(base)
            hi[which], lo[which] = base[which].copy(), base[which].copy()
            hi[which][idx] += eps
            lo[which][idx] -= eps
            fd = (loss(*hi) - loss(*lo)) / (2 * eps)
            assert abs(fd - grad[idx]) <= 1e-7, (which, idx, fd, grad[idx])


def test_special_cases():
    B, H, S, D = 1, 1, 8, 4
    g = torch.Generator().manual_seed(5)
    q, k, v, do = (torch.randn(B, H, S, D, generator=g, dtype=torch.float64).numpy() for _ in range(4))
    # one-hot rows: o[r] = v[c] whatever q and k are, so dq = dk = 0 and dv scatters do
    perm = torch.randperm(S, generator=g).numpy()
    mask = np.zeros((S, S), bool)
    mask[np.arange(S), perm] = True
    dq, dk, dv = oracle.backward_dense_fp64(q, k, v, mask, do)
    assert np.abs(dq).max() <= 1e-14 and np.abs(dk).max() <= 1e-14  # dP - delta cancels to rounding
    assert np.array_equal(dv[0, 0, perm], do[0, 0])
    # dead rows contribute nothing; identical keys give uniform P, hence dv[j] = sum_i do[i] / S and dq = 0
    kk = np.broadcast_to(k[:, :, :1], k.shape).copy()
    mask = np.ones((S, S), bool)
    mask[3] = False
    dq, dk, dv = oracle.backward_dense_fp64(q, kk, v, mask, do)
    live = np.arange(S) != 3
    assert np.abs(dq).max() <= 1e-15
    assert np.abs(dv[0, 0] - do[0, 0][live].sum(0) / S).max() <= 1e-15
