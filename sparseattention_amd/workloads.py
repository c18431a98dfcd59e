"""Synthetic masks and inputs of the benchmark configurations.

The reference's harness builds its masks in ``random_blocked_mask``
(``sparseattention/test_attn.py:17-29``): a grid of square blocks, each empty, full or - for a
flat 10 % of blocks - filled with fair coin flips.  The generators here produce that family and
the structured masks (causal, documents, sliding window + prefix) the benchmark is quoted on.
All take a seed and are deterministic: random draws come from a CPU generator, whatever the
target device.
"""
from __future__ import annotations

import torch


def causal_mask(S: int, device="cpu") -> torch.Tensor:
    """bool [S,S], True where kv <= q."""
    idx = torch.arange(S, device=device)
    return idx[None, :] <= idx[:, None]


def random_block_mask(S: int, block: int, p_empty: float, seed: int, device="cpu", partial_fraction: float = 0.1,
                      batch: int | None = None) -> torch.Tensor:
    """Random block mask, bool [S,S] (or [batch,1,S,S]).

    The S x S plane is tiled with ``block`` x ``block`` blocks.  One uniform draw u per block:
    u >= 1 - partial_fraction -> the block's entries are i.i.d. Bernoulli(0.5) (this overrides
    the other two cases, as in test_attn.py:21-22); otherwise u <= p_empty -> all False; else
    all True.  The diagonal is then forced True so that no query row is left without a key.
    """
    if S % block:
        raise ValueError("S must be a multiple of block")
    g = torch.Generator(device="cpu").manual_seed(seed)
    n = S // block
    planes = batch if batch is not None else 1
    u = torch.rand(planes, n, n, generator=g)
    label = torch.ones(planes, n, n, dtype=torch.uint8)
    label[u <= p_empty] = 0
    label[u >= 1.0 - partial_fraction] = 2
    coin = torch.randint(0, 2, (planes, S, S), generator=g, dtype=torch.uint8)
    label = label.repeat_interleave(block, 1).repeat_interleave(block, 2)
    mask = torch.where(label == 2, coin, label).to(torch.bool)
    del coin, label
    mask.diagonal(dim1=-2, dim2=-1).fill_(True)
    mask = mask.to(device)
    return mask.unsqueeze(1) if batch is not None else mask[0]


def document_lengths(S: int, seed: int, lo: int = 256, hi: int = 4096) -> list[int]:
    """Document lengths uniform in [lo, hi], the last one truncated so that they sum to S."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    lens, total = [], 0
    while total < S:
        n = int(torch.randint(lo, hi + 1, (1,), generator=g))
        n = min(n, S - total)
        lens.append(n)
        total += n
    return lens


def document_mask(S: int, seed: int, device="cpu", lo: int = 256, hi: int = 4096) -> torch.Tensor:
    """Causal attention within each document, none across documents.  bool [S,S]."""
    lens = document_lengths(S, seed, lo, hi)
    doc = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(device)
    idx = torch.arange(S, device=device)
    mask = torch.empty(S, S, dtype=torch.bool, device=device)
    step = 2048
    for r0 in range(0, S, step):
        r1 = min(S, r0 + step)
        mask[r0:r1] = (doc[r0:r1, None] == doc[None, :]) & (idx[None, :] <= idx[r0:r1, None])
    return mask


def composed_mask(S: int, window: int = 1024, prefix: int = 2048, device="cpu") -> torch.Tensor:
    """(causal AND sliding window) OR bidirectional prefix:
    ``(kv <= q and q - kv < window) or (q < prefix and kv < prefix)``.  bool [S,S], built in row slabs."""
    idx = torch.arange(S, device=device)
    mask = torch.empty(S, S, dtype=torch.bool, device=device)
    step = 2048
    for r0 in range(0, S, step):
        r1 = min(S, r0 + step)
        q = idx[r0:r1, None]
        kv = idx[None, :]
        mask[r0:r1] = ((kv <= q) & (q - kv < window)) | ((q < prefix) & (kv < prefix))
    return mask


def qkv(B: int, H: int, S: int, D: int, dtype, seed: int, device="cpu", Sk: int | None = None):
    """q, k, v ~ N(0,1) from a seeded generator on ``device``."""
    g = torch.Generator(device=device).manual_seed(seed)
    Sk = S if Sk is None else Sk
    q = torch.randn(B, H, S, D, generator=g, device=device, dtype=torch.float32).to(dtype)
    k = torch.randn(B, H, Sk, D, generator=g, device=device, dtype=torch.float32).to(dtype)
    v = torch.randn(B, H, Sk, D, generator=g, device=device, dtype=torch.float32).to(dtype)
    return q, k, v
