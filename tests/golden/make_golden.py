"""Writes tests/golden/kat_*.npz: small known-answer cases for the classification and the forward.

Nothing here comes from the reference package.  Expected index lists are produced by the numpy
popcount classification (oracle.classify_numpy) and expected outputs by a dense float64 masked
softmax (oracle.forward_dense_fp64) on inputs that are exactly representable in bf16, so the same
files check the C oracle on the CPU and the HIP kernels on the GPU.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from sparseattention_amd import workloads as W  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def doc_mask(lengths):
    doc = torch.repeat_interleave(torch.arange(len(lengths)), torch.tensor(lengths))
    idx = torch.arange(len(doc))
    return (doc[:, None] == doc[None, :]) & (idx[None, :] <= idx[:, None])


CASES = {
    # name: (mask [S,S] bool, B, H, D, BQ, BK, seed)
    "random_block": (W.random_block_mask(128, 16, 0.5, seed=21), 1, 1, 64, 64, 32, 1),
    "causal": (W.causal_mask(256), 1, 1, 64, 128, 32, 2),
    "documents": (doc_mask([20, 50, 58]), 1, 1, 64, 64, 16, 3),
    "window_prefix": (W.composed_mask(128, window=24, prefix=40), 1, 1, 128, 32, 64, 4),
}


def main():
    for name, (mask, B, H, D, BQ, BK, seed) in CASES.items():
        S = mask.shape[0]
        q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=seed)
        qf, kf, vf = (t.float().numpy() for t in (q, k, v))
        m4 = np.broadcast_to(mask.numpy()[None, None], (B, H, S, S))
        meta = oracle.classify_numpy(m4, BQ, BK)
        out = oracle.forward_dense_fp64(qf, kf, vf, m4)
        np.savez_compressed(
            os.path.join(HERE, f"kat_{name}.npz"),
            mask=np.packbits(mask.numpy(), axis=-1), S=S, B=B, H=H, D=D, BQ=BQ, BK=BK,
            q=q.view(torch.int16).numpy(), k=k.view(torch.int16).numpy(), v=v.view(torch.int16).numpy(),
            unmasked_kv_ids=meta.unmasked_kv_ids[0, 0], unmasked_lens=meta.unmasked_lens[0, 0],
            masked_kv_ids=meta.masked_kv_ids[0, 0], masked_lens=meta.masked_lens[0, 0],
            out_fp64=out.astype(np.float32),
        )
        print(name, "written")


if __name__ == "__main__":
    main()
