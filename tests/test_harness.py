"""The benchmark harness (sparseattention_amd/test_attn.py): mask family, result layout, and a reduced sweep
on the GPU whose outputs must match masked SDPA."""
import json

import pytest
import torch

from sparseattention_amd import test_attn as harness


def test_random_blocked_mask_family():
    torch.manual_seed(1352)
    m = harness.random_blocked_mask(2, 256, 512, 64, 128, 0.3, device="cpu")
    assert m.shape == (2, 1, 256, 512) and m.dtype == torch.bool
    t = m[:, 0].reshape(2, 4, 64, 4, 128).float().mean((2, 4))
    # every block is all clear, all set, or a coin-flip block (about half set)
    assert (((t == 0) | (t == 1) | ((t > 0.4) & (t < 0.6)))).all()
    # same seed, same mask; the draw order (blocks, then coin-flip entries) is part of the contract
    torch.manual_seed(1352)
    assert torch.equal(m, harness.random_blocked_mask(2, 256, 512, 64, 128, 0.3, device="cpu"))
    torch.manual_seed(7)
    frac = [harness.random_blocked_mask(1, 1024, 1024, 32, 32, p, device="cpu").float().mean().item() for p in (0.1, 0.5, 0.9)]
    assert frac[0] < frac[1] < frac[2]
    assert abs(frac[1] - (0.4 + 0.05)) < 0.05  # P(set) = p - 0.1 for p > 0.1, plus half of the 10 % coin-flip blocks


@pytest.mark.gpu
def test_reduced_sweep_layout_and_match(gpu, tmp_path):
    res = harness.sweep(B=2, H=2, Sq=1024, Sk=1024, D=128, BLOCK_Q=128, BLOCK_K=32, mask_block=128,
                        p_values=[0.2, 0.5, 0.8], verbose=False)
    assert set(res) == {"config", "results"}
    assert set(res["config"]) == {"shape", "BLOCK_Q", "BLOCK_K", "total_flops"}
    assert res["config"]["total_flops"] == 4 * 2 * 2 * 1024 * 1024 * 128
    want = {"p", "fraction_unmasked", "useful_flops", "ref_time_ms", "sparse_time_ms", "flex_time_ms",
            "ref_tflops_per_sec", "sparse_tflops_per_sec", "flex_tflops_per_sec"}
    for r in res["results"]:
        assert want <= set(r)
        assert r["match"], f"p={r['p']}: max abs err {r['max_abs_err']}"
        assert r["sparse_time_ms"] > 0 and r["ref_time_ms"] > 0
    json.dumps(res)  # serialisable as written by main()
