"""Benchmark harness: masked SDPA against the block-sparse forward across block sparsity p.

Plays the part of the reference's sparseattention/test_attn.py: the same family of random block masks
(:17-29), the same per-point check and timing (:32-76), the same sweep p = 0.1 ... 0.9 at
B=8, H=16, S=4096, D=128, tiles 128x32 and the same attention_results.json layout (:79-128), so that a
result file can be laid beside the reference's.  Differences, on purpose:

  * timing uses HIP events around repeated launches (do_bench below), not triton.testing.do_bench;
  * FlexAttention is not run (it needs a tracing compiler); its fields are written as null;
  * the plot is optional (--plot) and skipped when matplotlib is not importable.

Run:  python -m sparseattention_amd.test_attn [--out attention_results.json] [--plot perf.png]
"""
from __future__ import annotations

import argparse
import json

import torch
from torch.nn import functional as F

from .mask_utils import compute_mask_kernel
from .sparse_attn_kernel import sparse_attention


def random_blocked_mask(B, Sq, Sk, BLOCK_Q, BLOCK_K, p, device="cuda"):
    """Bool mask [B,1,Sq,Sk] made of BLOCK_Q x BLOCK_K blocks: a block is set with probability p, and the
    blocks whose uniform draw falls in the top 10 % are filled with coin flips instead (the reference's
    family, test_attn.py:17-29; one torch.rand over the blocks, then one torch.randint over the entries of
    the coin-flip blocks, in that order, on the CPU generator)."""
    nq, nk = Sq // BLOCK_Q, Sk // BLOCK_K
    u = torch.rand(B * nq * nk)
    kind = torch.where(u >= 0.9, 2, torch.where(u > 1 - p, 1, 0)).to(torch.int)
    kind = kind.view(B, nq, nk)
    cells = kind.repeat_interleave(BLOCK_Q, 1).repeat_interleave(BLOCK_K, 2).view(B, 1, Sq, Sk)
    noisy = cells == 2
    cells[noisy] = torch.randint(0, 2, (int(noisy.sum()),)).to(torch.int)
    return cells.to(torch.bool).to(device)


def do_bench(fn, warmup_ms=25.0, rep=20):
    """Median time of fn() in ms: HIP events on the current stream around each of ``rep`` launches that follow each
    other without a host synchronisation in between, after at least ``warmup_ms`` of untimed launches (as
    triton.testing.do_bench warms up by time, test_attn.py:64-68: after the seconds of host work that make a mask the
    device has dropped to a low power state and its first launches run several times slow)."""
    import time

    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < warmup_ms:
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(rep)]
    for start, end in pairs:
        start.record()
        fn()
        end.record()
    torch.cuda.synchronize()
    times = sorted(start.elapsed_time(end) for start, end in pairs)
    return times[len(times) // 2]


def test_attn(B, H, Sq, Sk, D, mask, BLOCK_Q=32, BLOCK_K=128, dtype=torch.bfloat16, verbose=True):
    """One point of the sweep (test_attn.py:32-76): outputs compared with assert_close(atol=1e-2,
    rtol=1e-4) against masked SDPA, then both timed; the mask preprocessing is timed on its own."""
    q = torch.randn(B, H, Sq, D, dtype=dtype, device="cuda")
    k = torch.randn(B, H, Sk, D, dtype=dtype, device="cuda")
    v = torch.randn(B, H, Sk, D, dtype=dtype, device="cuda")
    mask_expanded = mask.expand(B, H, Sq, Sk)
    mask_metadata = compute_mask_kernel(mask_expanded, BLOCK_Q, BLOCK_K)

    ref_attn = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    sparse_attn = sparse_attention(q, k, v, mask_expanded, BLOCK_Q, BLOCK_K, mask_metadata=mask_metadata)
    # rows without any attended key: SDPA gives NaN, the sparse kernel 0; compare the rows that exist
    live = mask.any(-1).expand(B, H, Sq)
    match = True
    try:
        torch.testing.assert_close(sparse_attn[live], ref_attn[live], atol=1e-2, rtol=1e-4)
        if verbose:
            print("sparse and ref match!")
    except AssertionError as e:  # reported, not fatal, as in the reference
        match = False
        if verbose:
            print(e)

    ref_time = do_bench(lambda: F.scaled_dot_product_attention(q, k, v, attn_mask=mask))
    sparse_time = do_bench(
        lambda: sparse_attention(q, k, v, mask_expanded, BLOCK_Q, BLOCK_K, mask_metadata=mask_metadata))
    mask_time = do_bench(lambda: compute_mask_kernel(mask_expanded, BLOCK_Q, BLOCK_K))
    if verbose:
        print(f"MASK_TIME: {mask_time:.3f}ms")
        print(f"SPARSE_TIME: {sparse_time:.3f}ms")
        print(f"REF_TIME: {ref_time:.3f}ms")
    return {"ref_time": ref_time, "sparse_time": sparse_time, "flex_time": None, "mask_time": mask_time,
            "match": match, "max_abs_err": float((sparse_attn[live].float() - ref_attn[live].float()).abs().max())}


test_attn.__test__ = False  # a benchmark step with required arguments, not a pytest case


def sweep(B=8, H=16, Sq=4096, Sk=4096, D=128, BLOCK_Q=128, BLOCK_K=32, mask_block=128, p_values=None, seed=1352,
          verbose=True):
    """The reference's __main__ (test_attn.py:79-128) as a function; returns the attention_results dict."""
    torch.manual_seed(seed)
    total_flops = 2 * 2 * B * H * Sq * Sk * D
    out = {"config": {"shape": (B, H, Sq, Sk), "BLOCK_Q": BLOCK_Q, "BLOCK_K": BLOCK_K, "total_flops": total_flops},
           "results": []}
    for p in (p_values if p_values is not None else [i / 10 for i in range(1, 10)]):
        mask = random_blocked_mask(B, Sq, Sk, mask_block, mask_block, p)
        fraction_unmasked = float(mask.sum() / mask.numel())
        if verbose:
            print(f"p: {p:.2f}, fraction_unmasked: {fraction_unmasked:.2f}")
        r = test_attn(B, H, Sq, Sk, D, mask, BLOCK_Q, BLOCK_K, verbose=verbose)
        useful_flops = total_flops * fraction_unmasked
        ref_s = useful_flops / (r["ref_time"] / 1000)
        sparse_s = useful_flops / (r["sparse_time"] / 1000)
        out["results"].append({
            "p": p,
            "fraction_unmasked": fraction_unmasked,
            "useful_flops": useful_flops,
            "ref_time_ms": r["ref_time"],
            "sparse_time_ms": r["sparse_time"],
            "flex_time_ms": None,
            "ref_tflops_per_sec": ref_s / 1e12,
            "sparse_tflops_per_sec": sparse_s / 1e12,
            "flex_tflops_per_sec": None,
            "mask_time_ms": r["mask_time"],       # extra fields: not in the reference's file
            "match": r["match"],
            "max_abs_err": r["max_abs_err"],
        })
        if verbose:
            print(f"  FLOPS/s - ref: {ref_s / 1e12:.2f} TFLOPS/s, sparse: {sparse_s / 1e12:.2f} TFLOPS/s")
    return out


def plot(results, path):
    try:
        import matplotlib
        matplotlib.use("Agg")
        import matplotlib.pyplot as plt
    except ImportError:
        print("matplotlib is not importable: no plot")
        return False
    ps = [r["p"] for r in results["results"]]
    plt.figure(figsize=(10, 6))
    plt.plot(ps, [r["ref_tflops_per_sec"] for r in results["results"]], "b-o", label="Reference (SDPA)")
    plt.plot(ps, [r["sparse_tflops_per_sec"] for r in results["results"]], "r-s", label="Sparse kernel (HIP, MI355X)")
    plt.xlabel("Fraction of blocks unmasked")
    plt.ylabel("TFLOPS/s")
    plt.title("Attention performance vs sparsity")
    plt.legend()
    plt.grid(True, alpha=0.3)
    plt.savefig(path, dpi=120, bbox_inches="tight")
    return True


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--out", default="attention_results.json")
    ap.add_argument("--plot", default=None, help="also write the TFLOPS-vs-p figure to this path")
    ap.add_argument("--heads", type=int, default=16)
    args = ap.parse_args(argv)
    res = sweep(H=args.heads)
    with open(args.out, "w") as f:
        json.dump(res, f, indent=2)
    print(f"wrote {args.out}")
    if args.plot:
        plot(res, args.plot)


if __name__ == "__main__":
    main()
