#!/usr/bin/env python3
"""Benchmark of the block-sparse attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-sweep] [--no-cpu]

A step is one forward pass (sa_sparse_attention_fwd_ex) over the headline workload: causal bool mask
passed as a tensor, B=8 H=32 S=4096 D=128 bf16, tiles 128x32, inputs and the precomputed mask metadata
(tile lists and bit-packed partial tiles: what compute_mask_kernel returns by default) resident in HBM;
the reference also excludes preprocessing from the forward time and reports it separately
(test_attn.py:38,65,68).  Prints ONE JSON line.

  value      effective TFLOP/s by the reference's convention: 4*B*H*Sq*Sk*D * mean(mask) / time
             (test_attn.py:84, :108-111)
  roofline   the forward kernel against the dense bf16 MFMA peak, counting executed tiles only:
             (full + partial tiles) * 4*BQ*BK*D flop per launch / mean launch duration (HIP events)
  mask_classify   the preprocessing kernels on a 1 GiB mask against the HBM peak
  across_p   the same forward on random block masks of sparsity p, a dense mask and the causal one
  variants   the headline workload through the other routes of the library (bool-mask reads, the pairs schedule,
             persistent workgroups)
  backward   dq, dk, dv of the headline workload (sparse_attention_backward) against the MFMA peak
  decode     the split-KV kernels for few query rows (sparse_attention_decode) against the HBM peak: K and V of
             the executed tiles are read once
  configs    the forward on the two long-sequence configurations (documents B4 H32 S16384, composed B1 H32 S32768),
             each with its own roofline against the MFMA peak
  tile_selection   every candidate tile size of select_block_sizes timed on four masks, next to what it picked
  cpu_baseline     torch's masked SDPA on CPU tensors of the whole workload: the reference's own check path
                   (test_attn.py:40) on the host cores; cpu_oracle_baseline: the C oracle (a port) on the same workload
                   mask_classify_cpu_baseline: compute_mask_slow (plain torch) on CPU tensors of a slab of the 1 GiB mask
  roofline.traffic  HBM bytes per launch from rocprofv3 counter runs (a constant here: traffic_source names the summary,
                   traffic_kernel_sources_sha16 the kernel sources it was read with, kernel_sources_sha16 the ones timed)
"""
import argparse
import gc
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak, TFLOP/s
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E peak, GB/s
PEAK_FP32_TFLOPS = 157.3   # MI355X dense fp32 MFMA peak, TFLOP/s

# HBM bytes per launch (read, written) measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE over
# `bench.py --traffic-probe` and scaled by what the same counters read for the 1 GiB device copy of the same run
# (`bench.py --traffic-summary` does the arithmetic).  profiles/hbm_traffic_all_kernels.txt holds the commands.
TRAFFIC_BYTES = {
    "forward, causal": (853480159, 268435456),
    "forward, dense": (808017050, 268436693),
    "forward, p=0.25": (1357508698, 268435456),
    "forward, p=0.5": (2852257992, 268435456),
    "forward, p=0.75": (2931904415, 268435456),
    "forward, p=0.9": (1417653896, 268435456),
    "backward, causal": (4305326450, 813694976),
    "forward, documents": (1721826894, 536870912),
    "forward, composed": (1612058763, 268435456),
    "mask_classify, composed mask 1 GiB": (1074106360, 308736),
    "decode, 1": (4295526174, 344064),
    "decode, 16": (1617159835, 5308501),
}
TRAFFIC_SOURCE = "profiles/hbm_traffic_all_kernels.txt"
# The sources each kernel is built from.  The counters were read with kernels built from sources of the digests in
# TRAFFIC_KERNEL_SOURCES_SHA16; the line carries those beside the digests of the sources in the tree, per kernel, so a
# reader sees whether a traffic figure belongs to the kernel that was timed.
KERNEL_FILES = {
    "forward": ("sparse_fwd_kernel.h", "sparse_fwd_c32.hip", "fwd_common.h", "kernels.h", "sparse_fwd.hip", "sparse_fwd_inst.hip"),
    "mask_classify": ("mask_classify.hip", "kernels.h"),
    "decode": ("sparse_decode.hip", "fwd_common.h", "kernels.h"),
    "backward": ("sparse_bwd.hip", "fwd_common.h", "kernels.h"),
}
TRAFFIC_KERNEL_SOURCES_SHA16 = {"forward": "bc08ea58e0414ab6", "mask_classify": "c6c9e6a7fb4bcc86", "decode": "39f4c61483f9cbce",
                                "backward": "44a7b516fda679c3"}


def kernel_sources_sha16(which=None):
    """First 16 hex digits of the SHA-256 over kernel sources (names and contents, in name order): the files of
    KERNEL_FILES[which], or every file under csrc/ when `which` is None."""
    import glob
    import hashlib

    files = sorted(glob.glob(os.path.join(ROOT, "sparseattention_amd", "csrc", "*")))
    if which is not None:
        files = [f for f in files if os.path.basename(f) in KERNEL_FILES[which]]
    h = hashlib.sha256()
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def traffic_of(workload, which):
    """The traffic entries of a roofline object: read + written bytes per launch (None when never measured)."""
    rw = TRAFFIC_BYTES.get(workload)
    return {"traffic": (rw[0] + rw[1]) if rw else None, "traffic_read_written": list(rw) if rw else None,
            "traffic_source": TRAFFIC_SOURCE if rw else None,
            "traffic_kernel_sources_sha16": TRAFFIC_KERNEL_SOURCES_SHA16[which],
            "kernel_sources_sha16": kernel_sources_sha16(which)}


def forward_roofline(executed_flop, hbm_bytes, kernel_ms, workload, kernel):
    """The forward against both of its floors: executed-tile flop at the bf16 MFMA peak, and q, k, v, o once through
    HBM.  `bound` is the larger floor; achieved / peak / frac are quoted against it, both fractions side by side."""
    t = kernel_ms * 1e-3
    mfma_floor, hbm_floor = executed_flop / (PEAK_BF16_TFLOPS * 1e12), hbm_bytes / (PEAK_HBM_GBS * 1e9)
    tf, gbs = executed_flop / t / 1e12, hbm_bytes / t / 1e9
    out = {"bound": "mfma" if mfma_floor >= hbm_floor else "hbm"}
    if out["bound"] == "mfma":
        out.update({"achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4)})
    else:
        out.update({"achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)})
    out.update({"mfma_frac": round(tf / PEAK_BF16_TFLOPS, 4), "hbm_frac": round(gbs / PEAK_HBM_GBS, 4),
                "mfma_floor_ms": round(mfma_floor * 1e3, 4), "hbm_floor_ms": round(hbm_floor * 1e3, 4),
                "flop_per_launch": executed_flop, "hbm_bytes_algorithmic": hbm_bytes, "kernel": kernel,
                "kernel_ms": kernel_ms})
    out.update(traffic_of(workload, "forward"))
    return out


SETTLE_LAUNCHES = 30
SETTLE_MS = 40.0

B, H, S, D = 8, 32, 4096, 128
BQ, BK = 128, 32
FLOP_PER_TILE = 4 * BQ * BK * D


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-sweep", action="store_true", help="skip the across-p table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--no-classify", action="store_true", help="skip the mask-classification timing")
    ap.add_argument("--no-decode", action="store_true", help="skip the few-query-rows (decode) timing")
    ap.add_argument("--no-backward", action="store_true", help="skip the backward-pass timing")
    ap.add_argument("--no-long", action="store_true", help="skip the forward on the documents and composed configurations")
    ap.add_argument("--no-tiles", action="store_true", help="skip the timing of the tile-size candidates")
    ap.add_argument("--power-trace", type=float, default=0.0, metavar="SECONDS",
                    help="instead of the benchmark: run each forward workload (and a device copy, a library GEMM) for "
                         "SECONDS without a gap while a child process, started before this one touches the GPU, samples "
                         "socket power, power cap, engine clock and temperatures from the amdgpu hwmon / sysfs files; "
                         "prints one JSON line with the figures per workload")
    ap.add_argument("--power-sampler", default=None, metavar="FILE", help=argparse.SUPPRESS)
    ap.add_argument("--traffic-probe", action="store_true",
                    help="instead of the benchmark: launch every timed workload of this script three times between "
                         "marker kernels (for a rocprofv3 --pmc FETCH_SIZE or WRITE_SIZE run over this command), then a "
                         "1 GiB device copy to scale the counters by; prints the workload names in order")
    ap.add_argument("--counter-summary", default=None, metavar="CSV",
                    help="instead of the benchmark: read the counter_collection.csv of a rocprofv3 --pmc run over "
                         "`bench.py --traffic-probe` and print every counter in it per launch of every workload (no GPU needed)")
    ap.add_argument("--traffic-summary", nargs=2, default=None, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="instead of the benchmark: read the two counter_collection.csv files of such runs and print "
                         "HBM bytes read and written per launch of every workload (no GPU needed)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy a few times, so that a counter run over this command "
                         "holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    return ap.parse_args()


def time_launches(fn, steps, warmup):
    """Wall time per step (host clock, synchronised on both sides) and mean per-launch duration from HIP
    events recorded on the stream the kernel is launched on (torch's current stream)."""
    import torch

    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    # A collection of the interpreter's cyclic garbage costs tens of milliseconds of host time: inside the timed region
    # a microsecond-scale step would report it as its own, and between warm-up and timed region it lets the device
    # fall idle, after which the next ten launches run up to 40 % slow.  So it happens before the warm-up.
    gc.collect()
    gc.disable()
    try:
        # the device settles over its first ten to twenty launches after an idle gap: with a short warm-up, further
        # untimed launches go in front of it
        for _ in range(max(0, SETTLE_LAUNCHES - warmup)):
            fn()
        # ... and by time as well: after seconds of host work (a mask built on the CPU) the device sits in a low power
        # state, from which short kernels need tens of milliseconds of load to come back
        torch.cuda.synchronize()
        t_settle = time.perf_counter()
        while (time.perf_counter() - t_settle) * 1e3 < SETTLE_MS:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            starts[i].record()
            fn()
            ends[i].record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    finally:
        gc.enable()
    ev_ms = sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / steps
    return wall_ms, ev_ms


def forward_case(name, mask2d, q, k, v, steps, warmup, schedule=None, pack_partial=None, block_k=BK, block_q=BQ):
    import torch
    from sparseattention_amd import compute_mask_kernel, sparse_attention

    B, H, S, D = q.shape
    BQ = block_q
    me = mask2d[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, block_k, pack_partial=pack_partial, schedule=schedule, list_stats=True)
    from sparseattention_amd.sparse_attn_kernel import _short_list_kernel
    kernel = ("sparse_fwd_c32_kernel" if _short_list_kernel(md, q.dtype, D, BQ, block_k, None)
              else "sparse_fwd_kernel" + (" (FULL entries walked from a start that depends on the Q tile)"
                                          if md.list_rotation and schedule is None else ""))
    tiles_plane = int(md.unmasked_lens[0, 0].sum()) + int(md.masked_lens[0, 0].sum())
    partial_plane = int(md.masked_lens[0, 0].sum())
    # mean of the mask in row slabs (a [32768,32768] float copy would take 4 GiB)
    frac = sum(float(mask2d[r0:r0 + 2048].sum()) for r0 in range(0, S, 2048)) / (S * S)
    wall_ms, ev_ms = time_launches(lambda: sparse_attention(q, k, v, me, BQ, block_k, mask_metadata=md), steps, warmup)
    executed = tiles_plane * B * H * 4 * BQ * block_k * D
    useful = 4 * B * H * S * S * D * frac
    return {
        "mask": name,
        "fraction_unmasked": round(frac, 5),
        "executed_tile_fraction": round(tiles_plane / ((S // BQ) * (S // block_k)), 5),
        "partial_tiles_per_plane": partial_plane,
        "ms": round(wall_ms, 4),
        "kernel_ms": round(ev_ms, 4),
        "effective_tflops": round(useful / (wall_ms * 1e-3) / 1e12, 2),
        "executed_tflops": round(executed / (ev_ms * 1e-3) / 1e12, 2),
        "list_entries_mean_longest": [round(md.list_stats[0], 2), md.list_stats[1]],
        "_executed_flop": executed,
        "_useful_flop": useful,
        "_hbm_bytes": 2 * q.numel() * 2 + 2 * k.numel() * 2,  # q read, o written, k and v read once
        "_kernel": kernel,
    }


def classify_case(steps, warmup):
    """Preprocessing on the largest single-plane mask of the configurations (S=32768, 1 GiB)."""
    import torch
    from sparseattention_amd import _native, workloads as W

    lib = _native.load()
    Sbig = 32768
    mask = W.composed_mask(Sbig, device="cuda")[None, None]
    nQ, nK = Sbig // BQ, Sbig // BK
    fid = torch.empty(1, 1, nQ, nK, dtype=torch.int32, device="cuda")
    pid = torch.empty_like(fid)
    fl = torch.empty(1, 1, nQ, dtype=torch.int32, device="cuda")
    pl = torch.empty_like(fl)
    ms = _native.strides(mask.stride())
    need = lib.sa_mask_classify_workspace_bytes(ms, 1, 1, Sbig, Sbig, BQ, BK)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = _native.strides
    stream = torch.cuda.current_stream().cuda_stream

    def run():
        rc = lib.sa_mask_classify(mask.data_ptr(), ms, 1, 1, Sbig, Sbig, BQ, BK, fid.data_ptr(), st(fid.stride()),
                                  fl.data_ptr(), st(fl.stride()), pid.data_ptr(), st(pid.stride()), pl.data_ptr(),
                                  st(pl.stride()), ws.data_ptr(), need, stream)
        _native.check(rc)

    wall_ms, ev_ms = time_launches(run, steps, warmup)
    # the optional extra step: one bit per entry of the PARTIAL tiles (1920 of 262144 tiles here)
    packed = torch.empty(lib.sa_mask_pack_partial_bytes(ms, 1, 1, Sbig, Sbig, BQ, BK), dtype=torch.uint8, device="cuda")

    def run_pack():
        rc = lib.sa_mask_pack_partial(mask.data_ptr(), ms, 1, 1, Sbig, Sbig, BQ, BK, pid.data_ptr(), st(pid.stride()),
                                      pl.data_ptr(), st(pl.stride()), packed.data_ptr(), st((0, 0)), stream)
        _native.check(rc)

    _, pack_ms = time_launches(run_pack, steps, warmup)
    nbytes = Sbig * Sbig + nQ * (2 * nK + 2) * 4  # mask read once + lists and counts written
    return {
        "workload": "sa_mask_classify on the composed mask, bool [32768,32768] = 1 GiB, tiles 128x32",
        "ms": round(ev_ms, 4),
        "pack_partial_ms": round(pack_ms, 4),
        "roofline": {"bound": "hbm", "achieved": round(nbytes / (ev_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(nbytes / (ev_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                     **traffic_of("mask_classify, composed mask 1 GiB", "mask_classify"),
                     "algorithmic_bytes": nbytes},
    }


def terms_case(steps, warmup):
    """The same composed mask from its formula: lists and packed PARTIAL tiles without the 1 GiB tensor."""
    import torch
    from sparseattention_amd import block_term, causal_term, compute_mask_terms

    Sbig = 32768
    terms = [causal_term(window=1024), block_term((0, 2048), (0, 2048))]
    md = compute_mask_terms(terms, 1, 32, Sbig, Sbig, BQ, BK, device="cuda")
    full, part = int(md.unmasked_lens[0, 0].sum()), int(md.masked_lens[0, 0].sum())
    _, ev_ms = time_launches(lambda: compute_mask_terms(terms, 1, 32, Sbig, Sbig, BQ, BK, device="cuda"), steps, warmup)
    return {
        "workload": "compute_mask_terms on (k<=q and q-k<1024) or (q<2048 and k<2048), S=32768, tiles 128x32: "
                    "classification from the formula, lists, packed PARTIAL tiles; no mask tensor",
        "full_tiles": full, "partial_tiles": part, "ms": round(ev_ms, 4),
        "entries_per_s": round(Sbig * Sbig / (ev_ms * 1e-3), 1),
    }


def classify_small_case(steps, warmup):
    """Preprocessing of the headline mask itself ([4096,4096] = 16 MiB): launch-latency bound."""
    import torch
    from sparseattention_amd import compute_mask_kernel, workloads as W

    me = W.causal_mask(S, "cuda")[None, None].expand(B, H, S, S)
    wall_ms, ev_ms = time_launches(lambda: compute_mask_kernel(me, BQ, BK, pack_partial=False), steps, warmup)
    _, full_ms = time_launches(lambda: compute_mask_kernel(me, BQ, BK, schedule="pairs"), steps, warmup)
    return {"workload": "compute_mask_kernel on the causal mask [4096,4096] = 16 MiB (latency bound)",
            "ms": round(ev_ms, 4), "with_pack_and_schedule_ms": round(full_ms, 4)}


def backward_case(q, k, v, steps, warmup):
    """dq, dk, dv of the headline workload (causal, B8 H32 S4096 D128 bf16); the backward tiles the mask 128 x 64
    both ways.  Algorithmic work per executed tile: the five products of the derivative (S, dP, dQ, dK, dV) of
    2*128*64*128 flop each; the three passes of the kernel recompute S twice and dP once, eight products in all."""
    import torch
    from sparseattention_amd import (compute_backward_metadata, compute_mask_kernel, sparse_attention,
                                     sparse_attention_backward, workloads as W)

    me = W.causal_mask(S, "cuda")[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, BK)
    bmd = compute_backward_metadata(me)
    o, lse = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md, return_lse=True)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(3)).to("cuda", torch.bfloat16)
    wall_ms, ev_ms = time_launches(lambda: sparse_attention_backward(do, q, k, v, o, lse, me, bmd), steps, warmup)
    tq = int(bmd.by_query.unmasked_lens[0, 0].sum()) + int(bmd.by_query.masked_lens[0, 0].sum())
    tk = int(bmd.by_key.unmasked_lens[0, 0].sum()) + int(bmd.by_key.masked_lens[0, 0].sum())
    per_product = 2 * 128 * 64 * D
    algorithmic = (3 * tq + 2 * tk) * per_product * B * H  # S, dP, dQ once per query-side tile; dK, dV per key-side tile
    executed = (3 * tq + 5 * tk) * per_product * B * H
    achieved = algorithmic / (ev_ms * 1e-3) / 1e12
    return {
        "workload": "dq, dk, dv of configs[1] (causal, B=8 H=32 S=4096 D=128 bf16), tiles 128x64 of the mask and of "
                    "its transpose, o and lse from the forward, metadata precomputed",
        "executed_tiles_per_plane": {"by_query": tq, "by_key": tk},
        "ms": round(wall_ms, 4), "kernel_ms": round(ev_ms, 4),
        "executed_tflops": round(executed / (ev_ms * 1e-3) / 1e12, 1),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), **traffic_of("backward, causal", "backward"),
                     "kernel": "sparse_bwd_kernel x3 (+ bwd_prepare_kernel)", "flop_per_launch": algorithmic},
    }


def decode_case(steps, warmup):
    """Few query rows against a 32k context (B8 H32 D128 bf16, KV tiles of 128): HBM-bound."""
    import torch
    from sparseattention_amd import compute_mask_kernel, sparse_attention_decode, workloads as W

    Sk, BKd = 32768, 128
    rows = []
    k = v = None
    for case, (name, Sq) in enumerate((("1 query row, every key", 1),
                                       ("16 query rows, causal window 4096 + 512 sink keys + 25% of the far tiles", 16))):
        q, k2, v2 = W.qkv(B, H, Sq, D, torch.bfloat16, seed=1, device="cuda", Sk=Sk)
        if k is None:
            k, v = k2, v2
        del k2, v2
        mask = decode_mask(Sq, Sk, BKd)
        me = mask.expand(B, H, Sq, Sk)
        md = compute_mask_kernel(me, Sq, BKd)
        tiles = int(md.unmasked_lens.sum()) + int(md.masked_lens.sum())
        nbytes = tiles * BKd * D * 2 * 2 + 2 * B * H * Sq * D * 2  # K and V rows of the executed tiles, q read, o written
        wall_ms, ev_ms = time_launches(lambda: sparse_attention_decode(q, k, v, me, BKd, mask_metadata=md), steps, warmup)
        rows.append({
            "workload": f"{name}; Sk=32768, B=8 H=32 D=128 bf16, BLOCK_K=128",
            "executed_tile_fraction": round(tiles / (B * H * (Sk // BKd)), 5),
            "ms": round(wall_ms, 4), "kernel_ms": round(ev_ms, 4),
            "roofline": {"bound": "hbm", "achieved": round(nbytes / (ev_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(nbytes / (ev_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                         **traffic_of("decode, %d" % Sq, "decode"),
                         "algorithmic_bytes": nbytes,
                         "kernel": "sparse_decode_kernel (+ decode_merge_kernel)"},
        })
    return rows


def fp32_case(steps, warmup):
    """The headline workload with float32 q, k, v (the reference's kernel takes the element type of its inputs,
    sparse_attn_kernel.py:98-101): v_mfma_f32_32x32x2_f32, nothing rounded below float32; against the fp32 MFMA peak."""
    import torch
    from sparseattention_amd import compute_mask_kernel, sparse_attention, workloads as W

    q, k, v = W.qkv(B, H, S, D, torch.float32, seed=0, device="cuda")
    me = W.causal_mask(S, "cuda")[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, BK)
    tiles = int(md.unmasked_lens[0, 0].sum()) + int(md.masked_lens[0, 0].sum())
    wall_ms, ev_ms = time_launches(lambda: sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md), steps, warmup)
    flop = tiles * B * H * FLOP_PER_TILE
    tf = flop / (ev_ms * 1e-3) / 1e12
    return {"workload": "configs[1] with float32 q, k, v, o (causal, B=8 H=32 S=4096 D=128, tiles 128x32, metadata precomputed)",
            "ms": round(wall_ms, 4), "kernel_ms": round(ev_ms, 4),
            "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tf / PEAK_FP32_TFLOPS, 4), "traffic": None, "flop_per_launch": flop,
                         "kernel": "sparse_fwd_f32_mfma_kernel", "dtype": "f32"}}


def long_configs(steps, warmup):
    """The forward on configs[3] (documents) and configs[4] (composed): tiles 128x32, packed partial tiles, metadata
    precomputed; executed-tile flop against the MFMA peak."""
    import torch
    from sparseattention_amd import workloads as W

    rows = []
    for name, Bc, Hc, Sc, make in (
            ("configs[3]: documents, B=4 H=32 S=16384 D=128 bf16; doc lengths uniform in [256,4096], causal within a document; "
             "bool mask [16384,16384] (256 MiB) shared by all planes", 4, 32, 16384, lambda: W.document_mask(16384, seed=0, device="cuda")),
            ("configs[4]: composed, B=1 H=32 S=32768 D=128 bf16; (kv<=q and q-kv<1024) or (q<2048 and kv<2048); bool mask "
             "[32768,32768] (1 GiB) shared by all heads", 1, 32, 32768, lambda: W.composed_mask(32768, device="cuda"))):
        q, k, v = W.qkv(Bc, Hc, Sc, D, torch.bfloat16, seed=0, device="cuda")
        mask = make()
        r = forward_case(name, mask, q, k, v, steps, warmup)
        rows.append({
            "workload": name + "; tiles BLOCK_Q=128 BLOCK_K=32",
            "fraction_unmasked": r["fraction_unmasked"], "executed_tile_fraction": r["executed_tile_fraction"],
            "executed_tiles_per_plane": int(r["_executed_flop"] // (Bc * Hc * FLOP_PER_TILE)),
            "partial_tiles_per_plane": r["partial_tiles_per_plane"],
            "ms": r["ms"], "kernel_ms": r["kernel_ms"], "effective_tflops": r["effective_tflops"],
            "list_entries_mean_longest": r["list_entries_mean_longest"],
            "roofline": forward_roofline(r["_executed_flop"], r["_hbm_bytes"], r["kernel_ms"],
                                         "forward, " + name.split(":")[1].split(",")[0].strip(), r["_kernel"]),
        })
        del q, k, v, mask
        torch.cuda.empty_cache()
    return rows


def tile_selection_case(steps, warmup):
    """select_block_sizes against the clock: every candidate tile size is classified and timed on four masks (the
    forward at B=2 H=32 D=128 bf16, so that the large masks fit beside q, k, v), next to the candidate the cost model
    picks.  `regret` = time of the pick / best measured time - 1."""
    import torch
    from sparseattention_amd import (compute_mask_kernel, select_block_sizes, sparse_attention, workloads as W)
    from sparseattention_amd.mask_utils import DEFAULT_TILE_CANDIDATES

    out = []
    for name, Sc, make in (("causal S=4096", 4096, lambda: W.causal_mask(4096, "cuda")),
                           ("random blocks p=0.75 S=4096", 4096, lambda: W.random_block_mask(4096, 128, 0.75, seed=75, device="cuda")),
                           ("documents S=16384", 16384, lambda: W.document_mask(16384, seed=0, device="cuda")),
                           ("composed S=32768", 32768, lambda: W.composed_mask(32768, device="cuda"))):
        Bc, Hc = (2, 32) if Sc <= 16384 else (1, 32)
        q, k, v = W.qkv(Bc, Hc, Sc, D, torch.bfloat16, seed=0, device="cuda")
        me = make()[None, None].expand(Bc, Hc, Sc, Sc)
        pick_q, pick_k, _, report = select_block_sizes(me)
        timed = {}
        for bq, bk in DEFAULT_TILE_CANDIDATES:
            md = compute_mask_kernel(me, bq, bk)
            _, ev = time_launches(lambda: sparse_attention(q, k, v, me, bq, bk, mask_metadata=md), steps, warmup)
            timed[f"{bq}x{bk}"] = round(ev, 4)
            del md
        best = min(timed, key=timed.get)
        out.append({"mask": name, "B": Bc, "H": Hc, "picked": f"{pick_q}x{pick_k}", "best_measured": best,
                    "regret": round(timed[f"{pick_q}x{pick_k}"] / timed[best] - 1.0, 4), "kernel_ms": timed,
                    "model_cost": {f"{r[0]}x{r[1]}": round(r[4] / 1e6, 2) for r in report}})
        del q, k, v, me
        torch.cuda.empty_cache()
    return out


def cpu_baselines():
    """Bounded CPU legs on the host cores: cpu_baseline = torch's masked SDPA on CPU tensors, the reference's own CPU
    path (test_attn.py:40); cpu_oracle_baseline = the C oracle (a port of the reference algorithm)."""
    import torch
    import torch.nn.functional as F

    import oracle
    from sparseattention_amd import workloads as W

    mask = W.causal_mask(S)
    frac = float(mask.float().mean())
    out = {}
    # (a) oracle: the whole workload (about ten seconds of host time)
    hp = B * H
    q, k, v = W.qkv(1, hp, S, D, torch.bfloat16, seed=0)
    qf, kf, vf = (t.float().numpy() for t in (q, k, v))
    m4 = mask.numpy()[None, None]
    meta = oracle.classify(m4.repeat(hp, 1), BQ, BK)
    t0 = time.perf_counter()
    oracle.forward(qf, kf, vf, m4, BQ, BK, meta=meta, p_round=1)
    dt = time.perf_counter() - t0
    useful = 4 * 1 * hp * S * S * D * frac
    out["cpu_oracle_baseline"] = {
        "value": round(useful / dt / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.max_threads(), "kind": "port",
        "sample": f"C oracle two-pass forward (oracle/sparse_oracle.c, OpenMP) on all {hp} (b,h) planes of the workload "
                  f"(causal S={S} D={D}, bf16 inputs widened to fp32, tiles {BQ}x{BK}): {dt:.2f} s, effective TFLOP/s",
        "ms_full_workload": round(dt * 1e3 * B * H / hp, 1),
    }
    del q, k, v, qf, kf, vf
    # (b) torch SDPA with the tensor mask on CPU
    hs = B * H
    q, k, v = W.qkv(1, hs, S, D, torch.bfloat16, seed=0)
    F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
        ts.append(time.perf_counter() - t0)
    dt = sorted(ts)[1]
    useful = 4 * 1 * hs * S * S * D * frac
    out["cpu_baseline"] = {
        "value": round(useful / dt / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "reference",
        "sample": f"the reference's CPU path for this workload is one library call, torch {torch.__version__} "
                  f"F.scaled_dot_product_attention(q,k,v,attn_mask=mask) (test_attn.py:40; none of the reference's own "
                  f"code runs): CPU bf16 tensors, all {hs} (b,h) planes of the workload (causal S={S} D={D}), one "
                  f"warm-up, median of 3 passes: {dt:.3f} s, effective TFLOP/s",
        "ms_full_workload": round(dt * 1e3 * B * H / hs, 1),
        "host_cpu_count": os.cpu_count(),
    }
    del q, k, v
    # (c) preprocessing on the CPU: the vectorised restatement of the reference's classification loop
    # (compute_mask_slow, mask_utils.py:14-44) on the first 4096 rows of the composed S = 32768 mask
    from sparseattention_amd import compute_mask_slow

    rows = 4096
    big = W.composed_mask(32768)[:rows][None, None]
    t0 = time.perf_counter()
    compute_mask_slow(big, BQ, BK)
    dt = time.perf_counter() - t0
    out["mask_classify_cpu_baseline"] = {
        "value": round(big.numel() / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"compute_mask_slow (plain torch on CPU tensors) on the first {rows} of the 32768 rows of the composed "
                  f"mask, 128 MiB of the 1 GiB, tiles {BQ}x{BK}: {dt:.2f} s, mask bytes per second",
    }
    return out


def power_sampler(path):
    """The child of --power-trace: never touches the GPU runtime, reads the amdgpu driver's files every 10 ms and
    appends `time power_W cap_W sclk_MHz junction_C mem_C` lines to `path` until `path + ".stop"` exists."""
    import glob

    dev = sorted(glob.glob("/sys/class/drm/card*/device"))
    dev = [d for d in dev if glob.glob(d + "/hwmon/hwmon*/power1_input")]
    if not dev:
        open(path, "w").write("no amdgpu hwmon files\n")
        return
    dev = dev[0]
    hw = glob.glob(dev + "/hwmon/hwmon*")[0]

    def rd(f, default="0"):
        try:
            with open(f) as fh:
                return fh.read()
        except OSError:
            return default

    def sclk():
        for line in rd(dev + "/pp_dpm_sclk", "").splitlines():
            if line.rstrip().endswith("*"):
                return float(line.split(":")[1].lower().replace("mhz", "").replace("*", ""))
        return 0.0

    with open(path, "w") as out:
        while not os.path.exists(path + ".stop"):
            out.write("%.4f %.1f %.1f %.0f %.1f %.1f\n" % (
                time.time(), float(rd(hw + "/power1_input")) / 1e6, float(rd(hw + "/power1_cap")) / 1e6, sclk(),
                float(rd(hw + "/temp2_input")) / 1e3, float(rd(hw + "/temp3_input")) / 1e3))
            out.flush()
            time.sleep(0.01)


def power_trace(seconds):
    """Every workload SECONDS long without a gap between launches, under the sampler; per workload the mean launch
    time over the second half (the settled state) and the sampler's readings over the same span."""
    import subprocess
    import tempfile

    tmp = tempfile.mkdtemp(prefix="sa_power_")
    path = os.path.join(tmp, "samples.txt")
    child = subprocess.Popen([sys.executable, os.path.abspath(__file__), "--power-sampler", path])
    time.sleep(0.5)  # idle readings first
    import torch
    from sparseattention_amd import compute_mask_kernel, sparse_attention, workloads as W

    torch.cuda.set_device(0)
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=0, device="cuda")
    spans = []

    def sustained(name, fn, flop):
        torch.cuda.synchronize()
        t0 = time.time()
        n = 0
        half = None
        while time.time() - t0 < seconds:
            for _ in range(25):
                fn()
            torch.cuda.synchronize()
            n += 25
            if half is None and time.time() - t0 >= seconds / 2:
                half = (time.time(), n)
        t1 = time.time()
        spans.append({"workload": name, "t0": half[0], "t1": t1, "ms_per_launch": round((t1 - half[0]) / (n - half[1]) * 1e3, 4),
                      "executed_flop": flop})
        time.sleep(0.3)  # (a gap in the samples between workloads)

    masks = [("causal", W.causal_mask(S, "cuda")), ("dense", torch.ones(S, S, dtype=torch.bool, device="cuda")),
             ("random blocks p=0.9", W.random_block_mask(S, 128, 0.9, seed=90, device="cuda")),
             ("no tile attended (q read, zeros written)", torch.zeros(S, S, dtype=torch.bool, device="cuda"))]
    for name, m in masks:
        me = m[None, None].expand(B, H, S, S)
        md = compute_mask_kernel(me, BQ, BK, list_stats=True)
        tiles = int(md.unmasked_lens[0, 0].sum()) + int(md.masked_lens[0, 0].sum())
        flop = tiles * B * H * FLOP_PER_TILE
        sustained("forward, " + name, lambda: sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md, kernel="default"), flop)
        if name == "causal":  # the same mask and work through the 256-row kernel (8 waves, one workgroup per CU)
            md2 = compute_mask_kernel(me, 256, BK)
            t2 = int(md2.unmasked_lens[0, 0].sum()) + int(md2.masked_lens[0, 0].sum())
            sustained("forward, causal, tiles 256x32 (8-wave two-phase kernel)",
                      lambda: sparse_attention(q, k, v, me, 256, BK, mask_metadata=md2), t2 * B * H * 2 * FLOP_PER_TILE)
        if name.endswith("p=0.9"):
            sustained("forward, " + name + ", short-list kernel",
                      lambda: sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md, kernel="short"), flop)
    # backward of the causal workload (algorithmic flop: five products per executed 128x64 tile)
    from sparseattention_amd import compute_backward_metadata, sparse_attention_backward, sparse_attention_decode

    me = masks[0][1][None, None].expand(B, H, S, S)
    bmd = compute_backward_metadata(me)
    o, lse = sparse_attention(q, k, v, me, BQ, BK, return_lse=True)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(3)).to("cuda", torch.bfloat16)
    tq = int(bmd.by_query.unmasked_lens[0, 0].sum()) + int(bmd.by_query.masked_lens[0, 0].sum())
    tk = int(bmd.by_key.unmasked_lens[0, 0].sum()) + int(bmd.by_key.masked_lens[0, 0].sum())
    sustained("backward, causal (algorithmic flop)", lambda: sparse_attention_backward(do, q, k, v, o, lse, me, bmd),
              (3 * tq + 2 * tk) * 2 * 128 * 64 * D * B * H)
    del o, lse, do, bmd
    # decode: one query row against every key of a 32k context (HBM-bound)
    qd, kd, vd = W.qkv(B, H, 1, D, torch.bfloat16, seed=1, device="cuda", Sk=32768)
    md_d = compute_mask_kernel(torch.ones(B, H, 1, 32768, dtype=torch.bool, device="cuda"), 1, 128)
    mk_d = torch.ones(1, 32768, dtype=torch.bool, device="cuda").expand(B, H, 1, 32768)
    sustained("decode, 1 query row, Sk=32768 (4 GiB of K/V per launch)",
              lambda: sparse_attention_decode(qd, kd, vd, mk_d, 128, mask_metadata=md_d), 0)
    del qd, kd, vd
    src = torch.ones(1 << 28, dtype=torch.int32, device="cuda")
    dst = torch.empty_like(src)
    sustained("device copy 1 GiB (torch)", lambda: dst.copy_(src), 0)
    del src, dst
    a = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    bm = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    sustained("bf16 GEMM 8192^3 (torch / hipBLASLt)", lambda: a @ bm, 2 * 8192 ** 3)
    open(path + ".stop", "w").close()
    child.wait(timeout=10)
    rows = [tuple(float(x) for x in ln.split()) for ln in open(path).read().splitlines() if ln[:1].isdigit()]
    idle = [r for r in rows if r[0] < rows[0][0] + 0.4] if rows else []
    out = {"power_trace_seconds_per_workload": seconds, "samples": len(rows),
           "idle": {"power_W": round(sum(r[1] for r in idle) / max(1, len(idle)), 1)} if idle else None, "workloads": []}
    for sp in spans:
        rs = [r for r in rows if sp["t0"] <= r[0] <= sp["t1"]]
        n = max(1, len(rs))
        tf = sp["executed_flop"] / (sp["ms_per_launch"] * 1e-3) / 1e12 if sp["executed_flop"] else None
        pw = sum(r[1] for r in rs) / n
        out["workloads"].append({
            "workload": sp["workload"], "ms_per_launch": sp["ms_per_launch"],
            "executed_tflops": round(tf, 1) if tf else None, "samples": len(rs),
            "power_W_mean": round(pw, 1), "power_W_max": round(max((r[1] for r in rs), default=0.0), 1),
            "power_cap_W": round(rs[0][2], 1) if rs else None,
            "sclk_MHz_mean": round(sum(r[3] for r in rs) / n, 0), "sclk_MHz_min": min((r[3] for r in rs), default=0.0),
            "junction_C_max": max((r[4] for r in rs), default=0.0), "mem_C_max": max((r[5] for r in rs), default=0.0),
            "W_per_executed_tflops": round(pw / tf, 3) if tf else None})
    print(json.dumps(out))


TRAFFIC_PROBE_LAUNCHES = 3
MARKER_KERNEL = "validate_lists_kernel"  # (sa_validate_metadata: nothing else in a probe run launches it)


def traffic_probe():
    """Every workload this script times, TRAFFIC_PROBE_LAUNCHES launches each between two marker kernels (what runs
    outside the markers - classification, warm-up - is not counted), the 1 GiB copy last."""
    import torch
    from sparseattention_amd import (_native, compute_backward_metadata, compute_mask_kernel, sparse_attention,
                                     sparse_attention_backward, sparse_attention_decode, workloads as W)

    lib = _native.load()
    st = _native.strides
    tiny = compute_mask_kernel(torch.ones(1, 1, 128, 128, dtype=torch.bool, device="cuda"), 128, 32, pack_partial=False)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    names = []

    def marker():
        _native.check(lib.sa_validate_metadata(
            tiny.unmasked_kv_ids.data_ptr(), st(tiny.unmasked_kv_ids.stride()), tiny.unmasked_lens.data_ptr(), st(tiny.unmasked_lens.stride()),
            tiny.masked_kv_ids.data_ptr(), st(tiny.masked_kv_ids.stride()), tiny.masked_lens.data_ptr(), st(tiny.masked_lens.stride()),
            1, 1, 128, 128, 128, 32, flag.data_ptr(), torch.cuda.current_stream().cuda_stream))

    def measured(name, fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        marker()
        for _ in range(TRAFFIC_PROBE_LAUNCHES):
            fn()
        marker()
        torch.cuda.synchronize()
        names.append(name)

    def forward(name, mask2d, q, k, v):
        Bc, Hc, Sc, _ = q.shape
        me = mask2d[None, None].expand(Bc, Hc, Sc, Sc)
        md = compute_mask_kernel(me, BQ, BK, list_stats=True)
        measured("forward, " + name, lambda: sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md))

    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=0, device="cuda")
    forward("causal", W.causal_mask(S, "cuda"), q, k, v)
    forward("dense", torch.ones(S, S, dtype=torch.bool, device="cuda"), q, k, v)
    for p_ in (0.25, 0.5, 0.75, 0.9):
        forward(f"p={p_}", W.random_block_mask(S, 128, p_, seed=int(p_ * 100), device="cuda"), q, k, v)
    me = W.causal_mask(S, "cuda")[None, None].expand(B, H, S, S)
    bmd = compute_backward_metadata(me)
    o, lse = sparse_attention(q, k, v, me, BQ, BK, return_lse=True)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(3)).to("cuda", torch.bfloat16)
    measured("backward, causal", lambda: sparse_attention_backward(do, q, k, v, o, lse, me, bmd))
    del q, k, v, o, lse, do, bmd, me
    torch.cuda.empty_cache()
    for name, Bc, Hc, Sc, make in (("documents", 4, 32, 16384, lambda: W.document_mask(16384, seed=0, device="cuda")),
                                   ("composed", 1, 32, 32768, lambda: W.composed_mask(32768, device="cuda"))):
        q, k, v = W.qkv(Bc, Hc, Sc, D, torch.bfloat16, seed=0, device="cuda")
        forward(name, make(), q, k, v)
        del q, k, v
        torch.cuda.empty_cache()
    big = W.composed_mask(32768, device="cuda")[None, None]
    measured("mask_classify, composed mask 1 GiB", lambda: compute_mask_kernel(big, BQ, BK, pack_partial=False))
    del big
    torch.cuda.empty_cache()
    Sk, BKd = 32768, 128
    kd = vd = None
    for Sq in (1, 16):
        qd, k2, v2 = W.qkv(B, H, Sq, D, torch.bfloat16, seed=1, device="cuda", Sk=Sk)
        if kd is None:
            kd, vd = k2, v2
        del k2, v2
        mask = decode_mask(Sq, Sk, BKd)
        med = mask.expand(B, H, Sq, Sk)
        mdd = compute_mask_kernel(med, Sq, BKd)
        measured("decode, %d" % Sq, lambda: sparse_attention_decode(qd, kd, vd, med, BKd, mask_metadata=mdd))
    del kd, vd
    torch.cuda.empty_cache()
    src = torch.ones(1 << 28, dtype=torch.int32, device="cuda")  # 1 GiB read + 1 GiB written per copy
    dst = torch.empty_like(src)
    measured("copy 1 GiB", lambda: dst.copy_(src))
    print(json.dumps({"traffic_probe_workloads": names, "launches_each": TRAFFIC_PROBE_LAUNCHES,
                      "kernel_sources_sha16": {w: kernel_sources_sha16(w) for w in KERNEL_FILES}}))


PROBE_WORKLOADS = ["forward, causal", "forward, dense", "forward, p=0.25", "forward, p=0.5", "forward, p=0.75", "forward, p=0.9",
                   "backward, causal", "forward, documents", "forward, composed", "mask_classify, composed mask 1 GiB",
                   "decode, 1", "decode, 16", "copy 1 GiB"]


def counter_summary(path):
    """Every counter of a --pmc run over --traffic-probe, summed over the dispatches of a workload's marked span and
    divided by its launches."""
    import csv

    rows = list(csv.DictReader(open(path)))
    rows.sort(key=lambda r: int(r["Dispatch_Id"]))
    counters = sorted({r["Counter_Name"] for r in rows})
    out = {n: {} for n in PROBE_WORKLOADS}
    for c in counters:
        sums, inside, acc = [], False, 0.0
        for r in rows:
            if r["Counter_Name"] != c:
                continue
            if MARKER_KERNEL in r["Kernel_Name"]:
                if inside:
                    sums.append(acc / TRAFFIC_PROBE_LAUNCHES)
                inside, acc = not inside, 0.0
            elif inside:
                acc += float(r["Counter_Value"])
        if len(sums) != len(PROBE_WORKLOADS):
            raise SystemExit(f"{path}: {len(sums)} marked spans of {c}, expected {len(PROBE_WORKLOADS)}")
        for n, v in zip(PROBE_WORKLOADS, sums):
            out[n][c] = v
    print(json.dumps(out, indent=1))


def traffic_summary(fetch_csv, write_csv):
    """Per workload of a --traffic-probe run: counter units summed over the dispatches between an odd marker and the
    next even one, per launch, scaled so that the copy of 1 GiB reads 2^30 bytes."""
    import csv

    names = PROBE_WORKLOADS

    def per_workload(path, counter):
        rows = [r for r in csv.DictReader(open(path)) if r["Counter_Name"] == counter]
        rows.sort(key=lambda r: int(r["Dispatch_Id"]))
        sums, inside, acc = [], False, 0.0
        for r in rows:
            if MARKER_KERNEL in r["Kernel_Name"]:
                if inside:
                    sums.append(acc / TRAFFIC_PROBE_LAUNCHES)
                inside, acc = not inside, 0.0
            elif inside:
                acc += float(r["Counter_Value"])
        if len(sums) != len(names):
            raise SystemExit(f"{path}: {len(sums)} marked spans, expected {len(names)}")
        return sums

    fetch, write = per_workload(fetch_csv, "FETCH_SIZE"), per_workload(write_csv, "WRITE_SIZE")
    f_unit, w_unit = (1 << 30) / fetch[-1], (1 << 30) / write[-1]
    out = {"bytes_per_FETCH_SIZE_unit": round(f_unit, 2), "bytes_per_WRITE_SIZE_unit": round(w_unit, 2), "workloads": {}}
    for n, f, w in zip(names, fetch, write):
        out["workloads"][n] = [round(f * f_unit), round(w * w_unit)]
    print(json.dumps(out, indent=1))


def decode_mask(Sq, Sk, BKd):
    """The two decode workloads' masks: every key for one query row; else a causal window of 4096 keys, 512 sink keys
    and a quarter of the far KV tiles."""
    import torch

    if Sq == 1:
        return torch.ones(Sq, Sk, dtype=torch.bool, device="cuda")
    pos_q = torch.arange(Sk - Sq, Sk, device="cuda")[:, None]
    pos_k = torch.arange(Sk, device="cuda")[None, :]
    far = (torch.rand(Sk // BKd, generator=torch.Generator().manual_seed(2)) < 0.25).to("cuda").repeat_interleave(BKd)
    return (pos_k <= pos_q) & ((pos_q - pos_k < 4096) | (pos_k < 512) | far[None, :])


def main():
    args = parse()
    if args.traffic_summary:
        traffic_summary(*args.traffic_summary)
        return
    if args.counter_summary:
        counter_summary(args.counter_summary)
        return
    if args.power_sampler:
        power_sampler(args.power_sampler)
        return
    if args.power_trace > 0:
        power_trace(args.power_trace)
        return
    if args.traffic_probe:
        traffic_probe()
        return
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); the path has no multi-GPU leg.",
              file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no ROCm GPU visible; the forward path has no CPU fallback.", file=sys.stderr)
        sys.exit(2)
    from sparseattention_amd import _native, workloads as W

    _native.load()
    torch.cuda.set_device(0)
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=0, device="cuda")

    head = forward_case("causal", W.causal_mask(S, "cuda"), q, k, v, args.steps, args.warmup)
    result = {
        "metric": "effective TFLOP/s of the block-sparse forward (4*B*H*S*S*D*mean(mask)/time), B8 H32 S4096 D128 bf16",
        "value": head["effective_tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        # untimed launches in front of the warm-up: this many, then more until settle_ms of load have passed
        "settle_launches": max(0, SETTLE_LAUNCHES - args.warmup), "settle_ms": SETTLE_MS,
        "ms_per_step": head["ms"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: causal bool mask [4096,4096] passed as a tensor, B=8 H=32 S=4096 D=128 bf16, "
                               "q/k/v ~ N(0,1), tiles BLOCK_Q=128 BLOCK_K=32, mask metadata precomputed "
                               "(tile lists, bit-packed partial tiles, list statistics; one workgroup per Q tile)",
                   "executed_tiles_per_plane": int(head["_executed_flop"] // (B * H * FLOP_PER_TILE)),
                   "partial_tiles_per_plane": head["partial_tiles_per_plane"],
                   "list_entries_mean_longest": head["list_entries_mean_longest"]},
        "roofline": forward_roofline(head["_executed_flop"], head["_hbm_bytes"], head["kernel_ms"], "forward, causal",
                                     head["_kernel"]),
    }
    if not args.no_sweep:
        # (a launch after an idle gap runs up to 40 % slow and the next ten settle: never fewer than 10 warm-ups)
        vs, vw = max(20, args.steps // 2), max(10, args.warmup)
        causal = W.causal_mask(S, "cuda")
        result["variants"] = {
            name: round(forward_case(name, causal, q, k, v, vs, vw, schedule=sch, pack_partial=pk)["kernel_ms"], 4)
            for name, sch, pk in (("pairs_schedule_packed_ms", "pairs", True), ("no_schedule_packed_ms", None, True),
                                  ("no_schedule_bool_mask_ms", None, False),
                                  ("persistent_schedule_packed_ms", "persistent", True))}
        # the same mask tiled 128 x 64 (the same executed area; the forward consumes keys in chunks of 64 either way)
        result["variants"]["tiles_128x64_ms"] = round(
            forward_case("causal 128x64", causal, q, k, v, vs, vw, block_k=64)["kernel_ms"], 4)
        del causal
        rows = [head]
        sweep_steps, sweep_warm = max(20, args.steps // 2), max(10, args.warmup)
        rows.append(forward_case("dense (all True)", torch.ones(S, S, dtype=torch.bool, device="cuda"), q, k, v,
                                 sweep_steps, sweep_warm))
        for p in (0.25, 0.5, 0.75, 0.9):
            m = W.random_block_mask(S, 128, p, seed=int(p * 100), device="cuda")
            rows.append(forward_case(f"random blocks p={p}", m, q, k, v, sweep_steps, sweep_warm))
        result["across_p"] = [dict({kk: vv for kk, vv in r.items() if not kk.startswith("_")},
                                   roofline=forward_roofline(r["_executed_flop"], r["_hbm_bytes"], r["kernel_ms"],
                                                             "forward, " + r["mask"].replace(" (all True)", "").replace("random blocks ", ""),
                                                             r["_kernel"]))
                              for r in rows]
    if not args.no_classify:
        result["mask_classify"] = classify_case(max(10, args.steps // 2), max(3, args.warmup // 2))
        result["mask_terms"] = terms_case(max(10, args.steps // 2), max(3, args.warmup // 2))
        result["mask_classify_headline"] = classify_small_case(max(10, args.steps // 2), max(3, args.warmup // 2))
    if not args.no_backward:
        result["backward"] = backward_case(q, k, v, max(10, args.steps // 5), max(5, args.warmup // 2))
    del q, k, v
    torch.cuda.empty_cache()
    if not args.no_sweep:
        result["fp32_forward"] = fp32_case(max(5, args.steps // 10), max(3, args.warmup // 5))
        torch.cuda.empty_cache()
    if not args.no_long:
        result["configs"] = long_configs(max(20, args.steps // 2), max(10, args.warmup))
    if not args.no_tiles:
        result["tile_selection"] = tile_selection_case(max(10, args.steps // 5), max(10, args.warmup // 2))
    if not args.no_decode:
        result["decode"] = decode_case(max(20, args.steps // 2), max(10, args.warmup))
    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.int32, device="cuda")  # 1 GiB read + 1 GiB written per copy
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if not args.no_cpu:
        result.update(cpu_baselines())
    print(json.dumps(result))


if __name__ == "__main__":
    main()
