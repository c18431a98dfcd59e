"""What the wrappers and kernels do with arguments the reference would reject or guard: tensors on the wrong device
(the reference's launcher raises a Python error), tile lists that do not fit Sk (the reference masks every K/V and
mask load with kv_offset < SEQLEN_K, sparse_attn_kernel.py:35,39,60), and the exact CPU-plumbing workload on the GPU."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from helpers import assert_metadata_equal
from sparseattention_amd import (MaskMetadata, _native, compute_backward_metadata, compute_mask_kernel,
                                 compute_mask_slow, sparse_attention, sparse_attention_backward,
                                 sparse_attention_decode, workloads as W)
from sparseattention_amd.mask_utils import validation_key
from sparseattention_amd.sparse_attn_kernel import merge_attention_parts, validate_metadata

pytestmark = pytest.mark.gpu
TOL = 2e-2


def sdpa32(q, k, v, mask):
    return F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)


def test_tensors_on_the_wrong_device_raise_before_any_launch(gpu):
    B, H, S, D = 1, 2, 256, 64
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=1, device=gpu)
    mask = W.causal_mask(S, gpu)
    md = compute_mask_kernel(mask[None, None].expand(B, H, S, S), 128, 32)
    for bad in ("k", "v", "mask"):
        args = {"k": k, "v": v, "mask": mask}
        args[bad] = args[bad].cpu()
        with pytest.raises(ValueError, match=bad):
            sparse_attention(q, args["k"], args["v"], args["mask"], 128, 32, mask_metadata=md)
    with pytest.raises(ValueError, match="v is on cpu"):
        sparse_attention_decode(q[:, :, :8], k, v.cpu(), mask[:8], 32)
    o, lse = sparse_attention(q, k, v, mask, 128, 32, return_lse=True)
    do = torch.ones_like(o)
    for bad in ("k", "o", "do", "lse"):
        a = {"do": do, "k": k, "o": o, "lse": lse}
        a[bad] = a[bad].cpu()
        with pytest.raises(ValueError, match=f"{bad} is on cpu"):
            sparse_attention_backward(a["do"], q, a["k"], v, a["o"], a["lse"], mask)
    with pytest.raises(ValueError, match="lse_parts is on cpu"):
        merge_attention_parts(o[None], lse[None].cpu())
    # metadata on the host (e.g. from compute_mask_slow on a CPU mask)
    with pytest.raises(ValueError, match="mask_metadata"):
        sparse_attention(q, k, v, mask, 128, 32, mask_metadata=compute_mask_slow(mask.cpu()[None, None].expand(B, H, S, S), 128, 32))


def test_metadata_that_does_not_fit_is_refused_by_the_wrappers(gpu):
    B, H, S, D, BQ, BK = 1, 1, 512, 64, 128, 32
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=2, device=gpu)
    mask = W.random_block_mask(S, 32, 0.5, seed=2, device=gpu)[None, None]
    good = compute_mask_kernel(mask, BQ, BK, pack_partial=False)
    # the lists of compute_mask_slow (unused slots hold -1) are fine
    slow = compute_mask_slow(mask, BQ, BK)
    assert torch.equal(sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=slow),
                       sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=good))
    clone = lambda md: MaskMetadata(md.unmasked_kv_ids.clone(), md.unmasked_lens.clone(), md.masked_kv_ids.clone(),  # noqa: E731
                                    md.masked_lens.clone())
    stale = clone(slow)
    stale.unmasked_lens[0, 0, 1] += 1  # reaches into the -1 slots
    with pytest.raises(ValueError, match="unmasked_kv_ids"):
        sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=stale)
    long = clone(good)
    long.masked_lens[0, 0, 0] = S // BK + 1
    with pytest.raises(ValueError, match="counts"):
        sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=long)
    # an object that passed once is checked again after an in-place edit of its lists
    edited = clone(good)
    sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=edited)
    edited.masked_lens[0, 0, 0] = S // BK + 1
    with pytest.raises(ValueError, match="counts"):
        sparse_attention(q, k, v, mask, BQ, BK, mask_metadata=edited)
    # lists made for a longer Sk: indices past this Sk
    other = compute_mask_kernel(torch.ones(1, 1, S, 2 * S, dtype=torch.bool, device=gpu), BQ, BK, pack_partial=False)
    with pytest.raises(ValueError):
        validate_metadata(other, S, BK)


def _fwd_raw(q, k, v, mask, md, BQ, BK, packed=None):
    """The forward straight through the C ABI (no validation of the lists on the way)."""
    lib = _native.load()
    S = _native.strides
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    o = torch.full_like(q, float("nan"))
    me = mask.expand(B, H, Sq, Sk)
    rc = lib.sa_sparse_attention_fwd_ex(
        q.data_ptr(), S(q.stride()), k.data_ptr(), S(k.stride()), v.data_ptr(), S(v.stride()), o.data_ptr(), S(o.stride()),
        me.data_ptr(), S(me.stride()),
        md.unmasked_kv_ids.data_ptr(), S(md.unmasked_kv_ids.stride()), md.unmasked_lens.data_ptr(), S(md.unmasked_lens.stride()),
        md.masked_kv_ids.data_ptr(), S(md.masked_kv_ids.stride()), md.masked_lens.data_ptr(), S(md.masked_lens.stride()),
        packed.data_ptr() if packed is not None else None, S(packed.stride()[:2]) if packed is not None else None,
        None, 0, 0, B, H, Sq, Sk, D, BQ, BK, 0, D ** -0.5 / math.log(2), torch.cuda.current_stream().cuda_stream)
    _native.check(rc)
    torch.cuda.synchronize()
    return o


@pytest.mark.parametrize("BK", [16, 32, 64])
def test_kernels_skip_list_entries_that_do_not_fit(gpu, BK):
    # Through the C ABI, lists with counts beyond the row of tiles and indices outside [0, Sk/BK): the forward treats
    # such entries as absent, so the result is that of the mask without those tiles.
    B, H, S, D, BQ = 1, 2, 512, 64, 128
    nK = S // BK
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=3, device=gpu)
    mask = W.random_block_mask(S, 64, 0.4, seed=3, device=gpu)
    me = mask[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, BK, pack_partial=True)
    bad = MaskMetadata(md.unmasked_kv_ids.contiguous().clone(), md.unmasked_lens.contiguous().clone(),
                       md.masked_kv_ids.contiguous().clone(), md.masked_lens.contiguous().clone())
    pos = torch.arange(nK, device=gpu)
    for ids, lens in ((bad.unmasked_kv_ids, bad.unmasked_lens), (bad.masked_kv_ids, bad.masked_lens)):
        ids[pos.expand_as(ids) >= lens[..., None]] = 1 << 28  # what torch.empty may leave in the unused slots
    expect_mask = me.clone()
    # one FULL and one PARTIAL entry of Q tile 1 (both planes) point outside: those tiles drop out
    for ids, lens, repl in ((bad.unmasked_kv_ids, bad.unmasked_lens, nK + 3), (bad.masked_kv_ids, bad.masked_lens, -1)):
        assert int(lens[0, 0, 1]) >= 1
        tile = int(ids[0, 0, 1, 0])
        ids[:, :, 1, 0] = repl
        expect_mask[:, :, BQ:2 * BQ, tile * BK:(tile + 1) * BK] = False
    # counts beyond the row: the slots they reach hold indices out of range, which are skipped.  A FULL count that
    # takes the whole row of tiles leaves no room for PARTIAL entries: Q tile 2 keeps its FULL tiles only.
    bad.unmasked_lens[:, :, 2] = nK + 100
    expect_mask[:, :, 2 * BQ:3 * BQ] &= _tiles_mask(md.unmasked_kv_ids, md.unmasked_lens, 2, BQ, BK, S, gpu)
    bad.masked_lens[:, :, 3] = 1 << 20
    bad.unmasked_lens[:, :, 0] = -5  # a negative count reads as 0
    expect_mask[:, :, :BQ] &= ~_tiles_mask(md.unmasked_kv_ids, md.unmasked_lens, 0, BQ, BK, S, gpu)
    want = sdpa32(q, k, v, expect_mask)
    dead = ~expect_mask.any(-1)
    want[dead] = 0.0
    for packed in (None, md.packed_masks):
        o = _fwd_raw(q, k, v, mask, bad, BQ, BK, packed)
        assert torch.isfinite(o).all()
        assert (o.float() - want).abs().max() <= TOL


def _tiles_mask(ids, lens, qt, BQ, BK, S, dev):
    """bool [B,H,BQ,S]: the key columns of the listed tiles of Q tile qt."""
    B, H = ids.shape[:2]
    out = torch.zeros(B, H, 1, S, dtype=torch.bool, device=dev)
    for b in range(B):
        for h in range(H):
            for j in ids[b, h, qt, :int(lens[b, h, qt])].tolist():
                out[b, h, 0, j * BK:(j + 1) * BK] = True
    return out.expand(B, H, BQ, S)


def test_decode_clamps_lists_that_do_not_fit(gpu):
    # C ABI, counts beyond the row of tiles and indices out of range: the decode kernels clamp both (counts to the nKt
    # tiles of the row, indices into [0, nKt)), so the result is attention over the CLAMPED lists, tiles repeated as
    # often as they are listed.  That value is formed here from the lists on the host and compared.
    lib = _native.load()
    S = _native.strides
    B, H, Sq, Sk, D, BK = 1, 2, 8, 1024, 64, 32
    nKt = Sk // BK
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=4, device=gpu, Sk=Sk)
    mask = (torch.rand(Sq, Sk, generator=torch.Generator().manual_seed(4)) < 0.5).to(gpu)
    me = mask[None, None].expand(B, H, Sq, Sk)
    fid = torch.full((B, H, 1, nKt), 1 << 27, dtype=torch.int32, device=gpu)
    pid = ((3 * torch.arange(nKt, dtype=torch.int32, device=gpu)) % nKt).expand(B, H, 1, nKt).contiguous()
    pid[..., 1::2] = -3
    fl = torch.full((B, H, 1), 7, dtype=torch.int32, device=gpu)
    pl = torch.full((B, H, 1), nKt + 9, dtype=torch.int32, device=gpu)
    o = torch.empty_like(q)
    rc = lib.sa_sparse_attention_decode(
        q.data_ptr(), S(q.stride()), k.data_ptr(), S(k.stride()), v.data_ptr(), S(v.stride()), o.data_ptr(), S(o.stride()),
        me.data_ptr(), S(me.stride()), fid.data_ptr(), S(fid.stride()), fl.data_ptr(), S(fl.stride()),
        pid.data_ptr(), S(pid.stride()), pl.data_ptr(), S(pl.stride()), B, H, Sq, Sk, D, BK, 0, D ** -0.5 / math.log(2),
        1, None, 0, None, None, torch.cuda.current_stream().cuda_stream)
    _native.check(rc)
    torch.cuda.synchronize()
    # host arithmetic of the clamp: F = 7 FULL entries, all tile nKt - 1; then nKt - 7 PARTIAL entries
    F_, P_ = 7, min(nKt + 9, nKt - 7)
    tiles = [(nKt - 1, False)] * F_ + [(min(max(int(t), 0), nKt - 1), True) for t in pid[0, 0, 0, :P_].tolist()]
    cols = torch.cat([torch.arange(t * BK, (t + 1) * BK, device=gpu) for t, _ in tiles])
    keep = torch.cat([mask[:, t * BK:(t + 1) * BK] if part else torch.ones(Sq, BK, dtype=torch.bool, device=gpu)
                      for t, part in tiles], dim=1)
    want = sdpa32(q, k[:, :, cols], v[:, :, cols], keep)
    assert (o.float() - want).abs().max() <= TOL


def _tile_weights(md, packed_source, mask_rc, R, C, nR, nS, dev):
    """[R, C] float: how often the lists of plane (0, 0) of `md` (resident tiles of 128 rows, streamed tiles of 64
    columns, counts and indices clamped as the backward kernels clamp them) attend to each entry of `mask_rc`.
    packed_source: None = PARTIAL entries read the mask at the (clamped) tile they name; else the int ids tensor the
    packed tiles were made from: slot s carries the entries of the tile that slot named THEN."""
    Wt = torch.zeros(R, C, device=dev)
    for rt in range(nR):
        F_ = min(max(int(md.unmasked_lens[0, 0, rt]), 0), nS)
        P_ = min(max(int(md.masked_lens[0, 0, rt]), 0), nS - F_)
        rows = slice(128 * rt, 128 * rt + 128)
        for e in range(F_):
            t = min(max(int(md.unmasked_kv_ids[0, 0, rt, e]), 0), nS - 1)
            Wt[rows, 64 * t:64 * t + 64] += 1.0
        for e in range(P_):
            t = min(max(int(md.masked_kv_ids[0, 0, rt, e]), 0), nS - 1)
            src = t if packed_source is None else int(packed_source[0, 0, rt, e])
            Wt[rows, 64 * t:64 * t + 64] += mask_rc[rows, 64 * src:64 * src + 64].float()
    return Wt


@pytest.mark.parametrize("pack", [False, True])
def test_backward_clamps_lists_that_do_not_fit(gpu, pack):
    # Counts beyond the row of tiles, negative counts and indices out of range, straight to the kernels: they clamp
    # both, so each pass computes the gradient terms of the CLAMPED lists (tiles repeated as listed; with packed tiles a
    # slot keeps the entries it was packed with).  Expected values from those lists by host arithmetic + dense fp32.
    B, H, S, D = 1, 1, 256, 64
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=5, device=gpu)
    m2 = W.causal_mask(S, gpu)
    mask = m2[None, None].expand(B, H, S, S)
    o, lse = sparse_attention(q, k, v, mask, 128, 32, return_lse=True)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(6)).to(gpu, torch.bfloat16)
    bmd = compute_backward_metadata(mask, pack_partial=pack)
    nR, nS = S // 128, S // 64
    packed_from = []
    for md in (bmd.by_query, bmd.by_key):
        for name in ("unmasked_kv_ids", "unmasked_lens", "masked_kv_ids", "masked_lens"):
            setattr(md, name, getattr(md, name).contiguous().clone())
        packed_from.append(md.masked_kv_ids.clone())
        md.unmasked_kv_ids[:] = torch.tensor([1 << 25, 1, -7, 2], dtype=torch.int32, device=gpu)
        md.unmasked_lens[:] = torch.tensor([3, 1 << 16], dtype=torch.int32, device=gpu)
        # (every causal tile row at 128 x 64 has two PARTIAL tiles, so slots 0 and 1 of `packed` are filled)
        md.masked_kv_ids[..., 0] = -1
        md.masked_kv_ids[..., 1] = 9
        md.masked_lens[:] = torch.tensor([2, -4], dtype=torch.int32, device=gpu)
        md._validated_for = validation_key(md, S, 64)  # straight to the kernels
    got = sparse_attention_backward(do, q, k, v, o, lse, None if pack else mask, bmd)
    torch.cuda.synchronize()
    Wq = _tile_weights(bmd.by_query, packed_from[0] if pack else None, m2, S, S, nR, nS, gpu)
    Wk = _tile_weights(bmd.by_key, packed_from[1] if pack else None, m2.t(), S, S, nR, nS, gpu).t()
    scale = D ** -0.5
    q32, k32, v32, o32, do32 = (t[0, 0].float() for t in (q, k, v, o, do))
    P = torch.exp(q32 @ k32.t() * scale - lse[0, 0][:, None])
    dS = P * (do32 @ v32.t() - (do32 * o32).sum(-1, keepdim=True))
    want = (scale * (Wq * dS) @ k32, scale * (Wk * dS).t() @ q32, (Wk * P).t() @ do32)
    for g, w, name in zip(got, want, ("dq", "dk", "dv")):
        ref = max(1.0, float(w.abs().max()))
        err = float((g[0, 0].float() - w).abs().max()) / ref
        assert err <= TOL, f"{name} off by {err:.3e} of its scale {ref:.2f}"


def test_pack_skips_list_entries_that_do_not_fit(gpu):
    # sa_mask_pack_partial with a caller's own lists: a count beyond the row of tiles is clamped to it and a slot whose
    # index is outside [0, nK) is left untouched, so nothing outside the mask is read and nothing outside `packed` is
    # written (guard planes on both sides of the buffer stay as they were).
    lib = _native.load()
    S_ = _native.strides
    S, BQ, BK = 512, 128, 32
    nQ, nK, tb = S // BQ, S // BK, BQ * BK // 8
    mask = W.random_block_mask(S, 32, 0.5, seed=21, device=gpu, partial_fraction=0.4)[None, None]
    md = compute_mask_kernel(mask, BQ, BK, pack_partial=True)
    want = md.packed_masks.contiguous().clone()
    ids = md.masked_kv_ids.contiguous().clone()
    lens = md.masked_lens.contiguous().clone()
    n0 = int(lens[0, 0, 0])
    assert n0 >= 2
    pos = torch.arange(nK, device=gpu)
    ids[pos.expand_as(ids) >= lens[..., None]] = 1 << 28      # what torch.empty may have left past the counts
    ids[0, 0, 0, 1] = nK + 5                                   # inside the count, outside the mask
    ids[0, 0, 1, 0] = -2
    lens[0, 0, 0] = nK + 1000                                  # count beyond the row of tiles
    lens[0, 0, 2] = -3                                         # negative count: nothing to pack
    guard = torch.full((3, nQ, nK, tb), 0xA5, dtype=torch.uint8, device=gpu)
    packed = guard[1:2].unsqueeze(0)
    rc = lib.sa_mask_pack_partial(mask.data_ptr(), S_(mask.stride()), 1, 1, S, S, BQ, BK, ids.data_ptr(), S_(ids.stride()),
                                  lens.data_ptr(), S_(lens.stride()), packed.data_ptr(), S_((0, 0)),
                                  torch.cuda.current_stream().cuda_stream)
    _native.check(rc)
    torch.cuda.synchronize()
    assert (guard[0] == 0xA5).all() and (guard[2] == 0xA5).all()
    got = guard[1]
    assert torch.equal(got[0, 0], want[0, 0, 0, 0]) and (got[0, 1] == 0xA5).all()      # slot 1 skipped
    assert torch.equal(got[0, 2:n0], want[0, 0, 0, 2:n0]) and (got[0, n0:] == 0xA5).all()
    assert (got[1, 0] == 0xA5).all() and (got[2] == 0xA5).all()
    n3 = int(lens[0, 0, 3])
    assert torch.equal(got[3, :n3], want[0, 0, 3, :n3])


def test_decode_route_with_default_metadata(gpu):
    # compute_mask_kernel packs PARTIAL tiles by default; sparse_attention with fewer than 32 query rows reaches the
    # split-KV kernels with that metadata (they read the packed tiles) and with the reference's four tensors alone
    B, H, Sq, Sk, D, BK = 2, 2, 8, 1024, 64, 32
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=13, device=gpu, Sk=Sk)
    mask = (torch.rand(Sq, Sk, generator=torch.Generator().manual_seed(14)) < 0.3).to(gpu)
    mask[:, :BK] = True
    me = mask[None, None].expand(B, H, Sq, Sk)
    md = compute_mask_kernel(me, Sq, BK)
    assert md.packed_masks is not None
    o = sparse_attention(q, k, v, me, Sq, BK, md)
    assert torch.equal(o, sparse_attention_decode(q, k, v, me, BK, md))
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
    md2 = compute_mask_kernel(me, Sq, BK, schedule=None, pack_partial=False)
    assert torch.equal(o, sparse_attention(q, k, v, me, Sq, BK, md2))
    # with the packed tiles no mask tensor is needed; without them it is
    assert torch.equal(o, sparse_attention(q, k, v, None, Sq, BK, md))
    with pytest.raises(ValueError, match="mask"):
        sparse_attention(q, k, v, None, Sq, BK, md2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_cpu_plumbing_workload_on_the_gpu(gpu, dtype):
    # B=1 H=4 S=512 D=64, q/k/v ~ N(0,1) from seed 0 in fp32, mask: 32x32 blocks empty w.p. 0.5, 10 % of the blocks
    # coin flips, diagonal True.  Lists bit-exact against the oracle; the fp32 inputs cast to the kernel's dtypes against
    # fp32 masked SDPA of the fp32 inputs.
    B, H, S, D = 1, 4, 512, 64
    q32, k32, v32 = W.qkv(B, H, S, D, torch.float32, seed=0)
    mask = W.random_block_mask(S, 32, 0.5, seed=0)
    want = F.scaled_dot_product_attention(q32, k32, v32, attn_mask=mask)
    q, k, v = (t.to(gpu, dtype) for t in (q32, k32, v32))
    me = mask.to(gpu)[None, None].expand(B, H, S, S)
    for BQ, BK in ((32, 32), (128, 32), (64, 64)):
        md = compute_mask_kernel(me, BQ, BK)
        assert_metadata_equal(md, oracle.classify(mask.numpy()[None, None].repeat(H, 1), BQ, BK), f"{BQ}x{BK}")
        o = sparse_attention(q, k, v, me, BQ, BK, md)
        assert (o.float().cpu() - want).abs().max() <= TOL


def test_device_side_check_of_lists(gpu):
    # sa_validate_metadata: error bits in a device int, no host synchronisation on the way
    lib = _native.load()
    S_ = _native.strides
    B, H, S, BQ, BK = 2, 3, 1024, 128, 32
    nK = S // BK
    mask = W.random_block_mask(S, 128, 0.5, seed=9, device=gpu, batch=B).expand(B, H, S, S)
    md = compute_mask_kernel(mask, BQ, BK, pack_partial=False)

    def check(md_):
        flag = torch.zeros(1, dtype=torch.int32, device=gpu)
        rc = lib.sa_validate_metadata(
            md_.unmasked_kv_ids.data_ptr(), S_(md_.unmasked_kv_ids.stride()), md_.unmasked_lens.data_ptr(), S_(md_.unmasked_lens.stride()),
            md_.masked_kv_ids.data_ptr(), S_(md_.masked_kv_ids.stride()), md_.masked_lens.data_ptr(), S_(md_.masked_lens.stride()),
            B, H, S, S, BQ, BK, flag.data_ptr(), torch.cuda.current_stream().cuda_stream)
        _native.check(rc)
        return int(flag.item())

    assert check(md) == 0  # broadcast (stride-0) views as compute_mask_kernel returns them
    assert check(compute_mask_slow(mask, BQ, BK)) == 0  # -1 in the unused slots does not count
    own = lambda: MaskMetadata(md.unmasked_kv_ids.contiguous().clone(), md.unmasked_lens.contiguous().clone(),  # noqa: E731
                               md.masked_kv_ids.contiguous().clone(), md.masked_lens.contiguous().clone())
    bad = own()
    bad.unmasked_lens[1, 2, 3] = nK + 1
    assert check(bad) & 1
    bad = own()
    bad.masked_lens[0, 0, 0] = -2
    assert check(bad) == 1
    bad = own()
    b, h, t = (int(x) for x in torch.nonzero(bad.unmasked_lens > 0)[-1])  # some Q tile that has a FULL tile
    bad.unmasked_kv_ids[b, h, t, 0] = nK
    assert check(bad) == 2
    bad = own()
    b, h, t = (int(x) for x in torch.nonzero(bad.masked_lens > 0)[0])
    bad.masked_kv_ids[b, h, t, int(bad.masked_lens[b, h, t]) - 1] = -1
    assert check(bad) == 4
    # and the Python check agrees
    with pytest.raises(ValueError):
        validate_metadata(bad, S, BK)
