"""sa_mask_classify_static (the entry point that allocates nothing: its class bytes live in a device array of the
library's own) against sa_mask_classify on the same masks, both through the C ABI: lens and ids[..., :len] bit-exact,
and both against the oracle.  Two calls in a row share the array, the second on a smaller input."""
import os

import pytest
import torch

import oracle
from helpers import assert_metadata_equal
from sparseattention_amd import MaskMetadata, _native, workloads as W

pytestmark = pytest.mark.gpu

SENTINEL = -7


def _outputs(B, H, nQ, nK, dev):
    fid = torch.full((B, H, nQ, nK), SENTINEL, dtype=torch.int32, device=dev)
    pid = torch.full((B, H, nQ, nK), SENTINEL, dtype=torch.int32, device=dev)
    fl = torch.full((B, H, nQ), SENTINEL, dtype=torch.int32, device=dev)
    pl = torch.full((B, H, nQ), SENTINEL, dtype=torch.int32, device=dev)
    return fid, fl, pid, pl


def _classify(mask, BQ, BK, static):
    """MaskMetadata from sa_mask_classify_static, or from sa_mask_classify with a torch workspace."""
    lib = _native.load()
    S = _native.strides
    B, H, Sq, Sk = mask.shape
    fid, fl, pid, pl = _outputs(B, H, Sq // BQ, Sk // BK, mask.device)
    ms = S(mask.stride())
    outs = (fid.data_ptr(), S(fid.stride()), fl.data_ptr(), S(fl.stride()),
            pid.data_ptr(), S(pid.stride()), pl.data_ptr(), S(pl.stride()))
    stream = torch.cuda.current_stream(mask.device).cuda_stream
    if static:
        rc = lib.sa_mask_classify_static(mask.data_ptr(), ms, B, H, Sq, Sk, BQ, BK, *outs, stream)
    else:
        need = int(lib.sa_mask_classify_workspace_bytes(ms, B, H, Sq, Sk, BQ, BK))
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=mask.device)
        rc = lib.sa_mask_classify(mask.data_ptr(), ms, B, H, Sq, Sk, BQ, BK, *outs, ws.data_ptr(), need, stream)
    _native.check(rc)
    torch.cuda.synchronize()
    return MaskMetadata(fid, fl, pid, pl)


def _same(a, b, what):
    for name in ("unmasked_kv_ids", "unmasked_lens", "masked_kv_ids", "masked_lens"):
        assert torch.equal(getattr(a, name), getattr(b, name)), f"{what}: {name} differ (untouched slots included)"


def test_two_calls_in_a_row_second_smaller(gpu):
    # first call: per-batch planes, wide kernel, 3 * 8 * 64 = 1536 class bytes in the library's array
    big = W.random_block_mask(2048, 32, 0.5, seed=11, device=gpu, batch=3).expand(3, 2, 2048, 2048)
    got = _classify(big, 256, 32, static=True)
    ref = _classify(big, 256, 32, static=False)
    _same(got, ref, "first call")
    assert_metadata_equal(got, oracle.classify(big.cpu().numpy(), 256, 32), "first call vs oracle")
    # second call: one smaller plane; the array still holds the first call's class bytes past its 4 * 16 = 64
    small = W.random_block_mask(512, 32, 0.6, seed=12, device=gpu)[None, None]
    got = _classify(small, 128, 32, static=True)
    ref = _classify(small, 128, 32, static=False)
    _same(got, ref, "second call")
    assert_metadata_equal(got, oracle.classify(small.cpu().numpy(), 128, 32), "second call vs oracle")
    # and the generic kernel (tile width that is no power of two) on the same array
    odd = (torch.rand(1, 2, 96, 120, generator=torch.Generator().manual_seed(13)) < 0.5).to(gpu)
    odd[0, 0, :24, :40] = True
    odd[0, 1, 24:48, 40:80] = False
    got = _classify(odd, 24, 40, static=True)
    ref = _classify(odd, 24, 40, static=False)
    _same(got, ref, "third call")
    assert_metadata_equal(got, oracle.classify(odd.cpu().numpy(), 24, 40), "third call vs oracle")


def test_largest_size_and_refusal_beyond_it(gpu):
    lib = _native.load()
    S = _native.strides
    cap = 1 << 20  # SA_STATIC_CLASSIFY_MAX_TILES
    header = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "sparseattn.h")).read()
    assert "#define SA_STATIC_CLASSIFY_MAX_TILES (1u << 20)" in header
    # exactly the cap: 16384 x 16384 entries in tiles of 16 x 16 -> 1024 x 1024 tiles
    Sx = 16384
    m = W.composed_mask(Sx, device=gpu)[None, None]
    got = _classify(m, 16, 16, static=True)
    ref = _classify(m, 16, 16, static=False)
    _same(got, ref, "cap-sized call")
    del got, ref
    # one Q-tile row more: refused on the host with SA_ERR_WORKSPACE, outputs untouched
    m2 = torch.ones(1, 1, Sx + 16, Sx, dtype=torch.bool, device=gpu)
    nQ, nK = (Sx + 16) // 16, Sx // 16
    assert nQ * nK > cap
    fl = torch.full((1, 1, nQ), SENTINEL, dtype=torch.int32, device=gpu)
    pl = torch.full((1, 1, nQ), SENTINEL, dtype=torch.int32, device=gpu)
    ids = torch.empty(1, 1, nQ, nK, dtype=torch.int32, device=gpu)
    rc = lib.sa_mask_classify_static(m2.data_ptr(), S(m2.stride()), 1, 1, Sx + 16, Sx, 16, 16,
                                     ids.data_ptr(), S(ids.stride()), fl.data_ptr(), S(fl.stride()),
                                     ids.data_ptr(), S(ids.stride()), pl.data_ptr(), S(pl.stride()),
                                     torch.cuda.current_stream(gpu).cuda_stream)
    assert rc == _native.SA_ERR_WORKSPACE
    assert b"SA_STATIC_CLASSIFY_MAX_TILES" in lib.sa_last_error()
    torch.cuda.synchronize()
    assert int((fl != SENTINEL).sum()) == 0 and int((pl != SENTINEL).sum()) == 0
    # a smaller call right after the cap-sized one and the refusal
    small = W.causal_mask(1024, gpu)[None, None]
    got = _classify(small, 128, 32, static=True)
    assert_metadata_equal(got, oracle.classify(small.cpu().numpy(), 128, 32), "after the cap-sized call")
