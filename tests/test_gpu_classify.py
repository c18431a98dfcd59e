"""Parity of the HIP tile classification (sa_mask_classify through the Python binding) with the
oracle: bit-exact lens and ids[..., :len] on the same inputs."""
import ctypes

import numpy as np
import pytest
import torch

import golden_io
import oracle
from helpers import assert_metadata_equal, causal_closed_form, lists_of
from sparseattention_amd import _native, compute_mask_kernel, workloads as W

pytestmark = pytest.mark.gpu


def check(mask_gpu, BQ, BK, what=""):
    got = compute_mask_kernel(mask_gpu, BQ, BK)
    torch.cuda.synchronize()
    want = oracle.classify(mask_gpu.cpu().numpy(), BQ, BK)
    assert_metadata_equal(got, want, what or f"{tuple(mask_gpu.shape)} {BQ}x{BK}")
    return got


@pytest.mark.parametrize("BQ,BK", [(128, 32), (32, 128), (64, 64), (128, 16), (16, 16), (32, 1024), (256, 256), (8, 64), (6, 32), (1, 16)])
def test_wide_path_tile_shapes(gpu, BQ, BK):
    S = 1536 if 1536 % BQ == 0 and 1536 % BK == 0 else 2048
    m = W.random_block_mask(S, 32, 0.5, seed=BQ * 1000 + BK, device=gpu)[None, None]
    check(m, BQ, BK)


@pytest.mark.parametrize("Sq,Sk", [(128, 48), (64, 16), (256, 1040), (96, 2064), (512, 1024)])
def test_wide_path_ragged_widths(gpu, Sq, Sk):
    g = torch.Generator().manual_seed(Sq + Sk)
    blocks = torch.randint(0, 3, (Sq // 32, Sk // 16), generator=g)
    m = blocks.repeat_interleave(32, 0).repeat_interleave(16, 1)
    m = torch.where(m == 2, torch.randint(0, 2, (Sq, Sk), generator=g), m).bool().to(gpu)[None, None]
    for BQ, BK in ((32, 16), (Sq, 16), (32, Sk if Sk <= 1024 and Sk & (Sk - 1) == 0 else 16)):
        check(m, BQ, BK)


@pytest.mark.parametrize("BQ,BK", [(32, 8), (24, 40), (128, 2048), (5, 3), (32, 48)])
def test_generic_path_tile_shapes(gpu, BQ, BK):
    Sq = BQ * 7
    Sk = BK * 5 if BK < 2048 else 4096
    g = torch.Generator().manual_seed(BQ + BK)
    m = (torch.rand(2, 1, Sq, Sk, generator=g) < 0.5)
    m[0, 0, :BQ, :BK] = True
    m[0, 0, BQ:2 * BQ, :BK] = False
    check(m.to(gpu).expand(2, 3, Sq, Sk), BQ, BK)


def test_generic_path_strided_and_misaligned_views(gpu):
    S = 256
    base = W.random_block_mask(S, 32, 0.5, seed=1, device=gpu)
    t = base.t()[None, None]                      # key stride != 1
    assert t.stride(-1) != 1
    check(t, 64, 32, "transposed")
    wide = torch.zeros(S, S + 32, dtype=torch.bool, device=gpu)
    wide[:, 1:S + 1] = base
    off = wide[:, 1:S + 1][None, None]            # base pointer off by one byte
    assert off.data_ptr() % 16 != 0
    check(off, 64, 32, "misaligned base")
    odd = torch.zeros(S, S + 8, dtype=torch.bool, device=gpu)
    odd[:, :S] = base                              # row pitch not a multiple of 16
    check(odd[:, :S][None, None], 128, 32, "odd row pitch")
    sub = base[::2, :][None, None]                # row stride 2*S: still the wide path
    check(sub, 32, 32, "row-strided")


def test_broadcast_planes(gpu):
    S, B, H = 512, 3, 4
    one = W.random_block_mask(S, 32, 0.5, seed=3, device=gpu)
    got = check(one[None, None].expand(B, H, S, S), 128, 32, "[1,1] expanded")
    assert got.unmasked_kv_ids.shape == (B, H, 4, 16) and got.unmasked_kv_ids.stride()[:2] == (0, 0)
    per_b = W.random_block_mask(S, 32, 0.5, seed=4, device=gpu, batch=B)
    got = check(per_b.expand(B, H, S, S), 128, 32, "[B,1] expanded")
    assert got.unmasked_lens.stride(1) == 0 and got.unmasked_lens.stride(0) != 0
    g = torch.Generator().manual_seed(0)
    full = (torch.rand(B, H, S, S, generator=g) < 0.9).to(gpu)
    full[:, :, :128, :64] = True
    check(full, 128, 32, "distinct planes")
    per_h = full[:1].expand(B, H, S, S)
    check(per_h, 64, 64, "[1,H] expanded")


def test_bytes_other_than_one_count_as_true(gpu):
    S = 128
    raw = torch.zeros(S, S, dtype=torch.uint8)
    raw[:64, :64] = 255
    raw[64:, 64:] = 2
    raw[70, 70] = 0
    raw[0:32, 96:128] = 128
    m = raw.to(gpu).view(torch.bool)[None, None]
    got = compute_mask_kernel(m, 32, 32)
    torch.cuda.synchronize()
    want = oracle.classify(raw.numpy()[None, None], 32, 32)
    assert_metadata_equal(got, want, "non-0/1 bytes")


def test_structured_masks_closed_forms(gpu):
    S = 4096
    got = check(W.causal_mask(S, gpu)[None, None], 128, 32, "causal 4096")
    full, part = lists_of(got)
    want_full, want_part = causal_closed_form(S, 128, 32)
    assert full == want_full and part == want_part
    assert int(got.unmasked_lens.sum()) == 1984 and int(got.masked_lens.sum()) == 128


@pytest.mark.parametrize("p", [0.25, 0.5, 0.75, 0.9])
def test_random_block_config_full_size(gpu, p):
    m = W.random_block_mask(4096, 128, p, seed=int(p * 100), device=gpu)
    check(m[None, None].expand(8, 32, 4096, 4096), 128, 32, f"random block p={p}")
    mb = W.random_block_mask(4096, 128, p, seed=int(p * 100) + 1, device=gpu, batch=2)
    check(mb.expand(2, 4, 4096, 4096), 128, 32, f"random block per batch p={p}")


def test_document_config_full_size(gpu):
    S = 16384
    m = W.document_mask(S, seed=0, device=gpu)[None, None]
    got = check(m.expand(4, 32, S, S), 128, 32, "documents 16384")
    lens = W.document_lengths(S, 0)
    assert sum(lens) == S
    # a Q tile never lists a key tile that starts after its last query or ends before its first document starts
    starts = np.cumsum([0] + lens[:-1])
    full, part = lists_of(got)
    for i, (f, pl) in enumerate(zip(full, part)):
        q0, q1 = i * 128, i * 128 + 127
        first_doc_start = max(s for s in starts if s <= q0)
        for j in f + pl:
            assert j * 32 <= q1 and (j + 1) * 32 - 1 >= first_doc_start


def test_composed_config_full_size(gpu):
    S = 32768
    m = W.composed_mask(S, device=gpu)[None, None]
    got = compute_mask_kernel(m.expand(1, 32, S, S), 128, 32)
    torch.cuda.synchronize()
    assert int(got.unmasked_lens[0, 0].sum()) == 7744 and int(got.masked_lens[0, 0].sum()) == 1920
    want = oracle.classify(m.cpu().numpy(), 128, 32)
    one_plane = type(got)(got.unmasked_kv_ids[:1, :1], got.unmasked_lens[:1, :1], got.masked_kv_ids[:1, :1], got.masked_lens[:1, :1])
    assert_metadata_equal(one_plane, want, "composed 32768")


@pytest.mark.parametrize("name", golden_io.names())
def test_golden_lists(gpu, name):
    g = golden_io.load(name)
    m = torch.from_numpy(g.mask).to(gpu)[None, None]
    got = compute_mask_kernel(m, g.BQ, g.BK)
    torch.cuda.synchronize()
    plane = type(got)(got.unmasked_kv_ids[0, 0], got.unmasked_lens[0, 0], got.masked_kv_ids[0, 0], got.masked_lens[0, 0])
    assert_metadata_equal(plane, g.meta, name)


def test_slots_past_the_count_are_left_untouched(gpu):
    # straight through the C ABI with caller-owned, pre-filled outputs and materialised planes
    lib = _native.load()
    B, H, S, BQ, BK = 2, 2, 256, 64, 32
    nQ, nK = S // BQ, S // BK
    m = W.random_block_mask(S, 32, 0.5, seed=9, device=gpu)[None, None].expand(B, H, S, S)
    sentinel = 123456
    fid = torch.full((B, H, nQ, nK), sentinel, dtype=torch.int32, device=gpu)
    pid = torch.full((B, H, nQ, nK), sentinel, dtype=torch.int32, device=gpu)
    fl = torch.full((B, H, nQ), sentinel, dtype=torch.int32, device=gpu)
    pl = torch.full((B, H, nQ), sentinel, dtype=torch.int32, device=gpu)
    ms = _native.strides(m.stride())
    need = lib.sa_mask_classify_workspace_bytes(ms, B, H, S, S, BQ, BK)
    assert need == nQ * nK
    ws = torch.empty(need, dtype=torch.uint8, device=gpu)
    S_ = _native.strides
    rc = lib.sa_mask_classify(m.data_ptr(), ms, B, H, S, S, BQ, BK, fid.data_ptr(), S_(fid.stride()), fl.data_ptr(),
                              S_(fl.stride()), pid.data_ptr(), S_(pid.stride()), pl.data_ptr(), S_(pl.stride()),
                              ws.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.sa_last_error()
    torch.cuda.synchronize()
    want = oracle.classify(m.cpu().numpy(), BQ, BK)
    got = type("M", (), dict(unmasked_kv_ids=fid, unmasked_lens=fl, masked_kv_ids=pid, masked_lens=pl))
    assert_metadata_equal(got, want, "materialised planes from a broadcast mask")
    pos = torch.arange(nK, device=gpu)
    assert (fid[pos >= fl[..., None]] == sentinel).all() and (pid[pos >= pl[..., None]] == sentinel).all()


def test_runs_on_a_side_stream(gpu):
    S = 1024
    m = W.random_block_mask(S, 64, 0.5, seed=5, device=gpu)[None, None]
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        got = compute_mask_kernel(m, 128, 32)
    s.synchronize()
    assert_metadata_equal(got, oracle.classify(m.cpu().numpy(), 128, 32), "side stream")
