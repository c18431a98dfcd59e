"""Pins of the oracle's bit-packing of PARTIAL tiles (oracle.pack_partial): numpy.packbits of the same tiles,
the closed form of causal diagonal tiles, bytes other than 0/1, strided and broadcast masks, untouched slots."""
import numpy as np
import pytest

import oracle


def tiles_by_packbits(mask, BQ, BK, meta):
    B, H, Sq, Sk = mask.shape
    nQ, nK = Sq // BQ, Sk // BK
    out = np.zeros((B, H, nQ, nK, BQ * BK // 8), np.uint8)
    for b in range(B):
        for h in range(H):
            for i in range(nQ):
                for s in range(meta.masked_lens[b, h, i]):
                    j = meta.masked_kv_ids[b, h, i, s]
                    tile = mask[b, h, i * BQ:(i + 1) * BQ, j * BK:(j + 1) * BK] != 0
                    out[b, h, i, s] = np.packbits(tile.reshape(-1), bitorder="little")
    return out


@pytest.mark.parametrize("BQ,BK", [(32, 16), (128, 32), (64, 64), (16, 8), (48, 24), (256, 128)])
def test_against_numpy_packbits(BQ, BK):
    rng = np.random.default_rng(BQ * 1000 + BK)
    Sq, Sk = 3 * BQ, 5 * BK
    blocks = rng.integers(0, 3, size=(2, 2, 3, 5))  # 0 empty, 1 full, 2 coin flips
    coin = rng.integers(0, 2, size=(2, 2, Sq, Sk)).astype(bool)
    lab = blocks.repeat(BQ, 2).repeat(BK, 3)
    mask = np.where(lab == 2, coin, lab == 1)
    meta = oracle.classify(mask, BQ, BK)
    assert meta.masked_lens.sum() > 0
    got = oracle.pack_partial(mask, BQ, BK, meta)
    assert got.shape == (2, 2, 3, 5, BQ * BK // 8)
    assert np.array_equal(got, tiles_by_packbits(mask, BQ, BK, meta))


def test_causal_diagonal_tiles_closed_form():
    # tiles 128x32 on the diagonal of a causal mask: Q tile i has PARTIAL KV tiles 4i..4i+3; in slot s, row r
    # attends to columns c with 32s + c <= r, i.e. bits 0..min(31, r-32s) are set
    S, BQ, BK = 512, 128, 32
    idx = np.arange(S)
    mask = (idx[None, :] <= idx[:, None])[None, None]
    packed = oracle.pack_partial(mask, BQ, BK)
    words = packed.view("<u4")  # [1,1,nQ,nK,BQ] one word per row
    for i in range(S // BQ):
        for s in range(4):
            for r in range(BQ):
                n = min(32, max(0, r - 32 * s + 1))
                assert int(words[0, 0, i, s, r]) == (1 << n) - 1, (i, s, r)


def test_nonzero_bytes_strides_broadcast_and_untouched_slots():
    rng = np.random.default_rng(7)
    raw = rng.integers(0, 256, size=(64, 96), dtype=np.uint8)
    raw[rng.random(raw.shape) < 0.6] = 0
    m = np.broadcast_to(raw[None, None], (2, 3, 64, 96))
    got = oracle.pack_partial(m, 32, 16, fill=0xAB)
    meta = oracle.classify(m, 32, 16)
    want = tiles_by_packbits(np.ascontiguousarray(m), 32, 16, meta)
    pos = np.arange(6) < meta.masked_lens[..., None]
    assert np.array_equal(got[pos], want[pos])
    assert (got[~pos] == 0xAB).all()
    # transposed view (key stride != 1)
    mt = np.ascontiguousarray(raw.T)[None, None].transpose(0, 1, 3, 2)
    assert mt.strides[-1] != 1
    assert np.array_equal(oracle.pack_partial(mt, 32, 16)[pos[:1, :1]], want[:1, :1][pos[:1, :1]])


def test_rejects_tiles_that_do_not_pack():
    with pytest.raises(ValueError):
        oracle.pack_partial(np.ones((1, 1, 32, 36), bool), 32, 12)
