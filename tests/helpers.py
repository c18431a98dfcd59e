"""Shared checks for the parity tests."""
import numpy as np
import torch


def assert_metadata_equal(got, want, what=""):
    """Bit-exact comparison of two metadata carriers: lens everywhere, ids only in [..., :len].

    Slots past the count are unspecified in the reference (torch.empty, mask_utils.py:91-94)."""
    def np_(t):
        return t.detach().cpu().numpy() if isinstance(t, torch.Tensor) else np.asarray(t)

    for ids_name, lens_name in (("unmasked_kv_ids", "unmasked_lens"), ("masked_kv_ids", "masked_lens")):
        g_ids, g_len = np_(getattr(got, ids_name)), np_(getattr(got, lens_name))
        w_ids, w_len = np_(getattr(want, ids_name)), np_(getattr(want, lens_name))
        assert g_ids.dtype == np.int32 and g_len.dtype == np.int32, f"{what}: {ids_name}/{lens_name} must be int32"
        assert g_ids.shape == w_ids.shape and g_len.shape == w_len.shape, f"{what}: shape of {ids_name}"
        assert np.array_equal(g_len, w_len), f"{what}: {lens_name} differ"
        valid = np.arange(w_ids.shape[-1]) < w_len[..., None]
        assert np.array_equal(g_ids[valid], w_ids[valid]), f"{what}: {ids_name}[..., :len] differ"


def causal_closed_form(S, BQ, BK):
    """Lists of a causal mask (kv <= q) by arithmetic, not by counting.

    KV tile j of Q tile i is full iff its last key <= the tile's first query:
    (j+1)*BK - 1 <= i*BQ; non-empty iff its first key <= the tile's last query: j*BK <= (i+1)*BQ - 1."""
    nQ, nK = S // BQ, S // BK
    full = [[j for j in range(nK) if (j + 1) * BK - 1 <= i * BQ] for i in range(nQ)]
    part = [[j for j in range(nK) if not ((j + 1) * BK - 1 <= i * BQ) and j * BK <= (i + 1) * BQ - 1] for i in range(nQ)]
    return full, part


def lists_of(meta, b=0, h=0):
    """Python lists of the valid ids of plane (b,h)."""
    fid = meta.unmasked_kv_ids[b, h].tolist() if isinstance(meta.unmasked_kv_ids, torch.Tensor) else meta.unmasked_kv_ids[b, h].tolist()
    pid = meta.masked_kv_ids[b, h].tolist()
    fl = meta.unmasked_lens[b, h].tolist()
    pl = meta.masked_lens[b, h].tolist()
    return [row[:n] for row, n in zip(fid, fl)], [row[:n] for row, n in zip(pid, pl)]
