"""Block-sparse attention forward (replaces the reference's ``sparseattention/sparse_attn_kernel.py``)."""
from __future__ import annotations

import math

import torch

from . import _native
from .mask_utils import MaskMetadata, Tiling, compute_mask_kernel, compute_mask_terms, validation_key

_DTYPES = {torch.bfloat16: _native.SA_DTYPE_BF16, torch.float16: _native.SA_DTYPE_FP16}
# the forward also takes float32 (kernels that compute in float32 throughout: on the fp32 matrix instruction at head
# dims 64 and 128 with Q tiles of 64 or 128 rows, on the vector units otherwise)
_FWD_DTYPES = {**_DTYPES, torch.float32: _native.SA_DTYPE_FP32}


def _kernel_ready(t: torch.Tensor) -> torch.Tensor:
    """The kernels want a unit stride in D, 16-byte aligned rows; copy only when that does not hold."""
    per16 = 16 // t.element_size()
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % per16 == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


def _kernel_head_dim(D: int, sizes) -> int:
    """The head dim the kernels run a request for ``D`` with: the smallest of ``sizes`` that holds it (q, k, v are then
    padded with zero columns, which change neither the scores nor the first D columns of the result; the softmax scale
    stays that of D).  A D beyond all of them is passed on, for the library to refuse."""
    return next((s for s in sizes if D <= s), D)


def _pad_head_dim(t: torch.Tensor, Dk: int) -> torch.Tensor:
    return t if t.shape[-1] == Dk else torch.nn.functional.pad(t, (0, Dk - t.shape[-1]))


def _pad_mask(mask: torch.Tensor, q_multiple: int, k_multiple: int) -> torch.Tensor:
    """``mask`` [B,H,Sq,Sk] with all-False rows and columns added up to multiples of the two numbers; only the
    distinct planes of a broadcast view are copied."""
    B, H, Sq, Sk = mask.shape
    if Sq % q_multiple == 0 and Sk % k_multiple == 0:
        return mask
    distinct = mask[: 1 if mask.stride(0) == 0 else B, : 1 if mask.stride(1) == 0 else H]
    padded = torch.nn.functional.pad(distinct, (0, -Sk % k_multiple, 0, -Sq % q_multiple), value=False)
    return padded.expand(B, H, *padded.shape[2:])


def _same_device(ref: torch.Tensor, **tensors) -> None:
    """Every tensor whose data pointer goes to a kernel must live where ``ref`` lives: a host pointer (or one of
    another GPU) in any slot would be a memory fault on the device, where the reference raises a Python error."""
    for name, t in tensors.items():
        if t is not None and t.device != ref.device:
            raise ValueError(f"{name} is on {t.device}, expected {ref.device} (every tensor argument must be on q's device)")


def validate_metadata(md: MaskMetadata, Sk: int, BLOCK_K: int) -> None:
    """Raise ValueError unless the lists can address K and V: ``0 <= lens``, ``unmasked_lens + masked_lens <= Sk/BLOCK_K``
    and ``0 <= ids[..., :len] < Sk/BLOCK_K`` (the reference guards its loads with ``kv_offset < SEQLEN_K``,
    sparse_attn_kernel.py:35,39,60).  Plain torch on the tensors' own device; reads two flags back, so it synchronises.
    The wrappers run it once per metadata object that did not come from this package's own preprocessing; the kernels
    additionally clamp counts and skip indices out of range, so unchecked metadata cannot fault either."""
    nK = Sk // BLOCK_K
    bad = []
    fl, pl = md.unmasked_lens, md.masked_lens
    if bool(((fl < 0) | (pl < 0) | (fl.to(torch.int64) + pl.to(torch.int64) > nK)).any()):
        bad.append(f"counts outside [0, {nK}] or unmasked_lens + masked_lens > {nK}")
    for name, ids, lens in (("unmasked_kv_ids", md.unmasked_kv_ids, fl), ("masked_kv_ids", md.masked_kv_ids, pl)):
        if ids.shape[-1] != nK:
            bad.append(f"{name} has {ids.shape[-1]} slots per Q tile, expected {nK}")
            continue
        live = torch.arange(nK, device=ids.device) < lens[..., None]
        if bool((live & ((ids < 0) | (ids >= nK))).any()):
            bad.append(f"{name}[..., :len] holds tile indices outside [0, {nK})")
    if bad:
        raise ValueError("mask_metadata does not fit Sk=%d, BLOCK_K=%d: %s" % (Sk, BLOCK_K, "; ".join(bad)))


def _checked_metadata(md: MaskMetadata, Sk: int, BLOCK_K: int) -> None:
    """validate_metadata once per (object, tiling, state of its list tensors); metadata made by compute_mask_kernel /
    compute_mask_terms is trusted (marked there), so the usual call path never synchronises.  Lists edited in place
    afterwards, or an object whose tensors were exchanged (dataclasses.replace, copy), are checked again."""
    key = validation_key(md, Sk, BLOCK_K)
    if getattr(md, "_validated_for", None) == key:
        return
    validate_metadata(md, Sk, BLOCK_K)
    try:
        md._validated_for = key
    except AttributeError:  # the reference's own dataclass, say: a carrier without the field is checked every time
        pass


_KERNEL_BLOCK_Q = (128, 64, 32, 256)  # in order of preference when the caller's size is not one of them


def kernel_tiles(Sq: int, Sk: int, D: int, BLOCK_Q: int, BLOCK_K: int):
    """The tile sizes the forward runs a request for ``BLOCK_Q`` x ``BLOCK_K`` tiles with: the same pair when the
    kernels tile by it (BLOCK_Q 32/64/128/256 — 64/128 at head dim 256 —, BLOCK_K a power of two >= 16), else the
    nearest pair they have that divides Sq and Sk, or None when there is none.  The reference takes any sizes its
    compiler accepts (sparse_attn_kernel.py:149-185); the result does not depend on them."""
    BLOCK_Q, BLOCK_K = int(BLOCK_Q), int(BLOCK_K)
    ok_k = BLOCK_K >= 16 and BLOCK_K & (BLOCK_K - 1) == 0 and Sk % BLOCK_K == 0
    if Sq < 32:  # the few-rows kernels: one Q tile of all rows, KV tiles of 16 keys or more, head dims up to 128
        if D > 128:
            return None
        if ok_k:
            return Sq, BLOCK_K
        return next(((Sq, bk) for bk in (32, 64) if Sk % bk == 0), None)
    ok_q = [b for b in _KERNEL_BLOCK_Q if Sq % b == 0 and (D <= 128 or b in (64, 128))]  # (D above 128 runs as 256)
    if not ok_q:
        return None
    bq = BLOCK_Q if BLOCK_Q in ok_q else ok_q[0]
    if ok_k:
        return bq, BLOCK_K
    return next(((bq, bk) for bk in (32, 64, 16) if Sk % bk == 0), None)


# Below this many listed keys per Q tile (mean over the Q tiles) the forward runs its short-list kernel when the
# metadata says so (MaskMetadata.list_stats) and the kernel has the sizes.  Measured on MI355X (B8 H32 S4096 D128,
# tiles 128x32, default / short-list kernel): 448 keys per Q tile 0.343 / 0.340 ms, 1222 keys 0.709 / 0.719 ms,
# 2100 keys and more +5 ... +8 %: the third workgroup per compute unit pays for itself on the shortest lists only.
SHORT_LIST_KEYS = 512


def _short_list_kernel(mask_metadata, dtype, D, BLOCK_Q, BLOCK_K, kernel) -> bool:
    """Whether this call runs the kernel for short lists (three workgroups per compute unit, 32 keys per step)."""
    if kernel not in (None, "auto", "default", "short", "rotated"):
        raise ValueError(f"kernel must be 'auto', 'default', 'rotated' or 'short' (got {kernel!r})")
    if kernel in ("default", "rotated"):
        return False
    has = (dtype in _DTYPES and D == 128 and BLOCK_Q == 128 and BLOCK_K >= 16 and BLOCK_K & (BLOCK_K - 1) == 0
           and getattr(mask_metadata, "packed_masks", None) is not None
           and getattr(mask_metadata, "schedule", None) is None)
    stats = getattr(mask_metadata, "list_stats", None)
    fits = stats is not None and stats[1] <= _native.SA_FWD_SHORT_LISTS_MAX_ENTRIES
    if kernel == "short":
        if not (has and fits):
            raise ValueError("kernel='short' needs bf16/fp16, head dim 128, BLOCK_Q 128, mask_metadata with packed_masks, "
                             "no schedule, and list_stats whose longest list has at most "
                             f"{_native.SA_FWD_SHORT_LISTS_MAX_ENTRIES} entries")
        return True
    return has and fits and stats[0] * BLOCK_K < SHORT_LIST_KEYS


def sparse_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor | None, BLOCK_Q, BLOCK_K,
                     mask_metadata: MaskMetadata | None = None, *, return_lse: bool = False, kernel: str | None = None):
    """softmax(q kᵀ / sqrt(D) + (mask ? 0 : -inf)) v, skipping KV tiles the mask empties.

    Signature and meaning follow sparse_attn_kernel.py:149-185: ``q`` [B,H,Sq,D], ``k``/``v``
    [B,H,Sk,D] (bf16, fp16, or float32 on kernels that compute in float32 throughout; on a
    ROCm GPU), ``mask`` bool broadcastable to [B,H,Sq,Sk] with
    True = attend, tile sizes ``BLOCK_Q`` x ``BLOCK_K``, and optionally the metadata from
    :func:`compute_mask_kernel` so that preprocessing is paid once for many calls.
    Returns ``o`` with q's shape, dtype and strides; with ``return_lse=True`` (not in the reference, which drops
    the row statistics after the division at sparse_attn_kernel.py:144) the pair ``(o, lse)`` where ``lse``
    [B,H,Sq] float32 is the log of the row's softmax denominator, -inf for rows that attend to nothing.
    ``mask`` may be None when ``mask_metadata`` carries ``packed_masks`` (the kernels then read no mask tensor), which
    is how masks given by a formula run (:func:`compute_mask_terms`).
    ``kernel`` (not in the reference, whose one kernel Triton autotunes at the first call, sparse_attn_kernel.py:66-72):
    "default" = two workgroups per compute unit, 64 keys per step; "short" = the form for masks that leave a Q tile
    few KV tiles (three workgroups per compute unit, 32 keys per step; bf16/fp16, D = 128, BLOCK_Q = 128, packed
    PARTIAL tiles, ``mask_metadata.list_stats`` with no list above 256 entries); None / "auto" = "short" when the
    metadata carries ``list_stats`` (``compute_mask_kernel(..., list_stats=True)``) that say the lists are short,
    else "default".  "rotated" = the default kernel with the FULL entries of Q tile qt walked from a start that depends
    on qt (for sliding windows; "auto" takes it when ``mask_metadata.list_rotation`` says so).  All agree within rounding.
    """
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [B,H,S,D]")
    B, H, Sq, D = q.shape
    Sk = k.shape[-2]
    if k.shape != (B, H, Sk, D) or v.shape != (B, H, Sk, D):
        raise ValueError(f"k/v shapes {tuple(k.shape)}/{tuple(v.shape)} do not match q {tuple(q.shape)}")
    if not q.is_cuda:
        raise RuntimeError("sparse_attention needs q, k, v on a ROCm GPU; there is no CPU path")
    _same_device(q, k=k, v=v, mask=mask)
    if q.dtype not in _FWD_DTYPES or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError(f"q, k, v must share dtype bfloat16, float16 or float32 (got {q.dtype}, {k.dtype}, {v.dtype})")
    f32 = q.dtype == torch.float32
    if mask is None and getattr(mask_metadata, "packed_masks", None) is None:
        raise ValueError("sparse_attention without a mask tensor needs mask_metadata with packed_masks")
    if mask is not None:
        mask = mask.expand(B, H, Sq, Sk)
    BLOCK_Q, BLOCK_K = int(BLOCK_Q), int(BLOCK_K)
    if f32 and 1 <= BLOCK_Q <= (256 if D <= 128 else 128) and BLOCK_K >= 1 and Sq % BLOCK_Q == 0 and Sk % BLOCK_K == 0:
        tiles = (BLOCK_Q, BLOCK_K)  # the float32 kernel tiles by any sizes up to 256 query rows (128 at head dims above 128)
    else:
        tiles = kernel_tiles(Sq, Sk, D, BLOCK_Q, BLOCK_K)
    row_multiple = 32 if D <= 128 else 64  # the smallest Q tile the kernels have
    if tiles is None and mask is not None and Sq % row_multiple and Sq % BLOCK_Q == 0 and Sk % BLOCK_K == 0:
        # A row count that no Q tile of the kernels divides (48, 80, ...; fewer than 32 rows at a head dim the few-rows
        # kernels do not have): zero rows are added to q and all-False rows to the mask, and their (zero) output rows
        # dropped again.  Nothing is kept between calls on this path.
        pad = -Sq % row_multiple
        padded_tiles = kernel_tiles(Sq + pad, Sk, D, BLOCK_Q, BLOCK_K)
        if padded_tiles is not None:
            out = sparse_attention(torch.nn.functional.pad(q, (0, 0, 0, pad)), k, v, _pad_mask(mask, row_multiple, 1),
                                   *padded_tiles, return_lse=return_lse)
            return (out[0][:, :, :Sq].contiguous(), out[1][:, :, :Sq].contiguous()) if return_lse \
                else out[:, :, :Sq].contiguous()
    if tiles != (BLOCK_Q, BLOCK_K):
        # Tile sizes the kernels do not tile by.  They only say how the mask is cut up, not what is computed, so the
        # mask is classified again at sizes the kernels have; the lists are kept on the caller's metadata.
        # what the reference asserts (mask_utils.py:89-90)
        assert Sq % BLOCK_Q == 0 and Sk % BLOCK_K == 0, \
            f"Sq={Sq} / Sk={Sk} must be multiples of BLOCK_Q={BLOCK_Q} / BLOCK_K={BLOCK_K}"
        if tiles is None or mask is None:
            raise ValueError(f"sparse_attention: no kernel tiles for BLOCK_Q={BLOCK_Q}, BLOCK_K={BLOCK_K} at Sq={Sq}, "
                             f"Sk={Sk}, D={D}" + ("" if tiles is None else " without a mask tensor to classify again"))
        again = getattr(mask_metadata, "_retiled", None)
        if again is None or again[0] != (tiles, mask.data_ptr(), tuple(mask.stride()), mask._version):
            again = ((tiles, mask.data_ptr(), tuple(mask.stride()), mask._version),
                     compute_mask_kernel(mask, *tiles, pack_partial=None if Sq >= 32 else False))
            if mask_metadata is not None:
                mask_metadata._retiled = again
        BLOCK_Q, BLOCK_K = tiles
        mask_metadata = again[1]

    if Sq == BLOCK_Q and Sq < 32 and BLOCK_K >= 16 and not f32:
        # one Q tile of fewer rows than the forward kernels tile by: the split-KV kernels (they use no schedule, and take
        # the packed tiles where the metadata carries them, so `mask` may be None there as it may for the forward)
        return sparse_attention_decode(q, k, v, mask, BLOCK_K, mask_metadata, return_lse=return_lse)
    sm_scale = D ** (-0.5) * 1 / math.log(2)  # exp2 replaces exp (sparse_attn_kernel.py:152)

    if mask_metadata is None:
        mask_metadata = compute_mask_kernel(mask, BLOCK_Q, BLOCK_K)
    fid, fl = mask_metadata.unmasked_kv_ids, mask_metadata.unmasked_lens
    pid, pl = mask_metadata.masked_kv_ids, mask_metadata.masked_lens
    nQ, nK = Sq // BLOCK_Q, Sk // BLOCK_K
    for name, t, shape in (("unmasked_kv_ids", fid, (B, H, nQ, nK)), ("masked_kv_ids", pid, (B, H, nQ, nK)),
                           ("unmasked_lens", fl, (B, H, nQ)), ("masked_lens", pl, (B, H, nQ))):
        if tuple(t.shape) != shape or t.dtype != torch.int32 or t.device != q.device:
            raise ValueError(f"mask_metadata.{name}: expected int32 {shape} on {q.device}, got {t.dtype} {tuple(t.shape)} on {t.device}")
    _checked_metadata(mask_metadata, Sk, BLOCK_K)
    if mask is not None:
        assert mask.dtype == torch.bool, "mask must be a torch.bool tensor"
    packed = getattr(mask_metadata, "packed_masks", None)
    if packed is not None:
        shape = (B, H, nQ, nK, BLOCK_Q * BLOCK_K // 8)
        if (tuple(packed.shape) != shape or packed.dtype != torch.uint8 or packed.device != q.device
                or packed.stride()[2:] != (nK * shape[4], shape[4], 1)):
            raise ValueError(f"mask_metadata.packed_masks: expected uint8 {shape} on {q.device} with contiguous "
                             f"tiles, got {packed.dtype} {tuple(packed.shape)} strides {packed.stride()}")

    sched = getattr(mask_metadata, "schedule", None)
    if sched is not None and (sched.dtype != torch.int32 or sched.device != q.device or not sched.is_contiguous()):
        raise ValueError("mask_metadata.schedule: expected a contiguous int32 tensor on q's device")

    Dk = _kernel_head_dim(D, (64, 128, 256))
    qc, kc, vc = (_kernel_ready(_pad_head_dim(t, Dk)) for t in (q, k, v))
    o = torch.empty_like(qc)
    lib = _native.load()
    S = _native.strides
    with torch.cuda.device(q.device):
        common = (qc.data_ptr(), S(qc.stride()), kc.data_ptr(), S(kc.stride()), vc.data_ptr(), S(vc.stride()),
                  o.data_ptr(), S(o.stride()),
                  mask.data_ptr() if mask is not None else None, S(mask.stride()) if mask is not None else None,
                  fid.data_ptr(), S(fid.stride()), fl.data_ptr(), S(fl.stride()),
                  pid.data_ptr(), S(pid.stride()), pl.data_ptr(), S(pl.stride()))
        tail = (B, H, Sq, Sk, Dk, int(BLOCK_Q), int(BLOCK_K), _FWD_DTYPES[q.dtype], sm_scale,
                torch.cuda.current_stream(q.device).cuda_stream)
        sched = getattr(mask_metadata, "schedule", None)
        if kernel == "rotated" and (sched is not None or q.dtype not in _DTYPES):
            raise ValueError("kernel='rotated' needs bf16/fp16 and mask_metadata without a schedule")
        lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device) if return_lse else None
        if _short_list_kernel(mask_metadata, q.dtype, Dk, int(BLOCK_Q), int(BLOCK_K), kernel):
            rc = lib.sa_sparse_attention_fwd_kernel(
                *common, packed.data_ptr(), S(packed.stride()[:2]), lse.data_ptr() if return_lse else None,
                S(lse.stride()) if return_lse else None, *tail[:-1], _native.SA_FWD_KERNEL_SHORT_LISTS, tail[-1])
        elif (sched is None and q.dtype in _DTYPES
              and (kernel == "rotated" or (kernel in (None, "auto") and getattr(mask_metadata, "list_rotation", 0) > 0))):
            # the default kernel with the FULL entries of Q tile qt walked from a start that depends on qt
            group = int(getattr(mask_metadata, "list_rotation", 0)) or 16
            rc = lib.sa_sparse_attention_fwd_kernel(
                *common, *((packed.data_ptr(), S(packed.stride()[:2])) if packed is not None else (None, None)),
                lse.data_ptr() if return_lse else None, S(lse.stride()) if return_lse else None, *tail[:-1],
                _native.SA_FWD_KERNEL_ROTATED | (group << 8), tail[-1])
        elif packed is not None or sched is not None or return_lse:
            pk = (packed.data_ptr(), S(packed.stride()[:2])) if packed is not None else (None, None)
            sc = ((sched.data_ptr(), sched.numel() * 4, int(getattr(mask_metadata, "schedule_mode", 0)))
                  if sched is not None else (None, 0, 0))
            if return_lse:
                rc = lib.sa_sparse_attention_fwd_lse(*common, *pk, *sc, lse.data_ptr(), S(lse.stride()), *tail)
            else:
                rc = lib.sa_sparse_attention_fwd_ex(*common, *pk, *sc, *tail)
        else:
            rc = lib.sa_sparse_attention_fwd(*common, *tail)
    _native.check(rc)
    if Dk != D:
        o = o[..., :D].contiguous()
    return (o, lse) if return_lse else o


def sparse_attention_tiled(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, tiling: Tiling, *, return_lse: bool = False):
    """:func:`sparse_attention` on the tile grid chosen by :func:`sparseattention_amd.select_tiling`: q, k, v get
    ``q_offset`` / ``k_offset`` zero rows in front (and zero rows at the end up to whole tiles), which the padded mask
    lets nothing attend to or from, and the rows of the result that belong to the caller's queries are returned.  With
    both offsets 0 and sizes that are whole tiles this is sparse_attention itself; otherwise it costs a copy of q, k, v."""
    Sq, Sk = q.shape[-2], k.shape[-2]
    Pq, Pk = tiling.padded_mask.shape[-2:]
    qo, ko = tiling.q_offset, tiling.k_offset
    if not (qo + Sq <= Pq and ko + Sk <= Pk):
        raise ValueError(f"tiling for a mask of {Pq - qo}x{Pk - ko} or smaller, got Sq={Sq}, Sk={Sk}")
    pad = torch.nn.functional.pad
    qp = q if (qo, Pq) == (0, Sq) else pad(q, (0, 0, qo, Pq - qo - Sq))
    kp = k if (ko, Pk) == (0, Sk) else pad(k, (0, 0, ko, Pk - ko - Sk))
    vp = v if (ko, Pk) == (0, Sk) else pad(v, (0, 0, ko, Pk - ko - Sk))
    out = sparse_attention(qp, kp, vp, tiling.padded_mask, tiling.BLOCK_Q, tiling.BLOCK_K, tiling.metadata,
                           return_lse=return_lse)
    if (qo, Pq) == (0, Sq):
        return out
    if return_lse:
        return out[0][:, :, qo:qo + Sq].contiguous(), out[1][:, :, qo:qo + Sq].contiguous()
    return out[:, :, qo:qo + Sq].contiguous()


def sparse_attention_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor | None, BLOCK_K,
                            mask_metadata: MaskMetadata | None = None, num_splits: int = 0, *,
                            return_lse: bool = False):
    """:func:`sparse_attention` for Sq <= 32 query rows (decode, speculative or chunked-prefill tails), BLOCK_Q = Sq.

    The reference lists decode kernels as future work (README.md:65); the result is defined by its forward
    (sparse_attn_kernel.py:149-185) called with ``BLOCK_Q = Sq``.  Every (b, h) has one Q tile, so its list of KV
    tiles is cut into ``num_splits`` ranges (0: chosen from the shape and the device) that run in parallel and are
    merged afterwards.  ``mask_metadata``: from ``compute_mask_kernel(mask, Sq, BLOCK_K)``; when it carries
    ``packed_masks`` (the default there) the kernels read those bits and ``mask`` may be None (at BLOCK_K = 16 with an odd
    number of query rows the bool mask is read instead).  ``return_lse``: as in :func:`sparse_attention`.
    """
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [B,H,S,D]")
    B, H, Sq, D = q.shape
    Sk = k.shape[-2]
    if k.shape != (B, H, Sk, D) or v.shape != (B, H, Sk, D):
        raise ValueError(f"k/v shapes {tuple(k.shape)}/{tuple(v.shape)} do not match q {tuple(q.shape)}")
    if not q.is_cuda:
        raise RuntimeError("sparse_attention_decode needs q, k, v on a ROCm GPU; there is no CPU path")
    _same_device(q, k=k, v=v, mask=mask)
    if q.dtype not in _DTYPES or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError(f"q, k, v must share dtype bfloat16 or float16 (got {q.dtype}, {k.dtype}, {v.dtype})")
    sm_scale = D ** (-0.5) * 1 / math.log(2)
    if mask is not None:
        mask = mask.expand(B, H, Sq, Sk)
    if mask_metadata is None:
        if mask is None:
            raise ValueError("sparse_attention_decode needs the mask or mask_metadata with packed_masks")
        mask_metadata = compute_mask_kernel(mask, Sq, BLOCK_K)
    fid, fl = mask_metadata.unmasked_kv_ids, mask_metadata.unmasked_lens
    pid, pl = mask_metadata.masked_kv_ids, mask_metadata.masked_lens
    nK = Sk // BLOCK_K
    for name, t, shape in (("unmasked_kv_ids", fid, (B, H, 1, nK)), ("masked_kv_ids", pid, (B, H, 1, nK)),
                           ("unmasked_lens", fl, (B, H, 1)), ("masked_lens", pl, (B, H, 1))):
        if tuple(t.shape) != shape or t.dtype != torch.int32 or t.device != q.device:
            raise ValueError(f"mask_metadata.{name}: expected int32 {shape} on {q.device}, got {t.dtype} {tuple(t.shape)} on {t.device}")
    _checked_metadata(mask_metadata, Sk, BLOCK_K)
    packed = getattr(mask_metadata, "packed_masks", None)
    if packed is not None:
        shape = (B, H, 1, nK, Sq * int(BLOCK_K) // 8)
        if (tuple(packed.shape) != shape or packed.dtype != torch.uint8 or packed.device != q.device
                or packed.stride()[2:] != (nK * shape[4], shape[4], 1)):
            raise ValueError(f"mask_metadata.packed_masks: expected uint8 {shape} on {q.device} with contiguous tiles, got "
                             f"{packed.dtype} {tuple(packed.shape)} strides {packed.stride()}")
        if int(BLOCK_K) == 16 and Sq % 2:  # (halfword rows: the kernels want an even number of them)
            packed = None
    if packed is None:
        if mask is None:
            raise ValueError("sparse_attention_decode without a mask tensor needs mask_metadata with packed_masks "
                             "(and an even number of query rows at BLOCK_K = 16)")
        assert mask.dtype == torch.bool, "mask must be a torch.bool tensor"
    Dk = _kernel_head_dim(D, (64, 128))
    qc, kc, vc = (_kernel_ready(_pad_head_dim(t, Dk)) for t in (q, k, v))
    o = torch.empty_like(qc)
    lib = _native.load()
    S = _native.strides
    with torch.cuda.device(q.device):
        if num_splits == 0:
            num_splits = lib.sa_decode_num_splits(B, H, Sq, Sk, int(BLOCK_K))
        ws_bytes = lib.sa_decode_workspace_bytes(B, H, Sq, Dk, int(num_splits))
        ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=q.device) if ws_bytes else None
        lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device) if return_lse else None
        rc = lib.sa_sparse_attention_decode_ex(
            qc.data_ptr(), S(qc.stride()), kc.data_ptr(), S(kc.stride()), vc.data_ptr(), S(vc.stride()),
            o.data_ptr(), S(o.stride()), mask.data_ptr() if mask is not None else None,
            S(mask.stride()) if mask is not None else None,
            fid.data_ptr(), S(fid.stride()), fl.data_ptr(), S(fl.stride()),
            pid.data_ptr(), S(pid.stride()), pl.data_ptr(), S(pl.stride()),
            packed.data_ptr() if packed is not None else None, S(packed.stride()[:2]) if packed is not None else None,
            B, H, Sq, Sk, Dk, int(BLOCK_K), _DTYPES[q.dtype], sm_scale, int(num_splits),
            ws.data_ptr() if ws is not None else None, ws_bytes,
            lse.data_ptr() if lse is not None else None, S(lse.stride()) if lse is not None else None,
            torch.cuda.current_stream(q.device).cuda_stream)
    _native.check(rc)
    if Dk != D:
        o = o[..., :D].contiguous()
    return (o, lse) if return_lse else o


class BackwardMetadata:
    """Tile lists the backward pass walks: of the mask per 128 queries (KV tiles of 64 keys) and of the transposed
    mask per 128 keys (tiles of 64 queries).  Built once per mask by :func:`compute_backward_metadata`.

    When both lists carry ``packed_masks`` (the PARTIAL tiles at one bit per entry), the backward reads those and
    neither the mask nor its transposed copy, so both bool tensors can be released after this preprocessing."""

    def __init__(self, by_query: MaskMetadata, by_key: MaskMetadata, transposed_mask: torch.Tensor | None = None):
        self.by_query = by_query
        self.by_key = by_key
        #: bool [B,H,Sk,Sq], the mask transposed as a tensor of its own (distinct planes, expanded), or None
        self.transposed_mask = transposed_mask


def compute_backward_metadata(mask: torch.Tensor, pack_partial: bool = True) -> BackwardMetadata:
    """``mask``: bool [B,H,Sq,Sk] (broadcast views are fine).  Sq and Sk that are not multiples of 128 are taken up to
    the next one with rows and columns that attend to nothing, as :func:`sparse_attention_backward` does with its
    tensors.

    ``pack_partial``: bit-pack the PARTIAL tiles of both tilings (2 * Sq*Sk/8 bytes per distinct plane at most) and
    drop the transposed copy; otherwise keep that copy (Sq*Sk bytes per distinct plane) for the key passes."""
    if mask.dim() != 4:
        raise ValueError("mask must be [B,H,Sq,Sk] (broadcast views are fine)")
    mask = _pad_mask(mask, 128, 128)
    # the transposed mask as a tensor of its own, distinct planes only, so that its classification reads rows
    B, H = mask.shape[:2]
    distinct = mask[: 1 if mask.stride(0) == 0 else B, : 1 if mask.stride(1) == 0 else H]
    transposed = distinct.transpose(-1, -2).contiguous().expand(B, H, mask.shape[3], mask.shape[2])
    return BackwardMetadata(compute_mask_kernel(mask, 128, 64, pack_partial=pack_partial),
                            compute_mask_kernel(transposed, 128, 64, pack_partial=pack_partial),
                            None if pack_partial else transposed)


def compute_backward_metadata_terms(terms, B: int, H: int, Sq: int, Sk: int, doc_q=None, doc_k=None,
                                    device=None) -> BackwardMetadata:
    """:func:`compute_backward_metadata` for a mask given by terms (:func:`compute_mask_terms`): both tilings with
    their packed PARTIAL tiles, the key-major one from the transposed terms, so that
    ``sparse_attention_backward(..., mask=None, bwd_metadata=...)`` runs without any mask tensor."""
    terms = list(terms)
    return BackwardMetadata(
        compute_mask_terms(terms, B, H, Sq, Sk, 128, 64, doc_q, doc_k, device),
        compute_mask_terms([t.transposed() for t in terms], B, H, Sk, Sq, 128, 64, doc_k, doc_q, device), None)


def sparse_attention_backward(do: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor,
                              lse: torch.Tensor, mask: torch.Tensor | None,
                              bwd_metadata: BackwardMetadata | None = None):
    """Gradients (dq, dk, dv) of :func:`sparse_attention` for the upstream gradient ``do``.

    The reference has no backward pass (README.md:65 lists it as future work); this differentiates its forward
    (sparse_attn_kernel.py:149-185).  ``o`` and ``lse`` come from ``sparse_attention(..., return_lse=True)`` with the
    same inputs.  bf16/fp16; the kernels have D = 64 and 128 and tile by 128 rows, other head dims up to 128 and
    other Sq, Sk are padded here (zero columns; rows that attend to nothing).  The backward tiles the mask its own way
    (128 x 64 both ways), whatever BLOCK_Q / BLOCK_K the forward used.  ``mask`` may be None when ``bwd_metadata``
    carries the packed PARTIAL tiles of both tilings.
    """
    B, H, Sq, D = q.shape
    Sk = k.shape[-2]
    if not q.is_cuda:
        raise RuntimeError("sparse_attention_backward needs its tensors on a ROCm GPU; there is no CPU path")
    _same_device(q, k=k, v=v, o=o, do=do, lse=lse, mask=mask)
    if q.dtype not in _DTYPES or any(t.dtype != q.dtype for t in (k, v, o, do)):
        raise TypeError("q, k, v, o, do must share dtype bfloat16 or float16")
    if k.shape != (B, H, Sk, D) or v.shape != k.shape or o.shape != q.shape or do.shape != q.shape:
        raise ValueError(f"shapes: q/o/do must be {(B, H, Sq, D)} and k/v {(B, H, Sk, D)} (got q {tuple(q.shape)}, "
                         f"k {tuple(k.shape)}, v {tuple(v.shape)}, o {tuple(o.shape)}, do {tuple(do.shape)})")
    if lse.dtype != torch.float32 or tuple(lse.shape) != (B, H, Sq):
        raise ValueError(f"lse: expected float32 {(B, H, Sq)}, got {lse.dtype} {tuple(lse.shape)}")
    if mask is not None:
        mask = mask.expand(B, H, Sq, Sk)
        assert mask.dtype == torch.bool, "mask must be a torch.bool tensor"
    if Sq % 128 or Sk % 128:
        # the kernels tile by 128 rows both ways: zero rows (lse = -inf: rows that attended to nothing) and mask rows
        # and columns that attend to nothing are added, and the gradients of the added rows dropped
        rows = lambda t, n: torch.nn.functional.pad(t, (0, 0, 0, -n % 128))  # noqa: E731
        dq, dk, dv = sparse_attention_backward(
            rows(do, Sq), rows(q, Sq), rows(k, Sk), rows(v, Sk), rows(o, Sq),
            torch.nn.functional.pad(lse, (0, -Sq % 128), value=float("-inf")),
            None if mask is None else _pad_mask(mask, 128, 128), bwd_metadata)
        return dq[:, :, :Sq].contiguous(), dk[:, :, :Sk].contiguous(), dv[:, :, :Sk].contiguous()
    if bwd_metadata is None:
        if mask is None:
            raise ValueError("sparse_attention_backward needs the mask or a BackwardMetadata with packed tiles")
        bwd_metadata = compute_backward_metadata(mask)
    sm_scale = D ** (-0.5) * 1 / math.log(2)
    Dk = _kernel_head_dim(D, (64, 128))
    qc, kc, vc, oc, doc = (_kernel_ready(_pad_head_dim(t, Dk)) for t in (q, k, v, o, do))
    dq, dk, dv = torch.empty_like(qc), torch.empty_like(kc), torch.empty_like(vc)
    lib = _native.load()
    S = _native.strides
    lists, packs = [], []
    for md, shape in ((bwd_metadata.by_query, (B, H, Sq // 128, Sk // 64)), (bwd_metadata.by_key, (B, H, Sk // 128, Sq // 64))):
        for t, shp in ((md.unmasked_kv_ids, shape), (md.unmasked_lens, shape[:3]), (md.masked_kv_ids, shape),
                       (md.masked_lens, shape[:3])):
            if tuple(t.shape) != shp or t.dtype != torch.int32 or t.device != q.device:
                raise ValueError(f"bwd_metadata: expected int32 {shp} on {q.device}, got {t.dtype} {tuple(t.shape)}")
            lists += [t.data_ptr(), S(t.stride())]
        _checked_metadata(md, 64 * shape[3], 64)
        pk = getattr(md, "packed_masks", None)
        if pk is not None and (tuple(pk.shape) != shape + (1024,) or pk.dtype != torch.uint8 or pk.device != q.device
                               or pk.stride()[2:] != (shape[3] * 1024, 1024, 1)):
            raise ValueError(f"bwd_metadata packed_masks: expected uint8 {shape + (1024,)} on {q.device} with "
                             f"contiguous tiles, got {pk.dtype} {tuple(pk.shape)} strides {pk.stride()}")
        packs += [pk.data_ptr(), S(pk.stride()[:2])] if pk is not None else [None, None]
    if mask is None and None in packs:
        raise ValueError("sparse_attention_backward without a mask needs packed_masks in both lists of bwd_metadata")
    mt = getattr(bwd_metadata, "transposed_mask", None)
    if mt is not None and (tuple(mt.shape) != (B, H, Sk, Sq) or mt.dtype != torch.bool or mt.device != q.device):
        raise ValueError(f"bwd_metadata.transposed_mask: expected bool {(B, H, Sk, Sq)} on {q.device}")
    with torch.cuda.device(q.device):
        ws_bytes = lib.sa_bwd_workspace_bytes(B, H, Sq)
        ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=q.device)
        rc = lib.sa_sparse_attention_bwd(
            qc.data_ptr(), S(qc.stride()), kc.data_ptr(), S(kc.stride()), vc.data_ptr(), S(vc.stride()),
            oc.data_ptr(), S(oc.stride()), doc.data_ptr(), S(doc.stride()), lse.data_ptr(), S(lse.stride()),
            dq.data_ptr(), S(dq.stride()), dk.data_ptr(), S(dk.stride()), dv.data_ptr(), S(dv.stride()),
            mask.data_ptr() if mask is not None else None, S(mask.stride()) if mask is not None else None,
            mt.data_ptr() if mt is not None else None, S(mt.stride()) if mt is not None else None,
            *packs, *lists, ws.data_ptr(), ws_bytes,
            B, H, Sq, Sk, Dk, _DTYPES[q.dtype], sm_scale, torch.cuda.current_stream(q.device).cuda_stream)
    _native.check(rc)
    if Dk != D:
        dq, dk, dv = (t[..., :D].contiguous() for t in (dq, dk, dv))
    return dq, dk, dv


class _SparseAttentionFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, mask, BLOCK_Q, BLOCK_K, mask_metadata, bwd_metadata):
        o, lse = sparse_attention(q, k, v, mask, BLOCK_Q, BLOCK_K, mask_metadata, return_lse=True)
        ctx.save_for_backward(q, k, v, o, lse, mask)
        ctx.bwd_metadata = bwd_metadata
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, mask = ctx.saved_tensors
        dq, dk, dv = sparse_attention_backward(do, q, k, v, o, lse, mask, ctx.bwd_metadata)
        return dq, dk, dv, None, None, None, None, None


def sparse_attention_trainable(q, k, v, mask, BLOCK_Q, BLOCK_K, mask_metadata: MaskMetadata | None = None,
                               bwd_metadata: BackwardMetadata | None = None) -> torch.Tensor:
    """:func:`sparse_attention` as a differentiable torch function (gradients for q, k, v through
    :func:`sparse_attention_backward`)."""
    return _SparseAttentionFunction.apply(q, k, v, mask, BLOCK_Q, BLOCK_K, mask_metadata, bwd_metadata)


def merge_attention_parts(o_parts: torch.Tensor, lse_parts: torch.Tensor, return_lse: bool = False):
    """Merge attention results computed over disjoint key ranges of the same queries.

    ``o_parts`` [n,B,H,Sq,D] (bf16/fp16) and ``lse_parts`` [n,B,H,Sq] (float32) as returned, per key range, by
    ``sparse_attention(..., return_lse=True)``: ``o = Σ_i exp(lse_i − lse) o_i`` with ``lse = logsumexp_i lse_i``.
    This is the exchange a key-axis sharding of the forward ends with (no counterpart in the reference).
    """
    if o_parts.dim() != 5 or lse_parts.shape != o_parts.shape[:4] or lse_parts.dtype != torch.float32:
        raise ValueError("o_parts must be [n,B,H,Sq,D] and lse_parts float32 [n,B,H,Sq]")
    if o_parts.dtype not in _DTYPES or not o_parts.is_cuda:
        raise TypeError("o_parts must be a bfloat16 or float16 tensor on a ROCm GPU")
    _same_device(o_parts, lse_parts=lse_parts)
    n, B, H, Sq, D = o_parts.shape
    if o_parts.stride(-1) != 1 or o_parts.data_ptr() % 16 or any(s % 8 for s in o_parts.stride()[:-1]):
        o_parts = o_parts.contiguous()
    o = torch.empty(B, H, Sq, D, dtype=o_parts.dtype, device=o_parts.device)
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device=o_parts.device) if return_lse else None
    S = _native.strides
    with torch.cuda.device(o_parts.device):
        rc = _native.load().sa_merge_attention_parts(
            o_parts.data_ptr(), S(o_parts.stride()), lse_parts.data_ptr(), S(lse_parts.stride()),
            o.data_ptr(), S(o.stride()), lse.data_ptr() if return_lse else None, S(lse.stride()) if return_lse else None,
            n, B, H, Sq, D, _DTYPES[o_parts.dtype], torch.cuda.current_stream(o_parts.device).cuda_stream)
    _native.check(rc)
    return (o, lse) if return_lse else o


def sparse_attention_kv_split(q, k, v, mask, BLOCK_Q, BLOCK_K, num_splits: int, return_lse: bool = False):
    """:func:`sparse_attention` with the key axis cut into ``num_splits`` equal ranges, each run as a forward of
    its own (own tile lists) and merged by :func:`merge_attention_parts`: what one device per range would do.
    Useful on one device when there are too few Q tiles to fill it (a few hundred query rows against long keys)."""
    B, H, Sq, D = q.shape
    Sk = k.shape[-2]
    if Sk % (num_splits * BLOCK_K):
        raise ValueError(f"Sk ({Sk}) must be a multiple of num_splits * BLOCK_K ({num_splits} * {BLOCK_K})")
    mask = mask.expand(B, H, Sq, Sk)
    step = Sk // num_splits
    o_parts = torch.empty(num_splits, B, H, Sq, D, dtype=q.dtype, device=q.device)
    lse_parts = torch.empty(num_splits, B, H, Sq, dtype=torch.float32, device=q.device)
    for i in range(num_splits):
        sl = slice(i * step, (i + 1) * step)
        o_parts[i], lse_parts[i] = sparse_attention(q, k[:, :, sl], v[:, :, sl], mask[..., sl], BLOCK_Q, BLOCK_K,
                                                    return_lse=True)
    return merge_attention_parts(o_parts, lse_parts, return_lse)
