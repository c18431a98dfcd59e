"""Mask preprocessing: which (Q tile, KV tile) pairs are full, partial or empty.

Mirrors the interface of the reference's ``sparseattention/mask_utils.py``:
``MaskMetadata`` (:6-11), ``compute_mask_slow`` (:14-44), ``compute_mask_kernel`` (:85-107).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

import torch

from . import _native


@dataclass
class MaskMetadata:
    """Per-Q-tile index lists.  Field names and order follow mask_utils.py:6-11.

    ``unmasked_kv_ids`` int32 [B,H,Sq/BQ,Sk/BK]: ascending indices of KV tiles whose mask tile is all True;
    ``unmasked_lens``  int32 [B,H,Sq/BQ]: how many leading slots of it are valid;
    ``masked_kv_ids`` / ``masked_lens``: the same for tiles with some but not all entries True.
    Slots past the count hold unspecified values.

    ``packed_masks`` is an addition to the reference's four fields (optional, last, default None, so code
    that builds the dataclass positionally keeps working): uint8 [B,H,Sq/BQ,Sk/BK,BQ*BK/8], the mask entries of
    the PARTIAL tiles at one bit each.  ``packed_masks[b,h,qt,slot]`` belongs to KV tile
    ``masked_kv_ids[b,h,qt,slot]``: rows first, entry (r, c) in bit ``c & 7`` of byte ``(r*BK + c) >> 3``.
    When present, :func:`sparse_attention` reads these bits and never touches the bool mask.

    ``schedule`` / ``schedule_mode`` are the second addition (optional, default None): int32
    [workgroups, rounds + 1, 4], which Q tiles each workgroup of the forward processes, in order (entry 0 of a
    row: the count; then ``((b << 16) | h, qt, unmasked_len, masked_len)`` per tile), made by
    ``compute_mask_kernel(..., schedule="pairs" | "persistent")``.  It depends on the counts, on B and H and, for
    "persistent", on the device; without it the forward launches one workgroup per Q tile.

    ``list_stats`` is the third addition (optional, default None): ``(mean, longest)`` number of listed KV tiles per
    Q tile, FULL and PARTIAL together, as Python numbers.  Reading them back synchronises the host with the device
    once, so they are filled only on request (``compute_mask_kernel(..., list_stats=True)`` or
    :func:`with_list_stats`); with them :func:`sparse_attention` picks the kernel form that suits the lists.
    ``list_rotation`` comes from the same read-back: a group size G > 0 when the FULL lists of neighbouring Q tiles
    slide along the keys (a sliding window), for which the forward then walks the FULL entries of Q tile qt from a
    start that depends on qt, so that neighbours read the same K/V rows at the same time (they are fetched from HBM
    once instead of once per Q tile); 0 (the default) walks every list from its front.

    Two book-keeping fields follow, neither compared nor shown: ``_validated_for`` = :func:`validation_key` of the
    ``(Sk, BLOCK_K)`` these lists have been checked against (set by the functions of this module, whose lists fit by
    construction, and by ``sparse_attention`` after it has checked a caller-built object; the key carries the address
    and the in-place version counter of the four list tensors, so lists edited in place or replaced are checked
    again), and ``_retiled`` = the lists of the same
    mask at tile sizes the kernels have, kept by ``sparse_attention`` when it was asked for sizes they do not have.
    """

    unmasked_kv_ids: torch.Tensor
    unmasked_lens: torch.Tensor
    masked_kv_ids: torch.Tensor
    masked_lens: torch.Tensor
    packed_masks: Optional[torch.Tensor] = None
    schedule: Optional[torch.Tensor] = None
    schedule_mode: int = 0
    list_stats: Optional[Tuple[float, int]] = None
    list_rotation: int = 0
    _validated_for: Optional[tuple] = field(default=None, repr=False, compare=False)
    _retiled: Optional[tuple] = field(default=None, repr=False, compare=False)


def with_list_stats(md: "MaskMetadata") -> "MaskMetadata":
    """Fills ``md.list_stats`` = (mean, longest) listed KV tiles per Q tile from the two count tensors and
    ``md.list_rotation`` (16 when the FULL lists slide along the keys from one Q tile to the next, as under a sliding
    window; else 0) with one host synchronisation (the distinct planes of broadcast lists are read once); returns
    ``md``."""
    fl, pl, fid = md.unmasked_lens, md.masked_lens, md.unmasked_kv_ids
    idx = tuple(slice(0, 1) if fl.stride(d) == 0 and pl.stride(d) == 0 and fid.stride(d) == 0 else slice(None)
                for d in range(2))
    fl_, pl_ = fl[idx].to(torch.int64), pl[idx].to(torch.int64)
    total = (fl_ + pl_).flatten()
    if total.numel() == 0:
        md.list_stats, md.list_rotation = (0.0, 0), 0
        return md
    # neighbouring Q tiles that both have FULL tiles, and those of them whose first FULL tile lies further on
    first = fid[idx][..., 0]
    both = (fl_[..., 1:] > 0) & (fl_[..., :-1] > 0)
    slides = both & (first[..., 1:] > first[..., :-1])
    got = torch.stack((total.sum(), total.max(), both.sum(), slides.sum(), fl_.sum())).tolist()
    md.list_stats = (got[0] / total.numel(), int(got[1]))
    # a sliding band: most neighbours slide, and the FULL lists are long enough for a rotation to matter
    md.list_rotation = 16 if got[2] > 0 and got[3] > 0.5 * got[2] and got[4] / total.numel() >= 8 else 0
    return md


def validation_key(md, Sk: int, BLOCK_K: int) -> tuple:
    """What "these lists were checked against Sk and BLOCK_K" is remembered under: the sizes plus, per list tensor,
    its address and torch's in-place version counter (shared by all views of a storage), so that an in-place edit
    of the lists or other tensors under the same object make the remembered check void."""
    return (int(Sk), int(BLOCK_K)) + tuple(
        (t.data_ptr(), t._version) for t in (md.unmasked_kv_ids, md.unmasked_lens, md.masked_kv_ids, md.masked_lens))


def _check_mask(mask: torch.Tensor, BLOCK_Q: int, BLOCK_K: int):
    if mask.dim() != 4:
        raise ValueError(f"mask must be [B,H,Sq,Sk] (got {tuple(mask.shape)}); use mask.expand(B,H,Sq,Sk)")
    B, H, Sq, Sk = mask.shape
    # the reference asserts these (mask_utils.py:18-20, :89-90)
    assert mask.dtype == torch.bool, "mask must be a torch.bool tensor"
    assert Sq % BLOCK_Q == 0, "Sq must be a multiple of BLOCK_Q"
    assert Sk % BLOCK_K == 0, "Sk must be a multiple of BLOCK_K"
    return B, H, Sq, Sk


def compute_mask_slow(mask: torch.Tensor, BLOCK_Q: int, BLOCK_K: int) -> MaskMetadata:
    """Specification of the classification, in plain torch on the mask's own device.

    Same results as the reference's loop (mask_utils.py:27-42) without the per-tile Python
    iterations: a tile whose popcount equals BLOCK_Q*BLOCK_K is listed as unmasked, one with a
    positive popcount as masked, indices ascending.  Slots past the count are filled with -1.
    """
    B, H, Sq, Sk = _check_mask(mask, BLOCK_Q, BLOCK_K)
    nQ, nK = Sq // BLOCK_Q, Sk // BLOCK_K
    # broadcast dimensions hold one distinct plane: count it once, expand the result
    uniq = mask[:1] if mask.stride(0) == 0 else mask
    uniq = uniq[:, :1] if mask.stride(1) == 0 else uniq
    counts = uniq.reshape(uniq.shape[0], uniq.shape[1], nQ, BLOCK_Q, nK, BLOCK_K).sum(dim=(3, 5), dtype=torch.int64)
    full = counts == BLOCK_Q * BLOCK_K
    part = (counts > 0) & ~full

    def compact(flags):
        lens = flags.sum(-1).to(torch.int32)
        order = torch.sort((~flags).to(torch.uint8), dim=-1, stable=True).indices.to(torch.int32)
        pos = torch.arange(nK, device=mask.device, dtype=torch.int32)
        ids = torch.where(pos < lens[..., None], order, torch.full_like(order, -1))
        return ids.expand(B, H, nQ, nK), lens.expand(B, H, nQ)

    fid, fl = compact(full)
    pid, pl = compact(part)
    return MaskMetadata(fid, fl, pid, pl)


def _make_schedule(lib, fl, pl, B, H, Sq, Sk, BLOCK_Q, BLOCK_K, schedule, dev):
    """(schedule tensor, mode) for ``compute_mask_kernel(..., schedule=...)``; (None, 0) without one."""
    if not schedule:
        return None, 0
    modes = {"persistent": _native.SA_SCHEDULE_PERSISTENT, "pairs": _native.SA_SCHEDULE_PAIRS,
             True: _native.SA_SCHEDULE_PAIRS}
    if schedule not in modes:
        raise ValueError(f"schedule must be 'pairs', 'persistent' or None (got {schedule!r})")
    mode = modes[schedule]
    nQ = Sq // BLOCK_Q
    nbytes = int(lib.sa_fwd_schedule_bytes(B, H, Sq, Sk, BLOCK_Q, BLOCK_K, mode))
    if nbytes == 0:
        raise ValueError(f"no scheduled forward for BLOCK_Q={BLOCK_Q}, BLOCK_K={BLOCK_K}, Sk={Sk}")
    sched = torch.empty(nbytes // 4, dtype=torch.int32, device=dev)
    rc = lib.sa_fwd_schedule(fl.data_ptr(), _native.strides(fl.stride()), pl.data_ptr(),
                             _native.strides(pl.stride()), B, H, Sq, Sk, BLOCK_Q, BLOCK_K, mode,
                             sched.data_ptr(), nbytes, torch.cuda.current_stream(dev).cuda_stream)
    _native.check(rc)
    if mode == _native.SA_SCHEDULE_PAIRS:
        sched = sched.view(-1, 3, 4)
    else:
        G = min(2 * torch.cuda.get_device_properties(dev).multi_processor_count, 512) & ~7
        sched = sched.view(G, nbytes // (16 * G), 4)
    return sched, mode


def compute_mask_kernel(mask: torch.Tensor, BLOCK_Q: int, BLOCK_K: int, pack_partial: Optional[bool] = None,
                        schedule=None, list_stats: bool = False) -> MaskMetadata:
    """Classify the mask's tiles on the GPU (replaces mask_utils.py:85-107).

    Memory beyond the reference's four tensors: with ``pack_partial`` (the default when BLOCK_K is a multiple of 8)
    ``Sq*Sk/8`` bytes per DISTINCT mask plane for ``packed_masks`` (128 MiB for a [32768,32768] mask; B*H times that
    for a mask that differs per batch element and head).  ``pack_partial=False`` allocates only the four tensors.

    ``mask``: bool [B,H,Sq,Sk] on a ROCm device, any strides.  Dimensions that are broadcast in
    ``mask`` (stride 0, e.g. from ``mask.expand(B,H,Sq,Sk)``) are classified once and the returned
    tensors are broadcast views over them, so every ``[b,h]`` plane reads the same values the
    reference would have written there.

    ``pack_partial``: also fill ``MaskMetadata.packed_masks`` (Sq*Sk/8 bytes per distinct mask plane).
    Default: whenever BLOCK_K is a multiple of 8; ``False`` gives exactly the reference's four tensors.
    ``schedule``: ``"pairs"`` or ``"persistent"`` also fills ``MaskMetadata.schedule`` (needs BLOCK_Q 32/64/128,
    BLOCK_K a power of two >= 16 and at most 1024 KV tiles per row); ``None``/``False`` leaves it out.
    "pairs": one workgroup per two Q tiles, tile r from the top with tile r from the bottom of a pair of planes.
    "persistent": as many workgroups as the device holds, each with a list of Q tiles ranked by cost; measured
    on MI355X it wins when the lists are short (a few hundred keys per Q tile) and loses a few percent to the
    hardware dispatcher when they are long, because a static hand-out cannot follow the uneven pace of the
    workgroups that share a compute unit.
    ``list_stats``: also read back how many KV tiles the lists hold per Q tile (mean and longest:
    ``MaskMetadata.list_stats``), which lets :func:`sparse_attention` choose the kernel form for short lists.  This is
    the one option that synchronises the host with the device; preprocessing is paid once per mask (README.md:46).
    """
    B, H, Sq, Sk = _check_mask(mask, BLOCK_Q, BLOCK_K)
    if not mask.is_cuda:
        raise RuntimeError("compute_mask_kernel needs the mask on a ROCm GPU; compute_mask_slow runs anywhere")
    lib = _native.load()
    nQ, nK = Sq // BLOCK_Q, Sk // BLOCK_K
    uB = 1 if (mask.stride(0) == 0 or B == 1) else B
    uH = 1 if (mask.stride(1) == 0 or H == 1) else H
    dev = mask.device
    with torch.cuda.device(dev):
        fid = torch.empty(uB, uH, nQ, nK, dtype=torch.int32, device=dev)
        pid = torch.empty(uB, uH, nQ, nK, dtype=torch.int32, device=dev)
        fl = torch.empty(uB, uH, nQ, dtype=torch.int32, device=dev)
        pl = torch.empty(uB, uH, nQ, dtype=torch.int32, device=dev)
        fid, pid = fid.expand(B, H, nQ, nK), pid.expand(B, H, nQ, nK)
        fl, pl = fl.expand(B, H, nQ), pl.expand(B, H, nQ)
        ms = _native.strides(mask.stride())
        need = lib.sa_mask_classify_workspace_bytes(ms, B, H, Sq, Sk, BLOCK_Q, BLOCK_K)
        workspace = torch.empty(max(int(need), 1), dtype=torch.uint8, device=dev)
        rc = lib.sa_mask_classify(
            mask.data_ptr(), ms, B, H, Sq, Sk, BLOCK_Q, BLOCK_K,
            fid.data_ptr(), _native.strides(fid.stride()), fl.data_ptr(), _native.strides(fl.stride()),
            pid.data_ptr(), _native.strides(pid.stride()), pl.data_ptr(), _native.strides(pl.stride()),
            workspace.data_ptr(), workspace.numel(), torch.cuda.current_stream(dev).cuda_stream,
        )
        _native.check(rc)
        # the kernels run on the current stream; the caching allocator may hand this block out again
        # only to work queued after them on the same stream, so dropping the reference here is safe
        del workspace
        packed = None
        if pack_partial is None:
            pack_partial = BLOCK_K % 8 == 0
        if pack_partial:
            if BLOCK_K % 8:
                raise ValueError(f"pack_partial needs BLOCK_K to be a multiple of 8 (got {BLOCK_K})")
            packed = torch.empty(uB, uH, nQ, nK, BLOCK_Q * BLOCK_K // 8, dtype=torch.uint8, device=dev)
            rc = lib.sa_mask_pack_partial(
                mask.data_ptr(), ms, B, H, Sq, Sk, BLOCK_Q, BLOCK_K,
                pid.data_ptr(), _native.strides(pid.stride()), pl.data_ptr(), _native.strides(pl.stride()),
                packed.data_ptr(), _native.strides(packed.stride()[:2]),
                torch.cuda.current_stream(dev).cuda_stream,
            )
            _native.check(rc)
            packed = packed.expand(B, H, nQ, nK, BLOCK_Q * BLOCK_K // 8)
        sched, mode = _make_schedule(lib, fl, pl, B, H, Sq, Sk, BLOCK_Q, BLOCK_K, schedule, dev)
    md = MaskMetadata(fid, fl, pid, pl, packed, sched, mode)
    md._validated_for = validation_key(md, Sk, BLOCK_K)  # lists made by the kernels above fit by construction
    return with_list_stats(md) if list_stats else md


# Tile sizes tried by select_block_sizes, and what one executed mask entry costs at each of them relative to tiles of
# 128 x 64 (measured on MI355X, D = 128 bf16, with bench.py's tile_selection leg: the same mask classified and run at
# every candidate; causal S=4096, random blocks p=0.75, documents S=16384 and the composed mask S=32768 agree within
# 3 %).  BLOCK_Q sets most of it (rows per workgroup: 64-row tiles fetch K/V twice as often per entry, 256-row tiles
# run the two-phase kernel); BLOCK_K only through the scalar bookkeeping per list entry (the forward consumes keys in
# chunks of 64 whatever the tile width).
DEFAULT_TILE_CANDIDATES = ((128, 32), (128, 64), (128, 128), (64, 32), (64, 64), (256, 32), (256, 64))
RELATIVE_COST_PER_ENTRY = {32: 2.0, 64: 1.45, 128: 1.0, 256: 1.1}
RELATIVE_COST_BLOCK_K = {16: 1.08, 32: 1.03, 64: 1.0}  # wider tiles: 1.005


def entry_cost(BLOCK_Q: int, BLOCK_K: int) -> float:
    """Relative cost of one executed mask entry at these tile sizes (see the tables above)."""
    return RELATIVE_COST_PER_ENTRY.get(BLOCK_Q, 1.0) * RELATIVE_COST_BLOCK_K.get(BLOCK_K, 1.005)


def select_block_sizes(mask: torch.Tensor, candidates=DEFAULT_TILE_CANDIDATES, partial_cost: float = 1.25):
    """Choose the tile sizes that leave the least attention work for this mask.

    The reference lists this as future work ("changing blocksizes ... to maximise the number of totally
    masked-out blocks", README.md:64).  Every candidate (BLOCK_Q, BLOCK_K) that divides the mask is
    classified (on the GPU when the mask lives there, else with compute_mask_slow) and priced as

        (full tiles + partial_cost * partial tiles) * BLOCK_Q * BLOCK_K * entry_cost(BLOCK_Q, BLOCK_K)

    summed over the distinct mask planes; partial tiles cost more because their mask is read and applied.
    Returns ``(BLOCK_Q, BLOCK_K, metadata, report)``: the cheapest candidate, its MaskMetadata (ready to pass
    to sparse_attention) and the list of ``(BLOCK_Q, BLOCK_K, full_tiles, partial_tiles, cost)`` rows.
    Reads the counts back to the host, so it synchronises with the device: call it once per mask.
    """
    if mask.dim() != 4:
        raise ValueError(f"mask must be [B,H,Sq,Sk] (got {tuple(mask.shape)})")
    B, H, Sq, Sk = mask.shape
    classify = compute_mask_kernel if mask.is_cuda else compute_mask_slow
    best, report = None, []
    for BQ, BK in candidates:
        if Sq % BQ or Sk % BK:
            continue
        md = classify(mask, BQ, BK)
        # broadcast planes hold the same counts: the sum over the expanded view weights every plane equally
        full = int(md.unmasked_lens.sum())
        part = int(md.masked_lens.sum())
        cost = (full + partial_cost * part) * BQ * BK * entry_cost(BQ, BK)
        report.append((BQ, BK, full, part, cost))
        if best is None or cost < best[0]:
            best = (cost, BQ, BK, md)
    if best is None:
        raise ValueError(f"no candidate tile size divides a mask of shape {tuple(mask.shape)}")
    return best[1], best[2], best[3], report


@dataclass
class Tiling:
    """A choice of tile sizes and of the tile grid's origin for one mask (:func:`select_tiling`).

    The grid of BLOCK_Q x BLOCK_K tiles starts ``q_offset`` rows above and ``k_offset`` columns left of the mask's
    first entry: the mask is taken as padded with that many all-False rows / columns in front (and at the end up to
    whole tiles).  ``metadata`` is the MaskMetadata of that padded mask, ``padded_mask`` the padded mask itself
    (the caller's mask when both offsets are 0 and no rounding up was needed)."""

    BLOCK_Q: int
    BLOCK_K: int
    q_offset: int
    k_offset: int
    metadata: MaskMetadata
    padded_mask: torch.Tensor
    report: list


def select_tiling(mask: torch.Tensor, candidates=DEFAULT_TILE_CANDIDATES, offsets: Sequence[Tuple[int, int]] = ((0, 0),),
                  partial_cost: float = 1.25) -> Tiling:
    """:func:`select_block_sizes` over tile sizes AND grid origins ("changing blocksizes / offsets to maximise the
    number of totally masked-out blocks", README.md:64): every candidate (BLOCK_Q, BLOCK_K) is tried with every
    ``(q_offset, k_offset)`` of ``offsets`` (0 <= offset < BLOCK; pairs that do not fit a candidate are skipped) on the
    mask padded accordingly, priced like select_block_sizes does.  A mask whose structure has a period of the tile
    size but starts off the grid (documents or windows that begin at row 32, say) loses its PARTIAL tiles at the
    right origin.  Run the result with :func:`sparseattention_amd.sparse_attention_tiled`.  Reads counts back to the
    host and copies the mask once per offset: call it once per mask."""
    if mask.dim() != 4:
        raise ValueError(f"mask must be [B,H,Sq,Sk] (got {tuple(mask.shape)})")
    B, H, Sq, Sk = mask.shape
    classify = compute_mask_kernel if mask.is_cuda else compute_mask_slow
    distinct = mask[: 1 if mask.stride(0) == 0 else B, : 1 if mask.stride(1) == 0 else H]
    best, report = None, []
    for BQ, BK in candidates:
        for qo, ko in offsets:
            if not (0 <= qo < BQ and 0 <= ko < BK):
                continue
            pq, pk = -(Sq + qo) % BQ, -(Sk + ko) % BK
            if (qo, ko, pq, pk) == (0, 0, 0, 0):
                padded = mask
            else:
                padded = torch.nn.functional.pad(distinct, (ko, pk, qo, pq), value=False).expand(B, H, Sq + qo + pq, Sk + ko + pk)
            md = classify(padded, BQ, BK)
            full, part = int(md.unmasked_lens.sum()), int(md.masked_lens.sum())
            cost = (full + partial_cost * part) * BQ * BK * entry_cost(BQ, BK)
            report.append((BQ, BK, qo, ko, full, part, cost))
            if best is None or cost < best[0]:
                best = (cost, BQ, BK, qo, ko, md, padded)
    if best is None:
        raise ValueError("no candidate tile size / offset pair fits")
    return Tiling(best[1], best[2], best[3], best[4], best[5], best[6], report)


# ---- masks given by a formula -----------------------------------------------------------------------------------
_TERM_BACK, _TERM_AHEAD, _TERM_Q_RANGE, _TERM_K_RANGE, _TERM_SAME_DOC = 1, 2, 4, 8, 16
MAX_MASK_TERMS = 8


@dataclass(frozen=True)
class MaskTerm:
    """One term of a mask given by a formula: the AND of the conditions that are set.

    ``back``: ``(q + offset) - k < back`` (how far behind the diagonal a key may lie); ``ahead``:
    ``k - (q + offset) < ahead`` (1: causal); ``q_range`` / ``k_range``: half-open index ranges; ``same_doc``:
    ``doc_q[b, q] == doc_k[b, k]``.  A mask is the OR of up to ``MAX_MASK_TERMS`` terms.  The reference takes tensor
    masks only and lists "algebraically defined masks ... to avoid materialisation + memory costs" as what could come
    next (README.md:63).
    """

    back: Optional[int] = None
    ahead: Optional[int] = None
    offset: int = 0
    q_range: Optional[Tuple[int, int]] = None
    k_range: Optional[Tuple[int, int]] = None
    same_doc: bool = False

    def encode(self):
        """The eight int32 of the C ABI: flags, offset, back, ahead, q_lo, q_hi, k_lo, k_hi."""
        flags = ((_TERM_BACK if self.back is not None else 0) | (_TERM_AHEAD if self.ahead is not None else 0)
                 | (_TERM_Q_RANGE if self.q_range is not None else 0) | (_TERM_K_RANGE if self.k_range is not None else 0)
                 | (_TERM_SAME_DOC if self.same_doc else 0))
        q_lo, q_hi = self.q_range if self.q_range is not None else (0, 0)
        k_lo, k_hi = self.k_range if self.k_range is not None else (0, 0)
        return [flags, int(self.offset), int(self.back or 0), int(self.ahead or 0), int(q_lo), int(q_hi), int(k_lo), int(k_hi)]

    def transposed(self) -> "MaskTerm":
        """The same condition with keys as rows: term(q, k) == term.transposed()(k, q)."""
        return MaskTerm(back=self.ahead, ahead=self.back, offset=-self.offset, q_range=self.k_range,
                        k_range=self.q_range, same_doc=self.same_doc)


def causal_term(window: Optional[int] = None, offset: int = 0, same_doc: bool = False) -> MaskTerm:
    """``k <= q + offset``, optionally only the last ``window`` such keys, optionally within one document."""
    return MaskTerm(back=window, ahead=1, offset=offset, same_doc=same_doc)


def block_term(q_range: Optional[Tuple[int, int]] = None, k_range: Optional[Tuple[int, int]] = None) -> MaskTerm:
    """Every (q, k) with q and k in the given half-open ranges (None: all), e.g. a bidirectional prefix or sink keys."""
    return MaskTerm(q_range=q_range, k_range=k_range)


def _check_docs(doc, B, S, name):
    if doc is None:
        return None
    if doc.dim() == 1:
        doc = doc[None]
    if doc.dim() != 2 or doc.shape[-1] != S or doc.shape[0] not in (1, B) or doc.dtype != torch.int32:
        raise ValueError(f"{name}: expected int32 [{B},{S}] or [{S}], got {doc.dtype} {tuple(doc.shape)}")
    return doc.expand(B, S)


def materialize_mask_terms(terms: Sequence[MaskTerm], B: int, Sq: int, Sk: int, doc_q=None, doc_k=None, device=None):
    """The bool mask [B,1,Sq,Sk] (or [1,1,Sq,Sk] without documents) that the terms describe, in plain torch: for
    checks, for the decode path (which reads a tensor) and for :func:`torch.nn.functional.scaled_dot_product_attention`."""
    doc_q, doc_k = _check_docs(doc_q, B, Sq, "doc_q"), _check_docs(doc_k, B, Sk, "doc_k")
    if device is None:
        device = doc_q.device if doc_q is not None else "cpu"
    q = torch.arange(Sq, device=device, dtype=torch.int64)[:, None]
    k = torch.arange(Sk, device=device, dtype=torch.int64)[None, :]
    out = torch.zeros(B if doc_q is not None else 1, 1, Sq, Sk, dtype=torch.bool, device=device)
    for t in terms:
        ok = torch.ones(1, 1, Sq, Sk, dtype=torch.bool, device=device)
        d = q + t.offset - k
        if t.back is not None:
            ok = ok & (d < t.back)
        if t.ahead is not None:
            ok = ok & (-d < t.ahead)
        if t.q_range is not None:
            ok = ok & (q >= t.q_range[0]) & (q < t.q_range[1])
        if t.k_range is not None:
            ok = ok & (k >= t.k_range[0]) & (k < t.k_range[1])
        if t.same_doc:
            if doc_q is None or doc_k is None:
                raise ValueError("a term with same_doc needs doc_q and doc_k")
            ok = ok & (doc_q[:, None, :, None] == doc_k[:, None, None, :])
        out = out | ok
    return out


def compute_mask_terms(terms: Sequence[MaskTerm], B: int, H: int, Sq: int, Sk: int, BLOCK_Q: int, BLOCK_K: int,
                       doc_q: Optional[torch.Tensor] = None, doc_k: Optional[torch.Tensor] = None, device=None,
                       pack_partial: bool = True, schedule=None) -> MaskMetadata:
    """:func:`compute_mask_kernel` for a mask given by terms: the same lists (and packed PARTIAL tiles, schedule) as
    for ``materialize_mask_terms(...)``, computed on the GPU from the formula without the Sq x Sk tensor.

    With ``pack_partial`` the result carries everything the forward needs: ``sparse_attention(q, k, v, None, BLOCK_Q,
    BLOCK_K, mask_metadata=md)``.  ``doc_q`` / ``doc_k``: int32 document numbers [B,Sq] / [B,Sk] (or [Sq] / [Sk]) on
    the GPU for terms with ``same_doc``.  ``device``: where to compute when there are no documents.
    """
    terms = list(terms)
    if not 1 <= len(terms) <= MAX_MASK_TERMS:
        raise ValueError(f"1..{MAX_MASK_TERMS} terms (got {len(terms)})")
    assert Sq % BLOCK_Q == 0, "Sq must be a multiple of BLOCK_Q"
    assert Sk % BLOCK_K == 0, "Sk must be a multiple of BLOCK_K"
    doc_q, doc_k = _check_docs(doc_q, B, Sq, "doc_q"), _check_docs(doc_k, B, Sk, "doc_k")
    if any(t.same_doc for t in terms) and (doc_q is None or doc_k is None):
        raise ValueError("a term with same_doc needs doc_q and doc_k")
    dev = torch.device(device) if device is not None else (doc_q.device if doc_q is not None else torch.device("cuda"))
    if dev.type != "cuda" or any(d is not None and d.device != dev for d in (doc_q, doc_k)):
        raise RuntimeError("compute_mask_terms runs on a ROCm GPU (documents on the same device); "
                           "materialize_mask_terms + compute_mask_slow run anywhere")
    lib = _native.load()
    nQ, nK = Sq // BLOCK_Q, Sk // BLOCK_K
    per_batch = B > 1 and any(d is not None and d.stride(0) != 0 for d in (doc_q, doc_k))
    uB = B if per_batch else 1
    flat = [w for t in terms for w in t.encode()]
    c_terms = (ctypes.c_int32 * len(flat))(*flat)
    S = _native.strides
    with torch.cuda.device(dev):
        fid = torch.empty(uB, 1, nQ, nK, dtype=torch.int32, device=dev).expand(B, H, nQ, nK)
        pid = torch.empty(uB, 1, nQ, nK, dtype=torch.int32, device=dev).expand(B, H, nQ, nK)
        fl = torch.empty(uB, 1, nQ, dtype=torch.int32, device=dev).expand(B, H, nQ)
        pl = torch.empty(uB, 1, nQ, dtype=torch.int32, device=dev).expand(B, H, nQ)
        packed = None
        if pack_partial:
            packed = torch.empty(uB, 1, nQ, nK, BLOCK_Q * BLOCK_K // 8, dtype=torch.uint8, device=dev)
            packed = packed.expand(B, H, nQ, nK, BLOCK_Q * BLOCK_K // 8)
        need = int(lib.sa_mask_terms_workspace_bytes(uB, Sq, Sk, BLOCK_Q, BLOCK_K))
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        rc = lib.sa_mask_classify_terms(
            c_terms, len(terms),
            doc_q.data_ptr() if doc_q is not None else None, S(doc_q.stride()) if doc_q is not None else None,
            doc_k.data_ptr() if doc_k is not None else None, S(doc_k.stride()) if doc_k is not None else None,
            B, H, Sq, Sk, BLOCK_Q, BLOCK_K,
            fid.data_ptr(), S(fid.stride()), fl.data_ptr(), S(fl.stride()),
            pid.data_ptr(), S(pid.stride()), pl.data_ptr(), S(pl.stride()),
            packed.data_ptr() if packed is not None else None, S(packed.stride()[:2]) if packed is not None else None,
            workspace.data_ptr(), workspace.numel(), torch.cuda.current_stream(dev).cuda_stream)
        _native.check(rc)
        del workspace
        sched, mode = _make_schedule(lib, fl, pl, B, H, Sq, Sk, BLOCK_Q, BLOCK_K, schedule, dev)
    md = MaskMetadata(fid, fl, pid, pl, packed, sched, mode)
    md._validated_for = validation_key(md, Sk, BLOCK_K)  # lists made by the kernels above fit by construction
    return md
