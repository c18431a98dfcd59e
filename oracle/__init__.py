"""CPU oracle for the block-sparse attention forward path.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this package.
The product (``sparseattention_amd``) never does: it fails loudly when its HIP library is
missing instead of falling back to anything in here.

Two restatements of the reference algorithm live here:

* ``sparse_oracle.c`` (built into ``liboracle.so`` by ``oracle/Makefile``), wrapped by
  :func:`classify`, :func:`forward` and :func:`pack_partial`;
* the numpy functions :func:`classify_numpy` and :func:`forward_dense_fp64`, written a
  different way (per-tile popcount by reshape; dense fp64 softmax) so that the two can be
  checked against each other and against closed forms.

Reference lines followed: ``sparseattention/mask_utils.py:14-44`` (classification) and
``sparseattention/sparse_attn_kernel.py:28-63, 103-146, 152`` (two-pass forward).
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``sparse_oracle.c`` with gcc (the recipe is ``oracle/Makefile``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    i32p = ctypes.POINTER(ctypes.c_int32)
    i64p = ctypes.POINTER(ctypes.c_int64)
    f32p = ctypes.POINTER(ctypes.c_float)
    u8p = ctypes.POINTER(ctypes.c_uint8)
    lib.oracle_classify.restype = ctypes.c_int
    lib.oracle_classify.argtypes = [u8p, i64p] + [ctypes.c_int] * 6 + [i32p] * 4
    lib.oracle_forward.restype = ctypes.c_int
    lib.oracle_forward.argtypes = (
        [f32p, f32p, f32p, f32p, u8p, i64p, i32p, i32p, i32p, i32p] + [ctypes.c_int] * 7 + [ctypes.c_float, ctypes.c_int]
    )
    lib.oracle_pack_partial.restype = ctypes.c_int
    lib.oracle_pack_partial.argtypes = [u8p, i64p] + [ctypes.c_int] * 6 + [i32p, i32p, u8p]
    lib.oracle_max_threads.restype = ctypes.c_int
    for fn in (lib.oracle_round_bf16, lib.oracle_round_fp16):
        fn.restype = ctypes.c_float
        fn.argtypes = [ctypes.c_float]
    _lib = lib
    return lib


def round_bf16(x: float) -> float:
    """fp32 -> nearest bf16 -> fp32, as the C oracle rounds P."""
    return float(_load().oracle_round_bf16(x))


def round_fp16(x: float) -> float:
    """fp32 -> nearest fp16 -> fp32, as the C oracle rounds P."""
    return float(_load().oracle_round_fp16(x))


def max_threads() -> int:
    """Threads the C oracle's OpenMP loops will use."""
    return int(_load().oracle_max_threads())


@dataclass
class OracleMetadata:
    """Same four fields, same order, as ``MaskMetadata`` (mask_utils.py:6-11), as numpy int32 arrays."""

    unmasked_kv_ids: np.ndarray
    unmasked_lens: np.ndarray
    masked_kv_ids: np.ndarray
    masked_lens: np.ndarray


def _ptr(a: np.ndarray, ty):
    return a.ctypes.data_as(ctypes.POINTER(ty))


def _mask_view(mask: np.ndarray):
    """Return (uint8 view, strides-in-bytes as int64[4]) for a 4-d bool/uint8 array of any strides."""
    if mask.ndim != 4:
        raise ValueError("mask must be 4-d [B,H,Sq,Sk] (broadcast views are fine)")
    if mask.dtype == np.bool_:
        mask = mask.view(np.uint8)
    if mask.dtype != np.uint8:
        raise ValueError("mask must be bool")
    strides = np.array(mask.strides, dtype=np.int64)
    return mask, strides


def classify(mask: np.ndarray, BQ: int, BK: int) -> OracleMetadata:
    """C restatement of ``compute_mask_slow`` (mask_utils.py:14-44).  Tail slots are -1."""
    lib = _load()
    B, H, Sq, Sk = mask.shape
    if Sq % BQ or Sk % BK:
        raise ValueError("Sq % BLOCK_Q and Sk % BLOCK_K must be 0")
    m8, strides = _mask_view(mask)
    nQ, nK = Sq // BQ, Sk // BK
    fid = np.empty((B, H, nQ, nK), np.int32)
    pid = np.empty((B, H, nQ, nK), np.int32)
    fl = np.empty((B, H, nQ), np.int32)
    pl = np.empty((B, H, nQ), np.int32)
    rc = lib.oracle_classify(
        _ptr(m8, ctypes.c_uint8), _ptr(strides, ctypes.c_int64), B, H, Sq, Sk, BQ, BK,
        _ptr(fid, ctypes.c_int32), _ptr(fl, ctypes.c_int32), _ptr(pid, ctypes.c_int32), _ptr(pl, ctypes.c_int32),
    )
    if rc != 0:
        raise RuntimeError(f"oracle_classify failed: {rc}")
    return OracleMetadata(fid, fl, pid, pl)


def classify_numpy(mask: np.ndarray, BQ: int, BK: int) -> OracleMetadata:
    """Vectorised popcount classification; independent of the C loop.  Tail slots are -1."""
    B, H, Sq, Sk = mask.shape
    nQ, nK = Sq // BQ, Sk // BK
    m = np.ascontiguousarray(np.broadcast_to(mask, (B, H, Sq, Sk))).astype(bool)
    counts = m.reshape(B, H, nQ, BQ, nK, BK).sum(axis=(3, 5), dtype=np.int64)
    full = counts == BQ * BK
    part = (counts > 0) & ~full

    def compact(flags):
        lens = flags.sum(-1).astype(np.int32)
        # stable sort puts flagged tile indices first, ascending
        order = np.argsort(~flags, axis=-1, kind="stable").astype(np.int32)
        pos = np.arange(nK, dtype=np.int32)
        ids = np.where(pos < lens[..., None], order, np.int32(-1)).astype(np.int32)
        return ids, lens

    fid, fl = compact(full)
    pid, pl = compact(part)
    return OracleMetadata(fid, fl, pid, pl)


def pack_partial(mask: np.ndarray, BQ: int, BK: int, meta: OracleMetadata | None = None, fill: int = 0) -> np.ndarray:
    """Bit-packed PARTIAL tiles, uint8 [B,H,nQ,nK,BQ*BK/8] (C loop ``oracle_pack_partial``).

    Tile ``[b,h,qt,slot]`` holds the entries of KV tile ``meta.masked_kv_ids[b,h,qt,slot]``, rows first,
    little-endian bits; slots past ``meta.masked_lens`` keep ``fill``.
    """
    lib = _load()
    B, H, Sq, Sk = mask.shape
    if Sq % BQ or Sk % BK or BK % 8:
        raise ValueError("Sq % BLOCK_Q, Sk % BLOCK_K and BLOCK_K % 8 must be 0")
    if meta is None:
        meta = classify(mask, BQ, BK)
    m8, strides = _mask_view(mask)
    nQ, nK = Sq // BQ, Sk // BK
    out = np.full((B, H, nQ, nK, BQ * BK // 8), fill, np.uint8)
    ids_p = np.ascontiguousarray(meta.masked_kv_ids, dtype=np.int32)
    len_p = np.ascontiguousarray(meta.masked_lens, dtype=np.int32)
    rc = lib.oracle_pack_partial(_ptr(m8, ctypes.c_uint8), _ptr(strides, ctypes.c_int64), B, H, Sq, Sk, BQ, BK,
                                 _ptr(ids_p, ctypes.c_int32), _ptr(len_p, ctypes.c_int32), _ptr(out, ctypes.c_uint8))
    if rc != 0:
        raise RuntimeError(f"oracle_pack_partial failed: {rc}")
    return out


def forward(q, k, v, mask, BQ: int, BK: int, meta: OracleMetadata | None = None, p_round: int = 0) -> np.ndarray:
    """C restatement of the two-pass forward (sparse_attn_kernel.py:28-63, 103-146).

    ``q, k, v``: float32 arrays [B,H,S,D] (widen bf16/fp16 inputs exactly before calling).
    ``p_round``: 0 keep P in fp32, 1 round P to bf16 before P·V, 2 round to fp16.
    Returns float32 [B,H,Sq,D].
    """
    lib = _load()
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    mask = np.broadcast_to(mask, (B, H, Sq, Sk))
    if meta is None:
        meta = classify(mask, BQ, BK)
    m8, strides = _mask_view(mask)
    out = np.empty_like(q)
    scale_log2 = D ** -0.5 / math.log(2.0)
    ids_f = np.ascontiguousarray(meta.unmasked_kv_ids, dtype=np.int32)
    len_f = np.ascontiguousarray(meta.unmasked_lens, dtype=np.int32)
    ids_p = np.ascontiguousarray(meta.masked_kv_ids, dtype=np.int32)
    len_p = np.ascontiguousarray(meta.masked_lens, dtype=np.int32)
    rc = lib.oracle_forward(
        _ptr(q, ctypes.c_float), _ptr(k, ctypes.c_float), _ptr(v, ctypes.c_float), _ptr(out, ctypes.c_float),
        _ptr(m8, ctypes.c_uint8), _ptr(strides, ctypes.c_int64),
        _ptr(ids_f, ctypes.c_int32), _ptr(len_f, ctypes.c_int32), _ptr(ids_p, ctypes.c_int32), _ptr(len_p, ctypes.c_int32),
        B, H, Sq, Sk, D, BQ, BK, ctypes.c_float(scale_log2), p_round,
    )
    if rc != 0:
        raise RuntimeError(f"oracle_forward failed: {rc}")
    return out


def forward_dense_fp64(q, k, v, mask) -> np.ndarray:
    """Dense masked softmax attention in float64: softmax(QK^T/sqrt(D) + (mask ? 0 : -inf)) V.

    Rows with no attended key give 0.  Quadratic memory: small shapes only.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    mask = np.broadcast_to(np.asarray(mask).astype(bool), (B, H, Sq, Sk))
    s = np.einsum("bhqd,bhkd->bhqk", q, k) / math.sqrt(D)
    s = np.where(mask, s, -np.inf)
    mx = s.max(axis=-1, keepdims=True)
    mx = np.where(np.isfinite(mx), mx, 0.0)
    p = np.exp(s - mx)
    den = p.sum(axis=-1, keepdims=True)
    p = np.divide(p, den, out=np.zeros_like(p), where=den > 0)
    return np.einsum("bhqk,bhkd->bhqd", p, v)


def backward_dense_fp64(q, k, v, mask, do):
    """Gradients of :func:`forward_dense_fp64` with respect to q, k, v for the upstream gradient ``do``, in float64.

    The reference has no backward pass (README.md:65 lists it as future work); this is the textbook derivative of
    o = softmax(q kᵀ/√D + (mask ? 0 : −∞)) v, the function sparse_attn_kernel.py:149-185 computes:
    P = softmax(S), dV = Pᵀ dO, dP = dO Vᵀ, dS = P ∘ (dP − rowsum(dO ∘ O)), dQ = dS K/√D, dK = dSᵀ Q/√D.
    Rows with no attended key have P = 0 and contribute nothing.  Quadratic memory: small shapes only.
    Returns (dq, dk, dv).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    do = np.asarray(do, dtype=np.float64)
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    mask = np.broadcast_to(np.asarray(mask).astype(bool), (B, H, Sq, Sk))
    scale = 1.0 / math.sqrt(D)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * scale
    s = np.where(mask, s, -np.inf)
    mx = s.max(axis=-1, keepdims=True)
    mx = np.where(np.isfinite(mx), mx, 0.0)
    p = np.exp(s - mx)
    den = p.sum(axis=-1, keepdims=True)
    p = np.divide(p, den, out=np.zeros_like(p), where=den > 0)
    o = np.einsum("bhqk,bhkd->bhqd", p, v)
    dv = np.einsum("bhqk,bhqd->bhkd", p, do)
    dp = np.einsum("bhqd,bhkd->bhqk", do, v)
    delta = (do * o).sum(axis=-1, keepdims=True)
    ds = p * (dp - delta)
    dq = np.einsum("bhqk,bhkd->bhqd", ds, k) * scale
    dk = np.einsum("bhqk,bhqd->bhkd", ds, q) * scale
    return dq, dk, dv


def mask_from_terms(terms, B: int, Sq: int, Sk: int, doc_q=None, doc_k=None, q_rows=None) -> np.ndarray:
    """The bool mask [B, rows, Sk] that the terms of the C ABI describe (``sa_mask_classify_terms``).

    ``terms``: int [n][8] = flags, offset, back, ahead, q_lo, q_hi, k_lo, k_hi with flags 1 BACK
    ((q + offset) - k < back), 2 AHEAD (k - (q + offset) < ahead), 4 Q_RANGE, 8 K_RANGE, 16 SAME_DOC
    (doc_q[b, q] == doc_k[b, k]); an entry attends when any term holds, a term holds when all its flagged
    conditions do.  The reference has no such masks (README.md:63 names them as future work); what pins this
    function are the tensor masks it must reproduce: ``numpy.tril`` for causal, banded triangles for windows, the
    reference's own mask semantics (mask_utils.py:34-40) through the tile totals of known masks, and a loop over
    single entries on small shapes.  ``q_rows``: a (start, stop) range of query rows to build (all by default), so
    that long masks can be classified strip by strip.
    """
    terms = np.asarray(terms, dtype=np.int64).reshape(-1, 8)
    q_lo_, q_hi_ = (0, Sq) if q_rows is None else q_rows
    q = np.arange(q_lo_, q_hi_, dtype=np.int64)[None, :, None]
    k = np.arange(Sk, dtype=np.int64)[None, None, :]
    out = np.zeros((B, q_hi_ - q_lo_, Sk), dtype=bool)
    for flags, offset, back, ahead, q_lo, q_hi, k_lo, k_hi in terms:
        ok = np.ones((1, q_hi_ - q_lo_, Sk), dtype=bool)
        d = q + offset - k
        if flags & 1:
            ok &= d < back
        if flags & 2:
            ok &= -d < ahead
        if flags & 4:
            ok &= (q >= q_lo) & (q < q_hi)
        if flags & 8:
            ok &= (k >= k_lo) & (k < k_hi)
        if flags & 16:
            dq = np.broadcast_to(np.asarray(doc_q), (B, Sq))[:, q_lo_:q_hi_, None]
            dk = np.broadcast_to(np.asarray(doc_k), (B, Sk))[:, None, :]
            ok = ok & (dq == dk)
        out |= ok
    return out
