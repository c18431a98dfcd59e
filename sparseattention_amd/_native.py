"""ctypes binding of libsparseattn_hip.so (the C ABI declared in include/sparseattn.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsparseattn_hip.so")

SA_ABI_VERSION = 14
SA_OK = 0
SA_ERR_INVALID_ARGUMENT = -1
SA_ERR_UNSUPPORTED = -2
SA_ERR_WORKSPACE = -3
SA_ERR_HIP = -4

SA_DTYPE_BF16 = 0
SA_DTYPE_FP16 = 1
SA_DTYPE_FP32 = 2  # forward only

SA_SCHEDULE_PERSISTENT = 0
SA_SCHEDULE_PAIRS = 1
SA_FWD_KERNEL_DEFAULT = 0
SA_FWD_KERNEL_SHORT_LISTS = 1
SA_FWD_KERNEL_ROTATED = 2
SA_FWD_SHORT_LISTS_MAX_ENTRIES = 256

#: every symbol include/sparseattn.h declares
EXPORTS = (
    "sa_abi_version",
    "sa_last_error",
    "sa_mask_classify_workspace_bytes",
    "sa_mask_classify",
    "sa_mask_classify_static",
    "sa_validate_metadata",
    "sa_sparse_attention_fwd",
    "sa_mask_pack_partial_bytes",
    "sa_mask_pack_partial",
    "sa_fwd_schedule_bytes",
    "sa_fwd_schedule",
    "sa_sparse_attention_fwd_ex",
    "sa_sparse_attention_fwd_lse",
    "sa_sparse_attention_fwd_kernel",
    "sa_decode_num_splits",
    "sa_decode_workspace_bytes",
    "sa_sparse_attention_decode",
    "sa_sparse_attention_decode_ex",
    "sa_merge_attention_parts",
    "sa_bwd_workspace_bytes",
    "sa_sparse_attention_bwd",
    "sa_mask_terms_workspace_bytes",
    "sa_mask_classify_terms",
)

_lib = None

_i64p = ctypes.POINTER(ctypes.c_int64)
_vp = ctypes.c_void_p


class SparseAttnError(RuntimeError):
    """A call into libsparseattn_hip.so returned an error code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libsparseattn_hip error {code}: {message}")
        self.code = code


def load() -> ctypes.CDLL:
    """Load the in-tree HIP library.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m sparseattention_amd.build` "
            "(hipcc, gfx950).  There is no CPU or PyTorch fallback for the attention path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.sa_abi_version.restype = ctypes.c_int
    lib.sa_abi_version.argtypes = []
    lib.sa_last_error.restype = ctypes.c_char_p
    lib.sa_last_error.argtypes = []
    lib.sa_mask_classify_workspace_bytes.restype = ctypes.c_size_t
    lib.sa_mask_classify_workspace_bytes.argtypes = [_i64p] + [ctypes.c_int] * 6
    lib.sa_mask_classify.restype = ctypes.c_int
    lib.sa_mask_classify.argtypes = (
        [_vp, _i64p] + [ctypes.c_int] * 6 + [_vp, _i64p] * 4 + [_vp, ctypes.c_size_t, _vp]
    )
    lib.sa_mask_classify_static.restype = ctypes.c_int
    lib.sa_mask_classify_static.argtypes = [_vp, _i64p] + [ctypes.c_int] * 6 + [_vp, _i64p] * 4 + [_vp]
    lib.sa_validate_metadata.restype = ctypes.c_int
    lib.sa_validate_metadata.argtypes = [_vp, _i64p] * 4 + [ctypes.c_int] * 6 + [_vp, _vp]
    lib.sa_sparse_attention_fwd.restype = ctypes.c_int
    lib.sa_sparse_attention_fwd.argtypes = (
        [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, _i64p] * 4 + [ctypes.c_int] * 8 + [ctypes.c_float, _vp]
    )
    lib.sa_mask_pack_partial_bytes.restype = ctypes.c_size_t
    lib.sa_mask_pack_partial_bytes.argtypes = [_i64p] + [ctypes.c_int] * 6
    lib.sa_mask_pack_partial.restype = ctypes.c_int
    lib.sa_mask_pack_partial.argtypes = [_vp, _i64p] + [ctypes.c_int] * 6 + [_vp, _i64p] * 3 + [_vp]
    lib.sa_fwd_schedule_bytes.restype = ctypes.c_size_t
    lib.sa_fwd_schedule_bytes.argtypes = [ctypes.c_int] * 7
    lib.sa_fwd_schedule.restype = ctypes.c_int
    lib.sa_fwd_schedule.argtypes = [_vp, _i64p] * 2 + [ctypes.c_int] * 7 + [_vp, ctypes.c_size_t, _vp]
    lib.sa_sparse_attention_fwd_ex.restype = ctypes.c_int
    lib.sa_sparse_attention_fwd_ex.argtypes = (
        [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, ctypes.c_size_t]
        + [ctypes.c_int] * 9 + [ctypes.c_float, _vp]
    )
    lib.sa_sparse_attention_fwd_lse.restype = ctypes.c_int
    lib.sa_sparse_attention_fwd_lse.argtypes = (
        [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, ctypes.c_size_t, ctypes.c_int]
        + [_vp, _i64p] + [ctypes.c_int] * 8 + [ctypes.c_float, _vp]
    )
    lib.sa_decode_num_splits.restype = ctypes.c_int
    lib.sa_decode_num_splits.argtypes = [ctypes.c_int] * 5
    lib.sa_decode_workspace_bytes.restype = ctypes.c_size_t
    lib.sa_decode_workspace_bytes.argtypes = [ctypes.c_int] * 5
    lib.sa_sparse_attention_decode.restype = ctypes.c_int
    lib.sa_sparse_attention_fwd_kernel.restype = ctypes.c_int
    lib.sa_sparse_attention_fwd_kernel.argtypes = (
        [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, _i64p] + [ctypes.c_int] * 8
        + [ctypes.c_float, ctypes.c_int, _vp]
    )
    lib.sa_sparse_attention_decode.argtypes = (
        [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, _i64p] * 4 + [ctypes.c_int] * 7 + [ctypes.c_float, ctypes.c_int]
        + [_vp, ctypes.c_size_t] + [_vp, _i64p] + [_vp]
    )
    lib.sa_sparse_attention_decode_ex.restype = ctypes.c_int
    lib.sa_sparse_attention_decode_ex.argtypes = (
        [_vp, _i64p] * 4 + [_vp, _i64p] + [_vp, _i64p] * 4 + [_vp, _i64p] + [ctypes.c_int] * 7 + [ctypes.c_float, ctypes.c_int]
        + [_vp, ctypes.c_size_t] + [_vp, _i64p] + [_vp]
    )
    lib.sa_merge_attention_parts.restype = ctypes.c_int
    lib.sa_merge_attention_parts.argtypes = [_vp, _i64p] * 4 + [ctypes.c_int] * 6 + [_vp]
    lib.sa_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.sa_bwd_workspace_bytes.argtypes = [ctypes.c_int] * 3
    lib.sa_sparse_attention_bwd.restype = ctypes.c_int
    lib.sa_sparse_attention_bwd.argtypes = (
        [_vp, _i64p] * 13 + [_vp, _i64p] * 8 + [_vp, ctypes.c_size_t] + [ctypes.c_int] * 6 + [ctypes.c_float, _vp]
    )
    lib.sa_mask_terms_workspace_bytes.restype = ctypes.c_size_t
    lib.sa_mask_terms_workspace_bytes.argtypes = [ctypes.c_int] * 5
    lib.sa_mask_classify_terms.restype = ctypes.c_int
    lib.sa_mask_classify_terms.argtypes = (
        [ctypes.POINTER(ctypes.c_int32), ctypes.c_int] + [_vp, _i64p] * 2 + [ctypes.c_int] * 6 + [_vp, _i64p] * 4
        + [_vp, _i64p] + [_vp, ctypes.c_size_t, _vp]
    )
    if lib.sa_abi_version() != SA_ABI_VERSION:
        raise RuntimeError(f"libsparseattn_hip ABI {lib.sa_abi_version()} != expected {SA_ABI_VERSION}")
    _lib = lib
    return lib


def strides(values):
    """int64[n] ctypes array from an iterable of strides."""
    values = tuple(int(v) for v in values)
    return (ctypes.c_int64 * len(values))(*values)


def check(rc: int) -> None:
    if rc != SA_OK:
        msg = load().sa_last_error().decode("utf-8", "replace")
        if rc == SA_ERR_INVALID_ARGUMENT:
            raise ValueError(f"libsparseattn_hip: {msg}")
        raise SparseAttnError(rc, msg)
