"""The C-ABI library: it loads, exports every symbol the header declares, and rejects bad
arguments on the host before any kernel is launched (so these run without a GPU)."""
import ctypes
import os
import re

import pytest
import torch

from sparseattention_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sparseattn.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sa_[a-z0-9_]+)\s*\(", text)))


def test_header_and_library_agree():
    names = declared_functions()
    assert names, "no functions found in the header"
    lib = _native.load()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in sparseattn.h but not exported"
    assert sorted(_native.EXPORTS) == names
    assert lib.sa_abi_version() == _native.SA_ABI_VERSION
    header = open(HEADER).read()
    assert f"#define SA_ABI_VERSION {_native.SA_ABI_VERSION}" in header
    for name in ("SA_ERR_INVALID_ARGUMENT", "SA_ERR_UNSUPPORTED", "SA_ERR_WORKSPACE", "SA_ERR_HIP"):
        assert re.search(rf"{name}\s*=\s*{getattr(_native, name)}\b", header)


def test_every_entry_point_cites_the_reference_interface_it_replaces():
    text = open(HEADER).read()
    assert "mask_utils.py:85-107" in text and "sparse_attn_kernel.py:149-185" in text


FAKE = 0x1000  # never dereferenced: every call below must fail validation first
S4 = _native.strides((0, 0, 64, 1))
S3 = _native.strides((0, 0, 1))
I4 = _native.strides((0, 0, 2, 1))


def classify(mask=FAKE, ms=S4, B=1, H=1, Sq=64, Sk=64, BQ=32, BK=32, ws=FAKE, ws_bytes=1 << 20, out=FAKE, ids_strides=I4):
    lib = _native.load()
    return lib.sa_mask_classify(mask, ms, B, H, Sq, Sk, BQ, BK, out, ids_strides, out, S3, out, ids_strides, out, S3, ws,
                                ws_bytes, None)


def fwd(q=FAKE, D=128, BQ=128, BK=32, dtype=0, Sq=256, Sk=256, scale=0.1, qs=None, B=1, H=1):
    lib = _native.load()
    qs = qs or _native.strides((Sq * D, Sq * D, D, 1))
    return lib.sa_sparse_attention_fwd(q, qs, FAKE, qs, FAKE, qs, FAKE, qs, FAKE, _native.strides((0, 0, Sk, 1)),
                                       FAKE, I4, FAKE, S3, FAKE, I4, FAKE, S3, B, H, Sq, Sk, D, BQ, BK, dtype, scale, None)


def last_error():
    return _native.load().sa_last_error().decode()


def test_classify_rejects_bad_arguments():
    assert classify(mask=None) == _native.SA_ERR_INVALID_ARGUMENT and "null" in last_error()
    assert classify(out=None) == _native.SA_ERR_INVALID_ARGUMENT
    assert classify(Sq=65) == _native.SA_ERR_INVALID_ARGUMENT and "BLOCK_Q" in last_error()
    assert classify(Sk=100) == _native.SA_ERR_INVALID_ARGUMENT and "BLOCK_K" in last_error()
    assert classify(BQ=0) == _native.SA_ERR_INVALID_ARGUMENT
    assert classify(B=0) == _native.SA_ERR_INVALID_ARGUMENT
    assert classify(ws=None) == _native.SA_ERR_WORKSPACE
    assert classify(ws_bytes=3) == _native.SA_ERR_WORKSPACE and "4 bytes required" in last_error()
    # folded output planes need a broadcast mask
    assert classify(B=2, ms=_native.strides((4096, 0, 64, 1))) == _native.SA_ERR_INVALID_ARGUMENT


def test_workspace_size_counts_distinct_planes_only():
    lib = _native.load()
    f = lib.sa_mask_classify_workspace_bytes
    assert f(_native.strides((0, 0, 4096, 1)), 8, 32, 4096, 4096, 128, 32) == 32 * 128
    assert f(_native.strides((1 << 24, 0, 4096, 1)), 8, 32, 4096, 4096, 128, 32) == 8 * 32 * 128
    assert f(_native.strides((1 << 29, 1 << 24, 4096, 1)), 8, 32, 4096, 4096, 128, 32) == 8 * 32 * 32 * 128
    assert f(_native.strides((0, 0, 4096, 1)), 8, 32, 4096, 4096, 100, 32) == 0


def test_forward_rejects_bad_arguments():
    assert fwd(q=None) == _native.SA_ERR_INVALID_ARGUMENT
    assert fwd(Sq=200) == _native.SA_ERR_INVALID_ARGUMENT
    assert fwd(scale=0.0) == _native.SA_ERR_INVALID_ARGUMENT
    assert fwd(scale=float("nan")) == _native.SA_ERR_INVALID_ARGUMENT
    assert fwd(D=96) == _native.SA_ERR_UNSUPPORTED and "head dim" in last_error()
    assert fwd(BQ=16, Sq=256) == _native.SA_ERR_UNSUPPORTED and "BLOCK_Q" in last_error()
    assert fwd(BQ=512, Sq=512) == _native.SA_ERR_UNSUPPORTED and "BLOCK_Q" in last_error()
    assert fwd(BK=8) == _native.SA_ERR_UNSUPPORTED and "BLOCK_K" in last_error()
    assert fwd(BK=4, Sk=252, Sq=256) == _native.SA_ERR_UNSUPPORTED
    assert fwd(dtype=7) == _native.SA_ERR_UNSUPPORTED and "dtype" in last_error()
    # float32 (dtype 2): any BLOCK_Q up to 256 (128 at head dim 256), strides in multiples of four elements
    f32 = _native.SA_DTYPE_FP32
    assert fwd(dtype=f32, BQ=512, Sq=512) == _native.SA_ERR_UNSUPPORTED and "float32" in last_error()
    assert fwd(dtype=f32, D=256, BQ=256) == _native.SA_ERR_UNSUPPORTED and "float32" in last_error()
    assert fwd(dtype=f32, D=96) == _native.SA_ERR_UNSUPPORTED and "head dim" in last_error()
    assert fwd(dtype=f32, qs=_native.strides((256 * 128, 256 * 128, 130, 1))) == _native.SA_ERR_UNSUPPORTED
    assert fwd(q=FAKE + 2) == _native.SA_ERR_UNSUPPORTED and "aligned" in last_error()
    assert fwd(qs=_native.strides((256 * 128, 256 * 128, 128, 2))) == _native.SA_ERR_UNSUPPORTED
    assert fwd(qs=_native.strides((256 * 128, 256 * 128, 132, 1))) == _native.SA_ERR_UNSUPPORTED


def pack(mask=FAKE, ms=S4, B=1, H=1, Sq=64, Sk=64, BQ=32, BK=32, ids=FAKE, packed=FAKE, ps=None):
    lib = _native.load()
    ps = ps or _native.strides((0, 0))
    return lib.sa_mask_pack_partial(mask, ms, B, H, Sq, Sk, BQ, BK, ids, I4, FAKE, S3, packed, ps, None)


def test_pack_rejects_bad_arguments_and_sizes_its_buffer():
    lib = _native.load()
    f = lib.sa_mask_pack_partial_bytes
    assert f(_native.strides((0, 0, 4096, 1)), 8, 32, 4096, 4096, 128, 32) == 4096 * 4096 // 8
    assert f(_native.strides((1 << 24, 0, 4096, 1)), 8, 32, 4096, 4096, 128, 32) == 8 * 4096 * 4096 // 8
    assert f(_native.strides((0, 0, 4096, 1)), 8, 32, 4096, 4096, 128, 4) == 0      # BLOCK_K % 8
    assert f(_native.strides((0, 0, 4096, 1)), 8, 32, 4096, 4096, 100, 32) == 0
    assert pack(mask=None) == _native.SA_ERR_INVALID_ARGUMENT and "null" in last_error()
    assert pack(packed=None) == _native.SA_ERR_INVALID_ARGUMENT
    assert pack(ids=None) == _native.SA_ERR_INVALID_ARGUMENT
    assert pack(Sq=65) == _native.SA_ERR_INVALID_ARGUMENT and "BLOCK_Q" in last_error()
    assert pack(BK=4) == _native.SA_ERR_UNSUPPORTED and "multiple of 8" in last_error()
    # two distinct batch planes need room for two packed planes
    assert pack(B=2, ms=_native.strides((4096, 0, 64, 1)), ps=_native.strides((8, 0))) == _native.SA_ERR_INVALID_ARGUMENT
    assert "overlap" in last_error()


def test_extended_forward_rejects_bad_arguments():
    lib = _native.load()
    qs = _native.strides((256 * 128, 256 * 128, 128, 1))

    def call(packed=FAKE, ps=_native.strides((0, 0)), mask=None, BK=32, B=1, sched=None, sched_bytes=0):
        return lib.sa_sparse_attention_fwd_ex(FAKE, qs, FAKE, qs, FAKE, qs, FAKE, qs, mask, None, FAKE, I4, FAKE, S3,
                                              FAKE, I4, FAKE, S3, packed, ps, sched, sched_bytes, 0, B, 1, 256, 256,
                                              128, 128, BK, 0, 0.1, None)

    # neither a mask nor packed bits
    assert call(packed=None) == _native.SA_ERR_INVALID_ARGUMENT and "mask" in last_error()
    assert call(ps=None) == _native.SA_ERR_INVALID_ARGUMENT
    assert call(packed=FAKE + 2) == _native.SA_ERR_UNSUPPORTED and "aligned" in last_error()
    assert call(B=2, ps=_native.strides((6, 0))) == _native.SA_ERR_UNSUPPORTED
    assert call(BK=8) == _native.SA_ERR_UNSUPPORTED and "BLOCK_K" in last_error()
    # the plain entry point insists on a mask
    assert lib.sa_sparse_attention_fwd(FAKE, qs, FAKE, qs, FAKE, qs, FAKE, qs, None, None, FAKE, I4, FAKE, S3, FAKE, I4,
                                       FAKE, S3, 1, 1, 256, 256, 128, 128, 32, 0, 0.1, None) == _native.SA_ERR_INVALID_ARGUMENT


def test_schedule_rejects_bad_arguments():
    lib = _native.load()

    def call(fl=FAKE, sched=FAKE, nbytes=16, Sq=256, BQ=128, BK=32, mode=0):
        return lib.sa_fwd_schedule(fl, S3, FAKE, S3, 1, 1, Sq, 256, BQ, BK, mode, sched, nbytes, None)

    assert call(fl=None) == _native.SA_ERR_INVALID_ARGUMENT and "null" in last_error()
    assert call(sched=None) == _native.SA_ERR_INVALID_ARGUMENT
    assert call(Sq=200) == _native.SA_ERR_INVALID_ARGUMENT
    # tile sizes without a persistent kernel (and, without a GPU, every size): unsupported, nothing launched
    assert call(BQ=256) == _native.SA_ERR_UNSUPPORTED and "scheduled" in last_error()
    assert call(BK=8) == _native.SA_ERR_UNSUPPORTED
    assert call(mode=7) == _native.SA_ERR_INVALID_ARGUMENT
    assert lib.sa_fwd_schedule_bytes(1, 1, 256, 256, 256, 32, 0) == 0
    assert lib.sa_fwd_schedule_bytes(1, 1, 256, 256, 100, 32, 1) == 0
    # pairs: one row of three entries per two Q tiles, in whole groups of 8 rows; no device needed for the size
    assert lib.sa_fwd_schedule_bytes(8, 32, 4096, 4096, 128, 32, 1) == 4096 * 3 * 16
    assert lib.sa_fwd_schedule_bytes(1, 1, 256, 256, 128, 32, 1) == 8 * 3 * 16
    assert lib.sa_fwd_schedule_bytes(1, 3, 384, 256, 128, 32, 1) == 8 * 3 * 16    # 3 + 2 workgroups -> 8 rows
    assert call(mode=1, nbytes=16) == _native.SA_ERR_WORKSPACE
    if not torch.cuda.is_available():
        assert lib.sa_fwd_schedule_bytes(1, 1, 256, 256, 128, 32, 0) == 0
        assert call() == _native.SA_ERR_UNSUPPORTED


def test_python_wrappers_refuse_to_run_without_a_gpu_tensor():
    from sparseattention_amd import compute_mask_kernel, sparse_attention

    m = torch.ones(1, 1, 64, 64, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="GPU"):
        compute_mask_kernel(m, 32, 32)
    q = torch.zeros(1, 1, 64, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        sparse_attention(q, q, q, m, 32, 32)
    with pytest.raises(AssertionError):
        compute_mask_kernel(m, 48, 32)  # same assertion as mask_utils.py:89


def test_check_maps_codes_to_exceptions():
    assert classify(Sq=65) == _native.SA_ERR_INVALID_ARGUMENT
    with pytest.raises(ValueError, match="BLOCK_Q"):
        _native.check(_native.SA_ERR_INVALID_ARGUMENT)
    assert fwd(D=96) == _native.SA_ERR_UNSUPPORTED
    with pytest.raises(_native.SparseAttnError) as ei:
        _native.check(_native.SA_ERR_UNSUPPORTED)
    assert ei.value.code == _native.SA_ERR_UNSUPPORTED


def test_product_code_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "sparseattention_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f
                assert "liboracle" not in text, f


def test_reference_import_paths_give_the_same_objects():
    # the reference's callers: from sparseattention.sparse_attn_kernel import sparse_attention;
    # from sparseattention.mask_utils import compute_mask_kernel (test_attn.py:11-12)
    import sparseattention.mask_utils as ref_mu
    import sparseattention.sparse_attn_kernel as ref_sa
    import sparseattention.test_attn as ref_ta
    import sparseattention_amd
    from sparseattention.mask_utils import MaskMetadata, compute_mask_kernel, compute_mask_slow
    from sparseattention.sparse_attn_kernel import sparse_attention

    assert sparse_attention is sparseattention_amd.sparse_attention is ref_sa.sparse_attention
    assert compute_mask_kernel is sparseattention_amd.compute_mask_kernel is ref_mu.compute_mask_kernel
    assert compute_mask_slow is sparseattention_amd.compute_mask_slow
    assert MaskMetadata is sparseattention_amd.MaskMetadata
    assert ref_ta.random_blocked_mask is sparseattention_amd.test_attn.random_blocked_mask
    import dataclasses
    assert [f.name for f in dataclasses.fields(MaskMetadata)][:4] == ["unmasked_kv_ids", "unmasked_lens", "masked_kv_ids",
                                                                     "masked_lens"]


def test_validate_metadata_on_cpu_tensors():
    from sparseattention_amd import compute_mask_slow
    from sparseattention_amd.sparse_attn_kernel import validate_metadata

    mask = (torch.rand(1, 2, 256, 256, generator=torch.Generator().manual_seed(0)) < 0.5)
    mask[0, 0, :64, :64] = True
    mask[0, 1, 64:128, 64:192] = False
    md = compute_mask_slow(mask, 64, 32)
    validate_metadata(md, 256, 32)  # the -1 in unused slots is fine
    with pytest.raises(ValueError, match="slots per Q tile"):
        validate_metadata(md, 512, 32)
    md.unmasked_lens = md.unmasked_lens.clone()
    md.unmasked_lens[0, 0, 0] += 1  # (the tile row holds PARTIAL tiles, so the next slot is a -1)
    with pytest.raises(ValueError, match=r"unmasked_kv_ids\[\.\.\., :len\]"):
        validate_metadata(md, 256, 32)
    md.unmasked_lens[0, 0, 0] = -1
    with pytest.raises(ValueError, match="counts"):
        validate_metadata(md, 256, 32)
    md.unmasked_lens[0, 0, 0] = 9
    with pytest.raises(ValueError, match="counts"):
        validate_metadata(md, 256, 32)


def test_device_check_names_the_tensor():
    from sparseattention_amd.sparse_attn_kernel import _same_device

    ref = torch.empty(1, device="meta")
    _same_device(ref, k=torch.empty(2, device="meta"), mask=None)
    with pytest.raises(ValueError, match="lse is on cpu"):
        _same_device(ref, k=torch.empty(2, device="meta"), lse=torch.empty(2))


def test_validate_metadata_rejects_bad_arguments_on_the_host():
    lib = _native.load()
    args = lambda **kw: [kw.get("ids", FAKE), I4, FAKE, S3, FAKE, I4, FAKE, S3, 1, 1, kw.get("Sq", 64), 64, 32, 32,
                         kw.get("flag", FAKE), None]  # noqa: E731
    assert lib.sa_validate_metadata(*args(ids=None)) == _native.SA_ERR_INVALID_ARGUMENT
    assert lib.sa_validate_metadata(*args(flag=None)) == _native.SA_ERR_INVALID_ARGUMENT
    assert lib.sa_validate_metadata(*args(Sq=65)) == _native.SA_ERR_INVALID_ARGUMENT
    assert lib.sa_validate_metadata(*args(flag=FAKE + 2)) == _native.SA_ERR_INVALID_ARGUMENT
