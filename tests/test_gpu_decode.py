"""Parity of the split-KV kernels for few query rows (sa_sparse_attention_decode through the Python binding).

The function is the forward with BLOCK_Q = Sq (the reference has no decode kernel of its own, README.md:65), so the
checkers are the same: the C oracle run with BQ = Sq on small shapes and torch's masked SDPA in fp32 on all shapes.
Tolerance: max-abs <= 2e-2 for bf16/fp16 inputs."""
import ctypes
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from sparseattention_amd import _native, compute_mask_kernel, sparse_attention, sparse_attention_decode, workloads as W

pytestmark = pytest.mark.gpu

TOL = 2e-2


def sdpa32(q, k, v, mask):
    return F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)


def oracle_out(q, k, v, mask, BK, p_round=1):
    B, H, Sq, _ = q.shape
    Sk = k.shape[2]
    m = mask.expand(B, H, Sq, Sk).cpu().numpy()
    return torch.from_numpy(oracle.forward(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), m,
                                           Sq, BK, p_round=p_round))


def tile_mask(shape, BK, seed, device, p_empty=0.4, p_partial=0.2, keep_first=True):
    """bool mask [..., Sq, Sk]: KV tiles of BK columns are empty / partly random / full; every row keeps one key."""
    g = torch.Generator().manual_seed(seed)
    *lead, Sq, Sk = shape
    nK = Sk // BK
    kind = torch.rand(*lead, 1, nK, generator=g)
    full = kind >= p_empty + p_partial
    part = (kind >= p_empty) & ~full
    bits = torch.rand(*lead, Sq, Sk, generator=g) < 0.5
    m = torch.where(part.repeat_interleave(BK, -1), bits, full.repeat_interleave(BK, -1).expand(*lead, Sq, Sk))
    if keep_first:
        m[..., 0] = True
    return m.to(device)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("Sq", [1, 2, 5, 8, 16, 31, 32])
@pytest.mark.parametrize("BK", [16, 32, 64, 256])
def test_rows_and_tiles_against_oracle_and_sdpa(gpu, D, Sq, BK):
    B, H, Sk = 2, 3, 2048
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=Sq + BK + D, device=gpu, Sk=Sk)
    mask = tile_mask((B, H, Sq, Sk), BK, seed=Sq * BK + D, device=gpu)
    o = sparse_attention_decode(q, k, v, mask, BK)
    torch.cuda.synchronize()
    assert o.shape == q.shape and o.dtype == q.dtype and not torch.isnan(o).any()
    want = oracle_out(q, k, v, mask, BK)
    err = (o.float().cpu() - want).abs()
    assert err.max() <= TOL and err.mean() <= 1e-3, f"vs oracle: max {err.max()}, mean {err.mean()}"
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL


@pytest.mark.parametrize("splits", [1, 2, 3, 7, 16, 64])
def test_every_split_count_gives_the_same_function(gpu, splits):
    B, H, Sq, Sk, D, BK = 1, 4, 4, 4096, 128, 64
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=3, device=gpu, Sk=Sk)
    mask = tile_mask((H, Sq, Sk), BK, seed=4, device=gpu)[None]
    md = compute_mask_kernel(mask.expand(B, H, Sq, Sk), Sq, BK)
    o = sparse_attention_decode(q, k, v, mask, BK, mask_metadata=md, num_splits=splits)
    assert (o.float().cpu() - oracle_out(q, k, v, mask, BK)).abs().max() <= TOL
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL


def test_fp16(gpu):
    B, H, Sq, Sk, D, BK = 2, 2, 8, 2048, 128, 128
    q, k, v = W.qkv(B, H, Sq, D, torch.float16, seed=5, device=gpu, Sk=Sk)
    mask = tile_mask((Sq, Sk), BK, seed=6, device=gpu)
    o = sparse_attention_decode(q, k, v, mask, BK)
    assert (o.float().cpu() - oracle_out(q, k, v, mask, BK, p_round=2)).abs().max() <= 2e-3
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= 2e-3


def test_rows_without_keys_and_planes_without_tiles_give_zero(gpu):
    B, H, Sq, Sk, D, BK = 2, 2, 6, 1024, 64, 32
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=7, device=gpu, Sk=Sk)
    mask = tile_mask((B, H, Sq, Sk), BK, seed=8, device=gpu, keep_first=False)
    mask[0, 0] = False          # a plane with no tile at all
    mask[1, 1, 2] = False       # a dead row among live ones
    mask[1, 0, :, 64:] = False  # everything in the first two tiles
    o = sparse_attention_decode(q, k, v, mask, BK, num_splits=4)
    assert not torch.isnan(o).any()
    assert (o[0, 0] == 0).all() and (o[1, 1, 2] == 0).all()
    assert (o.float().cpu() - oracle_out(q, k, v, mask, BK)).abs().max() <= TOL


def test_one_hot_rows_copy_value_rows_exactly(gpu):
    B, H, Sq, Sk, D, BK = 1, 2, 16, 2048, 128, 32
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=9, device=gpu, Sk=Sk)
    cols = torch.randint(0, Sk, (Sq,), generator=torch.Generator().manual_seed(10)).to(gpu)
    mask = torch.zeros(Sq, Sk, dtype=torch.bool, device=gpu)
    mask[torch.arange(Sq, device=gpu), cols] = True
    o = sparse_attention_decode(q, k, v, mask, BK, num_splits=8)
    assert torch.equal(o, v[:, :, cols, :])


def test_strided_storage_and_broadcast_mask(gpu):
    # [B,S,H,D] storage seen as [B,H,S,D]; a mask shared by all planes through zero strides
    B, H, Sq, Sk, D, BK = 2, 4, 3, 1024, 128, 64
    g = torch.Generator().manual_seed(11)
    q = torch.randn(B, Sq, H, D, generator=g).to(gpu, torch.bfloat16).transpose(1, 2)
    k = torch.randn(B, Sk, H, D, generator=g).to(gpu, torch.bfloat16).transpose(1, 2)
    v = torch.randn(B, Sk, H, D, generator=g).to(gpu, torch.bfloat16).transpose(1, 2)
    mask = tile_mask((Sq, Sk), BK, seed=12, device=gpu)
    o = sparse_attention_decode(q, k, v, mask, BK)
    assert o.stride() == q.stride()
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
    # a transposed (column-major) mask goes through the byte-wise loads
    mt = mask.t().contiguous().t()
    assert mt.stride(-1) != 1
    assert torch.equal(sparse_attention_decode(q, k, v, mt, BK), o)


def test_sparse_attention_routes_short_q_here(gpu):
    B, H, Sq, Sk, D, BK = 1, 2, 8, 1024, 64, 32
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=13, device=gpu, Sk=Sk)
    mask = tile_mask((Sq, Sk), BK, seed=14, device=gpu)
    assert torch.equal(sparse_attention(q, k, v, mask, Sq, BK), sparse_attention_decode(q, k, v, mask, BK))


def test_full_size_window_plus_random_tiles(gpu):
    # B8 H32, 16 query rows at the end of a 32k context: sliding window + attention sinks + random far tiles
    B, H, Sq, Sk, D, BK = 8, 32, 16, 32768, 128, 128
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=15, device=gpu, Sk=Sk)
    pos_q = torch.arange(Sk - Sq, Sk, device=gpu)[:, None]
    pos_k = torch.arange(Sk, device=gpu)[None, :]
    far = (torch.rand(Sk // BK, generator=torch.Generator().manual_seed(16)) < 0.25).to(gpu).repeat_interleave(BK)
    mask = (pos_k <= pos_q) & ((pos_q - pos_k < 4096) | (pos_k < 512) | far[None, :])
    md = compute_mask_kernel(mask.expand(B, H, Sq, Sk), Sq, BK)
    o = sparse_attention_decode(q, k, v, mask, BK, mask_metadata=md)
    for b, h in ((0, 0), (3, 17), (7, 31)):
        want = sdpa32(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], mask)
        assert (o[b:b + 1, h:h + 1].float() - want).abs().max() <= TOL
    # every plane: the output rows are convex combinations of value rows the mask allows
    assert not torch.isnan(o).any()
    vmax = v.float().abs().amax(dim=2, keepdim=True)
    assert (o.float().abs() <= vmax + 1e-2).all()


def test_errors(gpu):
    B, H, Sk, D = 1, 1, 1024, 128
    q, k, v = W.qkv(B, H, 33, D, torch.bfloat16, seed=17, device=gpu, Sk=Sk)
    mask = torch.ones(33, Sk, dtype=torch.bool, device=gpu)
    with pytest.raises(_native.SparseAttnError):
        sparse_attention_decode(q, k, v, mask, 32)  # more than 32 rows
    q8 = q[:, :, :8].contiguous()
    m8 = mask[:8]
    with pytest.raises(_native.SparseAttnError):
        sparse_attention_decode(q8, k, v, m8, 8)  # BLOCK_K below 16
    with pytest.raises(ValueError):
        sparse_attention_decode(q8, k, v, m8, 32, num_splits=300)
    # a workspace that is too small, through the raw ABI
    lib = _native.load()
    md = compute_mask_kernel(m8.expand(B, H, 8, Sk), 8, 32)
    S = _native.strides
    o = torch.empty_like(q8)
    me = m8.expand(B, H, 8, Sk)
    need = lib.sa_decode_workspace_bytes(B, H, 8, D, 4)
    assert need == B * H * 4 * 8 * (D + 2) * 4 and lib.sa_decode_workspace_bytes(B, H, 8, D, 1) == 0
    ws = torch.empty(need // 4 - 1, dtype=torch.float32, device=gpu)
    rc = lib.sa_sparse_attention_decode(
        q8.data_ptr(), S(q8.stride()), k.data_ptr(), S(k.stride()), v.data_ptr(), S(v.stride()), o.data_ptr(),
        S(o.stride()), me.data_ptr(), S(me.stride()), md.unmasked_kv_ids.data_ptr(), S(md.unmasked_kv_ids.stride()),
        md.unmasked_lens.data_ptr(), S(md.unmasked_lens.stride()), md.masked_kv_ids.data_ptr(),
        S(md.masked_kv_ids.stride()), md.masked_lens.data_ptr(), S(md.masked_lens.stride()), B, H, 8, Sk, D, 32,
        _native.SA_DTYPE_BF16, D ** -0.5 / math.log(2), 4, ws.data_ptr(), ws.numel() * 4, None, None,
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == _native.SA_ERR_WORKSPACE and b"workspace" in lib.sa_last_error()
    assert 1 <= lib.sa_decode_num_splits(8, 32, 1, 32768, 128) <= 256


def lse_fp64(q, k, mask):
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double()) / math.sqrt(q.shape[-1])
    return torch.logsumexp(s.masked_fill(~mask.expand(s.shape), -math.inf), dim=-1)


@pytest.mark.parametrize("splits", [1, 5])
def test_lse_output(gpu, splits):
    B, H, Sq, Sk, D, BK = 2, 2, 6, 2048, 128, 64
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=31, device=gpu, Sk=Sk)
    mask = tile_mask((B, H, Sq, Sk), BK, seed=32, device=gpu, keep_first=False)
    mask[1, 1, 3] = False
    o, lse = sparse_attention_decode(q, k, v, mask, BK, num_splits=splits, return_lse=True)
    assert torch.equal(o, sparse_attention_decode(q, k, v, mask, BK, num_splits=splits))
    want = lse_fp64(q, k, mask)
    assert lse.shape == (B, H, Sq) and lse.dtype == torch.float32
    assert lse[1, 1, 3] == -math.inf and torch.isinf(want[1, 1, 3])
    live = torch.isfinite(want)
    assert torch.equal(live, torch.isfinite(lse))
    # the row sum adds up P as rounded to bf16 (8 significant bits) for the P.V product: a sum that one term
    # dominates is off by up to 2^-8 of itself
    assert (lse[live].double() - want[live]).abs().max() <= 6e-3


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("Sq", [1, 2, 6, 16, 31, 32])
@pytest.mark.parametrize("BK", [16, 32, 128])
def test_packed_tiles_give_the_bits_of_the_bool_mask(gpu, D, Sq, BK):
    # the same call fed from the bit-packed PARTIAL tiles and from the bool mask: bit-identical; from the packed tiles no
    # mask tensor is needed (at BLOCK_K = 16 with an odd number of rows the wrapper reads the bool mask)
    B, H, Sk = 2, 2, 4096
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=Sq + BK, device=gpu, Sk=Sk)
    mask = tile_mask((B, 1, Sq, Sk), BK, seed=Sq + 7 * BK, device=gpu, p_partial=0.4).expand(B, H, Sq, Sk)
    md = compute_mask_kernel(mask, Sq, BK)
    assert md.packed_masks is not None
    md_bool = compute_mask_kernel(mask, Sq, BK, pack_partial=False)
    for splits in (1, 5):
        o_pack, lse_pack = sparse_attention_decode(q, k, v, mask, BK, md, num_splits=splits, return_lse=True)
        o_bool, lse_bool = sparse_attention_decode(q, k, v, mask, BK, md_bool, num_splits=splits, return_lse=True)
        assert torch.equal(o_pack, o_bool) and torch.equal(lse_pack, lse_bool)
    assert (o_pack.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
    if BK > 16 or Sq % 2 == 0:
        # blind to the mask tensor: none at all, or one with the wrong content
        assert torch.equal(sparse_attention_decode(q, k, v, None, BK, md, num_splits=5), o_pack)
        assert torch.equal(sparse_attention_decode(q, k, v, torch.zeros_like(mask), BK, md, num_splits=5), o_pack)
        if Sq < 32:  # (32 rows are a Q tile of the forward kernels)
            assert torch.equal(sparse_attention(q, k, v, None, Sq, BK, md), sparse_attention_decode(q, k, v, None, BK, md))
    else:
        with pytest.raises(ValueError, match="packed_masks"):
            sparse_attention_decode(q, k, v, None, BK, md)


def test_packed_entry_point_refusals(gpu):
    lib = _native.load()
    st = _native.strides
    B, H, Sq, Sk, D, BK = 1, 1, 3, 512, 64, 16
    q, k, v = W.qkv(B, H, Sq, D, torch.bfloat16, seed=1, device=gpu, Sk=Sk)
    mask = tile_mask((B, H, Sq, Sk), BK, seed=2, device=gpu)
    md = compute_mask_kernel(mask, Sq, BK)
    o = torch.empty_like(q)

    def raw(mask_t, packed):
        return lib.sa_sparse_attention_decode_ex(
            q.data_ptr(), st(q.stride()), k.data_ptr(), st(k.stride()), v.data_ptr(), st(v.stride()), o.data_ptr(), st(o.stride()),
            mask_t.data_ptr() if mask_t is not None else None, st(mask_t.stride()) if mask_t is not None else None,
            md.unmasked_kv_ids.data_ptr(), st(md.unmasked_kv_ids.stride()), md.unmasked_lens.data_ptr(), st(md.unmasked_lens.stride()),
            md.masked_kv_ids.data_ptr(), st(md.masked_kv_ids.stride()), md.masked_lens.data_ptr(), st(md.masked_lens.stride()),
            packed.data_ptr() if packed is not None else None, st(packed.stride()[:2]) if packed is not None else None,
            B, H, Sq, Sk, D, BK, 0, D ** -0.5 / math.log(2), 1, None, 0, None, None, torch.cuda.current_stream().cuda_stream)

    assert raw(None, None) == _native.SA_ERR_INVALID_ARGUMENT          # neither mask nor packed tiles
    assert raw(None, md.packed_masks) == _native.SA_ERR_UNSUPPORTED    # halfword rows, odd row count
    assert raw(mask, None) == 0
    torch.cuda.synchronize()
    assert (o.float() - sdpa32(q, k, v, mask)).abs().max() <= TOL
