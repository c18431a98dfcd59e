"""Host logic that maps a request for tile sizes and head dims onto what the kernels have (no GPU)."""
import pytest

from sparseattention_amd.sparse_attn_kernel import _kernel_head_dim, kernel_tiles


@pytest.mark.parametrize("args,want", [
    ((4096, 4096, 128, 128, 32), (128, 32)),   # the headline tiles are kept
    ((4096, 4096, 128, 256, 16), (256, 16)),
    ((4096, 4096, 128, 16, 32), (128, 32)),    # no kernel for 16 rows: the preferred size that divides Sq
    ((96, 4096, 128, 16, 32), (32, 32)),
    ((4096, 4096, 128, 512, 8), (128, 32)),    # nor for 8 keys
    ((4096, 48, 128, 128, 8), (128, 16)),      # 48 keys: only 16 divides
    ((4096, 40, 128, 128, 8), None),
    ((4096, 4096, 256, 32, 32), (128, 32)),    # head dim 256 has Q tiles of 64 and 128 rows
    ((4096, 4096, 192, 256, 64), (128, 64)),   # 192 runs as 256
    ((64, 4096, 256, 64, 32), (64, 32)),
    ((48, 4096, 128, 16, 32), None),           # no Q tile divides 48 rows: the wrapper pads the rows
    ((16, 4096, 128, 16, 64), (16, 64)),       # fewer than 32 rows: the few-rows kernels, one Q tile
    ((16, 4096, 128, 8, 16), (16, 16)),        # (tiles of 16 keys they have)
    ((16, 4096, 128, 8, 8), (16, 32)),
    ((16, 4096, 192, 16, 64), None),           # which stop at head dim 128
])
def test_kernel_tiles(args, want):
    assert kernel_tiles(*args) == want
    if want is not None:
        assert args[0] % want[0] == 0 and args[1] % want[1] == 0


def test_kernel_head_dim():
    sizes = (64, 128, 256)
    assert [_kernel_head_dim(d, sizes) for d in (16, 64, 65, 96, 128, 192, 256)] == [64, 64, 128, 128, 128, 256, 256]
    assert _kernel_head_dim(320, sizes) == 320  # passed on, for the library to refuse
