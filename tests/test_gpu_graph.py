"""The forward and decode launches under HIP graph capture: nothing in the library allocates, synchronises or keeps
host state between calls, so a captured step must replay to the eager result, every time, with new inputs in the
same buffers."""
import pytest
import torch

from sparseattention_amd import _native, compute_mask_kernel, sparse_attention, sparse_attention_decode, workloads as W

pytestmark = pytest.mark.gpu


def test_forward_and_decode_replay_to_the_eager_result(gpu):
    B, H, S, D, BQ, BK = 2, 4, 1024, 128, 128, 32
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=21, device=gpu)
    mask = W.random_block_mask(S, 64, 0.5, seed=22, device=gpu)
    me = mask[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, BK, schedule="pairs")
    Sq = 4
    qd = q[:, :, -Sq:].contiguous()
    md_dec = compute_mask_kernel(me[:, :, -Sq:], Sq, BK)
    splits = _native.load().sa_decode_num_splits(B, H, Sq, S, BK)

    def step():
        return (sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md),
                sparse_attention_decode(qd, k, v, me[:, :, -Sq:], BK, mask_metadata=md_dec, num_splits=max(splits, 2)))

    step()  # first launches set the kernels' shared-memory attribute: outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph):
            o_g, od_g = step()
    torch.cuda.current_stream().wait_stream(side)
    gen = torch.Generator().manual_seed(23)
    for it in range(4):
        if it:  # new inputs in the captured buffers, with the program's own eager work and a sync in between
            q.copy_(torch.randn(q.shape, generator=gen).to(gpu, q.dtype))
            k.copy_(torch.randn(k.shape, generator=gen).to(gpu, k.dtype))
            qd.copy_(q[:, :, -Sq:])
            torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        o_e, od_e = step()
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e), f"forward replay {it} differs from the eager result"
        assert torch.equal(od_g, od_e), f"decode replay {it} differs from the eager result"
