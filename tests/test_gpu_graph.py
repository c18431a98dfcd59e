"""The forward, decode and backward launches under HIP graph capture: nothing in the library allocates, synchronises or keeps
host state between calls, so a captured step must replay to the eager result, every time, with new inputs in the
same buffers."""
import pytest
import torch

from sparseattention_amd import (_native, compute_backward_metadata, compute_mask_kernel, sparse_attention,
                                 sparse_attention_backward, sparse_attention_decode, workloads as W)

pytestmark = pytest.mark.gpu


def test_forward_decode_and_backward_replay_to_the_eager_result(gpu):
    B, H, S, D, BQ, BK = 2, 4, 1024, 128, 128, 32
    q, k, v = W.qkv(B, H, S, D, torch.bfloat16, seed=21, device=gpu)
    mask = W.random_block_mask(S, 64, 0.5, seed=22, device=gpu)
    me = mask[None, None].expand(B, H, S, S)
    md = compute_mask_kernel(me, BQ, BK, schedule="pairs")
    Sq = 4
    qd = q[:, :, -Sq:].contiguous()
    md_dec = compute_mask_kernel(me[:, :, -Sq:], Sq, BK)
    splits = _native.load().sa_decode_num_splits(B, H, Sq, S, BK)
    bmd = compute_backward_metadata(me)
    do = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(24)).to(gpu, q.dtype)

    def step():
        o, lse = sparse_attention(q, k, v, me, BQ, BK, mask_metadata=md, return_lse=True)
        od = sparse_attention_decode(qd, k, v, me[:, :, -Sq:], BK, mask_metadata=md_dec, num_splits=max(splits, 2))
        return (o, od) + sparse_attention_backward(do, q, k, v, o, lse, me, bmd)

    step()  # first launches set the kernels' shared-memory attribute: outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph):
            captured = step()
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
        eager = step()
        torch.cuda.synchronize()
        for name, g, e in zip(("forward", "decode", "dq", "dk", "dv"), captured, eager):
            assert torch.equal(g, e), f"{name}: replay {it} differs from the eager result"
