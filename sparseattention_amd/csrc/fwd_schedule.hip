// Hand-out of Q tiles to the persistent workgroups of the block-sparse forward (no counterpart in the reference,
// whose launch grid is one program per Q tile, sparse_attn_kernel.py:167).
//
// The forward's cost per Q tile is known before it runs: the lengths of the two lists.  One wave per XCD deals
// the tiles of that XCD's eighth of the (b,h)-major order out in rounds of one tile per workgroup: the tiles of a
// round are ranked by cost, the workgroups by the work they already hold, and the costliest tile goes to the
// least loaded workgroup.  Rounds follow the order in which the planes are laid out, so at any time the
// workgroups of an XCD work on the same few K/V planes, and under regular masks (causal: cost rises with the
// tile index) the loads even out every other round.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace sa {

namespace {

// grid 8 (one wave per XCD), 64 threads; lane j is workgroup 8*j + x.
__global__ __launch_bounds__(64) void schedule_kernel(const ScheduleParams p) {
    __shared__ int by_rank[64];
    const int lane = threadIdx.x, x = blockIdx.x;
    const int W = p.G >> 3;
    const int64_t N = (int64_t)p.B * p.H * p.nQ;
    const int64_t NX = (N + 7) / 8;
    const int64_t first = x * NX, end = first + NX < N ? first + NX : N;
    const int BH = p.B * p.H;
    const bool is_wg = lane < W;
    int load = is_wg ? 0 : 0x7fffffff;  // lanes that stand for no workgroup rank last and take the idle slots
    int count = 0;
    int4 *row = reinterpret_cast<int4 *>(p.sched) + (int64_t)(8 * lane + x) * (p.R + 1);
    for (int r = 0; r < p.R; r++) {
        const int64_t lin = first + (int64_t)r * W + lane;
        const bool valid = is_wg && lin < end;
        int bh = 0, qt = 0, F = 0, P = 0, cost = -1;
        if (valid) {
            // planes two at a time with their Q tiles interleaved, last Q tile first
            const int pair = (int)(lin / (2 * p.nQ)), rr = (int)(lin - (int64_t)pair * 2 * p.nQ);
            const bool paired = 2 * pair + 1 < BH;
            bh = 2 * pair + (paired ? (rr & 1) : 0);
            qt = p.nQ - 1 - (paired ? (rr >> 1) : rr);
            const int b = bh / p.H, h = bh - b * p.H;
            F = p.full_lens[b * p.fls[0] + h * p.fls[1] + qt * p.fls[2]];
            P = p.part_lens[b * p.pls[0] + h * p.pls[1] + qt * p.pls[2]];
            // cost in quarter chunks: 4 per chunk of 64 keys, 1 more per chunk with PARTIAL entries, 8 per tile
            const int ne = F + P > 0 ? F + P : 1;
            const int chunks = p.lbk >= 6 ? ne << (p.lbk - 6) : (ne + (64 >> p.lbk) - 1) >> (6 - p.lbk);
            const int pchunks = p.lbk >= 6 ? P << (p.lbk - 6) : (P + (64 >> p.lbk) - 1) >> (6 - p.lbk);
            cost = 4 * chunks + pchunks + 8;
            bh = (b << 16) | h;
        }
        // rank of this lane's tile (costliest first) and of this lane's workgroup (least loaded first)
        int rank_tile = 0, rank_wg = 0;
        for (int m = 0; m < 64; m++) {
            const int cm = __shfl(cost, m), lm = __shfl(load, m);
            rank_tile += (cm > cost || (cm == cost && m < lane)) ? 1 : 0;
            rank_wg += (lm < load || (lm == load && m < lane)) ? 1 : 0;
        }
        by_rank[rank_tile] = lane;
        __syncthreads();
        const int src = by_rank[rank_wg];
        __syncthreads();
        const int t_bh = __shfl(bh, src), t_qt = __shfl(qt, src), t_F = __shfl(F, src), t_P = __shfl(P, src);
        const int t_cost = __shfl(cost, src);
        if (is_wg && t_cost >= 0) {
            row[1 + count] = int4{t_bh, t_qt, t_F, t_P};
            count++;
            load += t_cost;
        }
    }
    if (is_wg) row[0] = int4{count, 0, 0, 0};
}

// Pairs: workgroup w takes two Q tiles of one pair of planes, the r-th costliest-first and the r-th from the other
// end (under causal-like masks a long list with a short one, so that all workgroups carry the same load and
// the hardware dispatcher still evens out what differs).  The last plane of an odd count pairs its own tiles.
// One thread per schedule row g; rows are handed to XCDs in turn, so row g holds workgroup (g & 7) * G/8 + g / 8.
__global__ __launch_bounds__(256) void schedule_pairs_kernel(const ScheduleParams p) {
    const int g = blockIdx.x * 256 + threadIdx.x;
    if (g >= p.G) return;
    const int BH = p.B * p.H;
    const int pairs = BH >> 1;
    const int64_t w = (int64_t)(g & 7) * (p.G >> 3) + (g >> 3);
    int4 *row = reinterpret_cast<int4 *>(p.sched) + (int64_t)g * (p.R + 1);
    int bh[2], qt[2], n = 0;
    if (w < (int64_t)pairs * p.nQ) {
        const int pp = (int)(w / p.nQ), r = (int)(w - (int64_t)pp * p.nQ);
        // position r of the pair's interleaved order: plane r & 1, tile nQ-1 - r/2; its mirror 2nQ-1-r
        const int r2 = 2 * p.nQ - 1 - r;
        bh[0] = 2 * pp + (r & 1), qt[0] = p.nQ - 1 - (r >> 1);
        bh[1] = 2 * pp + (r2 & 1), qt[1] = p.nQ - 1 - (r2 >> 1);
        n = 2;
    } else if (BH & 1) {
        const int64_t r = w - (int64_t)pairs * p.nQ;  // the unpaired plane: tile nQ-1-r with tile r
        if (r < (p.nQ + 1) / 2) {
            bh[0] = BH - 1, qt[0] = p.nQ - 1 - (int)r;
            n = 1;
            if ((int)r != p.nQ - 1 - (int)r) {
                bh[1] = BH - 1, qt[1] = (int)r;
                n = 2;
            }
        }
    }
    for (int i = 0; i < n; i++) {
        const int b = bh[i] / p.H, h = bh[i] - b * p.H;
        row[1 + i] = int4{(b << 16) | h, qt[i], p.full_lens[b * p.fls[0] + h * p.fls[1] + qt[i] * p.fls[2]],
                          p.part_lens[b * p.pls[0] + h * p.pls[1] + qt[i] * p.pls[2]]};
    }
    row[0] = int4{n, 0, 0, 0};
}

}  // namespace

hipError_t launch_schedule(const ScheduleParams &p, hipStream_t stream) {
    if (p.pairs) hipLaunchKernelGGL(schedule_pairs_kernel, dim3((p.G + 255) / 256), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(schedule_kernel, dim3(8), dim3(64), 0, stream, p);
    return hipGetLastError();
}

}  // namespace sa
