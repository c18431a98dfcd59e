// Tile classification of a boolean attention mask on gfx950 (MI355X).
//
// Replaces the Triton kernel _compute_mask_inner (sparseattention/mask_utils.py:47-82), which walks the
// KV tiles of one Q-tile row serially and loads 32-byte row segments.  Here the work is split in two:
//
//   classify_wide_kernel / classify_generic_kernel
//       one class byte per (plane, Q tile, KV tile): 0 = empty, 1 = partial, 2 = full.  The wide kernel
//       streams the mask with 16-byte loads, 1 KiB contiguous per wave per row, and every byte of a
//       distinct plane is read exactly once.
//   compact_kernel
//       one wave per (b, h, Q tile): ballot + popcount prefix over the class bytes, writing the two
//       ascending index lists and their counts (mask_utils.py:72-82).
//   pack_partial_kernel (optional, no counterpart in the reference)
//       one bit per entry of every PARTIAL tile, so that the forward reads BQ*BK/8 contiguous bytes per
//       partial tile instead of BQ row segments of the mask (sparse_attn_kernel.py:42-46).
//
// A byte != 0 counts as "attend", so masks that were viewed from uint8 storage behave like torch.sum.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace sa {

namespace {

// 0x80 in every byte of x that is non-zero.
__device__ __forceinline__ uint32_t nonzero_bytes(uint32_t x) {
    return (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWideCols = 1024;  // mask columns covered by one workgroup: 64 lanes x 16 bytes
constexpr int kRowUnroll = 8;    // independent 16-byte loads in flight per lane

// grid (ceil(Sk/1024), nQ, distinct planes), 256 threads.  The four waves of a workgroup take rows
// w, w+4, ... of the same BQ x 1024 slab, so consecutive lanes always read consecutive 16-byte
// pieces of one mask row; the per-wave results meet in LDS.
__global__ __launch_bounds__(256) void classify_wide_kernel(const ClassifyParams p) {
    __shared__ unsigned long long sh_all[4];
    __shared__ unsigned long long sh_any[4];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int qt = blockIdx.y;
    const int plane = blockIdx.z;
    const int ub = plane / p.uH, uh = plane - ub * p.uH;
    const int col = blockIdx.x * kWideCols + lane * 16;
    const bool in_range = col < p.Sk;

    uint32_t any = 0u, all = 0x80808080u;
    if (in_range) {
        const uint8_t *base = p.mask + (int64_t)ub * p.sb + (int64_t)uh * p.sh + (int64_t)qt * p.BQ * p.sq + col;
        int r = wave;
        for (; r + 4 * (kRowUnroll - 1) < p.BQ; r += 4 * kRowUnroll) {
            u32x4 v[kRowUnroll];
#pragma unroll
            for (int u = 0; u < kRowUnroll; u++)
                v[u] = __builtin_nontemporal_load((const u32x4 *)(base + (int64_t)(r + 4 * u) * p.sq));
#pragma unroll
            for (int u = 0; u < kRowUnroll; u++) {
                any |= v[u].x | v[u].y | v[u].z | v[u].w;
                all &= nonzero_bytes(v[u].x) & nonzero_bytes(v[u].y) & nonzero_bytes(v[u].z) & nonzero_bytes(v[u].w);
            }
        }
        for (; r < p.BQ; r += 4) {
            const u32x4 v = __builtin_nontemporal_load((const u32x4 *)(base + (int64_t)r * p.sq));
            any |= v.x | v.y | v.z | v.w;
            all &= nonzero_bytes(v.x) & nonzero_bytes(v.y) & nonzero_bytes(v.z) & nonzero_bytes(v.w);
        }
    }
    const unsigned long long ball_all = __ballot(all == 0x80808080u);
    const unsigned long long ball_any = __ballot(any != 0u);
    if (lane == 0) {
        sh_all[wave] = ball_all;
        sh_any[wave] = ball_any;
    }
    __syncthreads();

    const int tiles = kWideCols >> p.lbk;  // KV tiles per slab, <= 64
    const int t = threadIdx.x;
    if (t < tiles) {
        const int kt = blockIdx.x * tiles + t;
        if (kt < p.nK) {
            const unsigned long long a = sh_all[0] & sh_all[1] & sh_all[2] & sh_all[3];
            const unsigned long long o = sh_any[0] | sh_any[1] | sh_any[2] | sh_any[3];
            const int lpt = p.BK >> 4;  // lanes per tile
            const unsigned long long field = lpt == 64 ? ~0ull : (((1ull << lpt) - 1ull) << (t * lpt));
            const uint8_t cls = (a & field) == field ? 2 : ((o & field) != 0ull ? 1 : 0);
            p.cls[((int64_t)plane * p.nQ + qt) * p.nK + kt] = cls;
        }
    }
}

// One thread per tile, any strides, any tile shape.
__global__ __launch_bounds__(256) void classify_generic_kernel(const ClassifyParams p) {
    const int64_t total = (int64_t)p.uB * p.uH * p.nQ * p.nK;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    const int kt = (int)(t % p.nK);
    const int qt = (int)((t / p.nK) % p.nQ);
    const int plane = (int)(t / ((int64_t)p.nK * p.nQ));
    const int ub = plane / p.uH, uh = plane - ub * p.uH;
    const uint8_t *base = p.mask + (int64_t)ub * p.sb + (int64_t)uh * p.sh + (int64_t)qt * p.BQ * p.sq +
                          (int64_t)kt * p.BK * p.sk;
    int64_t count = 0;
    for (int r = 0; r < p.BQ; r++) {
        const uint8_t *row = base + (int64_t)r * p.sq;
        for (int c = 0; c < p.BK; c++) count += row[(int64_t)c * p.sk] != 0;
    }
    p.cls[t] = count == (int64_t)p.BQ * p.BK ? 2 : (count > 0 ? 1 : 0);
}

// One wave per (b, h, Q tile) row of the outputs; 4 rows per workgroup.
__global__ __launch_bounds__(256) void compact_kernel(const CompactParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)p.oB * p.oH * p.nQ) return;
    const int qt = (int)(row % p.nQ);
    const int h = (int)((row / p.nQ) % p.oH);
    const int b = (int)(row / ((int64_t)p.nQ * p.oH));
    const int ub = p.bcast_b ? 0 : b, uh = p.bcast_h ? 0 : h;
    const uint8_t *cls = p.cls + (((int64_t)ub * p.uH + uh) * p.nQ + qt) * p.nK;
    int32_t *fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + qt * p.fis[2];
    int32_t *pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + qt * p.pis[2];
    const unsigned long long below = (1ull << lane) - 1ull;
    int nf = 0, np = 0;
    for (int k0 = 0; k0 < p.nK; k0 += 64) {
        const int kt = k0 + lane;
        const int c = kt < p.nK ? cls[kt] : 0;
        const unsigned long long bf = __ballot(c == 2);
        const unsigned long long bp = __ballot(c == 1);
        if (c == 2) fid[(int64_t)(nf + __popcll(bf & below)) * p.fis[3]] = kt;
        if (c == 1) pid[(int64_t)(np + __popcll(bp & below)) * p.pis[3]] = kt;
        nf += __popcll(bf);
        np += __popcll(bp);
    }
    if (lane == 0) {
        p.full_lens[b * p.fls[0] + h * p.fls[1] + qt * p.fls[2]] = nf;
        p.part_lens[b * p.pls[0] + h * p.pls[1] + qt * p.pls[2]] = np;
    }
}

// grid (slot lanes, nQ, distinct planes), 256 threads.  Workgroup x takes a run of consecutive PARTIAL slots of its Q
// tile, at least four: neighbouring tiles share the 128-byte lines of the mask rows (four tiles of 32 keys per line),
// and the workgroups of one Q tile run on different XCDs, each with an L2 of its own.  A thread makes one output
// byte at a time from 8 neighbouring mask entries of one row.
// The lists may be a caller's own: the count is clamped to the nK slots a Q tile has in `packed`, and a slot whose
// index lies outside [0, nK) is left untouched, so neither the reads of the mask nor the writes of `packed` leave
// their tensors whatever the lists hold.
__global__ __launch_bounds__(256) void pack_partial_kernel(const PackParams p) {
    const int qt = blockIdx.y;
    const int plane = blockIdx.z;
    const int ub = plane / p.uH, uh = plane - ub * p.uH;
    const int len = min(max(p.part_lens[ub * p.pls[0] + uh * p.pls[1] + qt * p.pls[2]], 0), p.nK);
    const int32_t *ids = p.part_ids + ub * p.pis[0] + uh * p.pis[1] + qt * p.pis[2];
    const int bpr = p.BK >> 3;                 // output bytes per tile row
    const int tile_bytes = p.BQ * bpr;
    const uint8_t *rows = p.mask + (int64_t)ub * p.sb + (int64_t)uh * p.sh + (int64_t)qt * p.BQ * p.sq;
    uint8_t *out_q = p.packed + (int64_t)ub * p.ob + (int64_t)uh * p.oh + (int64_t)qt * p.nK * tile_bytes;
    const int per = max(4, (len + (int)gridDim.x - 1) / (int)gridDim.x);
    const int slot_end = min(len, ((int)blockIdx.x + 1) * per);
    for (int slot = blockIdx.x * per; slot < slot_end; slot++) {
        const int id = ids[(int64_t)slot * p.pis[3]];
        if ((unsigned)id >= (unsigned)p.nK) continue;  // (uniform over the workgroup)
        const int64_t col0 = (int64_t)id * p.BK;
        uint8_t *out = out_q + (int64_t)slot * tile_bytes;
        for (int o = threadIdx.x; o < tile_bytes; o += 256) {
            const int r = o / bpr, cb = o - r * bpr;
            const uint8_t *src = rows + (int64_t)r * p.sq + (col0 + 8 * cb) * p.sk;
            uint32_t lo, hi;
            if (p.vec8) {
                const uint2 w = *(const uint2 *)src;
                lo = w.x;
                hi = w.y;
            } else {
                lo = hi = 0u;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    lo |= (uint32_t)src[(int64_t)i * p.sk] << (8 * i);
                    hi |= (uint32_t)src[(int64_t)(4 + i) * p.sk] << (8 * i);
                }
            }
            // 0x80 per non-zero byte -> one bit per byte, entry i of the group in bit i
            const uint32_t a = nonzero_bytes(lo) >> 7, b = nonzero_bytes(hi) >> 7;
            // (bits 0, 8, 16, 24 times 2^21 + 2^14 + 2^7 + 1 meet in bits 21..24, without carries)
            const uint32_t nib_lo = ((a * 0x00204081u) >> 21) & 0xfu, nib_hi = ((b * 0x00204081u) >> 21) & 0xfu;
            out[o] = (uint8_t)(nib_lo | (nib_hi << 4));
        }
    }
}

// One wave per (b, h, Q tile) row of the lists: bit 0 of *flag when a count is negative or the two counts exceed nK,
// bit 1 when a FULL index inside its count lies outside [0, nK), bit 2 the same for a PARTIAL index.
__global__ __launch_bounds__(256) void validate_lists_kernel(const ValidateParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)p.B * p.H * p.nQ) return;
    const int qt = (int)(row % p.nQ);
    const int h = (int)((row / p.nQ) % p.H);
    const int b = (int)(row / ((int64_t)p.nQ * p.H));
    const int nf = p.full_lens[b * p.fls[0] + h * p.fls[1] + qt * p.fls[2]];
    const int np = p.part_lens[b * p.pls[0] + h * p.pls[1] + qt * p.pls[2]];
    int bad = (nf < 0 || np < 0 || (int64_t)nf + np > p.nK) ? 1 : 0;
    const int32_t *fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + qt * p.fis[2];
    const int32_t *pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + qt * p.pis[2];
    const int cf = nf < 0 ? 0 : (nf > p.nK ? p.nK : nf), cp = np < 0 ? 0 : (np > p.nK ? p.nK : np);  // slots that exist
    for (int e = lane; e < cf; e += 64)
        if ((unsigned)fid[(int64_t)e * p.fis[3]] >= (unsigned)p.nK) bad |= 2;
    for (int e = lane; e < cp; e += 64)
        if ((unsigned)pid[(int64_t)e * p.pis[3]] >= (unsigned)p.nK) bad |= 4;
    if (bad) atomicOr(p.flag, bad);
}

}  // namespace

hipError_t launch_validate(const ValidateParams &p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.B * p.H * p.nQ;
    hipLaunchKernelGGL(validate_lists_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_pack(const PackParams &p, hipStream_t stream) {
    const int lanes = p.nK < 8 ? p.nK : 8;
    hipLaunchKernelGGL(pack_partial_kernel, dim3(lanes, p.nQ, p.uB * p.uH), dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_classify(const ClassifyParams &p, bool wide, hipStream_t stream) {
    if (wide) {
        const dim3 grid((p.Sk + kWideCols - 1) / kWideCols, p.nQ, p.uB * p.uH);
        hipLaunchKernelGGL(classify_wide_kernel, grid, dim3(256), 0, stream, p);
    } else {
        const int64_t total = (int64_t)p.uB * p.uH * p.nQ * p.nK;
        hipLaunchKernelGGL(classify_generic_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p);
    }
    return hipGetLastError();
}

hipError_t launch_compact(const CompactParams &p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.oB * p.oH * p.nQ;
    hipLaunchKernelGGL(compact_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace sa
