// Backward pass of the block-sparse attention on gfx950 (MI355X): dQ, dK, dV from dO.
//
// The reference has no backward pass ("Backwards pass + decode kernels", README.md:65); the function differentiated
// is its forward, o = softmax(q k^T * scale + (mask ? 0 : -inf)) v (sparse_attn_kernel.py:149-185), with the row
// log-sum-exp the forward hands out (FwdParams::lse):
//     P = exp(S - lse),  dV = P^T dO,  dP = dO V^T,  dS = P o (dP - rowsum(dO o O)),  dQ = scale dS K,  dK = scale dS^T Q.
//
// One kernel serves the three gradients.  A workgroup owns a tile of 128 RESIDENT rows (queries for dQ, keys for dK
// and dV), 32 per wave, whose operands stay in registers, and walks the list of 64-row tiles of the STREAMED side
// (keys for dQ, queries for dK/dV) that the mask leaves for it: FULL tiles, then PARTIAL ones, as in the forward; for
// dK/dV the lists are those of the transposed mask.  Per 32 streamed rows:
//     S^T  = Y . X^T        Y streamed (K | Q | Q), X resident and pre-scaled (Q | K | K)       -> P^T = exp2(S^T - L)
//     dP^T = Z . G^T        Z streamed (V | dO | -), G resident (dO | V | -)                    -> dS^T = P^T o (dP^T - Delta)
//     acc^T += Y^T . dS^T   (dQ, dK)      or      acc^T += Z^T . P^T   (dV)
// L and Delta belong to the query: per lane when queries are resident, per score register (read from LDS) when they
// are streamed.  Streamed chunks of 64 rows arrive by direct loads global -> LDS in two stages, one barrier per chunk.
// A chunk buffer is read both ways - row-wise as MFMA A operand (ds_read_b128) and transposed (ds_read_b64_tr_b16) -
// so the 16-byte pieces of a row are swizzled with a function of the row that keeps both patterns free of bank
// conflicts (bwd_swizzle).
#include "fwd_common.h"

namespace sa {

namespace {

constexpr int kBwdListCap = 2048;  // list entries kept in LDS (streamed length up to 131072)

// XOR applied to the 16-byte piece index of LDS row `row`.
// D = 128 (16 pieces per row, rows 256 bytes apart): bits 0-1 and 2-3 of the row swapped.  16 consecutive rows get 16
// different values (row-wise reads of one piece), and the 4 rows of a transposing read get 4 different 64-byte groups.
// D = 64 (8 pieces, rows 128 bytes apart, so rows of equal parity share their banks): row bit 1 goes to bit 2, bits
// 3 and 2 to bits 1 and 0.  The 8 rows of equal parity among 16 get 8 different values, and the two rows of equal
// parity in a transposing read get different 64-byte groups.
template <int D>
__device__ __forceinline__ int bwd_swizzle(int row) {
    if constexpr (D == 128) return ((row & 3) << 2) | ((row >> 2) & 3);
    else return (((row >> 1) & 1) << 2) | (((row >> 3) & 1) << 1) | ((row >> 2) & 1);
}

// LANE_STATS: queries are the resident side (dQ).  OUT_P: the output product takes P and Z (dV) instead of dS and Y.
template <int DT, int D, bool LANE_STATS, bool OUT_P>
__global__ __launch_bounds__(256, 2) void sparse_bwd_kernel(const BwdParams p) {
    using E = Elem<DT>;
    static_assert(D == 128 || D == 64, "head dim");
    constexpr int ROWB = D * 2;
    constexpr int CBUF = 64 * ROWB;  // one streamed chunk of one tensor
    constexpr int NC = D / 16, NDB = D / 32;
    constexpr int PPR = ROWB / 16;   // 16-byte pieces per row
    constexpr int RPI = 64 / PPR;    // rows per wave-wide direct load (1 KiB)
    constexpr int NLD = 16 / RPI;    // direct loads per wave per chunk and tensor
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    // [Y stage 0,1][Z stage 0,1][stats stage 0,1: 64 L then 64 Delta floats][list]
    constexpr int STAT0 = 4 * CBUF;
    constexpr int LIST0 = STAT0 + 2 * 512;
    int *const ent = reinterpret_cast<int *>(smem + LIST0);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    // Workgroup -> (plane, resident tile) as in sparse_fwd_kernel: consecutive workgroup ids go to the 8 XCDs in turn,
    // so each XCD gets a contiguous range of the plane-major order (the tiles that share K/V or Q/dO meet in one L2),
    // planes two at a time with their tiles interleaved, the tile that is heaviest under causal-like masks first
    // (the last queries, the first keys: p.first_tile_first).
    const int total = gridDim.x, per = total >> 3;
    int lin = blockIdx.x;
    if (lin < (per << 3)) lin = (lin & 7) * per + (lin >> 3);
    int pair = lin / (2 * p.nR);
    const int pr = lin - pair * 2 * p.nR;
    if (((p.B * p.H) & 15) == 0) {  // every eighth pair of planes to an XCD: masks that differ per batch element load them alike
        const int ppx = (p.B * p.H) >> 4;
        const int x = pair / ppx;
        pair = (pair - x * ppx) * 8 + x;
    }
    const bool paired = 2 * pair + 1 < p.B * p.H;
    const int bh = 2 * pair + (paired ? (pr & 1) : 0);
    const int order = paired ? (pr >> 1) : pr;
    const int rt = p.first_tile_first ? order : p.nR - 1 - order;  // resident tile
    const int b = bh / p.H, h = bh - b * p.H;
    const int rrow = rt * 128 + wave * 32 + l32;

    const uint16_t *ybase = p.y + b * p.ys[0] + h * p.ys[1];
    const uint16_t *zbase = p.z + b * p.zs[0] + h * p.zs[1];
    const int32_t *fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + rt * p.fis[2];
    const int32_t *pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + rt * p.pis[2];
    // Counts and tile indices are clamped to the nS streamed tiles there are (the reference guards every K/V and mask
    // load with kv_offset < SEQLEN_K, sparse_attn_kernel.py:35,39,60): stale or foreign metadata then gives wrong
    // numbers, never an access outside the tensors or past the list's LDS copy (nS <= kBwdListCap, checked by the host).
    const int F = min(max(p.full_lens[b * p.fls[0] + h * p.fls[1] + rt * p.fls[2]], 0), p.nS);
    const int T = F + min(max(p.part_lens[b * p.pls[0] + h * p.pls[1] + rt * p.pls[2]], 0), p.nS - F);  // chunks = list entries
    const uint8_t *mrow = p.mask + b * p.ms[0] + h * p.ms[1] + (int64_t)rrow * p.mrs;
    // this lane's row in a packed tile: 8 bytes per row, 1024 per tile, nS tiles per resident tile
    const uint8_t *prow = p.packed + b * p.pks[0] + h * p.pks[1] + (int64_t)rt * p.nS * 1024 + (wave * 32 + l32) * 8;
    const float *statL = p.stat_l + b * p.sts[0] + h * p.sts[1];
    const float *statD = p.stat_d + b * p.sts[0] + h * p.sts[1];
    // bytes from a query's L to its Delta (both live in one workspace, less than 4 GiB apart)
    const uint32_t stat_gap = (uint32_t)((const uint8_t *)p.stat_d - (const uint8_t *)p.stat_l);

    // resident operands: lane (l32, hh) keeps d = 16c + 8hh .. +7 of its row; X carries the softmax scale / ln 2
    u32x4 xf[NC], gf[OUT_P ? 1 : NC];
    {
        const uint16_t *xp = p.x + b * p.xs[0] + h * p.xs[1] + (int64_t)rrow * p.xs[2] + 8 * hh;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            xf[c] = *(const u32x4 *)(xp + 16 * c);
#pragma unroll
            for (int e = 0; e < 4; e++) xf[c][e] = E::scale2(xf[c][e], p.scale);
        }
        if constexpr (!OUT_P) {
            const uint16_t *gp = p.g + b * p.gs[0] + h * p.gs[1] + (int64_t)rrow * p.gs[2] + 8 * hh;
#pragma unroll
            for (int c = 0; c < NC; c++) gf[c] = *(const u32x4 *)(gp + 16 * c);
        }
    }
    float laneL = 0.f, laneD = 0.f;
    if constexpr (LANE_STATS) {
        laneL = statL[(int64_t)rrow * p.sts[2]];
        laneD = statD[(int64_t)rrow * p.sts[2]];
    }
    f32x16 acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.f;

    // LDS offsets inside a chunk buffer: row-wise operand reads (row 32kb + l32, piece 2c + hh) and transposing
    // reads (rows 16kc + 4hh + j and + 8 of a 32-row block, 32-wide d block db), both through bwd_swizzle
    int noff[NC];
#pragma unroll
    for (int c = 0; c < NC; c++) noff[c] = l32 * ROWB + 16 * ((2 * c + hh) ^ bwd_swizzle<D>(l32));
    int toff[2][NDB];
    {
        const int j = (lane & 15) >> 2;
        const int x = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int row = 4 * hh + j + 8 * u;
#pragma unroll
            for (int db = 0; db < NDB; db++) {
                // bwd_swizzle of row 16kc + 4hh + j + 8u, split into its 64-byte-group and its piece-in-group part
                const int grp = D == 128 ? j : (j >> 1), pc = D == 128 ? ((hh + 2 * u) & 3) : ((u << 1) | hh);
                toff[u][db] = row * ROWB + 64 * (db ^ grp) + 16 * (x ^ pc) + 8 * (lane & 1);
            }
        }
    }
    // direct loads: load i of this wave fills rows RPI (4i + wave) .. + RPI - 1 of the chunk; the lane writes LDS
    // piece lane % PPR of its row and therefore fetches the swizzled source piece
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const SA_LDS uint8_t *)smem);
    uint32_t ld_yoff[NLD], ld_zoff[NLD];
#pragma unroll
    for (int i = 0; i < NLD; i++) {
        const int r = RPI * (4 * i + wave_u) + lane / PPR;
        const int piece = (lane % PPR) ^ bwd_swizzle<D>(r);
        ld_yoff[i] = (uint32_t)((r * p.ys[2] + 8 * piece) * 2);
        ld_zoff[i] = (uint32_t)((r * p.zs[2] + 8 * piece) * 2);
    }

    // the tile's list (FULL entries, then PARTIAL ones) as first streamed rows
    for (int e = tid; e < T; e += 256) {
        const int idx = e < F ? fid[(int64_t)e * p.fis[3]] : pid[(int64_t)(e - F) * p.pis[3]];
        ent[e] = min(max(idx, 0), p.nS - 1) << 6;
    }
    __syncthreads();

    // everything chunk t needs from memory, into stage st
    auto issue = [&](int t, int st, uint32_t(&mk)[8]) {
        const int col = __builtin_amdgcn_readfirstlane(ent[t]);
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const uint32_t dst = 1024 * (4 * i + wave_u);  // RPI rows per load
            dma16(ybase + (int64_t)col * p.ys[2], ld_yoff[i], lds0 + st * CBUF + dst);
            dma16(zbase + (int64_t)col * p.zs[2], ld_zoff[i], lds0 + (2 + st) * CBUF + dst);
        }
        if constexpr (!LANE_STATS) {
            if (wave_u == 0 && lane < 32) {  // 64 L values, then 64 Delta values, 16 bytes per lane (row stride 1)
                const uint32_t off = (lane < 16 ? 0u : stat_gap) + 16u * (lane & 15);
                dma16(statL + col, off, lds0 + STAT0 + st * 512);
            }
        }
        if (t >= F && p.packed != nullptr) {  // the row's 64 bits of the tile in slot t - F
            const u32x2 w = *(const u32x2 *)(prow + (int64_t)(t - F) * 1024);
            mk[0] = w.x;
            mk[1] = w.y;
#pragma unroll
            for (int i = 2; i < 8; i++) mk[i] = 0u;
        } else if (t >= F) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int64_t cc = col + 32 * kb + 8 * g + 4 * hh;
                    if (p.mask_vec4) {
                        mk[4 * kb + g] = *(const uint32_t *)(mrow + cc);
                    } else {
                        const uint8_t *m0 = mrow + cc * p.mcs;
                        mk[4 * kb + g] = (uint32_t)m0[0] | ((uint32_t)m0[p.mcs] << 8) | ((uint32_t)m0[2 * p.mcs] << 16) |
                                         ((uint32_t)m0[3 * p.mcs] << 24);
                    }
                }
        }
    };

    auto compute = [&](int t, int st, const uint32_t(&mk)[8]) {
        const uint8_t *yb = smem + st * CBUF, *zb = smem + (2 + st) * CBUF;
        const float *sl = reinterpret_cast<const float *>(smem + STAT0 + st * 512);
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            f32x16 s, dp;
#pragma unroll
            for (int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; c++) s = E::mfma(*(const u32x4 *)(yb + 32 * kb * ROWB + noff[c]), xf[c], s);
            if constexpr (!OUT_P) {
#pragma unroll
                for (int i = 0; i < 16; i++) dp[i] = 0.f;
#pragma unroll
                for (int c = 0; c < NC; c++) dp = E::mfma(*(const u32x4 *)(zb + 32 * kb * ROWB + noff[c]), gf[c], dp);
            }
            if (t >= F) {
                // w: bit 8g + jj says whether this lane's entry (streamed row 32kb + 8g + 4hh + jj) attends
                uint32_t w;
                if (p.packed != nullptr) {  // bit k of the packed word: streamed row 32kb + k
                    w = mk[kb] >> (4 * hh);
                } else {  // one byte per entry: the non-zero bytes of each dword become four bits
                    w = 0u;
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const uint32_t m = mk[4 * kb + g];
                        const uint32_t nz = ((((m & 0x7f7f7f7fu) + 0x7f7f7f7fu) | m) >> 7) & 0x01010101u;
                        w |= ((nz * 0x01020408u) >> 24) << (8 * g);
                    }
                }
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int jj = 0; jj < 4; jj++)
                        if (((w >> (8 * g + jj)) & 1u) == 0u) s[4 * g + jj] = kNegInf;
            }
            // P^T = exp2(S^T - L) and, unless OUT_P, dS^T = P^T o (dP^T - Delta); rounded to the input type
            uint32_t pw[8];
#pragma unroll
            for (int g = 0; g < 4; g++) {
                f32x4 L4, D4;
                if constexpr (LANE_STATS) {
                    L4 = f32x4{laneL, laneL, laneL, laneL};
                    D4 = f32x4{laneD, laneD, laneD, laneD};
                } else {
                    L4 = *(const f32x4 *)(sl + 32 * kb + 8 * g + 4 * hh);
                    D4 = *(const f32x4 *)(sl + 64 + 32 * kb + 8 * g + 4 * hh);
                }
                float w[4];
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const float pr = __builtin_amdgcn_exp2f(s[4 * g + jj] - L4[jj]);
                    w[jj] = OUT_P ? pr : pr * (dp[4 * g + jj] - D4[jj]);
                }
                pw[2 * g] = E::pack2(w[0], w[1]);
                pw[2 * g + 1] = E::pack2(w[2], w[3]);
            }
            const uint8_t *tb = (OUT_P ? zb : yb) + 32 * kb * ROWB;
#pragma unroll
            for (int kc = 0; kc < 2; kc++) {
                const u32x4 pk4 = u32x4{pw[4 * kc], pw[4 * kc + 1], pw[4 * kc + 2], pw[4 * kc + 3]};
#pragma unroll
                for (int db = 0; db < NDB; db++) {
                    const u32x2 lo = E::tr_read(tb + 16 * kc * ROWB + toff[0][db]);
                    const u32x2 hi = E::tr_read(tb + 16 * kc * ROWB + toff[1][db]);
                    acc[db] = E::mfma(u32x4{lo.x, lo.y, hi.x, hi.y}, pk4, acc[db]);
                }
            }
        }
    };

    {
        uint32_t mk[2][8];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 8; i++) mk[j][i] = 0u;
        if (T > 0) issue(0, 0, mk[0]);
        for (int t0 = 0; t0 < T; t0 += 2) {
            static_for<2>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int t = t0 + j;
                if (t >= T) return;
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // own pieces of chunk t and its mask words
#pragma unroll
                for (int i = 0; i < 8; i++) asm volatile("" ::"v"(mk[j][i]));
                __syncthreads();  // everyone's pieces; and everyone is done with the other stage
                if (t + 1 < T) issue(t + 1, j ^ 1, mk[j ^ 1]);
                compute(t, j, mk[j]);
            });
        }
    }

    // out = acc * out_scale; acc holds the transposed tile: lane (row l32, hh), register 4g + jj of block db is
    // d = 32 db + 8g + 4hh + jj.  A lane's 8-byte pieces would make every store instruction touch 32 rows, so the
    // wave's 32 rows go through a private slice of the (now idle) chunk buffers, rows 16 bytes apart from the banks'
    // period, and leave as whole rows, 16 bytes per lane.
    __syncthreads();  // every wave is done with the chunk buffers
    constexpr int OROW = ROWB + 16;
    static_assert(4 * 32 * OROW <= 4 * CBUF, "the rows of the four waves fit the chunk buffers");
    uint8_t *const ob = smem + wave * 32 * OROW;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const u32x2 w = {E::pack2(acc[db][4 * g] * p.out_scale, acc[db][4 * g + 1] * p.out_scale),
                             E::pack2(acc[db][4 * g + 2] * p.out_scale, acc[db][4 * g + 3] * p.out_scale)};
            *(u32x2 *)(ob + l32 * OROW + 2 * (32 * db + 8 * g + 4 * hh)) = w;
        }
    constexpr int PPR_O = ROWB / 16;  // 16-byte pieces per row
    uint16_t *const o0 = p.out + b * p.outs[0] + h * p.outs[1] + (int64_t)(rt * 128 + wave * 32) * p.outs[2];
#pragma unroll
    for (int i = 0; i < 32 * PPR_O / 64; i++) {
        const int idx = 64 * i + lane, r = idx / PPR_O, pc = idx % PPR_O;
        const u32x4 x = *(const u32x4 *)(ob + r * OROW + 16 * pc);
        // (written once, whole rows: a streaming store leaves the streamed operands' lines in L2 alone)
        __builtin_nontemporal_store(x, (u32x4 *)(o0 + (int64_t)r * p.outs[2] + 8 * pc));
    }
}

// Per query row: Delta = sum_d dO o O, and L = lse / ln 2 (+inf for rows that attended to nothing, so that their
// P = exp2(S - L) is 0).  D/8 lanes per row, 8 elements each.
template <int DT, int D>
__global__ __launch_bounds__(256) void bwd_prepare_kernel(const BwdPrepParams p) {
    constexpr int LPR = D / 8;  // lanes per row
    const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
    const int part = threadIdx.x % LPR;
    if (row >= (int64_t)p.B * p.H * p.Sq) return;
    const int q = (int)(row % p.Sq);
    const int bh = (int)(row / p.Sq);
    const int b = bh / p.H, h = bh - b * p.H;
    // (read once, whole rows: streaming loads, which this device serves faster than loads that keep their lines in L2)
    const u32x4 a = __builtin_nontemporal_load((const u32x4 *)(p.o + b * p.os[0] + h * p.os[1] + (int64_t)q * p.os[2] + 8 * part));
    const u32x4 g = __builtin_nontemporal_load((const u32x4 *)(p.d_o + b * p.dos[0] + h * p.dos[1] + (int64_t)q * p.dos[2] + 8 * part));
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const uint32_t ae = a[e], ge = g[e];  // (a bit cast applied to the vector element itself reads element 0)
        if constexpr (DT == 0) {
            sum += __uint_as_float(ae << 16) * __uint_as_float(ge << 16);
            sum += __uint_as_float(ae & 0xffff0000u) * __uint_as_float(ge & 0xffff0000u);
        } else {
            const f16x2 x = __builtin_bit_cast(f16x2, ae), y = __builtin_bit_cast(f16x2, ge);
            sum += (float)x.x * (float)y.x + (float)x.y * (float)y.y;
        }
    }
#pragma unroll
    for (int m = LPR / 2; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, LPR);
    if (part == 0) {
        const float lse = p.lse[b * p.ls[0] + h * p.ls[1] + (int64_t)q * p.ls[2]];
        p.stat_l[row] = lse == kNegInf ? __builtin_inff() : lse * 1.44269504089f;
        p.stat_d[row] = sum;
    }
}

template <int DT, int D, bool LANE_STATS, bool OUT_P>
hipError_t launch_bwd_one(const BwdParams &p, hipStream_t stream) {
    constexpr int smem = 4 * 64 * D * 2 + 2 * 512 + kBwdListCap * 4;
    auto kern = sparse_bwd_kernel<DT, D, LANE_STATS, OUT_P>;
    static unsigned long long attr_done = 0;
    if (const hipError_t e0 = allow_dynamic_smem(kern, smem, attr_done); e0 != hipSuccess) return e0;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.nR * (unsigned)p.B * (unsigned)p.H), dim3(256), smem, stream, p);
    return hipGetLastError();
}

template <int DT, int D>
hipError_t launch_bwd_pass(const BwdParams &p, bool lane_stats, bool out_p, hipStream_t stream) {
    if (lane_stats) return launch_bwd_one<DT, D, true, false>(p, stream);
    return out_p ? launch_bwd_one<DT, D, false, true>(p, stream) : launch_bwd_one<DT, D, false, false>(p, stream);
}

template <int DT, int D>
hipError_t launch_prepare_one(const BwdPrepParams &p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.B * p.H * p.Sq;
    constexpr int RPB = 256 / (D / 8);  // rows per workgroup
    hipLaunchKernelGGL((bwd_prepare_kernel<DT, D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_bwd(const BwdParams &p, int dtype, int D, bool lane_stats, bool out_p, hipStream_t stream) {
    if (dtype == 0 && D == 128) return launch_bwd_pass<0, 128>(p, lane_stats, out_p, stream);
    if (dtype == 0 && D == 64) return launch_bwd_pass<0, 64>(p, lane_stats, out_p, stream);
    if (dtype == 1 && D == 128) return launch_bwd_pass<1, 128>(p, lane_stats, out_p, stream);
    if (dtype == 1 && D == 64) return launch_bwd_pass<1, 64>(p, lane_stats, out_p, stream);
    return hipErrorInvalidValue;
}

hipError_t launch_bwd_prepare(const BwdPrepParams &p, int dtype, int D, hipStream_t stream) {
    if (dtype == 0 && D == 128) return launch_prepare_one<0, 128>(p, stream);
    if (dtype == 0 && D == 64) return launch_prepare_one<0, 64>(p, stream);
    if (dtype == 1 && D == 128) return launch_prepare_one<1, 128>(p, stream);
    if (dtype == 1 && D == 64) return launch_prepare_one<1, 64>(p, stream);
    return hipErrorInvalidValue;
}

}  // namespace sa
