// Block-sparse attention forward for float32 q, k, v, o on the matrix unit (v_mfma_f32_32x32x2_f32), gfx950.
//
// Same function as sparse_fwd_kernel (the Triton kernels sparse_attention_kernel / _sparse_inner,
// sparseattention/sparse_attn_kernel.py:74-146 and :10-63, which take the element type of their inputs, :98-101, :145),
// in float32 throughout: nothing is rounded below float32, P enters the P.V product as it leaves the exponential.
// The plain vector-unit kernel of sparse_fwd_f32.hip stays for the sizes this one does not have.
//
// One workgroup per (Q tile of BQ = 32 NW rows, b, h); wave w owns query rows [32w, 32w+32).  The list (FULL tiles,
// then PARTIAL tiles) is consumed 32 keys at a time through two LDS stages of K and V rows, filled by direct loads
// global -> LDS one chunk ahead; the mask words of a chunk and the raw list travel the same way, so the loop holds no
// load the compiler knows of and one "s_waitcnt vmcnt(0)" per chunk covers everything.
//
// MFMA operands (lane = 32 hh + l32; every instruction contracts over 2 indices, one per lane half):
//   S^T = K . Q^T   A = K: lane (l32, hh) supplies key l32, d = (D/2) hh + c in step c (its half row is contiguous:
//                   one 16-byte LDS read feeds four steps); B = Q^T in registers with the same order of d.
//                   The result leaves lane (l32, hh) holding query l32 and keys 8g + 4hh + j in register 4g + j.
//   O^T = V^T . P^T step (g, j) contracts over the two keys 8g + j and 8g + 4 + j: B = P^T is register 4g + j of
//                   the scores as it stands (lane half hh holds key 8g + 4hh + j), A = V^T: lane (l32, hh) reads
//                   V[key 8g + 4hh + j][32 db + l32], 32 consecutive floats per lane half.
// LDS rows are unpadded (a direct load writes 64 lanes x 16 bytes contiguously); the 16-byte pieces of a row are
// XORed with the row's low four bits for K (the 16 rows read together fall into 16 bank groups) and with 8 * bit 2 of
// the row for V (the two lane halves read rows four apart: they fall into different halves of the banks).
//
// Online softmax in the reference's order (sparse_attn_kernel.py:53-58): row maximum, rescale, exponentials, row sum,
// accumulate; exp2 units with the scale folded into Q.  Rows that attend to nothing give 0.
#include "fwd_common.h"

namespace sa {

namespace {

constexpr int kF32ListCap = 1024;  // list entries kept in LDS (the launcher refuses longer rows of tiles)

__device__ __forceinline__ void f32_dma4(const void *lane_addr, uint32_t lds_addr) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %0, off"
        :
        : "v"(lane_addr), "s"(lds_addr)
        : "memory");
}
__device__ __forceinline__ void f32_dma16(const void *lane_addr, uint32_t lds_addr) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, off"
        :
        : "v"(lane_addr), "s"(lds_addr)
        : "memory");
}

// MODE 0: BK = 16 (two list entries per chunk), MODE 1: BK = 32, MODE 2: BK >= 64 (BK/32 chunks per entry).
// PK: mask entries of PARTIAL tiles from the bit-packed tiles; else from the bool mask (key stride 1, rows and base
// 16-byte aligned: checked by the launcher).
template <int D, int NW, int MODE, bool PK>
__global__ __launch_bounds__(NW * 64, NW >= 4 ? 2 : 1) void sparse_fwd_f32_mfma_kernel(const FwdParams p) {
    constexpr int ROWB = D * 4, PPR = ROWB / 16;  // bytes and 16-byte pieces per K/V row
    constexpr int KBUF = 32 * ROWB;               // one stage of K (or V): 32 rows
    constexpr int MBUF = NW * 1024;               // one stage of mask words: 64 lanes x 16 bytes per wave
    constexpr int OFF_V = 2 * KBUF, OFF_M = 4 * KBUF, OFF_L = OFF_M + 2 * MBUF;
    constexpr int EPC = MODE == 0 ? 2 : 1;
    constexpr int LBKC = MODE == 0 ? 4 : 5;
    constexpr int RPI = 1024 / ROWB;   // rows per direct load
    constexpr int NLD = 32 / RPI / NW; // direct loads per wave and chunk, each for K and for V
    static_assert(32 % (RPI * NW) == 0, "staging layout");

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    int *const ring = reinterpret_cast<int *>(smem + OFF_L);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // Workgroup -> (b, h, Q tile) as in sparse_fwd_kernel: the hardware hands consecutive workgroup ids to the 8 XCDs
    // in turn; the remap gives every XCD whole planes (so that the Q tiles sharing a K/V plane meet in one L2 and every
    // XCD gets the same mix of long and short lists), planes two at a time with their Q tiles interleaved, last Q tile
    // first.
    int b, h, qt;
    {
        const int total = gridDim.x, per = total >> 3;
        int lin = blockIdx.x;
        if (lin < (per << 3)) lin = (lin & 7) * per + (lin >> 3);
        int pair = lin / (2 * p.nQ);
        const int r = lin - pair * 2 * p.nQ;
        if (((p.B * p.H) & 15) == 0) {
            const int ppx = (p.B * p.H) >> 4;
            const int x = pair / ppx;
            pair = (pair - x * ppx) * 8 + x;
        }
        const bool paired = 2 * pair + 1 < p.B * p.H;
        const int bh = 2 * pair + (paired ? (r & 1) : 0);
        qt = p.nQ - 1 - (paired ? (r >> 1) : r);
        b = bh / p.H;
        h = bh - b * p.H;
    }
    const int qrow = qt * (NW * 32) + wave * 32 + l32;

    const float *const kbase = reinterpret_cast<const float *>(p.k) + b * p.ks[0] + h * p.ks[1];
    const float *const vbase = reinterpret_cast<const float *>(p.v) + b * p.vs[0] + h * p.vs[1];
    const int32_t *const fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + qt * p.fis[2];
    const int32_t *const pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + qt * p.pis[2];
    const int F = min(min(max(p.full_lens[b * p.fls[0] + h * p.fls[1] + qt * p.fls[2]], 0), p.nK), kF32ListCap);
    const int NE = F + min(min(max(p.part_lens[b * p.pls[0] + h * p.pls[1] + qt * p.pls[2]], 0), p.nK - F), kF32ListCap - F);
    const int T = MODE == 2 ? (NE << (p.lbk - 5)) : ((NE + EPC - 1) / EPC);
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const SA_LDS uint8_t *)smem);

    // Q^T operand: d = (D/2) hh + c for step c, scaled once (softmax scale / ln 2)
    float qf[D / 2];
    {
        const float *qp = reinterpret_cast<const float *>(p.q) + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2] + (D / 2) * hh;
#pragma unroll
        for (int c = 0; c < D / 2; c += 4) {
            const f32x4 x = *(const f32x4 *)(qp + c);
#pragma unroll
            for (int e = 0; e < 4; e++) qf[c + e] = x[e] * p.scale;
        }
    }

    // ---- per-lane constants ------------------------------------------------------------------------------------
    const int koff0 = l32 * ROWB + 16 * ((hh * (PPR / 2)) ^ (l32 & 15));  // read i of the row half: koff0 ^ (16 i)
    const int voff0 = 4 * hh * ROWB + 128 * hh + 16 * (l32 >> 2) + 4 * (l32 & 3);  // d block db: ^ (128 db); key: + row * ROWB
    // direct loads: load n (0 .. 32/RPI - 1) fills rows [RPI n, RPI n + RPI) of a stage, lane -> row n RPI + ld_r, LDS
    // piece ld_slot, which holds the source piece ld_slot ^ swizzle(row)
    const int ld_r = lane / PPR, ld_slot = lane % PPR;
    const int64_t ld_kbase = ((int64_t)ld_r * p.ks[2]) * 4, ld_vbase = ((int64_t)ld_r * p.vs[2]) * 4;
    const int64_t tile_bytes = (int64_t)(NW * 4) * p.BK;
    const uint8_t *const pbase = PK ? p.packed + b * p.pks[0] + h * p.pks[1] + (int64_t)qt * p.nK * tile_bytes : nullptr;
    const uint8_t *const mrow0 = PK ? nullptr : p.mask + b * p.ms[0] + h * p.ms[1] + (int64_t)(qt * (NW * 32)) * p.ms[2];

    struct Plan {
        int col[EPC];    // first key column of every entry of the chunk
        int slot[EPC];   // its slot among the PARTIAL entries (0 when it is not PARTIAL)
        unsigned flags;  // bit j: entry j exists; bit 4 + j: it is PARTIAL
    };
    auto plan_entry = [&](Plan &pl, int j, int e, int idx, int sub) {
        const bool exists = e < NE && (unsigned)idx < (unsigned)p.nK;
        const bool partial = exists && e >= F;
        pl.col[j] = exists ? ((MODE == 2 ? (idx << p.lbk) : (idx << LBKC)) + 32 * sub) : 0;
        pl.slot[j] = partial ? e - F : 0;
        pl.flags |= (exists ? 1u : 0u) << j | (partial ? 16u : 0u) << j;
    };
    auto plan_of = [&](int t, Plan &pl) {  // chunk t (t < T) from the LDS copy of the list
        pl.flags = 0u;
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            const int e = MODE == 2 ? (t >> (p.lbk - 5)) : t * EPC + j;
            const int sub = MODE == 2 ? (t & ((1 << (p.lbk - 5)) - 1)) : 0;
            plan_entry(pl, j, e, __builtin_amdgcn_readfirstlane(ring[min(e, kF32ListCap - 1)]), sub);
        }
    };
    // all direct loads of a chunk into stage `buf`
    auto stage_chunk = [&](int buf, const Plan &pl, int t) {
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const int n = NW * i + wave_u;  // this load's place in the chunk
            const int row0 = RPI * n;
            const int j = MODE == 0 ? (row0 >> 4) : 0;
            const int in_entry = MODE == 0 ? (row0 & 15) : row0;
            const int kswz = (row0 & 15) ^ 0, vswz = 8 * ((row0 >> 2) & 1);
            // (rows row0 .. row0 + RPI - 1 differ from row0 in bits that ld_r supplies: RPI <= 4 divides 16 and 4)
            const int col = (MODE == 0 && j ? pl.col[EPC - 1] : pl.col[0]) + in_entry;
            const uint8_t *ks_ = reinterpret_cast<const uint8_t *>(kbase + (int64_t)col * p.ks[2]) + ld_kbase +
                                 16 * (ld_slot ^ ((kswz | ld_r) & 15));
            const uint8_t *vs_ = reinterpret_cast<const uint8_t *>(vbase + (int64_t)col * p.vs[2]) + ld_vbase +
                                 16 * (ld_slot ^ (vswz ^ (8 * ((ld_r >> 2) & 1))));
            f32_dma16(ks_, lds0 + buf * KBUF + row0 * ROWB);
            f32_dma16(vs_, lds0 + OFF_V + buf * KBUF + row0 * ROWB);
        }
        // mask words of this wave's 32 rows
        const uint32_t mdst = lds0 + OFF_M + buf * MBUF + wave_u * 1024;
        if constexpr (PK) {
            // one dword per lane: the row's 32 bits of the chunk (BK = 16: lane half hh takes entry hh's dword that holds
            // rows 2r, 2r + 1)
            const int r = wave * 32 + l32;
            const uint8_t *src;
            if constexpr (MODE == 0) src = pbase + (int64_t)(hh ? pl.slot[EPC - 1] : pl.slot[0]) * tile_bytes + (r & ~1) * 2;
            else if constexpr (MODE == 1) src = pbase + (int64_t)pl.slot[0] * tile_bytes + r * 4;
            else src = pbase + (int64_t)pl.slot[0] * tile_bytes + (int64_t)r * (p.BK >> 3) + 4 * (t & ((1 << (p.lbk - 5)) - 1));
            f32_dma4(src, mdst);
        } else {
            // 16 mask bytes per lane: keys 16 hh .. 16 hh + 15 of the chunk (BK = 16: entry hh)
            const int col = MODE == 0 ? (hh ? pl.col[EPC - 1] : pl.col[0]) : pl.col[0] + 16 * hh;
            f32_dma16(mrow0 + (int64_t)(wave * 32 + l32) * p.ms[2] + col, mdst);
        }
    };

    // ---- state ----
    float m_i = kNegInf, l_i = 0.f;  // of this lane's query row; l_i over this lane half's keys only
    f32x16 acc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.f;

    if (T > 0) {
        // the list: wave w brings entries 64 w + lane, 64 (w + NW) + lane, ...
        for (int base = 64 * wave_u; base < NE; base += 64 * NW) {
            const int e = min(base + lane, NE - 1);
            const int32_t *src = e < F ? fid + (int64_t)e * p.fis[3] : pid + (int64_t)(e - F) * p.pis[3];
            f32_dma4(src, lds0 + OFF_L + 4 * base);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        Plan pl;
        plan_of(0, pl);
        stage_chunk(0, pl, 0);
        unsigned fl_cur = pl.flags;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();

        auto chunk = [&](auto buf_c, int tc) {
            constexpr int BUF = decltype(buf_c)::value;
            // the next chunk goes to the other stage (past the last chunk: the last one once more, harmless)
            Plan pn;
            const int tn = tc + 1 < T ? tc + 1 : T - 1;
            plan_of(tn, pn);
            stage_chunk(BUF ^ 1, pn, tn);

            // ---- S^T = K . Q^T ----
            const uint8_t *kb_ = smem + BUF * KBUF;
            f32x16 s;
#pragma unroll
            for (int i = 0; i < 16; i++) s[i] = 0.f;
            int kbo = koff0;
            asm volatile("" : "+v"(kbo));
#pragma unroll
            for (int i = 0; i < PPR / 2; i++) {
                const f32x4 kv = *(const f32x4 *)(kb_ + (kbo ^ (16 * i)));
#pragma unroll
                for (int e = 0; e < 4; e++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[e], qf[4 * i + e], s, 0, 0, 0);
            }

            // ---- mask (chunks with a PARTIAL or missing entry only) ----
            constexpr unsigned ALL = (1u << EPC) - 1u;
            if (fl_cur != ALL) {
                const uint8_t *mb_ = smem + OFF_M + BUF * MBUF + wave * 1024;
                if constexpr (PK) {
                    uint32_t w;
                    if constexpr (MODE == 0) {
                        const uint32_t a = *(const uint32_t *)(mb_ + 4 * l32), c2 = *(const uint32_t *)(mb_ + 128 + 4 * l32);
                        const int sh = 16 * (l32 & 1);
                        const uint32_t w0 = (fl_cur & 16u) ? ((a >> sh) & 0xffffu) : ((fl_cur & 1u) ? 0xffffu : 0u);
                        const uint32_t w1 = (fl_cur & 32u) ? ((c2 >> sh) & 0xffffu) : ((fl_cur & 2u) ? 0xffffu : 0u);
                        w = w0 | (w1 << 16);
                    } else {
                        const uint32_t a = *(const uint32_t *)(mb_ + 4 * l32);
                        w = (fl_cur & 16u) ? a : ((fl_cur & 1u) ? ~0u : 0u);
                    }
                    w >>= 4 * hh;
#pragma unroll
                    for (int g = 0; g < 4; g++)
#pragma unroll
                        for (int jj = 0; jj < 4; jj++)
                            if (((w >> (8 * g + jj)) & 1u) == 0u) s[4 * g + jj] = kNegInf;
                } else {
                    // the row's 32 bytes: keys 0..15 in the first 512 bytes of the wave's slice, 16..31 in the second
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const int j = MODE == 0 ? (g >> 1) : 0;  // list entry of this group of keys
                        const bool exists = (fl_cur >> j) & 1u, partial = (fl_cur >> (4 + j)) & 1u;
                        const uint32_t raw = *(const uint32_t *)(mb_ + 512 * (g >> 1) + 16 * l32 + 8 * (g & 1) + 4 * hh);
                        const uint32_t w = partial ? raw : (exists ? 0x01010101u : 0u);
#pragma unroll
                        for (int jj = 0; jj < 4; jj++)
                            if (((w >> (8 * jj)) & 0xffu) == 0u) s[4 * g + jj] = kNegInf;
                    }
                }
            }

            // ---- online softmax (sparse_attn_kernel.py:53-58) ----
            float mx = kNegInf;
#pragma unroll
            for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[i]);
            mx = half_swap_max(mx);
            const float m_new = fmaxf(m_i, mx);
            const float m_use = m_new == kNegInf ? 0.f : m_new;          // a row that has seen no key yet
            const float alpha = m_i == kNegInf ? 0.f : __builtin_amdgcn_exp2f(m_i - m_use);
            m_i = m_new;
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                s[i] = __builtin_amdgcn_exp2f(s[i] - m_use);
                psum += s[i];
            }
            l_i = l_i * alpha + psum;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0ull) {
#pragma unroll
                for (int db = 0; db < D / 32; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[db][i] *= alpha;
            }

            // ---- O^T += V^T . P^T ----
            const uint8_t *vb_ = smem + OFF_V + BUF * KBUF;
            int vbo = voff0;
            asm volatile("" : "+v"(vbo));
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int db = 0; db < D / 32; db++) {
                        const float vv = *(const float *)(vb_ + (8 * g + j) * ROWB + (vbo ^ (128 * db)));
                        acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv, s[4 * g + j], acc[db], 0, 0, 0);
                    }
            fl_cur = pn.flags;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next chunk has landed
            __syncthreads();                                   // and every wave is done with this one
        };
        for (int t = 0; t < T; t += 2) {
            chunk(std::integral_constant<int, 0>{}, t);
            if (t + 1 < T) chunk(std::integral_constant<int, 1>{}, t + 1);
        }
    }

    // ---- O = acc / l (sparse_attn_kernel.py:144); rows without a key give 0 ----
    {
        const uint32_t lu = __float_as_uint(l_i);
        const auto sw = __builtin_amdgcn_permlane32_swap(lu, lu, false, false);
        const float l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (p.lse != nullptr && hh == 0)
            p.lse[b * p.lses[0] + h * p.lses[1] + (int64_t)qrow * p.lses[2]] =
                l_tot > 0.f ? (m_i + __builtin_amdgcn_logf(l_tot)) * 0.69314718056f : kNegInf;
        float *orow = reinterpret_cast<float *>(p.o) + b * p.os[0] + h * p.os[1] + (int64_t)qrow * p.os[2] + 4 * hh;
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const f32x4 w = {acc[db][4 * g] * inv, acc[db][4 * g + 1] * inv, acc[db][4 * g + 2] * inv,
                                 acc[db][4 * g + 3] * inv};
                *(f32x4 *)(orow + 32 * db + 8 * g) = w;
            }
    }
}

template <int D, int NW, int MODE, bool PK>
hipError_t launch_one(const FwdParams &p, hipStream_t stream) {
    constexpr int smem = 4 * 32 * D * 4 + 2 * NW * 1024 + kF32ListCap * 4;
    auto kern = sparse_fwd_f32_mfma_kernel<D, NW, MODE, PK>;
    static unsigned long long attr_done = 0;
    if (const hipError_t e0 = allow_dynamic_smem(kern, smem, attr_done); e0 != hipSuccess) return e0;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.nQ * (unsigned)(p.B * p.H)), dim3(NW * 64), smem, stream, p);
    return hipGetLastError();
}

template <int D, int NW, bool PK>
hipError_t launch_mode(const FwdParams &p, hipStream_t stream) {
    if (p.BK == 16) return launch_one<D, NW, 0, PK>(p, stream);
    if (p.BK == 32) return launch_one<D, NW, 1, PK>(p, stream);
    return launch_one<D, NW, 2, PK>(p, stream);
}

template <int D, bool PK>
hipError_t launch_bq(const FwdParams &p, int BQ, hipStream_t stream) {
    switch (BQ) {
        case 32:
            // (a lone wave issues all 32 direct loads of a chunk itself; at D = 128 their addresses overflow the scalar
            // registers, and the vector-unit kernel serves that size)
            if constexpr (D > 64) return hipErrorInvalidValue;
            else return launch_mode<D, 1, PK>(p, stream);
        case 64: return launch_mode<D, 2, PK>(p, stream);
        case 128: return launch_mode<D, 4, PK>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

// Whether the matrix-unit kernel takes this float32 call: head dim 64 or 128, BLOCK_Q 32 (head dim 64 only) / 64 / 128, BLOCK_K a power of
// two >= 16 with at most kF32ListCap tiles per row, K/V rows 16-byte aligned, and either packed PARTIAL tiles or a
// bool mask whose rows can be fetched 16 bytes at a time.
bool fwd_f32_mfma_has(const FwdParams &p, int D, int BQ) {
    if ((D != 64 && D != 128) || (BQ != 32 && BQ != 64 && BQ != 128) || (D == 128 && BQ == 32)) return false;
    // (the kernels shift by p.lbk: it must be the logarithm of BLOCK_K)
    if (p.BK < 16 || (p.BK & (p.BK - 1)) || p.lbk < 4 || (1 << p.lbk) != p.BK || p.nK > kF32ListCap) return false;
    if (p.packed != nullptr) return true;
    return p.mask != nullptr && p.ms[3] == 1 && ((uintptr_t)p.mask & 15) == 0 && p.ms[0] % 16 == 0 && p.ms[1] % 16 == 0 &&
           p.ms[2] % 16 == 0;
}

hipError_t launch_fwd_f32_mfma(const FwdParams &p, int D, int BQ, hipStream_t stream) {
    if (!fwd_f32_mfma_has(p, D, BQ)) return hipErrorInvalidValue;
    if (p.packed != nullptr) return D == 64 ? launch_bq<64, true>(p, BQ, stream) : launch_bq<128, true>(p, BQ, stream);
    return D == 64 ? launch_bq<64, false>(p, BQ, stream) : launch_bq<128, false>(p, BQ, stream);
}

}  // namespace sa
