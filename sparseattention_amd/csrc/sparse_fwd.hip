// Block-sparse flash-attention forward for gfx950 (MI355X).
//
// Replaces the Triton kernels sparse_attention_kernel / _sparse_inner
// (sparseattention/sparse_attn_kernel.py:74-146 and :10-63).
//
// Work decomposition
//   One workgroup per (Q tile of BQ rows, b, h); NW = BQ/32 waves, wave w owns query rows
//   [32w, 32w+32) of the tile.  The listed KV tiles of that Q tile (all FULL tiles, then all PARTIAL
//   tiles, as the reference orders them) form one stream that is consumed in chunks of 64 key rows:
//   BK=16 -> 4 list entries per chunk, BK=32 -> 2, BK>=64 -> BK/64 chunks per entry.  Softmax is
//   row-wise, so gathered tiles that are not neighbours in K can share a chunk.
//
// Register layout (v_mfma_f32_32x32x16_{bf16,f16}; lane = 32*hh + l32)
//   S^T = K . Q^T   A = K rows (kv = l32 of each 32-row block), B = Q^T (q = l32), contraction over d;
//                   the result leaves lane (l32, hh) holding query l32 and keys 8g+4hh+j
//                   (g,j in 0..3, register 4g+j) of each 32-key block.  Every lane owns one query
//                   row, so row max / row sum are in-lane reductions plus one exchange with lane^32.
//   O^T = V^T . P^T A = V^T (d = l32 of each 32-wide block), B = P^T (q = l32), contraction over keys.
//                   Registers 8c..8c+7 of a S^T block are exactly the B operand of the c-th
//                   16-key MFMA step, so P never leaves registers; the matching A operand is read
//                   from row-major V in LDS with the transposing ds_read_b64_tr_b16.
//
// LDS: two buffers each for K and V (64 rows per buffer); row pitch D*2+16 bytes for K (conflict-free
// 16-byte reads down a column of rows) and D*2+64 for V (the four rows of a transposing read fall in
// different bank quarters).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace sa {

namespace {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

#define SA_LDS __attribute__((address_space(3)))

template <int DT>
struct Elem;

template <>
struct Elem<0> {  // bf16
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        const f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    static __device__ __forceinline__ u32x2 tr_read(const uint8_t *lds_ptr) {
        return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((SA_LDS bf16x4 *)lds_ptr));
    }
};

template <>
struct Elem<1> {  // fp16
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        const f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
    static __device__ __forceinline__ u32x2 tr_read(const uint8_t *lds_ptr) {
        // the transposing read only moves 16-bit lanes around, so the bf16 flavour serves fp16 too
        return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((SA_LDS bf16x4 *)lds_ptr));
    }
};

// Exchange a value between lane and lane^32 and combine: returns op(x[lane], x[lane^32]) in all lanes.
__device__ __forceinline__ float half_swap_max(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

constexpr float kNegInf = -__builtin_inff();

// MODE 0: BK = 16, MODE 1: BK = 32, MODE 2: BK >= 64 (runtime log2 in p.lbk).
template <int DT, int D, int NW, int MODE>
__global__ __launch_bounds__(NW * 64, NW >= 4 ? 2 : 1) void sparse_fwd_kernel(const FwdParams p) {
    using E = Elem<DT>;
    constexpr int NT = NW * 64;          // threads
    constexpr int DV = D / 8;            // 16-byte pieces per K/V row
    constexpr int RPP = NT / DV;         // rows staged per pass of the whole workgroup
    constexpr int NL = 64 / RPP;         // passes per 64-row chunk
    constexpr int KSTR = D * 2 + 16;     // LDS row pitch of K, bytes
    constexpr int VSTR = D * 2 + 64;     // LDS row pitch of V, bytes
    constexpr int KBUF = 64 * KSTR, VBUF = 64 * VSTR;
    constexpr int EPC = MODE == 0 ? 4 : (MODE == 1 ? 2 : 1);  // list entries per chunk
    constexpr int LBKC = MODE == 0 ? 4 : 5;                   // log2(BK) when MODE < 2
    static_assert(RPP >= 1 && 64 % RPP == 0, "staging layout");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t *const ksm = smem;
    uint8_t *const vsm = smem + 2 * KBUF;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;

    // Workgroup -> (b, h, Q tile).  Hardware hands consecutive workgroup ids to the 8 XCDs in turn; the
    // remap gives each XCD a contiguous range of the (b,h)-major order so that the Q tiles sharing one
    // K/V plane run on the XCD whose L2 already holds it.  Within a plane the last Q tile goes first
    // (under causal-like masks it has the longest list).
    const int total = gridDim.x, per = total >> 3;
    int lin = blockIdx.x;
    if (lin < (per << 3)) lin = (lin & 7) * per + (lin >> 3);
    const int bh = lin / p.nQ;
    const int qt = p.nQ - 1 - (lin - bh * p.nQ);
    const int b = bh / p.H, h = bh - b * p.H;

    const uint16_t *kbase = p.k + b * p.ks[0] + h * p.ks[1];
    const uint16_t *vbase = p.v + b * p.vs[0] + h * p.vs[1];
    const int qrow = qt * (NW * 32) + wave * 32 + l32;  // the query row this lane owns
    const uint8_t *mrow = p.mask + b * p.ms[0] + h * p.ms[1] + (int64_t)qrow * p.ms[2];

    const int32_t *fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + qt * p.fis[2];
    const int32_t *pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + qt * p.pis[2];
    const int F = p.full_lens[b * p.fls[0] + h * p.fls[1] + qt * p.fls[2]];
    const int P = p.part_lens[b * p.pls[0] + h * p.pls[1] + qt * p.pls[2]];
    const int NE = F + P;
    const int T = MODE == 2 ? (NE << (p.lbk - 6)) : ((NE + EPC - 1) / EPC);

    // Q^T operand: lane (l32, hh) keeps d = 16c + 8hh .. +7 of its query row for every 16-wide step c.
    u32x4 qf[D / 16];
    {
        const uint16_t *qp = p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2] + 8 * hh;
#pragma unroll
        for (int c = 0; c < D / 16; c++) qf[c] = *(const u32x4 *)(qp + 16 * c);
    }

    float m_run = kNegInf;  // running row maximum, in exp2 units (score * scale)
    float l_run = 0.f;      // running row sum over this lane's half of the keys
    f32x16 acc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.f;

    // First key column of every list entry in chunk t, plus which entries exist / are partial.
    auto chunk_entries = [&](int t, int(&col)[EPC], unsigned &valid, unsigned &part) {
        valid = 0u;
        part = 0u;
        if constexpr (MODE == 2) {
            const int sh = p.lbk - 6;
            const int e = t >> sh, sub = t & ((1 << sh) - 1);
            const int idx = e < F ? fid[(int64_t)e * p.fis[3]] : pid[(int64_t)(e - F) * p.pis[3]];
            col[0] = (idx << p.lbk) + (sub << 6);
            valid = 1u;
            part = e >= F ? 1u : 0u;
        } else {
#pragma unroll
            for (int j = 0; j < EPC; j++) {
                const int e = t * EPC + j;
                col[j] = 0;
                if (e < NE) {
                    const int idx = e < F ? fid[(int64_t)e * p.fis[3]] : pid[(int64_t)(e - F) * p.pis[3]];
                    col[j] = idx << LBKC;
                    valid |= 1u << j;
                    if (e >= F) part |= 1u << j;
                }
            }
        }
    };

    // Global -> registers for one chunk: thread covers row i*RPP + tid/DV, 16-byte piece tid%DV.
    auto load_chunk = [&](const int(&col)[EPC], unsigned valid, u32x4(&gk)[NL], u32x4(&gv)[NL]) {
        const int r0 = tid / DV, dv = tid % DV;
#pragma unroll
        for (int i = 0; i < NL; i++) {
            const int r = i * RPP + r0;
            int j = 0, within = r;
            if constexpr (MODE != 2) {
                j = r >> LBKC;
                within = r & ((1 << LBKC) - 1);
            }
            int c0 = col[0];
            bool ok = valid & 1u;
#pragma unroll
            for (int jj = 1; jj < EPC; jj++)
                if (j == jj) {
                    c0 = col[jj];
                    ok = (valid >> jj) & 1u;
                }
            const int64_t srow = c0 + within;
            if (ok) {
                gk[i] = *(const u32x4 *)(kbase + srow * p.ks[2] + dv * 8);
                gv[i] = *(const u32x4 *)(vbase + srow * p.vs[2] + dv * 8);
            } else {
                gk[i] = u32x4{0u, 0u, 0u, 0u};
                gv[i] = u32x4{0u, 0u, 0u, 0u};
            }
        }
    };
    auto store_chunk = [&](int buf, const u32x4(&gk)[NL], const u32x4(&gv)[NL]) {
        const int r0 = tid / DV, dv = tid % DV;
#pragma unroll
        for (int i = 0; i < NL; i++) {
            const int r = i * RPP + r0;
            *(u32x4 *)(ksm + buf * KBUF + r * KSTR + dv * 16) = gk[i];
            *(u32x4 *)(vsm + buf * VBUF + r * VSTR + dv * 16) = gv[i];
        }
    };

    auto compute = [&](int buf, const int(&col)[EPC], unsigned valid, unsigned part) {
        const uint8_t *kb_ = ksm + buf * KBUF;
        const uint8_t *vb_ = vsm + buf * VBUF;
        const bool special = part != 0u || valid != ((1u << EPC) - 1u);  // wave-uniform

        // Mask bytes for this lane's 4-key groups, fetched before the MFMAs so the latency overlaps.
        uint32_t mk[2][4];
        if (special) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    int j, within;
                    if constexpr (MODE == 0) {
                        j = 2 * kb + (g >> 1);
                        within = 8 * (g & 1) + 4 * hh;
                    } else if constexpr (MODE == 1) {
                        j = kb;
                        within = 8 * g + 4 * hh;
                    } else {
                        j = 0;
                        within = 32 * kb + 8 * g + 4 * hh;
                    }
                    uint32_t w = 0u;  // entry absent: all four keys masked out
                    if ((valid >> j) & 1u) {
                        w = 0x01010101u;  // FULL entry: all four keys attended
                        if ((part >> j) & 1u) {
                            const int64_t c = col[j] + within;
                            if (p.mask_vec4) {
                                w = *(const uint32_t *)(mrow + c);
                            } else {
                                w = (uint32_t)mrow[c * p.ms[3]] | ((uint32_t)mrow[(c + 1) * p.ms[3]] << 8) |
                                    ((uint32_t)mrow[(c + 2) * p.ms[3]] << 16) | ((uint32_t)mrow[(c + 3) * p.ms[3]] << 24);
                            }
                        }
                    }
                    mk[kb][g] = w;
                }
        }

        // S^T = K . Q^T
        f32x16 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) s[kb][i] = 0.f;
#pragma unroll
            for (int c = 0; c < D / 16; c++) {
                const u32x4 a = *(const u32x4 *)(kb_ + (32 * kb + l32) * KSTR + (16 * c + 8 * hh) * 2);
                s[kb] = E::mfma(a, qf[c], s[kb]);
            }
        }

        if (special) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (((mk[kb][g] >> (8 * j)) & 0xffu) == 0u) s[kb][4 * g + j] = kNegInf;
        }

        // Online softmax in exp2 units (sparse_attn_kernel.py:47-58).
        float mx = kNegInf;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[kb][i]);
        mx = half_swap_max(mx);
        const float m_new = fmaxf(m_run, mx * p.scale);
        const float m_ref = m_new == kNegInf ? 0.f : m_new;  // keeps exp2(-inf - -inf) out of the picture
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
        m_run = m_new;

        float rs = 0.f;
        u32x4 pb[2][2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int c = 0; c < 2; c++) {
                float pf[8];
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    pf[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][8 * c + i], p.scale, -m_ref));
                    rs += pf[i];
                }
                pb[kb][c] = u32x4{E::pack2(pf[0], pf[1]), E::pack2(pf[2], pf[3]), E::pack2(pf[4], pf[5]),
                                  E::pack2(pf[6], pf[7])};
            }
        l_run = l_run * alpha + rs;

#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[db][i] *= alpha;

        // O^T += V^T . P^T.  Transposing read: within each 16-lane group, lane t supplies the address of
        // 4 consecutive d of key row (t>>2) and receives the 4 key rows of d column t.
        const int tr_row = 4 * hh + ((lane & 15) >> 2);
        const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int kc = 0; kc < 4; kc++) {
                const uint8_t *vp = vb_ + (16 * kc + tr_row) * VSTR + (32 * db + tr_col) * 2;
                const u32x2 lo = E::tr_read(vp);
                const u32x2 hi = E::tr_read(vp + 8 * VSTR);
                acc[db] = E::mfma(u32x4{lo.x, lo.y, hi.x, hi.y}, pb[kc >> 1][kc & 1], acc[db]);
            }
    };

    if (T > 0) {
        int col_cur[EPC], col_nxt[EPC];
        unsigned valid_cur, part_cur, valid_nxt = 0u, part_nxt = 0u;
        u32x4 gk[NL], gv[NL];
        chunk_entries(0, col_cur, valid_cur, part_cur);
        load_chunk(col_cur, valid_cur, gk, gv);
        store_chunk(0, gk, gv);
        __syncthreads();
        for (int t = 0; t < T; t++) {
            const bool more = t + 1 < T;
            if (more) {
                chunk_entries(t + 1, col_nxt, valid_nxt, part_nxt);
                load_chunk(col_nxt, valid_nxt, gk, gv);
            }
            compute(t & 1, col_cur, valid_cur, part_cur);
            if (more) {
                store_chunk((t + 1) & 1, gk, gv);
#pragma unroll
                for (int j = 0; j < EPC; j++) col_cur[j] = col_nxt[j];
                valid_cur = valid_nxt;
                part_cur = part_nxt;
            }
            __syncthreads();
        }
    }

    // Epilogue: O = acc / l (sparse_attn_kernel.py:144); rows that attended to nothing give 0.
    const float l_tot = half_swap_sum(l_run);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    uint16_t *orow = p.o + b * p.os[0] + h * p.os[1] + (int64_t)qrow * p.os[2] + 4 * hh;
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const u32x2 w = {E::pack2(acc[db][4 * g] * inv, acc[db][4 * g + 1] * inv),
                             E::pack2(acc[db][4 * g + 2] * inv, acc[db][4 * g + 3] * inv)};
            *(u32x2 *)(orow + 32 * db + 8 * g) = w;
        }
}

template <int DT, int D, int NW, int MODE>
hipError_t launch_one(const FwdParams &p, hipStream_t stream) {
    constexpr int smem = 2 * 64 * (D * 2 + 16) + 2 * 64 * (D * 2 + 64);
    auto kern = sparse_fwd_kernel<DT, D, NW, MODE>;
    static bool attr_set = false;  // benign race: every thread sets the same value
    if (!attr_set) {
        const hipError_t e =
            hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const unsigned grid = (unsigned)p.nQ * (unsigned)p.B * (unsigned)p.H;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), smem, stream, p);
    return hipGetLastError();
}

template <int DT, int D, int NW>
hipError_t launch_mode(const FwdParams &p, hipStream_t stream) {
    if (p.BK == 16) return launch_one<DT, D, NW, 0>(p, stream);
    if (p.BK == 32) return launch_one<DT, D, NW, 1>(p, stream);
    return launch_one<DT, D, NW, 2>(p, stream);
}

template <int DT, int D>
hipError_t launch_bq(const FwdParams &p, int BQ, hipStream_t stream) {
    switch (BQ) {
        case 32: return launch_mode<DT, D, 1>(p, stream);
        case 64: return launch_mode<DT, D, 2>(p, stream);
        case 128: return launch_mode<DT, D, 4>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

template <int DT>
hipError_t launch_d(const FwdParams &p, int D, int BQ, hipStream_t stream) {
    switch (D) {
        case 64: return launch_bq<DT, 64>(p, BQ, stream);
        case 128: return launch_bq<DT, 128>(p, BQ, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_fwd(const FwdParams &p, int dtype, int D, int BQ, hipStream_t stream) {
    if (dtype == 0) return launch_d<0>(p, D, BQ, stream);
    if (dtype == 1) return launch_d<1>(p, D, BQ, stream);
    return hipErrorInvalidValue;
}

}  // namespace sa
