// Block-sparse attention for few query rows against a long K/V ("decode") on gfx950 (MI355X).
//
// Same function as the forward (sparse_attention with BLOCK_Q = Sq, sparseattention/sparse_attn_kernel.py:74-146,
// :10-63) for Sq <= 32: there is one Q tile per (b, h), so the forward's one-workgroup-per-Q-tile launch would
// leave the device empty and walk each list serially.  Here the list of a (b, h) is cut into `nsplit` ranges of
// 32-key chunks, one workgroup each; inside a workgroup the four waves take chunks in turn, every wave with a
// K/V stream of its own (no barrier in the loop) and its own online-softmax state for all query rows; waves, then
// workgroups, are merged by the usual rescaling.  The kernel is HBM-bound: every K and V byte of an executed tile is
// read once, 2 flop per byte and query row.
//
// Per chunk of 32 keys a wave
//   * holds K as MFMA operand straight from global memory (lane = key, 8 x 16 bytes of its row half; the
//     contraction order is permuted the same way in Q, which costs nothing),
//   * receives V in its own LDS stage by direct loads (swizzled rows, transposing reads: fwd_common.h),
//   * computes S^T = K . Q^T (32 keys x 32 query rows, rows past Sq are padding), masks PARTIAL tiles from the bool
//     mask, updates the lagging reference value, P = exp2(S^T - m), O^T += V^T . P^T, row sums by a small MFMA,
// while the loads of its next chunk (and the list index of the one after) are in flight.
#include "fwd_common.h"

namespace sa {

namespace {

constexpr int kDecodeWaves = 4;

template <int D>
constexpr int decode_smem_bytes() {
    constexpr int stream = kDecodeWaves * 2 * 32 * D * 2;         // per wave two V stages of 32 rows
    constexpr int merge = kDecodeWaves * 32 * (D + 2) * 4;        // per wave 32 rows of D + 2 floats
    return stream > merge ? stream : merge;
}

// Merge of partial rows: `n` parts of (D values, reference value m, row sum l) at `part + i * stride` floats; this
// thread owns NV consecutive values starting at d0.  Returns the merged reference value and sum, values in out[].
template <int NV>
__device__ __forceinline__ void merge_parts(const float *part, int n, int64_t stride, int D, int d0, float (&out)[NV],
                                            float &M, float &L) {
    M = kNegInf;
    for (int i = 0; i < n; i++) M = fmaxf(M, part[i * stride + D]);
    L = 0.f;
#pragma unroll
    for (int j = 0; j < NV; j++) out[j] = 0.f;
    if (M == kNegInf) return;  // no part saw an attended key
    for (int i = 0; i < n; i++) {
        const float *pp = part + i * stride;
        const float w = __builtin_amdgcn_exp2f(pp[D] - M);  // 0 for parts without an attended key (m = -inf)
        L += w * pp[D + 1];
#pragma unroll
        for (int j = 0; j < NV; j++) out[j] += w * pp[d0 + j];
    }
}

// PK: the mask entries of PARTIAL tiles come bit-packed from p.packed (sa_mask_pack_partial with BQ = Sq) instead of from
// the bool mask.  B16: BLOCK_K = 16, two list entries per chunk of 32 keys (else BLOCK_K >= 32, BLOCK_K/32 chunks per
// entry).
template <int DT, int D, bool PK, bool B16>
__global__ __launch_bounds__(kDecodeWaves * 64, 2) void sparse_decode_kernel(const DecodeParams p) {
    using E = Elem<DT>;
    constexpr int ROWB = D * 2;
    constexpr int VBUF = 32 * ROWB;   // one chunk of V
    constexpr int RPI = 1024 / ROWB;  // rows written by one wave-wide direct load
    constexpr int NLD = 32 / RPI;     // direct loads per chunk
    constexpr int PPR = ROWB / 16;
    constexpr int NC = D / 16, NDB = D / 32;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    const int split = blockIdx.x, bh = blockIdx.y;
    const int b = bh / p.H, h = bh - b * p.H;

    const uint16_t *kbase = p.k + b * p.ks[0] + h * p.ks[1];
    const uint16_t *vbase = p.v + b * p.vs[0] + h * p.vs[1];
    const int32_t *fid = p.full_ids + b * p.fis[0] + h * p.fis[1];
    const int32_t *pid = p.part_ids + b * p.pis[0] + h * p.pis[1];
    // Counts and tile indices are clamped to what Sk holds (the reference guards every K/V and mask load with
    // kv_offset < SEQLEN_K, sparse_attn_kernel.py:35,39,60): stale or foreign metadata then gives wrong numbers, never
    // an access outside K, V or the mask.
    const int nKt = p.Sk >> p.lbk;
    const int F = min(max(p.full_lens[b * p.fls[0] + h * p.fls[1]], 0), nKt);
    const int NE = F + min(max(p.part_lens[b * p.pls[0] + h * p.pls[1]], 0), nKt - F);
    constexpr int EPC = B16 ? 2 : 1;   // list entries per chunk
    const int sh = B16 ? 0 : p.lbk - 5;  // chunks per list entry, log2
    const int T = B16 ? (NE + 1) >> 1 : NE << sh;
    // this workgroup's chunks [t_lo, t_hi); this wave takes t_lo + wave, + 4, ...
    const int t_lo = (int)((unsigned)T * (unsigned)split / (unsigned)p.nsplit),
              t_hi = (int)((unsigned)T * (unsigned)(split + 1) / (unsigned)p.nsplit);  // T * nsplit < 2^31 (checked by the caller)
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);

    // query row of this lane (rows past Sq are padding: zero queries, row 0's mask, never stored)
    const bool live = l32 < p.Sq;
    const int qrow = live ? l32 : 0;
    const uint8_t *mrow = PK ? nullptr : p.mask + b * p.ms[0] + h * p.ms[1] + (int64_t)qrow * p.ms[2];
    // this row's bits in the packed tile of a PARTIAL slot: BK/8 bytes per row, Sq rows per tile
    const int64_t tile_bytes = (int64_t)p.Sq * (p.BK >> 3);
    const uint8_t *prow = PK ? p.packed + b * p.pks[0] + h * p.pks[1] + (int64_t)qrow * (p.BK >> 3) : nullptr;

    // Q^T operand, scaled once: lane (l32, hh) keeps d = (D/2) hh + 8c .. +7 of its row for step c (K uses the same
    // order, so each lane's K bytes are contiguous)
    u32x4 qf[NC];
    {
        const uint16_t *qp = p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2] + (D / 2) * hh;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            qf[c] = *(const u32x4 *)(qp + 8 * c);
#pragma unroll
            for (int e = 0; e < 4; e++) qf[c][e] = live ? E::scale2(qf[c][e], p.scale) : 0u;
        }
    }

    // online-softmax state of this lane's query row (see sparse_fwd_kernel.h); scores start from 0 here and the
    // reference value is subtracted before the exponential
    float m_ref = 0.f;
    float raise_above = -3.0e38f;
    f32x4 acc_l = {0.f, 0.f, 0.f, 0.f};
    const uint32_t sel1 = (((lane >> 4) ^ lane) & 1) == 0 ? E::ones4().x : 0u;
    const u32x4 sum_sel = {sel1, sel1, sel1, sel1};
    f32x16 acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.f;

    // V: transposing-read offsets and direct-load source offsets, as in sparse_fwd_kernel.h with one wave per chunk
    int voff[NDB];
    {
        const int tr_row = 4 * hh + ((lane & 15) >> 2);
        const int x = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
        const int sw = v_swizzle<D>(tr_row) >> 2;
#pragma unroll
        for (int db = 0; db < NDB; db++) voff[db] = tr_row * ROWB + 64 * (db ^ sw) + 16 * x + 8 * (lane & 1);
    }
    const int ld_r0 = lane / PPR, ld_slot = lane % PPR;
    uint32_t ld_voff[NLD];
#pragma unroll
    for (int i = 0; i < NLD; i++) {
        const int r = RPI * i + ld_r0;
        ld_voff[i] = (uint32_t)((r * p.vs[2] + 8 * (ld_slot ^ v_swizzle<D>(r))) * 2);
    }
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const SA_LDS uint8_t *)smem);
    uint8_t *const vmine = smem + wave_u * 2 * VBUF;
    const uint32_t vmine_lds = lds0 + wave_u * 2 * VBUF;
    const int64_t koff_lane = (int64_t)l32 * p.ks[2] + (D / 2) * hh;

    // list entries of chunk t (clamped into the row of tiles; an entry past the count reads as entry 0 and is masked out)
    auto idx_load = [&](int t, int(&idx)[EPC]) {
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            const int e0 = B16 ? 2 * t + j : (t >> sh);
            const int e = e0 < NE ? e0 : 0;
            const int v = e < F ? fid[(int64_t)e * p.fis[2]] : pid[(int64_t)(e - F) * p.pis[2]];
            idx[j] = min(max(v, 0), nKt - 1);
        }
    };
    // first key column of every entry of chunk t
    auto cols_of = [&](int t, const int(&idx)[EPC], int(&col)[EPC]) {
#pragma unroll
        for (int j = 0; j < EPC; j++)
            col[j] = (__builtin_amdgcn_readfirstlane(idx[j]) << p.lbk) + (B16 ? 0 : ((t & ((1 << sh) - 1)) << 5));
    };
    // what chunk t's entries are: bit j = entry j exists, bit 4 + j = it is PARTIAL
    auto flags_of = [&](int t) -> unsigned {
        unsigned f = 0u;
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            const int e = B16 ? 2 * t + j : (t >> sh);
            if (e < NE) f |= (1u << j) | (e >= F ? (16u << j) : 0u);
        }
        return f;
    };
    constexpr unsigned ALL = (1u << EPC) - 1u;
    constexpr int NMW = PK ? EPC : 4;  // mask words per lane and chunk
    // everything chunk t needs from memory: K into registers, V into LDS stage `st`, mask words if it has a PARTIAL entry
    auto issue = [&](int t, const int(&col)[EPC], int st, u32x4(&kf)[NC], uint32_t(&mk)[NMW]) {
        const int kcol = B16 ? ((l32 < 16 ? col[0] : col[EPC - 1]) - (l32 & 16)) : col[0];  // (+ l32: this lane's key)
        const uint16_t *kp = kbase + (int64_t)kcol * p.ks[2] + koff_lane;
#pragma unroll
        for (int c = 0; c < NC; c++) kf[c] = *(const u32x4 *)(kp + 8 * c);
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            // rows [RPI i, RPI i + RPI) of the chunk: with BLOCK_K = 16 the second half belongs to the second entry
            const int vcol = B16 ? (RPI * i < 16 ? col[0] : col[EPC - 1] - 16) : col[0];
            dma16<true>(vbase + (int64_t)vcol * p.vs[2], ld_voff[i], vmine_lds + st * VBUF + RPI * i * ROWB);
        }
        const unsigned fl = flags_of(t);
        if (fl >> 4) {
            if constexpr (PK) {
#pragma unroll
                for (int j = 0; j < EPC; j++) {
                    const int e = B16 ? 2 * t + j : (t >> sh);
                    const uint8_t *a = prow + (int64_t)((fl >> (4 + j)) & 1u ? e - F : 0) * tile_bytes;
                    if constexpr (B16) mk[j] = *(const uint16_t *)a;
                    else mk[j] = *(const uint32_t *)(a + 4 * (t & ((1 << sh) - 1)));
                }
            } else {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int64_t cc = (B16 ? (g < 2 ? col[0] + 8 * g : col[EPC - 1] + 8 * (g - 2)) : col[0] + 8 * g) + 4 * hh;
                    if (p.mask_vec4) {
                        mk[g] = *(const uint32_t *)(mrow + cc);
                    } else {
                        const uint8_t *m0 = mrow + cc * p.ms[3];
                        mk[g] = (uint32_t)m0[0] | ((uint32_t)m0[p.ms[3]] << 8) | ((uint32_t)m0[2 * p.ms[3]] << 16) |
                                ((uint32_t)m0[3 * p.ms[3]] << 24);
                    }
                }
            }
        }
    };
    // one chunk: scores, mask, softmax update, O^T += V^T . P^T
    auto compute = [&](int t, int st, const u32x4(&kf)[NC], const uint32_t(&mk)[NMW]) {
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; c++) s = E::mfma(kf[c], qf[c], s);
        const unsigned fl = flags_of(t);
        if (fl != ALL) {  // a PARTIAL entry, or (BLOCK_K = 16) a second entry past the end of the list
            if constexpr (PK) {
                // bit k of w: key k of the chunk; FULL entries count as all ones, missing ones as zero
                uint32_t w;
                if constexpr (B16) {
                    const uint32_t w0 = (fl & 16u) ? (mk[0] & 0xffffu) : ((fl & 1u) ? 0xffffu : 0u);
                    const uint32_t w1 = (fl & 32u) ? (mk[EPC - 1] & 0xffffu) : ((fl & 2u) ? 0xffffu : 0u);
                    w = w0 | (w1 << 16);
                } else {
                    w = (fl & 16u) ? mk[0] : ((fl & 1u) ? ~0u : 0u);
                }
                w >>= 4 * hh;  // this lane's keys are 8g + 4hh + jj
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int jj = 0; jj < 4; jj++)
                        if (((w >> (8 * g + jj)) & 1u) == 0u) s[4 * g + jj] = kNegInf;
            } else {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int j = B16 ? (g >> 1) : 0;
                    const uint32_t w = ((fl >> (4 + j)) & 1u) ? mk[g] : (((fl >> j) & 1u) ? 0x01010101u : 0u);
#pragma unroll
                    for (int jj = 0; jj < 4; jj++)
                        if (((w >> (8 * jj)) & 0xffu) == 0u) s[4 * g + jj] = kNegInf;
                }
            }
        }
        float mx = kNegInf;
#pragma unroll
        for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[i]);
        mx = half_swap_max(mx);
        const float rel = mx - m_ref;
        const bool raise = rel > raise_above;  // false for rows without an attended key so far (mx = -inf)
        if (__builtin_amdgcn_ballot_w64(raise) != 0ull) {
            const float a = raise ? (raise_above == kMaxSlack ? __builtin_amdgcn_exp2f(-rel) : 0.f) : 1.f;
            m_ref = raise ? mx : m_ref;
            raise_above = raise ? kMaxSlack : raise_above;
#pragma unroll
            for (int i = 0; i < 2; i++) acc_l[i] *= a;
#pragma unroll
            for (int db = 0; db < NDB; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[db][i] *= a;
        }
        uint32_t pw[8];
#pragma unroll
        for (int i = 0; i < 16; i += 2)
            pw[i >> 1] = E::pack2(__builtin_amdgcn_exp2f(s[i] - m_ref), __builtin_amdgcn_exp2f(s[i + 1] - m_ref));
        const uint8_t *vb_ = vmine + st * VBUF;
#pragma unroll
        for (int kc = 0; kc < 2; kc++) {
            const u32x4 pk4 = u32x4{pw[4 * kc], pw[4 * kc + 1], pw[4 * kc + 2], pw[4 * kc + 3]};
#pragma unroll
            for (int db = 0; db < NDB; db++) {
                const uint8_t *vp = vb_ + 16 * kc * ROWB + voff[db];
                const u32x2 lo = E::tr_read(vp), hi = E::tr_read(vp + 8 * ROWB);
                acc[db] = E::mfma(u32x4{lo.x, lo.y, hi.x, hi.y}, pk4, acc[db]);
            }
            acc_l = E::mfma16(sum_sel, pk4, acc_l);
        }
    };

    // ---- this wave's chunk stream: chunk t computes while chunk t + 4 loads and the index of t + 8 is fetched ----
    {
        u32x4 kf[2][NC];
        uint32_t mk[2][NMW];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int g = 0; g < NMW; g++) mk[j][g] = 0u;
        int t = t_lo + wave_u;
        int idxs[2][EPC] = {};  // idxs[s]: list indices of the chunk that goes into stage s next
        if (t < t_hi) {
            idx_load(t, idxs[0]);
            if (t + kDecodeWaves < t_hi) idx_load(t + kDecodeWaves, idxs[1]);
            int col[EPC];
            cols_of(t, idxs[0], col);
            issue(t, col, 0, kf[0], mk[0]);
        }
        for (; t < t_hi; t += 2 * kDecodeWaves) {
            static_for<2>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int tt = t + j * kDecodeWaves;  // the chunk in stage j
                if (tt >= t_hi) return;
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // chunk tt has landed, and the index of the next
                // (the compiler accounts for these loads here, where it costs nothing, instead of in front of their
                // first use, where its wait would take the direct loads of the next chunk along)
#pragma unroll
                for (int c = 0; c < NC; c++) asm volatile("" ::"v"(kf[j][c]));
#pragma unroll
                for (int g = 0; g < NMW; g++) asm volatile("" ::"v"(mk[j][g]));
#pragma unroll
                for (int e = 0; e < EPC; e++) asm volatile("" ::"v"(idxs[j ^ 1][e]));
                const int tn = tt + kDecodeWaves;
                if (tn < t_hi) {
                    int col_n[EPC];
                    cols_of(tn, idxs[j ^ 1], col_n);
                    if (tn + kDecodeWaves < t_hi) idx_load(tn + kDecodeWaves, idxs[j]);
                    issue(tn, col_n, j ^ 1, kf[j ^ 1], mk[j ^ 1]);
                }
                compute(tt, j, kf[j], mk[j]);
            });
        }
    }

    // ---- merge the four waves through LDS (the V stages are free once every wave is done) ----
    __syncthreads();
    float *const part = reinterpret_cast<float *>(smem);
    constexpr int PST = D + 2;  // floats per row of a part
    {
        float *mine = part + (wave * 32 + l32) * PST;
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int jj = 0; jj < 4; jj++) mine[32 * db + 8 * g + 4 * hh + jj] = acc[db][4 * g + jj];
        if (hh == 0) {
            mine[D] = raise_above == kMaxSlack ? m_ref : kNegInf;
            mine[D + 1] = l32 < 16 ? acc_l[0] : acc_l[1];
        }
    }
    __syncthreads();
    {
        constexpr int NV = D / 8;  // 8 threads per query row
        const int q = tid >> 3, d0 = (tid & 7) * NV;
        if (q < p.Sq) {
            float out[NV], M, L;
            merge_parts<NV>(part + q * PST, kDecodeWaves, 32 * PST, D, d0, out, M, L);
            if (p.nsplit == 1) {
                const float inv = L > 0.f ? 1.f / L : 0.f;
                if (p.lse != nullptr && (tid & 7) == 0)
                    p.lse[b * p.lses[0] + h * p.lses[1] + q * p.lses[2]] =
                        L > 0.f ? (M + __builtin_amdgcn_logf(L)) * 0.69314718056f : kNegInf;
                uint16_t *orow = p.o + b * p.os[0] + h * p.os[1] + (int64_t)q * p.os[2] + d0;
#pragma unroll
                for (int j = 0; j < NV; j += 2) *(uint32_t *)(orow + j) = E::pack2(out[j] * inv, out[j + 1] * inv);
            } else {
                float *w = p.ws + (((int64_t)bh * p.nsplit + split) * p.Sq + q) * PST;
#pragma unroll
                for (int j = 0; j < NV; j++) w[d0 + j] = out[j];
                if ((tid & 7) == 0) {
                    w[D] = M;
                    w[D + 1] = L;
                }
            }
        }
    }
}

// Merge of the nsplit partial results of every (b, h): grid B*H, 256 threads, 8 per query row.
template <int DT, int D>
__global__ __launch_bounds__(256) void decode_merge_kernel(const DecodeParams p) {
    using E = Elem<DT>;
    constexpr int NV = D / 8, PST = D + 2;
    const int tid = threadIdx.x, bh = blockIdx.x;
    const int b = bh / p.H, h = bh - b * p.H;
    const int q = tid >> 3, d0 = (tid & 7) * NV;
    if (q >= p.Sq) return;
    float out[NV], M, L;
    merge_parts<NV>(p.ws + ((int64_t)bh * p.nsplit * p.Sq + q) * PST, p.nsplit, (int64_t)p.Sq * PST, D, d0, out, M, L);
    const float inv = L > 0.f ? 1.f / L : 0.f;
    if (p.lse != nullptr && (tid & 7) == 0)
        p.lse[b * p.lses[0] + h * p.lses[1] + q * p.lses[2]] =
            L > 0.f ? (M + __builtin_amdgcn_logf(L)) * 0.69314718056f : kNegInf;
    uint16_t *orow = p.o + b * p.os[0] + h * p.os[1] + (int64_t)q * p.os[2] + d0;
#pragma unroll
    for (int j = 0; j < NV; j += 2) *(uint32_t *)(orow + j) = E::pack2(out[j] * inv, out[j + 1] * inv);
}

// Merge of n attention results over disjoint key ranges: o = sum_i exp(lse_i - lse) o_i, lse = log sum_i exp(lse_i).
// One thread per 8 output elements.
template <int DT>
__global__ __launch_bounds__(256) void merge_parts_kernel(const MergeParams p) {
    using E = Elem<DT>;
    const int per_row = p.D / 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t row = idx / per_row;
    const int part = (int)(idx - row * per_row);
    if (row >= (int64_t)p.B * p.H * p.Sq) return;
    const int q = (int)(row % p.Sq);
    const int bh = (int)(row / p.Sq);
    const int b = bh / p.H, h = bh - b * p.H;
    const float *lp = p.lse_parts + b * p.lps[1] + h * p.lps[2] + (int64_t)q * p.lps[3];
    float M = kNegInf;
    for (int i = 0; i < p.n; i++) M = fmaxf(M, lp[i * p.lps[0]]);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float L = 0.f;
    if (M != kNegInf) {
        for (int i = 0; i < p.n; i++) {
            const float w = __expf(lp[i * p.lps[0]] - M);  // 0 for parts whose keys this row does not attend to
            L += w;
            const u32x4 x = *(const u32x4 *)(p.o_parts + i * p.ops[0] + b * p.ops[1] + h * p.ops[2] +
                                             (int64_t)q * p.ops[3] + 8 * part);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t xe = x[e];
                if constexpr (DT == 0) {
                    acc[2 * e] += w * __uint_as_float(xe << 16);
                    acc[2 * e + 1] += w * __uint_as_float(xe & 0xffff0000u);
                } else {
                    const f16x2 hx = __builtin_bit_cast(f16x2, xe);
                    acc[2 * e] += w * (float)hx.x;
                    acc[2 * e + 1] += w * (float)hx.y;
                }
            }
        }
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    u32x4 out;
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = E::pack2(acc[2 * e] * inv, acc[2 * e + 1] * inv);
    *(u32x4 *)(p.o + b * p.os[0] + h * p.os[1] + (int64_t)q * p.os[2] + 8 * part) = out;
    if (p.lse != nullptr && part == 0)
        p.lse[b * p.lses[0] + h * p.lses[1] + (int64_t)q * p.lses[2]] = L > 0.f ? M + __logf(L) : kNegInf;
}

template <int DT, int D, bool PK, bool B16>
hipError_t launch_decode_kind(const DecodeParams &p, hipStream_t stream) {
    constexpr int smem = decode_smem_bytes<D>();
    auto kern = sparse_decode_kernel<DT, D, PK, B16>;
    static unsigned long long attr_done = 0;  // devices on which this kernel may use `smem` bytes of LDS
    if (const hipError_t e0 = allow_dynamic_smem(kern, smem, attr_done); e0 != hipSuccess) return e0;
    hipLaunchKernelGGL(kern, dim3(p.nsplit, p.B * p.H), dim3(kDecodeWaves * 64), smem, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || p.nsplit == 1) return e;
    hipLaunchKernelGGL((decode_merge_kernel<DT, D>), dim3(p.B * p.H), dim3(256), 0, stream, p);
    return hipGetLastError();
}

template <int DT, int D>
hipError_t launch_decode_one(const DecodeParams &p, hipStream_t stream) {
    const bool pk = p.packed != nullptr, b16 = p.BK == 16;
    if (pk) return b16 ? launch_decode_kind<DT, D, true, true>(p, stream) : launch_decode_kind<DT, D, true, false>(p, stream);
    return b16 ? launch_decode_kind<DT, D, false, true>(p, stream) : launch_decode_kind<DT, D, false, false>(p, stream);
}

}  // namespace

hipError_t launch_merge_parts(const MergeParams &p, int dtype, hipStream_t stream) {
    const int64_t threads = (int64_t)p.B * p.H * p.Sq * (p.D / 8);
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (dtype == 0) hipLaunchKernelGGL((merge_parts_kernel<0>), dim3(grid), dim3(256), 0, stream, p);
    else if (dtype == 1) hipLaunchKernelGGL((merge_parts_kernel<1>), dim3(grid), dim3(256), 0, stream, p);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_decode(const DecodeParams &p, int dtype, int D, hipStream_t stream) {
    if (dtype == 0 && D == 128) return launch_decode_one<0, 128>(p, stream);
    if (dtype == 0 && D == 64) return launch_decode_one<0, 64>(p, stream);
    if (dtype == 1 && D == 128) return launch_decode_one<1, 128>(p, stream);
    if (dtype == 1 && D == 64) return launch_decode_one<1, 64>(p, stream);
    return hipErrorInvalidValue;
}

}  // namespace sa
