// Tile classification and bit-packing of an attention mask that is given by a formula, on gfx950 (MI355X).
//
// The reference parses a materialised bool tensor (sparseattention/mask_utils.py:47-82) and names masks defined
// algebraically, without materialisation and its memory cost, as the first thing that could come next
// (README.md:12, :63).  Here the mask of entry (b, q, k) is the OR of up to kMaxMaskTerms terms, each the AND of
// the conditions its flags switch on:
//
//   BACK      (q + offset) - k < back        (how far behind the diagonal a key may lie)
//   AHEAD     k - (q + offset) < ahead       (ahead = 1: causal)
//   Q_RANGE   q_lo <= q < q_hi
//   K_RANGE   k_lo <= k < k_hi
//   SAME_DOC  doc_q[b][q] == doc_k[b][k]
//
//   classify_terms_kernel   one class byte per (distinct batch plane, Q tile, KV tile), the layout compact_kernel
//                           reads (mask_classify.hip), so the lists come out as for a tensor mask;
//   pack_terms_kernel       the PARTIAL tiles at one bit per entry in the layout of pack_partial_kernel, so the
//                           forward and the backward run without any mask tensor.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace sa {

namespace {

// For one query row a term admits an interval of keys (and of those the keys of the row's document).  With q uniform
// over a wave the interval lives in scalar registers and a lane pays two compares per term.
__device__ __forceinline__ void term_interval(const MaskTerm &m, int q, int &lo, int &hi) {
    lo = max(q + m.a, m.k_lo);
    hi = min(q + m.b, m.k_hi);
    if (q < m.q_lo || q >= m.q_hi) hi = lo;
}

__device__ __forceinline__ bool eval_terms(const TermsParams &p, int q, int k, int dq, int dk) {
    bool any = false;
    for (int t = 0; t < p.n_terms; t++) {
        int lo, hi;
        term_interval(p.terms[t], q, lo, hi);
        any = any || (k >= lo && k < hi && (!p.terms[t].doc || dq == dk));
    }
    return any;
}

// grid (regions of max(BK, 64) keys, nQ, distinct planes), one wave per workgroup.  Both ends of a row's interval
// move right (or stay) as q grows, so the first and the last row of the Q tile decide most regions at once: no term
// reaches the region (EMPTY), or one term covers it from every row (FULL), document conditions judged by the ranges of
// the document numbers on both sides.  The rest
// is evaluated: lane = key within a strip of 64 keys, per query row one ballot gives the row's 64 entries, whose set
// bits are counted per tile in scalar registers.
__global__ __launch_bounds__(64) void classify_terms_kernel(const TermsParams p) {
    const int lane = threadIdx.x;
    const int qt = blockIdx.y, ub = blockIdx.z;
    const int W = p.BK < 64 ? 64 : p.BK;      // keys per region
    const int k_reg = blockIdx.x * W;
    const int k_end = min(k_reg + W, p.Sk);
    const int tiles = W / p.BK;               // tiles per region: 4, 2 or 1
    const int q0 = qt * p.BQ, q1 = q0 + p.BQ - 1;
    uint8_t *cls = p.cls + ((int64_t)ub * p.nQ + qt) * p.nK + k_reg / p.BK;
    const bool owns = lane < tiles && k_reg / p.BK + lane < p.nK;

    const int32_t *dqp = p.doc_q ? p.doc_q + (int64_t)ub * p.dqs[0] : nullptr;
    const int32_t *dkp = p.doc_k ? p.doc_k + (int64_t)ub * p.dks[0] : nullptr;
    // Documents of the tile's rows and of the region's keys, as ranges of their numbers: ranges that do not meet
    // silence a document condition here, ranges of one and the same number satisfy it everywhere.
    bool docs_apart = false, docs_one = false;
    if (dqp && dkp) {
        int qmin = INT32_MAX, qmax = INT32_MIN, kmin = INT32_MAX, kmax = INT32_MIN;
        for (int r = lane; r < p.BQ; r += 64) {
            const int d = dqp[(int64_t)(q0 + r) * p.dqs[1]];
            qmin = min(qmin, d);
            qmax = max(qmax, d);
        }
        for (int k = k_reg + lane; k < k_end; k += 64) {
            const int d = dkp[(int64_t)k * p.dks[1]];
            kmin = min(kmin, d);
            kmax = max(kmax, d);
        }
#pragma unroll
        for (int sh = 32; sh >= 1; sh >>= 1) {
            qmin = min(qmin, __shfl_xor(qmin, sh));
            qmax = max(qmax, __shfl_xor(qmax, sh));
            kmin = min(kmin, __shfl_xor(kmin, sh));
            kmax = max(kmax, __shfl_xor(kmax, sh));
        }
        docs_apart = qmax < kmin || kmax < qmin;
        docs_one = qmin == qmax && kmin == kmax && qmin == kmin;
    }

    bool none = true, whole = false;
    for (int t = 0; t < p.n_terms; t++) {
        const MaskTerm &m = p.terms[t];
        const int r0 = max(q0, m.q_lo), r1 = min(q1, m.q_hi - 1);  // rows of the tile the term speaks about
        if (r0 > r1 || (m.doc && docs_apart)) continue;
        int lo0, hi0, lo1, hi1;
        term_interval(m, r0, lo0, hi0);
        term_interval(m, r1, lo1, hi1);
        // hi(q) <= hi1 and lo(q) >= lo0 on these rows
        if (hi1 > k_reg && lo0 < k_end) none = false;
        if ((!m.doc || docs_one) && r0 == q0 && r1 == q1 && lo1 <= k_reg && hi0 >= k_end) whole = true;
    }
    if (none || whole) {
        if (owns) cls[lane] = whole ? 2 : 0;
        return;
    }

    unsigned cnt[4] = {0u, 0u, 0u, 0u};
    for (int ks = k_reg; ks < k_end; ks += 64) {
        const int k = ks + lane;
        const bool k_in = k < p.Sk;
        const int dk = (dkp && k_in) ? dkp[(int64_t)k * p.dks[1]] : 0;
        for (int r0 = 0; r0 < p.BQ; r0 += 64) {
            // the documents of 64 query rows, one per lane, handed out row by row below
            const int rq = q0 + r0 + lane;
            const int dq_lane = (dqp && r0 + lane < p.BQ) ? dqp[(int64_t)rq * p.dqs[1]] : 0;
            const int rows = p.BQ - r0 < 64 ? p.BQ - r0 : 64;
            for (int r = 0; r < rows; r++) {
                const int dq = __builtin_amdgcn_readlane(dq_lane, r);
                const unsigned long long bits = __ballot(k_in && eval_terms(p, q0 + r0 + r, k, dq, dk));
                if (p.BK >= 64) {
                    cnt[0] += (unsigned)__popcll(bits);
                } else if (p.BK == 32) {
                    cnt[0] += (unsigned)__popc((unsigned)bits);
                    cnt[1] += (unsigned)__popc((unsigned)(bits >> 32));
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) cnt[j] += (unsigned)__popc((unsigned)(bits >> (16 * j)) & 0xffffu);
                }
            }
        }
    }
    if (owns) {
        const unsigned c = lane == 0 ? cnt[0] : (lane == 1 ? cnt[1] : (lane == 2 ? cnt[2] : cnt[3]));
        const unsigned full = (unsigned)p.BQ * (unsigned)p.BK;
        cls[lane] = c == full ? 2 : (c != 0u ? 1 : 0);
    }
}

// grid (slot lanes, nQ, distinct planes), 256 threads.  Workgroup x takes the PARTIAL slots x, x + gridDim.x, ... of
// its Q tile; a thread makes one 32-bit word of a packed tile: entries 32w .. 32w + 31 in row-major order.
__global__ __launch_bounds__(256) void pack_terms_kernel(const TermsParams p) {
    const int qt = blockIdx.y, ub = blockIdx.z;
    const int len = p.part_lens[ub * p.pls[0] + qt * p.pls[2]];
    const int32_t *ids = p.part_ids + ub * p.pis[0] + qt * p.pis[2];
    const int tile_words = p.BQ * p.BK / 32;
    const int32_t *dqp = p.doc_q ? p.doc_q + (int64_t)ub * p.dqs[0] : nullptr;
    const int32_t *dkp = p.doc_k ? p.doc_k + (int64_t)ub * p.dks[0] : nullptr;
    uint32_t *out_q = reinterpret_cast<uint32_t *>(p.packed + (int64_t)ub * p.ob) + (int64_t)qt * p.nK * tile_words;
    for (int slot = blockIdx.x; slot < len; slot += gridDim.x) {
        const int col0 = ids[(int64_t)slot * p.pis[3]] * p.BK;
        uint32_t *out = out_q + (int64_t)slot * tile_words;
        for (int w = threadIdx.x; w < tile_words; w += 256) {
            uint32_t word = 0u;
            int r_prev = -1, dq = 0;
            for (int i = 0; i < 32; i++) {
                const int e = 32 * w + i;
                const int r = e / p.BK, c = e - r * p.BK;
                const int q = qt * p.BQ + r, k = col0 + c;
                if (dqp && r != r_prev) {
                    dq = dqp[(int64_t)q * p.dqs[1]];
                    r_prev = r;
                }
                const int dk = dkp ? dkp[(int64_t)k * p.dks[1]] : 0;
                if (eval_terms(p, q, k, dq, dk)) word |= 1u << i;
            }
            out[w] = word;
        }
    }
}

}  // namespace

hipError_t launch_classify_terms(const TermsParams &p, hipStream_t stream) {
    const int W = p.BK < 64 ? 64 : p.BK;
    hipLaunchKernelGGL(classify_terms_kernel, dim3((p.Sk + W - 1) / W, p.nQ, p.uB), dim3(64), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_pack_terms(const TermsParams &p, hipStream_t stream) {
    const int lanes = p.nK < 8 ? p.nK : 8;
    hipLaunchKernelGGL(pack_terms_kernel, dim3(lanes, p.nQ, p.uB), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace sa
