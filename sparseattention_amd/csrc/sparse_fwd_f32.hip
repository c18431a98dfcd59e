// Block-sparse attention forward for float32 q, k, v, o: the reference's kernel takes whatever element type its
// inputs have (sparse_attn_kernel.py:98-101, :145), so float32 runs too.  This is the plain form of the algorithm
// (sparse_attn_kernel.py:28-63, :103-146) on the vector units, in float32 throughout, for callers that check
// numbers against an fp32 reference; the bf16 / fp16 kernels of sparse_fwd_kernel.h are the ones that are tuned.
//
// One workgroup per (Q tile, b, h), four lanes per query row.  A lane keeps a quarter of its row's queries and of
// its output accumulators in registers (the part-th 16-byte piece of every 64 bytes, so that the four lanes of a row
// read 64 consecutive bytes); K and V rows go through LDS 32 keys at a time, and every lane with the same quarter
// reads the same LDS address (a broadcast).  Per 32 keys: scores by dot products reduced over the four lanes, mask of
// PARTIAL tiles from the packed bits or the bool tensor, online softmax in exp2 units with the reference's update
// order (row maximum, rescale, exponentials, row sum, accumulate), then P.V.  FULL tiles first, PARTIAL tiles after,
// as in the reference.  Rows that attend to nothing give 0.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fwd_common.h"
#include "kernels.h"

namespace sa {

namespace {

constexpr int kKC = 32;  // keys per LDS chunk
constexpr float kNegInfF = -__builtin_huge_valf();

// At head dim 256 a lane's queries and accumulators take 128 registers: workgroups of at most 512 threads there, so
// that a lane may have 256.
template <int D>
__global__ __launch_bounds__(D > 128 ? 512 : 1024) void sparse_fwd_f32_kernel(const FwdParams p, const int BQ) {
    constexpr int NP = D / 16;  // 16-byte pieces per lane and row
    extern __shared__ __attribute__((aligned(16))) float lds[];  // [kKC][D] of K, then of V
    float *const ks = lds, *const vs = lds + kKC * D;

    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int r = tid >> 2, part = tid & 3;
    const bool row_ok = r < BQ;  // (the block is padded to whole waves)
    const int bh = blockIdx.x / p.nQ, qt = blockIdx.x - bh * p.nQ;
    const int b = bh / p.H, h = bh - b * p.H;
    const int row = qt * BQ + (row_ok ? r : 0);

    const float *qp = reinterpret_cast<const float *>(p.q) + b * p.qs[0] + h * p.qs[1] + (int64_t)row * p.qs[2];
    const float *kbase = reinterpret_cast<const float *>(p.k) + b * p.ks[0] + h * p.ks[1];
    const float *vbase = reinterpret_cast<const float *>(p.v) + b * p.vs[0] + h * p.vs[1];
    float4 q[NP], acc[NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        q[i] = *reinterpret_cast<const float4 *>(qp + 16 * i + 4 * part);
        acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float m_i = kNegInfF, l_i = 0.f;

    // counts clamped to the row of tiles, indices outside it skipped (the reference guards its loads with
    // kv_offset < SEQLEN_K, sparse_attn_kernel.py:35,39,60)
    const int F = min(max(p.full_lens[b * p.fls[0] + h * p.fls[1] + qt * p.fls[2]], 0), p.nK);
    const int P = min(max(p.part_lens[b * p.pls[0] + h * p.pls[1] + qt * p.pls[2]], 0), p.nK - F);
    const int32_t *fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + qt * p.fis[2];
    const int32_t *pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + qt * p.pis[2];
    const uint8_t *mrow = p.mask ? p.mask + b * p.ms[0] + h * p.ms[1] + (int64_t)row * p.ms[2] : nullptr;
    const int64_t tile_bytes = (int64_t)BQ * p.BK / 8;
    const uint8_t *ptile = p.packed ? p.packed + b * p.pks[0] + h * p.pks[1] + (int64_t)qt * p.nK * tile_bytes : nullptr;

    for (int e = 0; e < F + P; e++) {
        const bool partial = e >= F;
        const int idx = partial ? pid[(int64_t)(e - F) * p.pis[3]] : fid[(int64_t)e * p.fis[3]];
        if ((unsigned)idx >= (unsigned)p.nK) continue;  // (the same for every thread of the workgroup)
        const int col0 = idx * p.BK;
        for (int sub = 0; sub < p.BK; sub += kKC) {
            const int nkeys = min(kKC, p.BK - sub);
            __syncthreads();  // everyone is done with the previous chunk
            for (int x = tid; x < nkeys * (D / 4); x += nthreads) {
                const int kr = x / (D / 4), pc = x - kr * (D / 4);
                const int64_t krow = col0 + sub + kr;
                reinterpret_cast<float4 *>(ks)[kr * (D / 4) + pc] =
                    *reinterpret_cast<const float4 *>(kbase + krow * p.ks[2] + 4 * pc);
                reinterpret_cast<float4 *>(vs)[kr * (D / 4) + pc] =
                    *reinterpret_cast<const float4 *>(vbase + krow * p.vs[2] + 4 * pc);
            }
            __syncthreads();

            // scores of this row against the chunk's keys, in exp2 units (sparse_attn_kernel.py:48-52)
            float s[kKC];
            float mx = kNegInfF;
#pragma unroll
            for (int kk = 0; kk < kKC; kk++) {
                float d = 0.f;
                if (kk < nkeys) {
                    const float4 *kr = reinterpret_cast<const float4 *>(ks + kk * D) + part;
#pragma unroll
                    for (int i = 0; i < NP; i++) {
                        const float4 kv = kr[4 * i];
                        d += q[i].x * kv.x + q[i].y * kv.y + q[i].z * kv.z + q[i].w * kv.w;
                    }
                    d += __shfl_xor(d, 1);
                    d += __shfl_xor(d, 2);
                    d *= p.scale;
                    if (partial) {
                        const int c = sub + kk;  // column inside the tile
                        bool keep;
                        if (ptile) {
                            const int64_t bit = (int64_t)(row_ok ? r : 0) * p.BK + c;
                            keep = (ptile[(int64_t)(e - F) * tile_bytes + (bit >> 3)] >> (bit & 7)) & 1;
                        } else {
                            keep = mrow[(int64_t)(col0 + c) * p.ms[3]] != 0;
                        }
                        if (!keep) d = kNegInfF;
                    }
                } else {
                    d = kNegInfF;
                }
                s[kk] = d;
                mx = fmaxf(mx, d);
            }
            // online softmax (sparse_attn_kernel.py:53-58); a row that has seen no key yet keeps m = -inf and l = 0
            const float m_new = fmaxf(m_i, mx);
            if (m_new != kNegInfF) {
                const float alpha = exp2f(m_i - m_new);  // 0 while m_i is -inf
                float psum = 0.f;
#pragma unroll
                for (int i = 0; i < NP; i++) {
                    acc[i].x *= alpha;
                    acc[i].y *= alpha;
                    acc[i].z *= alpha;
                    acc[i].w *= alpha;
                }
#pragma unroll
                for (int kk = 0; kk < kKC; kk++) {
                    if (kk < nkeys) {
                        const float pk = exp2f(s[kk] - m_new);
                        psum += pk;
                        const float4 *vr = reinterpret_cast<const float4 *>(vs + kk * D) + part;
#pragma unroll
                        for (int i = 0; i < NP; i++) {
                            const float4 vv = vr[4 * i];
                            acc[i].x += pk * vv.x;
                            acc[i].y += pk * vv.y;
                            acc[i].z += pk * vv.z;
                            acc[i].w += pk * vv.w;
                        }
                    }
                }
                l_i = l_i * alpha + psum;
                m_i = m_new;
            }
        }
    }

    if (!row_ok) return;
    const float inv = l_i > 0.f ? 1.f / l_i : 0.f;  // sparse_attn_kernel.py:144; 0 for rows without a key
    float *op = reinterpret_cast<float *>(p.o) + b * p.os[0] + h * p.os[1] + (int64_t)row * p.os[2];
#pragma unroll
    for (int i = 0; i < NP; i++)
        *reinterpret_cast<float4 *>(op + 16 * i + 4 * part) =
            make_float4(acc[i].x * inv, acc[i].y * inv, acc[i].z * inv, acc[i].w * inv);
    if (p.lse != nullptr && part == 0)
        p.lse[b * p.lses[0] + h * p.lses[1] + (int64_t)row * p.lses[2]] =
            l_i > 0.f ? (m_i + log2f(l_i)) * 0.6931471805599453f : kNegInfF;
}

template <int D>
hipError_t launch_d(const FwdParams &p, int BQ, hipStream_t stream) {
    constexpr int smem = 2 * kKC * D * 4;
    auto kern = sparse_fwd_f32_kernel<D>;
    static unsigned long long attr_done = 0;  // devices on which this kernel may use `smem` bytes of LDS
    if (const hipError_t e0 = allow_dynamic_smem(kern, smem, attr_done); e0 != hipSuccess) return e0;
    const int threads = (4 * BQ + 63) / 64 * 64;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.nQ * (unsigned)(p.B * p.H)), dim3(threads), smem, stream, p, BQ);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_fwd_f32(const FwdParams &p, int D, int BQ, hipStream_t stream) {
    if (BQ < 1 || BQ > (D > 128 ? 128 : 256)) return hipErrorInvalidValue;
    if (fwd_f32_mfma_has(p, D, BQ)) return launch_fwd_f32_mfma(p, D, BQ, stream);
    switch (D) {
        case 64: return launch_d<64>(p, BQ, stream);
        case 128: return launch_d<128>(p, BQ, stream);
        case 256: return launch_d<256>(p, BQ, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace sa
