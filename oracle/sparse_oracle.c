/*
 * CPU oracle for the block-sparse attention forward path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithm of the reference package
 * (tomatillos/sparseattention) for the one path this repository accelerates:
 *
 *   oracle_classify   follows  sparseattention/mask_utils.py:14-44   (compute_mask_slow)
 *   oracle_forward    follows  sparseattention/sparse_attn_kernel.py:28-63   (_sparse_inner: one pass)
 *                              sparseattention/sparse_attn_kernel.py:103-146 (state init, pass order, epilogue)
 *                              sparseattention/sparse_attn_kernel.py:152     (scale folded with 1/ln 2)
 *
 * Only tests, the smoke check and the benchmark's CPU-baseline leg may load it; the
 * product (the HIP library) never links or calls anything in here.
 *
 * How it is pinned (tests/test_oracle_*.py): the classification against closed forms
 * (causal, sliding-window/prefix tile counts, all-true, all-false, single-entry flips) and
 * against a vectorised numpy popcount; the forward against torch's masked
 * scaled_dot_product_attention (the routine the reference's own check calls,
 * sparseattention/test_attn.py:40), against an fp64 dense softmax, and against exact special
 * cases (one-hot rows, constant keys).
 *
 * Deliberate differences from the reference, both required to agree with its own checker
 * (masked SDPA) on inputs the reference mishandles:
 *   - rows whose running maximum is still -inf use 0 as the subtrahend, so exp2(-inf - -inf)
 *     never produces NaN (the reference marks this as a todo, sparse_attn_kernel.py:53);
 *   - rows with no attended key produce 0 instead of 0/0.
 * Slots of the index lists at positions >= the stored count are set to -1 here; the
 * reference leaves them uninitialised (torch.empty, mask_utils.py:22-25), so callers must
 * never compare them.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_abi_version(void) { return 1; }

int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Round an fp32 value to the nearest bf16 (ties to even) and widen it back. */
static inline float round_to_bf16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return x; /* NaN stays NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&x, &u, 4);
    return x;
}

/* Round an fp32 value to the nearest fp16 (ties to even, overflow to inf) and widen it back. */
static inline float round_to_fp16(float x) {
    if (!(fabsf(x) <= 3.4028234664e38f)) return x; /* inf and NaN unchanged */
    const float ax = fabsf(x);
    if (ax >= 65520.f) return x < 0 ? -INFINITY : INFINITY; /* beyond the largest half + half an ulp */
    /* spacing of fp16 values around ax: 2^(e-10) for normals (e >= -14), 2^-24 for subnormals */
    int e;
    frexpf(ax, &e); /* ax = f * 2^e with f in [0.5,1) -> binade exponent is e-1 */
    int ulp_exp = (e - 1) - 10;
    if (ulp_exp < -24) ulp_exp = -24;
    const float ulp = ldexpf(1.f, ulp_exp);
    const float r = nearbyintf(ax / ulp) * ulp; /* default rounding mode: ties to even; exact in fp32 */
    return x < 0 ? -r : r;
}

/* Exported so that tests can compare the two rounding helpers with torch's casts directly. */
float oracle_round_bf16(float x) { return round_to_bf16(x); }
float oracle_round_fp16(float x) { return round_to_fp16(x); }

/*
 * Tile classification.  mask is addressed as mask[b*ms[0] + h*ms[1] + q*ms[2] + k*ms[3]]
 * (strides in bytes == elements, any value including 0); a byte != 0 means "attend".
 * Outputs are contiguous: ids [B,H,nQ,nK] int32, lens [B,H,nQ] int32.
 * Per tile: count == BQ*BK -> appended to the full list; 0 < count -> appended to the partial
 * list; count == 0 -> in neither (mask_utils.py:34-40).  KV tile indices ascend.
 */
int oracle_classify(const uint8_t *mask, const int64_t *ms, int B, int H, int Sq, int Sk, int BQ, int BK,
                    int32_t *full_ids, int32_t *full_lens, int32_t *part_ids, int32_t *part_lens) {
    if (!mask || !ms || BQ <= 0 || BK <= 0 || Sq % BQ || Sk % BK) return -1;
    const int nQ = Sq / BQ, nK = Sk / BK;
    const long total = (long)B * H * nQ;
#pragma omp parallel for schedule(static)
    for (long t = 0; t < total; t++) {
        const int i = (int)(t % nQ);
        const int h = (int)((t / nQ) % H);
        const int b = (int)(t / ((long)nQ * H));
        const uint8_t *plane = mask + (int64_t)b * ms[0] + (int64_t)h * ms[1];
        int32_t *fid = full_ids + t * nK, *pid = part_ids + t * nK;
        int nf = 0, np = 0;
        for (int j = 0; j < nK; j++) {
            long count = 0;
            for (int r = 0; r < BQ; r++) {
                const uint8_t *row = plane + (int64_t)(i * BQ + r) * ms[2] + (int64_t)j * BK * ms[3];
                for (int c = 0; c < BK; c++) count += row[(int64_t)c * ms[3]] != 0;
            }
            if (count == (long)BQ * BK) fid[nf++] = j;
            else if (count > 0) pid[np++] = j;
        }
        for (int j = nf; j < nK; j++) fid[j] = -1;
        for (int j = np; j < nK; j++) pid[j] = -1;
        full_lens[t] = nf;
        part_lens[t] = np;
    }
    return 0;
}

/*
 * One pass of the flash loop over one index list (sparse_attn_kernel.py:32-61).
 * State per query row: m (running max, base-2 scaled units), l (running sum), acc[D].
 */
static void one_pass(const float *q_tile, const float *k_plane, const float *v_plane, const uint8_t *mask_plane,
                     int64_t msq, int64_t msk, const int32_t *ids, int len, int q0, int BQ, int BK, int D,
                     float scale, int use_mask, int p_round, float *m, float *l, float *acc, float *s_buf) {
    for (int it = 0; it < len; it++) {
        const int kv0 = ids[it] * BK;
        for (int r = 0; r < BQ; r++) {
            const float *qr = q_tile + (long)r * D;
            float *s = s_buf; /* one row of scores, BK wide */
            float rowmax = -INFINITY;
            for (int c = 0; c < BK; c++) {
                const float *kr = k_plane + (long)(kv0 + c) * D;
                float dot = 0.f;
                for (int d = 0; d < D; d++) dot += qr[d] * kr[d];
                float x = dot * scale;
                if (use_mask && !mask_plane[(int64_t)(q0 + r) * msq + (int64_t)(kv0 + c) * msk]) x = -INFINITY;
                s[c] = x;
                if (x > rowmax) rowmax = x;
            }
            const float m_new = rowmax > m[r] ? rowmax : m[r];
            const float m_ref = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = exp2f(m[r] - m_ref);
            float rowsum = 0.f;
            float *a = acc + (long)r * D;
            for (int d = 0; d < D; d++) a[d] *= alpha;
            for (int c = 0; c < BK; c++) {
                float p = exp2f(s[c] - m_ref);
                rowsum += p;
                if (p_round == 1) p = round_to_bf16(p);
                else if (p_round == 2) p = round_to_fp16(p);
                if (p != 0.f) {
                    const float *vr = v_plane + (long)(kv0 + c) * D;
                    for (int d = 0; d < D; d++) a[d] += p * vr[d];
                }
            }
            l[r] = l[r] * alpha + rowsum;
            m[r] = m_new;
        }
    }
}

/*
 * Two-pass list-driven forward.  q,k,v,out: contiguous fp32 [B,H,S,D] (bf16/fp16 inputs are
 * widened exactly by the caller).  mask strides ms[4] as in oracle_classify.  Metadata
 * contiguous as produced by oracle_classify.  scale_log2 = D^-0.5 / ln 2.
 * p_round: 0 keep P in fp32, 1 round P to bf16 before P.V, 2 round to fp16
 * (the reference casts P to V's dtype, sparse_attn_kernel.py:61).
 */
int oracle_forward(const float *q, const float *k, const float *v, float *out, const uint8_t *mask,
                   const int64_t *ms, const int32_t *full_ids, const int32_t *full_lens, const int32_t *part_ids,
                   const int32_t *part_lens, int B, int H, int Sq, int Sk, int D, int BQ, int BK, float scale_log2,
                   int p_round) {
    if (!q || !k || !v || !out || !mask || !ms || BQ <= 0 || BK <= 0 || Sq % BQ || Sk % BK) return -1;
    const int nQ = Sq / BQ, nK = Sk / BK;
    const long total = (long)B * H * nQ;
    int failed = 0;
#pragma omp parallel
    {
        float *m = (float *)malloc(sizeof(float) * BQ);
        float *l = (float *)malloc(sizeof(float) * BQ);
        float *acc = (float *)malloc(sizeof(float) * (size_t)BQ * D);
        float *s_buf = (float *)malloc(sizeof(float) * BK);
        if (!m || !l || !acc || !s_buf) {
#pragma omp atomic write
            failed = 1;
        } else {
#pragma omp for schedule(dynamic, 1)
            for (long t = 0; t < total; t++) {
                const int i = (int)(t % nQ);
                const int h = (int)((t / nQ) % H);
                const int b = (int)(t / ((long)nQ * H));
                const long bh = (long)b * H + h;
                const float *q_tile = q + (bh * Sq + (long)i * BQ) * D;
                const float *k_plane = k + bh * Sk * D;
                const float *v_plane = v + bh * Sk * D;
                const uint8_t *mask_plane = mask + (int64_t)b * ms[0] + (int64_t)h * ms[1];
                for (int r = 0; r < BQ; r++) { m[r] = -INFINITY; l[r] = 0.f; }
                memset(acc, 0, sizeof(float) * (size_t)BQ * D);
                /* full tiles first, no mask; then partial tiles with the mask (:113-142) */
                one_pass(q_tile, k_plane, v_plane, mask_plane, ms[2], ms[3], full_ids + t * nK, full_lens[t], i * BQ, BQ,
                         BK, D, scale_log2, 0, p_round, m, l, acc, s_buf);
                one_pass(q_tile, k_plane, v_plane, mask_plane, ms[2], ms[3], part_ids + t * nK, part_lens[t], i * BQ, BQ,
                         BK, D, scale_log2, 1, p_round, m, l, acc, s_buf);
                float *o_tile = out + (bh * Sq + (long)i * BQ) * D;
                for (int r = 0; r < BQ; r++) {
                    for (int d = 0; d < D; d++)
                        o_tile[(long)r * D + d] = l[r] > 0.f ? acc[(long)r * D + d] / l[r] : 0.f; /* :144 */
                }
            }
        }
        free(m); free(l); free(acc); free(s_buf);
    }
    return failed ? -2 : 0;
}

/*
 * One bit per mask entry of every PARTIAL tile (the optional packed route of the HIP library; the reference
 * has no such step: it re-reads the bool tile in every forward, sparse_attn_kernel.py:42-46).
 *
 * part_ids [B,H,nQ,nK] / part_lens [B,H,nQ] are the PARTIAL lists of oracle_classify.  out is
 * [B,H,nQ,nK,BQ*BK/8] bytes, zero-filled by the caller: tile (qt, slot) holds the BQ x BK entries of KV tile
 * part_ids[..., qt, slot], rows first, entry (r, c) in bit (c & 7) of byte (r*BK + c) >> 3; a byte != 0 in
 * the mask sets the bit.  Slots >= the count stay as the caller left them.
 * Pinned by tests/test_oracle_pack.py against numpy.packbits(bitorder="little") of the same tiles and
 * against the closed form of the causal diagonal tiles.
 */
int oracle_pack_partial(const uint8_t *mask, const int64_t *ms, int B, int H, int Sq, int Sk, int BQ, int BK,
                        const int32_t *part_ids, const int32_t *part_lens, uint8_t *out) {
    if (BQ <= 0 || BK <= 0 || Sq % BQ || Sk % BK || BK % 8) return -1;
    const int nQ = Sq / BQ, nK = Sk / BK;
    const long tile_bytes = (long)BQ * BK / 8;
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++)
            for (int i = 0; i < nQ; i++) {
                const long row = ((long)b * H + h) * nQ + i;
                for (int s = 0; s < part_lens[row]; s++) {
                    const int j = part_ids[row * nK + s];
                    uint8_t *tile = out + (row * nK + s) * tile_bytes;
                    for (int r = 0; r < BQ; r++)
                        for (int c = 0; c < BK; c++) {
                            const uint8_t m = mask[(int64_t)b * ms[0] + (int64_t)h * ms[1] +
                                                   (int64_t)(i * BQ + r) * ms[2] + (int64_t)(j * BK + c) * ms[3]];
                            const long bit = (long)r * BK + c;
                            if (m) tile[bit >> 3] |= (uint8_t)(1u << (bit & 7));
                            else tile[bit >> 3] &= (uint8_t)~(1u << (bit & 7));
                        }
                }
            }
    return 0;
}
