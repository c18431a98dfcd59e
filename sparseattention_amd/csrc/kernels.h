// Internal declarations shared by the C-ABI translation unit and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sa {

// ---- mask classification -------------------------------------------------------------------------
struct ClassifyParams {
    const uint8_t *mask;
    int64_t sb, sh, sq, sk;  // mask strides in bytes over the DISTINCT planes (sb/sh unused when uB/uH == 1)
    uint8_t *cls;            // [uB*uH, nQ, nK] class bytes: 0 empty, 1 partial, 2 full
    int uB, uH;              // distinct planes along b and h
    int Sq, Sk, BQ, BK, nQ, nK;
    int lbk;                 // log2(BK) (wide kernel only)
};

struct CompactParams {
    const uint8_t *cls;
    int uH;                // distinct planes along h in cls
    int bcast_b, bcast_h;  // 1: every output plane along that dimension reads class plane 0
    int oB, oH;            // output planes to write
    int nQ, nK;
    int32_t *full_ids, *full_lens, *part_ids, *part_lens;
    int64_t fis[4], fls[3], pis[4], pls[3];  // output strides in elements
};

// Bit-packing of the PARTIAL tiles: tile (qt, slot) of a distinct plane is the slot-th entry of that Q tile's
// PARTIAL list; its BQ x BK mask entries become BQ*BK/8 bytes, row-major, entry (r, c) in bit (c & 7) of byte
// (r*BK + c) >> 3.
struct PackParams {
    const uint8_t *mask;
    int64_t sb, sh, sq, sk;  // mask strides in bytes over the distinct planes
    const int32_t *part_ids, *part_lens;
    int64_t pis[4], pls[3];  // list strides in elements, indexed with the distinct-plane coordinates
    uint8_t *packed;
    int64_t ob, oh;  // bytes between the packed planes along b and h
    int uB, uH;
    int BQ, BK, nQ, nK;
    int vec8;  // 1: key stride 1 and every row segment 8-byte aligned, so 8 entries load as one qword
};

// Q tiles dealt out to G persistent workgroups (G a multiple of 8, G/8 <= 64).  Workgroup g = 8*j + x is taken
// to run on XCD x (hardware hands consecutive workgroup ids to the XCDs in turn) and gets Q tiles of the x-th
// eighth of the (b,h)-major order, so that the tiles sharing a K/V plane meet in one L2.
// sched: int32 [G][R+1][4]; entry 0 of a row = {count, 0, 0, 0}, entries 1..count = {(b << 16) | h, qt, F, P}.
struct ScheduleParams {
    const int32_t *full_lens, *part_lens;
    int64_t fls[3], pls[3];
    int B, H, nQ;
    int G, R;
    int lbk;  // log2(BK): chunks of 64 keys per entry = BK/64, entries per chunk = 64/BK
    int pairs;  // 1: two Q tiles per workgroup, one workgroup per pair of tiles (G = number of pairs, R = 2)
    int32_t *sched;
};

// Check of caller-supplied lists against the nK tiles a row of tiles has; *flag collects error bits (never cleared here).
struct ValidateParams {
    const int32_t *full_ids, *full_lens, *part_ids, *part_lens;
    int64_t fis[4], fls[3], pis[4], pls[3];
    int B, H, nQ, nK;
    int32_t *flag;
};
hipError_t launch_validate(const ValidateParams &p, hipStream_t stream);

hipError_t launch_classify(const ClassifyParams &p, bool wide, hipStream_t stream);
hipError_t launch_schedule(const ScheduleParams &p, hipStream_t stream);
hipError_t launch_compact(const CompactParams &p, hipStream_t stream);
hipError_t launch_pack(const PackParams &p, hipStream_t stream);

// ---- masks given by a formula ---------------------------------------------------------------------
// Entry (b, q, k) attends when any term holds; a term is the AND of the conditions its flags switch on.
constexpr int kMaxMaskTerms = 8;
constexpr int kTermBack = 1;      // (q + offset) - k < back
constexpr int kTermAhead = 2;     // k - (q + offset) < ahead
constexpr int kTermQRange = 4;    // q_lo <= q < q_hi
constexpr int kTermKRange = 8;    // k_lo <= k < k_hi
constexpr int kTermSameDoc = 16;  // doc_q[b][q] == doc_k[b][k]
// A term as the kernels evaluate it: for query row q it admits the keys of
//   [max(q + a, k_lo), min(q + b, k_hi))   when q_lo <= q < q_hi, none otherwise,
// and of those the keys of q's document when `doc` is set.  a, b are clamped to +-2^30 and the ranges to the
// mask's extent on the host, so that with Sq, Sk <= 2^29 everything stays inside int32.
struct MaskTerm {
    int32_t a, b, k_lo, k_hi, q_lo, q_hi, doc;
};
struct TermsParams {
    MaskTerm terms[kMaxMaskTerms];
    int n_terms;
    const int32_t *doc_q, *doc_k;  // [uB, Sq] and [uB, Sk] document numbers, or null
    int64_t dqs[2], dks[2];        // their strides in elements
    int uB;                        // distinct planes (the mask never depends on the head)
    int Sq, Sk, BQ, BK, nQ, nK;
    uint8_t *cls;                  // [uB, nQ, nK] class bytes (classification)
    // packing: the PARTIAL lists of the distinct planes and the output in PackParams layout
    const int32_t *part_ids, *part_lens;
    int64_t pis[4], pls[3];
    uint8_t *packed;
    int64_t ob;  // bytes between packed planes along b
};
hipError_t launch_classify_terms(const TermsParams &p, hipStream_t stream);
hipError_t launch_pack_terms(const TermsParams &p, hipStream_t stream);

// ---- block-sparse forward ------------------------------------------------------------------------
struct FwdParams {
    const uint16_t *q, *k, *v;
    uint16_t *o;
    const uint8_t *mask;
    const int32_t *full_ids, *full_lens, *part_ids, *part_lens;
    int64_t qs[3], ks[3], vs[3], os[3];  // b, h, s strides in elements (d stride is 1)
    int64_t ms[4];                        // mask strides in bytes
    int64_t fis[4], fls[3], pis[4], pls[3];
    int B, H, Sq, Sk, nQ;
    int BK, lbk;    // KV tile width and its log2
    int mask_vec4;  // 1: mask columns are contiguous and 4-byte aligned, so 4 entries load as one dword
    // Bit-packed PARTIAL tiles (PackParams layout), or null: then the mask itself is read.
    const uint8_t *packed;
    int64_t pks[2];  // bytes between packed planes along b and h (0 where the mask is broadcast)
    int nK;          // KV tiles per row of tiles (slots per Q tile in `packed`)
    // Schedule of persistent workgroups (ScheduleParams layout), or null: then one workgroup per Q tile.
    const int32_t *sched;
    int sched_G, sched_R;  // workgroups, and entries per row after the header entry
    float scale;    // softmax scale / ln 2
    // 0, or the group size G of the rotated walk of the FULL entries (sparse_fwd_kernel, one workgroup per Q tile):
    // Q tile qt starts 2 * (G - 1 - qt mod G) chunks into its FULL entries.
    int rot;
    // Optional second output: natural-log sum of exp(scaled score) over the attended keys of every query row
    // (-inf for rows without one), or null.
    float *lse;
    int64_t lses[3];  // b, h, row strides in elements
};

// dtype: 0 bf16, 1 fp16.  Returns hipErrorInvalidValue when no instantiation matches (D, BQ).
hipError_t launch_fwd(const FwdParams &p, int dtype, int D, int BQ, hipStream_t stream);
// The forward for short lists (sparse_fwd_c32.hip): three workgroups per compute unit, 32 keys per step.  It exists
// for bf16 / fp16, D = 128, BLOCK_Q = 128, bit-packed PARTIAL tiles, no schedule (fwd_c32_has), and cuts lists at
// 256 entries.  Results agree with launch_fwd within rounding (the keys meet the online softmax in other groupings).
bool fwd_c32_has(const FwdParams &p, int dtype, int D, int BQ);
hipError_t launch_fwd_c32(const FwdParams &p, int dtype, int D, int BQ, hipStream_t stream);
// float32 q, k, v, o (the pointers of FwdParams then address floats; strides stay in elements): any BQ from 1 to 256
// (to 128 at D = 256), any BK; reads the packed tiles when given, else the mask; no schedules.
hipError_t launch_fwd_f32(const FwdParams &p, int D, int BQ, hipStream_t stream);
// The same on the matrix unit (sparse_fwd_f32_mfma.hip) for the sizes it has (fwd_f32_mfma_has); launch_fwd_f32 takes
// it whenever it can.
bool fwd_f32_mfma_has(const FwdParams &p, int D, int BQ);
hipError_t launch_fwd_f32_mfma(const FwdParams &p, int D, int BQ, hipStream_t stream);

// Few query rows against a long K/V (decode): one Q tile of Sq <= 32 rows per (b, h), its list of KV tiles split
// over `nsplit` workgroups whose partial results a second kernel merges.
struct DecodeParams {
    const uint16_t *q, *k, *v;
    uint16_t *o;
    const uint8_t *mask;
    const int32_t *full_ids, *full_lens, *part_ids, *part_lens;
    int64_t qs[3], ks[3], vs[3], os[3];  // b, h, s strides in elements (d stride is 1)
    int64_t ms[4];                        // mask strides in bytes
    int64_t fis[3], fls[2], pis[3], pls[2];  // b, h (and entry) strides of the lists of the one Q tile
    int B, H, Sq, Sk;
    int BK, lbk;    // KV tile width (a power of two >= 16) and its log2
    int mask_vec4;  // 1: mask columns are contiguous and 4-byte aligned
    // Bit-packed PARTIAL tiles of the one Q tile (PackParams layout with BQ = Sq), or null: then the mask itself is read.
    const uint8_t *packed;
    int64_t pks[2];  // bytes between packed planes along b and h
    int nsplit;     // workgroups per (b, h)
    float *ws;      // [B*H][nsplit][Sq][D + 2] floats: unnormalised rows, then reference value and row sum
    float scale;    // softmax scale / ln 2
    float *lse;     // optional second output as in FwdParams, or null
    int64_t lses[3];
};
hipError_t launch_decode(const DecodeParams &p, int dtype, int D, hipStream_t stream);

// Merge of n attention results computed over disjoint key ranges (outputs and row log-sum-exps).
struct MergeParams {
    const uint16_t *o_parts;  // [n,B,H,Sq,D]
    const float *lse_parts;   // [n,B,H,Sq]
    uint16_t *o;
    float *lse;               // optional
    int64_t ops[4], lps[4];   // part, b, h, row strides in elements (d stride is 1)
    int64_t os[3], lses[3];
    int n, B, H, Sq, D;
};
hipError_t launch_merge_parts(const MergeParams &p, int dtype, hipStream_t stream);

// ---- backward ------------------------------------------------------------------------------------
// One pass of the backward kernel (sparse_bwd.hip): tiles of 128 resident rows walk their lists of 64-row streamed
// tiles.  dQ: resident q (x = q, g = dO), streamed keys (y = k, z = v), statistics per resident row.
// dK / dV: resident keys (x = k, g = v), streamed queries (y = q, z = dO), statistics per streamed row, lists and
// mask strides of the transposed mask.  D = 64 or 128.
struct BwdParams {
    const uint16_t *x, *g, *y, *z;
    uint16_t *out;
    int64_t xs[3], gs[3], ys[3], zs[3], outs[3];  // b, h, row strides in elements (d stride is 1)
    const uint8_t *mask;
    int64_t ms[2];     // mask strides along b and h in bytes
    int64_t mrs, mcs;  // mask strides along the resident and the streamed rows in bytes
    int mask_vec4;     // 1: mcs == 1 and 4-byte aligned rows
    // Bit-packed PARTIAL tiles of this pass's tiling (PackParams layout, tiles of 128 x 64), or null: then `mask`.
    const uint8_t *packed;
    int64_t pks[2];    // bytes between packed planes along b and h
    int nS;            // streamed tiles per resident tile (slots in `packed`)
    const int32_t *full_ids, *full_lens, *part_ids, *part_lens;  // per resident tile, streamed tiles of 64
    int64_t fis[4], fls[3], pis[4], pls[3];
    const float *stat_l, *stat_d;  // per query: lse / ln 2 (+inf for dead rows) and rowsum(dO o O)
    int64_t sts[3];                // their b, h, row strides in elements (row stride 1 when queries are streamed)
    int B, H, nR;                  // nR: resident tiles
    int first_tile_first;          // launch order of a plane's tiles: 0 last tile first (queries), 1 first tile first (keys)
    float scale;                   // softmax scale / ln 2 (folded into x)
    float out_scale;               // softmax scale for dQ and dK, 1 for dV
};
hipError_t launch_bwd(const BwdParams &p, int dtype, int D, bool lane_stats, bool out_p, hipStream_t stream);

struct BwdPrepParams {
    const uint16_t *o, *d_o;
    const float *lse;
    int64_t os[3], dos[3], ls[3];
    float *stat_l, *stat_d;  // [B*H*Sq] each, contiguous
    int B, H, Sq;
};
hipError_t launch_bwd_prepare(const BwdPrepParams &p, int dtype, int D, hipStream_t stream);

}  // namespace sa
