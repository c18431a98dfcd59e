/*
 * sparseattn.h - C ABI of the MI355X (gfx950) block-sparse attention forward library
 * (libsparseattn_hip.so).
 *
 * The library replaces the two device kernels of tomatillos/sparseattention and nothing else:
 *
 *   sa_mask_classify          replaces the launch in compute_mask_kernel
 *                             (sparseattention/mask_utils.py:85-107, kernel :47-82)
 *   sa_sparse_attention_fwd   replaces the launch in sparse_attention
 *                             (sparseattention/sparse_attn_kernel.py:149-185, kernels :10-63, :74-146)
 *   sa_mask_pack_partial, sa_fwd_schedule, sa_sparse_attention_fwd_ex
 *                             optional accelerators of the same forward, prepared once per mask: the mask
 *                             entries of PARTIAL tiles packed to one bit each (read instead of the mask tile
 *                             loads of sparse_attn_kernel.py:42-46), and a schedule that deals the Q tiles
 *                             out to workgroups that stay resident (instead of the grid of
 *                             sparse_attn_kernel.py:167)
 *
 * Conventions
 *   - All pointers are DEVICE pointers owned by the caller.  The library allocates nothing,
 *     frees nothing and keeps no pointer after a call returns.
 *   - Strides are in ELEMENTS of the tensor they describe (bytes for the bool mask), exactly what
 *     torch.Tensor.stride() returns, and may be 0 on broadcast dimensions.
 *   - `stream` is a hipStream_t (NULL = the default stream).  Calls only enqueue work; they never
 *     synchronise the host with the device.
 *   - Return value: SA_OK or a negative SA_ERR_* code; sa_last_error() then gives a message
 *     (thread-local).  Argument errors are detected on the host before any kernel is launched.
 *   - Mask semantics: a byte != 0 means "this query may attend to this key" (torch bool masks).
 *     A tile of BQ x BK entries is FULL when every entry is set, EMPTY when none is, otherwise
 *     PARTIAL (mask_utils.py:34-40).
 */
#ifndef SPARSEATTN_H
#define SPARSEATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SA_ABI_VERSION 14

enum sa_status {
    SA_OK = 0,
    SA_ERR_INVALID_ARGUMENT = -1, /* null pointer, non-positive size, Sq % BQ != 0, Sk % BK != 0 ... */
    SA_ERR_UNSUPPORTED = -2,      /* valid request the gfx950 kernels have no instantiation for */
    SA_ERR_WORKSPACE = -3,        /* workspace missing or smaller than sa_mask_classify_workspace_bytes */
    SA_ERR_HIP = -4               /* the HIP runtime refused the launch */
};

enum sa_dtype {
    SA_DTYPE_BF16 = 0,
    SA_DTYPE_FP16 = 1,
    SA_DTYPE_FP32 = 2 /* the forward entry points only (sa_sparse_attention_fwd, _fwd_ex, _fwd_lse) */
};

/* Conditions of one term of a mask given by a formula (sa_mask_classify_terms). */
enum sa_term_flags {
    SA_TERM_BACK = 1,     /* (q + offset) - k < back                                   */
    SA_TERM_AHEAD = 2,    /* k - (q + offset) < ahead        (ahead = 1: causal)       */
    SA_TERM_Q_RANGE = 4,  /* q_lo <= q < q_hi                                          */
    SA_TERM_K_RANGE = 8,  /* k_lo <= k < k_hi                                          */
    SA_TERM_SAME_DOC = 16 /* doc_q[b][q] == doc_k[b][k]                                */
};
#define SA_MAX_MASK_TERMS 8

enum sa_schedule_mode {
    SA_SCHEDULE_PERSISTENT = 0, /* as many workgroups as the device holds at once, each walks many Q tiles */
    SA_SCHEDULE_PAIRS = 1       /* one workgroup per two Q tiles, a long list with a short one under causal masks */
};

/* ABI version of the loaded library (== SA_ABI_VERSION it was built with). */
int sa_abi_version(void);

/* Message for the last error returned on the calling thread ("" if none). */
const char *sa_last_error(void);

/*
 * Bytes of device scratch sa_mask_classify needs for this problem: one class byte per tile of
 * every DISTINCT mask plane (dimensions whose mask stride is 0 count once).  Returns 0 on
 * invalid arguments.
 */
size_t sa_mask_classify_workspace_bytes(const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ,
                                        int BK);

/*
 * Tile classification.  Replaces compute_mask_kernel's launch (mask_utils.py:96-106).
 *
 *   mask        bool [B,H,Sq,Sk] addressed through mask_strides (any strides, 0 allowed).
 *   full_ids    int32 [B,H,Sq/BQ,Sk/BK]: ascending KV-tile indices of FULL tiles ("unmasked_kv_ids");
 *   full_lens   int32 [B,H,Sq/BQ]: how many of them are valid ("unmasked_lens");
 *   part_ids / part_lens: the same for PARTIAL tiles ("masked_kv_ids", "masked_lens").
 *               Slots at positions >= the count are left untouched, as in the reference, which
 *               allocates them with torch.empty (mask_utils.py:91-94).
 *   Output strides may be 0 on b and/or h when the mask's stride is 0 there (the result is the
 *   same for every plane; it is then computed and written once).
 *   workspace   device scratch of at least sa_mask_classify_workspace_bytes(...) bytes; contents
 *               need not be initialised and are garbage afterwards.
 *
 * Any BQ, BK with Sq % BQ == 0 and Sk % BK == 0 is accepted.  Masks whose last dimension is
 * contiguous and 16-byte aligned with 16 <= BK <= 1024, BK a power of two, take the wide-load
 * kernel; everything else takes a slower generic kernel with identical results.
 */
int sa_mask_classify(const uint8_t *mask, const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ,
                     int BK, int32_t *full_ids, const int64_t full_ids_strides[4], int32_t *full_lens,
                     const int64_t full_lens_strides[3], int32_t *part_ids, const int64_t part_ids_strides[4],
                     int32_t *part_lens, const int64_t part_lens_strides[3], void *workspace,
                     size_t workspace_bytes, void *stream);

/*
 * sa_mask_classify for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference: its launcher allocates its outputs with
 * torch.empty on every call (mask_utils.py:91-94) and has no scratch.  Same arguments, checks, kernels and results as
 * sa_mask_classify, without `workspace`: the class bytes go to a device array of SA_STATIC_CLASSIFY_MAX_TILES bytes
 * that belongs to the library (one copy per GPU it runs on, held until the process ends).  The call allocates and
 * frees nothing.  The first call on a device asks the runtime for that array's address (hipGetSymbolAddress) and keeps
 * it; make that first call outside a stream capture.
 *
 *   - More tiles over the distinct mask planes (sa_mask_classify_workspace_bytes) than SA_STATIC_CLASSIFY_MAX_TILES:
 *     SA_ERR_WORKSPACE, nothing is launched.
 *   - Every call on a GPU uses that GPU's one array: calls that may run at the same time on one GPU (two streams, two
 *     threads) race on it; order them on one stream or with events.  Nothing needs clearing between calls: every byte
 *     the second kernel reads is written by the first.
 */
#define SA_STATIC_CLASSIFY_MAX_TILES (1u << 20)
int sa_mask_classify_static(const uint8_t *mask, const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ,
                            int BK, int32_t *full_ids, const int64_t full_ids_strides[4], int32_t *full_lens,
                            const int64_t full_lens_strides[3], int32_t *part_ids,
                            const int64_t part_ids_strides[4], int32_t *part_lens,
                            const int64_t part_lens_strides[3], void *stream);

/*
 * Block-sparse flash-attention forward.  Replaces sparse_attention_kernel's launch
 * (sparse_attn_kernel.py:167-184).
 *
 *   q,o  [B,H,Sq,D]; k,v [B,H,Sk,D]; dtype selects bf16 or fp16 for all four.  The last
 *   dimension must be contiguous (stride 1), every other stride a multiple of 8 elements and
 *   the base pointers 16-byte aligned; otherwise SA_ERR_UNSUPPORTED (copy to a contiguous tensor).
 *   mask and the four metadata tensors are as in sa_mask_classify; only ids[..., :len] are read.
 *   sm_scale_log2 = softmax scale divided by ln 2 (the reference uses D^-0.5 / ln 2,
 *   sparse_attn_kernel.py:152); scores are exponentiated with exp2.
 *
 * For each query tile: FULL tiles first without reading the mask, then PARTIAL tiles with the
 * mask applied, online softmax state in fp32, P rounded to the input dtype before P.V
 * (sparse_attn_kernel.py:61).  Rows with no attended key produce 0 (the reference produces NaN).
 *
 * Supported: D in {64,128,256}; BQ in {32,64,128,256} (64 and 128 at D = 256, where a given schedule is not used);
 * BK a power of two >= 16.
 * dtype SA_DTYPE_FP32 (the reference's kernel takes whatever element type its inputs have,
 * sparse_attn_kernel.py:98-101, :145): q, k, v, o are float, strides multiples of 4 elements; a plain kernel on the
 * vector units that keeps everything in float32 (P is not rounded), for checks against fp32 references, not for speed;
 * any BQ from 1 to 256 (to 128 at D = 256) and any BK that divide Sq and Sk; a schedule is not used.
 * ids[..., :len] should hold valid KV-tile indices (< Sk/BK).  Counts are clamped to Sk/BK and an index outside
 * [0, Sk/BK) is skipped, as the reference's masked loads would (sparse_attn_kernel.py:35,39,60); sa_validate_metadata
 * tells whether that happened.
 */
int sa_sparse_attention_fwd(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                            const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                            const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                            const int64_t full_ids_strides[4], const int32_t *full_lens,
                            const int64_t full_lens_strides[3], const int32_t *part_ids,
                            const int64_t part_ids_strides[4], const int32_t *part_lens,
                            const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk, int D, int BQ, int BK,
                            int dtype, float sm_scale_log2, void *stream);

/*
 * Check of caller-supplied lists before they are handed to a forward, decode or backward call or to
 * sa_mask_pack_partial, on the device and without a host synchronisation: the counterpart of the guard the reference puts on every K/V and mask load
 * (kv_offset < SEQLEN_K, sparse_attn_kernel.py:35,39,60).  ORs into *flag (a device int32 the caller has set to 0):
 *   1  a count is negative, or full_len + part_len exceeds Sk/BK for some Q tile
 *   2  a FULL index inside its count is outside [0, Sk/BK)      4  the same for a PARTIAL index
 * The caller reads the flag when it likes (with the results, say).  The kernels do not depend on it: they clamp
 * counts to the row of tiles and skip (forward, sa_mask_pack_partial) or clamp (decode, backward) indices out of range,
 * so lists that fail this check give wrong numbers (or unwritten packed slots), never an access outside the tensors.
 */
int sa_validate_metadata(const int32_t *full_ids, const int64_t full_ids_strides[4], const int32_t *full_lens,
                         const int64_t full_lens_strides[3], const int32_t *part_ids, const int64_t part_ids_strides[4],
                         const int32_t *part_lens, const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk,
                         int BQ, int BK, int32_t *flag, void *stream);

/*
 * Bytes of the buffer sa_mask_pack_partial fills: Sq*Sk/8 for every DISTINCT mask plane (room for every
 * tile being PARTIAL, so that no count has to be read back to the host).  Returns 0 on invalid arguments
 * (BK must be a multiple of 8).
 */
size_t sa_mask_pack_partial_bytes(const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ, int BK);

/*
 * One bit per mask entry of every PARTIAL tile.  No counterpart in the reference, which re-reads the bool
 * tile in every forward (sparse_attn_kernel.py:42-46); the reference README lists cheaper mask storage as
 * an open problem (README.md:12, :63).
 *
 *   mask, part_ids, part_lens   as in sa_mask_classify, whose outputs the two lists must be (run on the
 *                               same stream before this call).
 *   packed           device buffer of sa_mask_pack_partial_bytes(...) bytes.  For the distinct plane
 *                    (b, h) the tile that is entry `slot` of the PARTIAL list of Q tile `qt` lies at
 *                        packed + b*packed_strides[0] + h*packed_strides[1] + (qt*(Sk/BK) + slot) * BQ*BK/8
 *                    as BQ*BK/8 bytes, rows first: entry (r, c) of the tile is bit (c & 7) of byte
 *                    (r*BK + c) >> 3, set when the mask byte is non-zero.  Slots >= the count are left
 *                    untouched.
 *   packed_strides   bytes between planes along b and h; give 0 where the mask stride is 0 (that
 *                    dimension is then packed once).
 */
int sa_mask_pack_partial(const uint8_t *mask, const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ,
                         int BK, const int32_t *part_ids, const int64_t part_ids_strides[4],
                         const int32_t *part_lens, const int64_t part_lens_strides[3], uint8_t *packed,
                         const int64_t packed_strides[2], void *stream);

/*
 * Classification (and optionally the packed PARTIAL tiles) of a mask that is given by a formula instead of a tensor:
 * the same outputs as sa_mask_classify + sa_mask_pack_partial on the materialised mask, without the Sq x Sk tensor.
 * The reference parses tensors only (mask_utils.py:85-107) and names algebraic masks, and the memory they save, as
 * what could come next (README.md:12, :63).  With the packed tiles the forward (sa_sparse_attention_fwd_ex,
 * mask = NULL) and the backward (q_packed / k_packed) need no mask tensor at all.
 *
 * Entry (b, h, q, k) attends when ANY of the n_terms terms holds; a term holds when ALL the conditions its flags
 * switch on hold (enum sa_term_flags).  The mask does not depend on h, and on b only through the documents.
 *
 *   terms            HOST pointer: int32 [n_terms][8] = {flags, offset, back, ahead, q_lo, q_hi, k_lo, k_hi};
 *                    1 <= n_terms <= SA_MAX_MASK_TERMS.  Causal: {SA_TERM_AHEAD, 0, 0, 1, ...}; causal window of w
 *                    keys: {SA_TERM_BACK | SA_TERM_AHEAD, 0, w, 1, ...}; with Sq != Sk, offset = Sk - Sq aligns the
 *                    last query with the last key.  The transposed mask (keys as rows) is the same formula with
 *                    offset negated, back and ahead swapped, the ranges swapped and doc_q, doc_k swapped.
 *   doc_q, doc_k     device int32 [B, Sq] and [B, Sk] document numbers with strides in elements (batch stride 0: shared
 *                    by the batch), or NULL when no term has SA_TERM_SAME_DOC
 *   lists            as in sa_mask_classify; the head stride may always be 0, the batch stride only when the documents
 *                    do not differ between batch elements
 *   packed           optional (NULL: lists only): as in sa_mask_pack_partial; plane (b, 0) is written for every
 *                    distinct b, packed_strides[1] must be 0 when H > 1, base and batch stride multiples of 4 bytes
 *   workspace        sa_mask_terms_workspace_bytes(distinct batch planes, ...) bytes of device memory
 * BLOCK_K: a power of two >= 16.
 */
size_t sa_mask_terms_workspace_bytes(int distinct_b, int Sq, int Sk, int BQ, int BK);
int sa_mask_classify_terms(const int32_t *terms, int n_terms, const int32_t *doc_q, const int64_t doc_q_strides[2],
                           const int32_t *doc_k, const int64_t doc_k_strides[2], int B, int H, int Sq, int Sk, int BQ,
                           int BK, int32_t *full_ids, const int64_t full_ids_strides[4], int32_t *full_lens,
                           const int64_t full_lens_strides[3], int32_t *part_ids, const int64_t part_ids_strides[4],
                           int32_t *part_lens, const int64_t part_lens_strides[3], uint8_t *packed,
                           const int64_t packed_strides[2], void *workspace, size_t workspace_bytes, void *stream);

/*
 * Schedule of the forward: which Q tiles a workgroup processes, in order.  No counterpart in the reference, whose
 * grid is one program per Q tile (sparse_attn_kernel.py:167).  A workgroup that walks several Q tiles runs one
 * chunk stream across them: the next tile's first K/V rows, its queries and its list are on their way while the
 * current tile is computed, so the start-up latencies of a workgroup (arguments, counts, lists, first K/V tiles,
 * dispatch) are paid once per workgroup instead of once per Q tile.
 *
 *   SA_SCHEDULE_PAIRS       one workgroup per two Q tiles of a pair of planes, tile r from the top with tile r
 *                           from the bottom; the hardware dispatcher still balances the workgroups.
 *   SA_SCHEDULE_PERSISTENT  two workgroups per compute unit of the CURRENT device; the Q tiles are dealt out in
 *                           rounds by their cost (the list lengths), costliest tile to the least loaded workgroup.
 *
 * sa_fwd_schedule_bytes   size of the schedule buffer; 0 when the forward has no kernel for scheduled tiles at
 *                         these sizes (BQ must be 32, 64 or 128, BK a power of two >= 16 with Sk/BK <= 1024), on
 *                         invalid arguments, or (persistent mode) without a device.
 * sa_fwd_schedule         fills it from the two count tensors of sa_mask_classify (same stream, after it).  The
 *                         result depends on the counts, B, H, the tile sizes, the mode and (persistent mode) the
 *                         device only: compute it once per mask and reuse it for every forward over that mask.
 */
size_t sa_fwd_schedule_bytes(int B, int H, int Sq, int Sk, int BQ, int BK, int mode);
int sa_fwd_schedule(const int32_t *full_lens, const int64_t full_lens_strides[3], const int32_t *part_lens,
                    const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk, int BQ, int BK, int mode,
                    int32_t *schedule, size_t schedule_bytes, void *stream);

/*
 * sa_sparse_attention_fwd with the optional accelerators; results are bit-identical to it.
 *
 *   packed, packed_strides   output of sa_mask_pack_partial for the same mask, tile sizes and lists (strides may
 *                            be 0 on broadcast dimensions), or NULL.  When given, `mask` is not read and may be
 *                            NULL, so the bool tensor can be released once the lists and the packed bits exist.
 *   schedule, schedule_bytes, schedule_mode
 *                            output of sa_fwd_schedule for the same counts, sizes and mode (on this device), or
 *                            NULL (then, and when schedule_bytes is not sa_fwd_schedule_bytes(...), one
 *                            workgroup per Q tile is launched as in sa_sparse_attention_fwd).
 */
int sa_sparse_attention_fwd_ex(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                               const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                               const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                               const int64_t full_ids_strides[4], const int32_t *full_lens,
                               const int64_t full_lens_strides[3], const int32_t *part_ids,
                               const int64_t part_ids_strides[4], const int32_t *part_lens,
                               const int64_t part_lens_strides[3], const uint8_t *packed,
                               const int64_t packed_strides[2], const int32_t *schedule, size_t schedule_bytes,
                               int schedule_mode, int B, int H, int Sq, int Sk, int D, int BQ, int BK, int dtype,
                               float sm_scale_log2, void *stream);

/*
 * sa_sparse_attention_fwd_ex with a second output: lse[b,h,row] = ln sum over the attended keys of
 * exp(q.k * softmax scale), float32, -inf for rows that attend to nothing (what a caller needs to merge results
 * over disjoint key ranges, or to run a backward pass; the reference keeps the row maximum and sum in registers,
 * sparse_attn_kernel.py:107-108, and drops them after the division at :144).  lse, lse_strides (elements; b, h,
 * row) may be NULL: then this is sa_sparse_attention_fwd_ex.  `o` is bit-identical either way.
 */
int sa_sparse_attention_fwd_lse(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                                const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                                const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                                const int64_t full_ids_strides[4], const int32_t *full_lens,
                                const int64_t full_lens_strides[3], const int32_t *part_ids,
                                const int64_t part_ids_strides[4], const int32_t *part_lens,
                                const int64_t part_lens_strides[3], const uint8_t *packed,
                                const int64_t packed_strides[2], const int32_t *schedule, size_t schedule_bytes,
                                int schedule_mode, float *lse, const int64_t lse_strides[3], int B, int H, int Sq,
                                int Sk, int D, int BQ, int BK, int dtype, float sm_scale_log2, void *stream);

/*
 * sa_sparse_attention_fwd_lse (without a schedule) with the choice of the kernel that runs it.  No counterpart in the
 * reference, whose one kernel is tuned by Triton's autotuner over eight configurations at its first call
 * (sparse_attn_kernel.py:66-72); here the caller, who knows the mask, chooses.
 *
 *   SA_FWD_KERNEL_DEFAULT      what sa_sparse_attention_fwd runs: two workgroups per compute unit, 64 keys per step;
 *                              the fastest form for lists of some tens of KV tiles and more.
 *   SA_FWD_KERNEL_SHORT_LISTS  three workgroups per compute unit, 32 keys per step, K/V requested two steps ahead:
 *                              for masks that leave a Q tile few KV tiles (a Q tile then spends much of its life
 *                              waiting for its first loads, which a third resident workgroup covers).  Needs bf16 or
 *                              fp16, D = 128, BQ = 128 and the packed PARTIAL tiles (else SA_ERR_UNSUPPORTED), and it
 *                              reads at most SA_FWD_SHORT_LISTS_MAX_ENTRIES entries of a Q tile's two lists taken
 *                              together (FULL entries first): the caller must know that no list is longer, e.g. from
 *                              the counts of sa_mask_classify.
 *   SA_FWD_KERNEL_ROTATED_BY(G)  the default kernel, with Q tile qt walking its FULL entries (all but the first chunk
 *                              of 64 keys) from a start BQ/64 * (G - 1 - qt mod G) chunks further on, wrapping
 *                              around; 2 <= G <= 64, a power of two (a Q tile whose FULL list is shorter than the
 *                              largest start halves G until it fits); bf16 or fp16 (else SA_ERR_UNSUPPORTED).
 *                              For banded masks (sliding windows): the windows of neighbouring Q tiles
 *                              are BQ keys apart, so walked from the front they read the same K/V rows two chunks
 *                              apart and find them evicted from L2; walked this way G neighbours read them at the
 *                              same time.  The reference fixes FULL entries before PARTIAL ones
 *                              (sparse_attn_kernel.py:113-142), which stays; the order inside the FULL list is its
 *                              list order there and this rotation of it here.
 * All compute the same function; their results differ by rounding only (the keys meet the online softmax in other
 * groupings or another order).
 */
enum sa_fwd_kernel { SA_FWD_KERNEL_DEFAULT = 0, SA_FWD_KERNEL_SHORT_LISTS = 1, SA_FWD_KERNEL_ROTATED = 2 };
#define SA_FWD_KERNEL_ROTATED_BY(G) (SA_FWD_KERNEL_ROTATED | ((G) << 8))
#define SA_FWD_SHORT_LISTS_MAX_ENTRIES 256
int sa_sparse_attention_fwd_kernel(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                                   const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                                   const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                                   const int64_t full_ids_strides[4], const int32_t *full_lens,
                                   const int64_t full_lens_strides[3], const int32_t *part_ids,
                                   const int64_t part_ids_strides[4], const int32_t *part_lens,
                                   const int64_t part_lens_strides[3], const uint8_t *packed,
                                   const int64_t packed_strides[2], float *lse, const int64_t lse_strides[3], int B,
                                   int H, int Sq, int Sk, int D, int BQ, int BK, int dtype, float sm_scale_log2,
                                   int kernel, void *stream);

/*
 * The forward for few query rows against a long K/V (decode): Sq <= 32 rows form the single Q tile of every (b, h),
 * BLOCK_Q = Sq.  The result is that of sparse_attention (sparseattention/sparse_attn_kernel.py:149-185) called with
 * BLOCK_Q = Sq; the reference has no kernel of its own for this shape ("Backwards pass + decode kernels" is item 3
 * of its README's list of what could come next, README.md:65), and its one-program-per-Q-tile launch
 * (sparse_attn_kernel.py:166) would leave one program per (b, h).  Here the list of every (b, h) is cut into
 * num_splits ranges of 32-key chunks, one workgroup each, and a second kernel merges the partial results.
 *
 *   lists        output of sa_mask_classify for the same mask with BQ = Sq: shapes [B,H,1,Sk/BK] and [B,H,1]
 *                (stride entry 2 is ignored)
 *   BK           power of two >= 16
 *   num_splits   workgroups per (b, h), 1..256, or 0 for sa_decode_num_splits(...)
 *   workspace    sa_decode_workspace_bytes(...) bytes of device memory, 16-byte aligned (may be NULL when that is 0,
 *                i.e. for one split); contents on return are unspecified
 *   lse, lse_strides   optional second output as in sa_sparse_attention_fwd_lse, or NULL
 * q, k, v, o, D, dtype, sm_scale_log2, stream: as for sa_sparse_attention_fwd.
 */
int sa_decode_num_splits(int B, int H, int Sq, int Sk, int BK);
size_t sa_decode_workspace_bytes(int B, int H, int Sq, int D, int num_splits);
int sa_sparse_attention_decode(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                               const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                               const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                               const int64_t full_ids_strides[4], const int32_t *full_lens,
                               const int64_t full_lens_strides[3], const int32_t *part_ids,
                               const int64_t part_ids_strides[4], const int32_t *part_lens,
                               const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk, int D, int BK,
                               int dtype, float sm_scale_log2, int num_splits, void *workspace, size_t workspace_bytes,
                               float *lse, const int64_t lse_strides[3], void *stream);

/*
 * sa_sparse_attention_decode with the bit-packed PARTIAL tiles (sa_mask_pack_partial with BQ = Sq for the same mask and
 * lists; strides may be 0 on broadcast dimensions), or NULL.  When given, `mask` is not read and may be NULL, so the
 * metadata that sa_mask_classify + sa_mask_pack_partial make for a mask serves the few-rows kernels as it serves the
 * forward, and the bool tensor can be released.  At BK = 16 the packed rows are halfwords: Sq must then be even.
 * Results are bit-identical to sa_sparse_attention_decode.
 */
int sa_sparse_attention_decode_ex(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                                  const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                                  const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                                  const int64_t full_ids_strides[4], const int32_t *full_lens,
                                  const int64_t full_lens_strides[3], const int32_t *part_ids,
                                  const int64_t part_ids_strides[4], const int32_t *part_lens,
                                  const int64_t part_lens_strides[3], const uint8_t *packed,
                                  const int64_t packed_strides[2], int B, int H, int Sq, int Sk, int D, int BK, int dtype,
                                  float sm_scale_log2, int num_splits, void *workspace, size_t workspace_bytes, float *lse,
                                  const int64_t lse_strides[3], void *stream);

/*
 * Merge of n attention results over disjoint key ranges of the same queries (what sharding the key axis over
 * devices, or over launches, ends with; the reference has no counterpart - it never hands out the row statistics):
 *   o = sum_i exp(lse_i - lse) o_i,   lse = log sum_i exp(lse_i)     (rows with every lse_i = -inf give 0 and -inf)
 * o_parts [n,B,H,Sq,D] and lse_parts [n,B,H,Sq] are outputs of sa_sparse_attention_fwd_lse (or of the decode entry)
 * for the n key ranges; strides in elements, last dimension of o_parts and o contiguous.  lse may be NULL.
 */
int sa_merge_attention_parts(const void *o_parts, const int64_t o_parts_strides[5], const float *lse_parts,
                             const int64_t lse_parts_strides[4], void *o, const int64_t o_strides[4], float *lse,
                             const int64_t lse_strides[3], int n, int B, int H, int Sq, int D, int dtype,
                             void *stream);

/*
 * Backward pass: dq, dk, dv from the upstream gradient d_o, for the function sa_sparse_attention_fwd computes
 * (sparseattention/sparse_attn_kernel.py:149-185).  The reference has none ("Backwards pass + decode kernels",
 * README.md:65); the derivative is the textbook one: P = exp(S - lse), dV = P^T dO, dP = dO V^T,
 * dS = P o (dP - rowsum(dO o O)), dQ = scale dS K, dK = scale dS^T Q.
 *
 *   o, lse          outputs of sa_sparse_attention_fwd_lse for the same q, k, v, mask
 *   q_* lists       sa_mask_classify of the mask with BQ = 128, BK = 64:  ids [B,H,Sq/128,Sk/64], lens [B,H,Sq/128]
 *   k_* lists       sa_mask_classify of the TRANSPOSED mask (strides 2 and 3 swapped, Sq and Sk swapped) with
 *                   BQ = 128, BK = 64:  ids [B,H,Sk/128,Sq/64], lens [B,H,Sk/128]
 *   mask_t          optional: the transposed mask as a tensor [B,H,Sk,Sq] of its own (broadcast strides allowed), or
 *                   NULL.  With it the dK and dV passes read the entries of PARTIAL tiles four at a time instead
 *                   of byte-wise down the columns of `mask`.
 *   q_packed, k_packed   optional: outputs of sa_mask_pack_partial for the two tilings above (the mask with BQ = 128,
 *                   BK = 64 and the q_* lists; the transposed mask with BQ = 128, BK = 64 and the k_* lists), or
 *                   NULL.  A pass that has its packed buffer reads no mask; with both, `mask` and `mask_t` may be
 *                   NULL, so the bool tensors can be released after preprocessing.
 *   workspace       sa_bwd_workspace_bytes(B, H, Sq) bytes of device memory, 16-byte aligned
 * D = 64 or 128, bf16 or fp16, Sq and Sk multiples of 128; tensors as for the forward (last dimension contiguous).
 * The tile sizes of the backward are its own: they need not be those the forward ran with.
 */
size_t sa_bwd_workspace_bytes(int B, int H, int Sq);
int sa_sparse_attention_bwd(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                            const void *v, const int64_t v_strides[4], const void *o, const int64_t o_strides[4],
                            const void *d_o, const int64_t do_strides[4], const float *lse,
                            const int64_t lse_strides[3], void *dq, const int64_t dq_strides[4], void *dk,
                            const int64_t dk_strides[4], void *dv, const int64_t dv_strides[4], const uint8_t *mask,
                            const int64_t mask_strides[4], const uint8_t *mask_t, const int64_t mask_t_strides[4],
                            const uint8_t *q_packed, const int64_t q_packed_strides[2], const uint8_t *k_packed,
                            const int64_t k_packed_strides[2], const int32_t *q_full_ids,
                            const int64_t q_full_ids_strides[4], const int32_t *q_full_lens,
                            const int64_t q_full_lens_strides[3], const int32_t *q_part_ids,
                            const int64_t q_part_ids_strides[4], const int32_t *q_part_lens,
                            const int64_t q_part_lens_strides[3], const int32_t *k_full_ids,
                            const int64_t k_full_ids_strides[4], const int32_t *k_full_lens,
                            const int64_t k_full_lens_strides[3], const int32_t *k_part_ids,
                            const int64_t k_part_ids_strides[4], const int32_t *k_part_lens,
                            const int64_t k_part_lens_strides[3], void *workspace, size_t workspace_bytes, int B,
                            int H, int Sq, int Sk, int D, int dtype, float sm_scale_log2, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SPARSEATTN_H */
