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
// LDS: two buffers each for K and V (64 rows per buffer), filled straight from global memory
// (global_load_lds_dwordx4, 1 KiB per wave instruction) one chunk ahead of the MFMAs.  Rows are
// unpadded; bank conflicts are avoided by XOR-swizzling the 16-byte pieces of a row (k_swizzle,
// v_swizzle).
#pragma once
#include "fwd_common.h"

namespace sa {

namespace {

// Issue priority of a wave by phase of its chunk (s_setprio; 0 outside the two phases).  The two waves that share
// a SIMD both want the matrix pipe most of the time; served alternately they leave their MFMA phases together and
// then do their vector and scalar work together, with the pipe idle.  Letting the wave in its P.V phase (MFMAs
// with exponentials between them) go ahead of one in its S phase (MFMAs only), and either ahead of the
// bookkeeping between chunks, keeps them apart: 3 % on the causal and 2 % on the dense workload at D = 128.
constexpr int kPrioS = 1;
constexpr int kPrioPV = 2;

// "At most n vector-memory operations of this wave still in flight", n a small run-time value.
__device__ __forceinline__ void wait_vm_at_most(int n, int step) {
    if (n <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (n == 1) {
        if (step == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else if (step == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if (step == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
        if (step == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if (step == 4) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else if (step == 8) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
}

// MODE 0: BK = 16, MODE 1: BK = 32, MODE 2: BK >= 64 (runtime log2 in p.lbk).
// NS: LDS stages per operand (2 or 4); chunks are fetched NS-1 ahead of the one being computed.
// PP: the two waves that share a SIMD (w and w+4 of an 8-wave workgroup) run half a chunk apart, one in its
// S phase while the other is in its P.V phase (see the main loop).
// PK: the mask entries of PARTIAL tiles come bit-packed from p.packed (one bit per entry, rows first) instead of
// from the bool mask.
// PS: persistent workgroups.  The grid is as large as the device holds at once, and every workgroup walks its own
// row of p.sched (Q tiles dealt out by schedule_kernel).  The chunk stream runs on across Q tiles: while the last
// chunk of one tile is computed, the first chunk of the next is fetched and its queries are loaded, and the
// lists of the tiles after that are on their way, so that the latencies a fresh workgroup would pay one after
// the other (arguments, counts, lists, first K/V chunk) are paid once per workgroup instead of once per tile.
template <int DT, int D, int NW, int MODE, int NS, bool PP, bool PK, bool PS>
__global__ __launch_bounds__(NW * 64, (NW >= 4 && D <= 128) ? 2 : 1) void sparse_fwd_kernel(const FwdParams p) {
    static_assert(!PS || (!PP && NS == 2), "persistent workgroups use the two-stage loop");
    using E = Elem<DT>;
    constexpr int ROWB = D * 2;                   // bytes per K/V row in LDS
    constexpr int KBUF = 64 * ROWB, VBUF = 64 * ROWB;
    constexpr int RPI = 1024 / ROWB;              // rows written by one wave-wide direct load (1 KiB)
    constexpr int NLD = 64 / (RPI * NW);          // direct loads per wave per chunk, each for K and for V
    constexpr int PPR = ROWB / 16;                // 16-byte pieces per row
    constexpr int EPC = MODE == 0 ? 4 : (MODE == 1 ? 2 : 1);  // list entries per chunk
    constexpr int LBKC = MODE == 0 ? 4 : 5;                   // log2(BK) when MODE < 2
    static_assert(64 % (RPI * NW) == 0, "staging layout");

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    static_assert(NS == 2 || NS == 4, "stage count");
    // [K stage 0..NS-1][V stage 0..NS-1][first key column of every list entry, kListCap ints]
    int *const ent = reinterpret_cast<int *>(smem + NS * KBUF + NS * VBUF);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;

    // Workgroup -> (b, h, Q tile).  Hardware hands consecutive workgroup ids to the 8 XCDs in turn; the
    // remap gives each XCD whole planes (every eighth pair of the (b,h)-major order) so that the Q tiles sharing one
    // K/V plane run on the XCD whose L2 already holds it.  Planes are taken two at a time with their Q tiles
    // interleaved, last Q tile first (under causal-like masks it has the longest list): the slots that finish
    // the short tiles of one pair then pick up the long tiles of the next, which evens out the load.
    // The Q tile at hand: plane (b, h), tile qt, F FULL and NE - F PARTIAL entries, T chunks.  A persistent
    // workgroup moves from tile to tile; the others keep the values they start with.
    int b, h, qt, F, NE, T;
    const uint16_t *kbase, *vbase;
    const uint8_t *mrow, *prow;
    const int32_t *fid, *pid;
    int64_t orow_off;  // this lane's first output element
    int64_t lse_off;   // this lane's row in p.lse
    // this lane's row in a packed tile: BK/8 bytes per row, NW*32 rows per tile
    const int64_t tile_bytes = (int64_t)(NW * 4) * p.BK;
    const int sh4 = 4 * hh;
    // (see the loads next to the counts below)
    constexpr bool kEarlyFirstChunk = !PS && !PP && D <= 128;  // (at D = 256 the registers are all taken)
    int early_f[EPC] = {}, early_p[EPC] = {};
    // what load_mask needs to know of a Q tile
    struct MaskSrc {
        const uint8_t *mrow, *prow;
        int F, NE;
    };
    auto mask_src_of = [&](int b_, int h_, int qt_, int F_, int NE_) -> MaskSrc {
        const int qrow_ = qt_ * (NW * 32) + wave * 32 + l32;  // the query row this lane owns
        MaskSrc m;
        m.mrow = p.mask + b_ * p.ms[0] + h_ * p.ms[1] + (int64_t)qrow_ * p.ms[2];
        m.prow = p.packed + b_ * p.pks[0] + h_ * p.pks[1] + (int64_t)qt_ * p.nK * tile_bytes +
                 (wave * 32 + l32) * (p.BK >> 3);
        m.F = F_;
        m.NE = NE_;
        return m;
    };
    auto chunks_of = [&](int ne) -> int {
        if constexpr (PS) {  // a tile without entries still runs one chunk of absent entries, which yields zeros
            return MODE == 2 ? ((ne > 0 ? ne : 1) << (p.lbk - 6)) : (ne > 0 ? (ne + EPC - 1) / EPC : 1);
        } else {
            return MODE == 2 ? (ne << (p.lbk - 6)) : ((ne + EPC - 1) / EPC);
        }
    };
    // Counts are clamped to the nK tiles a row of tiles has, and an index outside [0, nK) becomes an ABSENT entry
    // (tagged_entry, ps_list_deposit): the reference guards every K/V and mask load with kv_offset < SEQLEN_K
    // (sparse_attn_kernel.py:35,39,60), so stale or foreign metadata must not become an access outside K, V, the
    // packed tiles or the list's LDS copy.
    auto clamp_full = [&](int F_) -> int { return min(max(F_, 0), p.nK); };
    auto clamp_part = [&](int F_, int P_) -> int { return min(max(P_, 0), p.nK - clamp_full(F_)); };
    auto set_item = [&](int b_, int h_, int qt_, int F_, int P_) {
        b = b_;
        h = h_;
        qt = qt_;
        F = clamp_full(F_);
        NE = F + clamp_part(F_, P_);
        T = chunks_of(NE);
        kbase = p.k + b * p.ks[0] + h * p.ks[1];
        vbase = p.v + b * p.vs[0] + h * p.vs[1];
        const MaskSrc m = mask_src_of(b, h, qt, F, NE);
        mrow = m.mrow;
        prow = m.prow;
        fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + qt * p.fis[2];
        pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + qt * p.pis[2];
        const int qrow_ = qt * (NW * 32) + wave * 32 + l32;
        orow_off = b * p.os[0] + h * p.os[1] + (int64_t)qrow_ * p.os[2] + 4 * hh;
        lse_off = b * p.lses[0] + h * p.lses[1] + (int64_t)qrow_ * p.lses[2];
    };
    // Q^T operand: lane (l32, hh) keeps d = 16c + 8hh .. +7 of its query row for every 16-wide step c.
    u32x4 qf[D / 16];
    auto load_q = [&](int b_, int h_, int qt_) {
        const int qrow_ = qt_ * (NW * 32) + wave * 32 + l32;
        const uint16_t *qp = p.q + b_ * p.qs[0] + h_ * p.qs[1] + (int64_t)qrow_ * p.qs[2] + 8 * hh;
#pragma unroll
        for (int c = 0; c < D / 16; c++) qf[c] = *(const u32x4 *)(qp + 16 * c);
    };
    // The scale (softmax scale / ln 2) goes into Q once, so that the S MFMAs deliver exp2 arguments.
    auto scale_q = [&]() {
#pragma unroll
        for (int c = 0; c < D / 16; c++)
#pragma unroll
            for (int e = 0; e < 4; e++) qf[c][e] = E::scale2(qf[c][e], p.scale);
    };
    // Row of this workgroup in the schedule: entry 0 = {number of Q tiles, -, -, -}, then one entry
    // {(b << 16) | h, qt, F, P} per Q tile.
    const int4 *const sched_row = reinterpret_cast<const int4 *>(p.sched) + (int64_t)blockIdx.x * (p.sched_R + 1);
    int n_items = 1;
    if constexpr (PS) {
        n_items = __builtin_amdgcn_readfirstlane(sched_row[0].x);
        if (n_items <= 0) return;
        const int4 e0 = sched_row[1];
        const int bh0 = __builtin_amdgcn_readfirstlane(e0.x);
        set_item(bh0 >> 16, bh0 & 0xffff, __builtin_amdgcn_readfirstlane(e0.y), __builtin_amdgcn_readfirstlane(e0.z),
                 __builtin_amdgcn_readfirstlane(e0.w));
    } else {
        const int total = gridDim.x, per = total >> 3;
        int lin = blockIdx.x;
        if (lin < (per << 3)) lin = (lin & 7) * per + (lin >> 3);
        int pair = lin / (2 * p.nQ);
        const int r = lin - pair * 2 * p.nQ;
        // Which pairs of planes an XCD gets: every eighth one, so that a mask that differs between batch elements
        // (whose planes are neighbours in this order) loads the XCDs alike; a contiguous range when the pairs do
        // not divide evenly.
        if (((p.B * p.H) & 15) == 0) {
            const int ppx = (p.B * p.H) >> 4;  // pairs per XCD
            const int x = pair / ppx;
            pair = (pair - x * ppx) * 8 + x;
        }
        const bool paired = 2 * pair + 1 < p.B * p.H;  // the last plane of an odd count goes alone
        const int bh = 2 * pair + (paired ? (r & 1) : 0);
        const int qt0 = p.nQ - 1 - (paired ? (r >> 1) : r);
        const int b0 = bh / p.H, h0 = bh - b0 * p.H;
        // The queries come from HBM, the longest wait of a tile's start: requested first of all.  Then the counts and,
        // with them, the first slots of both lists (uniform addresses: scalar loads under one wait), so that the first
        // K/V chunk can be requested one memory round trip earlier, before the list has made its way to LDS.  Slots
        // past a count hold anything; early_entry() picks the ones that count.
        const int32_t *const fl0 = p.full_lens + (b0 * p.fls[0] + h0 * p.fls[1] + qt0 * p.fls[2]);
        const int32_t *const pl0 = p.part_lens + (b0 * p.pls[0] + h0 * p.pls[1] + qt0 * p.pls[2]);
        if constexpr (kEarlyFirstChunk) {
            load_q(b0, h0, qt0);
            const int32_t *f0 = p.full_ids + b0 * p.fis[0] + h0 * p.fis[1] + qt0 * p.fis[2];
            const int32_t *p0 = p.part_ids + b0 * p.pis[0] + h0 * p.pis[1] + qt0 * p.pis[2];
            const int32_t *addr[2 + 2 * EPC];
            int got[2 + 2 * EPC];
            addr[0] = fl0;
            addr[1] = pl0;
            static_for<EPC>([&](auto i_c) {
                constexpr int i = decltype(i_c)::value;
                const int slot = i < p.nK ? i : p.nK - 1;  // (a row of fewer than EPC tiles: stay inside it)
                addr[2 + i] = f0 + (int64_t)slot * p.fis[3];
                addr[2 + EPC + i] = p0 + (int64_t)slot * p.pis[3];
            });
            scalar_gather(addr, got);
            static_for<EPC>([&](auto i_c) {
                constexpr int i = decltype(i_c)::value;
                early_f[i] = got[2 + i];
                early_p[i] = got[2 + EPC + i];
            });
            set_item(b0, h0, qt0, got[0], got[1]);
        } else {
            set_item(b0, h0, qt0, *fl0, *pl0);
        }
    }

    // (the plain loop requests its first K/V chunk and its list before its queries, see there)
    if constexpr (!kEarlyFirstChunk) {
        load_q(b, h, qt);
        scale_q();
    }

    // Online-softmax state of this lane's query row.  Exponentials are taken against a reference value m_ref
    // (exp2 units).  The S MFMAs start from the accumulator -m_ref (neg_m: the same value in all 16 registers,
    // one query per lane), so a score leaves the matrix unit as the exp2 argument itself.  raise_above is the
    // largest such argument tolerated before m_ref moves: kMaxSlack, or "anything finite" until the row has
    // seen its first attended key.
    float m_ref = 0.f;
    float raise_above = -3.0e38f;
    f32x16 neg_m;
#pragma unroll
    for (int i = 0; i < 16; i++) neg_m[i] = 0.f;
    // Running row sums of P, kept by a 16x16x32 MFMA whose B operand is P itself.  In that instruction lane l
    // supplies column l%16 and key group l/16, so the P registers of query rows r and r+16 land in the same
    // column; the A operand separates them again: its row i is all ones over the key groups of parity i&1 and
    // zero elsewhere.  Result register 0 of lane l is then the row sum of query l%16 and register 1 that of
    // query l%16 + 16; a lane reads the one that belongs to its own row.
    f32x4 acc_l = {0.f, 0.f, 0.f, 0.f};
    const uint32_t sel1 = (((lane >> 4) ^ lane) & 1) == 0 ? E::ones4().x : 0u;
    const u32x4 sum_sel = {sel1, sel1, sel1, sel1};
    f32x16 acc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.f;

    // ---- per-lane LDS offsets (bytes, relative to the start of a K or V buffer) -------------------
    // K operand of step c: row 32kb + l32, piece 2c + hh, swizzled.  (2c + hh) ^ s == (2c) ^ (hh ^ s).
    int koff[D / 16];
    {
        const int t = hh ^ k_swizzle<D>(l32);
#pragma unroll
        for (int c = 0; c < D / 16; c++) koff[c] = l32 * ROWB + 16 * ((2 * c) ^ t);
    }
    // V^T operand (transposing read): within each 16-lane group, lane t supplies the address of 4
    // consecutive d of key row (t >> 2) and receives the 4 key rows of d column t.
    int voff[D / 32];
    {
        const int tr_row = 4 * hh + ((lane & 15) >> 2);        // + 16kc (+8 for the second read)
        const int x = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);  // piece within the 32-wide d block
        const int sw = v_swizzle<D>(tr_row) >> 2;               // 16kc and 8 leave the swizzle bits alone
#pragma unroll
        for (int db = 0; db < D / 32; db++) voff[db] = tr_row * ROWB + 64 * (db ^ sw) + 16 * x + 8 * (lane & 1);
    }
    // Direct-load staging: load i of this wave fills rows [RPI*(NW*i + wave), +RPI) of the chunk; lane
    // writes row ld_row(i), LDS piece lane % PPR, and therefore fetches the swizzled source piece.
    // The source address splits into a wave-uniform part (plane base + first row of the list entry, scalar
    // arithmetic per chunk) and a per-lane byte offset that never changes (row within the entry, swizzled
    // piece), so staging a chunk costs no vector arithmetic.
    const int ld_r0 = lane / PPR, ld_slot = lane % PPR;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const SA_LDS uint8_t *)smem);
    uint32_t ld_koff[NLD], ld_voff[NLD];
#pragma unroll
    for (int i = 0; i < NLD; i++) {
        const int r = RPI * (NW * i + wave_u) + ld_r0;
        const int within = MODE == 2 ? r : (r & ((1 << LBKC) - 1));
        ld_koff[i] = (uint32_t)((within * p.ks[2] + 8 * (ld_slot ^ k_swizzle<D>(r))) * 2);
        ld_voff[i] = (uint32_t)((within * p.vs[2] + 8 * (ld_slot ^ v_swizzle<D>(r))) * 2);
    }

    // The Q tile's list (FULL entries, then PARTIAL entries) as first key columns, copied to LDS once:
    // loads issued after the first barrier cannot use the scalar cache, and a vector load of an index in
    // front of every chunk would put a full memory round trip on the critical path.
    // Every entry carries its kind in the top bits, and the list is padded with ABSENT entries to whole chunks, so
    // that a chunk's entries say by themselves which of them exist and which are PARTIAL:
    //   bits 0..29 first key column, bit 30 PARTIAL, bit 31 ABSENT (column 0: its scores are discarded).
    constexpr int kPartialBit = 1 << 30;
    constexpr int kAbsent = (int)0x80000000u;
    const int list_cnt = MODE == 2 ? NE : (NE + EPC - 1) / EPC * EPC;
    const bool list_in_lds = !PS && list_cnt <= kListCap;
    // (the strides as scalars, read here: left inside the lane-dependent branch below they are fetched from the
    // argument block by a vector load of their own, a memory round trip in front of every list load)
    int64_t fis3 = p.fis[3], pis3 = p.pis[3];
    asm volatile("" : "+s"(fis3), "+s"(pis3));
    auto tagged_entry = [&](int e) -> int {  // from global memory
        if (e >= NE) return kAbsent;
        const int idx = e < F ? fid[(int64_t)e * fis3] : pid[(int64_t)(e - F) * pis3];
        if ((unsigned)idx >= (unsigned)p.nK) return kAbsent;
        return (MODE == 2 ? (idx << p.lbk) : (idx << LBKC)) | (e >= F ? kPartialBit : 0);
    };
    // list slot E of the tile's first chunk, from the slots that came with the counts, tagged like an LDS entry
    auto early_entry = [&](auto e_c) -> int {
        constexpr int e = decltype(e_c)::value;
        if (e >= NE) return kAbsent;
        int idx = early_f[e];
        if (e >= F) {
            idx = early_p[0];
            static_for<e>([&](auto j_c) {  // e - F is one of 0 .. e
                constexpr int j = decltype(j_c)::value + 1;
                // (a value that passed through an asm statement is no array element any more: the compiler would
                // otherwise fold this chain of selects into one load at a variable index, from scratch memory)
                int cand = __builtin_amdgcn_readfirstlane(early_p[j]);
                asm volatile("" : "+s"(cand));
                if (e - F == j) idx = cand;
            });
        }
        if ((unsigned)idx >= (unsigned)p.nK) return kAbsent;
        return (MODE == 2 ? (idx << p.lbk) : (idx << LBKC)) | (e >= F ? kPartialBit : 0);
    };
    // Where list entry e goes in the LDS copy.  With p.rot = G > 0 the chunks that hold FULL entries only, but for the
    // first (requested before the list is copied), are walked from a start that depends on the Q tile: tile qt starts
    // BQ/64 * (G - 1 - qt mod G) chunks further on, wrapping around.  Neighbouring Q tiles of a banded mask (a sliding
    // window) have windows BQ keys apart and run at the same time; walked from the front they read the same keys two
    // chunks apart, with everything the other resident workgroups read in between, and find them gone from L2.
    // Walked this way G neighbours read the same keys at the same time.  The order inside a list changes the result by
    // rounding only (sparse_attn_kernel.py:113-142 fixes FULL entries before PARTIAL ones, which stays).
    const int rot_first = MODE == 2 ? 1 : EPC;                                    // entries of the first chunk
    const int rot_n = MODE == 2 ? max(F - 1, 0) : max((F / EPC) * EPC - EPC, 0);  // entries that take part
    int rot_by = 0;
    if (!PS && p.rot > 0 && rot_n > 0) {
        // the group shrinks (by halves) until its largest start lies inside the entries that take part: neighbours of a
        // band have lists of one length, so they agree on it
        constexpr int CPT = NW >= 2 ? NW / 2 : 1;  // chunks of 64 keys per Q tile height
        const int n_chunks = MODE == 2 ? (rot_n << (p.lbk - 6)) : rot_n / EPC;
        int G = p.rot;
        while (G > 1 && CPT * (G - 1) >= n_chunks) G >>= 1;
        const int chunks = CPT * (G - 1 - (qt % G));
        rot_by = (MODE == 2 ? (chunks >> (p.lbk - 6)) : chunks * EPC) % rot_n;
    }
    auto list_pos = [&](int e) -> int {
        if (PS || e < rot_first || e >= rot_first + rot_n) return e;
        int x = e - rot_first - rot_by;
        if (x < 0) x += rot_n;
        return rot_first + x;
    };
    auto copy_list = [&]() {
        if (list_in_lds) {
            for (int e = tid; e < list_cnt; e += NW * 64) ent[list_pos(e)] = tagged_entry(e);
        }
    };
    // First key column of every list entry in chunk t (t < T), plus which entries exist / are partial, in two
    // steps: entries_read issues the reads of the list (the values are the same in all lanes), entries_use turns
    // them into scalars.  The main loop reads the entries of a chunk one iteration before it needs them, so
    // that no wave waits for the list.
    auto entry_read = [&](int e) -> int {
        if (__builtin_expect(list_in_lds, 1)) return ent[e];
        return tagged_entry(e);
    };
    auto entries_read = [&](int t, int(&raw)[EPC]) {
        if constexpr (MODE == 2) {
            raw[0] = entry_read(t >> (p.lbk - 6));
        } else {
#pragma unroll
            for (int j = 0; j < EPC; j++) raw[j] = entry_read(t * EPC + j);
        }
    };
    auto entries_use = [&](int t, const int(&raw)[EPC], int(&col)[EPC], unsigned &valid, unsigned &part) {
        valid = 0u;
        part = 0u;
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            const int v = __builtin_amdgcn_readfirstlane(raw[j]);
            col[j] = v & (kPartialBit - 1);
            if constexpr (MODE == 2) col[j] += (t & ((1 << (p.lbk - 6)) - 1)) << 6;
            if (v >= 0) valid |= 1u << j;
            if (v & kPartialBit) part |= 1u << j;
        }
    };
    auto chunk_entries = [&](int t, int(&col)[EPC], unsigned &valid, unsigned &part) {
        int raw[EPC];
        entries_read(t, raw);
        entries_use(t, raw, col, valid, part);
    };
    // Persistent workgroups keep the lists of two Q tiles in LDS (kPsListCap entries each), every entry with its
    // kind in the top bits, padded with ABSENT entries to whole chunks:
    //   bits 0..29 first key column, bit 30 PARTIAL, bit 31 ABSENT.
    constexpr int NT = NW * 64;
    constexpr int PER = kPsListCap / NT;  // list entries per thread
    const int lbk_rt = MODE == 2 ? p.lbk : LBKC;
    auto ps_list_issue = [&](int b_, int h_, int qt_, int F_, int P_, int(&lr)[PER]) {  // indices -> registers
        const int32_t *f_ = p.full_ids + b_ * p.fis[0] + h_ * p.fis[1] + qt_ * p.fis[2];
        const int32_t *p_ = p.part_ids + b_ * p.pis[0] + h_ * p.pis[1] + qt_ * p.pis[2];
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int e = tid + NT * i;
            // slots past the count are read too (slot 0 of the row: always there) and flagged ABSENT on deposit
            const int32_t *a = e < F_ ? f_ + (int64_t)e * p.fis[3]
                                      : p_ + (int64_t)(e < F_ + P_ ? e - F_ : 0) * p.pis[3];
            lr[i] = *a;
        }
    };
    auto ps_list_deposit = [&](int F_, int P_, const int(&lr)[PER], int *dst) {  // registers -> LDS
        const int ne = F_ + P_;
        const int cnt = MODE == 2 ? (ne > 0 ? ne : 1) : chunks_of(ne) * EPC;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int e = tid + NT * i;
            if (e < cnt)
                dst[e] = (e >= ne || (unsigned)lr[i] >= (unsigned)p.nK) ? kAbsent
                                                                         : ((lr[i] << lbk_rt) | (e >= F_ ? kPartialBit : 0));
        }
    };
    auto ps_entries_read = [&](const int *el, int t, int(&raw)[EPC]) {
        if constexpr (MODE == 2) {
            raw[0] = el[t >> (p.lbk - 6)];
        } else {
#pragma unroll
            for (int j = 0; j < EPC; j++) raw[j] = el[t * EPC + j];
        }
    };
    auto ps_entries_use = [&](int t, const int(&raw)[EPC], int(&col)[EPC], unsigned &valid, unsigned &part) {
        valid = 0u;
        part = 0u;
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            const int v = __builtin_amdgcn_readfirstlane(raw[j]);
            col[j] = v & (kPartialBit - 1);
            if constexpr (MODE == 2) col[j] += (t & ((1 << (p.lbk - 6)) - 1)) << 6;
            if (v >= 0) valid |= 1u << j;
            if (v & kPartialBit) part |= 1u << j;
        }
    };

    // Global -> LDS for one chunk, without passing through registers: 2*NLD direct loads per wave (piece 2i is
    // load i of K, piece 2i+1 load i of V).  A wave that issues them back to back sits at the issue stage until
    // the address unit has taken them all, while every other wave of the CU does the same; the main loop
    // therefore hands them out one at a time between the MFMA bundles of the chunk being computed.
    struct StagePlan {
        const uint16_t *kp[EPC], *vp[EPC];  // first row of every list entry of the chunk (scalar registers)
    };
    // first row of a list entry as an element offset: key column and row stride are both below 2^32 (the strides
    // are checked on the host), so one 32 x 32 -> 64 bit product does
    const uint32_t ks2 = (uint32_t)p.ks[2], vs2 = (uint32_t)p.vs[2];
    auto row_off = [](int col, uint32_t stride) -> int64_t { return (int64_t)((uint64_t)(uint32_t)col * stride); };
    auto plan_chunk = [&](const int(&col)[EPC], StagePlan &pl) {
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            pl.kp[j] = kbase + row_off(col[j], ks2);
            pl.vp[j] = vbase + row_off(col[j], vs2);
        }
    };
    auto stage_piece = [&](int buf, int piece, const StagePlan &pl) {
        const int i = piece >> 1;
        // rows [rbase, rbase + RPI) lie inside one list entry; when the rows of all waves of load i do, the
        // entry is known at compile time
        constexpr bool kEntryByLoad = MODE == 2 || RPI * NW <= (1 << LBKC);
        const int rbase = RPI * (NW * i + wave_u);
        const uint16_t *ks_ = pl.kp[0], *vs_ = pl.vp[0];
        if constexpr (MODE != 2) {
            const int j = kEntryByLoad ? ((RPI * NW * i) >> LBKC) : (rbase >> LBKC);
#pragma unroll
            for (int jj = 1; jj < EPC; jj++) {
                const uint16_t *kc = pl.kp[jj], *vc = pl.vp[jj];
                // With more than two candidates and an entry that depends on the wave, the compiler would turn
                // this chain into one load at a variable index, which keeps the plan in scratch memory; values
                // that passed through an (empty) asm statement are no loads any more.
                if constexpr (!kEntryByLoad && EPC > 2) asm volatile("" : "+s"(kc), "+s"(vc));
                if (j == jj) {
                    ks_ = kc;
                    vs_ = vc;
                }
            }
        }
        if ((piece & 1) == 0) dma16(ks_, ld_koff[i], lds0 + buf * KBUF + rbase * ROWB);
        else dma16(vs_, ld_voff[i], lds0 + NS * KBUF + buf * VBUF + rbase * ROWB);
    };
    auto stage_chunk = [&](int buf, const int(&col)[EPC]) {  // all pieces at once (prologue)
        StagePlan pl;
        plan_chunk(col, pl);
#pragma unroll
        for (int i = 0; i < 2 * NLD; i++) stage_piece(buf, i, pl);
    };

    // Mask bytes of this lane's eight 4-key groups in a chunk (non-zero byte = attended key).  Called for
    // chunks with a PARTIAL or absent entry only.  FULL entries are read too (their bytes are all set);
    // absent entries re-read the chunk's first entry and are discarded when the mask is applied.
    // No branches, eight independent loads, and no use of the loaded values here.
    constexpr int NMW = PK ? (MODE == 0 ? 4 : 2) : 8;  // mask words per lane and chunk
    auto load_mask = [&](int t, const int(&col)[EPC], uint32_t(&mk)[NMW], const MaskSrc &ms) {
        const uint8_t *const mrow = ms.mrow, *const prow = ms.prow;
        const int F = ms.F, NE = ms.NE;
        if constexpr (PK) {
            // the row's bits of every entry of chunk t: one word (BK = 32), one halfword (BK = 16) per entry, or
            // the two words of the chunk's 64 keys (BK >= 64).  Entries that are not PARTIAL read slot 0.
            if constexpr (MODE == 2) {
                const int sh = p.lbk - 6;
                const int e = t >> sh, sub = t & ((1 << sh) - 1);
                const uint8_t *a = prow + (int64_t)(e >= F ? e - F : 0) * tile_bytes + 8 * sub;
                mk[0] = *(const uint32_t *)a;
                mk[1] = *(const uint32_t *)(a + 4);
            } else {
#pragma unroll
                for (int j = 0; j < EPC; j++) {
                    const int e = t * EPC + j;
                    const uint8_t *a = prow + (int64_t)((e >= F && e < NE) ? e - F : 0) * tile_bytes;
                    if constexpr (MODE == 1) mk[j] = *(const uint32_t *)a;
                    else mk[j] = *(const uint16_t *)a;
                }
            }
            return;
        }
        int64_t c[2][4];
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
                c[kb][g] = col[j] + within;
            }
        if (p.mask_vec4) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) mk[4 * kb + g] = *(const uint32_t *)(mrow + c[kb][g]);
        } else {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const uint8_t *m0 = mrow + c[kb][g] * p.ms[3];
                    mk[4 * kb + g] = (uint32_t)m0[0] | ((uint32_t)m0[p.ms[3]] << 8) |
                                     ((uint32_t)m0[2 * p.ms[3]] << 16) | ((uint32_t)m0[3 * p.ms[3]] << 24);
                }
        }
    };

    // The mask of 32-key block KB of a chunk, applied to its scores: entries the mask leaves out become -inf.
    // Bit j of `valid` / `part`: list entry j of the chunk exists / is PARTIAL.
    auto apply_mask_block = [&](f32x16 &sb, auto kb_c, unsigned valid, unsigned part, const uint32_t(&mk)[NMW]) {
        constexpr int kb = decltype(kb_c)::value;
        if constexpr (PK) {
            // bit k of w: key k of this 32-key block; FULL entries count as all ones, absent ones as zero
            auto word = [&](int j, uint32_t ones) -> uint32_t {
                return ((part >> j) & 1u) ? mk[j] : (((valid >> j) & 1u) ? ones : 0u);
            };
            uint32_t w;
            if constexpr (MODE == 0) w = word(2 * kb, 0xffffu) | (word(2 * kb + 1, 0xffffu) << 16);
            else if constexpr (MODE == 1) w = word(kb, ~0u);
            else w = (valid & 1u) ? mk[kb] : 0u;  // a chunk of a PARTIAL entry (or of an absent one)
            w >>= sh4;  // this lane's keys are 8g + 4hh + jj
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const uint32_t keep = (uint32_t)__builtin_amdgcn_sbfe((int)w, 8 * g + jj, 1);  // 0 or ~0
                    const uint32_t x = __float_as_uint(sb[4 * g + jj]);
                    sb[4 * g + jj] = __uint_as_float((x & keep) | (0xff800000u & ~keep));
                }
        } else {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int j = MODE == 0 ? 2 * kb + (g >> 1) : (MODE == 1 ? kb : 0);  // list entry of this group
                const uint32_t w = ((valid >> j) & 1u) ? mk[4 * kb + g] : 0u;
#pragma unroll
                for (int jj = 0; jj < 4; jj++)
                    if (((w >> (8 * jj)) & 0xffu) == 0u) sb[4 * g + jj] = kNegInf;
            }
        }
    };

    // One chunk from stage BUF, in two phases.
    // S phase: s = K . Q^T - m_ref.  When `fetch`, the pieces of the chunk planned in `pl` are sent to stage
    // FBUF between its MFMA bundles.
    auto phase_s = [&](auto buf_c, f32x16(&s)[2], auto fbuf_c, bool fetch, const StagePlan &pl) {
        constexpr int BUF = decltype(buf_c)::value;
        constexpr int FBUF = decltype(fbuf_c)::value;
        const uint8_t *kb_ = smem + BUF * KBUF;

        // S^T = K . Q^T in bundles of two MFMAs (the two key blocks of d step c), operand reads kPfS bundles
        // ahead.  Within a bundle the MFMA that uses the younger read goes first, so one wait covers both.
        constexpr int NC = D / 16;
        constexpr int kPfS = 3;
        u32x4 kf0[NC], kf1[NC];
        auto k_read = [&](int c) {
            kf0[c] = *(const u32x4 *)(kb_ + koff[c]);
            kf1[c] = *(const u32x4 *)(kb_ + 32 * ROWB + koff[c]);
        };
#pragma unroll
        for (int c = 0; c < kPfS; c++) k_read(c);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(kPrioS);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < NC; c++) {
            s[1] = E::mfma(kf1[c], qf[c], c == 0 ? neg_m : s[1]);
            s[0] = E::mfma(kf0[c], qf[c], c == 0 ? neg_m : s[0]);
            if (c + kPfS < NC) k_read(c + kPfS);
            if (fetch) {
#pragma unroll
                for (int i = 2 * NLD * c / NC; i < 2 * NLD * (c + 1) / NC; i++) stage_piece(FBUF, i, pl);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
    };
    // P.V phase: mask, online softmax, O^T += V^T . P^T.  between(b, NB) is called once per MFMA bundle b of NB;
    // the main loop uses it to spread scalar bookkeeping over the phase, where it hides behind the MFMAs.
    auto phase_pv = [&](auto buf_c, f32x16(&s)[2], bool special, unsigned valid, unsigned part,
                        const uint32_t(&mk)[NMW], auto &&between) {
        constexpr int BUF = decltype(buf_c)::value;
        const uint8_t *vb_ = smem + NS * KBUF + BUF * VBUF;
        if (special) {
            apply_mask_block(s[0], std::integral_constant<int, 0>{}, valid, part, mk);
            apply_mask_block(s[1], std::integral_constant<int, 1>{}, valid, part, mk);
        }

        // Online softmax in exp2 units (sparse_attn_kernel.py:47-58), with a lagging reference value: s holds
        // score*scale - m_ref.  Only when some row's largest argument exceeds raise_above does m_ref move.
        float mx = kNegInf;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[kb][i]);
        mx = half_swap_max(mx);
        const bool raise = mx > raise_above;  // false for rows without an attended key so far (mx = -inf)
        if (__builtin_amdgcn_ballot_w64(raise) != 0ull) {
            // rows that raise: m_ref += mx, the arguments drop by mx, what was accumulated shrinks by 2^-mx
            // (nothing was accumulated if this is the row's first attended key: factor 0, not 2^-mx, which
            // may be infinite)
            const float delta = raise ? mx : 0.f;
            const float a = raise ? (raise_above == kMaxSlack ? __builtin_amdgcn_exp2f(-mx) : 0.f) : 1.f;
            m_ref += delta;
            raise_above = raise ? kMaxSlack : raise_above;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int i = 0; i < 16; i++) s[kb][i] -= delta;
            // (= -m_ref either way; formed in place the sixteen registers need no copy on the path that does not raise,
            // but at D = 256, where every register is taken, that form spills)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                if constexpr (D <= 128) neg_m[i] -= delta;
                else neg_m[i] = -m_ref;
            }
#pragma unroll
            for (int i = 0; i < 2; i++) acc_l[i] *= a;  // the lane only ever reads the one of its own row
#pragma unroll
            for (int db = 0; db < D / 32; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[db][i] *= a;
        }

        // P = exp2(s), rounded to the input dtype, and O^T += V^T . P^T.
        // MFMA (key step kc, d block db) needs only the kc-th group of 8 P values, so the loop is a software
        // pipeline of bundles pinned by scheduling barriers: two MFMAs (d blocks 2h, 2h+1 of one key step) |
        // the transposing reads for a later bundle | half of the next key step's exponentials.
        // The row sum comes from one small MFMA per key step (see acc_l): it adds up the 16 keys of the step,
        // both lane halves included, and it adds up the ROUNDED values, the ones that enter P.V, so the output
        // is an exact convex combination of value rows (the reference sums the unrounded ones; the difference
        // is bounded by the rounding of P).
        constexpr int NDB = D / 32;
        constexpr int NB = 4 * NDB / 2;  // bundles; bundle b: key step b / (NDB/2), d blocks 2*(b % (NDB/2)) + {0,1}
        constexpr int BPK = NDB / 2;     // bundles per key step
        constexpr int kPfV = 2;
        constexpr int PER = 8 / BPK;     // P values of the next key step produced per bundle
        uint32_t pw[16];                 // P, two keys per dword, in MFMA operand order
        auto p_values = [&](int kc, int first, int count) {
#pragma unroll
            for (int i = first; i < first + count; i += 2) {
                const float x0 = __builtin_amdgcn_exp2f(s[kc >> 1][8 * (kc & 1) + i]);
                const float x1 = __builtin_amdgcn_exp2f(s[kc >> 1][8 * (kc & 1) + i + 1]);
                pw[4 * kc + (i >> 1)] = E::pack2(x0, x1);
            }
        };
        u32x2 vlo[2 * NB], vhi[2 * NB];
        auto v_read = [&](int b) {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int kc = b / BPK, db = 2 * (b % BPK) + u;
                const uint8_t *vp = vb_ + 16 * kc * ROWB + voff[db];
                vlo[2 * b + u] = E::tr_read(vp);
                vhi[2 * b + u] = E::tr_read(vp + 8 * ROWB);
            }
        };
#pragma unroll
        for (int b = 0; b < kPfV; b++) v_read(b);
        p_values(0, 0, 8);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(kPrioPV);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const int kc = b / BPK;
            const u32x4 pk4 = u32x4{pw[4 * kc], pw[4 * kc + 1], pw[4 * kc + 2], pw[4 * kc + 3]};
#pragma unroll
            for (int u = 1; u >= 0; u--) {
                const int db = 2 * (b % BPK) + u, i = 2 * b + u;
                acc[db] = E::mfma(u32x4{vlo[i].x, vlo[i].y, vhi[i].x, vhi[i].y}, pk4, acc[db]);
            }
            if (b % BPK == BPK - 1) acc_l = E::mfma16(sum_sel, pk4, acc_l);
            if (b + kPfV < NB) v_read(b + kPfV);
            if (kc + 1 < 4) p_values(kc + 1, PER * (b % BPK), PER);
            between(b, NB);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
    };

    // Makes the compiler account for a completed vector-memory load here (it emits its own wait, which
    // costs nothing once the data has landed) instead of in front of a later use, where the wait would
    // also cover direct loads it does not know about.
    auto settle = [](const uint32_t(&mk)[NMW]) {
#pragma unroll
        for (int i = 0; i < NMW; i++) asm volatile("" ::"v"(mk[i]));
    };

    // O = acc / l (sparse_attn_kernel.py:144); rows that attended to nothing give 0.
    auto store_o = [&]() {
        const float l_tot = l32 < 16 ? acc_l[0] : acc_l[1];
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        // sum over the attended keys of exp(scaled score) = l * 2^m_ref
        if (p.lse != nullptr && hh == 0)
            p.lse[lse_off] = l_tot > 0.f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * 0.69314718056f : kNegInf;
        uint16_t *orow = p.o + orow_off;
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const u32x2 w = {E::pack2(acc[db][4 * g] * inv, acc[db][4 * g + 1] * inv),
                                 E::pack2(acc[db][4 * g + 2] * inv, acc[db][4 * g + 3] * inv)};
                *(u32x2 *)(orow + 32 * db + 8 * g) = w;
            }
    };

    // The same through LDS, for paths that end with every K/V stage free (no wave reads them any more, no direct load
    // is on its way): a lane owns 8-byte pieces of its own row, which makes every store instruction touch 32 rows; a
    // wave-private copy of its 32 rows in LDS (rows 16 bytes apart from the banks' period) read back 16 bytes per
    // lane turns them into stores of whole rows, an eighth of the memory transactions.
    auto store_o_rows = [&]() {
        const float l_tot = l32 < 16 ? acc_l[0] : acc_l[1];
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (p.lse != nullptr && hh == 0)
            p.lse[lse_off] = l_tot > 0.f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * 0.69314718056f : kNegInf;
        constexpr int OROW = ROWB + 16;
        static_assert(NW * 32 * OROW <= 2 * NS * 64 * ROWB, "the rows of all waves fit the K/V stages");
        uint8_t *const ob = smem + wave * 32 * OROW;
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const u32x2 w = {E::pack2(acc[db][4 * g] * inv, acc[db][4 * g + 1] * inv),
                                 E::pack2(acc[db][4 * g + 2] * inv, acc[db][4 * g + 3] * inv)};
                *(u32x2 *)(ob + l32 * OROW + 2 * (32 * db + 8 * g + 4 * hh)) = w;
            }
        // 64 lanes x 16 bytes = 1024 / ROWB rows per store
        uint16_t *const o0 = p.o + b * p.os[0] + h * p.os[1] + (int64_t)(qt * (NW * 32) + wave * 32) * p.os[2];
#pragma unroll
        for (int i = 0; i < 32 * PPR / 64; i++) {
            const int idx = 64 * i + lane, r = idx / PPR, pc = idx % PPR;
            const u32x4 x = *(const u32x4 *)(ob + r * OROW + 16 * pc);
            // (written once, whole rows: a streaming store leaves the lines of K and V in L2 alone)
            __builtin_nontemporal_store(x, (u32x4 *)(o0 + (int64_t)r * p.os[2] + 8 * pc));
        }
    };

    if constexpr (PS) {
        // Persistent loop.  Per Q tile of this workgroup's row, the pipeline is
        //   two tiles ahead  its schedule entry is loaded;
        //   one tile ahead   its list indices are loaded into registers (issued when the tile before it starts)
        //                    and written to the free LDS list when that tile starts;
        //   last chunk of the tile before: its first chunk is fetched into the free K/V stage and, once the
        //                    last S phase is over, its queries are loaded over the old ones.
        // Everything issued during a tile has landed by the time it is used: every chunk ends in vmcnt(0).
        int *const el0 = reinterpret_cast<int *>(smem + NS * KBUF + NS * VBUF);
        auto elist = [&](int which) -> int * { return el0 + which * kPsListCap; };
        int lb = 0;  // LDS list of the tile at hand
        int it = 0;  // its position in the row
        bool has_nx = 1 < n_items, has_n2 = 2 < n_items;
        int nx_bh = 0, nx_qt = 0, nx_F = 0, nx_P = 0;  // the next tile
        int n2_bh = 0, n2_qt = 0, n2_F = 0, n2_P = 0;  // the one after
        int lr[PER];
        auto rfl = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
        ps_list_issue(b, h, qt, F, NE - F, lr);
        ps_list_deposit(F, NE - F, lr, elist(0));
        if (has_nx) {
            const int4 e1 = sched_row[2];
            nx_bh = rfl(e1.x), nx_qt = rfl(e1.y), nx_F = clamp_full(rfl(e1.z)), nx_P = clamp_part(rfl(e1.z), rfl(e1.w));
            ps_list_issue(nx_bh >> 16, nx_bh & 0xffff, nx_qt, nx_F, nx_P, lr);
            ps_list_deposit(nx_F, nx_P, lr, elist(1));
        }
        if (has_n2) {
            const int4 e2 = sched_row[3];
            n2_bh = rfl(e2.x), n2_qt = rfl(e2.y), n2_F = clamp_full(rfl(e2.z)), n2_P = clamp_part(rfl(e2.z), rfl(e2.w));
            ps_list_issue(n2_bh >> 16, n2_bh & 0xffff, n2_qt, n2_F, n2_P, lr);  // stays in registers for now
        }
        int4 e3 = 3 < n_items ? sched_row[4] : int4{0, 0, 0, 0};

        int col[EPC], coln[EPC];
        unsigned valid, part;
        uint32_t mk[2][NMW] = {};
        bool sp[2] = {false, false};
        unsigned vl[2] = {0u, 0u}, pt[2] = {0u, 0u};
        constexpr unsigned ALL = (1u << EPC) - 1u;
        StagePlan pl;
        int raw[EPC];
        __syncthreads();  // the lists in LDS are complete
        // first chunk of the first tile, and the look-ahead state of a tile that starts at the parity-0 stage:
        // `pl`, coln, sp/vl/pt[1] describe chunk 1, raw holds the entries of chunk 2 (clamped to the last chunk)
        ps_entries_read(elist(0), 0, raw);
        ps_entries_use(0, raw, col, valid, part);
        stage_chunk(0, col);
        sp[0] = part != 0u || valid != ALL;
        vl[0] = valid;
        pt[0] = part;
        if (sp[0]) load_mask(0, col, mk[0], MaskSrc{mrow, prow, F, NE});
        ps_entries_read(elist(0), 1 < T ? 1 : 0, raw);
        ps_entries_use(1 < T ? 1 : 0, raw, coln, valid, part);
        sp[1] = 1 < T && (part != 0u || valid != ALL);
        vl[1] = valid;
        pt[1] = part;
        plan_chunk(coln, pl);
        ps_entries_read(elist(0), 2 < T ? 2 : T - 1, raw);
#pragma unroll
        for (int c = 0; c < D / 16; c++) asm volatile("" ::"v"(qf[c]));
        settle(mk[0]);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();

        int tc = 0;
        bool done = false;
        while (!done) {
            static_for<2>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                constexpr int cur = j & 1, nxt = cur ^ 1;
                if (done) return;
                const bool last = tc == T - 1;
                const bool cross = last && has_nx;  // the chunk fetched now is the first one of the next tile
                const bool fetch = !last || has_nx;
                MaskSrc msn{mrow, prow, F, NE};
                const int nb_ = nx_bh >> 16, nh_ = nx_bh & 0xffff;
                if (cross) {
                    int rx[EPC];
                    ps_entries_read(elist(lb ^ 1), 0, rx);
                    ps_entries_use(0, rx, coln, valid, part);
                    const uint16_t *kn = p.k + nb_ * p.ks[0] + nh_ * p.ks[1];
                    const uint16_t *vn = p.v + nb_ * p.vs[0] + nh_ * p.vs[1];
#pragma unroll
                    for (int e = 0; e < EPC; e++) {
                        pl.kp[e] = kn + row_off(coln[e], ks2);
                        pl.vp[e] = vn + row_off(coln[e], vs2);
                    }
                    sp[nxt] = part != 0u || valid != ALL;
                    vl[nxt] = valid;
                    pt[nxt] = part;
                    if (sp[nxt]) msn = mask_src_of(nb_, nh_, nx_qt, nx_F, nx_F + nx_P);
                }
                if (sp[nxt]) load_mask(cross ? 0 : tc + 1, coln, mk[nxt], msn);
                f32x16 s[2];
                phase_s(jc, s, std::integral_constant<int, nxt>{}, fetch, pl);
                if (cross) load_q(nb_, nh_, nx_qt);  // the old queries have done their last S phase
                const int t2 = tc + 2 < T ? tc + 2 : T - 1, t3 = tc + 3 < T ? tc + 3 : T - 1;
                int col2[EPC];
                unsigned valid2 = 0u, part2 = 0u;
                StagePlan pl2;
                const int *const el = elist(lb);
                phase_pv(jc, s, sp[cur], vl[cur], pt[cur], mk[cur], [&](int bb, int nb) {
                    const int per = (2 * EPC + nb - 1) / nb;  // plan entries per bundle
                    if (bb == 0) ps_entries_use(t2, raw, col2, valid2, part2);
#pragma unroll
                    for (int i = bb * per; i < (bb + 1) * per && i < 2 * EPC; i++) {
                        if (i & 1) pl2.vp[i >> 1] = vbase + row_off(col2[i >> 1], vs2);
                        else pl2.kp[i >> 1] = kbase + row_off(col2[i >> 1], ks2);
                    }
                    if (bb == nb - 1) ps_entries_read(el, t3, raw);
                });
                pl = pl2;
#pragma unroll
                for (int e = 0; e < EPC; e++) coln[e] = col2[e];
                const bool sp2 = tc + 2 < T && (part2 != 0u || valid2 != ALL);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the fetched chunk and its mask words have landed
                settle(mk[nxt]);  // on every path: the compiler cannot tell that loads and uses share a condition
                // same for the queries (new ones are loaded when `cross`): accounted for here on every path, so that
                // the S phases of the loop carry no wait for them
#pragma unroll
                for (int c = 0; c < D / 16; c++) asm volatile("" ::"v"(qf[c]));
                sp[cur] = sp2;
                vl[cur] = valid2;
                pt[cur] = part2;
                if (!last) {
                    tc++;
                    __syncthreads();
                    return;
                }
                // ---- the tile is finished --------------------------------------------------------------
                store_o();
                if (!has_nx) {
                    done = true;
                    return;
                }
                set_item(nb_, nh_, nx_qt, nx_F, nx_P);
                lb ^= 1;
                it++;
                tc = 0;
                // the list that waited in registers goes to the LDS list the finished tile used
                if (has_n2) ps_list_deposit(n2_F, n2_P, lr, elist(lb ^ 1));
                has_nx = has_n2;
                nx_bh = n2_bh, nx_qt = n2_qt, nx_F = n2_F, nx_P = n2_P;
                has_n2 = it + 2 < n_items;
                if (has_n2) {
                    n2_bh = rfl(e3.x), n2_qt = rfl(e3.y), n2_F = clamp_full(rfl(e3.z)), n2_P = clamp_part(rfl(e3.z), rfl(e3.w));
                    ps_list_issue(n2_bh >> 16, n2_bh & 0xffff, n2_qt, n2_F, n2_P, lr);
                }
                if (it + 3 < n_items) e3 = sched_row[1 + it + 3];
                // fresh softmax state; the new queries were loaded during the last P.V phase
                m_ref = 0.f;
                raise_above = -3.0e38f;
#pragma unroll
                for (int i = 0; i < 16; i++) neg_m[i] = 0.f;
#pragma unroll
                for (int i = 0; i < 4; i++) acc_l[i] = 0.f;
#pragma unroll
                for (int db = 0; db < D / 32; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[db][i] = 0.f;
                scale_q();
                // look-ahead state of the new tile; its chunk 0 sits in stage nxt, so chunk 1 goes to stage cur
                const int *const eln = elist(lb);
                int rx[EPC];
                ps_entries_read(eln, 1 < T ? 1 : 0, rx);
                ps_entries_use(1 < T ? 1 : 0, rx, coln, valid, part);
                sp[cur] = 1 < T && (part != 0u || valid != ALL);
                vl[cur] = valid;
                pt[cur] = part;
                plan_chunk(coln, pl);
                ps_entries_read(eln, 2 < T ? 2 : T - 1, raw);
                __syncthreads();
            });
        }
        return;
    } else if constexpr (PP) {
        // Ping-pong schedule.  Every wave runs  barrier | S phase | barrier | P.V phase  per chunk; waves 4..7
        // enter the sequence one barrier later than waves 0..3, so between two barriers one wave of each SIMD
        // issues the MFMA-only S phase while the other does softmax and P.V, and the matrix unit always has a
        // taker.  Chunk t is needed first by waves 0..3 after barrier 2t and last by waves 4..7 before barrier
        // 2t+3; it is fetched two chunks ahead into a ring of 4 stages, whose slot was given up before barrier
        // 2t-1.  Before arriving at barrier 2t every wave has waited for its own pieces of chunk t.
        static_assert(!PP || (NW == 8 && NS == 4), "ping-pong layout");
        if (T > 0) {
            const int late = wave_u >> 2;  // 1: this wave runs half a chunk behind
            int col[EPC], coln[EPC];       // entries of the chunk at hand / of the next chunk to look at
            unsigned valid, part, validn = 0u, partn = 0u;
            uint32_t mk[2][NMW] = {};
            bool sp[2] = {false, false};
            unsigned vl[2] = {0u, 0u}, pt[2] = {0u, 0u};
            constexpr unsigned ALL = (1u << EPC) - 1u;
            constexpr int kOpsPerChunk = 2 * NLD;
            copy_list();
            __syncthreads();  // the list in LDS is complete
            chunk_entries(0, col, valid, part);
            stage_chunk(0, col);
            sp[0] = part != 0u || valid != ALL;
            vl[0] = valid;
            pt[0] = part;
            if (sp[0]) load_mask(0, col, mk[0], MaskSrc{mrow, prow, F, NE});
#pragma unroll
            for (int j = 0; j < EPC; j++) coln[j] = col[j];
            if (1 < T) {
                chunk_entries(1, coln, validn, partn);
                stage_chunk(1, coln);
            }
#pragma unroll
            for (int c = 0; c < D / 16; c++) asm volatile("" ::"v"(qf[c]));
            int raw[EPC] = {};  // list entries of the chunk after next, read ahead
            if (2 < T) entries_read(2, raw);
            settle(mk[0]);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (late) __syncthreads();
            for (int t = 0; t < T; t += NS) {
                static_for<NS>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    constexpr int cur = j & 1, nxt = cur ^ 1;
                    const int tc = t + j;
                    if (tc < T) {
                        // own pieces of chunk tc have landed; chunk tc+1 may be in flight
                        wait_vm_at_most((tc + 1 < T ? tc + 1 : T - 1) - tc, kOpsPerChunk);
                        if (sp[cur]) settle(mk[cur]);  // (the compiler's wait for them takes the chunk in flight along)
                        __syncthreads();
                        sp[nxt] = false;
                        if (tc + 1 < T) {  // coln: entries of chunk tc+1
                            sp[nxt] = partn != 0u || validn != ALL;
                            vl[nxt] = validn;
                            pt[nxt] = partn;
                            if (sp[nxt]) load_mask(tc + 1, coln, mk[nxt], MaskSrc{mrow, prow, F, NE});
                        }
                        const bool fetch = tc + 2 < T;
                        if (fetch) {
                            entries_use(tc + 2, raw, coln, validn, partn);
                            if (tc + 3 < T) entries_read(tc + 3, raw);
                        }
                        StagePlan pl;
                        plan_chunk(coln, pl);
                        f32x16 s[2];
                        phase_s(jc, s, std::integral_constant<int, (j + 2) % NS>{}, fetch, pl);
                        // own pieces of chunk tc+1 have landed; chunk tc+2 may be in flight
                        wait_vm_at_most((tc + 2 < T ? tc + 2 : T - 1) - (tc + 1), kOpsPerChunk);
                        __syncthreads();
                        phase_pv(jc, s, sp[cur], vl[cur], pt[cur], mk[cur], [](int, int) {});
                    }
                });
            }
            if (!late) __syncthreads();
        }
    } else if (T > 0) {
        static_assert(PP || NS == 2, "two stages: the chunk being computed and the one being fetched");
        int col[EPC], coln[EPC];  // entries of chunk 0 / of the chunk that the current iteration fetches
        unsigned valid, part;
        uint32_t mk[2][NMW] = {};  // mask words of the chunk being computed / of the next one, by chunk parity
        bool sp[2] = {false, false};
        unsigned vl[2] = {0u, 0u}, pt[2] = {0u, 0u};
        constexpr unsigned ALL = (1u << EPC) - 1u;
        StagePlan pl;  // where the chunk fetched by the current iteration comes from
        // The first chunk is requested from the list slots that came with the counts, before the list itself is
        // copied (its loads would otherwise have to land first: one memory round trip per Q tile).
        if constexpr (kEarlyFirstChunk) {
            // The queries were requested first of all; now the first K/V chunk, then the list.
            int raw0[EPC];
            static_for<EPC>([&](auto j_c) { raw0[decltype(j_c)::value] = early_entry(j_c); });
            entries_use(0, raw0, col, valid, part);
            stage_chunk(0, col);
            // (and its mask words, when it has a PARTIAL or absent entry: where every tile is PARTIAL they were the
            // last thing a Q tile waited for before its loop)
            sp[0] = part != 0u || valid != ALL;
            vl[0] = valid;
            pt[0] = part;
            if (sp[0]) load_mask(0, col, mk[0], MaskSrc{mrow, prow, F, NE});
            const bool mine = list_in_lds && tid < list_cnt;
            int first_slots = 0;
            if (mine) first_slots = tagged_entry(tid);
            if (mine) ent[list_pos(tid)] = first_slots;
            if (list_in_lds)
                for (int e = tid + NW * 64; e < list_cnt; e += NW * 64) ent[list_pos(e)] = tagged_entry(e);
        } else {
            copy_list();
        }
        __syncthreads();  // the list in LDS is complete
        if constexpr (kEarlyFirstChunk) {
            scale_q();
        } else {
            chunk_entries(0, col, valid, part);
            stage_chunk(0, col);
            sp[0] = part != 0u || valid != ALL;
            vl[0] = valid;
            pt[0] = part;
            if (sp[0]) load_mask(0, col, mk[0], MaskSrc{mrow, prow, F, NE});
        }
        chunk_entries(1 < T ? 1 : 0, coln, valid, part);
        sp[1] = 1 < T && (part != 0u || valid != ALL);
        vl[1] = valid;
        pt[1] = part;
        plan_chunk(coln, pl);
        int raw[EPC];  // list entries of the chunk after next, read ahead
        entries_read(2 < T ? 2 : T - 1, raw);
#pragma unroll
        for (int c = 0; c < D / 16; c++) asm volatile("" ::"v"(qf[c]));
        settle(mk[0]);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // Two chunks per trip so that the LDS stage is a compile-time constant.  Iteration tc computes chunk tc
        // while chunk tc+1 is fetched (its pieces go out between the S bundles) and, during the P.V phase, turns
        // the list entries of chunk tc+2 into the fetch plan of the next iteration.  Indices past the last chunk
        // are clamped to it: the values are computed and never used.
        for (int t = 0; t < T; t += 2) {
            static_for<2>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                constexpr int cur = j & 1, nxt = cur ^ 1;
                const int tc = t + j;
                if (tc < T) {
                    if (sp[nxt]) load_mask(tc + 1, coln, mk[nxt], MaskSrc{mrow, prow, F, NE});
                    f32x16 s[2];
                    // the fetch is unconditional: after the last chunk the plan is the clamped one and the last
                    // chunk is fetched once more, into the stage nobody reads any more (cheaper than a branch in
                    // front of every direct load)
                    phase_s(jc, s, std::integral_constant<int, nxt>{}, true, pl);
                    const int t2 = tc + 2 < T ? tc + 2 : T - 1, t3 = tc + 3 < T ? tc + 3 : T - 1;
                    int col2[EPC];
                    unsigned valid2 = 0u, part2 = 0u;
                    StagePlan pl2;
                    phase_pv(jc, s, sp[cur], vl[cur], pt[cur], mk[cur], [&](int b, int nb) {
                        const int per = (2 * EPC + nb - 1) / nb;  // plan entries per bundle
                        if (b == 0) entries_use(t2, raw, col2, valid2, part2);
#pragma unroll
                        for (int i = b * per; i < (b + 1) * per && i < 2 * EPC; i++) {
                            if (i & 1) pl2.vp[i >> 1] = vbase + row_off(col2[i >> 1], vs2);
                            else pl2.kp[i >> 1] = kbase + row_off(col2[i >> 1], ks2);
                        }
                        if (b == nb - 1) entries_read(t3, raw);
                    });
                    pl = pl2;
#pragma unroll
                    for (int e = 0; e < EPC; e++) coln[e] = col2[e];
                    // chunk tc+2 will be computed from the slot of chunk tc
                    const bool sp2 = tc + 2 < T && (part2 != 0u || valid2 != ALL);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // chunk tc+1 and its mask words have landed
                    settle(mk[nxt]);  // on every path: the compiler cannot tell that loads and uses share a condition
                    sp[cur] = sp2;
                    vl[cur] = valid2;
                    pt[cur] = part2;
                    __syncthreads();
                }
            });
        }
    }

    if constexpr (PP) __syncthreads();  // the late waves of the ping-pong schedule have read their last stage
    store_o_rows();
}

template <int DT, int D, int NW, int MODE, bool PK, bool PS>
hipError_t launch_one(const FwdParams &p, hipStream_t stream) {
    // Eight waves fill a CU's register file on their own, so that workgroup can have most of the LDS: 4 stages.
    constexpr int NS = NW == 8 ? 4 : 2;
    static_assert(kListCap == 2 * kPsListCap, "one long list or two short ones in the same LDS");
    constexpr int smem = 2 * NS * 64 * D * 2 + kListCap * 4;  // NS stages of 64 rows for K and for V + the list(s)
    auto kern = sparse_fwd_kernel<DT, D, NW, MODE, NS, NW == 8, PK, PS>;
    static unsigned long long attr_done = 0;  // devices on which this kernel may use `smem` bytes of LDS
    if (const hipError_t e0 = allow_dynamic_smem(kern, smem, attr_done); e0 != hipSuccess) return e0;
    const unsigned grid = PS ? (unsigned)p.sched_G : (unsigned)p.nQ * (unsigned)p.B * (unsigned)p.H;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), smem, stream, p);
    return hipGetLastError();
}

template <int DT, int D, int NW, bool PK, bool PS>
hipError_t launch_mode(const FwdParams &p, hipStream_t stream) {
    if (p.BK == 16) return launch_one<DT, D, NW, 0, PK, PS>(p, stream);
    if (p.BK == 32) return launch_one<DT, D, NW, 1, PK, PS>(p, stream);
    return launch_one<DT, D, NW, 2, PK, PS>(p, stream);
}

template <int DT, int D, bool PK, bool PS>
hipError_t launch_bq(const FwdParams &p, int BQ, hipStream_t stream) {
    switch (BQ) {
        case 32:
            if constexpr (D > 128) return hipErrorInvalidValue;  // a lone wave would spill its registers there
            else return launch_mode<DT, D, 1, PK, PS>(p, stream);
        case 64: return launch_mode<DT, D, 2, PK, PS>(p, stream);
        case 128: return launch_mode<DT, D, 4, PK, PS>(p, stream);
        case 256:
            // 8-wave workgroups are not persistent, and their four stages do not fit the LDS at D = 256
            if constexpr (PS || D > 128) return hipErrorInvalidValue;
            else return launch_mode<DT, D, 8, PK, false>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

// Every kernel for one element type, one source of the PARTIAL tiles' mask entries and one way of handing out
// Q tiles.  Each combination is instantiated in a translation unit of its own (sparse_fwd_inst.hip compiled
// with SA_FWD_DT / SA_FWD_PK / SA_FWD_PS).
template <int DT, bool PK, bool PS>
hipError_t launch_fwd_variant(const FwdParams &p, int D, int BQ, hipStream_t stream) {
    switch (D) {
        case 64: return launch_bq<DT, 64, PK, PS>(p, BQ, stream);
        case 128: return launch_bq<DT, 128, PK, PS>(p, BQ, stream);
        case 256:
            // one workgroup per CU (its two stages of K and V take 128 KiB of LDS) with the whole register file:
            // one wave per SIMD; no schedules
            if constexpr (PS) return hipErrorInvalidValue;
            else return launch_bq<DT, 256, PK, false>(p, BQ, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace sa
