// Block-sparse flash-attention forward for gfx950 (MI355X), the form for SHORT lists: three workgroups per compute
// unit instead of two, keys consumed 32 at a time instead of 64.
//
// Same function as sparse_fwd_kernel (sparse_fwd_kernel.h; the Triton kernels sparse_attention_kernel / _sparse_inner,
// sparseattention/sparse_attn_kernel.py:74-146 and :10-63), same work decomposition (one workgroup of four waves per
// Q tile of 128 rows, wave w owns rows [32w, 32w+32)), same MFMA operand layouts.  What differs:
//
//   * A Q tile whose list is short spends a large part of its life outside its loop (arguments, counts, first K/V
//     rows: dependent memory round trips), and with two workgroups per compute unit nothing covers that time.  This
//     kernel stays below 168 vector registers so that a third workgroup fits: scores of 32 keys (16 registers) instead
//     of 64, and the reference value of the softmax is written into the score registers by moves instead of being
//     held in 16 registers of its own.
//   * K, V and the mask words of a chunk go through a ring of THREE LDS stages and are requested two chunks ahead:
//     a chunk of 32 keys is computed in less time than an L2 round trip takes when the neighbours are starting up.
//     The mask words (one dword per query row and chunk, from the bit-packed PARTIAL tiles) and the raw list travel
//     by direct loads global -> LDS as K and V do, so the loop issues a constant five such loads per wave and chunk
//     and no load the compiler knows of: "s_waitcnt vmcnt(5)" at the top of an iteration is exact.
//   * The list stays in LDS as the raw tile indices (at most kC32ListCap entries, FULL then PARTIAL); which entries
//     exist, which are PARTIAL and which point outside the row of tiles is decided with scalar instructions when an
//     entry is turned into addresses.
//
// Requirements (checked by launch_fwd_c32): D = 128, BLOCK_Q = 128, bit-packed PARTIAL tiles, one workgroup per
// Q tile.  Lists longer than kC32ListCap entries are cut there: the caller selects this kernel only when it knows
// the longest list (the wrapper does, from the counts).
#include "fwd_common.h"

namespace sa {

namespace {

constexpr int kC32ListCap = 256;

// 4 bytes per lane from per-lane global addresses straight into LDS: lane i writes lds_addr + 4*i.
// (m0 and its wait state inside the statement, as in dma16.)
__device__ __forceinline__ void dma4(const void *lane_addr, uint32_t lds_addr) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %0, off"
        :
        : "v"(lane_addr), "s"(lds_addr)
        : "memory");
}
// the same from a wave-uniform base and a per-lane byte offset
__device__ __forceinline__ void dma4_off(const void *base, uint32_t lane_offset, uint32_t lds_addr) {
    const uint64_t b = (uint64_t)(uintptr_t)base;
    const uint64_t ub = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32)) << 32);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %0, %1"
        :
        : "v"(lane_offset), "s"(ub), "s"(lds_addr)
        : "memory");
}

constexpr int kC32PrioS = 1;
constexpr int kC32PrioPV = 2;

// MODE 0: BK = 16 (two list entries per chunk), MODE 1: BK = 32, MODE 2: BK >= 64 (BK/32 chunks per entry).
template <int DT, int MODE>
__global__ __launch_bounds__(256, 3) void sparse_fwd_c32_kernel(const FwdParams p) {
    using E = Elem<DT>;
    constexpr int D = 128, NW = 4, ROWB = D * 2, NS = 3;
    constexpr int KBUF = 32 * ROWB;  // one stage of K (or V): 32 rows
    constexpr int MBUF = NW * 256;   // one stage of mask words: 64 dwords per wave
    constexpr int OFF_V = NS * KBUF, OFF_M = 2 * NS * KBUF, OFF_L = OFF_M + NS * MBUF;
    constexpr int EPC = MODE == 0 ? 2 : 1;   // list entries per chunk
    constexpr int LBKC = MODE == 0 ? 4 : 5;  // log2(BK) when MODE < 2
    constexpr int NEARLY = 2 * EPC;          // list slots fetched with the counts: those of chunks 0 and 1

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    int *const ring = reinterpret_cast<int *>(smem + OFF_L);  // raw tile indices, FULL entries then PARTIAL ones

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);

    // Workgroup -> (b, h, Q tile): every XCD gets whole planes, pairs of planes with their Q tiles interleaved, last
    // Q tile first (the same order as sparse_fwd_kernel, for the same reasons).
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
    const int qrow = qt * 128 + wave * 32 + l32;  // the query row this lane owns

    // Q^T operand: lane (l32, hh) keeps d = 16c + 8hh .. +7 of its query row for every 16-wide step c.  Requested first
    // of all: the queries come from HBM.
    u32x4 qf[D / 16];
    {
        const uint16_t *qp = p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2] + 8 * hh;
#pragma unroll
        for (int c = 0; c < D / 16; c++) qf[c] = *(const u32x4 *)(qp + 16 * c);
    }

    // Counts and the first slots of both lists by scalar loads under one wait.
    const int32_t *const fid = p.full_ids + b * p.fis[0] + h * p.fis[1] + qt * p.fis[2];
    const int32_t *const pid = p.part_ids + b * p.pis[0] + h * p.pis[1] + qt * p.pis[2];
    int64_t fis3 = p.fis[3], pis3 = p.pis[3];
    asm volatile("" : "+s"(fis3), "+s"(pis3));
    int F, NE, T;
    int early_f[NEARLY], early_p[NEARLY];
    {
        const int32_t *addr[2 + 2 * NEARLY];
        int got[2 + 2 * NEARLY];
        addr[0] = p.full_lens + (b * p.fls[0] + h * p.fls[1] + qt * p.fls[2]);
        addr[1] = p.part_lens + (b * p.pls[0] + h * p.pls[1] + qt * p.pls[2]);
        static_for<NEARLY>([&](auto i_c) {
            constexpr int i = decltype(i_c)::value;
            const int slot = i < p.nK ? i : p.nK - 1;  // (a row of fewer tiles: stay inside it)
            addr[2 + i] = fid + (int64_t)slot * fis3;
            addr[2 + NEARLY + i] = pid + (int64_t)slot * pis3;
        });
        scalar_gather(addr, got);
        static_for<NEARLY>([&](auto i_c) {
            constexpr int i = decltype(i_c)::value;
            early_f[i] = got[2 + i];
            early_p[i] = got[2 + NEARLY + i];
        });
        // counts clamped to the row of tiles and to what the LDS copy of the list holds
        F = min(min(max(got[0], 0), p.nK), kC32ListCap);
        NE = F + min(min(max(got[1], 0), p.nK - F), kC32ListCap - F);
        T = MODE == 2 ? (NE << (p.lbk - 5)) : ((NE + EPC - 1) / EPC);
    }

    const uint16_t *const kbase = p.k + b * p.ks[0] + h * p.ks[1];
    const uint16_t *const vbase = p.v + b * p.vs[0] + h * p.vs[1];
    const int64_t tile_bytes = (int64_t)16 * p.BK;  // 128 rows of BK/8 bytes
    // packed tiles of this Q tile's PARTIAL slots (slot s at s * tile_bytes)
    const uint8_t *const pbase = p.packed + b * p.pks[0] + h * p.pks[1] + (int64_t)qt * p.nK * tile_bytes;
    const uint32_t ks2 = (uint32_t)p.ks[2], vs2 = (uint32_t)p.vs[2];
    auto row_off = [](int col, uint32_t stride) -> int64_t { return (int64_t)((uint64_t)(uint32_t)col * stride); };
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const SA_LDS uint8_t *)smem);

    // ---- per-lane constants ------------------------------------------------------------------------------------
    // K operand of step c: row l32, 16-byte piece 2c + hh, swizzled by the row: l32*ROWB + 16*((2c) ^ t) with
    // t = hh ^ swizzle, which is the offset of step 0 with bits 5..7 flipped by c.  One register and an XOR per read
    // instead of eight registers (the registers are what this kernel is short of).
    const int koff0 = l32 * ROWB + 16 * (hh ^ k_swizzle<D>(l32));
    // V^T operand (transposing read): within each 16-lane group, lane t supplies the address of 4 consecutive d of key
    // row (t >> 2) and receives the 4 key rows of d column t.  The 32-wide d block db flips bits 6..7 of the offset.
    int voff0;
    {
        const int tr_row = 4 * hh + ((lane & 15) >> 2);
        const int x = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
        const int sw = v_swizzle<D>(tr_row) >> 2;
        voff0 = tr_row * ROWB + 64 * sw + 16 * x + 8 * (lane & 1);
    }
    // Direct loads of a chunk: load i (0, 1) of this wave fills rows [16i + 4*wave, +4) of a stage, 16 bytes per lane;
    // the lane fetches the swizzled source piece of its row.  Rows 16i + r and r share their swizzle, so one per-lane
    // offset serves both loads (the 16 rows in between go into the scalar base).
    const int ld_r = 4 * wave_u + (lane >> 4), ld_slot = lane & 15;
    const uint32_t ld_koff = (uint32_t)((ld_r * p.ks[2] + 8 * (ld_slot ^ k_swizzle<D>(ld_r))) * 2);
    const uint32_t ld_voff = (uint32_t)((ld_r * p.vs[2] + 8 * (ld_slot ^ v_swizzle<D>(ld_r))) * 2);
    // Mask words: per chunk the wave fetches one dword per lane into its 256 bytes of the M stage.
    //   BK = 32   the row's 32 bits of the chunk's tile (both lane halves fetch the same word)
    //   BK >= 64  the same, 4 bytes further on per chunk within the tile
    //   BK = 16   lane half hh fetches from entry hh of the chunk the dword that holds the 16 bits of rows 2r, 2r+1
    const uint32_t ld_moff = MODE == 0 ? (uint32_t)((wave * 32 + (l32 & ~1)) * 2) : (uint32_t)((wave * 32 + l32) * (p.BK >> 3));
    const int mread = OFF_M + wave * 256 + 4 * l32;  // where this lane reads its word(s) back (+128: the second half's)

    // ---- list entries -> what a chunk needs ---------------------------------------------------------------------
    // bits of Plan::flags: bit j = entry j of the chunk exists, bit 4 + j = it is PARTIAL
    struct Plan {
        const uint16_t *kp[EPC], *vp[EPC];
        const uint8_t *mp[EPC];
        unsigned flags;
    };
    // entry e of the list (raw index idx, both uniform) as entry j of a chunk's plan; sub: the chunk's place inside a
    // tile wider than 32 keys
    auto plan_entry = [&](Plan &pl, int j, int e, int idx, int sub) {
        const bool exists = e < NE && (unsigned)idx < (unsigned)p.nK;
        const bool partial = exists && e >= F;
        const int col = exists ? ((MODE == 2 ? (idx << p.lbk) : (idx << LBKC)) + 32 * sub) : 0;
        pl.kp[j] = kbase + row_off(col, ks2);
        pl.vp[j] = vbase + row_off(col, vs2);
        pl.mp[j] = pbase + (int64_t)((uint64_t)(uint32_t)(partial ? e - F : 0) * (uint32_t)tile_bytes) + 4 * sub;
        pl.flags |= (exists ? 1u : 0u) << j | (partial ? 16u : 0u) << j;
    };
    // chunk t of the list from the LDS copy (t clamped by the caller); two steps, the LDS read and its use
    auto ring_read = [&](int t, int(&raw)[EPC]) {
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            const int e = MODE == 2 ? (t >> (p.lbk - 5)) : t * EPC + j;
            raw[j] = ring[min(e, kC32ListCap - 1)];
        }
    };
    auto ring_use = [&](int t, const int(&raw)[EPC], Plan &pl) {
        pl.flags = 0u;
#pragma unroll
        for (int j = 0; j < EPC; j++) {
            const int e = MODE == 2 ? (t >> (p.lbk - 5)) : t * EPC + j;
            const int sub = MODE == 2 ? (t & ((1 << (p.lbk - 5)) - 1)) : 0;
            plan_entry(pl, j, e, __builtin_amdgcn_readfirstlane(raw[j]), sub);
        }
    };
    // the same for chunks 0 and 1 from the slots that came with the counts
    auto early_plan = [&](auto t_c, Plan &pl) {
        constexpr int t = decltype(t_c)::value;
        pl.flags = 0u;
        static_for<EPC>([&](auto j_c) {
            constexpr int j = decltype(j_c)::value;
            constexpr int e = MODE == 2 ? 0 : t * EPC + j;  // (BK >= 64: chunks 0 and 1 lie in entry 0)
            int idx = early_f[e];
            if (e >= F) {
                idx = early_p[0];
                static_for<e>([&](auto i_c) {  // e - F is one of 0 .. e
                    constexpr int i = decltype(i_c)::value + 1;
                    int cand = __builtin_amdgcn_readfirstlane(early_p[i]);
                    asm volatile("" : "+s"(cand));  // (keeps the chain of selects from becoming an indexed load)
                    if (e - F == i) idx = cand;
                });
            }
            plan_entry(pl, j, e, idx, MODE == 2 ? t : 0);
        });
    };

    // The five direct loads of a chunk, one at a time (the loop spreads them over its S phase).
    auto stage_piece = [&](auto buf_c, int piece, const Plan &pl) {
        constexpr int BUF = decltype(buf_c)::value;
        const int i = piece & 1;  // rows 16i .. 16i + 15 of the stage
        const uint16_t *ks_ = pl.kp[0], *vs_ = pl.vp[0];
        if constexpr (MODE == 0) {
            if (i == 1) {
                ks_ = pl.kp[1];
                vs_ = pl.vp[1];
            }
        } else {
            ks_ += (int64_t)(16 * i) * ks2;
            vs_ += (int64_t)(16 * i) * vs2;
        }
        const uint32_t dst = (uint32_t)((16 * i + 4 * wave_u) * ROWB);
        if (piece < 2) dma16(ks_, ld_koff, lds0 + BUF * KBUF + dst);
        else if (piece < 4) dma16(vs_, ld_voff, lds0 + OFF_V + BUF * KBUF + dst);
        else {
            const uint32_t mdst = lds0 + OFF_M + BUF * MBUF + wave_u * 256;
            if constexpr (MODE == 0) dma4((hh ? pl.mp[1] : pl.mp[0]) + ld_moff, mdst);
            else dma4_off(pl.mp[0], ld_moff, mdst);
        }
    };
    auto stage_chunk = [&](auto buf_c, const Plan &pl) {
#pragma unroll
        for (int i = 0; i < 5; i++) stage_piece(buf_c, i, pl);
    };

    // ---- start-up: list -> LDS, chunks 0 and 1 requested ------------------------------------------------------------
    unsigned fl0, fl1, fl2 = 0u;  // flags of the chunk at hand, of the next one and of the one after
    Plan pl;                      // plan of the chunk that the current iteration requests
    if (T > 0) {
        {
            Plan p0, p1;
            early_plan(std::integral_constant<int, 0>{}, p0);
            stage_chunk(std::integral_constant<int, 0>{}, p0);
            fl0 = p0.flags;
            early_plan(std::integral_constant<int, 1>{}, p1);  // (past the last chunk: entries that do not exist)
            stage_chunk(std::integral_constant<int, 1>{}, p1);
            fl1 = p1.flags;
        }
        // the list: wave w brings entries [64w, 64w + 64), each lane the slot of its entry in the list it belongs to
        if (64 * wave_u < NE) {
            const int e = min(64 * wave + lane, NE - 1);
            const int32_t *src = e < F ? fid + (int64_t)e * fis3 : pid + (int64_t)(e - F) * pis3;
            dma4(src, lds0 + OFF_L + 256 * wave_u);
        }
    }

    // Online-softmax state of this lane's query row, exp2 domain (the scale / ln 2 is folded into Q).  Exponentials are
    // taken against a reference value m_ref that is raised only when the row maximum exceeds it by more than kMaxSlack;
    // the score registers start every chunk at -m_ref, so a score leaves the matrix unit as the exp2 argument.
    float m_ref = 0.f;
    float raise_above = -3.0e38f;
    f32x4 acc_l = {0.f, 0.f, 0.f, 0.f};  // row sums of P by a 16x16x32 MFMA (see sparse_fwd_kernel)
    const uint32_t sel1 = (((lane >> 4) ^ lane) & 1) == 0 ? E::ones4().x : 0u;
    const u32x4 sum_sel = {sel1, sel1, sel1, sel1};
    f32x16 acc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.f;
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; i++) s[i] = 0.f;

    if (T > 0) {
        // queries scaled once (the compiler's wait for them is a wait for everything requested so far: the first two
        // chunks and the list, which the loop needs anyway)
#pragma unroll
        for (int c = 0; c < D / 16; c++)
#pragma unroll
            for (int e = 0; e < 4; e++) qf[c][e] = E::scale2(qf[c][e], p.scale);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // list, chunk 0 and chunk 1 are in LDS
        int raw[EPC];
        ring_read(2 < T ? 2 : T - 1, raw);
        ring_use(2 < T ? 2 : T - 1, raw, pl);
        fl2 = pl.flags;
        ring_read(3 < T ? 3 : T - 1, raw);

        // One chunk from stage BUF; requests the chunk planned in `pl` into stage FBUF on the way.
        auto chunk = [&](auto buf_c, auto fbuf_c, int tc) {
            constexpr int BUF = decltype(buf_c)::value;
            const uint8_t *kb_ = smem + BUF * KBUF;
            const uint8_t *vb_ = smem + OFF_V + BUF * KBUF;
            // ---- S phase: s = K . Q^T - m_ref, operand reads two steps ahead ----
            constexpr int NC = D / 16, kPfS = 2;
            u32x4 kf[NC];
            // (opaque per chunk, so that the eight offsets are formed here and not kept in registers across the loop)
            int kbase_off = koff0, vbase_off = voff0;
            asm volatile("" : "+v"(kbase_off), "+v"(vbase_off));
#pragma unroll
            for (int c = 0; c < kPfS; c++) kf[c] = *(const u32x4 *)(kb_ + (kbase_off ^ (c << 5)));
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(kC32PrioS);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int c = 0; c < NC; c++) {
                s = E::mfma(kf[c], qf[c], s);
                if (c + kPfS < NC) kf[c + kPfS] = *(const u32x4 *)(kb_ + (kbase_off ^ ((c + kPfS) << 5)));
                if (c < 5) stage_piece(fbuf_c, c, pl);
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);

            // ---- mask (chunks with a PARTIAL or missing entry only) ----
            constexpr unsigned ALL = (1u << EPC) - 1u;
            if (fl0 != ALL) {
                uint32_t w;
                if constexpr (MODE == 0) {
                    const uint32_t a = *(const uint32_t *)(smem + BUF * MBUF + mread);
                    const uint32_t c2 = *(const uint32_t *)(smem + BUF * MBUF + mread + 128);
                    const int sh = 16 * (l32 & 1);
                    const uint32_t w0 = (fl0 & 16u) ? ((a >> sh) & 0xffffu) : ((fl0 & 1u) ? 0xffffu : 0u);
                    const uint32_t w1 = (fl0 & 32u) ? ((c2 >> sh) & 0xffffu) : ((fl0 & 2u) ? 0xffffu : 0u);
                    w = w0 | (w1 << 16);
                } else {
                    const uint32_t a = *(const uint32_t *)(smem + BUF * MBUF + mread);
                    w = (fl0 & 16u) ? a : ((fl0 & 1u) ? ~0u : 0u);
                }
                w >>= 4 * hh;  // this lane's keys are 8g + 4hh + jj
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) {
                        const uint32_t keep = (uint32_t)__builtin_amdgcn_sbfe((int)w, 8 * g + jj, 1);  // 0 or ~0
                        const uint32_t x = __float_as_uint(s[4 * g + jj]);
                        s[4 * g + jj] = __uint_as_float((x & keep) | (0xff800000u & ~keep));
                    }
            }

            // ---- online softmax (sparse_attn_kernel.py:47-58) with the lagging reference value ----
            float mx = kNegInf;
#pragma unroll
            for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[i]);
            mx = half_swap_max(mx);
            const bool raise = mx > raise_above;
            if (__builtin_amdgcn_ballot_w64(raise) != 0ull) {
                const float delta = raise ? mx : 0.f;
                const float a = raise ? (raise_above == kMaxSlack ? __builtin_amdgcn_exp2f(-mx) : 0.f) : 1.f;
                m_ref += delta;
                raise_above = raise ? kMaxSlack : raise_above;
#pragma unroll
                for (int i = 0; i < 16; i++) s[i] -= delta;
#pragma unroll
                for (int i = 0; i < 2; i++) acc_l[i] *= a;
#pragma unroll
                for (int db = 0; db < D / 32; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[db][i] *= a;
            }

            // ---- P = exp2(s) rounded to the input type, O^T += V^T . P^T, row sums; bundles of two MFMAs ----
            constexpr int NB = 4;  // bundle b: key step b >> 1, d blocks 2 * (b & 1) + {0, 1}
            uint32_t pw[8];
            auto p_values = [&](int kc, int first, int count) {
#pragma unroll
                for (int i = first; i < first + count; i += 2) {
                    const float x0 = __builtin_amdgcn_exp2f(s[8 * kc + i]);
                    const float x1 = __builtin_amdgcn_exp2f(s[8 * kc + i + 1]);
                    pw[4 * kc + (i >> 1)] = E::pack2(x0, x1);
                }
            };
            u32x2 vlo[2 * NB], vhi[2 * NB];
            auto v_read = [&](int bb) {
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int kc = bb >> 1, db = 2 * (bb & 1) + u;
                    const uint8_t *vp = vb_ + 16 * kc * ROWB + (vbase_off ^ (db << 6));
                    vlo[2 * bb + u] = E::tr_read(vp);
                    vhi[2 * bb + u] = E::tr_read(vp + 8 * ROWB);
                }
            };
            v_read(0);
            p_values(0, 0, 8);
            const float nm = -m_ref;
            // the plan of the chunk after next (requested by the next iteration), spread over the bundles
            const int t3 = tc + 3 < T ? tc + 3 : T - 1, t4 = tc + 4 < T ? tc + 4 : T - 1;
            Plan pl2;
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(kC32PrioPV);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int bb = 0; bb < NB; bb++) {
                const int kc = bb >> 1;
                const u32x4 pk4 = u32x4{pw[4 * kc], pw[4 * kc + 1], pw[4 * kc + 2], pw[4 * kc + 3]};
#pragma unroll
                for (int u = 1; u >= 0; u--) {
                    const int db = 2 * (bb & 1) + u, i = 2 * bb + u;
                    acc[db] = E::mfma(u32x4{vlo[i].x, vlo[i].y, vhi[i].x, vhi[i].y}, pk4, acc[db]);
                }
                if (bb & 1) acc_l = E::mfma16(sum_sel, pk4, acc_l);
                if (bb + 1 < NB) v_read(bb + 1);
                if (bb < 2) p_values(1, 4 * bb, 4);
                // the score registers whose exponentials are taken go back to -m_ref for the next chunk
                if (bb >= 1) {
#pragma unroll
                    for (int i = 0; i < 16; i++)
                        if (i / 6 == bb - 1 || (bb == 3 && i >= 12)) s[i] = nm;
                }
                if (bb == 0) ring_use(t3, raw, pl2);
                if (bb == NB - 1) ring_read(t4, raw);
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            pl = pl2;
            fl0 = fl1;
            fl1 = fl2;
            fl2 = pl2.flags;
        };

        // Iteration tc computes chunk tc from stage tc % 3 and requests chunk tc + 2 into the stage that chunk tc - 1
        // has left.  At its top at most the five loads of chunk tc + 1 may still be on their way; the barrier also
        // tells that every wave is done with chunk tc - 1.  Past the last chunk the plan is the last chunk's once
        // more (cheaper than a branch in front of every load).
        for (int t = 0; t < T; t += 3) {
            static_for<3>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int tc = t + j;
                if (tc < T) {
                    asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
                    __syncthreads();
                    chunk(jc, std::integral_constant<int, (j + 2) % 3>{}, tc);
                }
            });
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the requests past the last chunk
        __syncthreads();                                   // every wave is done with the stages
    }

    // ---- O = acc / l (sparse_attn_kernel.py:144), rows that attended to nothing give 0; whole rows leave through a
    // wave-private slice of the stages, 16 bytes per lane ----
    {
        // (the lane's coordinates formed again from its id: kept across the loop they would cost registers there)
        int tid2 = threadIdx.x;
        asm volatile("" : "+v"(tid2));
        const int lane2 = tid2 & 63, wave2 = tid2 >> 6, l32b = tid2 & 31, hhb = (tid2 >> 5) & 1;
        const float l_tot = l32b < 16 ? acc_l[0] : acc_l[1];
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (p.lse != nullptr && hhb == 0)
            p.lse[b * p.lses[0] + h * p.lses[1] + (int64_t)(qt * 128 + wave2 * 32 + l32b) * p.lses[2]] =
                l_tot > 0.f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * 0.69314718056f : kNegInf;
        constexpr int OROW = ROWB + 16;
        static_assert(NW * 32 * OROW <= 2 * NS * KBUF, "the rows of all waves fit the K/V stages");
        uint8_t *const ob = smem + wave2 * 32 * OROW;
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const u32x2 w = {E::pack2(acc[db][4 * g] * inv, acc[db][4 * g + 1] * inv),
                                 E::pack2(acc[db][4 * g + 2] * inv, acc[db][4 * g + 3] * inv)};
                *(u32x2 *)(ob + l32b * OROW + 2 * (32 * db + 8 * g + 4 * hhb)) = w;
            }
        uint16_t *const o0 = p.o + b * p.os[0] + h * p.os[1] + (int64_t)(qt * 128 + wave2 * 32) * p.os[2];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int idx = 64 * i + lane2, r = idx >> 4, pc = idx & 15;
            const u32x4 x = *(const u32x4 *)(ob + r * OROW + 16 * pc);
            __builtin_nontemporal_store(x, (u32x4 *)(o0 + (int64_t)r * p.os[2] + 8 * pc));  // (streaming, as in sparse_fwd_kernel)
        }
    }
}

template <int DT, int MODE>
hipError_t launch_c32(const FwdParams &p, hipStream_t stream) {
    constexpr int smem = 2 * 3 * 32 * 256 + 3 * 1024 + kC32ListCap * 4;  // 52 KiB: three workgroups per compute unit
    auto kern = sparse_fwd_c32_kernel<DT, MODE>;
    static unsigned long long attr_done = 0;
    if (const hipError_t e0 = allow_dynamic_smem(kern, smem, attr_done); e0 != hipSuccess) return e0;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.nQ * (unsigned)p.B * (unsigned)p.H), dim3(256), smem, stream, p);
    return hipGetLastError();
}

template <int DT>
hipError_t launch_c32_mode(const FwdParams &p, hipStream_t stream) {
    if (p.BK == 16) return launch_c32<DT, 0>(p, stream);
    if (p.BK == 32) return launch_c32<DT, 1>(p, stream);
    return launch_c32<DT, 2>(p, stream);
}

}  // namespace

bool fwd_c32_has(const FwdParams &p, int dtype, int D, int BQ) {
    return (dtype == 0 || dtype == 1) && D == 128 && BQ == 128 && p.packed != nullptr && p.sched == nullptr &&
           p.BK >= 16 && (p.BK & (p.BK - 1)) == 0;
}

hipError_t launch_fwd_c32(const FwdParams &p, int dtype, int D, int BQ, hipStream_t stream) {
    if (!fwd_c32_has(p, dtype, D, BQ)) return hipErrorInvalidValue;
    return dtype == 0 ? launch_c32_mode<0>(p, stream) : launch_c32_mode<1>(p, stream);
}

}  // namespace sa
