// C ABI of libsparseattn_hip.so: argument validation, broadcast-plane folding and kernel dispatch.
// The declarations and their contracts live in include/sparseattn.h.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "kernels.h"
#include "sparseattn.h"

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int log2_exact(int x) {  // -1 unless x is a power of two
    if (x <= 0 || (x & (x - 1))) return -1;
    int l = 0;
    while ((1 << l) < x) l++;
    return l;
}

bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Shape checks shared by both entry points.  Returns SA_OK or an error code (message set).
int check_tiling(int B, int H, int Sq, int Sk, int BQ, int BK) {
    if (B <= 0 || H <= 0 || Sq <= 0 || Sk <= 0) return fail(SA_ERR_INVALID_ARGUMENT, "B, H, Sq, Sk must be positive (got %d, %d, %d, %d)", B, H, Sq, Sk);
    if (BQ <= 0 || BK <= 0) return fail(SA_ERR_INVALID_ARGUMENT, "BLOCK_Q and BLOCK_K must be positive (got %d, %d)", BQ, BK);
    if (Sq % BQ) return fail(SA_ERR_INVALID_ARGUMENT, "Sq (%d) must be a multiple of BLOCK_Q (%d)", Sq, BQ);
    if (Sk % BK) return fail(SA_ERR_INVALID_ARGUMENT, "Sk (%d) must be a multiple of BLOCK_K (%d)", Sk, BK);
    return SA_OK;
}

// The two launches of the classification (class bytes, then compaction into the lists), after the argument checks
// the entry points share.  `workspace` holds one class byte per tile of every distinct plane; the caller has checked
// its size.  `who` names the entry point in error messages.
int classify_impl(const char *who, const uint8_t *mask, const int64_t mask_strides[4], int B, int H, int Sq, int Sk,
                  int BQ, int BK, int32_t *full_ids, const int64_t full_ids_strides[4], int32_t *full_lens,
                  const int64_t full_lens_strides[3], int32_t *part_ids, const int64_t part_ids_strides[4],
                  int32_t *part_lens, const int64_t part_lens_strides[3], void *workspace, void *stream) {
    const int nQ = Sq / BQ, nK = Sk / BK;
    const bool bcast_b = mask_strides[0] == 0 || B == 1;
    const bool bcast_h = mask_strides[1] == 0 || H == 1;
    // An output dimension may be folded (stride 0) only where every plane holds the same result.
    const int64_t ob[4] = {full_ids_strides[0], full_lens_strides[0], part_ids_strides[0], part_lens_strides[0]};
    const int64_t oh[4] = {full_ids_strides[1], full_lens_strides[1], part_ids_strides[1], part_lens_strides[1]};
    int zb = 0, zh = 0;
    for (int i = 0; i < 4; i++) {
        zb += ob[i] == 0;
        zh += oh[i] == 0;
    }
    if (B > 1 && zb != 0 && (zb != 4 || !bcast_b))
        return fail(SA_ERR_INVALID_ARGUMENT, "%s: output batch stride 0 needs a batch-broadcast mask and must be 0 on all four outputs", who);
    if (H > 1 && zh != 0 && (zh != 4 || !bcast_h))
        return fail(SA_ERR_INVALID_ARGUMENT, "%s: output head stride 0 needs a head-broadcast mask and must be 0 on all four outputs", who);

    sa::ClassifyParams cp{};
    cp.mask = mask;
    cp.sb = mask_strides[0];
    cp.sh = mask_strides[1];
    cp.sq = mask_strides[2];
    cp.sk = mask_strides[3];
    cp.cls = static_cast<uint8_t *>(workspace);
    cp.uB = bcast_b ? 1 : B;
    cp.uH = bcast_h ? 1 : H;
    cp.Sq = Sq;
    cp.Sk = Sk;
    cp.BQ = BQ;
    cp.BK = BK;
    cp.nQ = nQ;
    cp.nK = nK;
    cp.lbk = log2_exact(BK);
    if (nQ > 65535 || (int64_t)cp.uB * cp.uH > 65535)
        return fail(SA_ERR_UNSUPPORTED, "%s: more than 65535 Q tiles or distinct mask planes", who);

    // Wide kernel: 16-byte loads along a contiguous, aligned key dimension; a tile spans 1..64 lanes.
    const bool wide = cp.lbk >= 4 && BK <= 1024 && (cp.sk == 1 || Sk == 1) && aligned(mask, 16) && cp.sq % 16 == 0 &&
                      (cp.uB == 1 || cp.sb % 16 == 0) && (cp.uH == 1 || cp.sh % 16 == 0);
    hipError_t e = sa::launch_classify(cp, wide, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "%s: classify launch failed: %s", who, hipGetErrorString(e));

    sa::CompactParams kp{};
    kp.cls = cp.cls;
    kp.uH = cp.uH;
    kp.bcast_b = bcast_b;
    kp.bcast_h = bcast_h;
    kp.oB = (B > 1 && zb == 4) ? 1 : B;
    kp.oH = (H > 1 && zh == 4) ? 1 : H;
    kp.nQ = nQ;
    kp.nK = nK;
    kp.full_ids = full_ids;
    kp.full_lens = full_lens;
    kp.part_ids = part_ids;
    kp.part_lens = part_lens;
    for (int i = 0; i < 4; i++) {
        kp.fis[i] = full_ids_strides[i];
        kp.pis[i] = part_ids_strides[i];
    }
    for (int i = 0; i < 3; i++) {
        kp.fls[i] = full_lens_strides[i];
        kp.pls[i] = part_lens_strides[i];
    }
    e = sa::launch_compact(kp, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "%s: compaction launch failed: %s", who, hipGetErrorString(e));
    return SA_OK;
}

// Class bytes of sa_mask_classify_static: device memory that belongs to the library, one copy per GPU the library
// runs on, held until the process ends.  Host code never uses this name as an address (on the host it is only a
// stand-in for the symbol): static_scratch() asks the runtime for the array's address on the current device.
constexpr size_t kStaticScratchBytes = SA_STATIC_CLASSIFY_MAX_TILES;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};  // address of `scratch` on device i, once it has been asked for

// Address of `scratch` on the current device (each GPU holds its own copy at its own address), or an error code
// with the message set when the runtime does not give it.  The first call on a device asks the runtime, later calls
// read the pointer kept then.  Two threads racing through the first call store the same value twice.
int static_scratch(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_mask_classify_static: hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices)
        return fail(SA_ERR_UNSUPPORTED, "sa_mask_classify_static: device ordinal %d (supported: below %d)", dev, kMaxDevices);
    void *ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(SA_ERR_HIP, "sa_mask_classify_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
    }
    *out = ptr;
    return SA_OK;
}

}  // namespace

extern "C" {

int sa_abi_version(void) { return SA_ABI_VERSION; }

const char *sa_last_error(void) { return g_error; }

size_t sa_mask_classify_workspace_bytes(const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ, int BK) {
    if (!mask_strides || check_tiling(B, H, Sq, Sk, BQ, BK) != SA_OK) return 0;
    const size_t uB = (mask_strides[0] == 0) ? 1 : (size_t)B;
    const size_t uH = (mask_strides[1] == 0) ? 1 : (size_t)H;
    return uB * uH * (size_t)(Sq / BQ) * (size_t)(Sk / BK);
}

int sa_mask_classify(const uint8_t *mask, const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ, int BK,
                     int32_t *full_ids, const int64_t full_ids_strides[4], int32_t *full_lens,
                     const int64_t full_lens_strides[3], int32_t *part_ids, const int64_t part_ids_strides[4],
                     int32_t *part_lens, const int64_t part_lens_strides[3], void *workspace, size_t workspace_bytes,
                     void *stream) {
    g_error[0] = 0;
    if (!mask || !mask_strides || !full_ids || !full_ids_strides || !full_lens || !full_lens_strides || !part_ids ||
        !part_ids_strides || !part_lens || !part_lens_strides)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify: null pointer argument");
    if (const int rc = check_tiling(B, H, Sq, Sk, BQ, BK)) return rc;
    const size_t need = sa_mask_classify_workspace_bytes(mask_strides, B, H, Sq, Sk, BQ, BK);
    if (!workspace || workspace_bytes < need)
        return fail(SA_ERR_WORKSPACE, "sa_mask_classify: workspace of %zu bytes required, %zu given", need,
                    workspace ? workspace_bytes : (size_t)0);
    return classify_impl("sa_mask_classify", mask, mask_strides, B, H, Sq, Sk, BQ, BK, full_ids, full_ids_strides,
                         full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens, part_lens_strides,
                         workspace, stream);
}

int sa_mask_classify_static(const uint8_t *mask, const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ,
                            int BK, int32_t *full_ids, const int64_t full_ids_strides[4], int32_t *full_lens,
                            const int64_t full_lens_strides[3], int32_t *part_ids,
                            const int64_t part_ids_strides[4], int32_t *part_lens,
                            const int64_t part_lens_strides[3], void *stream) {
    g_error[0] = 0;
    if (!mask || !mask_strides || !full_ids || !full_ids_strides || !full_lens || !full_lens_strides || !part_ids ||
        !part_ids_strides || !part_lens || !part_lens_strides)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_static: null pointer argument");
    if (const int rc = check_tiling(B, H, Sq, Sk, BQ, BK)) return rc;
    const size_t need = sa_mask_classify_workspace_bytes(mask_strides, B, H, Sq, Sk, BQ, BK);
    if (need > kStaticScratchBytes)
        return fail(SA_ERR_WORKSPACE,
                    "sa_mask_classify_static: %zu tiles over the distinct mask planes, the library's own scratch holds "
                    "%zu (SA_STATIC_CLASSIFY_MAX_TILES); use sa_mask_classify with a workspace of the caller's",
                    need, kStaticScratchBytes);
    // Every class byte the compaction reads is written by the classification launch in front of it, so nothing of
    // the previous call's contents has to be cleared.
    void *ws = nullptr;
    if (const int rc = static_scratch(&ws)) return rc;
    return classify_impl("sa_mask_classify_static", mask, mask_strides, B, H, Sq, Sk, BQ, BK, full_ids,
                         full_ids_strides, full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens,
                         part_lens_strides, ws, stream);
}

}  // extern "C"

namespace {

// Workgroups the persistent forward launches on the current device (2 per compute unit, a multiple of 8, at
// most 512), entries per schedule row, and the bytes of the schedule; 0 when there is no persistent kernel for
// the problem or no device.
size_t schedule_shape(int B, int H, int Sq, int Sk, int BQ, int BK, int mode, int *G_out, int *R_out) {
    if (B <= 0 || H <= 0 || Sq <= 0 || Sk <= 0 || BQ <= 0 || BK <= 0 || Sq % BQ || Sk % BK) return 0;
    if (BQ != 32 && BQ != 64 && BQ != 128) return 0;
    if (log2_exact(BK) < 4 || Sk / BK > 1024 || B >= 32768 || H >= 65536) return 0;
    if (mode == SA_SCHEDULE_PAIRS) {
        // one workgroup per two Q tiles (per one for the middle tile of an unpaired plane), rounded up to whole
        // groups of 8 rows
        const int nQ = Sq / BQ;
        const int64_t BH = (int64_t)B * H;
        int64_t W = (BH / 2) * nQ + ((BH & 1) ? (nQ + 1) / 2 : 0);
        W = (W + 7) / 8 * 8;
        if (W > 0x7fffffffLL) return 0;
        if (G_out) *G_out = (int)W;
        if (R_out) *R_out = 2;
        return (size_t)W * 3 * 16;
    }
    if (mode != SA_SCHEDULE_PERSISTENT) return 0;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    int G = 2 * cus;
    if (G > 512) G = 512;
    G &= ~7;
    if (G < 8) return 0;
    const int64_t N = (int64_t)B * H * (Sq / BQ);
    const int64_t NX = (N + 7) / 8;
    const int64_t R = (NX + G / 8 - 1) / (G / 8);
    if (R > 0x3fffffff) return 0;
    if (G_out) *G_out = G;
    if (R_out) *R_out = (int)R;
    return (size_t)G * (size_t)(R + 1) * 16;
}

int forward_impl(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4], const void *v,
                 const int64_t v_strides[4], void *o, const int64_t o_strides[4], const uint8_t *mask,
                 const int64_t mask_strides[4], const int32_t *full_ids, const int64_t full_ids_strides[4],
                 const int32_t *full_lens, const int64_t full_lens_strides[3], const int32_t *part_ids,
                 const int64_t part_ids_strides[4], const int32_t *part_lens, const int64_t part_lens_strides[3],
                 const uint8_t *packed, const int64_t packed_strides[2], bool use_packed, const int32_t *schedule,
                 size_t schedule_bytes, int schedule_mode, float *lse, const int64_t lse_strides[3], int B, int H,
                 int Sq, int Sk, int D, int BQ, int BK, int dtype, float sm_scale_log2, void *stream,
                 int kernel = SA_FWD_KERNEL_DEFAULT) {
    g_error[0] = 0;
    const int rot_group = kernel >> 8;
    kernel &= 0xff;
    if ((kernel != SA_FWD_KERNEL_DEFAULT && kernel != SA_FWD_KERNEL_SHORT_LISTS && kernel != SA_FWD_KERNEL_ROTATED) ||
        (kernel == SA_FWD_KERNEL_ROTATED ? (rot_group < 2 || rot_group > 64 || (rot_group & (rot_group - 1))) : rot_group != 0))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd_kernel: kernel %d, group %d (0 = default, 1 = short lists, SA_FWD_KERNEL_ROTATED_BY(G) with G = 2, 4, ... 64)", kernel, rot_group);
    if (!q || !k || !v || !o || !q_strides || !k_strides || !v_strides || !o_strides || !full_ids ||
        !full_ids_strides || !full_lens || !full_lens_strides || !part_ids || !part_ids_strides || !part_lens ||
        !part_lens_strides)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd: null pointer argument");
    if (use_packed ? (!packed || !packed_strides) : (!mask || !mask_strides))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd: null pointer argument (%s)",
                    use_packed ? "packed" : "mask");
    if (const int rc = check_tiling(B, H, Sq, Sk, BQ, BK)) return rc;
    if (D <= 0) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd: D must be positive (got %d)", D);
    if (!(sm_scale_log2 > 0.f) || !(sm_scale_log2 < 3.0e38f))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd: sm_scale_log2 must be positive and finite");
    const bool f32 = dtype == SA_DTYPE_FP32;  // the float32 kernels: any BLOCK_Q up to 256, any BLOCK_K
    if (dtype != SA_DTYPE_BF16 && dtype != SA_DTYPE_FP16 && !f32)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: dtype code %d (supported: 0 = bf16, 1 = fp16, 2 = fp32)", dtype);
    if (f32 && kernel == SA_FWD_KERNEL_ROTATED)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd_kernel: the rotated walk needs bf16 or fp16");
    if (D != 64 && D != 128 && D != 256)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: head dim %d (supported: 64, 128, 256)", D);
    int lbk = 0;
    if (f32) {
        if (use_packed && BK % 8 != 0)
            return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd: packed tiles need BLOCK_K to be a multiple of 8 (got %d)", BK);
        if (BQ > (D > 128 ? 128 : 256))
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: BLOCK_Q %d in float32 (supported: 1 to 256, to 128 at head dim 256)", BQ);
    } else {
        if (BQ != 32 && BQ != 64 && BQ != 128 && BQ != 256)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: BLOCK_Q %d (supported: 32, 64, 128, 256)", BQ);
        if (D == 256 && BQ != 64 && BQ != 128)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: BLOCK_Q %d at head dim 256 (supported there: 64, 128)", BQ);
        lbk = log2_exact(BK);
        if (lbk < 4) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: BLOCK_K %d (supported: powers of two >= 16)", BK);
    }
    const int64_t *st[4] = {q_strides, k_strides, v_strides, o_strides};
    const void *ptr[4] = {q, k, v, o};
    const char *name[4] = {"q", "k", "v", "o"};
    const int per16 = f32 ? 4 : 8;  // elements in 16 bytes
    for (int t = 0; t < 4; t++) {
        if (st[t][3] != 1 && D != 1)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: %s must be contiguous in its last dimension (stride %lld)", name[t], (long long)st[t][3]);
        if (!aligned(ptr[t], 16) || st[t][0] % per16 || st[t][1] % per16 || st[t][2] % per16)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: %s needs a 16-byte aligned base and strides that are multiples of %d elements", name[t], per16);
    }
    if (o_strides[2] == 0 || (B > 1 && o_strides[0] == 0) || (H > 1 && o_strides[1] == 0))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd: o must not alias itself (zero stride)");
    if (Sk >= (1 << 30)) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: Sk %d (supported: below 2^30)", Sk);
    // (the kernels form row offsets of K and V from 32-bit factors)
    if (!f32 && (k_strides[2] < 0 || v_strides[2] < 0 || k_strides[2] >= (1 << 24) || v_strides[2] >= (1 << 24)))
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: row strides of k and v must lie in [0, 2^24) elements (%lld, %lld)",
                    (long long)k_strides[2], (long long)v_strides[2]);
    if ((int64_t)B * H * (Sq / BQ) > 0x7fffffffLL)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd: more than 2^31-1 workgroups");

    sa::FwdParams fp{};
    fp.q = static_cast<const uint16_t *>(q);
    fp.k = static_cast<const uint16_t *>(k);
    fp.v = static_cast<const uint16_t *>(v);
    fp.o = static_cast<uint16_t *>(o);
    fp.mask = mask;
    fp.full_ids = full_ids;
    fp.full_lens = full_lens;
    fp.part_ids = part_ids;
    fp.part_lens = part_lens;
    for (int i = 0; i < 3; i++) {
        fp.qs[i] = q_strides[i];
        fp.ks[i] = k_strides[i];
        fp.vs[i] = v_strides[i];
        fp.os[i] = o_strides[i];
        fp.fls[i] = full_lens_strides[i];
        fp.pls[i] = part_lens_strides[i];
    }
    for (int i = 0; i < 4; i++) {
        fp.ms[i] = mask_strides ? mask_strides[i] : 0;
        fp.fis[i] = full_ids_strides[i];
        fp.pis[i] = part_ids_strides[i];
    }
    fp.packed = use_packed ? packed : nullptr;
    fp.pks[0] = use_packed ? packed_strides[0] : 0;
    fp.pks[1] = use_packed ? packed_strides[1] : 0;
    fp.nK = Sk / BK;
    fp.sched = nullptr;
    if (schedule && D <= 128 && !f32) {  // head dim 256 and float32 have no scheduled kernels; the order of Q tiles does not change results
        int G = 0, R = 0;
        const size_t want = schedule_shape(B, H, Sq, Sk, BQ, BK, schedule_mode, &G, &R);
        if (want != 0 && want == schedule_bytes) {
            if (!aligned(schedule, 16))
                return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd_ex: schedule needs a 16-byte aligned base");
            fp.sched = schedule;
            fp.sched_G = G;
            fp.sched_R = R;
        }
    }
    fp.B = B;
    fp.H = H;
    fp.Sq = Sq;
    fp.Sk = Sk;
    fp.nQ = Sq / BQ;
    fp.BK = BK;
    fp.lbk = f32 ? (log2_exact(BK) > 0 ? log2_exact(BK) : 0) : lbk;  // (float32: any BLOCK_K; 0 unless a power of two)
    fp.mask_vec4 = (!use_packed && mask_strides[3] == 1 && aligned(mask, 4) && mask_strides[0] % 4 == 0 &&
                    mask_strides[1] % 4 == 0 && mask_strides[2] % 4 == 0)
                       ? 1
                       : 0;
    fp.scale = sm_scale_log2;
    fp.rot = kernel == SA_FWD_KERNEL_ROTATED ? rot_group : 0;
    fp.lse = nullptr;
    if (lse) {
        if (!lse_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd_lse: null pointer argument (lse_strides)");
        if (!aligned(lse, 4) || (Sq > 1 && lse_strides[2] == 0) || (B > 1 && lse_strides[0] == 0) || (H > 1 && lse_strides[1] == 0))
            return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd_lse: lse must be 4-byte aligned and must not alias itself (zero stride)");
        fp.lse = lse;
        for (int i = 0; i < 3; i++) fp.lses[i] = lse_strides[i];
    }
    if (kernel == SA_FWD_KERNEL_SHORT_LISTS) {
        if (f32 || !sa::fwd_c32_has(fp, dtype, D, BQ))
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd_kernel: the short-list kernel needs bf16 or fp16, head dim 128, BLOCK_Q 128, packed PARTIAL tiles and no schedule");
        if (Sk / BK > SA_FWD_SHORT_LISTS_MAX_ENTRIES * 64)  // (its packed-slot arithmetic stays inside 32 bits far beyond this)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd_kernel: Sk/BLOCK_K %d", Sk / BK);
        const hipError_t e1 = sa::launch_fwd_c32(fp, dtype, D, BQ, static_cast<hipStream_t>(stream));
        if (e1 != hipSuccess) return fail(SA_ERR_HIP, "sa_sparse_attention_fwd_kernel: launch failed: %s", hipGetErrorString(e1));
        return SA_OK;
    }
    const hipError_t e = f32 ? sa::launch_fwd_f32(fp, D, BQ, static_cast<hipStream_t>(stream))
                             : sa::launch_fwd(fp, dtype, D, BQ, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_sparse_attention_fwd: launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}

// Distinct planes of a mask along b and h, and whether `strides` may fold them.
struct Planes {
    int uB, uH;
    bool bcast_b, bcast_h;
};
Planes planes_of(const int64_t mask_strides[4], int B, int H) {
    Planes pl;
    pl.bcast_b = mask_strides[0] == 0 || B == 1;
    pl.bcast_h = mask_strides[1] == 0 || H == 1;
    pl.uB = pl.bcast_b ? 1 : B;
    pl.uH = pl.bcast_h ? 1 : H;
    return pl;
}

}  // namespace

extern "C" {

int sa_sparse_attention_fwd(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                            const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                            const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                            const int64_t full_ids_strides[4], const int32_t *full_lens,
                            const int64_t full_lens_strides[3], const int32_t *part_ids,
                            const int64_t part_ids_strides[4], const int32_t *part_lens,
                            const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk, int D, int BQ, int BK,
                            int dtype, float sm_scale_log2, void *stream) {
    return forward_impl(q, q_strides, k, k_strides, v, v_strides, o, o_strides, mask, mask_strides, full_ids,
                        full_ids_strides, full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens,
                        part_lens_strides, nullptr, nullptr, false, nullptr, 0, 0, nullptr, nullptr, B, H, Sq, Sk, D, BQ,
                        BK, dtype, sm_scale_log2, stream);
}

int sa_sparse_attention_fwd_ex(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                               const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                               const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                               const int64_t full_ids_strides[4], const int32_t *full_lens,
                               const int64_t full_lens_strides[3], const int32_t *part_ids,
                               const int64_t part_ids_strides[4], const int32_t *part_lens,
                               const int64_t part_lens_strides[3], const uint8_t *packed,
                               const int64_t packed_strides[2], const int32_t *schedule, size_t schedule_bytes,
                               int schedule_mode, int B, int H, int Sq, int Sk, int D, int BQ, int BK, int dtype,
                               float sm_scale_log2, void *stream) {
    const bool use_packed = packed != nullptr;
    if (use_packed) {
        g_error[0] = 0;
        if (!packed_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd_ex: null pointer argument (packed_strides)");
        if ((B > 1 && packed_strides[0] % 4) || (H > 1 && packed_strides[1] % 4) || !aligned(packed, 4))
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd_ex: packed needs a 4-byte aligned base and plane strides");
    }
    return forward_impl(q, q_strides, k, k_strides, v, v_strides, o, o_strides, mask, mask_strides, full_ids,
                        full_ids_strides, full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens,
                        part_lens_strides, packed, packed_strides, use_packed, schedule, schedule_bytes, schedule_mode,
                        nullptr, nullptr, B, H, Sq, Sk, D, BQ, BK, dtype, sm_scale_log2, stream);
}

int sa_sparse_attention_fwd_lse(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                                const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                                const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                                const int64_t full_ids_strides[4], const int32_t *full_lens,
                                const int64_t full_lens_strides[3], const int32_t *part_ids,
                                const int64_t part_ids_strides[4], const int32_t *part_lens,
                                const int64_t part_lens_strides[3], const uint8_t *packed,
                                const int64_t packed_strides[2], const int32_t *schedule, size_t schedule_bytes,
                                int schedule_mode, float *lse, const int64_t lse_strides[3], int B, int H, int Sq,
                                int Sk, int D, int BQ, int BK, int dtype, float sm_scale_log2, void *stream) {
    const bool use_packed = packed != nullptr;
    if (use_packed) {
        g_error[0] = 0;
        if (!packed_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd_lse: null pointer argument (packed_strides)");
        if ((B > 1 && packed_strides[0] % 4) || (H > 1 && packed_strides[1] % 4) || !aligned(packed, 4))
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd_lse: packed needs a 4-byte aligned base and plane strides");
    }
    return forward_impl(q, q_strides, k, k_strides, v, v_strides, o, o_strides, mask, mask_strides, full_ids,
                        full_ids_strides, full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens,
                        part_lens_strides, packed, packed_strides, use_packed, schedule, schedule_bytes, schedule_mode,
                        lse, lse_strides, B, H, Sq, Sk, D, BQ, BK, dtype, sm_scale_log2, stream);
}

int sa_sparse_attention_fwd_kernel(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                                   const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                                   const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                                   const int64_t full_ids_strides[4], const int32_t *full_lens,
                                   const int64_t full_lens_strides[3], const int32_t *part_ids,
                                   const int64_t part_ids_strides[4], const int32_t *part_lens,
                                   const int64_t part_lens_strides[3], const uint8_t *packed,
                                   const int64_t packed_strides[2], float *lse, const int64_t lse_strides[3], int B,
                                   int H, int Sq, int Sk, int D, int BQ, int BK, int dtype, float sm_scale_log2,
                                   int kernel, void *stream) {
    const bool use_packed = packed != nullptr;
    if (use_packed) {
        g_error[0] = 0;
        if (!packed_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_fwd_kernel: null pointer argument (packed_strides)");
        if ((B > 1 && packed_strides[0] % 4) || (H > 1 && packed_strides[1] % 4) || !aligned(packed, 4))
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_fwd_kernel: packed needs a 4-byte aligned base and plane strides");
    }
    return forward_impl(q, q_strides, k, k_strides, v, v_strides, o, o_strides, mask, mask_strides, full_ids,
                        full_ids_strides, full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens,
                        part_lens_strides, packed, packed_strides, use_packed, nullptr, 0, 0, lse, lse_strides, B, H, Sq,
                        Sk, D, BQ, BK, dtype, sm_scale_log2, stream, kernel);
}

int sa_validate_metadata(const int32_t *full_ids, const int64_t full_ids_strides[4], const int32_t *full_lens,
                         const int64_t full_lens_strides[3], const int32_t *part_ids, const int64_t part_ids_strides[4],
                         const int32_t *part_lens, const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk,
                         int BQ, int BK, int32_t *flag, void *stream) {
    g_error[0] = 0;
    if (!full_ids || !full_ids_strides || !full_lens || !full_lens_strides || !part_ids || !part_ids_strides ||
        !part_lens || !part_lens_strides || !flag)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_validate_metadata: null pointer argument");
    if (const int rc = check_tiling(B, H, Sq, Sk, BQ, BK)) return rc;
    if (!aligned(flag, 4)) return fail(SA_ERR_INVALID_ARGUMENT, "sa_validate_metadata: flag must be 4-byte aligned");
    sa::ValidateParams vp{};
    vp.full_ids = full_ids;
    vp.full_lens = full_lens;
    vp.part_ids = part_ids;
    vp.part_lens = part_lens;
    for (int i = 0; i < 4; i++) {
        vp.fis[i] = full_ids_strides[i];
        vp.pis[i] = part_ids_strides[i];
    }
    for (int i = 0; i < 3; i++) {
        vp.fls[i] = full_lens_strides[i];
        vp.pls[i] = part_lens_strides[i];
    }
    vp.B = B;
    vp.H = H;
    vp.nQ = Sq / BQ;
    vp.nK = Sk / BK;
    vp.flag = flag;
    const hipError_t e = sa::launch_validate(vp, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_validate_metadata: launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}

size_t sa_fwd_schedule_bytes(int B, int H, int Sq, int Sk, int BQ, int BK, int mode) {
    return schedule_shape(B, H, Sq, Sk, BQ, BK, mode, nullptr, nullptr);
}

int sa_fwd_schedule(const int32_t *full_lens, const int64_t full_lens_strides[3], const int32_t *part_lens,
                    const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk, int BQ, int BK, int mode,
                    int32_t *schedule, size_t schedule_bytes, void *stream) {
    g_error[0] = 0;
    if (!full_lens || !full_lens_strides || !part_lens || !part_lens_strides || !schedule)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_fwd_schedule: null pointer argument");
    if (const int rc = check_tiling(B, H, Sq, Sk, BQ, BK)) return rc;
    int G = 0, R = 0;
    if (mode != SA_SCHEDULE_PERSISTENT && mode != SA_SCHEDULE_PAIRS)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_fwd_schedule: mode %d (0 = persistent, 1 = pairs)", mode);
    const size_t want = schedule_shape(B, H, Sq, Sk, BQ, BK, mode, &G, &R);
    if (want == 0)
        return fail(SA_ERR_UNSUPPORTED, "sa_fwd_schedule: no scheduled forward for BLOCK_Q %d, BLOCK_K %d, Sk %d (BLOCK_Q 32/64/128, BLOCK_K a power of two >= 16, Sk/BLOCK_K <= 1024), or no device", BQ, BK, Sk);
    if (schedule_bytes != want)
        return fail(SA_ERR_WORKSPACE, "sa_fwd_schedule: schedule of %zu bytes required, %zu given", want, schedule_bytes);
    if (!aligned(schedule, 16)) return fail(SA_ERR_UNSUPPORTED, "sa_fwd_schedule: schedule needs a 16-byte aligned base");
    sa::ScheduleParams sp{};
    sp.full_lens = full_lens;
    sp.part_lens = part_lens;
    for (int i = 0; i < 3; i++) {
        sp.fls[i] = full_lens_strides[i];
        sp.pls[i] = part_lens_strides[i];
    }
    sp.B = B;
    sp.H = H;
    sp.nQ = Sq / BQ;
    sp.G = G;
    sp.R = R;
    sp.lbk = log2_exact(BK);
    sp.pairs = mode == SA_SCHEDULE_PAIRS ? 1 : 0;
    sp.sched = schedule;
    const hipError_t e = sa::launch_schedule(sp, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_fwd_schedule: launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}

size_t sa_mask_pack_partial_bytes(const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ, int BK) {
    if (!mask_strides || check_tiling(B, H, Sq, Sk, BQ, BK) != SA_OK || BK % 8) return 0;
    const Planes pl = planes_of(mask_strides, B, H);
    return (size_t)pl.uB * pl.uH * (size_t)Sq * (size_t)Sk / 8;
}

int sa_mask_pack_partial(const uint8_t *mask, const int64_t mask_strides[4], int B, int H, int Sq, int Sk, int BQ,
                         int BK, const int32_t *part_ids, const int64_t part_ids_strides[4],
                         const int32_t *part_lens, const int64_t part_lens_strides[3], uint8_t *packed,
                         const int64_t packed_strides[2], void *stream) {
    g_error[0] = 0;
    if (!mask || !mask_strides || !part_ids || !part_ids_strides || !part_lens || !part_lens_strides || !packed ||
        !packed_strides)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_pack_partial: null pointer argument");
    if (const int rc = check_tiling(B, H, Sq, Sk, BQ, BK)) return rc;
    if (BK % 8) return fail(SA_ERR_UNSUPPORTED, "sa_mask_pack_partial: BLOCK_K %d (must be a multiple of 8)", BK);
    const Planes pl = planes_of(mask_strides, B, H);
    const int64_t plane_bytes = (int64_t)Sq * Sk / 8;
    if ((pl.uB > 1 && packed_strides[0] < plane_bytes) || (pl.uH > 1 && packed_strides[1] < plane_bytes))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_pack_partial: packed planes overlap (strides %lld, %lld; %lld bytes per plane)",
                    (long long)packed_strides[0], (long long)packed_strides[1], (long long)plane_bytes);
    const int nQ = Sq / BQ, nK = Sk / BK;
    if (nQ > 65535 || (int64_t)pl.uB * pl.uH > 65535)
        return fail(SA_ERR_UNSUPPORTED, "sa_mask_pack_partial: more than 65535 Q tiles or distinct mask planes");

    sa::PackParams pp{};
    pp.mask = mask;
    pp.sb = mask_strides[0];
    pp.sh = mask_strides[1];
    pp.sq = mask_strides[2];
    pp.sk = mask_strides[3];
    pp.part_ids = part_ids;
    pp.part_lens = part_lens;
    for (int i = 0; i < 4; i++) pp.pis[i] = part_ids_strides[i];
    for (int i = 0; i < 3; i++) pp.pls[i] = part_lens_strides[i];
    pp.packed = packed;
    pp.ob = packed_strides[0];
    pp.oh = packed_strides[1];
    pp.uB = pl.uB;
    pp.uH = pl.uH;
    pp.BQ = BQ;
    pp.BK = BK;
    pp.nQ = nQ;
    pp.nK = nK;
    pp.vec8 = ((pp.sk == 1 || Sk == 1) && aligned(mask, 8) && pp.sq % 8 == 0 && (pl.uB == 1 || pp.sb % 8 == 0) &&
               (pl.uH == 1 || pp.sh % 8 == 0))
                  ? 1
                  : 0;
    const hipError_t e = sa::launch_pack(pp, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_mask_pack_partial: launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}

size_t sa_mask_terms_workspace_bytes(int distinct_b, int Sq, int Sk, int BQ, int BK) {
    if (distinct_b <= 0 || check_tiling(distinct_b, 1, Sq, Sk, BQ, BK) != SA_OK) return 0;
    return (size_t)distinct_b * (size_t)(Sq / BQ) * (size_t)(Sk / BK);
}

int sa_mask_classify_terms(const int32_t *terms, int n_terms, const int32_t *doc_q, const int64_t doc_q_strides[2],
                           const int32_t *doc_k, const int64_t doc_k_strides[2], int B, int H, int Sq, int Sk, int BQ,
                           int BK, int32_t *full_ids, const int64_t full_ids_strides[4], int32_t *full_lens,
                           const int64_t full_lens_strides[3], int32_t *part_ids, const int64_t part_ids_strides[4],
                           int32_t *part_lens, const int64_t part_lens_strides[3], uint8_t *packed,
                           const int64_t packed_strides[2], void *workspace, size_t workspace_bytes, void *stream) {
    g_error[0] = 0;
    if (!terms || !full_ids || !full_ids_strides || !full_lens || !full_lens_strides || !part_ids ||
        !part_ids_strides || !part_lens || !part_lens_strides || (doc_q && !doc_q_strides) ||
        (doc_k && !doc_k_strides) || (packed && !packed_strides))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: null pointer argument");
    if (n_terms < 1 || n_terms > sa::kMaxMaskTerms)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: %d terms (1..%d)", n_terms, sa::kMaxMaskTerms);
    if (const int rc = check_tiling(B, H, Sq, Sk, BQ, BK)) return rc;
    const int lbk = log2_exact(BK);
    if (lbk < 4) return fail(SA_ERR_UNSUPPORTED, "sa_mask_classify_terms: BLOCK_K %d (supported: powers of two >= 16)", BK);
    if ((int64_t)BQ * BK > 0x7fffffffLL)
        return fail(SA_ERR_UNSUPPORTED, "sa_mask_classify_terms: tiles of more than 2^31-1 entries");

    sa::TermsParams tp{};
    tp.n_terms = n_terms;
    for (int t = 0; t < n_terms; t++) {
        const int32_t *w = terms + 8 * t;
        if (w[0] < 0 || w[0] > 31) return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: term %d has unknown flags %d", t, w[0]);
        if ((w[0] & SA_TERM_SAME_DOC) && !(doc_q && doc_k))
            return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: term %d compares documents, doc_q and doc_k are needed", t);
        // the term as an interval of keys per query row (sa::MaskTerm), in 64 bits before clamping
        const int64_t big = (int64_t)1 << 30;
        auto clamp = [](int64_t x, int64_t lo, int64_t hi) { return x < lo ? lo : (x > hi ? hi : x); };
        sa::MaskTerm &m = tp.terms[t];
        m.a = (int32_t)((w[0] & SA_TERM_BACK) ? clamp((int64_t)w[1] - w[2] + 1, -big, big) : -big);
        m.b = (int32_t)((w[0] & SA_TERM_AHEAD) ? clamp((int64_t)w[1] + w[3], -big, big) : big);
        m.k_lo = (int32_t)((w[0] & SA_TERM_K_RANGE) ? clamp(w[6], 0, Sk) : 0);
        m.k_hi = (int32_t)((w[0] & SA_TERM_K_RANGE) ? clamp(w[7], 0, Sk) : Sk);
        m.q_lo = (int32_t)((w[0] & SA_TERM_Q_RANGE) ? clamp(w[4], 0, Sq) : 0);
        m.q_hi = (int32_t)((w[0] & SA_TERM_Q_RANGE) ? clamp(w[5], 0, Sq) : Sq);
        m.doc = (w[0] & SA_TERM_SAME_DOC) ? 1 : 0;
    }
    if (Sq > (1 << 29) || Sk > (1 << 29))
        return fail(SA_ERR_UNSUPPORTED, "sa_mask_classify_terms: more than 2^29 queries or keys");
    // the mask depends on the batch element only through the document numbers
    const bool per_batch = B > 1 && ((doc_q && doc_q_strides[0] != 0) || (doc_k && doc_k_strides[0] != 0));
    const int uB = per_batch ? B : 1;
    const int nQ = Sq / BQ, nK = Sk / BK;
    if (nQ > 65535 || uB > 65535)
        return fail(SA_ERR_UNSUPPORTED, "sa_mask_classify_terms: more than 65535 Q tiles or distinct mask planes");
    const size_t need = sa_mask_terms_workspace_bytes(uB, Sq, Sk, BQ, BK);
    if (!workspace || workspace_bytes < need)
        return fail(SA_ERR_WORKSPACE, "sa_mask_classify_terms: workspace of %zu bytes required, %zu given", need,
                    workspace ? workspace_bytes : (size_t)0);
    const int64_t ob[4] = {full_ids_strides[0], full_lens_strides[0], part_ids_strides[0], part_lens_strides[0]};
    const int64_t oh[4] = {full_ids_strides[1], full_lens_strides[1], part_ids_strides[1], part_lens_strides[1]};
    int zb = 0, zh = 0;
    for (int i = 0; i < 4; i++) {
        zb += ob[i] == 0;
        zh += oh[i] == 0;
    }
    if (B > 1 && zb != 0 && (zb != 4 || per_batch))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: output batch stride 0 needs a mask shared by the batch and must be 0 on all four outputs");
    if (H > 1 && zh != 0 && zh != 4)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: output head stride 0 must be 0 on all four outputs");
    if (packed) {
        const int64_t plane_bytes = (int64_t)Sq * Sk / 8;
        if (!aligned(packed, 4) || packed_strides[0] % 4)
            return fail(SA_ERR_UNSUPPORTED, "sa_mask_classify_terms: packed needs a 4-byte aligned base and batch stride");
        if (uB > 1 && packed_strides[0] < plane_bytes)
            return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: packed planes overlap (stride %lld, %lld bytes per plane)",
                        (long long)packed_strides[0], (long long)plane_bytes);
        if (H > 1 && packed_strides[1] != 0)
            return fail(SA_ERR_INVALID_ARGUMENT, "sa_mask_classify_terms: the mask is the same for every head: packed_strides[1] must be 0");
    }

    tp.doc_q = doc_q;
    tp.doc_k = doc_k;
    for (int i = 0; i < 2; i++) {
        tp.dqs[i] = doc_q ? doc_q_strides[i] : 0;
        tp.dks[i] = doc_k ? doc_k_strides[i] : 0;
    }
    tp.uB = uB;
    tp.Sq = Sq;
    tp.Sk = Sk;
    tp.BQ = BQ;
    tp.BK = BK;
    tp.nQ = nQ;
    tp.nK = nK;
    tp.cls = static_cast<uint8_t *>(workspace);
    hipError_t e = sa::launch_classify_terms(tp, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_mask_classify_terms: classify launch failed: %s", hipGetErrorString(e));

    sa::CompactParams kp{};
    kp.cls = tp.cls;
    kp.uH = 1;
    kp.bcast_b = !per_batch;
    kp.bcast_h = true;
    kp.oB = (B > 1 && zb == 4) ? 1 : B;
    kp.oH = (H > 1 && zh == 4) ? 1 : H;
    kp.nQ = nQ;
    kp.nK = nK;
    kp.full_ids = full_ids;
    kp.full_lens = full_lens;
    kp.part_ids = part_ids;
    kp.part_lens = part_lens;
    for (int i = 0; i < 4; i++) {
        kp.fis[i] = full_ids_strides[i];
        kp.pis[i] = part_ids_strides[i];
    }
    for (int i = 0; i < 3; i++) {
        kp.fls[i] = full_lens_strides[i];
        kp.pls[i] = part_lens_strides[i];
    }
    e = sa::launch_compact(kp, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_mask_classify_terms: compaction launch failed: %s", hipGetErrorString(e));
    if (!packed) return SA_OK;

    tp.part_ids = part_ids;
    tp.part_lens = part_lens;
    for (int i = 0; i < 4; i++) tp.pis[i] = part_ids_strides[i];
    for (int i = 0; i < 3; i++) tp.pls[i] = part_lens_strides[i];
    tp.packed = packed;
    tp.ob = packed_strides[0];
    e = sa::launch_pack_terms(tp, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_mask_classify_terms: packing launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}

int sa_decode_num_splits(int B, int H, int Sq, int Sk, int BK) {
    if (B <= 0 || H <= 0 || Sq <= 0 || Sq > 32 || Sk <= 0 || BK < 16 || Sk % BK) return 0;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    // two workgroups per compute unit over all (b, h), at least eight 32-key chunks per workgroup
    const int64_t bh = (int64_t)B * H;
    int64_t n = (2 * (int64_t)cus + bh - 1) / bh;
    const int64_t most = Sk / 256 > 0 ? Sk / 256 : 1;
    if (n > most) n = most;
    if (n > 256) n = 256;
    if (n < 1) n = 1;
    return (int)n;
}

size_t sa_decode_workspace_bytes(int B, int H, int Sq, int D, int num_splits) {
    if (B <= 0 || H <= 0 || Sq <= 0 || D <= 0 || num_splits <= 1) return 0;
    return (size_t)B * H * num_splits * Sq * (size_t)(D + 2) * sizeof(float);
}

}  // extern "C"

namespace {
int decode_impl(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4], const void *v,
                const int64_t v_strides[4], void *o, const int64_t o_strides[4], const uint8_t *mask,
                const int64_t mask_strides[4], const int32_t *full_ids, const int64_t full_ids_strides[4],
                const int32_t *full_lens, const int64_t full_lens_strides[3], const int32_t *part_ids,
                const int64_t part_ids_strides[4], const int32_t *part_lens, const int64_t part_lens_strides[3],
                const uint8_t *packed, const int64_t packed_strides[2], int B, int H, int Sq, int Sk, int D, int BK,
                int dtype, float sm_scale_log2, int num_splits, void *workspace, size_t workspace_bytes, float *lse,
                const int64_t lse_strides[3], void *stream) {
    g_error[0] = 0;
    if (!q || !k || !v || !o || !q_strides || !k_strides || !v_strides || !o_strides ||
        !full_ids || !full_ids_strides || !full_lens || !full_lens_strides || !part_ids || !part_ids_strides ||
        !part_lens || !part_lens_strides)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_decode: null pointer argument");
    if (packed ? !packed_strides : (!mask || !mask_strides))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_decode: null pointer argument (%s)", packed ? "packed_strides" : "mask");
    if (packed && (!aligned(packed, 4) || (B > 1 && packed_strides[0] % 4) || (H > 1 && packed_strides[1] % 4)))
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode_ex: packed needs a 4-byte aligned base and plane strides");
    if (const int rc = check_tiling(B, H, Sq, Sk, Sq > 0 ? Sq : 1, BK)) return rc;
    if (Sq > 32) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: Sq %d (supported: 1..32 query rows)", Sq);
    if (D != 64 && D != 128) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: head dim %d (supported: 64, 128)", D);
    if (!(sm_scale_log2 > 0.f) || !(sm_scale_log2 < 3.0e38f))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_decode: sm_scale_log2 must be positive and finite");
    if (dtype != SA_DTYPE_BF16 && dtype != SA_DTYPE_FP16)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: dtype code %d (supported: 0 = bf16, 1 = fp16)", dtype);
    const int lbk = log2_exact(BK);
    if (lbk < 4) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: BLOCK_K %d (supported: powers of two >= 16)", BK);
    // (a packed tile is Sq * BLOCK_K / 8 bytes; the kernel reads its rows as dwords, at BLOCK_K = 16 as halfwords)
    if (packed && BK == 16 && (Sq & 1))
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode_ex: packed tiles at BLOCK_K 16 need an even number of query rows (got %d)", Sq);
    const int64_t *st[4] = {q_strides, k_strides, v_strides, o_strides};
    const void *ptr[4] = {q, k, v, o};
    const char *name[4] = {"q", "k", "v", "o"};
    for (int t = 0; t < 4; t++) {
        if (st[t][3] != 1)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: %s must be contiguous in its last dimension (stride %lld)", name[t], (long long)st[t][3]);
        if (!aligned(ptr[t], 16) || st[t][0] % 8 || st[t][1] % 8 || st[t][2] % 8)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: %s needs a 16-byte aligned base and strides that are multiples of 8 elements", name[t]);
    }
    if ((Sq > 1 && o_strides[2] == 0) || (B > 1 && o_strides[0] == 0) || (H > 1 && o_strides[1] == 0))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_decode: o must not alias itself (zero stride)");
    if ((int64_t)B * H > 65535) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: more than 65535 (b, h) planes");
    if (num_splits == 0) num_splits = sa_decode_num_splits(B, H, Sq, Sk, BK);
    if (num_splits < 1 || num_splits > 256)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_decode: num_splits %d (1..256, or 0 for the default)", num_splits);
    if ((int64_t)(Sk / 32) * num_splits > 0x7fffffffLL)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_decode: Sk / 32 * num_splits exceeds 2^31-1");
    const size_t need = sa_decode_workspace_bytes(B, H, Sq, D, num_splits);
    if (need != 0 && (!workspace || workspace_bytes < need || !aligned(workspace, 16)))
        return fail(SA_ERR_WORKSPACE, "sa_sparse_attention_decode: 16-byte aligned workspace of %zu bytes required, %zu given", need,
                    workspace ? workspace_bytes : (size_t)0);

    sa::DecodeParams dp{};
    dp.q = static_cast<const uint16_t *>(q);
    dp.k = static_cast<const uint16_t *>(k);
    dp.v = static_cast<const uint16_t *>(v);
    dp.o = static_cast<uint16_t *>(o);
    dp.mask = packed ? nullptr : mask;
    dp.packed = packed;
    dp.pks[0] = packed ? packed_strides[0] : 0;
    dp.pks[1] = packed ? packed_strides[1] : 0;
    dp.full_ids = full_ids;
    dp.full_lens = full_lens;
    dp.part_ids = part_ids;
    dp.part_lens = part_lens;
    for (int i = 0; i < 3; i++) {
        dp.qs[i] = q_strides[i];
        dp.ks[i] = k_strides[i];
        dp.vs[i] = v_strides[i];
        dp.os[i] = o_strides[i];
    }
    for (int i = 0; i < 4; i++) dp.ms[i] = packed ? 0 : mask_strides[i];
    // the lists of the one Q tile: b and h strides, and the stride along the entries
    dp.fis[0] = full_ids_strides[0];
    dp.fis[1] = full_ids_strides[1];
    dp.fis[2] = full_ids_strides[3];
    dp.pis[0] = part_ids_strides[0];
    dp.pis[1] = part_ids_strides[1];
    dp.pis[2] = part_ids_strides[3];
    dp.fls[0] = full_lens_strides[0];
    dp.fls[1] = full_lens_strides[1];
    dp.pls[0] = part_lens_strides[0];
    dp.pls[1] = part_lens_strides[1];
    dp.B = B;
    dp.H = H;
    dp.Sq = Sq;
    dp.Sk = Sk;
    dp.BK = BK;
    dp.lbk = lbk;
    dp.mask_vec4 = (!packed && mask_strides[3] == 1 && aligned(mask, 4) && mask_strides[0] % 4 == 0 &&
                    mask_strides[1] % 4 == 0 && mask_strides[2] % 4 == 0)
                       ? 1
                       : 0;
    dp.nsplit = num_splits;
    dp.ws = static_cast<float *>(workspace);
    dp.scale = sm_scale_log2;
    dp.lse = nullptr;
    if (lse) {
        if (!lse_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_decode: null pointer argument (lse_strides)");
        if (!aligned(lse, 4) || (Sq > 1 && lse_strides[2] == 0) || (B > 1 && lse_strides[0] == 0) || (H > 1 && lse_strides[1] == 0))
            return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_decode: lse must be 4-byte aligned and must not alias itself (zero stride)");
        dp.lse = lse;
        for (int i = 0; i < 3; i++) dp.lses[i] = lse_strides[i];
    }
    const hipError_t e = sa::launch_decode(dp, dtype, D, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_sparse_attention_decode: launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}
}  // namespace

extern "C" {

int sa_sparse_attention_decode(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                               const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                               const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                               const int64_t full_ids_strides[4], const int32_t *full_lens,
                               const int64_t full_lens_strides[3], const int32_t *part_ids,
                               const int64_t part_ids_strides[4], const int32_t *part_lens,
                               const int64_t part_lens_strides[3], int B, int H, int Sq, int Sk, int D, int BK,
                               int dtype, float sm_scale_log2, int num_splits, void *workspace, size_t workspace_bytes,
                               float *lse, const int64_t lse_strides[3], void *stream) {
    return decode_impl(q, q_strides, k, k_strides, v, v_strides, o, o_strides, mask, mask_strides, full_ids,
                       full_ids_strides, full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens,
                       part_lens_strides, nullptr, nullptr, B, H, Sq, Sk, D, BK, dtype, sm_scale_log2, num_splits, workspace,
                       workspace_bytes, lse, lse_strides, stream);
}

int sa_sparse_attention_decode_ex(const void *q, const int64_t q_strides[4], const void *k, const int64_t k_strides[4],
                                  const void *v, const int64_t v_strides[4], void *o, const int64_t o_strides[4],
                                  const uint8_t *mask, const int64_t mask_strides[4], const int32_t *full_ids,
                                  const int64_t full_ids_strides[4], const int32_t *full_lens,
                                  const int64_t full_lens_strides[3], const int32_t *part_ids,
                                  const int64_t part_ids_strides[4], const int32_t *part_lens,
                                  const int64_t part_lens_strides[3], const uint8_t *packed,
                                  const int64_t packed_strides[2], int B, int H, int Sq, int Sk, int D, int BK, int dtype,
                                  float sm_scale_log2, int num_splits, void *workspace, size_t workspace_bytes, float *lse,
                                  const int64_t lse_strides[3], void *stream) {
    return decode_impl(q, q_strides, k, k_strides, v, v_strides, o, o_strides, mask, mask_strides, full_ids,
                       full_ids_strides, full_lens, full_lens_strides, part_ids, part_ids_strides, part_lens,
                       part_lens_strides, packed, packed_strides, B, H, Sq, Sk, D, BK, dtype, sm_scale_log2, num_splits,
                       workspace, workspace_bytes, lse, lse_strides, stream);
}

size_t sa_bwd_workspace_bytes(int B, int H, int Sq) {
    if (B <= 0 || H <= 0 || Sq <= 0) return 0;
    return (size_t)B * H * Sq * 2 * sizeof(float);
}

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
                            int H, int Sq, int Sk, int D, int dtype, float sm_scale_log2, void *stream) {
    g_error[0] = 0;
    if (!mask && !(q_packed && k_packed))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_bwd: null pointer argument (mask, without both packed buffers)");
    if ((q_packed && !q_packed_strides) || (k_packed && !k_packed_strides))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_bwd: null pointer argument (packed strides)");
    const void *ptrs[] = {q, k, v, o, d_o, lse, dq, dk, dv, q_full_ids, q_full_lens, q_part_ids, q_part_lens,
                          k_full_ids, k_full_lens, k_part_ids, k_part_lens, q_strides, k_strides, v_strides, o_strides,
                          do_strides, lse_strides, dq_strides, dk_strides, dv_strides,
                          q_full_ids_strides, q_full_lens_strides, q_part_ids_strides, q_part_lens_strides,
                          k_full_ids_strides, k_full_lens_strides, k_part_ids_strides, k_part_lens_strides};
    for (const void *ptr : ptrs)
        if (!ptr) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_bwd: null pointer argument");
    if (const int rc = check_tiling(B, H, Sq, Sk, 128, 128)) return rc;  // tiles of 128 resident and 64 streamed rows both ways
    if (D != 64 && D != 128) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: head dim %d (supported: 64, 128)", D);
    if (dtype != SA_DTYPE_BF16 && dtype != SA_DTYPE_FP16)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: dtype code %d (supported: 0 = bf16, 1 = fp16)", dtype);
    if (!(sm_scale_log2 > 0.f) || !(sm_scale_log2 < 3.0e38f))
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_bwd: sm_scale_log2 must be positive and finite");
    if (Sq / 64 > 2048 || Sk / 64 > 2048)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: more than 2048 tiles of 64 rows along Sq or Sk");
    if ((int64_t)B * H * ((Sq > Sk ? Sq : Sk) / 128) > 0x7fffffffLL)
        return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: more than 2^31-1 workgroups");
    const int64_t *st[9] = {q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides};
    const void *tp[8] = {q, k, v, o, d_o, dq, dk, dv};
    const char *name[8] = {"q", "k", "v", "o", "do", "dq", "dk", "dv"};
    for (int t = 0; t < 8; t++) {
        if (st[t][3] != 1)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: %s must be contiguous in its last dimension", name[t]);
        if (!aligned(tp[t], 16) || st[t][0] % 8 || st[t][1] % 8 || st[t][2] % 8)
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: %s needs a 16-byte aligned base and strides that are multiples of 8 elements", name[t]);
    }
    for (int t = 5; t < 8; t++)
        if (st[t][2] == 0 || (B > 1 && st[t][0] == 0) || (H > 1 && st[t][1] == 0))
            return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_bwd: %s must not alias itself (zero stride)", name[t]);
    const size_t need = sa_bwd_workspace_bytes(B, H, Sq);
    if (!workspace || workspace_bytes < need || !aligned(workspace, 16))
        return fail(SA_ERR_WORKSPACE, "sa_sparse_attention_bwd: 16-byte aligned workspace of %zu bytes required, %zu given", need,
                    workspace ? workspace_bytes : (size_t)0);
    if (need / 2 >= (size_t)1 << 32) return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: B*H*Sq too large");
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const float sm_scale = sm_scale_log2 * 0.69314718056f;

    // per query row: L = lse / ln 2 and Delta = rowsum(dO o O)
    float *stat_l = static_cast<float *>(workspace);
    float *stat_d = stat_l + (size_t)B * H * Sq;
    sa::BwdPrepParams pp{};
    pp.o = static_cast<const uint16_t *>(o);
    pp.d_o = static_cast<const uint16_t *>(d_o);
    pp.lse = lse;
    for (int i = 0; i < 3; i++) {
        pp.os[i] = o_strides[i];
        pp.dos[i] = do_strides[i];
        pp.ls[i] = lse_strides[i];
    }
    pp.stat_l = stat_l;
    pp.stat_d = stat_d;
    pp.B = B;
    pp.H = H;
    pp.Sq = Sq;
    hipError_t e = sa::launch_bwd_prepare(pp, dtype, D, hs);
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_sparse_attention_bwd: launch failed: %s", hipGetErrorString(e));

    auto set3 = [](int64_t(&dst)[3], const int64_t *src) {
        for (int i = 0; i < 3; i++) dst[i] = src[i];
    };
    if (mask && !mask_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_bwd: null pointer argument (mask_strides)");
    const uint8_t *pk[2] = {q_packed, k_packed};
    const int64_t *pks[2] = {q_packed_strides, k_packed_strides};
    for (int i = 0; i < 2; i++)
        if (pk[i] && (!aligned(pk[i], 8) || (B > 1 && pks[i][0] % 8) || (H > 1 && pks[i][1] % 8)))
            return fail(SA_ERR_UNSUPPORTED, "sa_sparse_attention_bwd: packed buffers need 8-byte aligned bases and plane strides");
    const int64_t no_strides[4] = {0, 0, 0, 0};
    if (!mask) mask_strides = no_strides;
    sa::BwdParams bp{};
    bp.mask = mask;
    bp.ms[0] = mask_strides[0];
    bp.ms[1] = mask_strides[1];
    bp.stat_l = stat_l;
    bp.stat_d = stat_d;
    bp.sts[0] = (int64_t)H * Sq;
    bp.sts[1] = Sq;
    bp.sts[2] = 1;
    bp.B = B;
    bp.H = H;
    bp.scale = sm_scale_log2;
    const bool m4 = mask && aligned(mask, 4) && mask_strides[0] % 4 == 0 && mask_strides[1] % 4 == 0;

    // dQ: queries resident, keys streamed
    bp.x = static_cast<const uint16_t *>(q);
    bp.g = static_cast<const uint16_t *>(d_o);
    bp.y = static_cast<const uint16_t *>(k);
    bp.z = static_cast<const uint16_t *>(v);
    bp.out = static_cast<uint16_t *>(dq);
    set3(bp.xs, q_strides);
    set3(bp.gs, do_strides);
    set3(bp.ys, k_strides);
    set3(bp.zs, v_strides);
    set3(bp.outs, dq_strides);
    bp.mrs = mask_strides[2];
    bp.mcs = mask_strides[3];
    bp.mask_vec4 = (m4 && bp.mcs == 1 && bp.mrs % 4 == 0) ? 1 : 0;
    bp.full_ids = q_full_ids;
    bp.full_lens = q_full_lens;
    bp.part_ids = q_part_ids;
    bp.part_lens = q_part_lens;
    for (int i = 0; i < 4; i++) {
        bp.fis[i] = q_full_ids_strides[i];
        bp.pis[i] = q_part_ids_strides[i];
    }
    set3(bp.fls, q_full_lens_strides);
    set3(bp.pls, q_part_lens_strides);
    bp.packed = q_packed;
    bp.pks[0] = q_packed ? q_packed_strides[0] : 0;
    bp.pks[1] = q_packed ? q_packed_strides[1] : 0;
    bp.nS = Sk / 64;
    bp.nR = Sq / 128;
    bp.first_tile_first = 0;
    bp.out_scale = sm_scale;
    e = sa::launch_bwd(bp, dtype, D, true, false, hs);
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_sparse_attention_bwd: launch failed: %s", hipGetErrorString(e));

    // dK and dV: keys resident, queries streamed; the mask is walked transposed, or read from the caller's
    // transposed copy [B,H,Sk,Sq], whose rows are contiguous in the streamed direction
    const uint8_t *mk = mask;
    int64_t mk_b = mask_strides[0], mk_h = mask_strides[1], mk_r = mask_strides[3], mk_c = mask_strides[2];
    if (mask_t) {
        if (!mask_t_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_sparse_attention_bwd: null pointer argument (mask_t_strides)");
        mk = mask_t;
        mk_b = mask_t_strides[0];
        mk_h = mask_t_strides[1];
        mk_r = mask_t_strides[2];
        mk_c = mask_t_strides[3];
    }
    bp.mask = mk;
    bp.ms[0] = mk_b;
    bp.ms[1] = mk_h;
    bp.x = static_cast<const uint16_t *>(k);
    bp.g = static_cast<const uint16_t *>(v);
    bp.y = static_cast<const uint16_t *>(q);
    bp.z = static_cast<const uint16_t *>(d_o);
    set3(bp.xs, k_strides);
    set3(bp.gs, v_strides);
    set3(bp.ys, q_strides);
    set3(bp.zs, do_strides);
    bp.mrs = mk_r;
    bp.mcs = mk_c;
    bp.mask_vec4 = (aligned(mk, 4) && mk_b % 4 == 0 && mk_h % 4 == 0 && mk_c == 1 && mk_r % 4 == 0) ? 1 : 0;
    bp.full_ids = k_full_ids;
    bp.full_lens = k_full_lens;
    bp.part_ids = k_part_ids;
    bp.part_lens = k_part_lens;
    for (int i = 0; i < 4; i++) {
        bp.fis[i] = k_full_ids_strides[i];
        bp.pis[i] = k_part_ids_strides[i];
    }
    set3(bp.fls, k_full_lens_strides);
    set3(bp.pls, k_part_lens_strides);
    bp.packed = k_packed;
    bp.pks[0] = k_packed ? k_packed_strides[0] : 0;
    bp.pks[1] = k_packed ? k_packed_strides[1] : 0;
    bp.nS = Sq / 64;
    bp.nR = Sk / 128;
    bp.first_tile_first = 1;
    bp.out = static_cast<uint16_t *>(dk);
    set3(bp.outs, dk_strides);
    bp.out_scale = sm_scale;
    e = sa::launch_bwd(bp, dtype, D, false, false, hs);
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_sparse_attention_bwd: launch failed: %s", hipGetErrorString(e));
    bp.out = static_cast<uint16_t *>(dv);
    set3(bp.outs, dv_strides);
    bp.out_scale = 1.f;
    e = sa::launch_bwd(bp, dtype, D, false, true, hs);
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_sparse_attention_bwd: launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}

int sa_merge_attention_parts(const void *o_parts, const int64_t o_parts_strides[5], const float *lse_parts,
                             const int64_t lse_parts_strides[4], void *o, const int64_t o_strides[4], float *lse,
                             const int64_t lse_strides[3], int n, int B, int H, int Sq, int D, int dtype,
                             void *stream) {
    g_error[0] = 0;
    if (!o_parts || !o_parts_strides || !lse_parts || !lse_parts_strides || !o || !o_strides)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_merge_attention_parts: null pointer argument");
    if (n <= 0 || B <= 0 || H <= 0 || Sq <= 0 || D <= 0)
        return fail(SA_ERR_INVALID_ARGUMENT, "sa_merge_attention_parts: n, B, H, Sq, D must be positive");
    if (D % 8) return fail(SA_ERR_UNSUPPORTED, "sa_merge_attention_parts: D %d (supported: multiples of 8)", D);
    if (dtype != SA_DTYPE_BF16 && dtype != SA_DTYPE_FP16)
        return fail(SA_ERR_UNSUPPORTED, "sa_merge_attention_parts: dtype code %d (supported: 0 = bf16, 1 = fp16)", dtype);
    if (o_parts_strides[4] != 1 || o_strides[3] != 1)
        return fail(SA_ERR_UNSUPPORTED, "sa_merge_attention_parts: o_parts and o must be contiguous in their last dimension");
    if (!aligned(o_parts, 16) || !aligned(o, 16) || o_parts_strides[0] % 8 || o_parts_strides[1] % 8 ||
        o_parts_strides[2] % 8 || o_parts_strides[3] % 8 || o_strides[0] % 8 || o_strides[1] % 8 || o_strides[2] % 8)
        return fail(SA_ERR_UNSUPPORTED, "sa_merge_attention_parts: o_parts and o need 16-byte aligned bases and strides that are multiples of 8 elements");
    if (lse && !lse_strides) return fail(SA_ERR_INVALID_ARGUMENT, "sa_merge_attention_parts: null pointer argument (lse_strides)");
    if ((int64_t)B * H * Sq * (D / 8) / 256 > 0x7fffffffLL)
        return fail(SA_ERR_UNSUPPORTED, "sa_merge_attention_parts: more than 2^31-1 workgroups");
    sa::MergeParams mp{};
    mp.o_parts = static_cast<const uint16_t *>(o_parts);
    mp.lse_parts = lse_parts;
    mp.o = static_cast<uint16_t *>(o);
    mp.lse = lse;
    for (int i = 0; i < 4; i++) {
        mp.ops[i] = o_parts_strides[i];
        mp.lps[i] = lse_parts_strides[i];
    }
    for (int i = 0; i < 3; i++) {
        mp.os[i] = o_strides[i];
        mp.lses[i] = lse ? lse_strides[i] : 0;
    }
    mp.n = n;
    mp.B = B;
    mp.H = H;
    mp.Sq = Sq;
    mp.D = D;
    const hipError_t e = sa::launch_merge_parts(mp, dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(SA_ERR_HIP, "sa_merge_attention_parts: launch failed: %s", hipGetErrorString(e));
    return SA_OK;
}

}  // extern "C"
