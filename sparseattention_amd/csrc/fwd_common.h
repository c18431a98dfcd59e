// Helpers shared by the forward kernels: register types, per-dtype MFMA wrappers, the direct global->LDS
// load, the LDS row swizzles and the constants of the online softmax.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "kernels.h"

namespace sa {
namespace {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
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
    // 16x16x32 product; lane l supplies row/column l%16 and the 8 contraction indices 8*(l/16)..+7, and
    // receives column l%16, rows 4*(l/16)..+3
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        const f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    static __device__ __forceinline__ uint32_t scale2(uint32_t w, float s) {  // both halves times s, rounded again
        return pack2(__uint_as_float(w << 16) * s, __uint_as_float(w & 0xffff0000u) * s);
    }
    static __device__ __forceinline__ u32x2 tr_read(const uint8_t *lds_ptr) {
        return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((SA_LDS bf16x4 *)lds_ptr));
    }
    static __device__ __forceinline__ u32x4 ones4() {  // eight 1.0 values, an all-ones MFMA operand
        return u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    }
};

template <>
struct Elem<1> {  // fp16
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        const f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
    static __device__ __forceinline__ uint32_t scale2(uint32_t w, float s) {
        const f16x2 h = __builtin_bit_cast(f16x2, w);
        return pack2((float)h.x * s, (float)h.y * s);
    }
    static __device__ __forceinline__ u32x2 tr_read(const uint8_t *lds_ptr) {
        // the transposing read only moves 16-bit lanes around, so the bf16 flavour serves fp16 too
        return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((SA_LDS bf16x4 *)lds_ptr));
    }
    static __device__ __forceinline__ u32x4 ones4() {
        return u32x4{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
    }
};

// Exchange a value between lane and lane^32 and combine: returns op(x[lane], x[lane^32]) in all lanes.
__device__ __forceinline__ float half_swap_max(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

constexpr float kNegInf = -__builtin_inff();

// 16 bytes per lane from global memory (wave-uniform base + per-lane byte offset) straight into LDS:
// lane i of the wave writes LDS address lds_addr + 16*i.
// Issued through inline assembly on purpose: the compiler then does not track it, so it does not hold
// back later LDS reads of the OTHER buffer until the transfer lands.  Whoever reads the destination
// must execute "s_waitcnt vmcnt(0)" and a workgroup barrier first (the main loop does).
// The load takes its LDS address from m0, which needs a wait state after a scalar write.  The write of m0 and the
// s_nop therefore stay INSIDE this asm statement: handing the address over as an "{m0}" input leaves the copy into
// the (reserved) register to the compiler, with no guarantee of the wait state or that two loads do not share one
// copy, and a build of that form ended in a GPU memory fault.
// STREAM: the bytes are read once by the whole launch (the K/V rows of the few-rows kernels): the load carries the
// non-temporal hint, with which a streaming read runs at 7.1 TB/s on this device against 6.3 TB/s without.
template <bool STREAM = false>
__device__ __forceinline__ void dma16(const void *base, uint32_t lane_offset, uint32_t lds_addr) {
    // the base is wave-uniform by construction; say so in a way the register allocator cannot miss
    const uint64_t b = (uint64_t)(uintptr_t)base;
    // (readfirstlane returns a signed int: widen through uint32_t, or the low half sign-extends)
    const uint64_t ub = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32)) << 32);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    if constexpr (STREAM) {
        asm volatile(
            "s_mov_b32 m0, %2\n\t"
            "s_nop 0\n\t"
            "global_load_lds_dwordx4 %0, %1 nt"
            :
            : "v"(lane_offset), "s"(ub), "s"(lds_addr)
            : "memory");
    } else {
        asm volatile(
            "s_mov_b32 m0, %2\n\t"
            "s_nop 0\n\t"
            "global_load_lds_dwordx4 %0, %1"
            :
            : "v"(lane_offset), "s"(ub), "s"(lds_addr)
            : "memory");  // m0 is written; nothing else in these kernels keeps a value in it
    }
}

// N dwords from N wave-uniform addresses by scalar loads that are issued back to back and share ONE wait.  Left to
// the compiler, loads whose addresses it forms one after the other are waited for one after the other as well, a
// memory round trip each; at the start of a Q tile that is most of the time before the first K/V request.
template <int N>
__device__ __forceinline__ void scalar_gather(const int32_t *const (&a)[N], int (&o)[N]) {
    static_assert(N == 4 || N == 6 || N == 10, "counts + first slots of both lists for 1, 2 or 4 entries per chunk");
    const uint64_t *const q = reinterpret_cast<const uint64_t *>(&a[0]);  // (pointers as 64-bit scalars)
    if constexpr (N == 4) {
        asm volatile(
            "s_load_dword %0, %4, 0x0\n\ts_load_dword %1, %5, 0x0\n\ts_load_dword %2, %6, 0x0\n\t"
            "s_load_dword %3, %7, 0x0\n\ts_waitcnt lgkmcnt(0)"
            : "=&s"(o[0]), "=&s"(o[1]), "=&s"(o[2]), "=&s"(o[3])
            : "s"(q[0]), "s"(q[1]), "s"(q[2]), "s"(q[3])
            : "memory");
    } else if constexpr (N == 6) {
        asm volatile(
            "s_load_dword %0, %6, 0x0\n\ts_load_dword %1, %7, 0x0\n\ts_load_dword %2, %8, 0x0\n\t"
            "s_load_dword %3, %9, 0x0\n\ts_load_dword %4, %10, 0x0\n\ts_load_dword %5, %11, 0x0\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&s"(o[0]), "=&s"(o[1]), "=&s"(o[2]), "=&s"(o[3]), "=&s"(o[4]), "=&s"(o[5])
            : "s"(q[0]), "s"(q[1]), "s"(q[2]), "s"(q[3]), "s"(q[4]), "s"(q[5])
            : "memory");
    } else {
        asm volatile(
            "s_load_dword %0, %10, 0x0\n\ts_load_dword %1, %11, 0x0\n\ts_load_dword %2, %12, 0x0\n\t"
            "s_load_dword %3, %13, 0x0\n\ts_load_dword %4, %14, 0x0\n\ts_load_dword %5, %15, 0x0\n\t"
            "s_load_dword %6, %16, 0x0\n\ts_load_dword %7, %17, 0x0\n\ts_load_dword %8, %18, 0x0\n\t"
            "s_load_dword %9, %19, 0x0\n\ts_waitcnt lgkmcnt(0)"
            : "=&s"(o[0]), "=&s"(o[1]), "=&s"(o[2]), "=&s"(o[3]), "=&s"(o[4]), "=&s"(o[5]), "=&s"(o[6]), "=&s"(o[7]),
              "=&s"(o[8]), "=&s"(o[9])
            : "s"(q[0]), "s"(q[1]), "s"(q[2]), "s"(q[3]), "s"(q[4]), "s"(q[5]), "s"(q[6]), "s"(q[7]), "s"(q[8]), "s"(q[9])
            : "memory");
    }
}

// Swizzles of the 16-byte pieces inside an LDS row.  Rows are stored unpadded (D*2 bytes) because a
// direct global->LDS load writes 64 lanes x 16 bytes contiguously; instead the piece index is XORed
// with a function of the row so that
//   K: the 16 rows read together by one quarter-wave ds_read_b128 fall into 16 different bank groups,
//   V: the 4 rows touched by one half-wave transposing read fall into 4 different 64-byte bank groups.
template <int D>
__device__ __forceinline__ int k_swizzle(int row) {
    return D >= 128 ? (row & 15) : ((row >> 1) & 7);
}
template <int D>
__device__ __forceinline__ int v_swizzle(int row) {
    return D >= 128 ? 4 * (row & 3) : 4 * ((row >> 1) & 1);
}

// log2-domain slack before the running maximum is raised (and the accumulator rescaled).  Scores are
// exponentiated against a reference value that may lag the true row maximum by up to this much, so
// P stays <= 2^kMaxSlack; the final division by the row sum cancels the reference exactly.
constexpr float kMaxSlack = 8.0f;

// List entries kept in LDS per Q tile (8 KiB); longer lists are read from global memory per chunk.
constexpr int kListCap = 2048;
// Persistent workgroups keep two lists in the same space, of the Q tile at hand and of the next one.
constexpr int kPsListCap = 1024;

template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {  // f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// Raises a kernel's dynamic shared-memory limit to `bytes`, once per device: `done` is the caller's bit mask of the
// devices (ordinals below 64) that have it.  Two threads racing here set the same value twice.
template <class K>
hipError_t allow_dynamic_smem(K kern, int bytes, unsigned long long &done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = dev >= 0 && dev < 64 ? 1ull << dev : 0ull;
    if (bit != 0 && (__atomic_load_n(&done, __ATOMIC_RELAXED) & bit)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && bit != 0) __atomic_fetch_or(&done, bit, __ATOMIC_RELAXED);
    return e;
}

}  // namespace
}  // namespace sa
