// Loads that the compiler is not told about, for kernels that keep several items of weight data in
// flight into LDS while they compute.
//
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight to LDS (at
// m0 + 16 * lane), holding no registers while in flight.  Its builtin makes the compiler wait for
// every such load before each LDS read, which leaves nothing in flight; and any wait the compiler
// places for an ordinary load counts these too (vmcnt is one in-order counter) and drains them.  So
// both kinds are issued from inline asm here, and the kernel waits itself with s_waitcnt vmcnt(n),
// n = the number of load instructions it knows to be younger than the data it needs.
#pragma once
#include "qmm_internal.h"

namespace qmm {

typedef __attribute__((address_space(3))) void* lds_space_ptr;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// LDS byte address of a pointer into shared memory, as a wave-uniform scalar.
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_space_ptr)p);
}

// 16 bytes per lane from global memory to LDS at lds_base + 16 * lane (lds_base uniform).  m0 is put
// back; the s_nop is the wait state the hardware wants between a write of m0 and an LDS-direct load.
__device__ __forceinline__ void load16_to_lds(const void* g, uint32_t lds_base) {
    uint32_t keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(g), "s"(lds_base)
                 : "memory");
}
// The same for data that is read exactly once (weight streams): marked non-temporal, so that the caches do not
// keep it (a plain read of a 453 MB buffer runs at 7.0 TB/s with the mark against 6.3 TB/s without).
__device__ __forceinline__ void load16_to_lds_once(const void* g, uint32_t lds_base) {
    uint32_t keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(g), "s"(lds_base)
                 : "memory");
}

// The same with the address split into a wave-uniform 64-bit base (scalar registers) and a 32-bit byte offset per
// lane: a kernel that walks a tensor keeps the lane offsets fixed and advances the base with scalar arithmetic,
// which costs no vector instruction per load.
__device__ __forceinline__ void load16_to_lds(uint32_t lane_offset, const void* uniform_base, uint32_t lds_base) {
    uint32_t keep;
    // (the base is made uniform explicitly: an address the compiler cannot prove uniform would be handed over in vector registers)
    const uint64_t b = (uint64_t)(uintptr_t)uniform_base;
    const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) |
                        (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(lane_offset), "s"(sb), "s"(lds_base)
                 : "memory");
}

// Plain global loads into registers, hidden the same way.  The destination may only be used after
// wait_vmcnt and tie() on it.
__device__ __forceinline__ void hidden_load(u32x4& d, const void* g) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(d) : "v"(g) : "memory");
}
__device__ __forceinline__ void hidden_load(u32x2& d, const void* g) {
    asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(d) : "v"(g) : "memory");
}
template <typename T>
__device__ __forceinline__ void tie(T& d) {
    asm volatile("" : "+v"(d));
}

// Loads into FIXED accumulation registers (a[R], a[R + 1], ...), for data that stays in flight across loop
// back-edges.  A hidden load into an ordinary variable is only safe while the compiler never copies that
// variable between issue and use: a copy (which it may make where two definitions meet at a loop header, or
// when it splits a live range) moves the stale contents and frees the register the data later lands in, which
// by then holds something else.  Accumulation registers named here are never allocated by the compiler for
// anything that lives across these statements (they are declared clobbered), so the data is where it was sent;
// it is moved to ordinary registers with agpr_read after the wait.  A kernel that uses these must not need
// accumulation registers of its own in that range (check its resource report: AGPRs == the range reserved).
template <int R> __device__ __forceinline__ void agpr_load2(const void* g);
template <int R> __device__ __forceinline__ void agpr_load4(const void* g);
template <int R> __device__ __forceinline__ u32x2 agpr_read2();
template <int R> __device__ __forceinline__ u32x4 agpr_read4();
#define QMM_AGPR2(R0, R1)                                                                                                   \
    template <> __device__ __forceinline__ void agpr_load2<R0>(const void* g) {                                             \
        asm volatile("global_load_dwordx2 a[" #R0 ":" #R1 "], %0, off" ::"v"(g) : "memory", "a" #R0, "a" #R1);               \
    }                                                                                                                       \
    template <> __device__ __forceinline__ u32x2 agpr_read2<R0>() {                                                         \
        uint32_t x, y;                                                                                                      \
        asm volatile("v_accvgpr_read_b32 %0, a" #R0 "\n\tv_accvgpr_read_b32 %1, a" #R1 : "=v"(x), "=v"(y)::"memory");       \
        u32x2 v;                                                                                                            \
        v.x = x; v.y = y;                                                                                                   \
        return v;                                                                                                           \
    }
#define QMM_AGPR4(R0, R1, R2, R3)                                                                                           \
    template <> __device__ __forceinline__ void agpr_load4<R0>(const void* g) {                                             \
        asm volatile("global_load_dwordx4 a[" #R0 ":" #R3 "], %0, off" ::"v"(g)                                              \
                     : "memory", "a" #R0, "a" #R1, "a" #R2, "a" #R3);                                                       \
    }                                                                                                                       \
    template <> __device__ __forceinline__ u32x4 agpr_read4<R0>() {                                                         \
        uint32_t x, y, z, w;                                                                                                \
        asm volatile("v_accvgpr_read_b32 %0, a" #R0 "\n\tv_accvgpr_read_b32 %1, a" #R1 "\n\tv_accvgpr_read_b32 %2, a" #R2   \
                     "\n\tv_accvgpr_read_b32 %3, a" #R3                                                                     \
                     : "=v"(x), "=v"(y), "=v"(z), "=v"(w)::"memory");                                                       \
        u32x4 v;                                                                                                            \
        v.x = x; v.y = y; v.z = z; v.w = w;                                                                                 \
        return v;                                                                                                           \
    }
QMM_AGPR2(0, 1)
QMM_AGPR2(2, 3)
QMM_AGPR2(4, 5)
QMM_AGPR2(6, 7)
QMM_AGPR4(8, 9, 10, 11)
QMM_AGPR4(12, 13, 14, 15)
#undef QMM_AGPR2
#undef QMM_AGPR4

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Wait until at most `items` items of L load instructions each (items 0..3), plus X more if `extra`,
// are outstanding.
template <int L, int X>
__device__ __forceinline__ void wait_items(int items, bool extra) {
    if (extra) {
        if (items >= 3) wait_vmcnt<3 * L + X>();
        else if (items == 2) wait_vmcnt<2 * L + X>();
        else if (items == 1) wait_vmcnt<L + X>();
        else wait_vmcnt<X>();
    } else {
        if (items >= 3) wait_vmcnt<3 * L>();
        else if (items == 2) wait_vmcnt<2 * L>();
        else if (items == 1) wait_vmcnt<L>();
        else wait_vmcnt<0>();
    }
}

}  // namespace qmm
