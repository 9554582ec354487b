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

// A hidden load into an ordinary variable is only safe while the compiler never copies that variable between issue and
// use: a copy (which it may make where two definitions meet at a loop header, or when it splits a live range) moves the
// stale contents and frees the register the data later lands in, which by then holds something else.  Use hidden_load
// in straight-line prologues only; data that stays in flight across a loop back-edge goes global -> LDS (load16_to_lds).

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
