// Device-side helpers shared by every kernel: half conversions, block layouts
// of the GGUF encodings, nibble / 6-bit field decoding, wave reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qmm {

constexpr int kWave = 64;

constexpr int Q4_0_EPB = 32, Q4_0_BPB = 18;
constexpr int Q8_0_EPB = 32, Q8_0_BPB = 34;
constexpr int Q4_K_EPB = 256, Q4_K_BPB = 144;
constexpr int Q6_K_EPB = 256, Q6_K_BPB = 210;
constexpr int Q5_K_EPB = 256, Q5_K_BPB = 176;

__device__ __forceinline__ float h2f(uint16_t h) {
    union { uint16_t u; _Float16 f; } v;
    v.u = h;
    return (float)v.f;
}
__device__ __forceinline__ uint16_t f2h(float f) {
    union { uint16_t u; _Float16 h; } v;
    v.h = (_Float16)f;  // v_cvt_f16_f32: round-to-nearest-even
    return v.u;
}
__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
// Round-to-nearest-even with canonical NaN, the rule of the reference's
// software bf16 narrowing (stdlib/src/builtin/simd.mojo:3279-3300).
__device__ __forceinline__ uint16_t f2bf(float f) {
    uint32_t x = __float_as_uint(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(((x >> 16) & 0x8000u) | 0x7fc0u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

// lhs element i as fp32; InT is float or a bf16 bit pattern (uint16_t).
template <typename InT>
__device__ __forceinline__ float load_f32(const InT* p, int64_t i) {
    if constexpr (sizeof(InT) == 4) return p[i];
    else return bf2f(p[i]);
}

// The per-block rule of the Q8_0 activation quantiser (GGUF quantize_row_q8_0), shared by the stand-alone
// quantiser and by every Q4_0 matmul kernel that quantises its lhs itself: d = amax / 127 in fp32, the stored
// scale is d narrowed to fp16 (returned as its bit pattern), and a code is round-half-away(x * (1 / d)) with the
// fp32 d (all codes 0 for an all-zero block).
__device__ __forceinline__ float q8_0_block_rule(float amax, uint16_t& d_half) {
    const float d = amax / 127.0f;
    d_half = f2h(d);
    return d != 0.0f ? 1.0f / d : 0.0f;
}
__device__ __forceinline__ int q8_0_code(float v, float inv_d) { return (int)roundf(v * inv_d); }

__device__ __forceinline__ uint32_t byte_of(uint32_t w, int i) { return (w >> (8 * i)) & 0xffu; }

// Q4_K: 6-bit scale and min of sub-block j (0..7) from the 12 packed bytes,
// given as three little-endian dwords s[0..2].
__device__ __forceinline__ void q4k_scale_min(int j, const uint32_t s[3], uint32_t& sc, uint32_t& mn) {
    if (j < 4) {
        sc = byte_of(s[0], j) & 63u;
        mn = byte_of(s[1], j) & 63u;
    } else {
        uint32_t hi = byte_of(s[2], j - 4);
        sc = (hi & 0xFu) | ((byte_of(s[0], j - 4) >> 6) << 4);
        mn = (hi >> 4) | ((byte_of(s[1], j - 4) >> 6) << 4);
    }
}

// Sum over the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Cross-lane data movement inside the VALU (DPP), no LDS round trip.
// CTRL: 0xB1 swap lane pairs, 0x4E swap pairs of a quad, 0x141 mirror 8 lanes, 0x140 mirror 16 lanes.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// Sum over each aligned group of 8 lanes; every lane of the group gets it.
__device__ __forceinline__ float sum8(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    return v;
}

// Sum over the 64 lanes through DPP; the total is returned in every lane.
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);  // every lane of a 16-lane row holds the row sum
    const int b = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0)), r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32)), r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// The same sum, delivered in lane 63 only (the other lanes hold partial sums): after the four steps inside the
// 16-lane rows, row_bcast15 adds row 0's total into row 1 and row 2's into row 3, row_bcast31 adds row 1's
// into row 3.  Same association as wave_sum_dpp, (r0 + r1) + (r2 + r3), so the value is bit-identical.
__device__ __forceinline__ float wave_sum_dpp_lane63(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xa, 0xf, false));  // row_bcast15 -> rows 1, 3
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xc, 0xf, false));  // row_bcast31 -> rows 2, 3
    return v;
}

// Maxima over the 64 lanes of N unsigned values per lane at once (N = 2, 4 or 8); the results are wave-uniform.
// Used on the bit patterns of float magnitudes: with the sign cleared the unsigned order is the numeric order
// (NaN patterns sort above infinity).  Every step is one v_max_u32 with a DPP operand per value (the compiler keeps
// the lane permutation and the maximum apart and pads them with wait states); the N values of a step are
// independent, so only the first instruction of a step waits (s_nop 1: a DPP operand may be read two wait states
// after the instruction that wrote it).  Steps: swap lane pairs, swap pairs of a quad, mirror 8, mirror 16, then
// row_bcast15 into rows 1 and 3 and row_bcast31 into row 3: lane 63 holds the maximum.
#define QMM_UMAX1(CTRL, A) "v_max_u32_dpp " A ", " A ", " A " " CTRL " bank_mask:0xf\n\t"
#define QMM_UMAX_STEPS(M)                                                                                         \
    M("quad_perm:[1,0,3,2] row_mask:0xf") M("quad_perm:[2,3,0,1] row_mask:0xf") M("row_half_mirror row_mask:0xf") \
    M("row_mirror row_mask:0xf") M("row_bcast:15 row_mask:0xa") M("row_bcast:31 row_mask:0xc")
template <int N>
__device__ __forceinline__ void wave_umax_many(uint32_t (&v)[N]) {
    static_assert(N == 2 || N == 4 || N == 8, "2, 4 or 8 values");
    if constexpr (N == 2) {
#define QMM_STEP(C) asm volatile("s_nop 1\n\t" QMM_UMAX1(C, "%0") "s_nop 0\n\t" QMM_UMAX1(C, "%1") : "+v"(v[0]), "+v"(v[1]));
        QMM_UMAX_STEPS(QMM_STEP)
#undef QMM_STEP
    } else if constexpr (N == 4) {
#define QMM_STEP(C)                                                                                         \
    asm volatile("s_nop 1\n\t" QMM_UMAX1(C, "%0") QMM_UMAX1(C, "%1") QMM_UMAX1(C, "%2") QMM_UMAX1(C, "%3") \
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
        QMM_UMAX_STEPS(QMM_STEP)
#undef QMM_STEP
    } else {
#define QMM_STEP(C)                                                                                         \
    asm volatile("s_nop 1\n\t" QMM_UMAX1(C, "%0") QMM_UMAX1(C, "%1") QMM_UMAX1(C, "%2") QMM_UMAX1(C, "%3") \
                     QMM_UMAX1(C, "%4") QMM_UMAX1(C, "%5") QMM_UMAX1(C, "%6") QMM_UMAX1(C, "%7")             \
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
        QMM_UMAX_STEPS(QMM_STEP)
#undef QMM_STEP
    }
    asm volatile("s_nop 1");  // (the readlanes below are the compiler's: it does not see what the block above wrote last)
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = (uint32_t)__builtin_amdgcn_readlane((int)v[i], 63);
}
#undef QMM_UMAX_STEPS
// the magnitude bits of the largest of four floats (lane-local)
__device__ __forceinline__ uint32_t max_abs_bits(float x0, float x1, float x2, float x3) {
    const uint32_t a0 = __float_as_uint(x0) & 0x7fffffffu, a1 = __float_as_uint(x1) & 0x7fffffffu;
    const uint32_t a2 = __float_as_uint(x2) & 0x7fffffffu, a3 = __float_as_uint(x3) & 0x7fffffffu;
    return max(max(a0, a1), max(a2, a3));
}

// Largest value of a non-negative float over the 64 lanes, as its bit pattern (wave-uniform).
__device__ __forceinline__ uint32_t wave_max_nonneg_bits(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    const int b = __float_as_int(v);
    uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane(b, 0), r1 = (uint32_t)__builtin_amdgcn_readlane(b, 16);
    uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane(b, 32), r3 = (uint32_t)__builtin_amdgcn_readlane(b, 48);
    r0 = r0 > r1 ? r0 : r1;
    r2 = r2 > r3 ? r2 : r3;
    return r0 > r2 ? r0 : r2;
}

}  // namespace qmm
