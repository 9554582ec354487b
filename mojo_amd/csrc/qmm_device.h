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
