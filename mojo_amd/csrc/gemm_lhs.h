// lhs preparation shared by the prefill (m > 16) matrix-core kernels.
//
// Every prefill kernel multiplies exact small-integer weight codes, held as fp16
// subnormals, with the lhs narrowed to fp16.  This pass produces, for each lhs row:
//   a16  [m][k] fp16   the row scaled by a power of two into [2^9, 2^10) at its largest
//                      magnitude and stored in the order the matrix-core operand wants,
//   a16_lo             (fp32 lhs only) the residual  x*s - fp16(x*s), same order,
//   asum [m][k/256][16] fp16  sums of the scaled row over each 32-wide sub-block,
//                      8 hi parts then 8 lo parts per 256 columns,
//   inv  [m] fp32      the inverse of the row scale.
#pragma once
#include "qmm_internal.h"

namespace qmm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

union HalfPack {
    uint32_t u[4];
    half8 h;
};
__device__ __forceinline__ half8 pack4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    HalfPack p;
    p.u[0] = a; p.u[1] = b; p.u[2] = c; p.u[3] = d;
    return p.h;
}
__device__ __forceinline__ uint32_t pack_half2(float x, float y) {
    return (uint32_t)f2h(x) | ((uint32_t)f2h(y) << 16);
}
__device__ __forceinline__ uint32_t pk_mul(uint32_t x, uint32_t s) {
    union { uint32_t u; half2v h; } a, b, r;
    a.u = x; b.u = s;
    r.h = a.h * b.h;
    return r.u;
}
// x*s + c on packed fp16 pairs, fused (single rounding)
__device__ __forceinline__ uint32_t pk_fma(uint32_t x, uint32_t s, uint32_t c) {
    union { uint32_t u; half2v h; } a, b, d, r;
    a.u = x; b.u = s; d.u = c;
    r.h = __builtin_elementwise_fma(a.h, b.h, d.h);
    return r.u;
}

// acc += g * P, element by element, written as the two-operand multiply-add so that acc stays in its own
// registers.  Left to the compiler, the three-operand form puts the result where P was; the 16-register
// tuples of the matrix-core accumulators then swap roles and fragment the register file, and the
// multiply-adds get sunk past the next group's matrix-core instructions.
// The compiler does not see which registers an asm statement reads, so it cannot place the wait states the
// hardware wants between a matrix-core instruction that writes P and a vector instruction that reads it (they
// are not interlocked): twelve idle states in front cover the eight passes of v_mfma_f32_32x32x16_f16.
__device__ __forceinline__ void rescale_add(float16v& acc, float g, const float16v& P) {
    asm volatile("s_nop 7\n\ts_nop 3");
#pragma unroll
    for (int r = 0; r < 16; r++) {
        float t = acc[r];
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(t) : "v"(g), "v"(P[r]));
        acc[r] = t;
    }
}

// Operand orders inside every 64-wide chunk of a row; position f*16 + g*8 + slot holds column
//   kLhsOrderQ4K : 32*(f/2) + 16*g + 8*(f%2) + (0,2,1,3,4,6,5,7)[slot]
//   kLhsOrderGPTQ: 16*f + 8*g + (0,4,1,5,2,6,3,7)[slot], odd columns pre-multiplied by 1/16
//                  (their codes are used in place in the high nibble position, 16*q)
//   kLhsOrderQ4K16: 8*(pos/8) + (0,2,1,3,4,6,5,7)[slot]   (natural order, the two middle pairs of every 8 swapped:
//                  the operand order of the 16x16x32 small-batch kernel)
//   kLhsOrderTile: 32*g + 8*f + (0,2,1,3,4,6,5,7)[slot]   (slice f pairs 8 columns of the low-nibble sub-block
//                  with the same 8 of the high-nibble one: what one lane of the tile kernels unpacks from 8 code bytes)
constexpr int kLhsOrderQ4K = 0, kLhsOrderGPTQ = 1, kLhsOrderQ4K16 = 2, kLhsOrderTile = 3;

// One lhs row by one workgroup of 256 threads.
// With next > 0 the rows of a16 / a16_lo are lda = k + 256 next halfs long and the sub-block sums go behind the row's k
// columns instead of into asum, as `next` further blocks of 256 operand positions: the 32 positions of super-block b are
// 8 hi, 8 lo, 8 hi, 8 lo parts of its sums (what multiplies a weight-side block of 8 hi, 8 hi, 8 lo, 8 lo table parts to the
// full hi/lo product), zeros beyond the last super-block.
// twin_rows > 0 (fp32 lhs): the residual plane is rows twin_rows .. 2 twin_rows - 1 of ONE lhs of twice the rows (a16_lo =
// a16 + twin_rows * lda), which one pass of a GEMM multiplies like any other rows; their sub-block sums are written as zeros
// (the min term belongs to the hi rows, which carry the full sums) and their row scales repeat those of the hi rows.
template <typename AT, int ORDER>
__device__ __forceinline__ void prep_lhs_row(int row, const AT* __restrict__ a, int k, _Float16* __restrict__ a16,
                                             _Float16* __restrict__ a16_lo, _Float16* __restrict__ asum, float* __restrict__ inv,
                                             int64_t lda = 0, int next = 0, int twin_rows = 0) {
    if (lda == 0) lda = k;
    __shared__ uint32_t wmax[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const AT* ar = a + (int64_t)row * k;
    // Rows of up to 8192 elements stay in registers between the maximum search and the conversion (one read of the row).
    constexpr int kHeld = 8;
    float held[kHeld][4];
    const bool hold = k <= kHeld * 1024;
    float mx = 0.0f;
    if (hold) {
#pragma unroll
        for (int it = 0; it < kHeld; it++) {
            const int i = tid * 4 + it * 1024;
            if (i < k) {
#pragma unroll
                for (int q = 0; q < 4; q++) held[it][q] = load_f32(ar, i + q);
                mx = fmaxf(mx, fmaxf(fmaxf(fabsf(held[it][0]), fabsf(held[it][1])), fmaxf(fabsf(held[it][2]), fabsf(held[it][3]))));
            }
        }
    } else {
        for (int i = tid * 4; i < k; i += 1024) {
            float x0 = load_f32(ar, i), x1 = load_f32(ar, i + 1), x2 = load_f32(ar, i + 2), x3 = load_f32(ar, i + 3);
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3))));
        }
    }
    const uint32_t mb = wave_max_nonneg_bits(mx);
    if (lane == 0) wmax[wave] = mb;
    __syncthreads();
    uint32_t mxb = max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]));
    int e = (int)((mxb >> 23) & 0xffu) - 127;
    if (e < -100 || e > 127) e = 9;  // zero, denormal or non-finite row: leave unscaled
    const float s = __uint_as_float((uint32_t)(127 + 9 - e) << 23);
    if (tid == 0) {
        inv[row] = __uint_as_float((uint32_t)(127 - 9 + e) << 23);
        if (twin_rows > 0) inv[twin_rows + row] = inv[row];
    }
    auto emit = [&](int i, float x0, float x1, float x2, float x3) __attribute__((always_inline)) {
        const float h0 = h2f(f2h(x0)), h1 = h2f(f2h(x1)), h2 = h2f(f2h(x2)), h3 = h2f(f2h(x3));
        const int kl = i & 63;
        if constexpr (ORDER == kLhsOrderQ4K) {
            const int hin = kl >> 5, gg = (kl >> 4) & 1, odd = (kl >> 3) & 1;
            const int pos = (2 * hin + odd) * 16 + gg * 8 + (kl & 4);
            const int64_t o = (int64_t)row * lda + (i & ~63) + pos;
            *(uint2*)(a16 + o) = make_uint2(pack_half2(h0, h2), pack_half2(h1, h3));
            if (a16_lo) *(uint2*)(a16_lo + o) = make_uint2(pack_half2(x0 - h0, x2 - h2), pack_half2(x1 - h1, x3 - h3));
        } else if constexpr (ORDER == kLhsOrderTile) {
            const int gg = kl >> 5, f = (kl >> 3) & 3;
            const int64_t o = (int64_t)row * lda + (i & ~63) + f * 16 + gg * 8 + (kl & 4);
            *(uint2*)(a16 + o) = make_uint2(pack_half2(h0, h2), pack_half2(h1, h3));
            if (a16_lo) *(uint2*)(a16_lo + o) = make_uint2(pack_half2(x0 - h0, x2 - h2), pack_half2(x1 - h1, x3 - h3));
        } else if constexpr (ORDER == kLhsOrderQ4K16) {
            const int64_t o = (int64_t)row * lda + i;
            *(uint2*)(a16 + o) = make_uint2(pack_half2(h0, h2), pack_half2(h1, h3));
            if (a16_lo) *(uint2*)(a16_lo + o) = make_uint2(pack_half2(x0 - h0, x2 - h2), pack_half2(x1 - h1, x3 - h3));
        } else {
            // columns kl..kl+3 of an 8-group go to slots 0,2,4,6 (kl % 8 == 0) or 1,3,5,7 (kl % 8 == 4)
            const int64_t o = (int64_t)row * lda + (i & ~63) + (kl & ~7) + ((kl >> 2) & 1);
            const float sixteenth = 0.0625f;
            a16[o] = (_Float16)h0;
            a16[o + 2] = (_Float16)(h1 * sixteenth);
            a16[o + 4] = (_Float16)h2;
            a16[o + 6] = (_Float16)(h3 * sixteenth);
            if (a16_lo) {
                a16_lo[o] = (_Float16)(x0 - h0);
                a16_lo[o + 2] = (_Float16)((x1 - h1) * sixteenth);
                a16_lo[o + 4] = (_Float16)(x2 - h2);
                a16_lo[o + 6] = (_Float16)((x3 - h3) * sixteenth);
            }
        }
        const float sum = sum8((x0 + x1) + (x2 + x3));  // 8 consecutive lanes = one 32-wide sub-block
        if ((lane & 7) == 0) {
            const int blk = i >> 8, j = (i >> 5) & 7;
            const float sh = h2f(f2h(sum));
            if (next > 0) {
                _Float16* as = a16 + (int64_t)row * lda + k + blk * 32;
                as[j] = as[16 + j] = (_Float16)sh;
                as[8 + j] = as[24 + j] = (_Float16)(sum - sh);
                if (twin_rows > 0) {
                    _Float16* az = a16 + (int64_t)(twin_rows + row) * lda + k + blk * 32;
                    az[j] = az[8 + j] = az[16 + j] = az[24 + j] = (_Float16)0.0f;
                }
            } else {
                _Float16* as = asum + ((int64_t)row * (k >> 8) + blk) * 16;
                as[j] = (_Float16)sh;
                as[8 + j] = (_Float16)(sum - sh);
                if (twin_rows > 0) {
                    _Float16* az = asum + ((int64_t)(twin_rows + row) * (k >> 8) + blk) * 16;
                    az[j] = az[8 + j] = (_Float16)0.0f;
                }
            }
        }
    };
    if (hold) {
#pragma unroll
        for (int it = 0; it < kHeld; it++) {
            const int i = tid * 4 + it * 1024;
            if (i < k) emit(i, held[it][0] * s, held[it][1] * s, held[it][2] * s, held[it][3] * s);
        }
    } else {
        for (int i = tid * 4; i < k; i += 1024) emit(i, load_f32(ar, i) * s, load_f32(ar, i + 1) * s, load_f32(ar, i + 2) * s, load_f32(ar, i + 3) * s);
    }
    for (int i = (k >> 8) * 32 + tid; i < next * 256; i += 256) {
        a16[(int64_t)row * lda + k + i] = (_Float16)0.0f;
        if (twin_rows > 0) a16[(int64_t)(twin_rows + row) * lda + k + i] = (_Float16)0.0f;
    }
}

template <typename AT, int ORDER>
__global__ __launch_bounds__(256) void prep_lhs_kernel(const AT* __restrict__ a, int k, _Float16* __restrict__ a16,
                                                       _Float16* __restrict__ a16_lo, _Float16* __restrict__ asum,
                                                       float* __restrict__ inv, int twin_rows) {
    prep_lhs_row<AT, ORDER>((int)blockIdx.x, a, k, a16, a16_lo, asum, inv, 0, 0, twin_rows);
}

struct LhsPlanes {
    _Float16* a16;
    _Float16* a16_lo;  // null unless the lhs is fp32
    _Float16* asum;
    float* inv;
    int64_t bytes;
};

// row_pad: the planes are sized for m rounded up to a multiple of it (kernels that read whole row tiles past the
// last row; the pass leaves those rows unwritten, and nothing computed from them is ever stored).
inline LhsPlanes lhs_planes(void* workspace, int lhs_dtype, int64_t m, int64_t k, int64_t row_pad = 1, int64_t lda = 0) {
    auto up = [](int64_t v) { return (v + 255) / 256 * 256; };
    m = (m + row_pad - 1) / row_pad * row_pad;
    const int64_t k_sums = k;
    if (lda > k) k = lda;  // rows with extension blocks (see prep_lhs_row)
    LhsPlanes p;
    char* ws = (char*)workspace;
    int64_t off = 0;
    p.a16 = (_Float16*)(ws + off);
    off += up(m * k * 2);
    p.a16_lo = nullptr;
    if (lhs_dtype == QMM_F32) {
        p.a16_lo = (_Float16*)(ws + off);
        off += up(m * k * 2);
    }
    p.asum = (_Float16*)(ws + off);
    off += up(m * (k_sums / 256) * 32);
    p.inv = (float*)(ws + off);
    off += up(m * 4);
    p.bytes = off;
    return p;
}

// twin: an fp32 lhs whose planes `p` were laid out as ONE plane of 2 m rows (see prep_lhs_row)
template <int ORDER>
inline hipError_t launch_prep_lhs(const void* lhs, int lhs_dtype, int64_t m, int64_t k, const LhsPlanes& p,
                                  hipStream_t s, bool twin = false) {
    if (lhs_dtype == QMM_F32)
        prep_lhs_kernel<float, ORDER><<<dim3((unsigned)m), dim3(256), 0, s>>>((const float*)lhs, (int)k, p.a16,
                                                                            twin ? p.a16 + m * k : p.a16_lo, p.asum, p.inv,
                                                                            twin ? (int)m : 0);
    else
        prep_lhs_kernel<uint16_t, ORDER><<<dim3((unsigned)m), dim3(256), 0, s>>>((const uint16_t*)lhs, (int)k, p.a16,
                                                                               nullptr, p.asum, p.inv, 0);
    return hipGetLastError();
}

}  // namespace qmm
