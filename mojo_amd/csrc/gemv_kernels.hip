// Decode-shape kernels: out[m, n] = lhs[m, :] . dequant(rhs[n, :]) for m <= 16.
//
// The packed weights are streamed once; every wavefront owns one weight row,
// keeps one fp32 accumulator per lhs row and finishes with a cross-lane sum.
// No matrix-core instructions are used here.
#include <stdlib.h>

#include "qmm_internal.h"

namespace qmm {


template <typename AT>
__device__ __forceinline__ float4 load_a4(const AT* __restrict__ a, int64_t i) {
    if constexpr (sizeof(AT) == 4) {
        return *(const float4*)(a + i);
    } else {
        uint2 v = *(const uint2*)(a + i);
        return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                           __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
    }
}
template <typename AT>
__device__ __forceinline__ float load_a1(const AT* __restrict__ a, int64_t i) {
    if constexpr (sizeof(AT) == 4) return a[i];
    else return bf2f(a[i]);
}

__device__ __forceinline__ float ub0(uint32_t v) { return (float)(v & 0xffu); }
__device__ __forceinline__ float ub1(uint32_t v) { return (float)((v >> 8) & 0xffu); }
__device__ __forceinline__ float ub2(uint32_t v) { return (float)((v >> 16) & 0xffu); }
__device__ __forceinline__ float ub3(uint32_t v) { return (float)(v >> 24); }

// ---------------------------------------------------------------------------
// Q4_K: eight lanes per 144-byte super-block.  Lane u of a group loads the
// 16-byte header and the 16-byte code unit u (bytes 16+16u..): its low nibbles
// are 16 weights of sub-block 2c, its high nibbles 16 weights of sub-block
// 2c+1 (c = u/2).  With w = (d*sc)*q - dmin*m the row dot factors into
//   sum_sub (d*sc) * sum(q*a) - (dmin*m) * sum(a).
// ---------------------------------------------------------------------------
template <int MT, typename AT>
__global__ __launch_bounds__(256) void gemv_q4_k_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                        float* __restrict__ out, int m, int n, int k,
                                                        int64_t ldo) {
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int row = blockIdx.x * 4 + wave;
    if (row >= n) return;
    int nblk = k >> 8;
    const uint8_t* wrow = w + (int64_t)row * nblk * Q4_K_BPB;
    int sb = lane >> 3, u = lane & 7, c = u >> 1, h = u & 1;
    float acc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) acc[i] = 0.0f;
    for (int b = sb; b < nblk; b += 8) {
        const uint4* blk = (const uint4*)(wrow + (int64_t)b * Q4_K_BPB);
        uint4 hdr = blk[0];
        uint4 qs = blk[1 + u];
        float d = h2f((uint16_t)(hdr.x & 0xffffu)), dmin = h2f((uint16_t)(hdr.x >> 16));
        uint32_t s[3] = {hdr.y, hdr.z, hdr.w};
        uint32_t sc1, mn1, sc2, mn2;
        q4k_scale_min(2 * c, s, sc1, mn1);
        q4k_scale_min(2 * c + 1, s, sc2, mn2);
        float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
        float d2 = d * (float)sc2, m2 = dmin * (float)mn2;
        uint32_t qw[4] = {qs.x, qs.y, qs.z, qs.w};
        int kbase = b * 256 + 64 * c + 16 * h;
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            if (mi < m) {
                const AT* ar = a + (int64_t)mi * k + kbase;
                float slo = 0.0f, shi = 0.0f, alo = 0.0f, ahi = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float4 x = load_a4(ar, 4 * i);
                    float4 y = load_a4(ar, 32 + 4 * i);
                    uint32_t lo = qw[i] & 0x0F0F0F0Fu, hi = (qw[i] >> 4) & 0x0F0F0F0Fu;
                    slo = fmaf(x.x, ub0(lo), slo);
                    slo = fmaf(x.y, ub1(lo), slo);
                    slo = fmaf(x.z, ub2(lo), slo);
                    slo = fmaf(x.w, ub3(lo), slo);
                    shi = fmaf(y.x, ub0(hi), shi);
                    shi = fmaf(y.y, ub1(hi), shi);
                    shi = fmaf(y.z, ub2(hi), shi);
                    shi = fmaf(y.w, ub3(hi), shi);
                    alo += (x.x + x.y) + (x.z + x.w);
                    ahi += (y.x + y.y) + (y.z + y.w);
                }
                float t = fmaf(d1, slo, acc[mi]);
                t = fmaf(-m1, alo, t);
                t = fmaf(d2, shi, t);
                acc[mi] = fmaf(-m2, ahi, t);
            }
        }
    }
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        if (mi < m) {
            float v = wave_sum(acc[mi]);
            if (lane == 0) out[(int64_t)mi * ldo + row] = v;
        }
    }
}

// ---------------------------------------------------------------------------
// Q6_K: 32 lanes per 210-byte super-block, two super-blocks per wavefront
// step.  Lane l handles, in each 128-weight half, ql[l], ql[l+32] and qh[l]:
// four weights at offsets l, l+32, l+64, l+96.
// ---------------------------------------------------------------------------
template <int MT, typename AT>
__global__ __launch_bounds__(256) void gemv_q6_k_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                        float* __restrict__ out, int m, int n, int k,
                                                        int64_t ldo) {
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int row = blockIdx.x * 4 + wave;
    if (row >= n) return;
    int nblk = k >> 8;
    const uint8_t* wrow = w + (int64_t)row * nblk * Q6_K_BPB;
    int half_wave = lane >> 5, l = lane & 31;
    float acc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) acc[i] = 0.0f;
    for (int b = half_wave; b < nblk; b += 2) {
        const uint8_t* blk = wrow + (int64_t)b * Q6_K_BPB;
        float d = h2f((uint16_t)(blk[208] | (blk[209] << 8)));
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t l0 = blk[64 * h + l], l1 = blk[64 * h + 32 + l], hh = blk[128 + 32 * h + l];
            const int8_t* sc = (const int8_t*)(blk + 192 + 8 * h + (l >> 4));
            int q1 = (int)((l0 & 15u) | ((hh & 3u) << 4)) - 32;
            int q2 = (int)((l1 & 15u) | (((hh >> 2) & 3u) << 4)) - 32;
            int q3 = (int)((l0 >> 4) | (((hh >> 4) & 3u) << 4)) - 32;
            int q4 = (int)((l1 >> 4) | (((hh >> 6) & 3u) << 4)) - 32;
            float w1 = d * (float)sc[0] * (float)q1;
            float w2 = d * (float)sc[2] * (float)q2;
            float w3 = d * (float)sc[4] * (float)q3;
            float w4 = d * (float)sc[6] * (float)q4;
            int kbase = b * 256 + 128 * h + l;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                if (mi < m) {
                    const AT* ar = a + (int64_t)mi * k + kbase;
                    float t = fmaf(w1, load_a1(ar, 0), acc[mi]);
                    t = fmaf(w2, load_a1(ar, 32), t);
                    t = fmaf(w3, load_a1(ar, 64), t);
                    acc[mi] = fmaf(w4, load_a1(ar, 96), t);
                }
            }
        }
    }
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        if (mi < m) {
            float v = wave_sum(acc[mi]);
            if (lane == 0) out[(int64_t)mi * ldo + row] = v;
        }
    }
}

// ---------------------------------------------------------------------------
// Q4_0 x Q8_0: one lane per 18-byte block.  Codes 0..15 are dotted against the
// int8 activation codes with v_dot4 and the -8 offset is taken out through the
// precomputed activation code sum: sum (q-8)*a = sum q*a - 8*sum a.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int q4_0_block_isum(const uint8_t* __restrict__ wb, const int8_t* __restrict__ ab,
                                               int asum) {
    const uint16_t* w16 = (const uint16_t*)wb;  // blocks are 2-byte aligned
    const int* a32 = (const int*)ab;            // activation codes are 32-byte aligned
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t x = (uint32_t)w16[1 + 2 * i] | ((uint32_t)w16[2 + 2 * i] << 16);
        int lo = (int)(x & 0x0F0F0F0Fu), hi = (int)((x >> 4) & 0x0F0F0F0Fu);
        s = __builtin_amdgcn_sdot4(lo, a32[i], s, false);
        s = __builtin_amdgcn_sdot4(hi, a32[4 + i], s, false);
    }
    return s - 8 * asum;
}

template <int MT>
__global__ __launch_bounds__(256) void gemv_q4_0_kernel(const uint8_t* __restrict__ w,
                                                        const int8_t* __restrict__ a_codes,
                                                        const float* __restrict__ a_scale,
                                                        const int32_t* __restrict__ a_sum,
                                                        float* __restrict__ out, int m, int n, int k,
                                                        int64_t ldo) {
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int row = blockIdx.x * 4 + wave;
    if (row >= n) return;
    int nblk = k >> 5;
    const uint8_t* wrow = w + (int64_t)row * nblk * Q4_0_BPB;
    float acc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) acc[i] = 0.0f;
    for (int b = lane; b < nblk; b += 64) {
        const uint8_t* wb = wrow + (int64_t)b * Q4_0_BPB;
        float dw = h2f(*(const uint16_t*)wb);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            if (mi < m) {
                int64_t ab = (int64_t)mi * nblk + b;
                int isum = q4_0_block_isum(wb, a_codes + ab * 32, a_sum[ab]);
                acc[mi] = fmaf((float)isum, dw * a_scale[ab], acc[mi]);
            }
        }
    }
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        if (mi < m) {
            float v = wave_sum(acc[mi]);
            if (lane == 0) out[(int64_t)mi * ldo + row] = v;
        }
    }
}

// Raw int32 block sums against GGUF Q8_0 lhs blocks: out[m, n, k/32].
__global__ __launch_bounds__(256) void block_dots_q4_0_kernel(const uint8_t* __restrict__ a_q8,
                                                              const uint8_t* __restrict__ w, int64_t m,
                                                              int64_t n, int64_t nblk, int32_t* __restrict__ out) {
    int64_t total = m * n * nblk;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
        int64_t b = e % nblk, j = (e / nblk) % n, i = e / (nblk * n);
        const uint8_t* wb = w + (j * nblk + b) * Q4_0_BPB;
        const int8_t* ab = (const int8_t*)(a_q8 + (i * nblk + b) * Q8_0_BPB + 2);
        int s = 0;
        for (int t = 0; t < 16; t++) {
            int byte = wb[2 + t];
            s += ((byte & 15) - 8) * (int)ab[t] + ((byte >> 4) - 8) * (int)ab[t + 16];
        }
        out[e] = s;
    }
}

// ---------------------------------------------------------------------------
// GPTQ 4-bit: qweight is [k/8, n], so a lane owns one output column and walks
// down k; four wavefronts split k and combine through LDS.
// ---------------------------------------------------------------------------
template <int MT, typename AT>
__global__ __launch_bounds__(256) void gemv_gptq_kernel(const uint32_t* __restrict__ qweight,
                                                        const uint16_t* __restrict__ scales,
                                                        const uint32_t* __restrict__ qzeros,
                                                        const AT* __restrict__ a, float* __restrict__ out, int m,
                                                        int n, int k, int group, int64_t ldo) {
    __shared__ float red[4][MT][64];
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int col = blockIdx.x * 64 + lane;
    bool live = col < n;
    int ccol = live ? col : n - 1;
    int ngroups = k / group;
    float acc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) acc[i] = 0.0f;
    for (int g = wave; g < ngroups; g += 4) {
        float sc = h2f(scales[(int64_t)g * n + ccol]);
        int z = (int)((qzeros[(int64_t)g * (n >> 3) + (ccol >> 3)] >> (4 * (ccol & 7))) & 0xFu) + 1;
        float part[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) part[i] = 0.0f;
        for (int k8 = g * (group >> 3); k8 < (g + 1) * (group >> 3); k8++) {
            uint32_t x = qweight[(int64_t)k8 * n + ccol];
            float q[8];
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = (float)((int)((x >> (4 * i)) & 0xFu) - z);
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                if (mi < m) {
                    const AT* ar = a + (int64_t)mi * k + k8 * 8;
                    float4 x0 = load_a4(ar, 0), x1 = load_a4(ar, 4);
                    float t = part[mi];
                    t = fmaf(q[0], x0.x, t);
                    t = fmaf(q[1], x0.y, t);
                    t = fmaf(q[2], x0.z, t);
                    t = fmaf(q[3], x0.w, t);
                    t = fmaf(q[4], x1.x, t);
                    t = fmaf(q[5], x1.y, t);
                    t = fmaf(q[6], x1.z, t);
                    part[mi] = fmaf(q[7], x1.w, t);
                }
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi] = fmaf(sc, part[mi], acc[mi]);
    }
#pragma unroll
    for (int mi = 0; mi < MT; mi++) red[wave][mi][lane] = acc[mi];
    __syncthreads();
    if (wave == 0 && live) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            if (mi < m)
                out[(int64_t)mi * ldo + col] = (red[0][mi][lane] + red[1][mi][lane]) + (red[2][mi][lane] + red[3][mi][lane]);
        }
    }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
#define QMM_MT_SWITCH(m, CALL)   \
    if (m <= 1) { CALL(1); }     \
    else if (m <= 2) { CALL(2); } \
    else if (m <= 4) { CALL(4); } \
    else if (m <= 8) { CALL(8); } \
    else { CALL(16); }

// Q4_K through the decode kernels: the streaming kernel for one or two lhs rows, three and four rows as two
// passes over the weights, more rows through the generic kernel.  (qmm_matmul sends 2..16 rows to the
// small-batch matrix-core kernel instead; this is what is left when that is switched off.)
hipError_t launch_gemv_q4_k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                            float* out, int64_t ldo, hipStream_t s) {
    const bool rows_ok = !kernel_disabled("q4k_rows_v2");  // (the streaming / row kernels of gemv_q4k_valu.hip)
    if (m <= 2) {
        bool handled = false;
        hipError_t e = launch_gemv_q4_k_lanes(a, a_dtype, w, m, n, k, out, ldo, s, &handled);  // (declines when disabled)
        if (e != hipSuccess || handled) return e;
        if (rows_ok) return launch_gemv_q4_k_rows(a, a_dtype, w, m, n, k, out, ldo, s);
    } else if (m <= 4 && rows_ok) {
        const int64_t esz = a_dtype == QMM_F32 ? 4 : 2;
        hipError_t e = launch_gemv_q4_k_rows(a, a_dtype, w, 2, n, k, out, ldo, s);
        if (e != hipSuccess) return e;
        return launch_gemv_q4_k_rows((const char*)a + 2 * k * esz, a_dtype, w, m - 2, n, k, out + 2 * ldo, ldo, s);
    }
    dim3 grid((unsigned)((n + 3) / 4)), block(256);
#define CALL(MT)                                                                                          \
    if (a_dtype == QMM_F32)                                                                               \
        gemv_q4_k_kernel<MT, float><<<grid, block, 0, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo); \
    else                                                                                                  \
        gemv_q4_k_kernel<MT, uint16_t><<<grid, block, 0, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo)
    QMM_MT_SWITCH(m, CALL)
#undef CALL
    return hipGetLastError();
}

hipError_t launch_gemv_q6_k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                            float* out, int64_t ldo, hipStream_t s) {
    if (!kernel_disabled("q6k_staged")) {
        bool handled = false;
        hipError_t e = launch_gemv_q6_k_rows(a, a_dtype, w, m, n, k, out, ldo, s, &handled);
        if (e != hipSuccess || handled) return e;
    }
    dim3 grid((unsigned)((n + 3) / 4)), block(256);
#define CALL(MT)                                                                                          \
    if (a_dtype == QMM_F32)                                                                               \
        gemv_q6_k_kernel<MT, float><<<grid, block, 0, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo); \
    else                                                                                                  \
        gemv_q6_k_kernel<MT, uint16_t><<<grid, block, 0, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo)
    QMM_MT_SWITCH(m, CALL)
#undef CALL
    return hipGetLastError();
}

hipError_t launch_gemv_q4_0(const int8_t* a_codes, const float* a_scale, const int32_t* a_sum,
                            const uint8_t* w, int m, int64_t n, int64_t k, float* out, int64_t ldo,
                            hipStream_t s) {
    dim3 grid((unsigned)((n + 3) / 4)), block(256);
#define CALL(MT) gemv_q4_0_kernel<MT><<<grid, block, 0, s>>>(w, a_codes, a_scale, a_sum, out, m, (int)n, (int)k, ldo)
    QMM_MT_SWITCH(m, CALL)
#undef CALL
    return hipGetLastError();
}

hipError_t launch_gemv_gptq(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                            const uint32_t* qzeros, int m, int64_t n, int64_t k, int group, float* out,
                            int64_t ldo, hipStream_t s) {
    if (!kernel_disabled("gptq_cols")) {
        // up to four lhs rows per pass of the column kernel; more rows take more passes over the weights
        const int64_t esz = a_dtype == QMM_F32 ? 4 : 2;
        bool handled = true;
        for (int m0 = 0; m0 < m && handled; m0 += 4) {
            hipError_t e = launch_gemv_gptq_cols((const char*)a + (int64_t)m0 * k * esz, a_dtype, qweight, scales, qzeros,
                                                 min(4, m - m0), n, k, group, out + (int64_t)m0 * ldo, ldo, s, &handled);
            if (e != hipSuccess) return e;
        }
        if (handled) return hipSuccess;
    }
    dim3 grid((unsigned)((n + 63) / 64)), block(256);
#define CALL(MT)                                                                                       \
    if (a_dtype == QMM_F32)                                                                            \
        gemv_gptq_kernel<MT, float><<<grid, block, 0, s>>>(qweight, scales, qzeros, (const float*)a, out, m, \
                                                           (int)n, (int)k, group, ldo);                \
    else                                                                                               \
        gemv_gptq_kernel<MT, uint16_t><<<grid, block, 0, s>>>(qweight, scales, qzeros, (const uint16_t*)a, \
                                                              out, m, (int)n, (int)k, group, ldo)
    QMM_MT_SWITCH(m, CALL)
#undef CALL
    return hipGetLastError();
}

hipError_t launch_block_dots_q4_0(const uint8_t* a_q8, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                                  int32_t* out, hipStream_t s) {
    int64_t total = m * n * (k / 32);
    int64_t g = (total + 255) / 256;
    if (g > 65536) g = 65536;
    if (g < 1) g = 1;
    block_dots_q4_0_kernel<<<dim3((unsigned)g), dim3(256), 0, s>>>(a_q8, w, m, n, k / 32, out);
    return hipGetLastError();
}

}  // namespace qmm
