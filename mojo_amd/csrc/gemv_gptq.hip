// GPTQ decode kernel for m <= 4 lhs rows.
//
// qweight is [K/8, N] int32: a dword holds 8 consecutive k of one output column, and a row of
// dwords is contiguous in N.  A lane owns one output column; a wavefront's load of one k8 row is
// 256 contiguous bytes.  The eight wavefronts of a workgroup share 64 columns and split the groups
// of K between them; every wavefront issues all the loads of a group (group/8 dwords per lane)
// before it touches the first one, so the memory latency is paid once per group, not once per row.
// The activations a wavefront needs for a k8 row are the same for all its lanes; they are read with
// wave-uniform addresses.  Per-group activation sums (for the zero point) are computed once per
// workgroup into LDS:  sum_k a_k s (q_k - z) = s (sum a_k q_k - z asum_g).
#include <stdlib.h>

#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int kWaves = 8;

__device__ __forceinline__ float gub0(uint32_t x) { float r; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float gub1(uint32_t x) { float r; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float gub2(uint32_t x) { float r; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float gub3(uint32_t x) { float r; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(x)); return r; }

template <typename AT>
__device__ __forceinline__ float act(const AT* __restrict__ a, int64_t i) {
    return load_f32(a, i);
}

}  // namespace

// ROWS = k8 rows per group handled per inner step (group / 8 must be a multiple of it).
template <int MT, int ROWS, typename AT>
__global__ __launch_bounds__(64 * kWaves) void gemv_gptq_cols_kernel(const uint32_t* __restrict__ qweight,
                                                                     const uint16_t* __restrict__ scales,
                                                                     const uint32_t* __restrict__ qzeros,
                                                                     const AT* __restrict__ a, float* __restrict__ out,
                                                                     int m, int n, int k, int group, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) float gsm[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ngroups = k / group, rows_per_group = group >> 3;
    float* asum = gsm;                       // [MT][ngroups]
    float* red = gsm + MT * ngroups;         // [kWaves][MT][64]

    // per-group activation sums: one wavefront per (lhs row, group) item, lanes stride the group
    for (int gi = wave; gi < MT * ngroups; gi += kWaves) {
        const int mi = gi / ngroups, g = gi - mi * ngroups;
        float s = 0.0f;
        if (mi < m) {
            const AT* ar = a + (int64_t)mi * k + (int64_t)g * group;
            for (int i = lane; i < group; i += 64) s += act(ar, i);
        }
        s = wave_sum(s);
        if (lane == 0) asum[gi] = s;
    }
    __syncthreads();

    const int col = (int)blockIdx.x * 64 + lane;
    const int ccol = min(col, n - 1);
    const int zshift = 4 * (ccol & 7);
    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;

    for (int g = wave; g < ngroups; g += kWaves) {
        const float sc = h2f(scales[(int64_t)g * n + ccol]);
        const float z = (float)(((qzeros[(int64_t)g * (n >> 3) + (ccol >> 3)] >> zshift) & 0xFu) + 1u);
        float part[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) part[mi] = 0.0f;
        for (int r0 = 0; r0 < rows_per_group; r0 += ROWS) {
            const int64_t k8 = (int64_t)g * rows_per_group + r0;
            uint32_t x[ROWS];
#pragma unroll
            for (int j = 0; j < ROWS; j++) x[j] = (qweight + (k8 + j) * n)[ccol];
#pragma unroll
            for (int j = 0; j < ROWS; j++) {
                const uint32_t qe = x[j] & 0x0F0F0F0Fu, qo = (x[j] >> 4) & 0x0F0F0F0Fu;  // k 0,2,4,6 / k 1,3,5,7
                const float w0 = gub0(qe), w2 = gub1(qe), w4 = gub2(qe), w6 = gub3(qe);
                const float w1 = gub0(qo), w3 = gub1(qo), w5 = gub2(qo), w7 = gub3(qo);
#pragma unroll
                for (int mi = 0; mi < MT; mi++) {
                    const AT* ar = a + (int64_t)(mi < m ? mi : 0) * k + (k8 + j) * 8;  // wave-uniform address
                    float t = part[mi];
                    t = fmaf(w0, act(ar, 0), t);
                    t = fmaf(w1, act(ar, 1), t);
                    t = fmaf(w2, act(ar, 2), t);
                    t = fmaf(w3, act(ar, 3), t);
                    t = fmaf(w4, act(ar, 4), t);
                    t = fmaf(w5, act(ar, 5), t);
                    t = fmaf(w6, act(ar, 6), t);
                    part[mi] = fmaf(w7, act(ar, 7), t);
                }
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi] = fmaf(sc, fmaf(-z, asum[mi * ngroups + g], part[mi]), acc[mi]);
    }
#pragma unroll
    for (int mi = 0; mi < MT; mi++) red[(wave * MT + mi) * 64 + lane] = acc[mi];
    __syncthreads();
    if (wave == 0 && col < n) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            if (mi < m) {
                float v = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; w++) v += red[(w * MT + mi) * 64 + lane];
                out[(int64_t)mi * ldo + col] = v;
            }
        }
    }
}

hipError_t launch_gemv_gptq_cols(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                                 const uint32_t* qzeros, int m, int64_t n, int64_t k, int group, float* out,
                                 int64_t ldo, hipStream_t s, bool* handled) {
    *handled = false;
    if (m > 4 || group % 32) return hipSuccess;
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    const size_t lds = ((size_t)mt * (k / group) + (size_t)kWaves * mt * 64) * 4;
    if (lds > 64 * 1024) return hipSuccess;
    dim3 grid((unsigned)((n + 63) / 64)), block(64 * kWaves);
#define QMM_GPTQ_GO(MT_, ROWS_)                                                                                       \
    do {                                                                                                              \
        if (a_dtype == QMM_F32)                                                                                       \
            gemv_gptq_cols_kernel<MT_, ROWS_, float><<<grid, block, lds, s>>>(qweight, scales, qzeros, (const float*)a, \
                                                                             out, m, (int)n, (int)k, group, ldo);    \
        else                                                                                                          \
            gemv_gptq_cols_kernel<MT_, ROWS_, uint16_t><<<grid, block, lds, s>>>(                                     \
                qweight, scales, qzeros, (const uint16_t*)a, out, m, (int)n, (int)k, group, ldo);                     \
    } while (0)
#define QMM_GPTQ_MT(ROWS_)                  \
    do {                                    \
        if (mt == 1) QMM_GPTQ_GO(1, ROWS_); \
        else if (mt == 2) QMM_GPTQ_GO(2, ROWS_); \
        else QMM_GPTQ_GO(4, ROWS_);         \
    } while (0)
    if (group % 128 == 0) QMM_GPTQ_MT(16);
    else QMM_GPTQ_MT(4);
#undef QMM_GPTQ_MT
#undef QMM_GPTQ_GO
    *handled = true;
    return hipGetLastError();
}

}  // namespace qmm
