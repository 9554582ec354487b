// GPTQ decode kernel for m <= 4 lhs rows.
//
// qweight is [K/8, N] int32: a dword holds 8 consecutive k of one output column, and a row of
// dwords is contiguous in N.  A lane owns one output column; a wavefront's load of one k8 row is
// 256 contiguous bytes.  The eight wavefronts of a workgroup share 64 columns and split the groups
// of K between them; every wavefront issues all the loads of a group (group/8 dwords per lane)
// before it touches the first one, so the memory latency is paid once per group, not once per row.
// The activations a wavefront needs for a k8 row are the same for all its lanes: the wavefront loads
// a group's activations once (coalesced), parks them in LDS lines of its own and reads them back as
// broadcasts; their sum, for the zero point, falls out on the way:
// sum_k a_k s (q_k - z) = s (sum a_k q_k - z asum_g).  Nothing is shared between wavefronts before
// the final sum over the K shares.
#include <stdlib.h>

#include "qmm_internal.h"

namespace qmm {

namespace {

// Wavefronts per workgroup, which share 64 columns and split the groups of K: 16 (the loads of ONE group per wavefront are all
// that is in flight, so the wavefronts per compute unit decide the bandwidth: 14336 x 4096, g128, one lhs row: 8 -> 16
// wavefronts 11.25 -> 8.52 us; asking for the next group's weights before computing this one made it slower, 9.9 us).
constexpr int kWaves = 16;

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
    float* red = gsm;                                  // [kWaves][MT][64]
    float* mine = gsm + kWaves * MT * 64 + wave * MT * group;  // this wavefront's copy of a group's activations: [MT][group]

    const int col = (int)blockIdx.x * 64 + lane;
    const int ccol = min(col, n - 1);
    const int zshift = 4 * (ccol & 7);
    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;

    for (int g = wave; g < ngroups; g += kWaves) {
        const float sc = h2f(scales[(int64_t)g * n + ccol]);
        const float z = (float)(((qzeros[(int64_t)g * (n >> 3) + (ccol >> 3)] >> zshift) & 0xFu) + 1u);
        // The group's activations: loaded once by the wavefront (coalesced), parked in its own LDS lines and read
        // back as broadcasts (every lane needs the same value at the same time); their sum for the zero point on
        // the way.  LDS operations of one wavefront are performed in order, so no barrier is needed.
        float gsum[MT], part[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const AT* ar = a + (int64_t)min(mi, m - 1) * k + (int64_t)g * group;
            float s = 0.0f;
            for (int i = lane; i < group; i += 64) {
                const float v = act(ar, i);
                mine[mi * group + i] = v;
                s += v;
            }
            gsum[mi] = wave_sum(s);
            part[mi] = 0.0f;
        }
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
                    const float4* ap = (const float4*)(mine + mi * group + (r0 + j) * 8);  // the same address in every lane
                    const float4 a0 = ap[0], a1 = ap[1];
                    float t = part[mi];
                    t = fmaf(w0, a0.x, t);
                    t = fmaf(w1, a0.y, t);
                    t = fmaf(w2, a0.z, t);
                    t = fmaf(w3, a0.w, t);
                    t = fmaf(w4, a1.x, t);
                    t = fmaf(w5, a1.y, t);
                    t = fmaf(w6, a1.z, t);
                    part[mi] = fmaf(w7, a1.w, t);
                }
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi] = fmaf(sc, fmaf(-z, gsum[mi], part[mi]), acc[mi]);
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

// The same product for matrices of few columns (N / 64 workgroups would leave most compute units idle): a wavefront covers CW
// columns and KR = 64 / CW k8 rows per load instruction (lane l: column l % CW, row l / CW of every KR: CW * 4 contiguous bytes
// per row), so N / CW workgroups; consecutive column blocks run on one XCD, whose L2 then sees both halves of a 128-byte line.
// A lane takes NR = group / (8 KR) words per group; a wavefront has the loads of G groups in flight at a time.  The KR row lanes
// of a column meet in the final sum, in lane order.  Built with CW = 16 and G = 1: one-row calls on weights that no cache holds,
// 4096 x 4096 8.5 us with 64 columns per workgroup, 6.4 with 16, 9.8 with 32; 4096 x 14336 22.6 / 15.3 / 20.1; more groups in
// flight leave wavefronts without work and are slower (G = 4: 8.7 us on 4096 x 4096, 5.5 against 3.0 on 1024 x 1024).
template <int MT, int NR, int G, int CW, typename AT>
__global__ __launch_bounds__(64 * kWaves) void gemv_gptq_cols16_kernel(const uint32_t* __restrict__ qweight,
                                                                       const uint16_t* __restrict__ scales,
                                                                       const uint32_t* __restrict__ qzeros,
                                                                       const AT* __restrict__ a, float* __restrict__ out,
                                                                       int m, int n, int k, int64_t ldo, int per_xcd) {
    extern __shared__ __attribute__((aligned(16))) float gsm[];
    constexpr int KR = 64 / CW, GROUP = 8 * KR * NR;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cl = lane % CW, kr = lane / CW;
    const int ngroups = k / GROUP;
    float* red = gsm;                                               // [kWaves][MT][64]
    float* mine = gsm + kWaves * MT * 64 + wave * (G * MT * GROUP);  // this wavefront's copy of G groups' activations: [G][MT][GROUP]
    const int cb = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (cb * CW >= n) return;  // (the whole workgroup: the grid is rounded up to eight times per_xcd)
    const int col = cb * CW + cl;
    const int ccol = min(col, n - 1);
    const int zshift = 4 * (ccol & 7);
    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;

    for (int g0 = wave * G; g0 < ngroups; g0 += kWaves * G) {
        uint32_t x[G][NR];
        float sc[G], nz[G];
#pragma unroll
        for (int gi = 0; gi < G; gi++) {
            const int g = min(g0 + gi, ngroups - 1);
            const int64_t k8 = (int64_t)g * (KR * NR);
#pragma unroll
            for (int j = 0; j < NR; j++) x[gi][j] = (qweight + (k8 + KR * j + kr) * n)[ccol];
            // (a group past the end repeats the last one with scale 0; the zero-point term once per column, in row lane 0)
            sc[gi] = g0 + gi < ngroups ? h2f(scales[(int64_t)g * n + ccol]) : 0.0f;
            nz[gi] = kr == 0 ? -(float)(((qzeros[(int64_t)g * (n >> 3) + (ccol >> 3)] >> zshift) & 0xFu) + 1u) : 0.0f;
        }
        float gsum[G][MT];
#pragma unroll
        for (int gi = 0; gi < G; gi++) {
            const int g = min(g0 + gi, ngroups - 1);
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const AT* ar = a + (int64_t)min(mi, m - 1) * k + (int64_t)g * GROUP;
                float s = 0.0f;
                for (int i = lane; i < GROUP; i += 64) {
                    const float v = act(ar, i);
                    mine[(gi * MT + mi) * GROUP + i] = v;
                    s += v;
                }
                gsum[gi][mi] = wave_sum(s);
            }
        }
#pragma unroll
        for (int gi = 0; gi < G; gi++) {
            float part[MT];
#pragma unroll
            for (int mi = 0; mi < MT; mi++) part[mi] = 0.0f;
#pragma unroll
            for (int j = 0; j < NR; j++) {
                const uint32_t qe = x[gi][j] & 0x0F0F0F0Fu, qo = (x[gi][j] >> 4) & 0x0F0F0F0Fu;  // k 0,2,4,6 / k 1,3,5,7
                const float w0 = gub0(qe), w2 = gub1(qe), w4 = gub2(qe), w6 = gub3(qe);
                const float w1 = gub0(qo), w3 = gub1(qo), w5 = gub2(qo), w7 = gub3(qo);
#pragma unroll
                for (int mi = 0; mi < MT; mi++) {
                    const float4* ap = (const float4*)(mine + (gi * MT + mi) * GROUP + (KR * j + kr) * 8);  // KR addresses per wavefront
                    const float4 a0 = ap[0], a1 = ap[1];
                    float t = part[mi];
                    t = fmaf(w0, a0.x, t);
                    t = fmaf(w1, a0.y, t);
                    t = fmaf(w2, a0.z, t);
                    t = fmaf(w3, a0.w, t);
                    t = fmaf(w4, a1.x, t);
                    t = fmaf(w5, a1.y, t);
                    t = fmaf(w6, a1.z, t);
                    part[mi] = fmaf(w7, a1.w, t);
                }
            }
#pragma unroll
            for (int mi = 0; mi < MT; mi++) acc[mi] = fmaf(sc[gi], fmaf(nz[gi], gsum[gi][mi], part[mi]), acc[mi]);
        }
    }
#pragma unroll
    for (int mi = 0; mi < MT; mi++) red[(wave * MT + mi) * 64 + lane] = acc[mi];
    __syncthreads();
    if (tid < CW && cb * CW + tid < n) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            if (mi < m) {
                float v = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; w++)
#pragma unroll
                    for (int r = 0; r < KR; r++) v += red[(w * MT + mi) * 64 + CW * r + tid];
                out[(int64_t)mi * ldo + cb * CW + tid] = v;
            }
        }
    }
}

// Up to 4096 columns (a quarter of the compute units with 64 columns each).  More columns fill the part with 64 each, whose
// row loads are whole cache lines (weights from memory, one row: 5120 x 5120 10.0 us either way, 11008 x 4096 9.1 against
// 12.1 here, 14336 x 4096 9.7 against 13.9, 28672 x 8192 30 against 44).
bool gemv_gptq_cols16_wanted(int64_t n, int group) {
    return (group == 64 || group == 128 || group == 256) && n <= 4096 && n % 8 == 0 && !kernel_disabled("gptq_cols16");
}

hipError_t launch_gemv_gptq_cols(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                                 const uint32_t* qzeros, int m, int64_t n, int64_t k, int group, float* out,
                                 int64_t ldo, hipStream_t s, bool* handled) {
    *handled = false;
    if (m > 4 || group % 32) return hipSuccess;
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    // few columns: the kernel with 16 columns per workgroup
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    if (gemv_gptq_cols16_wanted(n, group)) {
        const size_t lds16 = ((size_t)kWaves * mt * group + (size_t)kWaves * mt * 64) * 4;
        const int per_xcd = (int)(((n + 15) / 16 + 7) / 8);
        dim3 grid16((unsigned)(8 * per_xcd)), block16(64 * kWaves);
#define QMM_GPTQ16(MT_, NR_, G_, CW_)                                                                                 \
    do {                                                                                                              \
        if (a_dtype == QMM_F32) {                                                                                     \
            if (lds16 > 64 * 1024) (void)allow_full_lds<gemv_gptq_cols16_kernel<MT_, NR_, G_, CW_, float>>();         \
            gemv_gptq_cols16_kernel<MT_, NR_, G_, CW_, float><<<grid16, block16, lds16, s>>>(qweight, scales, qzeros, (const float*)a, out, m, (int)n, (int)k, ldo, per_xcd); \
        } else {                                                                                                      \
            if (lds16 > 64 * 1024) (void)allow_full_lds<gemv_gptq_cols16_kernel<MT_, NR_, G_, CW_, uint16_t>>();      \
            gemv_gptq_cols16_kernel<MT_, NR_, G_, CW_, uint16_t><<<grid16, block16, lds16, s>>>(qweight, scales, qzeros, (const uint16_t*)a, out, m, (int)n, (int)k, ldo, per_xcd); \
        }                                                                                                             \
    } while (0)
#define QMM_GPTQ16_NR(NR_)                      \
    do {                                        \
        if (mt == 1) QMM_GPTQ16(1, NR_, 1, 16); \
        else if (mt == 2) QMM_GPTQ16(2, NR_, 1, 16); \
        else QMM_GPTQ16(4, NR_, 1, 16);         \
    } while (0)
        if (lds16 <= (size_t)kLdsPerCu) {
            if (group == 64) QMM_GPTQ16_NR(2);
            else if (group == 128) QMM_GPTQ16_NR(4);
            else QMM_GPTQ16_NR(8);
            *handled = true;
            return hipGetLastError();
        }
#undef QMM_GPTQ16_NR
#undef QMM_GPTQ16
    }
    const size_t lds = ((size_t)kWaves * mt * group + (size_t)kWaves * mt * 64) * 4;
    if (lds > (size_t)kLdsPerCu) return hipSuccess;
    dim3 grid((unsigned)((n + 63) / 64)), block(64 * kWaves);
#define QMM_GPTQ_GO(MT_, ROWS_)                                                                                       \
    do {                                                                                                              \
        if (a_dtype == QMM_F32) {                                                                                     \
            if (lds > 64 * 1024) (void)allow_full_lds<gemv_gptq_cols_kernel<MT_, ROWS_, float>>();                    \
            gemv_gptq_cols_kernel<MT_, ROWS_, float><<<grid, block, lds, s>>>(qweight, scales, qzeros, (const float*)a, \
                                                                             out, m, (int)n, (int)k, group, ldo);    \
        } else {                                                                                                      \
            if (lds > 64 * 1024) (void)allow_full_lds<gemv_gptq_cols_kernel<MT_, ROWS_, uint16_t>>();                 \
            gemv_gptq_cols_kernel<MT_, ROWS_, uint16_t><<<grid, block, lds, s>>>(                                     \
                qweight, scales, qzeros, (const uint16_t*)a, out, m, (int)n, (int)k, group, ldo);                     \
        }                                                                                                             \
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

// ---------------------------------------------------------------------------
// Act-order checkpoints (desc_act = True): g_idx[k] names the group of every k, in no particular order,
// so the scale and the zero point change from one k to the next.  Same lane-per-column shape as above;
// the 64 columns' (scale, -scale * zero) pairs of every group sit in LDS (TABLE; read from global memory
// when they do not fit), g_idx and the activations are read with wave-uniform addresses, and a weight
// is fma(scale, q, -scale * zero): both products and their difference are exact in fp32.
// Group indices outside [0, K / group) are clamped (the result is then meaningless, nothing is read
// out of bounds).
// ---------------------------------------------------------------------------
template <int MT, bool TABLE, typename AT>
__global__ __launch_bounds__(64 * kWaves) void gemv_gptq_act_order_kernel(
    const uint32_t* __restrict__ qweight, const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const int32_t* __restrict__ g_idx, const AT* __restrict__ a, float* __restrict__ out, int m, int n, int k, int group,
    int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) float gsm[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ngroups = k / group;
    float2* table = (float2*)gsm;                          // [ngroups][64]
    float* red = gsm + (TABLE ? 2 * 64 * ngroups : 0);     // [kWaves][MT][64]
    const int col = (int)blockIdx.x * 64 + lane;
    const int ccol = min(col, n - 1);
    const int zshift = 4 * (ccol & 7);
    auto pair_of = [&](int g) {
        const float sc = h2f(scales[(int64_t)g * n + ccol]);
        const float z = (float)(((qzeros[(int64_t)g * (n >> 3) + (ccol >> 3)] >> zshift) & 0xFu) + 1u);
        return make_float2(sc, -sc * z);
    };
    if constexpr (TABLE) {
        for (int g = wave; g < ngroups; g += kWaves) table[g * 64 + lane] = pair_of(g);
        __syncthreads();
    }
    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;
    // wavefront w walks the k8 rows [w * per, (w + 1) * per), four rows of loads at a time (K / 8 is a multiple of 4)
    constexpr int U = 4;
    const int rows = k >> 3;
    const int per = ((rows + kWaves - 1) / kWaves + U - 1) / U * U;
    const int r_end = min(rows, (wave + 1) * per);
    for (int r = wave * per; r < r_end; r += U) {
        uint32_t x[U];
#pragma unroll
        for (int j = 0; j < U; j++) x[j] = (qweight + (int64_t)(r + j) * n)[ccol];
#pragma unroll
        for (int j = 0; j < U; j++) {
            const int k0 = (r + j) * 8;
            const uint32_t qe = x[j] & 0x0F0F0F0Fu, qo = (x[j] >> 4) & 0x0F0F0F0Fu;  // k 0,2,4,6 / k 1,3,5,7
            const float q[8] = {gub0(qe), gub0(qo), gub1(qe), gub1(qo), gub2(qe), gub2(qo), gub3(qe), gub3(qo)};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int g = min(max(g_idx[k0 + i], 0), ngroups - 1);  // wave-uniform
                const float2 sz = TABLE ? table[g * 64 + lane] : pair_of(g);
                const float w = fmaf(sz.x, q[i], sz.y);
#pragma unroll
                for (int mi = 0; mi < MT; mi++)
                    acc[mi] = fmaf(w, act(a + (int64_t)(mi < m ? mi : 0) * k, k0 + i), acc[mi]);
            }
        }
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

// m <= 4 lhs rows; K % 32 == 0 and N % 8 == 0 are the caller's checks.
hipError_t launch_gemv_gptq_act_order(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                                      const uint32_t* qzeros, const int32_t* g_idx, int m, int64_t n, int64_t k, int group,
                                      float* out, int64_t ldo, hipStream_t s) {
    if (m < 1 || m > 4 || (k & 31)) return hipErrorInvalidValue;
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    const size_t red_bytes = (size_t)kWaves * mt * 64 * 4;
    const size_t table_bytes = (size_t)(k / group) * 64 * 8;
    const bool table = table_bytes + red_bytes <= 64 * 1024;
    const size_t lds = red_bytes + (table ? table_bytes : 0);
    dim3 grid((unsigned)((n + 63) / 64)), block(64 * kWaves);
#define QMM_GPTQ_AO(MT_, TB_)                                                                                          \
    do {                                                                                                              \
        if (a_dtype == QMM_F32)                                                                                       \
            gemv_gptq_act_order_kernel<MT_, TB_, float><<<grid, block, lds, s>>>(                                     \
                qweight, scales, qzeros, g_idx, (const float*)a, out, m, (int)n, (int)k, group, ldo);                 \
        else                                                                                                          \
            gemv_gptq_act_order_kernel<MT_, TB_, uint16_t><<<grid, block, lds, s>>>(                                  \
                qweight, scales, qzeros, g_idx, (const uint16_t*)a, out, m, (int)n, (int)k, group, ldo);              \
    } while (0)
#define QMM_GPTQ_AO_MT(TB_)                        \
    do {                                           \
        if (mt == 1) QMM_GPTQ_AO(1, TB_);          \
        else if (mt == 2) QMM_GPTQ_AO(2, TB_);     \
        else QMM_GPTQ_AO(4, TB_);                  \
    } while (0)
    if (table) QMM_GPTQ_AO_MT(true);
    else QMM_GPTQ_AO_MT(false);
#undef QMM_GPTQ_AO_MT
#undef QMM_GPTQ_AO
    return hipGetLastError();
}

}  // namespace qmm
