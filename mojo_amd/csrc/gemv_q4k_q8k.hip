// Q4_K decode with Q8_K-quantised activations (the integer dot of the ggml-lineage CPU kernels), up to
// four lhs rows.  Selected by QMM_FLAG_ACT_Q8K; the default Q4_K path keeps the lhs in floating point.
//
// Per (lhs row, weight row, super-block):
//   isum = sum_sub sc_sub * sum_32 q4 * q8,   msum = sum_sub mn_sub * (sum of the sub-block's 32 q8)
//   out += (d8 * d) * isum - (d8 * dmin) * msum
// with q8 the Q8_K codes of the lhs block (d8 = -max / 127 for the element of largest magnitude, codes
// rounded to nearest even).  The integer sums are exact, so they equal the CPU path's.
//
// Schedule: that of gemv_q4k_lanes.hip.  Every lane owns one 64-column chunk (sub-blocks 2c, 2c + 1)
// of a row part: the 64 Q8_K codes of that chunk, their two sums and d8 stay in registers for every lhs
// row (16 dwords per row), weight row parts go global -> LDS directly into a 3-slot ring, and per row a
// lane spends two v_dot4_i32_i8 per code dword and lhs row.  The workgroup quantises the lhs itself at
// the start (32 threads per 256-wide block, codes to LDS), after the first weight rows have been issued.
#include <stdlib.h>

#include <algorithm>

#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int kWaves = 8;     // wavefronts per workgroup
constexpr int kMaxRows = 64;  // rows a wavefront may own (LDS result slots)

// round to nearest, ties to even, through the fp32 adder
__device__ __forceinline__ int nearest_int(float f) {
    const float v = __fadd_rn(f, 12582912.f);
    return (__float_as_int(v) & 0x007fffff) - 0x00400000;
}

}  // namespace

// Quantise `nblocks` 256-wide blocks of x to Q8_K codes.  Block-local work of 32 consecutive threads
// (8 values each): returns this thread's 8 codes packed in two dwords, the block's d8 and the thread's
// code sum.  The first element of largest magnitude decides the sign of the scale, as in the CPU quantiser.
template <typename AT>
__device__ __forceinline__ void q8k_quantise8(const AT* __restrict__ xp, int idx_in_block, uint32_t& c0, uint32_t& c1,
                                              float& d8, int& sum8) {
    float v[8];
    if constexpr (sizeof(AT) == 4) {
        const float4 a = *(const float4*)xp, b = *(const float4*)(xp + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        const uint4 r = *(const uint4*)xp;
        v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
        v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
        v[4] = __uint_as_float(r.z << 16); v[5] = __uint_as_float(r.z & 0xffff0000u);
        v[6] = __uint_as_float(r.w << 16); v[7] = __uint_as_float(r.w & 0xffff0000u);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v[i]));
    // over the 32 threads of the block (two 16-lane rows of a wavefront)
    amax = fmaxf(amax, dpp_move<0xB1>(amax));
    amax = fmaxf(amax, dpp_move<0x4E>(amax));
    amax = fmaxf(amax, dpp_move<0x141>(amax));
    amax = fmaxf(amax, dpp_move<0x140>(amax));
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    // first element of that magnitude: smallest (index << 1 | sign bit)
    int key = 0x7fffffff;
#pragma unroll
    for (int i = 7; i >= 0; i--)
        if (fabsf(v[i]) == amax) key = ((idx_in_block + i) << 1) | (int)(__float_as_uint(v[i]) >> 31);
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0xB1, 0xf, 0xf, false));
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0x4E, 0xf, 0xf, false));
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0x141, 0xf, 0xf, false));
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0x140, 0xf, 0xf, false));
    key = min(key, __shfl_xor(key, 16, 64));
    const float mx = (key & 1) ? -amax : amax;
    int q[8];
    if (amax == 0.0f) {
        d8 = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = 0;
    } else {
        const float iscale = -127.f / mx;
        d8 = 1.0f / iscale;
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = min(127, nearest_int(__fmul_rn(iscale, v[i])));
    }
    sum8 = ((q[0] + q[1]) + (q[2] + q[3])) + ((q[4] + q[5]) + (q[6] + q[7]));
    c0 = (uint32_t)(q[0] & 0xff) | ((uint32_t)(q[1] & 0xff) << 8) | ((uint32_t)(q[2] & 0xff) << 16) | ((uint32_t)q[3] << 24);
    c1 = (uint32_t)(q[4] & 0xff) | ((uint32_t)(q[5] & 0xff) << 8) | ((uint32_t)(q[6] & 0xff) << 16) | ((uint32_t)q[7] << 24);
}

// Stand-alone quantiser: x [rows, k] -> Q8_K blocks (float d, 256 int8, 16 int16 sums of 16).  One wavefront
// half (32 threads) per block.
template <typename AT>
__global__ __launch_bounds__(256) void quantize_q8_k_kernel(const AT* __restrict__ x, int64_t nblocks, uint8_t* __restrict__ out) {
    const int64_t blk = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    const int l = threadIdx.x & 31;
    const int64_t bc = min(blk, nblocks - 1);  // whole 32-thread groups stay together for the cross-lane steps
    uint32_t c0, c1;
    float d8;
    int s8;
    q8k_quantise8(x + bc * 256 + 8 * l, 8 * l, c0, c1, d8, s8);
    const int s16 = s8 + __builtin_amdgcn_update_dpp(0, s8, 0xB1, 0xf, 0xf, false);  // 16 codes: two threads
    if (blk >= nblocks) return;
    uint8_t* ob = out + blk * 292;
    if (l == 0) *(float*)ob = d8;
    *(uint2*)(ob + 4 + 8 * l) = make_uint2(c0, c1);
    if ((l & 1) == 0) *(int16_t*)(ob + 260 + 2 * (l >> 1)) = (int16_t)s16;
}

// x [rows, k] -> d8 * code of its Q8_K quantisation as fp32 [rows, k]: the activations that the integer treatment multiplies,
// for the kernels that take a floating-point lhs.  Same quantiser, same 32 threads per block.
template <typename AT>
__global__ __launch_bounds__(256) void q8k_round_trip_kernel(const AT* __restrict__ x, int64_t nblocks, float* __restrict__ y) {
    const int64_t blk = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    const int l = threadIdx.x & 31;
    const int64_t bc = min(blk, nblocks - 1);
    uint32_t c0, c1;
    float d8;
    int s8;
    q8k_quantise8(x + bc * 256 + 8 * l, 8 * l, c0, c1, d8, s8);
    if (blk >= nblocks) return;
    float* yo = y + blk * 256 + 8 * l;
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[i] = d8 * (float)(int)(int8_t)((c0 >> (8 * i)) & 0xffu);
        v[4 + i] = d8 * (float)(int)(int8_t)((c1 >> (8 * i)) & 0xffu);
    }
    *(float4*)yo = make_float4(v[0], v[1], v[2], v[3]);
    *(float4*)(yo + 4) = make_float4(v[4], v[5], v[6], v[7]);
}

hipError_t launch_q8k_round_trip(const void* x, int x_dtype, int64_t rows, int64_t k, float* y, hipStream_t s) {
    const int64_t nblocks = rows * (k / 256), threads = nblocks * 32;
    const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
    if (x_dtype == QMM_F32) q8k_round_trip_kernel<float><<<grid, block, 0, s>>>((const float*)x, nblocks, y);
    else q8k_round_trip_kernel<uint16_t><<<grid, block, 0, s>>>((const uint16_t*)x, nblocks, y);
    return hipGetLastError();
}

template <int MT, int WPR, int L, typename AT>
__global__ __launch_bounds__(64 * kWaves, 2) void gemv_q4_k_q8k_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                                      float* __restrict__ out, int m, int n, int k, int64_t ldo,
                                                                      int ring_slots) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int part = wave % WPR;
    const int bpw = (nblk + WPR - 1) / WPR;                       // super-blocks per part (<= 16)
    const int blk0 = min(part * bpw, nblk - 1);
    const int nb = max(0, min(bpw, nblk - part * bpw));           // super-blocks of this part
    const int kRing = ring_slots;
    const int pieces = bpw * 9;       // 16-byte pieces of a full row part
    const int kSlot = pieces * 16;    // bytes of a slot
    uint8_t* ring = smem + wave * (kRing * kSlot);
    const uint32_t ring_lds = lds_address(ring);
    float* res = (float*)(smem + kWaves * kRing * kSlot) + wave * kMaxRows * MT;
    uint8_t* qbase = smem + kWaves * kRing * kSlot + kWaves * kMaxRows * MT * 4;
    uint32_t* lds_codes = (uint32_t*)qbase;                           // [MT][k / 4] dwords of four codes
    float* lds_d8 = (float*)(qbase + (size_t)MT * k);                  // [MT][nblk]
    int* lds_sum = (int*)(lds_d8 + MT * nblk);                        // [MT][k / 32] sums of 32 codes
    const int gs = (int)blockIdx.x * (kWaves / WPR) + wave / WPR, GS = (int)gridDim.x * (kWaves / WPR);
    const int my_rows = gs < n ? (n - gs + GS - 1) / GS : 0;

    const int last_piece = max(nb, 1) * 9 - 1;
    auto issue = [&](int ri, int slot) {
        const uint8_t* base = w + (int64_t)(gs + (int64_t)ri * GS) * row_bytes + (int64_t)blk0 * Q4_K_BPB;
#pragma unroll
        for (int i = 0; i < L; i++)
            if (lane + 64 * i < pieces)
                load16_to_lds_once(base + 16 * min(lane + 64 * i, last_piece), ring_lds + slot * kSlot + i * 1024);
    };
    // the first weight rows are issued before the lhs is touched: the compiler's waits for the lhs loads below also
    // wait for these rows, which the first decode needs anyway
    int issued = 0, islot = 0;
    for (; issued < min(kRing - 1, my_rows); issued++) {
        issue(issued, islot);
        islot = islot + 1 == kRing ? 0 : islot + 1;
    }

    // --- lhs -> Q8_K, once per workgroup: thread t takes 8 values of a block (32 threads per block)
    {
        const int t = (int)threadIdx.x;
        const int per_pass = 64 * kWaves * 8;  // values per pass of the workgroup
        for (int mi = 0; mi < MT; mi++) {
            const AT* ar = a + (int64_t)min(mi, m - 1) * k;
            for (int v0 = 0; v0 < k; v0 += per_pass) {
                const int vi = min(v0 + 8 * t, k - 256 + 8 * (t & 31));  // past the end: the last block again
                uint32_t c0, c1;
                float d8;
                int s8;
                q8k_quantise8(ar + vi, vi & 255, c0, c1, d8, s8);
                int s32 = s8 + __builtin_amdgcn_update_dpp(0, s8, 0xB1, 0xf, 0xf, false);
                s32 += __builtin_amdgcn_update_dpp(0, s32, 0x4E, 0xf, 0xf, false);  // 32 codes: four threads
                if (v0 + 8 * t < k) {
                    *(uint2*)(lds_codes + ((size_t)mi * k + vi) / 4) = make_uint2(c0, c1);
                    if ((t & 31) == 0) lds_d8[mi * nblk + (vi >> 8)] = d8;
                    if ((t & 3) == 0) lds_sum[mi * (k >> 5) + (vi >> 5)] = s32;
                }
            }
        }
    }
    __syncthreads();
    // the lane's chunk: super-block blk0 + lane / 4 (clamped: lanes past the part contribute nothing), chunk c
    const int lb = min(lane >> 2, max(nb, 1) - 1), c = lane & 3;
    const bool live = (lane >> 2) < nb;
    uint32_t qlo[MT][8], qhi[MT][8];
    float d8r[MT];
    int blo[MT], bhi[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        const int v0 = (blk0 + lb) * 256 + 64 * c;
        const uint4* cp = (const uint4*)(lds_codes + ((size_t)mi * k + v0) / 4);
        const uint4 c0 = cp[0], c1 = cp[1], c2 = cp[2], c3 = cp[3];
        qlo[mi][0] = c0.x; qlo[mi][1] = c0.y; qlo[mi][2] = c0.z; qlo[mi][3] = c0.w;
        qlo[mi][4] = c1.x; qlo[mi][5] = c1.y; qlo[mi][6] = c1.z; qlo[mi][7] = c1.w;
        qhi[mi][0] = c2.x; qhi[mi][1] = c2.y; qhi[mi][2] = c2.z; qhi[mi][3] = c2.w;
        qhi[mi][4] = c3.x; qhi[mi][5] = c3.y; qhi[mi][6] = c3.z; qhi[mi][7] = c3.w;
        d8r[mi] = live ? lds_d8[mi * nblk + blk0 + lb] : 0.0f;
        blo[mi] = lds_sum[mi * (k >> 5) + (v0 >> 5)];
        bhi[mi] = lds_sum[mi * (k >> 5) + (v0 >> 5) + 1];
    }
    const int sh = 16 * (c & 1);  // byte pair (2c, 2c + 1) mod 4 inside a dword of the 6-bit fields
    const bool upper = c >= 2;    // sub-blocks 4..7 use the split encoding

    int cslot = 0;
    for (int ri = 0; ri < my_rows; ri++) {
        if (issued < my_rows) {
            issue(issued, islot);
            islot = islot + 1 == kRing ? 0 : islot + 1;
            issued++;
        }
        wait_items<L, 0>(issued - 1 - ri, false);
        const uint8_t* blk = ring + cslot * kSlot + lb * Q4_K_BPB;
        cslot = cslot + 1 == kRing ? 0 : cslot + 1;
        const uint4 hdr = *(const uint4*)blk;
        const uint4 q0 = *(const uint4*)(blk + 16 + 32 * c), q1 = *(const uint4*)(blk + 32 + 32 * c);
        const uint32_t qd[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        int il[MT], ih[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) il[mi] = ih[mi] = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int lo = (int)(qd[i] & 0x0F0F0F0Fu), hi = (int)((qd[i] >> 4) & 0x0F0F0F0Fu);
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                il[mi] = __builtin_amdgcn_sdot4(lo, (int)qlo[mi][i], il[mi], false);
                ih[mi] = __builtin_amdgcn_sdot4(hi, (int)qhi[mi][i], ih[mi], false);
            }
        }
        const float d = h2f((uint16_t)(hdr.x & 0xffffu)), dmin = h2f((uint16_t)(hdr.x >> 16));
        const uint32_t p0 = (hdr.y >> sh) & 0xffffu, p1 = (hdr.z >> sh) & 0xffffu, p2 = (hdr.w >> sh) & 0xffffu;
        const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
        const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
        const int sc0 = (int)(sc_pair & 0xffu), sc1 = (int)(sc_pair >> 8), mn0 = (int)(mn_pair & 0xffu), mn1 = (int)(mn_pair >> 8);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            // |il| <= 32 * 15 * 127, times a 6-bit scale, twice: below 2^23, so the integers and their fp32 images are exact
            const int is = __mul24(sc0, il[mi]) + __mul24(sc1, ih[mi]);
            const int ms = __mul24(mn0, blo[mi]) + __mul24(mn1, bhi[mi]);
            float t = (d8r[mi] * d) * (float)is;
            t = fmaf(-(d8r[mi] * dmin), (float)ms, t);
            const float v = wave_sum_dpp(t);
            if (lane == 0) res[ri * MT + mi] = v;
        }
    }
    if constexpr (WPR == 1) {
        for (int idx = lane; idx < my_rows * MT; idx += 64) {
            const int r = idx / MT, mi = idx - r * MT;
            if (mi < m) out[(int64_t)mi * ldo + gs + (int64_t)r * GS] = res[idx];
        }
    } else {
        __syncthreads();
        if (part == 0) {
            for (int idx = lane; idx < my_rows * MT; idx += 64) {
                const int r = idx / MT, mi = idx - r * MT;
                float v = res[idx];
#pragma unroll
                for (int q = 1; q < WPR; q++) v += res[q * kMaxRows * MT + idx];
                if (mi < m) out[(int64_t)mi * ldo + gs + (int64_t)r * GS] = v;
            }
        }
    }
}

hipError_t launch_quantize_q8_k(const void* x, int x_dtype, int64_t rows, int64_t k, void* out, hipStream_t s) {
    const int64_t nblocks = rows * (k / 256);
    dim3 grid((unsigned)((nblocks * 32 + 255) / 256)), block(256);
    if (x_dtype == QMM_F32) quantize_q8_k_kernel<float><<<grid, block, 0, s>>>((const float*)x, nblocks, (uint8_t*)out);
    else quantize_q8_k_kernel<uint16_t><<<grid, block, 0, s>>>((const uint16_t*)x, nblocks, (uint8_t*)out);
    return hipGetLastError();
}

// m <= 4, K <= 16384 (reports other shapes through *handled = false).
hipError_t launch_gemv_q4_k_q8k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                int64_t ldo, hipStream_t s, bool* handled) {
    *handled = false;
    const int nblk = (int)(k / 256);
    if (m > 4 || nblk > 64) return hipSuccess;
    const int wpr = nblk <= 16 ? 1 : nblk <= 32 ? 2 : 4;
    const int bpw = (nblk + wpr - 1) / wpr;
    const int l = (bpw * 9 + 63) / 64;  // 1..3
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const size_t fixed = (size_t)kWaves * kMaxRows * mt * 4 + (size_t)mt * ((size_t)k + (size_t)nblk * 4 + (size_t)(k / 32) * 4);
    const size_t slot = (size_t)bpw * Q4_K_BPB;
    int ring = 3;
    if ((size_t)kWaves * ring * slot + fixed > (size_t)kLdsPerCu) ring = 2;
    const size_t lds = (size_t)kWaves * ring * slot + fixed;
    if (lds > (size_t)kLdsPerCu) return hipSuccess;
    const int streams = kWaves / wpr;
    int64_t wgs = cus;
    if (wgs * streams > n) wgs = (n + streams - 1) / streams;
    const int64_t min_wgs = (n + (int64_t)streams * kMaxRows - 1) / ((int64_t)streams * kMaxRows);
    if (wgs < min_wgs) wgs = min_wgs;  // no wavefront owns more rows than it has result slots
    dim3 grid((unsigned)wgs), block(64 * kWaves);
#define QMM_GO3(MT_, WPR_, L_, AT_)                                                                                   \
    do {                                                                                                              \
        hipError_t e_ = allow_full_lds<gemv_q4_k_q8k_kernel<MT_, WPR_, L_, AT_>>();                                   \
        if (e_ != hipSuccess) return e_;                                                                              \
        gemv_q4_k_q8k_kernel<MT_, WPR_, L_, AT_><<<grid, block, lds, s>>>(w, (const AT_*)a, out, m, (int)n, (int)k, ldo, ring); \
    } while (0)
#define QMM_GO2(MT_, WPR_, L_)                            \
    do {                                                  \
        if (a_dtype == QMM_F32) QMM_GO3(MT_, WPR_, L_, float); \
        else QMM_GO3(MT_, WPR_, L_, uint16_t);            \
    } while (0)
#define QMM_GO1(WPR_, L_)                 \
    do {                                  \
        if (mt == 1) QMM_GO2(1, WPR_, L_); \
        else if (mt == 2) QMM_GO2(2, WPR_, L_); \
        else QMM_GO2(4, WPR_, L_);        \
    } while (0)
#define QMM_GO0(WPR_)               \
    do {                            \
        if (l == 1) QMM_GO1(WPR_, 1); \
        else if (l == 2) QMM_GO1(WPR_, 2); \
        else QMM_GO1(WPR_, 3);      \
    } while (0)
    if (wpr == 1) QMM_GO0(1);
    else if (wpr == 2) QMM_GO0(2);
    else QMM_GO0(4);
#undef QMM_GO0
#undef QMM_GO1
#undef QMM_GO2
#undef QMM_GO3
    *handled = true;
    return hipGetLastError();
}

}  // namespace qmm
