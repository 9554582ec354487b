// Q5_K decode kernel (up to four lhs rows per pass).
//
// A Q5_K super-block is 176 bytes: the Q4_K header (f16 d, f16 dmin, 12 bytes of 6-bit scales and
// mins), qh[32] and qs[128].  Code (sub-block j, position l) has its low four bits in the low
// (j even) or high (j odd) nibble of qs[32 (j / 2) + l] and its fifth bit in bit j of qh[l].
//
// Shape of the work: a wavefront owns whole weight rows.  The super-blocks of a row are taken 16 at
// a time (a "group": 4096 columns); lane (block lb = lane / 4, chunk c = lane % 4) decodes the 64
// weights of sub-blocks 2c and 2c + 1 of its block: 32 code bytes, all 32 qh bytes (bits 2c and
// 2c + 1 of each), two scales and two mins.  Five aligned 16-byte loads per lane and item, issued
// one item ahead of the one being decoded.  The lhs is staged once per workgroup in LDS as float4s in
// the order [group][quartet i of the lane's 64 columns][lane], so that a lane's 16 reads are
// conflict-free; with a single lhs row and K <= 4096 the 64 activations stay in registers instead.
// 5-bit code bytes are assembled four at a time (nibble mask | fifth bits shifted to bit 4) and
// converted with v_cvt_f32_ubyteN; per sub-block  d sc sum(a q) - dmin mn sum(a).
#include <stdlib.h>

#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int kWavesQ5 = 4;
constexpr int kGroupCols = 4096;  // columns of a group: 16 super-blocks

__device__ __forceinline__ float ub0(uint32_t x) { float r; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float ub1(uint32_t x) { float r; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float ub2(uint32_t x) { float r; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float ub3(uint32_t x) { float r; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(x)); return r; }

struct Q5Item {
    uint4 hdr, qh0, qh1, qs0, qs1;
};

__device__ __forceinline__ float dot4(const float4 a, uint32_t q) {
    return fmaf(a.w, ub3(q), fmaf(a.z, ub2(q), fmaf(a.y, ub1(q), a.x * ub0(q))));
}

}  // namespace

// MT lhs rows (1, 2 or 4; rows past m repeat the last one and are not stored).
// HOIST: one lhs row and one group: the lane's activations live in registers for the whole kernel.
template <int MT, bool HOIST, typename AT>
__global__ __launch_bounds__(64 * kWavesQ5) void gemv_q5_k_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                                 float* __restrict__ out, int m, int n, int k, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) float4 xs[];  // [MT][ngroups][16][64]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk = k >> 8;
    const int ngroups = (nblk + 15) >> 4;
    const int64_t row_bytes = (int64_t)nblk * Q5_K_BPB;
    const int lb = lane >> 2, c = lane & 3;

    // lhs -> LDS: float4 t of (row mi, group g) covers columns 4096 g + 4 t; it belongs to lane t / 16, quartet t % 16
    const int per_row = ngroups * 1024;
    for (int idx = tid; idx < MT * per_row; idx += 64 * kWavesQ5) {
        const int mi = idx / per_row, r = idx - mi * per_row;
        const int g = r >> 10, t = r & 1023;
        const int col = g * kGroupCols + 4 * t;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (col < k) {
            const AT* ar = a + (int64_t)min(mi, m - 1) * k + col;
            v = make_float4(load_f32(ar, 0), load_f32(ar, 1), load_f32(ar, 2), load_f32(ar, 3));
        }
        xs[(mi * ngroups + g) * 1024 + (t & 15) * 64 + (t >> 4)] = v;
    }
    __syncthreads();

    const int total_waves = (int)gridDim.x * kWavesQ5, gw = (int)blockIdx.x * kWavesQ5 + wave;
    const int my_rows = gw < n ? (n - gw + total_waves - 1) / total_waves : 0;
    const int items = my_rows * ngroups;

    // sub-blocks 2c, 2c + 1: byte pair (2c, 2c + 1) mod 4 of the 6-bit fields; 4..7 use the split encoding
    const int sh = 16 * (c & 1);
    const bool upper = c >= 2;

    auto load_item = [&](int it) {
        const int ri = it / ngroups, g = it - ri * ngroups;
        const int blk = min(16 * g + lb, nblk - 1);
        const uint8_t* b = w + (int64_t)(gw + (int64_t)ri * total_waves) * row_bytes + (int64_t)blk * Q5_K_BPB;
        Q5Item x;
        x.hdr = *(const uint4*)b;
        x.qh0 = *(const uint4*)(b + 16);
        x.qh1 = *(const uint4*)(b + 32);
        x.qs0 = *(const uint4*)(b + 48 + 32 * c);
        x.qs1 = *(const uint4*)(b + 64 + 32 * c);
        return x;
    };

    float4 xh[16];
    float sum_lo_h = 0.f, sum_hi_h = 0.f;
    if constexpr (HOIST) {
#pragma unroll
        for (int i = 0; i < 16; i++) xh[i] = xs[i * 64 + lane];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            sum_lo_h += (xh[i].x + xh[i].y) + (xh[i].z + xh[i].w);
            sum_hi_h += (xh[8 + i].x + xh[8 + i].y) + (xh[8 + i].z + xh[8 + i].w);
        }
    }

    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;
    Q5Item cur;
    if (items > 0) cur = load_item(0);
    int ri = 0, g = 0;
    for (int it = 0; it < items; it++) {
        Q5Item nxt = cur;
        if (it + 1 < items) nxt = load_item(it + 1);
        const bool live = 16 * g + lb < nblk;
        // header: d, dmin, scales and mins of sub-blocks 2c and 2c + 1
        const float d = h2f((uint16_t)(cur.hdr.x & 0xffffu)), dmin = h2f((uint16_t)(cur.hdr.x >> 16));
        const uint32_t p0 = (cur.hdr.y >> sh) & 0xffffu, p1 = (cur.hdr.z >> sh) & 0xffffu, p2 = (cur.hdr.w >> sh) & 0xffffu;
        const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
        const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
        const float d_lo = d * (float)(sc_pair & 0xffu), d_hi = d * (float)(sc_pair >> 8);
        const float m_lo = dmin * (float)(mn_pair & 0xffu), m_hi = dmin * (float)(mn_pair >> 8);
        // code bytes, four positions per dword: low nibbles + fifth bit 2c, high nibbles + fifth bit 2c + 1
        const uint32_t qs[8] = {cur.qs0.x, cur.qs0.y, cur.qs0.z, cur.qs0.w, cur.qs1.x, cur.qs1.y, cur.qs1.z, cur.qs1.w};
        const uint32_t qh[8] = {cur.qh0.x, cur.qh0.y, cur.qh0.z, cur.qh0.w, cur.qh1.x, cur.qh1.y, cur.qh1.z, cur.qh1.w};
        uint32_t lo[8], hi[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t hb = qh[i] >> (2 * c);
            lo[i] = (qs[i] & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
            hi[i] = ((qs[i] >> 4) & 0x0F0F0F0Fu) | ((hb << 3) & 0x10101010u);
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            float s_lo = 0.f, s_hi = 0.f, a_lo = 0.f, a_hi = 0.f;
            if constexpr (HOIST) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    s_lo += dot4(xh[i], lo[i]);
                    s_hi += dot4(xh[8 + i], hi[i]);
                }
                a_lo = sum_lo_h;
                a_hi = sum_hi_h;
            } else {
                const float4* xr = xs + (mi * ngroups + g) * 1024 + lane;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float4 u = xr[i * 64], v = xr[(8 + i) * 64];
                    s_lo += dot4(u, lo[i]);
                    s_hi += dot4(v, hi[i]);
                    a_lo += (u.x + u.y) + (u.z + u.w);
                    a_hi += (v.x + v.y) + (v.z + v.w);
                }
            }
            const float v = (d_lo * s_lo - m_lo * a_lo) + (d_hi * s_hi - m_hi * a_hi);
            acc[mi] += live ? v : 0.0f;
        }
        if (++g == ngroups) {
            const int row = gw + ri * total_waves;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const float s = wave_sum_dpp(acc[mi]);
                if (lane == 0 && mi < m) out[(int64_t)mi * ldo + row] = s;
                acc[mi] = 0.0f;
            }
            g = 0;
            ri++;
        }
        cur = nxt;
    }
}

// Up to four lhs rows; the rows of lhs a pass can take are limited by the LDS copy of the lhs
// (16 KB per row and 4096 columns).  *handled stays false for shapes this kernel does not take.
hipError_t launch_gemv_q5_k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                            int64_t ldo, hipStream_t s, bool* handled) {
    *handled = false;
    const int64_t ngroups = (k / 256 + 15) / 16;
    if (m < 1 || m > 4 || (k & 255) || ((uintptr_t)w & 15)) return hipSuccess;
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    const size_t lds = (size_t)mt * ngroups * 16384;
    if (lds > 128 * 1024) return hipSuccess;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    const int per_cu = (int)std::max<size_t>(1, std::min<size_t>(4, (size_t)kLdsPerCu / lds));
    dim3 grid((unsigned)std::min<int64_t>((n + kWavesQ5 - 1) / kWavesQ5, (int64_t)cus * per_cu)), block(64 * kWavesQ5);
    hipError_t e = hipSuccess;
#define QMM_Q5K_GO(MT_, H_)                                                                                           \
    do {                                                                                                              \
        if (a_dtype == QMM_F32) {                                                                                     \
            e = allow_full_lds<gemv_q5_k_kernel<MT_, H_, float>>();                                                   \
            if (e == hipSuccess)                                                                                      \
                gemv_q5_k_kernel<MT_, H_, float><<<grid, block, lds, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo); \
        } else {                                                                                                      \
            e = allow_full_lds<gemv_q5_k_kernel<MT_, H_, uint16_t>>();                                                \
            if (e == hipSuccess)                                                                                      \
                gemv_q5_k_kernel<MT_, H_, uint16_t><<<grid, block, lds, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo); \
        }                                                                                                             \
    } while (0)
    if (mt == 1 && ngroups == 1) QMM_Q5K_GO(1, true);
    else if (mt == 1) QMM_Q5K_GO(1, false);
    else if (mt == 2) QMM_Q5K_GO(2, false);
    else QMM_Q5K_GO(4, false);
#undef QMM_Q5K_GO
    if (e != hipSuccess) return e;
    *handled = true;
    return hipGetLastError();
}

}  // namespace qmm
