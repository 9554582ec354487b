// GPTQ small-batch kernel (2..16 lhs rows per pass) on the matrix cores.
//
// A qweight word holds eight consecutive k of one column, which is exactly what a lane supplies of the B
// operand of v_mfma_f32_16x16x32_f16 (lane l: column l % 16, k = 8 * (l / 16) .. + 7): a lane loads the words of
// two neighbouring columns (8 bytes; the 16 lanes of a row read 128 contiguous bytes, the four rows four
// consecutive word rows), and one shift and one mask per register move the nibbles v and v + 4 of a word to
// bits 6..9 of the two halves of register v: the fp16 subnormals q * 2^-18.  (The nibble sits at the top of the
// subnormal's mantissa on purpose.  The matrix core does not normalise subnormal inputs before it aligns the
// products of a step: with the nibble in bits 0..3, q * 2^-24, the low bits of every product fall off the end of
// the adder, always towards minus infinity, and with non-negative codes that adds up to a bias that grows with
// K, 6e-5 at K = 14336 with unit-size activations.)  The lhs is the A operand in the matching order (a[v], a[v + 4] in
// register v), scaled per (row, wavefront) by a power of two and narrowed to fp16 (fp32 lhs: plus the residual
// as a second plane with accumulators of its own, two matrix-core instructions per step), so every product is
// exact and the sums are fp32.  Per group
//     acc += scale * (2^18 * P  -  zero * sum of the scaled lhs row over the group),
// two multiply-adds per output and group.
//
// Shape.  Wavefront w of a workgroup owns the 256 k values [256 w, 256 w + 256) for the whole kernel and keeps
// its lhs operands (16 rows x 256 k: 32 registers a plane), the group sums and the inverse row scales in
// registers; a workgroup of up to 16 wavefronts walks over strips of 32 columns.  K beyond 4096 is cut into equal
// chunks of at most 16 wavefront parts, one per value of blockIdx.y: the chunks write their partial results to a
// workspace, [chunk][row][N], and a second kernel adds them in chunk order.  The eight loads of a strip are replaced, as they are
// consumed, by those of the workgroup's next strip.  The wavefronts' partial sums of a strip meet in LDS and are
// added in wavefront order: results do not depend on timing.
#include <stdlib.h>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kPartK = 256;         // k values of a wavefront
constexpr int kKB = kPartK / 32;    // matrix-core steps of a wavefront per strip
constexpr int kStrip = 32;          // columns of a strip
constexpr int kMaxWaves = 16;
constexpr int kLoReg = 2;            // residual-plane operands of a wavefront kept in registers; the other kKB - kLoReg in LDS
constexpr int kLoLds = kKB - kLoReg;

__device__ __forceinline__ half8 nibble_operand(uint32_t w) {
    constexpr uint32_t kTop = 0x03C003C0u;  // mantissa bits 6..9 of both halves
    return pack4((w << 6) & kTop, (w << 2) & kTop, (w >> 2) & kTop, (w >> 6) & kTop);
}

// PLANES: 1 (bf16 lhs: exact in one fp16 plane) or 2 (fp32 lhs).  GK: 32-wide steps per group (group 64 / 128 / 256).
template <int PLANES, int GK, typename AT>
__global__ __launch_bounds__(64 * kMaxWaves) void gemv_gptq_mm_kernel(
    const uint32_t* __restrict__ qweight, const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const AT* __restrict__ a, float* __restrict__ out, int m, int n, int64_t lda, int64_t ldo, int nstrips,
    int parts_total, int64_t chunk_stride) {
    constexpr int NG = kKB / GK;  // groups of a wavefront's part
    extern __shared__ __attribute__((aligned(16))) float mm_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = (int)(blockDim.x >> 6);
    const int c = lane & 15, kq = lane >> 4;
    // this wavefront's 256 k: part `part` of the row; the wavefronts of the last chunk beyond the end of the row redo
    // the last part (every address stays valid, the barriers stay uniform) and contribute zeros
    const int part_raw = (int)blockIdx.y * nw + wave;
    const bool part_live = part_raw < parts_total;
    const int part = __builtin_amdgcn_readfirstlane(min(part_raw, parts_total - 1));
    out += (int64_t)blockIdx.y * chunk_stride;
    float* park = mm_lds;                                // [nw][512]
    float* tr = mm_lds + nw * 512 + wave * (NG + 1) * 16;  // this wavefront's [NG + 1][16]

    // --- the first strip's loads go out before anything else ---
    // word row of (part, step kb, lane row kq): 32 * part + 4 * kb + kq; columns n0 + 2c, n0 + 2c + 1.  Lanes
    // beyond N read the last column pair instead (their outputs are not stored).
    const uint32_t* wrow = qweight + (int64_t)(32 * part + kq) * n;
    const int n_half = n >> 3;
    auto col_of = [&](int strip) { return min(strip * kStrip + 2 * c, n - 2); };
    uint2 wq[kKB];
    uint32_t sc2[NG], zw[NG];
    auto load_strip = [&](int strip) {
        const int col = col_of(strip);
#pragma unroll
        for (int kb = 0; kb < kKB; kb++) wq[kb] = *(const uint2*)(wrow + (int64_t)(4 * kb) * n + col);
    };
    auto load_params = [&](int strip) {
        const int col = col_of(strip);
#pragma unroll
        for (int g = 0; g < NG; g++) {
            const int64_t gi = (int64_t)part * NG + g;
            sc2[g] = *(const uint32_t*)(scales + gi * n + col);
            zw[g] = qzeros[gi * n_half + (col >> 3)];
        }
    };
    int strip = (int)blockIdx.x;
    if (strip < nstrips) {
        load_strip(strip);
        load_params(strip);
    }

    // --- this wavefront's lhs part: lane (row c, k quarter kq) holds a[c][256 part + 32 kb + 8 kq + 0..7] ---
    // (fp32 lhs: main and residual operands, 64 registers, do not fit next to the loads in flight in the 128
    // registers of a 16-wavefront workgroup: with all of them in registers the compiler spilled a dozen to scratch
    // memory and 14336 x 4096 with 16 rows took 24.7 us; with six of the eight residual operands in LDS, each lane
    // reading back what it wrote, 21.3 us.  One plane alone: 18.5 us.)
    half8 ahi[kKB], alo[PLANES == 2 ? kLoReg : 1];
    half8* lo_w = (half8*)(mm_lds + nw * 512 + nw * (NG + 1) * 16) + wave * kLoLds * 64 + lane;  // [kLoLds][64] per wavefront
    {
        float x[kKB][8];
        const AT* ar = a + (int64_t)min(c, m - 1) * lda + part * kPartK + kq * 8;
#pragma unroll
        for (int kb = 0; kb < kKB; kb++) {
            if constexpr (sizeof(AT) == 4) {
                const float4 p = *(const float4*)(ar + kb * 32), q = *(const float4*)(ar + kb * 32 + 4);
                x[kb][0] = p.x; x[kb][1] = p.y; x[kb][2] = p.z; x[kb][3] = p.w;
                x[kb][4] = q.x; x[kb][5] = q.y; x[kb][6] = q.z; x[kb][7] = q.w;
            } else {
                const uint4 p = *(const uint4*)(ar + kb * 32);
                x[kb][0] = bf2f((uint16_t)p.x); x[kb][1] = bf2f((uint16_t)(p.x >> 16));
                x[kb][2] = bf2f((uint16_t)p.y); x[kb][3] = bf2f((uint16_t)(p.y >> 16));
                x[kb][4] = bf2f((uint16_t)p.z); x[kb][5] = bf2f((uint16_t)(p.z >> 16));
                x[kb][6] = bf2f((uint16_t)p.w); x[kb][7] = bf2f((uint16_t)(p.w >> 16));
            }
        }
        const bool row_live = c < m;
        uint32_t mx = 0;
#pragma unroll
        for (int kb = 0; kb < kKB; kb++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                x[kb][i] = row_live ? x[kb][i] : 0.0f;
                mx = max(mx, __float_as_uint(x[kb][i]) & 0x7fffffffu);
            }
        mx = max(mx, (uint32_t)__shfl_xor((int)mx, 16, kWave));
        mx = max(mx, (uint32_t)__shfl_xor((int)mx, 32, kWave));
        // scale = 2^(14 - exponent of the largest magnitude): the row lies below 2^15 (fp16 reaches 65504); an
        // all-zero row keeps scale 1; a non-finite row gets a finite scale and stays non-finite.
        const int e_max = (int)(mx >> 23);
        const int e_scale = mx == 0 ? 127 : min(max(268 - e_max, 1), 253);
        const float scale = __uint_as_float((uint32_t)e_scale << 23);
        const float inv_scale = __uint_as_float((uint32_t)(254 - e_scale) << 23);
        float gs[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) gs[g] = 0.0f;
#pragma unroll
        for (int kb = 0; kb < kKB; kb++) {
            uint32_t hi[4], lo[4];
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float s0 = x[kb][v] * scale, s1 = x[kb][v + 4] * scale;
                const _Float16 h0 = (_Float16)s0, h1 = (_Float16)s1;
                union { _Float16 h[2]; uint32_t u; } ph, pl;
                ph.h[0] = h0; ph.h[1] = h1;
                hi[v] = ph.u;
                pl.h[0] = (_Float16)(s0 - (float)h0); pl.h[1] = (_Float16)(s1 - (float)h1);
                lo[v] = pl.u;
                gs[kb / GK] += s0 + s1;
            }
            ahi[kb] = pack4(hi[0], hi[1], hi[2], hi[3]);
            if constexpr (PLANES == 2) {
                if (kb < kLoReg) alo[kb] = pack4(lo[0], lo[1], lo[2], lo[3]);
                else lo_w[(kb - kLoReg) * 64] = pack4(lo[0], lo[1], lo[2], lo[3]);
            }
        }
        // group sums over the four k quarters, then row c -> the lanes that hold row 4 * kq + r of the results
#pragma unroll
        for (int g = 0; g < NG; g++) {
            gs[g] += __shfl_xor(gs[g], 16, kWave);
            gs[g] += __shfl_xor(gs[g], 32, kWave);
            if (kq == 0) tr[g * 16 + c] = gs[g];
        }
        if (kq == 0) tr[NG * 16 + c] = inv_scale;
        __syncthreads();
    }

    const int zshift = 4 * ((2 * c) & 7);
    for (; strip < nstrips; strip += (int)gridDim.x) {
        const int next = strip + (int)gridDim.x;
        const bool more = next < nstrips;  // uniform
        float acc[2][4];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[j][r] = 0.0f;
        const uint32_t* wnext = wrow + col_of(more ? next : strip);
#pragma unroll
        for (int g = 0; g < NG; g++) {
            const float4 as4 = *(const float4*)(tr + g * 16 + 4 * kq);  // group sums of result rows 4 kq + 0..3
            const float asum[4] = {as4.x, as4.y, as4.z, as4.w};
            const float sz0 = h2f((uint16_t)sc2[g]), sz1 = h2f((uint16_t)(sc2[g] >> 16));
            const float zp0 = (float)(((zw[g] >> zshift) & 0xFu) + 1u), zp1 = (float)(((zw[g] >> (zshift + 4)) & 0xFu) + 1u);
            // the two columns of a lane one after the other (half the accumulators in flight); the loads of the
            // next strip replace this group's words once both have used them
#pragma unroll
            for (int j = 0; j < 2; j++) {
                // The residual plane has accumulators of its own: next to the large main sums its small products
                // would lose their low bits inside the matrix core.
                float4v P = {0.f, 0.f, 0.f, 0.f}, R = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < GK; kk++) {
                    const int kb = g * GK + kk;
                    const half8 b = nibble_operand(j == 0 ? wq[kb].x : wq[kb].y);
                    P = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi[kb], b, P, 0, 0, 0);
                    if constexpr (PLANES == 2)
                        R = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb < kLoReg ? alo[kb] : lo_w[(kb - kLoReg) * 64], b, R, 0, 0, 0);
                }
                if constexpr (PLANES == 2) P += R;
                const float sc = j == 0 ? sz0 : sz1, zp = j == 0 ? zp0 : zp1;
                const float scp = sc * 262144.0f, scz = -sc * zp;
#pragma unroll
                for (int r = 0; r < 4; r++) acc[j][r] = fmaf(scp, P[r], fmaf(scz, asum[r], acc[j][r]));
            }
            if (more) {
#pragma unroll
                for (int kk = 0; kk < GK; kk++) wq[g * GK + kk] = *(const uint2*)(wnext + (int64_t)(4 * (g * GK + kk)) * n);
            }
        }
        if (more) load_params(next);  // (this strip's are spent: no second set of registers)
        // partial sums of this wavefront's k range, back in the lhs row's own scale
        float* mine = park + wave * 512;
        const float4 iv4 = *(const float4*)(tr + NG * 16 + 4 * kq);  // inverse scales of result rows 4 kq + 0..3
        const float inv[4] = {iv4.x, iv4.y, iv4.z, iv4.w};
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) mine[(j * 4 + r) * 64 + lane] = part_live ? acc[j][r] * inv[r] : 0.0f;
        __syncthreads();
        for (int t = tid; t < 512; t += (int)blockDim.x) {
            float v = 0.0f;
            for (int w = 0; w < nw; w++) v += park[w * 512 + t];
            const int j = t >> 8, r = (t >> 6) & 3, l = t & 63;
            const int row = 4 * (l >> 4) + r, col = strip * kStrip + 2 * (l & 15) + j;
            if (row < m && col < n) {
                out[(int64_t)row * ldo + col] = v;
            }
        }
        if (more) __syncthreads();  // the next strip's partial sums go to the same place
    }
}

}  // namespace

bool gemv_gptq_mm_supported(const void* qweight, int64_t n, int64_t k, int group) {
    return !kernel_disabled("gptq_mm") && k % kPartK == 0 && n >= 8 && n % 8 == 0 && ((uintptr_t)qweight & 7) == 0 &&
           (group == 64 || group == 128 || group == 256);
}

namespace {

// K = chunks * (wavefronts per workgroup) * 256 at most, chunks as few as 16 wavefronts allow, of equal size
struct MmChunks {
    int chunks, nw;
};
MmChunks mm_chunks(int64_t k) {
    const int parts = (int)(k / kPartK);
    const int chunks = (parts + kMaxWaves - 1) / kMaxWaves;
    return {chunks, (parts + chunks - 1) / chunks};
}

// out[r][c] = sum over the chunks of part[chunk][r][c], in chunk order
__global__ __launch_bounds__(256) void gemv_gptq_mm_sum_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                               int m, int n, int64_t ldo, int chunks) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x, count = (int64_t)m * n;
    if (i >= count) return;
    float v = 0.0f;
    for (int ch = 0; ch < chunks; ch++) v += part[ch * count + i];
    out[(i / n) * ldo + i % n] = v;
}

}  // namespace

// Workspace of one call with up to 16 lhs rows: the chunks' partial results when K is beyond 4096.
int64_t gemv_gptq_mm_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    if (k % kPartK || k <= (int64_t)kMaxWaves * kPartK) return 0;
    return (int64_t)mm_chunks(k).chunks * std::min<int64_t>(m, 16) * n * 4;
}

// 1..16 lhs rows, K a multiple of 256, group 64 / 128 / 256, qweight 8-byte aligned: otherwise *handled stays
// false and nothing is launched.  `workspace` holds gemv_gptq_mm_workspace_bytes(m, n, k) bytes.
hipError_t launch_gemv_gptq_mm(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                               const uint32_t* qzeros, int m, int64_t n, int64_t k, int group, float* out, int64_t ldo,
                               void* workspace, hipStream_t s, bool* handled) {
    *handled = false;
    if (m < 1 || m > 16 || !gemv_gptq_mm_supported(qweight, n, k, group)) return hipSuccess;
    if (a_dtype != QMM_F32 && a_dtype != QMM_BF16) return hipSuccess;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    const int gk = group / 32, ng = kKB / gk;
    const int nstrips = (int)((n + kStrip - 1) / kStrip);
    const MmChunks cc = mm_chunks(k);
    if (cc.chunks > 1 && !workspace) return hipErrorInvalidValue;
    const int nw = cc.nw, parts_total = (int)(k / kPartK);
    const size_t lds = ((size_t)nw * 512 + (size_t)nw * (ng + 1) * 16) * sizeof(float) +  // at most 34 KB
                       (a_dtype == QMM_F32 ? (size_t)nw * kLoLds * 64 * 16 : 0);            // + 96 KB
    const int per_cu = std::max(1, kMaxWaves / nw);
    const int64_t wgs_x = std::max<int64_t>(1, std::min<int64_t>(nstrips, (int64_t)cus * per_cu / cc.chunks));
    dim3 grid((unsigned)wgs_x, (unsigned)cc.chunks), block(64 * nw);
    float* dst = cc.chunks > 1 ? (float*)workspace : out;
    const int64_t dst_ld = cc.chunks > 1 ? n : ldo, chunk_stride = cc.chunks > 1 ? (int64_t)m * n : 0;
#define QMM_GPTQ_MM(PL_, GK_, AT_)                                                                                   \
    do {                                                                                                             \
        if (lds > 64 * 1024) { /* (raised once, to the whole LDS) */                                                 \
            hipError_t e_ = allow_full_lds<gemv_gptq_mm_kernel<PL_, GK_, AT_>>();                                    \
            if (e_ != hipSuccess) return e_;                                                                         \
        }                                                                                                            \
        gemv_gptq_mm_kernel<PL_, GK_, AT_><<<grid, block, lds, s>>>(qweight, scales, qzeros, (const AT_*)a, dst, m,  \
                                                                    (int)n, k, dst_ld, nstrips, parts_total,         \
                                                                    chunk_stride);                                   \
    } while (0)
#define QMM_GPTQ_MM_GK(GK_)                                  \
    do {                                                     \
        if (a_dtype == QMM_F32) QMM_GPTQ_MM(2, GK_, float);  \
        else QMM_GPTQ_MM(1, GK_, uint16_t);                  \
    } while (0)
    if (gk == 2) QMM_GPTQ_MM_GK(2);
    else if (gk == 4) QMM_GPTQ_MM_GK(4);
    else QMM_GPTQ_MM_GK(8);
#undef QMM_GPTQ_MM_GK
#undef QMM_GPTQ_MM
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (cc.chunks > 1) {
        const int64_t count = (int64_t)m * n;
        gemv_gptq_mm_sum_kernel<<<dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s>>>((const float*)workspace, out, m,
                                                                                            (int)n, ldo, cc.chunks);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    *handled = true;
    return hipSuccess;
}

}  // namespace qmm
