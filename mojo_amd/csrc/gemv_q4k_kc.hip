// Q4_K small-batch kernel (2..16 lhs rows) for shapes with few weight rows and long K: every wavefront owns one
// super-block column, K is cut along blockIdx.y.
//
// The small-batch kernel in gemv_q4k_mm.hip gives a workgroup whole weight rows, so with N = 4096 a workgroup has a
// single 16-row tile and prepares the whole lhs (K values per lhs row) for it: on 4096 x 14336 that preparation
// costs as much as the weights.  Here the work is cut the other way, as in the GPTQ small-batch kernel
// (gemv_gptq_mm.hip): wavefront w of a workgroup owns super-block b = chunk * waves + w of every weight row, keeps the
// lhs operands of those 256 k (16 rows, fp16 main plane and, for an fp32 lhs, a residual plane with accumulators of
// its own) in registers, and the workgroup walks over strips of 32 weight rows (two matrix-core tiles of 16).  A lane
// (row c = l % 16, quarter kq = l / 16) loads the 16-byte header of its row's super-block and, for each of the four
// 64-weight pairs, the 8 quant bytes 32 p + 8 kq .. + 7: their low nibbles are its share of sub-block 2p, the high
// nibbles of sub-block 2p + 1.  One shift and one mask put two nibbles at the top of the fp16 subnormal mantissa,
// q * 2^-18; one packed multiply by sc makes it sc * q * 2^-18 (exact; a normal number from 16 on, which the matrix
// cores need to keep the low product bits).  acc += d * 2^18 * P  -  dmin * sum_s mn_s * (sum of the scaled lhs row over sub-block s).
// The wavefronts' partial sums meet in LDS and are added in wavefront order; the chunks' partial results go to the
// workspace, [chunk][row][N], and a second kernel adds them in chunk order.
#include <stdlib.h>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kMaxWaves = 16;
constexpr int kStripRows = 32;
constexpr int kLoReg = 2, kLoLds = 8 - kLoReg;  // residual operands in registers / in LDS (as in the GPTQ kernel)

struct KcChunks {
    int chunks, nw;
};
KcChunks kc_chunks(int64_t k) {
    const int parts = (int)(k / 256);
    const int chunks = (parts + kMaxWaves - 1) / kMaxWaves;
    return {chunks, (parts + chunks - 1) / chunks};
}

__global__ __launch_bounds__(256) void gemv_q4_k_kc_sum_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                               int m, int n, int64_t ldo, int chunks) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x, count = (int64_t)m * n;
    if (i >= count) return;
    float v = 0.0f;
    for (int ch = 0; ch < chunks; ch++) v += part[ch * count + i];
    out[(i / n) * ldo + i % n] = v;
}

// PLANES: 1 (bf16 lhs) or 2 (fp32 lhs)
template <int PLANES, typename AT>
__global__ __launch_bounds__(64 * kMaxWaves) void gemv_q4_k_kc_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                                      float* __restrict__ out, int m, int n, int64_t lda,
                                                                      int64_t ldo, int nstrips, int nblk, int64_t chunk_stride) {
    extern __shared__ __attribute__((aligned(16))) float kc_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = (int)(blockDim.x >> 6);
    const int c = lane & 15, kq = lane >> 4;
    // this wavefront's super-block; the wavefronts of the last chunk beyond the end of the row redo the last one
    // (addresses stay valid, barriers uniform) and contribute zeros
    const int blk_raw = (int)blockIdx.y * nw + wave;
    const bool blk_live = blk_raw < nblk;
    const int blk = __builtin_amdgcn_readfirstlane(min(blk_raw, nblk - 1));
    out += (int64_t)blockIdx.y * chunk_stride;
    float* park = kc_lds;                          // [nw][512]
    float* tr = kc_lds + nw * 512 + wave * 9 * 16;  // this wavefront's [8 sub-block sums + inverse scale][16 lhs rows]
    half8* lo_w = (half8*)(kc_lds + nw * 512 + nw * 9 * 16) + wave * kLoLds * 64 + lane;

    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const uint8_t* wblk = w + (int64_t)blk * Q4_K_BPB;
    // rows of this lane in a strip: strip * 32 + c and + 16 (rows beyond N read the last row; not stored)
    uint4 hdr[2];
    uint2 qs[2][4];
    auto load_strip = [&](int strip) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint8_t* p = wblk + (int64_t)min(strip * kStripRows + 16 * j + c, n - 1) * row_bytes;
            hdr[j] = *(const uint4*)p;
#pragma unroll
            for (int q = 0; q < 4; q++) qs[j][q] = *(const uint2*)(p + 16 + 32 * q + 8 * kq);
        }
    };
    int strip = (int)blockIdx.x;
    if (strip < nstrips) load_strip(strip);

    // --- lhs of this super-block: lane (row c, quarter kq) holds a[c][256 blk + 32 s + 8 kq + 0..7], s = 0..7 ---
    half8 ahi[8], alo[PLANES == 2 ? kLoReg : 1];
    {
        float x[8][8];
        const AT* ar = a + (int64_t)min(c, m - 1) * lda + blk * 256 + kq * 8;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            if constexpr (sizeof(AT) == 4) {
                const float4 p = *(const float4*)(ar + s * 32), q = *(const float4*)(ar + s * 32 + 4);
                x[s][0] = p.x; x[s][1] = p.y; x[s][2] = p.z; x[s][3] = p.w;
                x[s][4] = q.x; x[s][5] = q.y; x[s][6] = q.z; x[s][7] = q.w;
            } else {
                const uint4 p = *(const uint4*)(ar + s * 32);
                x[s][0] = bf2f((uint16_t)p.x); x[s][1] = bf2f((uint16_t)(p.x >> 16));
                x[s][2] = bf2f((uint16_t)p.y); x[s][3] = bf2f((uint16_t)(p.y >> 16));
                x[s][4] = bf2f((uint16_t)p.z); x[s][5] = bf2f((uint16_t)(p.z >> 16));
                x[s][6] = bf2f((uint16_t)p.w); x[s][7] = bf2f((uint16_t)(p.w >> 16));
            }
        }
        const bool row_live = c < m;
        uint32_t mx = 0;
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                x[s][i] = row_live ? x[s][i] : 0.0f;
                mx = max(mx, __float_as_uint(x[s][i]) & 0x7fffffffu);
            }
        mx = max(mx, (uint32_t)__shfl_xor((int)mx, 16, kWave));
        mx = max(mx, (uint32_t)__shfl_xor((int)mx, 32, kWave));
        // scale = 2^(14 - exponent of the largest magnitude): the row lies below 2^15 (fp16 reaches 65504) and the
        // residuals stay normal fp16 numbers; a zero row keeps scale 1; a non-finite row stays non-finite
        const int e_max = (int)(mx >> 23);
        const int e_scale = mx == 0 ? 127 : min(max(268 - e_max, 1), 253);
        const float scale = __uint_as_float((uint32_t)e_scale << 23);
        const float inv_scale = __uint_as_float((uint32_t)(254 - e_scale) << 23);
#pragma unroll
        for (int s = 0; s < 8; s++) {
            // operand order of a step: registers (k0, k2), (k1, k3), (k4, k6), (k5, k7), the order in which one mask
            // takes the nibbles of bytes 0 and 2, then 1 and 3, of a quant dword
            const int o0[4] = {0, 1, 4, 5}, o1[4] = {2, 3, 6, 7};
            uint32_t hi[4], lo[4];
            float ssum = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float s0 = x[s][o0[v]] * scale, s1 = x[s][o1[v]] * scale;
                const _Float16 h0 = (_Float16)s0, h1 = (_Float16)s1;
                union { _Float16 h[2]; uint32_t u; } ph, pl;
                ph.h[0] = h0; ph.h[1] = h1;
                hi[v] = ph.u;
                pl.h[0] = (_Float16)(s0 - (float)h0); pl.h[1] = (_Float16)(s1 - (float)h1);
                lo[v] = pl.u;
                ssum += s0 + s1;
            }
            ahi[s] = pack4(hi[0], hi[1], hi[2], hi[3]);
            if constexpr (PLANES == 2) {
                if (s < kLoReg) alo[s] = pack4(lo[0], lo[1], lo[2], lo[3]);
                else lo_w[(s - kLoReg) * 64] = pack4(lo[0], lo[1], lo[2], lo[3]);
            }
            ssum += __shfl_xor(ssum, 16, kWave);
            ssum += __shfl_xor(ssum, 32, kWave);
            if (kq == 0) tr[s * 16 + c] = ssum;
        }
        if (kq == 0) tr[8 * 16 + c] = inv_scale;
        __syncthreads();
    }

    const uint32_t M1 = 0x03C003C0u;  // mantissa bits 6..9 of both fp16 halves
    for (; strip < nstrips; strip += (int)gridDim.x) {
        const int next = strip + (int)gridDim.x;
        const bool more = next < nstrips;  // uniform
        float acc[2][4];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint4 h = hdr[j];
            const uint32_t s3[3] = {h.y, h.z, h.w};
            const float d = h2f((uint16_t)(h.x & 0xffffu)) * 262144.0f, ndmin = -h2f((uint16_t)(h.x >> 16));
            float4v P = {0.f, 0.f, 0.f, 0.f}, R = {0.f, 0.f, 0.f, 0.f};
            float msum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 8; s++) {
                uint32_t sc, mn;
                q4k_scale_min(s, s3, sc, mn);
                const uint32_t sp = (uint32_t)f2h((float)sc) * 0x00010001u;  // (sc, sc)
                const uint2 q = qs[j][s >> 1];
                // nibbles of bytes 0 and 2, then 1 and 3, moved to bits 6..9 of the fp16 halves: q * 2^-18
                const half8 b = (s & 1) ? pack4(pk_mul((q.x << 2) & M1, sp), pk_mul((q.x >> 6) & M1, sp),
                                                pk_mul((q.y << 2) & M1, sp), pk_mul((q.y >> 6) & M1, sp))
                                        : pack4(pk_mul((q.x << 6) & M1, sp), pk_mul((q.x >> 2) & M1, sp),
                                                pk_mul((q.y << 6) & M1, sp), pk_mul((q.y >> 2) & M1, sp));
                P = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi[s], b, P, 0, 0, 0);
                if constexpr (PLANES == 2)
                    R = __builtin_amdgcn_mfma_f32_16x16x32_f16(s < kLoReg ? alo[s] : lo_w[(s - kLoReg) * 64], b, R, 0, 0, 0);
                const float4 as4 = *(const float4*)(tr + s * 16 + 4 * kq);  // sums of lhs rows 4 kq + 0..3 over sub-block s
                const float fm = (float)mn;
                msum[0] = fmaf(fm, as4.x, msum[0]);
                msum[1] = fmaf(fm, as4.y, msum[1]);
                msum[2] = fmaf(fm, as4.z, msum[2]);
                msum[3] = fmaf(fm, as4.w, msum[3]);
            }
            if constexpr (PLANES == 2) P += R;
#pragma unroll
            for (int r = 0; r < 4; r++) acc[j][r] = fmaf(d, P[r], ndmin * msum[r]);
        }
        if (more) load_strip(next);
        float* mine = park + wave * 512;
        const float4 iv4 = *(const float4*)(tr + 8 * 16 + 4 * kq);
        const float inv[4] = {iv4.x, iv4.y, iv4.z, iv4.w};
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) mine[(j * 4 + r) * 64 + lane] = blk_live ? acc[j][r] * inv[r] : 0.0f;
        __syncthreads();
        for (int t = tid; t < 512; t += (int)blockDim.x) {
            float v = 0.0f;
            for (int ww = 0; ww < nw; ww++) v += park[ww * 512 + t];
            const int j = t >> 8, r = (t >> 6) & 3, l = t & 63;
            const int row = 4 * (l >> 4) + r, col = strip * kStripRows + 16 * j + (l & 15);
            if (row < m && col < n) out[(int64_t)row * ldo + col] = v;
        }
        if (more) __syncthreads();  // the next strip's partial sums go to the same place
    }
}

}  // namespace

bool gemv_q4_k_kc_supported(const void* w, int64_t k) {
    return !kernel_disabled("q4k_kc") && k % 256 == 0 && ((uintptr_t)w & 15) == 0;
}

// Partial results of the K chunks (none up to K = 4096).
int64_t gemv_q4_k_kc_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    if (k % 256 || k <= (int64_t)kMaxWaves * 256) return 0;
    return (int64_t)kc_chunks(k).chunks * std::min<int64_t>(m, 16) * n * 4;
}

// 1..16 lhs rows; `workspace` holds gemv_q4_k_kc_workspace_bytes(m, n, k) bytes.
hipError_t launch_gemv_q4_k_kc(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                               int64_t ldo, void* workspace, hipStream_t s, bool* handled) {
    *handled = false;
    if (m < 1 || m > 16 || n < 1 || !gemv_q4_k_kc_supported(w, k)) return hipSuccess;
    if (a_dtype != QMM_F32 && a_dtype != QMM_BF16) return hipSuccess;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    const int nstrips = (int)((n + kStripRows - 1) / kStripRows), nblk = (int)(k / 256);
    const KcChunks cc = kc_chunks(k);
    if (cc.chunks > 1 && !workspace) return hipErrorInvalidValue;
    const int nw = cc.nw;
    const size_t lds = ((size_t)nw * 512 + (size_t)nw * 9 * 16) * sizeof(float) +
                       (a_dtype == QMM_F32 ? (size_t)nw * kLoLds * 64 * 16 : 0);
    const int per_cu = std::max(1, kMaxWaves / nw);
    const int64_t wgs_x = std::max<int64_t>(1, std::min<int64_t>(nstrips, (int64_t)cus * per_cu / cc.chunks));
    dim3 grid((unsigned)wgs_x, (unsigned)cc.chunks), block(64 * nw);
    float* dst = cc.chunks > 1 ? (float*)workspace : out;
    const int64_t dst_ld = cc.chunks > 1 ? n : ldo, chunk_stride = cc.chunks > 1 ? (int64_t)m * n : 0;
#define QMM_Q4K_KC(PL_, AT_)                                                                                          \
    do {                                                                                                              \
        if (lds > 64 * 1024) { /* (the limit is raised once, to the whole LDS: two host threads cannot interleave it) */ \
            hipError_t e_ = allow_full_lds<gemv_q4_k_kc_kernel<PL_, AT_>>();                                          \
            if (e_ != hipSuccess) return e_;                                                                          \
        }                                                                                                             \
        gemv_q4_k_kc_kernel<PL_, AT_><<<grid, block, lds, s>>>(w, (const AT_*)a, dst, m, (int)n, k, dst_ld, nstrips,  \
                                                               nblk, chunk_stride);                                   \
    } while (0)
    if (a_dtype == QMM_F32) QMM_Q4K_KC(2, float);
    else QMM_Q4K_KC(1, uint16_t);
#undef QMM_Q4K_KC
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (cc.chunks > 1) {
        const int64_t count = (int64_t)m * n;
        gemv_q4_k_kc_sum_kernel<<<dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s>>>((const float*)workspace, out, m,
                                                                                            (int)n, ldo, cc.chunks);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    *handled = true;
    return hipSuccess;
}

}  // namespace qmm
