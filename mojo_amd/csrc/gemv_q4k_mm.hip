// Q4_K small-batch kernel (3 <= m <= 16 lhs rows): weight rows streamed through LDS, 16 x 16 x 32
// matrix-core products over exact integer codes.
//
// Arithmetic is that of the prefill kernel (gemm_q4k.hip): a masked nibble is the fp16 subnormal
// q*2^-24, one packed fp16 multiply folds the 6-bit sub-block scale in, the lhs is narrowed to fp16
// (hi, plus a residual plane for fp32 input) after an exact per-row power-of-two scaling, the fp32
// super-block scale is applied in the lanes and the min term is one extra matrix product per
// super-block (K = 32 slots hold  asum_hi x dmn_hi,  asum_lo x dmn_hi,  asum_hi x dmn_lo).
//
// Shape of the work: a workgroup of 8 wavefronts walks a list of 16-row weight tiles.  Wavefront w
// owns super-blocks 2w, 2w + 1 of the current group of 16 super-blocks (4096 columns): its lhs
// fragments for those two super-blocks (16 lhs rows, hi and residual planes) are loaded into
// registers once per group and reused for every tile of the workgroup, so the lhs traffic is
// amortised over the tiles (loading them per tile made the lhs planes, not the weights, the bulk
// of the traffic).  For a tile, the wavefront copies its two super-blocks of the 16 rows into
// private LDS with 16-byte loads (288 contiguous bytes per row; the next tile's loads are issued
// before the current one is decoded), each lane (row n = lane % 16, k-group lane / 16) reads its 8
// code bytes of a 64-wide chunk with one ds_read_b64 and they serve two matrix-core instructions,
// the low nibbles (sub-block 2c) and the high nibbles (sub-block 2c + 1).  The 8 partial results of
// a tile are added through LDS and accumulated over the groups of K in a per-tile LDS slot.
#include <stdlib.h>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

typedef float float4v __attribute__((ext_vector_type(4)));

namespace {

constexpr int kRunBlk = 2;                      // super-blocks per staged run
constexpr int kRowStride = 304;                 // LDS bytes per row: 288 + 16 (conflict-free ds_read_b64 / b128)
constexpr int kWaveBytes = 16 * kRowStride;     // 4864
constexpr float kTwo24f = 16777216.0f;
constexpr int kWaves = 8;                       // wavefronts per workgroup: two super-blocks each per group of 16
constexpr int kMaxTiles = 8;                    // tiles per workgroup (LDS slots for their results)

}  // namespace

template <int NPART>
__global__ __launch_bounds__(512) void gemv_q4_k_mm_kernel(const uint8_t* __restrict__ w, const _Float16* __restrict__ a16,
                                                           const _Float16* __restrict__ a16_lo,
                                                           const _Float16* __restrict__ asum, const float* __restrict__ inv,
                                                           float* __restrict__ out, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int nn = lane & 15, kg = lane >> 4;
    uint8_t* wbuf = smem + wave * kWaveBytes;
    float* red = (float*)(smem + kWaves * kWaveBytes);  // [kWaves][4][64]
    float* tot = red + kWaves * 4 * 64;                 // [kMaxTiles][4][64]
    const int ntiles = (n + 15) >> 4;
    const int my_tiles = (int)blockIdx.x < ntiles ? (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;

    // staging pieces: piece p = lane + 64 i of a tile: row p / 18, 16-byte piece p % 18 (288 pieces, 4.5 per lane)
    int prow[5], pidx[5];
#pragma unroll
    for (int i = 0; i < 5; i++) {
        const int p = min(lane + 64 * i, 16 * 18 - 1);
        prow[i] = p / 18;
        pidx[i] = p - prow[i] * 18;
    }
    const int mrow = min(nn, m - 1);  // lhs row whose fragments this lane holds (rows >= m repeat the last one)
    const _Float16* a_hi = a16 + (int64_t)mrow * k + 8 * kg;
    const _Float16* a_lo = NPART == 2 ? a16_lo + (int64_t)mrow * k + 8 * kg : nullptr;
    const _Float16* as_row = asum + (int64_t)mrow * nblk * 16 + (kg & 1) * 8;
    const uint32_t M1 = 0x000F000Fu, M2 = 0x00F000F0u;

    const int ngrp = (nblk + 2 * kWaves - 1) / (2 * kWaves);
    for (int grp = 0; grp < ngrp; grp++) {
        const int b0 = grp * 2 * kWaves + 2 * wave;       // this wavefront's two super-blocks of the group
        const int nb = max(0, min(kRunBlk, nblk - b0));
        // lhs fragments and sub-block sums of those super-blocks: registers, reused for every tile
        half8 fa[kRunBlk][8][NPART], fs[kRunBlk];
#pragma unroll
        for (int bb = 0; bb < kRunBlk; bb++) {
            const int blk = min(b0 + bb, nblk - 1);
            fs[bb] = *(const half8*)(as_row + (int64_t)blk * 16);
#pragma unroll
            for (int sl = 0; sl < 8; sl++) {
                fa[bb][sl][0] = *(const half8*)(a_hi + (int64_t)blk * 256 + 32 * sl);
                if constexpr (NPART == 2) fa[bb][sl][1] = *(const half8*)(a_lo + (int64_t)blk * 256 + 32 * sl);
            }
        }
        uint4 r0, r1, r2, r3, r4;
#define QMM_STAGE_LOAD(TILE)                                                                                          \
    do {                                                                                                              \
        const int n0_ = min((TILE), ntiles - 1) * 16, bc_ = min(b0, nblk - 1), np_ = max(nb, 1) * 9 - 1;              \
        const uint8_t* base_ = w + (int64_t)bc_ * Q4_K_BPB;                                                           \
        r0 = ((const uint4*)(base_ + (int64_t)min(n0_ + prow[0], n - 1) * row_bytes))[min(pidx[0], np_)];             \
        r1 = ((const uint4*)(base_ + (int64_t)min(n0_ + prow[1], n - 1) * row_bytes))[min(pidx[1], np_)];             \
        r2 = ((const uint4*)(base_ + (int64_t)min(n0_ + prow[2], n - 1) * row_bytes))[min(pidx[2], np_)];             \
        r3 = ((const uint4*)(base_ + (int64_t)min(n0_ + prow[3], n - 1) * row_bytes))[min(pidx[3], np_)];             \
        r4 = ((const uint4*)(base_ + (int64_t)min(n0_ + prow[4], n - 1) * row_bytes))[min(pidx[4], np_)];             \
    } while (0)
        QMM_STAGE_LOAD((int)blockIdx.x);
        for (int ti = 0; ti < my_tiles; ti++) {
            const int tile = (int)blockIdx.x + ti * (int)gridDim.x;
            __builtin_amdgcn_wave_barrier();  // the previous tile's LDS reads are issued (LDS is in order per wavefront)
            *(uint4*)(wbuf + prow[0] * kRowStride + pidx[0] * 16) = r0;
            *(uint4*)(wbuf + prow[1] * kRowStride + pidx[1] * 16) = r1;
            *(uint4*)(wbuf + prow[2] * kRowStride + pidx[2] * 16) = r2;
            *(uint4*)(wbuf + prow[3] * kRowStride + pidx[3] * 16) = r3;
            if (lane + 256 < 16 * 18) *(uint4*)(wbuf + prow[4] * kRowStride + pidx[4] * 16) = r4;
            QMM_STAGE_LOAD(tile + (int)gridDim.x);  // next tile (past the last: a harmless repeat)
            __builtin_amdgcn_wave_barrier();

            float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int bb = 0; bb < kRunBlk; bb++) {
                if (bb >= nb) break;
                const uint8_t* lb = wbuf + nn * kRowStride + bb * Q4_K_BPB;
                const uint4 hdr = *(const uint4*)lb;
                // 6-bit scales and mins of the 8 sub-blocks
                const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
                const uint32_t sc_lo = s0 & 0x3F3F3F3Fu, sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
                const uint32_t mn_lo = s1 & 0x3F3F3F3Fu, mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
                uint32_t sp[8];
                {
                    const float e0 = (float)(sc_lo & 0xffu), e1 = 0.0625f * (float)((sc_lo >> 8) & 0xffu);
                    const float e2 = (float)((sc_lo >> 16) & 0xffu), e3 = 0.0625f * (float)(sc_lo >> 24);
                    const float e4 = (float)(sc_hi & 0xffu), e5 = 0.0625f * (float)((sc_hi >> 8) & 0xffu);
                    const float e6 = (float)((sc_hi >> 16) & 0xffu), e7 = 0.0625f * (float)(sc_hi >> 24);
                    sp[0] = pack_half2(e0, e0); sp[1] = pack_half2(e1, e1);
                    sp[2] = pack_half2(e2, e2); sp[3] = pack_half2(e3, e3);
                    sp[4] = pack_half2(e4, e4); sp[5] = pack_half2(e5, e5);
                    sp[6] = pack_half2(e6, e6); sp[7] = pack_half2(e7, e7);
                }
                // min term: B slots (k-group 0,1: hi parts, 2: lo parts) of -(dmin*mn_j), A slots asum hi / lo
                {
                    const uint32_t ndm = ((hdr.x >> 16) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
                    const uint32_t mp[4] = {pack_half2((float)(mn_lo & 0xffu), (float)((mn_lo >> 8) & 0xffu)),
                                            pack_half2((float)((mn_lo >> 16) & 0xffu), (float)(mn_lo >> 24)),
                                            pack_half2((float)(mn_hi & 0xffu), (float)((mn_hi >> 8) & 0xffu)),
                                            pack_half2((float)((mn_hi >> 16) & 0xffu), (float)(mn_hi >> 24))};
                    uint32_t v[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const uint32_t hi = pk_mul(ndm, mp[i]);
                        const uint32_t lo = pk_fma(ndm, mp[i], hi ^ 0x80008000u);
                        v[i] = kg < 2 ? hi : (kg == 2 ? lo : 0u);  // slots 24..31 (asum_lo x dmn_lo) are dropped
                    }
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(fs[bb], pack4(v[0], v[1], v[2], v[3]), acc, 0, 0, 0);
                }
                float4v P = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const uint2 q = *(const uint2*)(lb + 16 + 32 * c + 8 * kg);
                    const uint32_t x0 = q.x, x1 = q.y, y0 = q.x >> 8, y1 = q.y >> 8;
                    const half8 blo = pack4(pk_mul(x0 & M1, sp[2 * c]), pk_mul(y0 & M1, sp[2 * c]),
                                            pk_mul(x1 & M1, sp[2 * c]), pk_mul(y1 & M1, sp[2 * c]));
                    const half8 bhi = pack4(pk_mul(x0 & M2, sp[2 * c + 1]), pk_mul(y0 & M2, sp[2 * c + 1]),
                                            pk_mul(x1 & M2, sp[2 * c + 1]), pk_mul(y1 & M2, sp[2 * c + 1]));
                    P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c][0], blo, P, 0, 0, 0);
                    P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c + 1][0], bhi, P, 0, 0, 0);
                    if constexpr (NPART == 2) {
                        P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c][1], blo, P, 0, 0, 0);
                        P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c + 1][1], bhi, P, 0, 0, 0);
                    }
                }
                const float dsc = h2f((uint16_t)(hdr.x & 0xffffu)) * kTwo24f;
#pragma unroll
                for (int r = 0; r < 4; r++) acc[r] = fmaf(dsc, P[r], acc[r]);
            }
            // add the 8 wavefronts' shares of this tile and accumulate over the groups of K
#pragma unroll
            for (int r = 0; r < 4; r++) red[(wave * 4 + r) * 64 + lane] = acc[r];
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float v = 0.0f;
#pragma unroll
                    for (int ww = 0; ww < kWaves; ww++) v += red[(ww * 4 + r) * 64 + lane];
                    float* t = tot + (ti * 4 + r) * 64 + lane;
                    *t = grp == 0 ? v : *t + v;
                }
            }
            __syncthreads();
        }
#undef QMM_STAGE_LOAD
    }
    // lane holds lhs rows 4 kg + r of weight row 16 tile + nn
    if (wave == 0) {
        for (int ti = 0; ti < my_tiles; ti++) {
            const int col = ((int)blockIdx.x + ti * (int)gridDim.x) * 16 + nn;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = 4 * kg + r;
                if (row < m && col < n) out[(int64_t)row * n + col] = tot[(ti * 4 + r) * 64 + lane] * inv[row];
            }
        }
    }
}

int64_t gemv_q4_k_mm_workspace_bytes(int lhs_dtype, int64_t m, int64_t k) { return lhs_planes(nullptr, lhs_dtype, m, k).bytes; }

hipError_t launch_gemv_q4_k_mm(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                               float* out, void* workspace, hipStream_t s) {
    const LhsPlanes p = lhs_planes(workspace, lhs_dtype, m, k);
    hipError_t e = launch_prep_lhs<kLhsOrderQ4K16>(lhs, lhs_dtype, m, k, p, s);
    if (e != hipSuccess) return e;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    const int64_t ntiles = (n + 15) / 16;
    // one workgroup per compute unit when that leaves each at most kMaxTiles tiles, more otherwise
    int64_t wgs = cus;
    if (wgs * kMaxTiles < ntiles) wgs = (ntiles + kMaxTiles - 1) / kMaxTiles;
    if (wgs > ntiles) wgs = ntiles;
    const size_t lds = (size_t)kWaves * kWaveBytes + (size_t)(kWaves + kMaxTiles) * 4 * 64 * 4;
    dim3 grid((unsigned)wgs), block(64 * kWaves);
    if (p.a16_lo)
        gemv_q4_k_mm_kernel<2><<<grid, block, lds, s>>>(w, p.a16, p.a16_lo, p.asum, p.inv, out, (int)m, (int)n, (int)k);
    else
        gemv_q4_k_mm_kernel<1><<<grid, block, lds, s>>>(w, p.a16, nullptr, p.asum, p.inv, out, (int)m, (int)n, (int)k);
    return hipGetLastError();
}

}  // namespace qmm
