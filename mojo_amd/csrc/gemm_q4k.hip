// Q4_K prefill kernel (m > 16 lhs rows): matrix-core GEMM over exact integer codes.
//
// Arithmetic.  As in the decode kernel, a masked nibble is the fp16 subnormal
// q*2^-24 and one packed fp16 multiply folds the 6-bit sub-block scale in
// (q*sc <= 945, exact).  lhs values are scaled per row by a power of two and
// narrowed to fp16 (exact for bf16 inputs of ordinary range), so every product
// inside v_mfma_f32_32x32x16_f16 is exact and the sums are fp32.  Per 256-wide
// super-block b the matrix cores produce P_b[m][n] = sum_k a[m][k]*(sc*q)[n][k];
// the fp32 super-block scale is applied in the lanes, acc += d[n,b] * P_b.  The
// min term  -sum_{b,j} (dmin*mn_j)[n] * (sum_{k in j} a[m][k])  is itself a matrix
// product over the 8 sub-blocks of a super-block: dmin*mn (17 bits) is split
// exactly into two fp16 values and the activation sums into hi + lo, and the two
// extra products per super-block accumulate straight into acc.
//
// A workgroup of 8 wavefronts computes a 128 x 256 output tile; wavefront
// (wm, wn) owns the 64 x 64 sub-tile at (64*wm, 64*wn).  lhs tiles go through
// LDS (double buffered, one 64-wide chunk per step); the packed weights are
// loaded by the lanes that use them and unpacked in registers.
#include <stdlib.h>

#include <type_traits>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int BM = 128, BN = 256;   // workgroup tile
constexpr int A_STRIDE = 72;        // halfs per LDS row of a 64-wide chunk (144 bytes: conflict-free b128 reads)
constexpr float kTwo24 = 16777216.0f;

}  // namespace

// ---------------------------------------------------------------------------
// main kernel
// ---------------------------------------------------------------------------
template <int NPART>
__global__ __launch_bounds__(512) void gemm_q4_k_kernel(const uint8_t* __restrict__ w, const _Float16* __restrict__ a16,
                                                        const _Float16* __restrict__ a16_lo,
                                                        const _Float16* __restrict__ asum,
                                                        const float* __restrict__ inv, float* __restrict__ out, int m,
                                                        int n, int k, int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(16))) _Float16 lds_a[2][NPART][BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 lds_s[BM * 16];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int nl = lane & 31, g = lane >> 5;
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;

    // Tile order: consecutive workgroup ids land on different XCDs, so give each XCD a
    // contiguous range of an order that keeps two lhs tile rows fixed while walking N.
    int tile_m, tile_n;
    {
        const int total = tiles_m * tiles_n;
        const int per_xcd = (total + 7) / 8;
        const int o = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
        if (o >= total) return;
        const int gm = 2, span = gm * tiles_n;
        const int grp = o / span, rem = o - grp * span;
        const int rows_here = min(gm, tiles_m - grp * gm);
        tile_n = rem / rows_here;
        tile_m = grp * gm + rem - tile_n * rows_here;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // lhs chunk loader: 128 rows x 64 halfs = 1024 x 16 bytes; 512 threads x 2.  Base pointers are
    // fixed per thread; a step only adds the chunk offset.  Two register sets (parity of the
    // step) keep two steps of loads in flight.
    const int nsteps = nblk * 4;
    const int a_row = tid >> 2, a_seg = tid & 3;
    const int64_t a_off = (int64_t)min(m0 + a_row, m - 1) * k + a_seg * 8;
    const uint4* a_base0 = (const uint4*)(a16 + a_off);
    const uint4* a_base1 = NPART == 2 ? (const uint4*)(a16_lo + a_off) : nullptr;
    // register sets as plain variables (set, part, segment)
    uint4 ax0_p0s0, ax0_p0s1, ax0_p1s0, ax0_p1s1, ax1_p0s0, ax1_p0s1, ax1_p1s0, ax1_p1s1;
    ax0_p1s0 = ax0_p1s1 = ax1_p1s0 = ax1_p1s1 = make_uint4(0, 0, 0, 0);
    _Float16* a_dst = &lds_a[0][0][a_row * A_STRIDE + a_seg * 8];
#define QMM_A_LOAD(SET, STEP)                                         \
    do {                                                              \
        const int chunk_ = min((STEP), nsteps - 1);                   \
        SET##_p0s0 = a_base0[chunk_ * 8];                             \
        SET##_p0s1 = a_base0[chunk_ * 8 + 4];                         \
        if constexpr (NPART == 2) {                                   \
            SET##_p1s0 = a_base1[chunk_ * 8];                         \
            SET##_p1s1 = a_base1[chunk_ * 8 + 4];                     \
        }                                                             \
    } while (0)
#define QMM_A_STORE(SET, BUF)                                                     \
    do {                                                                          \
        _Float16* d_ = a_dst + (size_t)(BUF) * NPART * BM * A_STRIDE;             \
        *(uint4*)d_ = SET##_p0s0;                                                 \
        *(uint4*)(d_ + 32) = SET##_p0s1;                                          \
        if constexpr (NPART == 2) {                                               \
            *(uint4*)(d_ + BM * A_STRIDE) = SET##_p1s0;                           \
            *(uint4*)(d_ + BM * A_STRIDE + 32) = SET##_p1s1;                      \
        }                                                                         \
    } while (0)

    // this lane's two weight columns
    const uint8_t* wcol0 = w + (int64_t)min(n0 + wn * 64 + nl, n - 1) * row_bytes;
    const uint8_t* wcol1 = w + (int64_t)min(n0 + wn * 64 + 32 + nl, n - 1) * row_bytes;
    const int q_lane_off = 16 + 16 * g;

    float16v acc[2][2], P[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc[mi][ni][r] = 0.0f;
                P[mi][ni][r] = 0.0f;
            }

    uint4 qx0_c0, qx0_c1, qx1_c0, qx1_c1;  // code units of the two columns, two register sets
#define QMM_Q_LOAD(SET, STEP)                                                              \
    do {                                                                                   \
        const int st_ = min((STEP), nsteps - 1);                                           \
        const int off_ = (st_ >> 2) * Q4_K_BPB + 32 * (st_ & 3) + q_lane_off;              \
        SET##_c0 = *(const uint4*)(wcol0 + off_);                                          \
        SET##_c1 = *(const uint4*)(wcol1 + off_);                                          \
    } while (0)

    // block headers and sub-block sums are fetched one super-block ahead
    uint4 hdr_n0, hdr_n1, as_n = make_uint4(0, 0, 0, 0);
    const uint4* as_src = (const uint4*)(asum + (int64_t)min(m0 + (tid >> 1), m - 1) * nblk * 16 + (tid & 1) * 8);
    auto hdr_prefetch = [&](int blk) {
        const int bc = min(blk, nblk - 1);
        hdr_n0 = *(const uint4*)(wcol0 + bc * Q4_K_BPB);
        hdr_n1 = *(const uint4*)(wcol1 + bc * Q4_K_BPB);
    };
    auto as_prefetch = [&](int blk) {
        if (tid < 256) as_n = as_src[min(blk, nblk - 1) * 2];
    };
    hdr_prefetch(0);
    as_prefetch(0);
    QMM_A_LOAD(ax0, 0);
    QMM_Q_LOAD(qx0, 0);
    QMM_Q_LOAD(qx1, 1);
    QMM_A_STORE(ax0, 0);
    if (tid < 256) *(uint4*)(&lds_s[(tid >> 1) * 16 + (tid & 1) * 8]) = as_n;
    QMM_A_LOAD(ax1, 1);
    QMM_A_LOAD(ax0, 2);
    as_prefetch(1);
    __syncthreads();

    float dscale[2] = {0.f, 0.f};
    uint32_t sp[2][8];
    // One step = one 64-wide chunk c of super-block blk.  The chunk index is a compile-time
    // constant so that register arrays and the parity-selected prefetch sets stay in registers.
    auto do_step = [&](int blk, auto CC) {
        constexpr int c = decltype(CC)::value;
        const int step = blk * 4 + c, buf = c & 1;
        uint4 qc0, qc1;
        if constexpr (c & 1) {
            qc0 = qx1_c0; qc1 = qx1_c1;
            QMM_Q_LOAD(qx1, step + 2);
        } else {
            qc0 = qx0_c0; qc1 = qx0_c1;
            QMM_Q_LOAD(qx0, step + 2);
        }
        if (c == 0) {
            // ---- super-block start: header decode, min-term products (sums already in lds_s)
            const uint4 hdr_c0 = hdr_n0, hdr_c1 = hdr_n1;
            hdr_prefetch(blk + 1);
            uint32_t dmn_hi[2][4], dmn_lo[2][4];
#pragma unroll
            for (int ni = 0; ni < 2; ni++) {
                const uint4 hdr = ni == 0 ? hdr_c0 : hdr_c1;
                dscale[ni] = h2f((uint16_t)(hdr.x & 0xffffu)) * kTwo24;
                const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
                const uint32_t sc_lo = s0 & 0x3F3F3F3Fu, sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
                const uint32_t mn_lo = s1 & 0x3F3F3F3Fu, mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
                const float e0 = (float)(sc_lo & 0xffu), e1 = 0.0625f * (float)((sc_lo >> 8) & 0xffu);
                const float e2 = (float)((sc_lo >> 16) & 0xffu), e3 = 0.0625f * (float)(sc_lo >> 24);
                const float e4 = (float)(sc_hi & 0xffu), e5 = 0.0625f * (float)((sc_hi >> 8) & 0xffu);
                const float e6 = (float)((sc_hi >> 16) & 0xffu), e7 = 0.0625f * (float)(sc_hi >> 24);
                sp[ni][0] = pack_half2(e0, e0); sp[ni][1] = pack_half2(e1, e1);
                sp[ni][2] = pack_half2(e2, e2); sp[ni][3] = pack_half2(e3, e3);
                sp[ni][4] = pack_half2(e4, e4); sp[ni][5] = pack_half2(e5, e5);
                sp[ni][6] = pack_half2(e6, e6); sp[ni][7] = pack_half2(e7, e7);
                // -(dmin * mn_j) as exact fp16 hi + lo, sub-blocks (0,1) (2,3) (4,5) (6,7)
                const uint32_t ndm = ((hdr.x >> 16) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
                const uint32_t mp[4] = {
                    pack_half2((float)(mn_lo & 0xffu), (float)((mn_lo >> 8) & 0xffu)),
                    pack_half2((float)((mn_lo >> 16) & 0xffu), (float)(mn_lo >> 24)),
                    pack_half2((float)(mn_hi & 0xffu), (float)((mn_hi >> 8) & 0xffu)),
                    pack_half2((float)((mn_hi >> 16) & 0xffu), (float)(mn_hi >> 24))};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    dmn_hi[ni][i] = pk_mul(ndm, mp[i]);
                    dmn_lo[ni][i] = pk_fma(ndm, mp[i], dmn_hi[ni][i] ^ 0x80008000u);
                }
            }
#pragma unroll
            for (int mi = 0; mi < 2; mi++) {
                // A operand: lanes g=0 carry the hi parts of the 8 sub-block sums, g=1 the lo parts
                const half8 av = *(const half8*)(&lds_s[(wm * 64 + mi * 32 + nl) * 16 + g * 8]);
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        av, pack4(dmn_hi[ni][0], dmn_hi[ni][1], dmn_hi[ni][2], dmn_hi[ni][3]), acc[mi][ni], 0, 0, 0);
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        av, pack4(dmn_lo[ni][0], dmn_lo[ni][1], dmn_lo[ni][2], dmn_lo[ni][3]), acc[mi][ni], 0, 0, 0);
                }
            }
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
#pragma unroll
                    for (int r = 0; r < 16; r++) P[mi][ni][r] = 0.0f;
        }

        // ---- one 64-wide chunk: four 16-wide operand slices
        const uint32_t M1 = 0x000F000Fu, M2 = 0x00F000F0u;
#pragma unroll
        for (int f = 0; f < 4; f++) {
            half8 bfrag[2];
#pragma unroll
            for (int ni = 0; ni < 2; ni++) {
                const uint4 qq = ni == 0 ? qc0 : qc1;
                const uint32_t x0 = (f & 1) ? qq.z : qq.x, x1 = (f & 1) ? qq.w : qq.y;
                const uint32_t mask = (f & 2) ? M2 : M1;
                const uint32_t s = sp[ni][2 * c + (f >> 1)];
                bfrag[ni] = pack4(pk_mul(x0 & mask, s), pk_mul((x0 >> 8) & mask, s), pk_mul(x1 & mask, s),
                                  pk_mul((x1 >> 8) & mask, s));
            }
#pragma unroll
            for (int p = 0; p < NPART; p++) {
#pragma unroll
                for (int mi = 0; mi < 2; mi++) {
                    const half8 afrag = *(const half8*)(&lds_a[buf][p][(wm * 64 + mi * 32 + nl) * A_STRIDE + f * 16 + g * 8]);
#pragma unroll
                    for (int ni = 0; ni < 2; ni++)
                        P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag[ni], P[mi][ni], 0, 0, 0);
                }
            }
        }
        // Ask the scheduler to interleave the unpack arithmetic with the matrix-core instructions
        // (one MFMA, then a group of vector ALU ops), so the two pipes run concurrently inside a
        // wavefront instead of in two phases.
#pragma unroll
        for (int i = 0; i < 16; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);  // 6 VALU
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 LDS read
        }
        if (c == 3) {
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[mi][ni][r] = fmaf(dscale[ni], P[mi][ni][r], acc[mi][ni][r]);
        }
        // next step's lhs chunk to the other LDS buffer; its register set then takes the loads of step + 3
        if constexpr (c & 1) {
            QMM_A_STORE(ax0, buf ^ 1);
            QMM_A_LOAD(ax0, step + 3);
        } else {
            QMM_A_STORE(ax1, buf ^ 1);
            QMM_A_LOAD(ax1, step + 3);
        }
        if (c == 3) {  // next super-block's sub-block sums
            if (tid < 256) *(uint4*)(&lds_s[(tid >> 1) * 16 + (tid & 1) * 8]) = as_n;
            as_prefetch(blk + 2);
        }
        __syncthreads();
    };
    for (int blk = 0; blk < nblk; blk++) {
        do_step(blk, std::integral_constant<int, 0>{});
        do_step(blk, std::integral_constant<int, 1>{});
        do_step(blk, std::integral_constant<int, 2>{});
        do_step(blk, std::integral_constant<int, 3>{});
    }

#undef QMM_A_LOAD
#undef QMM_A_STORE
#undef QMM_Q_LOAD
    // ---- epilogue: undo the row scale, store
#pragma unroll
    for (int mi = 0; mi < 2; mi++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
            if (row < m) {
                const float is = inv[row];
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    const int col = n0 + wn * 64 + ni * 32 + nl;
                    if (col < n) out[(int64_t)row * n + col] = acc[mi][ni][r] * is;
                }
            }
        }
    }
}

int64_t gemm_q4_k_workspace_bytes(int lhs_dtype, int64_t m, int64_t k) { return lhs_planes(nullptr, lhs_dtype, m, k).bytes; }

hipError_t launch_gemm_q4_k(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                            float* out, void* workspace, hipStream_t s) {
    // QMM_Q4K_GEMM=w4 selects the 4-wavefront kernel; the default is this file's 8-wavefront one.
    static const bool use_w4 = [] {
        const char* v = getenv("QMM_Q4K_GEMM");
        return v && v[0] == 'w' && v[1] == '4';
    }();
    if (use_w4) return launch_gemm_q4_k_w4(lhs, lhs_dtype, w, m, n, k, out, workspace, s);
    const LhsPlanes p = lhs_planes(workspace, lhs_dtype, m, k);
    hipError_t e = launch_prep_lhs<kLhsOrderQ4K>(lhs, lhs_dtype, m, k, p, s);
    if (e != hipSuccess) return e;
    const int tiles_m = (int)((m + BM - 1) / BM), tiles_n = (int)((n + BN - 1) / BN);
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    dim3 grid((unsigned)(per_xcd * 8)), block(512);
    if (lhs_dtype == QMM_F32)
        gemm_q4_k_kernel<2><<<grid, block, 0, s>>>(w, p.a16, p.a16_lo, p.asum, p.inv, out, (int)m, (int)n, (int)k, tiles_m, tiles_n);
    else
        gemm_q4_k_kernel<1><<<grid, block, 0, s>>>(w, p.a16, nullptr, p.asum, p.inv, out, (int)m, (int)n, (int)k, tiles_m, tiles_n);
    return hipGetLastError();
}

}  // namespace qmm
