// GPTQ (4-bit, AutoGPTQ v1 packing) prefill kernel for m > 16 lhs rows: the same
// matrix-core scheme as the Q4_K prefill kernel, on the [K/8, N] int32 layout.
//
// A packed dword holds 8 consecutive k of one output column.  With the lhs stored in
// the order (0,4,1,5,2,6,3,7) inside each 8-group and its odd columns pre-multiplied
// by 1/16, the four fp16 pairs  x & 0x000F000F,  x & 0x00F000F0,  (x>>8) & 0x000F000F,
// (x>>8) & 0x00F000F0  are the matrix-core B operand directly: fp16 subnormals q*2^-24
// (or 16q*2^-24), no multiply needed because the scale is per group, not per 32.
// The matrix core does not normalise subnormal inputs before it aligns the products of a
// step, and the low bits of long products then fall off the end of the adder, always towards
// minus infinity: with non-negative codes a bias that grows with K.  With unit-size
// activations at K = 14336 it is 1.5e-5 for a bf16 lhs (short products).  For an fp32 lhs it
// was 2e-4 with the main and the residual plane in one launch; now each plane is a launch of
// its own (the residual plane's small products no longer sit next to the main plane's large
// sums) and the nibbles are moved two bits up inside the subnormal's mantissa (x << 2 and
// x >> 6, masks shifted likewise: q*2^-22), which leaves 6e-6.
// Per group g the matrix cores produce  P[m][n] = sum_k a[m][k]*q[k][n]  exactly (fp32
// sums), and the lanes apply  acc += scale[g][n] * P.  The zero-point term
// -scale*zero * sum_k a[m][k]  is a second small matrix product over the 32-wide
// sub-block sums of a 256-column chunk, with scale*zero split exactly into two fp16
// values; zero = stored + 1 (AutoGPTQ v1 convention).
//
// Tile shape and data movement as in the Q4_K kernel: 128 x 256 outputs per workgroup of
// 8 wavefronts, lhs chunks through double-buffered LDS, weights loaded by the lanes that
// use them (a wavefront load covers 32 consecutive columns of two k8 rows: 128-byte runs).
#include <stdlib.h>

#include <algorithm>

#include <type_traits>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int BM = 128, BN = 256;
constexpr int A_STRIDE = 72;
constexpr float kTwo24 = 16777216.0f, kTwo22 = 4194304.0f;

}  // namespace

// GB = groups per 256-column chunk (group size 256 / GB: 256, 128 or 64).
// One launch multiplies one fp16 plane of the lhs (`a16`) with the weights.  `with_zero` adds the zero-point term (it
// uses the full-precision sub-block sums, so it belongs to exactly one launch); `accumulate` adds the result to
// what `out` already holds (second launch of an fp32 lhs: its residual plane, with accumulators of its own: next to
// the large sums of the main plane the small residual products would lose their low bits inside the matrix core).
// UP: how many bits the nibbles are moved up inside the fp16 halves (2 for an fp32 lhs, 0 for a bf16 lhs).
template <int UP, int GB, bool with_zero, bool accumulate>
__global__ __launch_bounds__(512) void gemm_gptq_kernel(const uint32_t* __restrict__ qweight,
                                                        const uint16_t* __restrict__ scales,
                                                        const uint32_t* __restrict__ qzeros,
                                                        const _Float16* __restrict__ a16,
                                                        const _Float16* __restrict__ asum, const float* __restrict__ inv,
                                                        float* __restrict__ out, int m, int n, int k, int tiles_m,
                                                        int tiles_n, int ksplit) {
    __shared__ __attribute__((aligned(16))) _Float16 lds_a[2][BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 lds_s[BM * 16];
    __shared__ __attribute__((aligned(16))) float lds_inv[BM];
    constexpr int SPG = 4 / GB;  // 64-wide steps per group

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int nl = lane & 31, g = lane >> 5;
    const int nblk_row = k >> 8;  // 256-column blocks of a whole row

    // A work unit is a tile's share of K: blocks [kb0, kb0 + nblk); with ksplit > 1 its result goes to slice ks of `out`, then
    // a [ksplit][m][n] buffer that a later launch adds up.  Every pointer below is moved to the share's first block.
    int tile_m, tile_n, kb0, nblk;
    {
        const int total = tiles_m * tiles_n * ksplit;
        const int per_xcd = (total + 7) / 8;
        const int u = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
        if (u >= total) return;
        const int o = u / ksplit, ks = u - o * ksplit;
        kb0 = ks * nblk_row / ksplit;
        nblk = (ks + 1) * nblk_row / ksplit - kb0;
        out += (int64_t)ks * m * n;
        const int gm = 2, span = gm * tiles_n;
        const int grp = o / span, rem = o - grp * span;
        const int rows_here = min(gm, tiles_m - grp * gm);
        tile_n = rem / rows_here;
        tile_m = grp * gm + rem - tile_n * rows_here;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    a16 += (int64_t)kb0 * 256;
    qweight += (int64_t)kb0 * 32 * n;
    scales += (int64_t)kb0 * GB * n;
    qzeros += (int64_t)kb0 * GB * (n >> 3);

    const int nsteps = nblk * 4;
    const int a_row = tid >> 2, a_seg = tid & 3;
    const int64_t a_off = (int64_t)min(m0 + a_row, m - 1) * k + a_seg * 8;
    const uint4* a_base0 = (const uint4*)(a16 + a_off);
    uint4 ax0_p0s0, ax0_p0s1, ax1_p0s0, ax1_p0s1;
    _Float16* a_dst = &lds_a[0][a_row * A_STRIDE + a_seg * 8];
#define QMM_A_LOAD(SET, STEP)                                         \
    do {                                                              \
        const int chunk_ = min((STEP), nsteps - 1);                   \
        SET##_p0s0 = a_base0[chunk_ * 8];                             \
        SET##_p0s1 = a_base0[chunk_ * 8 + 4];                         \
    } while (0)
#define QMM_A_STORE(SET, BUF)                                                     \
    do {                                                                          \
        _Float16* d_ = a_dst + (size_t)(BUF) * BM * A_STRIDE;                     \
        *(uint4*)d_ = SET##_p0s0;                                                 \
        *(uint4*)(d_ + 32) = SET##_p0s1;                                          \
    } while (0)

    // this lane's two weight columns; the lane half g takes the odd k8 rows
    const int col0 = min(n0 + wn * 64 + nl, n - 1), col1 = min(n0 + wn * 64 + 32 + nl, n - 1);
    // Loads are written as (wave-uniform pointer)[per-lane 32-bit offset] so that the address
    // arithmetic stays in scalar registers.
    const int64_t ldq = n;  // dwords per k8 row
    const int qoff0 = g * n + col0, qoff1 = g * n + col1;

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

    // code dwords of the two columns (4 k8 rows each), two register sets
    uint32_t qx0_a0, qx0_a1, qx0_a2, qx0_a3, qx0_b0, qx0_b1, qx0_b2, qx0_b3;
    uint32_t qx1_a0, qx1_a1, qx1_a2, qx1_a3, qx1_b0, qx1_b1, qx1_b2, qx1_b3;
#define QMM_Q_LOAD(SET, STEP)                                                       \
    do {                                                                            \
        const uint32_t* r_ = qweight + (int64_t)min((STEP), nsteps - 1) * 8 * ldq;  \
        SET##_a0 = r_[qoff0];                                                       \
        SET##_a1 = (r_ + 2 * ldq)[qoff0];                                           \
        SET##_a2 = (r_ + 4 * ldq)[qoff0];                                           \
        SET##_a3 = (r_ + 6 * ldq)[qoff0];                                           \
        SET##_b0 = r_[qoff1];                                                       \
        SET##_b1 = (r_ + 2 * ldq)[qoff1];                                           \
        SET##_b2 = (r_ + 4 * ldq)[qoff1];                                           \
        SET##_b3 = (r_ + 6 * ldq)[qoff1];                                           \
    } while (0)

    // group scales and zero words of the next 256-column chunk
    uint32_t sc_n[2][GB], zw_n[2][GB];
    const int zshift0 = 4 * (col0 & 7), zshift1 = 4 * (col1 & 7);
    const int ldz = n >> 3, zcol0 = col0 >> 3, zcol1 = col1 >> 3;
    auto hdr_prefetch = [&](int blk) {
        const int64_t g0 = (int64_t)min(blk, nblk - 1) * GB;
#pragma unroll
        for (int i = 0; i < GB; i++) {
            const uint16_t* sr = scales + (g0 + i) * n;
            const uint32_t* zr = qzeros + (g0 + i) * ldz;
            sc_n[0][i] = sr[col0];
            sc_n[1][i] = sr[col1];
            zw_n[0][i] = zr[zcol0];
            zw_n[1][i] = zr[zcol1];
        }
    };
    uint4 as_n = make_uint4(0, 0, 0, 0);
    const uint4* as_src = (const uint4*)(asum + ((int64_t)min(m0 + (tid >> 1), m - 1) * nblk_row + kb0) * 16 + (tid & 1) * 8);
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
    if (tid < BM) lds_inv[tid] = inv[min(m0 + tid, m - 1)];
    __syncthreads();

    float gscale[2][GB];
    auto do_step = [&](int blk, auto CC) {
        constexpr int c = decltype(CC)::value;
        const int step = blk * 4 + c, buf = c & 1;
        uint32_t qa[4], qb[4];
        if constexpr (c & 1) {
            qa[0] = qx1_a0; qa[1] = qx1_a1; qa[2] = qx1_a2; qa[3] = qx1_a3;
            qb[0] = qx1_b0; qb[1] = qx1_b1; qb[2] = qx1_b2; qb[3] = qx1_b3;
            QMM_Q_LOAD(qx1, step + 2);
        } else {
            qa[0] = qx0_a0; qa[1] = qx0_a1; qa[2] = qx0_a2; qa[3] = qx0_a3;
            qb[0] = qx0_b0; qb[1] = qx0_b1; qb[2] = qx0_b2; qb[3] = qx0_b3;
            QMM_Q_LOAD(qx0, step + 2);
        }
        if (c == 0) {
            // ---- chunk start: group scales, zero-point term (sub-block sums already in lds_s)
            uint32_t sz_hi[2][GB], sz_lo[2][GB];
#pragma unroll
            for (int ni = 0; ni < 2; ni++) {
#pragma unroll
                for (int i = 0; i < GB; i++) {
                    const uint32_t sb = sc_n[ni][i] & 0xffffu;
                    gscale[ni][i] = h2f((uint16_t)sb) * (UP == 2 ? kTwo22 : kTwo24);
                    const float z = (float)(((zw_n[ni][i] >> (ni == 0 ? zshift0 : zshift1)) & 0xFu) + 1u);
                    const uint32_t nsc = (sb ^ 0x8000u) * 0x00010001u;  // (-scale, -scale)
                    const uint32_t zp = pack_half2(z, z);
                    sz_hi[ni][i] = pk_mul(nsc, zp);
                    sz_lo[ni][i] = pk_fma(nsc, zp, sz_hi[ni][i] ^ 0x80008000u);
                }
            }
            hdr_prefetch(blk + 1);
            if constexpr (with_zero)
#pragma unroll
            for (int mi = 0; mi < 2; mi++) {
                // A operand: lanes g=0 carry the hi parts of the 8 sub-block sums, g=1 the lo parts
                const half8 av = *(const half8*)(&lds_s[(wm * 64 + mi * 32 + nl) * 16 + g * 8]);
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    // sub-block pair p (columns 64p..64p+63) belongs to group p*GB/4
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        av, pack4(sz_hi[ni][0], sz_hi[ni][GB / 4], sz_hi[ni][GB / 2], sz_hi[ni][3 * GB / 4]),
                        acc[mi][ni], 0, 0, 0);
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        av, pack4(sz_lo[ni][0], sz_lo[ni][GB / 4], sz_lo[ni][GB / 2], sz_lo[ni][3 * GB / 4]),
                        acc[mi][ni], 0, 0, 0);
                }
            }
        }

        // ---- one 64-wide chunk: four 16-wide operand slices, one packed dword per column each
        // nibble positions inside the fp16 halves: bits 2..5 / 6..9 for an fp32 lhs, 0..3 / 4..7 for a bf16 lhs
        // (one shift less; its products are three bits shorter and lose next to nothing)
        const uint32_t M1 = 0x000F000Fu << UP, M2 = 0x00F000F0u << UP;
#pragma unroll
        for (int f = 0; f < 4; f++) {
            half8 bfrag[2];
            const uint32_t qa_lo = UP ? qa[f] << UP : qa[f], qb_lo = UP ? qb[f] << UP : qb[f];
            bfrag[0] = pack4(qa_lo & M1, qa_lo & M2, (qa[f] >> (8 - UP)) & M1, (qa[f] >> (8 - UP)) & M2);
            bfrag[1] = pack4(qb_lo & M1, qb_lo & M2, (qb[f] >> (8 - UP)) & M1, (qb[f] >> (8 - UP)) & M2);
#pragma unroll
            for (int mi = 0; mi < 2; mi++) {
                const half8 afrag = *(const half8*)(&lds_a[buf][(wm * 64 + mi * 32 + nl) * A_STRIDE + f * 16 + g * 8]);
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
                    P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag[ni], P[mi][ni], 0, 0, 0);
            }
        }
        if constexpr ((c + 1) % SPG == 0) {  // group end: apply its scale
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        acc[mi][ni][r] = fmaf(gscale[ni][c / SPG], P[mi][ni][r], acc[mi][ni][r]);
                        P[mi][ni][r] = 0.0f;
                    }
            // Pin the updated accumulators here.  Otherwise the compiler sinks these multiply-adds
            // to the end of the chunk and keeps every group's P alive until then.
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++) asm volatile("" : "+v"(acc[mi][ni]));
        }
        if constexpr (c & 1) {
            QMM_A_STORE(ax0, buf ^ 1);
            QMM_A_LOAD(ax0, step + 3);
        } else {
            QMM_A_STORE(ax1, buf ^ 1);
            QMM_A_LOAD(ax1, step + 3);
        }
        if (c == 3) {  // next chunk's sub-block sums
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

    // ---- epilogue: undo the row scale (inverse scales come from LDS, four rows per read: a dependent
    // global load per output row cost a fifth of the tile time), store
    const int ocol0 = n0 + wn * 64 + nl, ocol1 = ocol0 + 32;
    const bool c0_ok = ocol0 < n, c1_ok = ocol1 < n;
#pragma unroll
    for (int mi = 0; mi < 2; mi++) {
        float4 iv[4];
#pragma unroll
        for (int j = 0; j < 4; j++) iv[j] = *(const float4*)(&lds_inv[wm * 64 + mi * 32 + 8 * j + 4 * g]);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
            const float4 q = iv[r >> 2];
            const float is = (r & 3) == 0 ? q.x : (r & 3) == 1 ? q.y : (r & 3) == 2 ? q.z : q.w;
            if (row < m) {
                float* o = out + (int64_t)row * n;
                if (c0_ok) o[ocol0] = accumulate ? fmaf(acc[mi][0][r], is, o[ocol0]) : acc[mi][0][r] * is;
                if (c1_ok) o[ocol1] = accumulate ? fmaf(acc[mi][1][r], is, o[ocol1]) : acc[mi][1][r] * is;
            }
        }
    }
}

bool gemm_gptq_supported(int64_t k, int group) {
    return k % 256 == 0 && (group == 64 || group == 128 || group == 256);
}

// An fp32 lhs of up to 256 rows: hi and residual plane as the two halves of ONE lhs of twice the rows, one pass over the weights
// into the workspace instead of two onto `out`, and a small launch that adds the halves (4096 x 4096 with 128 rows: 126 -> 70 us).
bool gemm_gptq_twin(int lhs_dtype, int64_t m) { return lhs_dtype == QMM_F32 && m <= 256 && twin_rows_allowed() && !kernel_disabled("gptq_twin_rows"); }

// Shares of K per tile when the tiles leave compute units without work: as many as make about one workgroup per compute unit,
// each at least two blocks of 256 columns long, sixteen at most (4096 x 4096 with 64 bf16 rows, 16 tiles: 40 -> 21 us).
int gemm_gptq_k_shares(int64_t m, int64_t n, int64_t k) {
    const int64_t tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN), nblk = k / 256;
    if (kernel_disabled("gptq_k_shares")) return 1;
    return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(256 / tiles, 16), nblk / 2));
}

int64_t gemm_gptq_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    const bool twin = gemm_gptq_twin(lhs_dtype, m);
    const int64_t me = twin ? 2 * m : m;
    const int ks = gemm_gptq_k_shares(me, n, k);
    return lhs_planes(nullptr, twin ? QMM_BF16 : lhs_dtype, me, k).bytes + (twin || ks > 1 ? (int64_t)ks * me * n * 4 : 0);
}

hipError_t launch_gemm_gptq(const void* lhs, int lhs_dtype, const uint32_t* qweight, const uint16_t* scales,
                            const uint32_t* qzeros, int64_t m, int64_t n, int64_t k, int group, float* out,
                            void* workspace, hipStream_t s) {
    const bool twin = gemm_gptq_twin(lhs_dtype, m);
    const int64_t m_given = m;
    float* const out_given = out;
    const LhsPlanes p = twin ? lhs_planes(workspace, QMM_BF16, 2 * m, k) : lhs_planes(workspace, lhs_dtype, m, k);
    hipError_t e = launch_prep_lhs<kLhsOrderGPTQ>(lhs, lhs_dtype, m, k, p, s, twin);
    if (e != hipSuccess) return e;
    if (twin) m *= 2;
    const int ks = gemm_gptq_k_shares(m, n, k);
    const bool to_workspace = twin || ks > 1;  // partial results [ks][m][n], added up (and the row halves with them) at the end
    if (to_workspace) out = (float*)((char*)workspace + p.bytes);
    const int tiles_m = (int)((m + BM - 1) / BM), tiles_n = (int)((n + BN - 1) / BN);
    const int total = tiles_m * tiles_n * ks;
    const int per_xcd = (total + 7) / 8;
    dim3 grid((unsigned)(per_xcd * 8)), block(512);
#define QMM_GPTQ_LAUNCH(GB_)                                                                                          \
    do {                                                                                                              \
        if (twin) { /* both planes as one lhs */                                                                      \
            gemm_gptq_kernel<2, GB_, true, false><<<grid, block, 0, s>>>(qweight, scales, qzeros, p.a16, p.asum,    \
                                                                         p.inv, out, (int)m, (int)n, (int)k, tiles_m, \
                                                                         tiles_n, ks);                               \
        } else if (lhs_dtype == QMM_F32) { /* main plane, then the residual plane added on top */                     \
            gemm_gptq_kernel<2, GB_, true, false><<<grid, block, 0, s>>>(qweight, scales, qzeros, p.a16, p.asum,    \
                                                                         p.inv, out, (int)m, (int)n, (int)k, tiles_m, \
                                                                         tiles_n, ks);                               \
            gemm_gptq_kernel<2, GB_, false, true><<<grid, block, 0, s>>>(qweight, scales, qzeros, p.a16_lo, p.asum, \
                                                                         p.inv, out, (int)m, (int)n, (int)k, tiles_m, \
                                                                         tiles_n, ks);                               \
        } else {                                                                                                      \
            gemm_gptq_kernel<0, GB_, true, false><<<grid, block, 0, s>>>(qweight, scales, qzeros, p.a16, p.asum,    \
                                                                         p.inv, out, (int)m, (int)n, (int)k, tiles_m, \
                                                                         tiles_n, ks);                               \
        }                                                                                                             \
    } while (0)
    if (group == 256) QMM_GPTQ_LAUNCH(1);
    else if (group == 128) QMM_GPTQ_LAUNCH(2);
    else if (group == 64) QMM_GPTQ_LAUNCH(4);
    else return hipErrorInvalidValue;
#undef QMM_GPTQ_LAUNCH
    if (to_workspace) return launch_sum_shares(out, out_given, m_given * n, twin ? 2 * ks : ks, s);
    return hipGetLastError();
}

}  // namespace qmm
