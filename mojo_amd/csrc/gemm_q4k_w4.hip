// Q4_K prefill kernel, four-wavefront variant: one wavefront per SIMD with the full
// 512-register budget, so that a wavefront owns a 128 x 64 output sub-tile (all lhs
// rows of the workgroup tile, 64 weight columns).
//
// Arithmetic is that of gemm_q4k.hip (exact integer codes as fp16 subnormals, per
// super-block fp32 rescale, min term as an extra matrix product).  What differs is the
// shape of the work inside a compute unit:
//   * every weight column is unpacked by exactly one wavefront (the 8-wavefront kernel
//     unpacks each column twice), so there are 2.5 vector ALU instructions per
//     matrix-core instruction instead of 5;
//   * with a single wavefront per SIMD nothing else hides latency, so the step is
//     software-pipelined by hand: lhs fragments for slice f+1 are read from LDS, and the
//     weight operand for slice f+1 is unpacked, while the matrix cores work on slice f;
//   * the single barrier of a step sits before its last slice, after the last LDS read of
//     the current chunk, so that the refill of that buffer and the first fragment reads
//     of the next chunk are issued under the last slice's matrix-core instructions.
#include <stdlib.h>

#include <type_traits>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int BM = 128, BN = 256;
constexpr int A_STRIDE = 72;  // halfs per LDS row of a 64-wide chunk (144 bytes: conflict-free b128 reads)
constexpr float kTwo24 = 16777216.0f;

}  // namespace

// One pass multiplies one fp16 plane of the lhs (`a16`) with the weights.  `with_min` adds the
// min term (it uses the full-precision sub-block sums, so it belongs to exactly one pass);
// `accumulate` adds the result to what `out` already holds (second pass of an fp32 lhs).
__global__ __launch_bounds__(256, 1) void gemm_q4_k_w4_kernel(const uint8_t* __restrict__ w,
                                                              const _Float16* __restrict__ a16,
                                                              const _Float16* __restrict__ asum,
                                                              const float* __restrict__ inv, float* __restrict__ out,
                                                              int m, int n, int k, int tiles_m, int tiles_n,
                                                              int with_min, int accumulate) {
    __shared__ __attribute__((aligned(16))) _Float16 lds_a[2][BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 lds_s[2][BM * 16];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wn = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 31, g = lane >> 5;
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;

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
    const int nsteps = nblk * 4;

    // lhs chunk staging: 128 rows x 128 bytes per step; thread t moves the 16-byte piece (t & 7)
    // of rows (t >> 3) + 32 j.  Two register sets (parity of the step) keep two steps in flight.
    const int a_row = tid >> 3, a_seg = tid & 7;
    const uint4* a_src0 = (const uint4*)(a16 + (int64_t)min(m0 + a_row, m - 1) * k + a_seg * 8);
    const uint4* a_src1 = (const uint4*)(a16 + (int64_t)min(m0 + a_row + 32, m - 1) * k + a_seg * 8);
    const uint4* a_src2 = (const uint4*)(a16 + (int64_t)min(m0 + a_row + 64, m - 1) * k + a_seg * 8);
    const uint4* a_src3 = (const uint4*)(a16 + (int64_t)min(m0 + a_row + 96, m - 1) * k + a_seg * 8);
    uint4 ax0_0, ax0_1, ax0_2, ax0_3, ax1_0, ax1_1, ax1_2, ax1_3;
    _Float16* a_dst = &lds_a[0][a_row * A_STRIDE + a_seg * 8];
#define QMM_A_LOAD(SET, STEP)                          \
    do {                                               \
        const int ch_ = min((STEP), nsteps - 1) * 8;   \
        SET##_0 = a_src0[ch_];                         \
        SET##_1 = a_src1[ch_];                         \
        SET##_2 = a_src2[ch_];                         \
        SET##_3 = a_src3[ch_];                         \
    } while (0)
#define QMM_A_STORE(SET, BUF)                                  \
    do {                                                       \
        _Float16* d_ = a_dst + (size_t)(BUF) * BM * A_STRIDE;  \
        *(uint4*)d_ = SET##_0;                                 \
        *(uint4*)(d_ + 32 * A_STRIDE) = SET##_1;               \
        *(uint4*)(d_ + 64 * A_STRIDE) = SET##_2;               \
        *(uint4*)(d_ + 96 * A_STRIDE) = SET##_3;               \
    } while (0)

    // this lane's two weight columns
    const uint8_t* wcol0 = w + (int64_t)min(n0 + wn * 64 + nl, n - 1) * row_bytes;
    const uint8_t* wcol1 = w + (int64_t)min(n0 + wn * 64 + 32 + nl, n - 1) * row_bytes;
    const int q_lane_off = 16 + 16 * g;
    uint4 qx0_c0, qx0_c1, qx1_c0, qx1_c1;
#define QMM_Q_LOAD(SET, STEP)                                                 \
    do {                                                                      \
        const int st_ = min((STEP), nsteps - 1);                              \
        const int off_ = (st_ >> 2) * Q4_K_BPB + 32 * (st_ & 3) + q_lane_off; \
        SET##_c0 = *(const uint4*)(wcol0 + off_);                             \
        SET##_c1 = *(const uint4*)(wcol1 + off_);                             \
    } while (0)

    float16v acc[4][2], P[4][2];
#pragma unroll
    for (int mi = 0; mi < 4; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc[mi][ni][r] = 0.0f;
                P[mi][ni][r] = 0.0f;
            }

    // block headers and sub-block sums are fetched one super-block ahead
    uint4 hdr_n0, hdr_n1, as_n;
    const uint4* as_src = (const uint4*)(asum + (int64_t)min(m0 + (tid >> 1), m - 1) * nblk * 16 + (tid & 1) * 8);
    auto hdr_prefetch = [&](int blk) {
        const int bc = min(blk, nblk - 1);
        hdr_n0 = *(const uint4*)(wcol0 + bc * Q4_K_BPB);
        hdr_n1 = *(const uint4*)(wcol1 + bc * Q4_K_BPB);
    };
    auto as_prefetch = [&](int blk) { as_n = as_src[min(blk, nblk - 1) * 2]; };

    // fragment registers: lhs fragments and unpacked weight operands, double-buffered by slice parity
    half8 afr[2][4], bfr[2][2], sfr[4];
    const _Float16* a_frag_base = &lds_a[0][nl * A_STRIDE + g * 8];
    const _Float16* s_frag_base = &lds_s[0][nl * 16 + g * 8];
    auto read_afr = [&](int buf, int f, int slot) {
#pragma unroll
        for (int mi = 0; mi < 4; mi++)
            afr[slot][mi] = *(const half8*)(a_frag_base + (size_t)buf * BM * A_STRIDE + mi * 32 * A_STRIDE + f * 16);
    };
    auto read_sfr = [&](int sbuf) {
#pragma unroll
        for (int mi = 0; mi < 4; mi++) sfr[mi] = *(const half8*)(s_frag_base + (size_t)sbuf * BM * 16 + mi * 32 * 16);
    };

    float dscale[2] = {0.f, 0.f};
    uint32_t sp[2][8], dmn_hi[2][4], dmn_lo[2][4];
    // header decode of one column: scale pairs for the unpack, -(dmin*mn) as fp16 hi + lo pairs
    auto decode = [&](const uint4 hdr, int ni) {
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
        const uint32_t ndm = ((hdr.x >> 16) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
        const uint32_t mp[4] = {pack_half2((float)(mn_lo & 0xffu), (float)((mn_lo >> 8) & 0xffu)),
                                pack_half2((float)((mn_lo >> 16) & 0xffu), (float)(mn_lo >> 24)),
                                pack_half2((float)(mn_hi & 0xffu), (float)((mn_hi >> 8) & 0xffu)),
                                pack_half2((float)((mn_hi >> 16) & 0xffu), (float)(mn_hi >> 24))};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            dmn_hi[ni][i] = pk_mul(ndm, mp[i]);
            dmn_lo[ni][i] = pk_fma(ndm, mp[i], dmn_hi[ni][i] ^ 0x80008000u);
        }
    };
    // one dword pair of the operand of slice f (chunk c) of column ni: half of a half8
    const uint32_t M1 = 0x000F000Fu, M2 = 0x00F000F0u;
    auto unpack_half = [&](const uint4 qq, int c, int f, int ni, int slot, int half) {
        const uint32_t x = half == 0 ? ((f & 1) ? qq.z : qq.x) : ((f & 1) ? qq.w : qq.y);
        const uint32_t mask = (f & 2) ? M2 : M1;
        const uint32_t s = sp[ni][2 * c + (f >> 1)];
        HalfPack hp;
        hp.h = bfr[slot][ni];
        hp.u[2 * half] = pk_mul(x & mask, s);
        hp.u[2 * half + 1] = pk_mul((x >> 8) & mask, s);
        bfr[slot][ni] = hp.h;
    };

    // ---- prologue: chunks 0 and 1 to LDS, sums of block 0, header 0 decoded, operand of slice 0
    hdr_prefetch(0);
    as_prefetch(0);
    QMM_A_LOAD(ax0, 0);
    QMM_A_LOAD(ax1, 1);
    QMM_Q_LOAD(qx0, 0);
    QMM_Q_LOAD(qx1, 1);
    QMM_A_STORE(ax0, 0);
    QMM_A_STORE(ax1, 1);
    *(uint4*)(&lds_s[0][(tid >> 1) * 16 + (tid & 1) * 8]) = as_n;
    QMM_A_LOAD(ax0, 2);
    QMM_A_LOAD(ax1, 3);
    as_prefetch(1);
    decode(hdr_n0, 0);
    decode(hdr_n1, 1);
    hdr_prefetch(1);
    __syncthreads();
    read_afr(0, 0, 0);
    read_sfr(0);
#pragma unroll
    for (int ni = 0; ni < 2; ni++) {
        bfr[0][ni] = pack4(0, 0, 0, 0);
        bfr[1][ni] = pack4(0, 0, 0, 0);
        unpack_half(ni == 0 ? qx0_c0 : qx0_c1, 0, 0, ni, 0, 0);
        unpack_half(ni == 0 ? qx0_c0 : qx0_c1, 0, 0, ni, 0, 1);
    }

    auto do_step = [&](int blk, auto CC) {
        constexpr int c = decltype(CC)::value;
        const int step = blk * 4 + c;
        constexpr int buf = c & 1;
        uint4 qc0, qc1, qn0, qn1;  // this step's codes, next step's codes
        if constexpr (c & 1) {
            qc0 = qx1_c0; qc1 = qx1_c1; qn0 = qx0_c0; qn1 = qx0_c1;
        } else {
            qc0 = qx0_c0; qc1 = qx0_c1; qn0 = qx1_c0; qn1 = qx1_c1;
        }
        if (c == 0) {
            // min term of this super-block (sums already in sfr, products decoded at the previous c == 3)
            if (with_min) {
#pragma unroll
                for (int mi = 0; mi < 4; mi++)
#pragma unroll
                    for (int ni = 0; ni < 2; ni++) {
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                            sfr[mi], pack4(dmn_hi[ni][0], dmn_hi[ni][1], dmn_hi[ni][2], dmn_hi[ni][3]), acc[mi][ni], 0, 0, 0);
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                            sfr[mi], pack4(dmn_lo[ni][0], dmn_lo[ni][1], dmn_lo[ni][2], dmn_lo[ni][3]), acc[mi][ni], 0, 0, 0);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int f = 0; f < 4; f++) {
            if (f < 3) {
                read_afr(buf, f + 1, (f + 1) & 1);
            } else {
                // All reads of this chunk's buffer are issued; after the barrier it can take chunk step + 2,
                // and the other buffer (filled during the previous step) is visible.
                __syncthreads();
                read_afr(buf ^ 1, 0, 0);
                if constexpr (c & 1) {
                    QMM_A_STORE(ax1, buf);
                    QMM_A_LOAD(ax1, step + 4);
                    QMM_Q_LOAD(qx1, step + 2);
                } else {
                    QMM_A_STORE(ax0, buf);
                    QMM_A_LOAD(ax0, step + 4);
                    QMM_Q_LOAD(qx0, step + 2);
                }
                if (c == 1) {  // sums of the next super-block into the other sums buffer
                    *(uint4*)(&lds_s[(blk + 1) & 1][(tid >> 1) * 16 + (tid & 1) * 8]) = as_n;
                    as_prefetch(blk + 2);
                }
                if (c == 3) read_sfr((blk + 1) & 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (c == 3 && f == 3) {
                // next super-block's header: its scales are needed for the operand unpacked below
                decode(hdr_n0, 0);
                decode(hdr_n1, 1);
                hdr_prefetch(blk + 2);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int mi = i >> 1, ni = i & 1;
                P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[f & 1][mi], bfr[f & 1][ni], P[mi][ni], 0, 0, 0);
                if (i < 4) {  // one quarter of the next slice's weight operands per matrix-core instruction
                    const int uni = i >> 1, uh = i & 1;
                    if (f < 3)
                        unpack_half(uni == 0 ? qc0 : qc1, c, f + 1, uni, (f + 1) & 1, uh);
                    else
                        unpack_half(uni == 0 ? qn0 : qn1, (c + 1) & 3, 0, uni, 0, uh);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    float dprev[2];
    for (int blk = 0; blk < nblk; blk++) {
        // decode() at the last step replaces dscale with the next block's; keep this block's for the rescale
        dprev[0] = dscale[0];
        dprev[1] = dscale[1];
        do_step(blk, std::integral_constant<int, 0>{});
        do_step(blk, std::integral_constant<int, 1>{});
        do_step(blk, std::integral_constant<int, 2>{});
        do_step(blk, std::integral_constant<int, 3>{});
#pragma unroll
        for (int mi = 0; mi < 4; mi++)
#pragma unroll
            for (int ni = 0; ni < 2; ni++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    acc[mi][ni][r] = fmaf(dprev[ni], P[mi][ni][r], acc[mi][ni][r]);
                    P[mi][ni][r] = 0.0f;
                }
            }
    }
#undef QMM_A_LOAD
#undef QMM_A_STORE
#undef QMM_Q_LOAD

    // ---- epilogue: undo the row scale, store
#pragma unroll
    for (int mi = 0; mi < 4; mi++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = m0 + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
            if (row < m) {
                const float is = inv[row];
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    const int col = n0 + wn * 64 + ni * 32 + nl;
                    if (col < n) {
                        float* o = out + (int64_t)row * n + col;
                        const float v = acc[mi][ni][r] * is;
                        *o = accumulate ? *o + v : v;
                    }
                }
            }
        }
    }
}

hipError_t launch_gemm_q4_k_w4(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                               float* out, void* workspace, hipStream_t s) {
    const LhsPlanes p = lhs_planes(workspace, lhs_dtype, m, k);
    hipError_t e = launch_prep_lhs<kLhsOrderQ4K>(lhs, lhs_dtype, m, k, p, s);
    if (e != hipSuccess) return e;
    const int tiles_m = (int)((m + BM - 1) / BM), tiles_n = (int)((n + BN - 1) / BN);
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    dim3 grid((unsigned)(per_xcd * 8)), block(256);
    gemm_q4_k_w4_kernel<<<grid, block, 0, s>>>(w, p.a16, p.asum, p.inv, out, (int)m, (int)n, (int)k, tiles_m, tiles_n, 1, 0);
    if (p.a16_lo)  // fp32 lhs: the residual plane, added on top
        gemm_q4_k_w4_kernel<<<grid, block, 0, s>>>(w, p.a16_lo, p.asum, p.inv, out, (int)m, (int)n, (int)k, tiles_m,
                                                   tiles_n, 0, 1);
    return hipGetLastError();
}

}  // namespace qmm
