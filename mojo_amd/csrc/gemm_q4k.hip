// Q4_K prefill kernel (m > 16 lhs rows): matrix-core GEMM over exact integer codes.
//
// Arithmetic.  As in the decode kernel, a masked nibble is the fp16 subnormal
// q*2^-24 and one packed fp16 multiply folds the 6-bit sub-block scale in,
// times 64 (sc*q*2^-18 with q*sc <= 945: exact, and normal from 16 on).  lhs values are scaled per row by a power of two and
// narrowed to fp16 (exact for bf16 inputs of ordinary range), so every product
// inside v_mfma_f32_32x32x16_f16 is exact and the sums are fp32.  Per 256-wide
// super-block b the matrix cores produce P_b[m][n] = sum_k a[m][k]*(sc*q)[n][k];
// the fp32 super-block scale is applied in the lanes, acc += d[n,b] * P_b.  The
// min term  -sum_{b,j} (dmin*mn_j)[n] * (sum_{k in j} a[m][k])  is itself a matrix
// product over the 8 sub-blocks of a super-block: dmin*mn (17 bits) is split
// exactly into two fp16 values and the activation sums into hi + lo, and the two
// extra products per super-block accumulate straight into acc.
//
// Shape.  Persistent workgroups loop over 64 x 256 output tiles (4 wavefronts, two
// workgroups per compute unit, so two wavefronts per SIMD that run out of phase) or
// 128 x 256 tiles (8 wavefronts, one workgroup per compute unit); wavefront (wm, wn)
// owns the 64 x 64 sub-tile at (64 wm, 64 wn).  lhs chunks (64 wide) go through
// double-buffered LDS; the packed weights are loaded by the lanes that use them and
// unpacked in registers.  The schedule, in the order the measurements on this part
// asked for it:
//   * lhs fragments for slice f+1 are read from LDS, and the weight operand for slice
//     f+1 is unpacked, while the matrix cores work on slice f (with two wavefronts per
//     SIMD about six vector ALU instructions per matrix-core instruction are free; an
//     LDS fragment read of 1 KB costs about 7.4 ns of the whole compute unit);
//   * the one barrier of a step sits before its last slice, after the last LDS read of
//     the chunk, so the refill of that buffer and the first fragment reads of the next
//     chunk are issued under the last slice's matrix-core instructions;
//   * the workgroup is persistent: the stores of a finished tile drain while the next
//     tile's loads are in flight;
//   * the per-row inverse scales of the epilogue come from LDS (a dependent global load
//     per output row cost a fifth of the tile time).
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int BN = 256;
constexpr int A_STRIDE = 72;  // halfs per LDS row of a 64-wide chunk (144 bytes: conflict-free b128 reads)
constexpr float kTwo18 = 262144.0f;

// Tile order inside an XCD's range: `gm` lhs tile rows stay fixed while the order walks N.
__device__ __forceinline__ void tile_coords(int o, int tiles_m, int tiles_n, int gm, int& tile_m, int& tile_n) {
    const int span = gm * tiles_n;
    const int grp = o / span, rem = o - grp * span;
    const int rows_here = min(gm, tiles_m - grp * gm);
    tile_n = rem / rows_here;
    tile_m = grp * gm + rem - tile_n * rows_here;
}

}  // namespace

// One pass multiplies one fp16 plane of the lhs (`a16`) with the weights.  `with_min` adds the
// min term (it uses the full-precision sub-block sums, so it belongs to exactly one pass);
// `accumulate` adds the result to what `out` already holds (second pass of an fp32 lhs).
template <int WM>
__global__ __launch_bounds__(256 * WM, 2 / WM) void gemm_q4_k_kernel(const uint8_t* __restrict__ w,
                                                           const _Float16* __restrict__ a16,
                                                           const _Float16* __restrict__ asum,
                                                           const float* __restrict__ inv, float* __restrict__ out,
                                                           int m, int n, int k, int tiles_m, int tiles_n,
                                                           int with_min, int accumulate, int ksplit) {
    constexpr int BM = 64 * WM;  // WM wavefront rows of 64 lhs rows each; 256 * WM threads
    __shared__ __attribute__((aligned(16))) _Float16 lds_a[2][BM * A_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 lds_s[2][BM * 16];
    __shared__ __attribute__((aligned(16))) float lds_inv[BM];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int nl = lane & 31, g = lane >> 5;
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int total = tiles_m * tiles_n * ksplit;  // work units: (tile, share of K)
    const int per_xcd = (total + 7) / 8;
    const int a_row = tid >> 2, a_seg = tid & 3;
    _Float16* a_dst = &lds_a[0][a_row * A_STRIDE + a_seg * 8];
    const _Float16* a_frag_base = &lds_a[0][(wm * 64 + nl) * A_STRIDE + g * 8];
    const _Float16* s_frag_base = &lds_s[0][(wm * 64 + nl) * 16 + g * 8];
    const int q_lane_off = 16 + 16 * g;

    // Units of one XCD (workgroup ids congruent mod 8 share an XCD and its L2) form a contiguous range of
    // an order that keeps a few lhs tile rows fixed while walking N; slot j of an XCD takes units j, j + S, ...
    // With ksplit > 1 (few lhs rows, hence few tiles) a unit is one tile's share of the super-blocks and
    // writes its partial result to slice `ks` of `out`, which is then a [ksplit][m][n] buffer that a
    // second kernel adds up in a fixed order.  (For large m, cutting only the leftover tiles of the last
    // round along K was tried and lost: a workgroup that has its compute unit to itself runs its last tile
    // about 1.6x faster, and the partial sums cost traffic.)
    for (int tq = (int)(blockIdx.x >> 3); tq < per_xcd; tq += (int)(gridDim.x >> 3)) {
        const int o = (int)(blockIdx.x & 7) * per_xcd + tq;
        if (o >= total) break;
        const int tile = o / ksplit, ks = o - tile * ksplit;
        const int kb0 = ks * nblk / ksplit;
        const int nb = (ks + 1) * nblk / ksplit - kb0, ns = nb * 4;
        int tile_m, tile_n;
        tile_coords(tile, tiles_m, tiles_n, 4 / WM, tile_m, tile_n);
        const int m0 = tile_m * BM, n0 = tile_n * BN;

        // lhs chunk staging: 128 rows x 128 bytes per step, two 16-byte pieces per thread; two
        // register sets (parity of the step) keep two steps of loads in flight.
        const uint4* a_src = (const uint4*)(a16 + (int64_t)min(m0 + a_row, m - 1) * k + kb0 * 256 + a_seg * 8);
        uint4 ax0_0, ax0_1, ax1_0, ax1_1;
#define QMM_A_LOAD(SET, STEP)                          \
    do {                                               \
        const int ch_ = min((STEP), ns - 1) * 8;       \
        SET##_0 = a_src[ch_];                          \
        SET##_1 = a_src[ch_ + 4];                      \
    } while (0)
#define QMM_A_STORE(SET, BUF)                                  \
    do {                                                       \
        _Float16* d_ = a_dst + (size_t)(BUF) * BM * A_STRIDE;  \
        *(uint4*)d_ = SET##_0;                                 \
        *(uint4*)(d_ + 32) = SET##_1;                          \
    } while (0)

        // this lane's two weight columns
        const uint8_t* wcol0 = w + (int64_t)min(n0 + wn * 64 + nl, n - 1) * row_bytes + kb0 * Q4_K_BPB;
        const uint8_t* wcol1 = w + (int64_t)min(n0 + wn * 64 + 32 + nl, n - 1) * row_bytes + kb0 * Q4_K_BPB;
        uint4 qx0_c0, qx0_c1, qx1_c0, qx1_c1;
#define QMM_Q_LOAD(SET, STEP)                                                 \
    do {                                                                      \
        const int st_ = min((STEP), ns - 1);                                  \
        const int off_ = (st_ >> 2) * Q4_K_BPB + 32 * (st_ & 3) + q_lane_off; \
        SET##_c0 = *(const uint4*)(wcol0 + off_);                             \
        SET##_c1 = *(const uint4*)(wcol1 + off_);                             \
    } while (0)

        float16v acc[2][2], P[2][2], zero16;
#pragma unroll
        for (int mi = 0; mi < 2; mi++)
#pragma unroll
            for (int ni = 0; ni < 2; ni++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    acc[mi][ni][r] = 0.0f;
                    P[mi][ni][r] = 0.0f;
                    zero16[r] = 0.0f;
                }

        // block headers and sub-block sums are fetched one super-block ahead
        uint4 hdr_n0, hdr_n1, as_n = make_uint4(0, 0, 0, 0);
        const uint4* as_src = (const uint4*)(asum + ((int64_t)min(m0 + (tid >> 1), m - 1) * nblk + kb0) * 16 + (tid & 1) * 8);
        auto hdr_prefetch = [&](int blk) {
            const int bc = min(blk, nb - 1);
            hdr_n0 = *(const uint4*)(wcol0 + bc * Q4_K_BPB);
            hdr_n1 = *(const uint4*)(wcol1 + bc * Q4_K_BPB);
        };
        auto as_prefetch = [&](int blk) {
            if (tid < 2 * BM) as_n = as_src[min(blk, nb - 1) * 2];
        };

        // fragment registers, double-buffered by slice parity
        half8 afr[2][2], bfr[2][2];
        auto read_afr = [&](int buf, int f, int slot) {
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
                afr[slot][mi] = *(const half8*)(a_frag_base + (size_t)buf * BM * A_STRIDE + mi * 32 * A_STRIDE + f * 16);
        };

        float dscale[2] = {0.f, 0.f};
        uint32_t sp[2][8];
        // Header decode of both columns for super-block `blk`: scale pairs for the unpack, and the min
        // term of that block, -(dmin*mn) as exact fp16 hi + lo pairs times the sub-block sums, which
        // goes straight into acc (the order of accumulation into acc does not matter).
        auto decode_and_min = [&](int sbuf, bool add_min) {
            half8 sfr[2];
#pragma unroll
            for (int mi = 0; mi < 2; mi++) sfr[mi] = *(const half8*)(s_frag_base + (size_t)sbuf * BM * 16 + mi * 32 * 16);
#pragma unroll
            for (int ni = 0; ni < 2; ni++) {
                const uint4 hdr = ni == 0 ? hdr_n0 : hdr_n1;
                dscale[ni] = h2f((uint16_t)(hdr.x & 0xffffu)) * kTwo18;
                const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
                const uint32_t sc_lo = s0 & 0x3F3F3F3Fu, sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
                const uint32_t mn_lo = s1 & 0x3F3F3F3Fu, mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
                // 64 * sc for the low nibbles (q * 2^-24), 4 * sc for the high ones (16 q * 2^-24): the operand is
                // sc * q * 2^-18, a normal fp16 number from sc * q = 16 on.  (With sc * q * 2^-24, always a subnormal,
                // the matrix core drops low bits of the products of small sc * q towards minus infinity: a bias
                // growing with K, 5e-5 at K = 14336 for sub-block scales of 1.)
                const float e0 = 64.0f * (float)(sc_lo & 0xffu), e1 = 4.0f * (float)((sc_lo >> 8) & 0xffu);
                const float e2 = 64.0f * (float)((sc_lo >> 16) & 0xffu), e3 = 4.0f * (float)(sc_lo >> 24);
                const float e4 = 64.0f * (float)(sc_hi & 0xffu), e5 = 4.0f * (float)((sc_hi >> 8) & 0xffu);
                const float e6 = 64.0f * (float)((sc_hi >> 16) & 0xffu), e7 = 4.0f * (float)(sc_hi >> 24);
                sp[ni][0] = pack_half2(e0, e0); sp[ni][1] = pack_half2(e1, e1);
                sp[ni][2] = pack_half2(e2, e2); sp[ni][3] = pack_half2(e3, e3);
                sp[ni][4] = pack_half2(e4, e4); sp[ni][5] = pack_half2(e5, e5);
                sp[ni][6] = pack_half2(e6, e6); sp[ni][7] = pack_half2(e7, e7);
                if (add_min) {
                    const uint32_t ndm = ((hdr.x >> 16) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
                    const uint32_t mp[4] = {pack_half2((float)(mn_lo & 0xffu), (float)((mn_lo >> 8) & 0xffu)),
                                            pack_half2((float)((mn_lo >> 16) & 0xffu), (float)(mn_lo >> 24)),
                                            pack_half2((float)(mn_hi & 0xffu), (float)((mn_hi >> 8) & 0xffu)),
                                            pack_half2((float)((mn_hi >> 16) & 0xffu), (float)(mn_hi >> 24))};
                    uint32_t hi[4], lo[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        hi[i] = pk_mul(ndm, mp[i]);
                        lo[i] = pk_fma(ndm, mp[i], hi[i] ^ 0x80008000u);
                    }
#pragma unroll
                    for (int mi = 0; mi < 2; mi++) {
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sfr[mi], pack4(hi[0], hi[1], hi[2], hi[3]),
                                                                            acc[mi][ni], 0, 0, 0);
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sfr[mi], pack4(lo[0], lo[1], lo[2], lo[3]),
                                                                            acc[mi][ni], 0, 0, 0);
                    }
                }
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

        // ---- tile prologue: chunks 0 and 1 to LDS, sums of block 0, header 0, operand of slice 0
        hdr_prefetch(0);
        as_prefetch(0);
        QMM_A_LOAD(ax0, 0);
        QMM_A_LOAD(ax1, 1);
        QMM_Q_LOAD(qx0, 0);
        QMM_Q_LOAD(qx1, 1);
        __syncthreads();  // every wavefront is done with the previous tile's LDS contents
        QMM_A_STORE(ax0, 0);
        QMM_A_STORE(ax1, 1);
        if (tid < 2 * BM) *(uint4*)(&lds_s[0][(tid >> 1) * 16 + (tid & 1) * 8]) = as_n;
        if (tid < BM) lds_inv[tid] = inv[min(m0 + tid, m - 1)];
        QMM_A_LOAD(ax0, 2);
        QMM_A_LOAD(ax1, 3);
        as_prefetch(1);
        __syncthreads();
        decode_and_min(0, with_min != 0);
        hdr_prefetch(1);
        read_afr(0, 0, 0);
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            bfr[0][ni] = pack4(0, 0, 0, 0);
            bfr[1][ni] = pack4(0, 0, 0, 0);
            unpack_half(ni == 0 ? qx0_c0 : qx0_c1, 0, 0, ni, 0, 0);
            unpack_half(ni == 0 ? qx0_c0 : qx0_c1, 0, 0, ni, 0, 1);
        }

        float dprev[2];
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
#pragma unroll
            for (int f = 0; f < 4; f++) {
                if (f < 3) {
                    read_afr(buf, f + 1, (f + 1) & 1);
                } else {
                    // All reads of this chunk's buffer are issued; after the barrier it can take chunk
                    // step + 2, and the other buffer (filled during the previous step) is visible.
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
                        if (tid < 2 * BM) *(uint4*)(&lds_s[(blk + 1) & 1][(tid >> 1) * 16 + (tid & 1) * 8]) = as_n;
                        as_prefetch(blk + 2);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (c == 3 && f == 3) {
                    // next super-block: its scales are needed for the operand unpacked below
                    dprev[0] = dscale[0];
                    dprev[1] = dscale[1];
                    decode_and_min((blk + 1) & 1, with_min != 0 && blk + 1 < nb);  // no block after the last
                    hdr_prefetch(blk + 2);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int mi = i >> 1, ni = i & 1;
                    // the first slice after a rescale starts from zero
                    P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[f & 1][mi], bfr[f & 1][ni],
                                                                      (f == 0 && c % 4 == 0) ? zero16 : P[mi][ni], 0, 0, 0);
                    // one quarter of the next slice's weight operands per matrix-core instruction
                    const int uni = i >> 1, uh = i & 1;
                    if (f < 3)
                        unpack_half(uni == 0 ? qc0 : qc1, c, f + 1, uni, (f + 1) & 1, uh);
                    else
                        unpack_half(uni == 0 ? qn0 : qn1, (c + 1) & 3, 0, uni, 0, uh);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        for (int blk = 0; blk < nb; blk++) {
            do_step(blk, std::integral_constant<int, 0>{});
            do_step(blk, std::integral_constant<int, 1>{});
            do_step(blk, std::integral_constant<int, 2>{});
            do_step(blk, std::integral_constant<int, 3>{});
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    rescale_add(acc[mi][ni], dprev[ni], P[mi][ni]);
                }
        }
#undef QMM_A_LOAD
#undef QMM_A_STORE
#undef QMM_Q_LOAD

        // ---- tile epilogue: undo the row scale (inverse scales come from LDS, four rows per read), store;
        // the stores drain under the next tile
        {
            const int col0 = n0 + wn * 64 + nl, col1 = col0 + 32;
            const bool c0_ok = col0 < n, c1_ok = col1 < n;
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
                        float* o = out + ((int64_t)ks * m + row) * n;
                        const float v0 = acc[mi][0][r] * is, v1 = acc[mi][1][r] * is;
                        if (accumulate) {
                            if (c0_ok) o[col0] += v0;
                            if (c1_ok) o[col1] += v1;
                        } else {
                            if (c0_ok) o[col0] = v0;
                            if (c1_ok) o[col1] = v1;
                        }
                    }
                }
            }
        }
    }
}

// out[i] (+)= part[0][i] + part[1][i] + ... in that order.  VEC: four neighbouring values per thread (count a multiple of 4,
// 16-byte aligned buffers); the loads of four shares are issued together, the additions keep their order.
template <bool VEC>
__global__ __launch_bounds__(256) void sum_k_shares_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                           int64_t count, int ksplit, int accumulate) {
    if constexpr (VEC) {
        const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
        if (i >= count) return;
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        float4 v = accumulate ? *(const float4*)(out + i) : make_float4(0.f, 0.f, 0.f, 0.f);
        int s = 0;
        for (; s + 4 <= ksplit; s += 4) {
            f32x4 p[4];
#pragma unroll
            for (int j = 0; j < 4; j++) p[j] = __builtin_nontemporal_load((const f32x4*)(part + (int64_t)(s + j) * count + i));
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v.x += p[j].x;
                v.y += p[j].y;
                v.z += p[j].z;
                v.w += p[j].w;
            }
        }
        for (; s < ksplit; s++) {
            const f32x4 p = __builtin_nontemporal_load((const f32x4*)(part + (int64_t)s * count + i));
            v.x += p.x;
            v.y += p.y;
            v.z += p.z;
            v.w += p.w;
        }
        *(float4*)(out + i) = v;
    } else {
        const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
        if (i >= count) return;
        float v = accumulate ? out[i] : 0.0f;
        for (int s = 0; s < ksplit; s++) v += part[(int64_t)s * count + i];
        out[i] = v;
    }
}

namespace {
void sum_shares(const float* part, float* out, int64_t count, int shares, int accumulate, hipStream_t s) {
    if (count % 4 == 0 && (((uintptr_t)part | (uintptr_t)out) & 15) == 0)
        sum_k_shares_kernel<true><<<dim3((unsigned)((count / 4 + 255) / 256)), dim3(256), 0, s>>>(part, out, count, shares, accumulate);
    else
        sum_k_shares_kernel<false><<<dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s>>>(part, out, count, shares, accumulate);
}
}  // namespace

hipError_t launch_sum_shares(const float* part, float* out, int64_t count, int shares, hipStream_t s) {
    sum_shares(part, out, count, shares, 0, s);
    return hipGetLastError();
}

namespace {

// Shares of K per tile, a function of the shape only: 1 when the tiles alone fill the machine; each share at least two
// super-blocks long.  Every share is another m x n partial result written and read back, so with several lhs row tiles the aim
// is about 256 work units (one per compute unit; microseconds with 1024 / 512 / 256 / 128 units aimed at, bf16 lhs: 512 x 4096 x
// 4096 60.7 / 45.9 / 42.7 / 52.8; 512 x 4096 x 14336 123 / 105 / 107 / 170; 200 x 14336 x 4096 77.6 / 67.7 / 59.9 / 56.7;
// 96 x 4096 x 14336 57.7 / 49.0 / 43.8 / 60.7).  One row tile (up to 64 rows) has small partial results: as many shares as fit
// one round of two workgroups per compute unit, sixteen at most (32 rows: 14336 x 4096, 56 tiles, 5 / 8 shares 35.2 / 29.3;
// 4096 x 14336, 16 tiles, 16 / 28 shares 33.5 / 35.7; 64 rows on 32000 x 4096, 125 tiles, 3 / 5 shares 51.6 / 60.2).
int k_shares(int64_t m, int64_t n, int64_t k, int bm) {
    const int64_t tiles = ((m + bm - 1) / bm) * ((n + BN - 1) / BN), nblk = k / 256;
    if (tiles >= 256) return 1;
    const int64_t cap = nblk / 2 > 1 ? nblk / 2 : 1;
    const int64_t want = m <= bm ? std::min<int64_t>(512 / tiles, 16) : 256 / tiles;  // (rounded down: 384 x 4096 x 4096, 96 tiles, 2 / 3 shares 40.1 / 42.3 us)
    return (int)std::max<int64_t>(1, std::min(want, cap));
}

}  // namespace

namespace {
// An fp32 lhs on a problem whose tiles are cut into K shares anyway, or of up to 256 rows: hi and residual plane as the two
// halves of one lhs of 2 m rows, one pass of the GEMM instead of two, and the pass that adds the K shares adds the two halves as
// well (twice the shares of m x n values each; without K shares it is a launch more and a pass over the weights less).
// 4096 x 4096 with 32 fp32 rows: 35 -> 20 us; 14336 x 4096 with 256: 157 -> 85.
bool twin_rows(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    return lhs_dtype == QMM_F32 && (k_shares(2 * m, n, k, 64) > 1 || m <= 256) && twin_rows_allowed() && !kernel_disabled("q4k_twin_rows");
}
}  // namespace

int64_t gemm_q4_k_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    if (gemm_q4_k_tile_wanted(m, n, k)) return gemm_q4_k_tile_workspace_bytes(lhs_dtype, m, k);
    if (twin_rows(lhs_dtype, m, n, k))
        return lhs_planes(nullptr, QMM_BF16, 2 * m, k).bytes + (int64_t)k_shares(2 * m, n, k, 64) * 2 * m * n * 4;
    const int ks = k_shares(m, n, k, 64);
    return lhs_planes(nullptr, lhs_dtype, m, k).bytes + (ks > 1 ? (int64_t)ks * m * n * 4 : 0);
}

hipError_t launch_gemm_q4_k(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                               float* out, void* workspace, hipStream_t s) {
    if (gemm_q4_k_tile_wanted(m, n, k)) return launch_gemm_q4_k_tile(lhs, lhs_dtype, w, m, n, k, out, workspace, s);
    const bool twin = twin_rows(lhs_dtype, m, n, k);
    const int64_t m_out = m;  // rows of the result
    LhsPlanes p = twin ? lhs_planes(workspace, QMM_BF16, 2 * m, k) : lhs_planes(workspace, lhs_dtype, m, k);
    hipError_t e = launch_prep_lhs<kLhsOrderQ4K>(lhs, lhs_dtype, m, k, p, s, twin);
    if (e != hipSuccess) return e;
    if (twin) m *= 2;  // (the GEMM's rows from here on)
    // 4-wavefront workgroups on 64-row tiles, two per compute unit, which run out of phase; with that shape
    // disabled ("q4k_gemm64"), 8-wavefront workgroups on 128-row tiles, one per compute unit.
    const int wm_env = kernel_disabled("q4k_gemm64") ? 2 : 1;
    const int ksplit = k_shares(m, n, k, 64);
    const int wm_rows = ksplit > 1 ? 1 : wm_env;
    const int bm = 64 * wm_rows;
    const int tiles_m = (int)((m + bm - 1) / bm), tiles_n = (int)((n + BN - 1) / BN);
    const int total = tiles_m * tiles_n * ksplit;
    const int per_xcd = (total + 7) / 8;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    // persistent workgroups: as many as fit on the device at once (two per compute unit for the 4-wavefront shape)
    const int wg = 8 * min(per_xcd, max(1, cus / 8) * (2 / wm_rows));
    dim3 grid((unsigned)wg), block(256 * wm_rows);
    float* part = ksplit > 1 || twin ? (float*)((char*)workspace + p.bytes) : nullptr;
    float* dst = part ? part : out;
    const int64_t count = m_out * n;
    const int sum_shares_n = twin ? 2 * ksplit : ksplit;
#define QMM_GEMM_GO(WM_)                                                                                          \
    do {                                                                                                          \
        gemm_q4_k_kernel<WM_><<<grid, block, 0, s>>>(w, p.a16, p.asum, p.inv, dst, (int)m, (int)n, (int)k,       \
                                                     tiles_m, tiles_n, 1, 0, ksplit);                             \
        if (part) sum_shares(part, out, count, sum_shares_n, 0, s);                                               \
        if (p.a16_lo) { /* fp32 lhs: the residual plane, added on top */                                          \
            gemm_q4_k_kernel<WM_><<<grid, block, 0, s>>>(w, p.a16_lo, p.asum, p.inv, dst, (int)m, (int)n,        \
                                                         (int)k, tiles_m, tiles_n, 0, part ? 0 : 1, ksplit);      \
            if (part) sum_shares(part, out, count, ksplit, 1, s);                                                 \
        }                                                                                                         \
    } while (0)
    if (wm_rows == 2)
        QMM_GEMM_GO(2);
    else
        QMM_GEMM_GO(1);
#undef QMM_GEMM_GO
    return hipGetLastError();
}

}  // namespace qmm
