// Q4_0 prefill (more than 64 lhs rows) on the fp16 matrix cores with exact integer operands.
//
// Arithmetic: that of the Q4_0 path everywhere in this library.  The lhs rows are quantised to Q8_0 (32-wide blocks, fp16
// scale d_a, int8 codes: the shared block rule of qmm_device.h) and a block of weights is 32 codes q - 8 in [-8, 7] with
// an fp16 scale d_w:
//     out[m, n] = sum over blocks b of  (d_a[m, b] * d_w[n, b]) * isum_b[m, n],   isum_b = sum_32 code_a * (q - 8).
// int8 codes and q - 8 are fp16 numbers, so v_mfma_f32_32x32x16_f16 forms isum_b exactly (|isum| <= 32 * 127 * 8 in fp32),
// two instructions per block and 32 x 32 sub-tile.  What makes Q4_0 expensive on a GPU is the scale: every (lhs row, weight
// column, block) has its own, so each block's dots need their own multiply by a rank-one matrix d_a d_w^T on the vector
// ALUs.  Here the matrix cores make that rank-one matrix too: one more instruction per sub-tile and block with d_a in
// element 0 of the A operand and d_w in element 0 of the B operand (all other elements zero) gives S[m, n] = d_a * d_w,
// exact (two fp16 factors), in the register layout of the dots; the lanes are left with one fused multiply-add per output
// element and block, acc += isum * S.  (The int8 kernels in gemm_q4_0.hip need a convert, a multiply and a multiply-add per
// element and block: 24 vector instructions per matrix-core instruction against about 6 here per product instruction.)
//
// Structure: that of gemm_planes.hip.  A prologue launch (a) turns the weights into a plane of q - 8 as fp16 in the LDS image
// of the GEMM's weight tiles plus a table of the block scales, (b) quantises the lhs rows and stores the codes as fp16 in
// natural k order plus a table of their scales, (c) zeroes the output tiles that the GEMM cuts in two along K.  The GEMM: one
// persistent workgroup of 8 wavefronts per compute unit, 256 x 128 tiles, K in steps of 64 (two blocks), lhs 32 KB + weights
// 16 KB per step global -> LDS directly into rings of three buffers, the scales of eight blocks (256 k) at a time into two
// alternating tables.  K must be a multiple of 256.
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "gemm_lhs.h"
#include "gemm_tile.h"
#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int TM = 256, TN = 128;
constexpr int kABuf = TM * 128, kBBuf = TN * 128;
constexpr int kDaBuf = TM * 16;  // fp16 scales of 8 blocks for 256 lhs rows
constexpr int kDwBuf = TN * 16;  // the same for 128 weight columns
constexpr int kOffA = 0, kOffB = kOffA + 3 * kABuf, kOffDa = kOffB + 3 * kBBuf, kOffDw = kOffDa + 2 * kDaBuf;
constexpr int kQ40Lds = kOffDw + 2 * kDwBuf;
static_assert(kQ40Lds <= kLdsPerCu, "Q4_0 plane kernel LDS");

struct Q40Space {
    _Float16* a16;    // [m_pad][k]      lhs codes, natural order
    uint16_t* da;     // [m_pad][k / 32] lhs block scales (fp16 bits)
    uint8_t* planes;  // [tiles_n][k / 64][16 KB]
    uint16_t* dw;     // [tiles_n][k / 256][128][8] weight block scales (fp16 bits)
    int64_t bytes;
};
// The lhs part at `lhs_base`, the weight part at `w_base` (directly behind the lhs part if null: one workspace holds both).
Q40Space q40_space(void* lhs_base, int64_t m, int64_t n, int64_t k, void* w_base = nullptr) {
    auto up = [](int64_t v) { return (v + 255) / 256 * 256; };
    const int64_t m_pad = (m + TM - 1) / TM * TM, tiles_n = (n + TN - 1) / TN;
    Q40Space p;
    int64_t off = 0;
    p.a16 = (_Float16*)((uint8_t*)lhs_base + off);
    off += up(m_pad * k * 2);
    p.da = (uint16_t*)((uint8_t*)lhs_base + off);
    off += up(m_pad * (k / 32) * 2);
    uint8_t* wb = w_base ? (uint8_t*)w_base - off : (uint8_t*)lhs_base;
    p.planes = wb + off;
    off += up(tiles_n * (k / 64) * kBBuf);
    p.dw = (uint16_t*)(wb + off);
    off += up(tiles_n * (k / 256) * kDwBuf);
    p.bytes = off;
    return p;
}

__device__ __forceinline__ uint32_t pack_codes(int a, int b) { return pack_half2((float)a, (float)b); }

// Weights: one workgroup of 256 threads per (n_tile, 256 k, quarter of the tile's columns); thread t takes the 16-byte piece
// t % 8 of column t / 8 in each of the four steps.  Piece p of a step holds k = 8 p .. 8 p + 7 (natural order).
__device__ __forceinline__ void q4_0_plane_part(int tile_n, int grp, int quarter, const uint8_t* __restrict__ w, int n, int nblk32,
                                                uint8_t* __restrict__ planes, uint16_t* __restrict__ dw) {
    constexpr int COLS = TN / 4, BYTES = 8 * Q4_0_BPB;  // 144 bytes of a column's eight blocks
    __shared__ __attribute__((aligned(16))) uint16_t stage[COLS * BYTES / 2];
    const int tid = (int)threadIdx.x, col0 = quarter * COLS;
    for (int i = tid; i < COLS * (BYTES / 2); i += 256) {
        const int c = i / (BYTES / 2), e = i - c * (BYTES / 2);
        const int64_t src_col = min(tile_n * TN + col0 + c, n - 1);
        stage[i] = ((const uint16_t*)(w + (src_col * nblk32 + (int64_t)grp * 8) * Q4_0_BPB))[e];
    }
    __syncthreads();
    const int piece = tid & 7, col = col0 + (tid >> 3);
    const bool live = tile_n * TN + col < n;
    const uint16_t* blk16 = stage + (tid >> 3) * (BYTES / 2);
    const uint32_t dst_in_tile = (uint32_t)(col * 128 + ((piece ^ ((col >> 1) & 7)) << 4));
    const int64_t steps_row = (int64_t)nblk32 / 2;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        // k = 64 c + 8 piece + (0..7): block 2 c + piece / 4, elements e0 .. e0 + 7 with e0 = 8 (piece % 4); elements 0..15 are
        // the low nibbles of the block's 16 code bytes, 16..31 the high nibbles
        const int j = 2 * c + (piece >> 2), e0 = 8 * (piece & 3);
        const uint16_t* qs = blk16 + j * 9 + 1 + ((e0 & 15) >> 1);
        const int sh = e0 >= 16 ? 4 : 0;
        int v[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t two = qs[i];
            v[2 * i] = live ? (int)((two >> sh) & 15u) - 8 : 0;
            v[2 * i + 1] = live ? (int)((two >> (8 + sh)) & 15u) - 8 : 0;
        }
        uint8_t* tile = planes + ((int64_t)tile_n * steps_row + (int64_t)grp * 4 + c) * kBBuf;
        *(uint4*)(tile + dst_in_tile) = make_uint4(pack_codes(v[0], v[1]), pack_codes(v[2], v[3]), pack_codes(v[4], v[5]), pack_codes(v[6], v[7]));
    }
    if (piece == 0) {
        uint32_t d[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = live ? (uint32_t)blk16[(2 * i) * 9] | (uint32_t)blk16[(2 * i + 1) * 9] << 16 : 0u;
        *(uint4*)(dw + (((int64_t)tile_n * (nblk32 / 8) + grp) * TN + col) * 8) = make_uint4(d[0], d[1], d[2], d[3]);
    }
}

// lhs: one row per workgroup; thread t takes 8 values of every 2048 (four threads per 32-wide block).
template <typename AT>
__device__ __forceinline__ void q4_0_lhs_row(int row, const AT* __restrict__ a, int k, _Float16* __restrict__ a16, uint16_t* __restrict__ da) {
    const int tid = (int)threadIdx.x;
    const AT* ar = a + (int64_t)row * k;
    for (int i = tid * 8; i < k; i += 2048) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = load_f32(ar, i + e);
        float amax = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                           fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
        amax = fmaxf(amax, dpp_move<0xB1>(amax));
        amax = fmaxf(amax, dpp_move<0x4E>(amax));  // the four threads of a block hold its amax
        uint16_t dh;
        const float id = q8_0_block_rule(amax, dh);
        int q[8];
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = q8_0_code(v[e], id);
        *(uint4*)(a16 + (int64_t)row * k + i) = make_uint4(pack_codes(q[0], q[1]), pack_codes(q[2], q[3]), pack_codes(q[4], q[5]), pack_codes(q[6], q[7]));
        if ((tid & 3) == 0) da[(int64_t)row * (k / 32) + (i >> 5)] = dh;
    }
}

template <typename AT>
__global__ __launch_bounds__(256) void q4_0_planes_prologue_kernel(const uint8_t* __restrict__ w, int nblk32, Q40Space sp, int conv,
                                                                   const AT* __restrict__ a, int k, int lhs_rows, SplitTiles z) {
    const int b = (int)blockIdx.x;
    if (b < conv) {
        const int t = b >> 2, grp = t / z.tiles_n;
        q4_0_plane_part(t - grp * z.tiles_n, grp, b & 3, w, z.n, nblk32, sp.planes, sp.dw);
    } else if (b < conv + lhs_rows) {
        q4_0_lhs_row<AT>(b - conv, a, k, sp.a16, sp.da);
    } else if (z.part) {
        zero_flat(z.out, z.part, (int64_t)z.m * z.n, b - conv - lhs_rows);
    } else {
        const int e = b - conv - lhs_rows;
        zero_split_tile_part(z, e >> 6, (e >> 3) & 7, e & 7);
    }
}

}  // namespace

__global__ __launch_bounds__(512, 1) void gemm_q4_0_planes_kernel(const uint8_t* __restrict__ planes, const uint16_t* __restrict__ dw,
                                                                 const _Float16* __restrict__ a16, const uint16_t* __restrict__ da,
                                                                 float* __restrict__ out, int m, int n, int k, int tiles_m, int tiles_n,
                                                                 int allow_split, float* __restrict__ part) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int nl = lane & 31, g = lane >> 5;
    const int ngrp_row = k >> 8;  // groups of eight blocks in a row
    const uint32_t fb0 = (uint32_t)(kOffB + (wn * 64 + nl) * 128 + ((g ^ ((nl >> 1) & 7)) << 4));
    const int a_minus_b = (kOffA + wm * 64 * 128) - (kOffB + wn * 64 * 128);
    const float16v zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const uint32_t lane16 = (uint32_t)(lane * 16);
    // scale operands: this lane's rows / columns of the two tables (element 0 of the g = 0 lanes carries the scale)
    const uint32_t da_at = (uint32_t)(kOffDa + (wm * 64 + nl) * 16), dw_at = (uint32_t)(kOffDw + (wn * 64 + nl) * 16);
    const uint32_t keep = g ? 0u : 0xffffu;

    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8, wgs_per_xcd = (int)(gridDim.x >> 3);
    const int xcd_base = (int)(blockIdx.x & 7) * per_xcd, n_x = max(0, min(per_xcd, total - xcd_base));
    // part != null: every tile in four K quarters, one unit each.  Quarters 0 and 1 meet in `out`, 2 and 3 in `part` (both zeroed
    // beforehand; two terms per element each, so neither sum depends on the order), and a launch behind this one adds `part` to `out`.
    int full;
    const int units = part ? 4 * n_x : xcd_units(n_x, wgs_per_xcd, ngrp_row, allow_split, full);
    for (int u = (int)(blockIdx.x >> 3); u < units; u += wgs_per_xcd) {
        TileUnit unit;
        if (part) {
            const int q = u & 3, b0 = q * ngrp_row / 4, b1 = (q + 1) * ngrp_row / 4;
            unit.tile = xcd_base + (u >> 2); unit.kb0 = b0; unit.nb = b1 - b0; unit.half = 1;
        } else {
            unit = xcd_unit(u, xcd_base, full, ngrp_row);
        }
        float* __restrict__ dst = part && (u & 2) ? part : out;
        const int ngrp = __builtin_amdgcn_readfirstlane(unit.nb), ns = ngrp * 4;  // this unit's share of K: groups, steps
        const int kg0 = __builtin_amdgcn_readfirstlane(unit.kb0), unit_half = __builtin_amdgcn_readfirstlane(unit.half);
        int tile_m, tile_n;
        tile_order(unit.tile, tiles_m, tiles_n, kTileGm, tile_m, tile_n);
        tile_m = __builtin_amdgcn_readfirstlane(tile_m);
        tile_n = __builtin_amdgcn_readfirstlane(tile_n);
        const int m0 = tile_m * TM, n0 = tile_n * TN;

        uint32_t a_off[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
            a_off[i] = (uint32_t)((lane >> 3) * (k * 2) + (((lane & 7) ^ ((4 * i + (lane >> 4)) & 7)) << 4));
        const uint8_t* a_base = (const uint8_t*)a16 + ((int64_t)(m0 + wave * 32) * k + (int64_t)kg0 * 256) * 2;
        const uint8_t* b_base = planes + ((int64_t)tile_n * ngrp_row + kg0) * 4 * kBBuf;
        // tables: lhs rows wave * 32 + lane (lanes 0..31), 16 bytes = eight block scales each; weight columns: 256 bytes per wavefront
        const uint32_t da_off = (uint32_t)(lane * ((k / 32) * 2));
        const uint8_t* da_base = (const uint8_t*)da + ((int64_t)(m0 + wave * 32) * (k / 32) + (int64_t)kg0 * 8) * 2;
        const uint8_t* dw_base = (const uint8_t*)dw + ((int64_t)tile_n * ngrp_row + kg0) * kDwBuf + wave * 256;

        auto issue_A1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const uint32_t dst = lds0 + kOffA + buf * kABuf + wave * 4096;
            load16_to_lds(a_off[i & 1], a_base + (int64_t)min(step, ns - 1) * 128 + (int64_t)i * 16 * k,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(dst + i * 1024)));
        };
        auto issue_B1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const int piece = (wave * 2 + i) * 1024;
            load16_to_lds(lane16, b_base + (int64_t)min(step, ns - 1) * kBBuf + piece,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffB + buf * kBBuf + piece)));
        };
        auto issue_tables = [&](int grp) __attribute__((always_inline)) {
            const int gc = min(grp, ngrp - 1), buf = grp & 1;
            if (lane < 32)
                load16_to_lds(da_off, da_base + (int64_t)gc * 16,
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffDa + buf * kDaBuf + wave * 512)));
            if (lane < 16)
                load16_to_lds(lane16, dw_base + (int64_t)gc * kDwBuf,
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffDw + buf * kDwBuf + wave * 256)));
        };

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
        half8 afr[2][2], bfr[2][2];

        // ---- tile prologue
        __syncthreads();  // every wavefront is done with the previous tile's LDS contents
        issue_tables(0);
#pragma unroll
        for (int i = 0; i < 4; i++) issue_A1(0, 0, i);
#pragma unroll
        for (int i = 0; i < 4; i++) issue_A1(1, 1, i);
        issue_B1(0, 0, 0);
        issue_B1(0, 0, 1);
        issue_B1(1, 1, 0);
        issue_B1(1, 1, 1);
        wait_vmcnt<0>();
        int abuf = 0;  // buffer of the current step (step % 3), lhs and weights alike
        __syncthreads();

        uint32_t fa = 0, fbb = 0;
        auto step_bases = [&](int ab) __attribute__((always_inline)) {
            int ao = a_minus_b + ab * kABuf, bo = ab * kBBuf;
            asm volatile("" : "+s"(ao), "+s"(bo));
            fa = fb0 + (uint32_t)ao;
            fbb = fb0 + (uint32_t)bo;
        };
        auto read_frags = [&](int f, int slot) __attribute__((always_inline)) {
#pragma unroll
            for (int mi = 0; mi < 2; mi++) afr[slot][mi] = *(const half8*)(smem + (uint32_t)((fa ^ (uint32_t)(f << 5)) + mi * 4096));
#pragma unroll
            for (int ni = 0; ni < 2; ni++) bfr[slot][ni] = *(const half8*)(smem + (uint32_t)((fbb ^ (uint32_t)(f << 5)) + ni * 4096));
        };
        auto mfma_slice = [&](int slot, auto&& between) __attribute__((always_inline)) {
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[slot][mi], bfr[slot][ni], P[mi][ni], 0, 0, 0);
                    between(mi * 2 + ni);
                    __builtin_amdgcn_sched_barrier(0);
                }
        };
        // the scale operands of block j (0..7) of the table in buffer tb: d_a of this lane's two row groups, d_w of its two column groups
        // (kept as whole operands: element 0 carries the scale, the other seven stay zero for the whole kernel)
        HalfPack oa[2], ob[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) oa[i].u[e] = ob[i].u[e] = 0u;
        auto read_scales = [&](int tb, int j) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                oa[i].u[0] = (uint32_t)(*(const uint16_t*)(smem + da_at + tb * kDaBuf + i * 512 + j * 2)) & keep;
                ob[i].u[0] = (uint32_t)(*(const uint16_t*)(smem + dw_at + tb * kDwBuf + i * 512 + j * 2)) & keep;
            }
        };
        auto scale_tile = [&](int t) __attribute__((always_inline)) {
            return __builtin_amdgcn_mfma_f32_32x32x16_f16(oa[t >> 1].h, ob[t & 1].h, zero16, 0, 0, 0);
        };
        // acc += isum * (d_a d_w^T) for the finished block whose dots are in P and whose scale operands are in oa / ob, sub-tile by
        // sub-tile in front of the instruction that restarts that sub-tile's P with the first slice of the next block (slot 0)
        auto finish_and_restart = [&](bool restart, auto&& between) __attribute__((always_inline)) {
            // one sub-tile: the multiply-adds, then the instruction that restarts its dots
            auto finish_tile = [&](int t, const float16v& S) __attribute__((always_inline)) {
                const int mi = t >> 1, ni = t & 1;
#pragma unroll
                for (int r = 0; r < 16; r++) acc[mi][ni][r] = fmaf(P[mi][ni][r], S[r], acc[mi][ni][r]);
                // (pins the update here: left alone, the compiler defers the multiply-adds of several blocks and keeps their
                // dots and scale products in scratch memory until then)
                asm volatile("" : "+v"(acc[mi][ni]));
                __builtin_amdgcn_sched_barrier(0);
                if (restart) P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][mi], bfr[0][ni], zero16, 0, 0, 0);
            };
            // two scale products are in flight ahead of the sub-tile that uses them
            const float16v S0 = scale_tile(0), S1 = scale_tile(1);
            __builtin_amdgcn_sched_barrier(0);
            finish_tile(0, S0);
            const float16v S2 = scale_tile(2);
            between(0);
            __builtin_amdgcn_sched_barrier(0);
            finish_tile(1, S1);
            const float16v S3 = scale_tile(3);
            between(1);
            __builtin_amdgcn_sched_barrier(0);
            finish_tile(2, S2);
            between(2);
            __builtin_amdgcn_sched_barrier(0);
            finish_tile(3, S3);
            between(3);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto nothing = [](int) __attribute__((always_inline)) {};

        // One phase = from the barrier inside step s - 1 to the barrier inside step s.  A step holds two blocks: X (slices 0, 1) and
        // Y (slices 2, 3).  In flight at the top: the second slice of the previous step's Y (operands in slot 1).
        auto phase = [&](int grp, auto CC) __attribute__((always_inline)) {
            constexpr int c = decltype(CC)::value;
            const int s = grp * 4 + c;
            const int tb = grp & 1;
            step_bases(abuf);
            read_frags(0, 0);
            __builtin_amdgcn_sched_barrier(0);
            const int ab2 = abuf == 0 ? 2 : abuf - 1;  // (step + 2) % 3
            if (s > 0) mfma_slice(1, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 0); });  // Y of step s - 1, second slice
            else issue_A1(s + 2, ab2, 0);
            issue_B1(s + 2, ab2, 0);
            if constexpr (c == 2) issue_tables(grp + 1);
            __builtin_amdgcn_sched_barrier(0);
            read_frags(1, 1);
            __builtin_amdgcn_sched_barrier(0);
            // Y of step s - 1 is complete (its scale operands were read during that step): finish it, start X
            if (s > 0) {
                finish_and_restart(true, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 1); });
            } else {
#pragma unroll
                for (int t = 0; t < 4; t++) P[t >> 1][t & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t >> 1], bfr[0][t & 1], zero16, 0, 0, 0);
                issue_A1(s + 2, ab2, 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            read_scales(tb, 2 * c);  // X's
            read_frags(2, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(1, [&](int i) __attribute__((always_inline)) {  // X, second slice
                if (i == 1) issue_B1(s + 2, ab2, 1);
                if (i == 3) issue_A1(s + 2, ab2, 2);
            });
            read_frags(3, 1);
            __builtin_amdgcn_sched_barrier(0);
            finish_and_restart(true, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 3); });  // finish X, start Y
            read_scales(tb, 2 * c + 1);  // Y's, used at the top of the next phase (or after the loop)
            // everything issued before this phase has landed: lhs and weights of step s + 1 (and, after phase 3, the tables)
            if constexpr (c == 2) wait_vmcnt<8>();
            else wait_vmcnt<6>();
            __syncthreads();
            abuf = abuf == 2 ? 0 : abuf + 1;
        };
        for (int grp = 0; grp < ngrp; grp++) {
            phase(grp, std::integral_constant<int, 0>{});
            phase(grp, std::integral_constant<int, 1>{});
            phase(grp, std::integral_constant<int, 2>{});
            phase(grp, std::integral_constant<int, 3>{});
        }
        mfma_slice(1, nothing);  // second slice of the last block
        finish_and_restart(false, nothing);

        // ---- tile epilogue: store
        {
            const int col0 = n0 + wn * 64 + nl, col1 = col0 + 32;
            const bool c0_ok = col0 < n, c1_ok = col1 < n;
#pragma unroll
            for (int mi = 0; mi < 2; mi++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                    if (row < m) {
                        float* o_ = dst + (int64_t)row * n;
                        const float v0 = acc[mi][0][r], v1 = acc[mi][1][r];
                        if (unit_half) {  // one of the two K halves of this tile: out holds zero or the other half
                            if (c0_ok) unsafeAtomicAdd(o_ + col0, v0);
                            if (c1_ok) unsafeAtomicAdd(o_ + col1, v1);
                        } else {
                            if (c0_ok) __builtin_nontemporal_store(v0, o_ + col0);
                            if (c1_ok) __builtin_nontemporal_store(v1, o_ + col1);
                        }
                    }
                }
            }
        }
    }
}

bool gemm_q4_0_planes_wanted(int64_t m, int64_t n, int64_t k) {
    // QMM_Q4_0_PLANES=1 (read once) sends every shape with more than 16 lhs rows here, for tests of the kernel on small problems
    static const bool force = getenv("QMM_Q4_0_PLANES") != nullptr && atoi(getenv("QMM_Q4_0_PLANES")) == 1;
    if (k % 256 || k < 256 || kernel_disabled("q4_0_planes")) return false;
    if (force) return m > 16;
    // Against passes of the 16-row int8 kernel (one launch that quantises the lhs, then a launch per 16 rows), both in microseconds
    // as fitted on this part (W: millions of weights).  Measured, 16 / 32 / 64 rows in passes and the planes at 65 rows: 4096 x 4096
    // 11.4 / 15.6 / 23.9 and 38; 14336 x 4096 12.8 / 22.4 / 41.3 and 90; 4096 x 14336 16.0 / 30.3 / 58.0 and 118; 1024 x 4096
    // 8.2 / 13.0 / 22 and 33.
    const double W = (double)n * (double)k * 1e-6;
    const double passes_us = 3.5 + (double)((m + 15) / 16) * (4.5 + 0.082 * W + (k > 4096 ? 3.0 : 0.0));
    const double planes_us = 28.0 + 1.0 * W + (k > 4096 ? 28.0 : 0.0) + 0.02 * (double)m;
    return m > 16 && passes_us > planes_us;
}

int64_t gemm_q4_0_planes_workspace_bytes(int64_t m, int64_t n, int64_t k);

namespace {
bool quarters_wanted(int64_t m, int64_t n, int64_t k) { return !kernel_disabled("planes_quarters") && few_tiles_for_quarters(m, n, k); }
int64_t part_bytes(int64_t m, int64_t n, int64_t k) { return quarters_wanted(m, n, k) ? (m * n * 4 + 255) / 256 * 256 : 0; }
// convert: the weight plane in `sp` is made from `w` in the preparation launch; otherwise it was made earlier.
// part: room for a second m x n result (quarter mode), used where few_tiles_for_quarters says so.
hipError_t run_q4_0_planes(const void* lhs, int lhs_dtype, const uint8_t* w, bool convert, int64_t m, int64_t n, int64_t k, float* out,
                           const Q40Space& sp, float* part, hipStream_t s) {
    if (!quarters_wanted(m, n, k)) part = nullptr;
    hipError_t e = allow_full_lds<gemm_q4_0_planes_kernel>();
    if (e != hipSuccess) return e;
    const int tiles_m = (int)((m + TM - 1) / TM), tiles_n = (int)((n + TN - 1) / TN), ngrp = (int)(k / 256);
    const int total = tiles_m * tiles_n, per_xcd = (total + 7) / 8;
    // Tiles for no more than half of the compute units: a workgroup per compute unit all the same, and the unit arithmetic cuts
    // every tile in two K halves (a tile's time is set by K).
    const int per_xcd_cus = std::max(1, compute_units() / 8);
    const bool halve_all = 2 * per_xcd <= per_xcd_cus && ngrp >= 2;
    const int wg = 8 * (halve_all || part ? per_xcd_cus : std::min(per_xcd, per_xcd_cus));
    SplitTiles z = split_tiles(out, m, n, tiles_m, tiles_n, ngrp, wg);
    if (part) {
        z.max_split = 0;
        z.part = part;
    }
    const int64_t zero_blocks = part ? (m * n + kZeroFlatFloats - 1) / kZeroFlatFloats : (int64_t)z.max_split * 64;
    const int64_t conv = convert ? (int64_t)tiles_n * ngrp * 4 : 0, blocks = conv + m + zero_blocks;
    if (blocks > INT32_MAX) return hipErrorInvalidValue;
    const dim3 pgrid((unsigned)blocks);
    if (lhs_dtype == QMM_F32)
        q4_0_planes_prologue_kernel<float><<<pgrid, dim3(256), 0, s>>>(w, (int)(k / 32), sp, (int)conv, (const float*)lhs, (int)k, (int)m, z);
    else
        q4_0_planes_prologue_kernel<uint16_t><<<pgrid, dim3(256), 0, s>>>(w, (int)(k / 32), sp, (int)conv, (const uint16_t*)lhs, (int)k, (int)m, z);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    gemm_q4_0_planes_kernel<<<dim3((unsigned)wg), dim3(512), kQ40Lds, s>>>(sp.planes, sp.dw, sp.a16, sp.da, out, (int)m, (int)n, (int)k,
                                                                         tiles_m, tiles_n, z.max_split > 0 ? 1 : 0, part);
    if (part) return launch_add_part(out, part, m * n, s);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_gemm_q4_0_planes(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out,
                                   void* workspace, hipStream_t s) {
    const Q40Space sp = q40_space(workspace, m, n, k);
    return run_q4_0_planes(lhs, lhs_dtype, w, true, m, n, k, out, sp, (float*)((uint8_t*)workspace + sp.bytes), s);
}
int64_t gemm_q4_0_planes_workspace_bytes(int64_t m, int64_t n, int64_t k) { return q40_space(nullptr, m, n, k).bytes + part_bytes(m, n, k); }

// The weight plane kept across calls: the conversion alone, and the GEMM over a plane made by it (workspace: the lhs part).
int64_t repacked_q4_0_bytes(int64_t n, int64_t k) { return q40_space(nullptr, 0, n, k).bytes; }
hipError_t launch_repack_q4_0(const uint8_t* w, int64_t n, int64_t k, void* packed, hipStream_t s) {
    const Q40Space sp = q40_space(nullptr, 0, n, k, packed);
    const int tiles_n = (int)((n + TN - 1) / TN);
    const int64_t conv = (int64_t)tiles_n * (k / 256) * 4;
    if (conv > INT32_MAX) return hipErrorInvalidValue;
    SplitTiles z{};
    z.n = (int)n;
    z.tiles_n = tiles_n;
    q4_0_planes_prologue_kernel<uint16_t><<<dim3((unsigned)conv), dim3(256), 0, s>>>(w, (int)(k / 32), sp, (int)conv, nullptr, (int)k, 0, z);
    return hipGetLastError();
}
int64_t repacked_q4_0_workspace_bytes(int64_t m, int64_t n, int64_t k) { return q40_space(nullptr, m, 0, k).bytes + part_bytes(m, n, k); }
hipError_t launch_gemm_q4_0_repacked(const void* lhs, int lhs_dtype, const void* packed, int64_t m, int64_t n, int64_t k, float* out,
                                     void* workspace, hipStream_t s) {
    float* part = (float*)((uint8_t*)workspace + q40_space(nullptr, m, 0, k).bytes);
    return run_q4_0_planes(lhs, lhs_dtype, nullptr, false, m, n, k, out, q40_space(workspace, m, n, k, const_cast<void*>(packed)), part, s);
}

}  // namespace qmm
