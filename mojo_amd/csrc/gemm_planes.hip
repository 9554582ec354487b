// Prefill on the matrix cores through weight planes, in two steps: a conversion pass turns the packed weights into planes
// of exact small integers in fp16, already in the LDS image of the matrix-core operand tiles, and a GEMM streams lhs and
// plane tiles global -> LDS directly and applies the fp32 scales of the scale blocks (K-quant super-blocks, GPTQ groups) in
// the lanes.  Q5_K (more than 32 lhs rows) and Q6_K (more than 64) always come here; Q4_K and GPTQ (plain groups of 128 or
// 256) from 513 rows on large matrices, when the caller's workspace holds the planes.
//
// Arithmetic (exact products, fp32 sums):
//   Q4_K / Q5_K  w = d * (sc * q) - dmin * mn,  q <= 15 / 31, sc <= 63: one plane, sc * q <= 1953 (an fp16 integer); the min
//         term as matrix-core products of the lhs sub-block sums with -(dmin * mn), both split into fp16 hi + lo parts:
//         extra instructions per super-block in gemm_planes_kernel, extension blocks of K in gemm_planes_wide_kernel.
//   Q6_K  w = d * (sc * q),  q in [-32, 31], sc an int8 per 16 weights: sc * q reaches 4096 and odd values above
//         2048 are no fp16 numbers, so sc = 16 hi + lo (hi = sc >> 4 in [-8, 7], lo = sc & 15) gives two planes,
//         (16 hi) * q (a multiple of 16 with at most 9 significant bits) and lo * q (<= 480), both exact.  Its GEMM
//         (gemm_planes2_kernel) multiplies both planes of a K step with the same lhs operands.
//   GPTQ  w = s * (q - zero),  q - zero in [-16, 14]: one plane, no zero-point term left.
// The planes cost workspace (2 bytes per weight and plane) and one pass over the weights (tens of microseconds at
// the sizes this path is chosen for); they buy a GEMM whose only vector-ALU work is the change of scale.
//
// Three GEMM kernels: gemm_planes_wide_kernel (one plane, 256 x 256 or 256 x 192 tiles, accumulators in units of the
// current block's scale; large problems), gemm_planes2_kernel (two planes, 256 x 128 tiles, the same accumulator scheme),
// gemm_planes_kernel (one plane, 256 x 128 tiles, a second accumulator set per super-block and the min term in the kernel;
// problems with fewer than 160 tiles of 256 x 256).
//
// Plane layout: [n_tile][plane * steps + step][128 columns][64 halfs] with the 16-byte pieces of a column's row at
// piece index p ^ ((column / 2) % 8) (the swizzle of the tile kernel's LDS buffers), piece p = 2 f + g holding the
// weights k = 64 step + 32 g + 8 f + (0,2,1,3,4,6,5,7)[slot] (the lhs order kLhsOrderTile): one (tile, step) is 16 KB
// of contiguous memory that goes to LDS as it is.  Tables per (n_tile, scale block): the scale as fp32 [128], and for
// gemm_planes_kernel the min operands -(dmin * mn) split exactly into fp16 hi + lo, [128 columns][8 hi, 8 lo].
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
constexpr int kABuf = TM * 128, kBBuf = TN * 128, kSBuf = TM * 32, kMBuf = TN * 32, kDBuf = TN * 4;
constexpr int kOffA = 0, kOffB = kOffA + 3 * kABuf, kOffS = kOffB + 3 * kBBuf, kOffM = kOffS + kSBuf, kOffD = kOffM + kMBuf;
constexpr int kOffInv = kOffD + kDBuf, kPlanesLds = kOffInv + TM * 4;
static_assert(kPlanesLds <= kLdsPerCu, "planes kernel LDS");

struct PlaneSpace {
    uint8_t* planes;  // [tiles_n][nplanes * steps][16 KB]
    float* dtab;      // [tiles_n][nblk][128]
    uint8_t* mtab;    // [tiles_n][nblk][128][32 bytes]   (Q5_K)
    int64_t bytes;
};
// nblk_tile: blocks of four steps per 128-column tile and plane (the super-blocks, plus the wide GEMM's extension blocks)
// dblocks: scale blocks per tile (GPTQ groups of 128: two per 256 k)
PlaneSpace plane_space(void* base, int64_t n, int64_t k, int nplanes, bool with_mtab, int64_t nblk_tile, int64_t dblocks = 0) {
    auto up = [](int64_t v) { return (v + 255) / 256 * 256; };
    const int64_t tiles_n = (n + TN - 1) / TN, nblk = k / 256;
    PlaneSpace p;
    int64_t off = 0;
    p.planes = (uint8_t*)base + off;
    off += up(tiles_n * nplanes * nblk_tile * 4 * kBBuf);
    p.dtab = (float*)((uint8_t*)base + off);
    off += up(tiles_n * (dblocks ? dblocks : nblk_tile) * kDBuf);
    p.mtab = with_mtab ? (uint8_t*)base + off : nullptr;
    off += with_mtab ? up(tiles_n * nblk * kMBuf) : 0;
    p.bytes = off;
    return p;
}

// Which GEMM serves a single-plane encoding: the 256 x 256 tiles from this many of them on.  Up to 256 tiles the wide kernel
// takes one round whatever their number, the 256 x 128 kernels' time grows with it (K halves balance their last round):
// 2048 rows x 4096 columns x 4096 (128 tiles) 105.8 against 92.5 us (Q5_K), 5120 columns (160 tiles) 112.5 against 132.7 us.
constexpr int kWideMinTiles = 160;
constexpr int kOptionalPlanesMinRows = 513;  // Q4_K and GPTQ have GEMM kernels that need no conversion pass: planes from three row tiles on
bool wide_tiles(int encoding, int64_t m, int64_t n) {
    if (encoding == QMM_Q6_K || kernel_disabled("planes_wide")) return false;
    const int64_t tiles_m = (m + TM - 1) / TM, tiles_nw = (n + 2 * TN - 1) / (2 * TN);
    return tiles_m * tiles_nw >= kWideMinTiles;
}
// blocks per tile: with the wide GEMM, Q4_K / Q5_K carry their min operands as one extension block per eight super-blocks
int64_t blocks_per_tile(int encoding, int64_t m, int64_t n, int64_t k) {
    const int64_t nblk = k / 256;
    return wide_tiles(encoding, m, n) ? nblk + (nblk + 7) / 8 : nblk;
}

__device__ __forceinline__ uint32_t pack_ints(int a, int b) { return pack_half2((float)a, (float)b); }

}  // namespace

// The conversion.  One workgroup of 256 threads per (n_tile, super-block, quarter of the tile's columns).  The 32 blocks of its
// columns are first copied into LDS (16-byte loads where the rows allow it, two-byte loads otherwise: rows of Q6_K blocks start
// on even addresses only) at a stride that is a multiple of four bytes, so that the code bytes can be read eight at a time; thread t then takes piece
// t % 8 of column t / 8 of each of the four steps, so that eight neighbouring threads write one 128-byte row of the tile.
// nblk_tile > nblk (the wide GEMM's layout for Q4_K / Q5_K): every 128-column tile has nblk_tile - nblk further blocks of four
// steps behind its nblk super-blocks, with scale 1, that hold the min operands: the 32 positions of super-block b in them are
// -(dmin * mn) of its eight sub-blocks as 8 hi, 8 hi, 8 lo, 8 lo parts (lhs side: the sub-block sums as hi, lo, hi, lo), zeros
// beyond the last super-block; no mtab then.  Blocks with d = 0 get a plane of zeros (the wide GEMM keeps no unit for them).
template <int ENC>
__device__ __forceinline__ void planes_from_kquant(int tile_n, int rb, int quarter, const uint8_t* __restrict__ w, int n, int nblk,
                                                   int nblk_tile, uint8_t* __restrict__ planes, float* __restrict__ dtab,
                                                   uint8_t* __restrict__ mtab) {
    constexpr int BPB = ENC == QMM_Q6_K ? Q6_K_BPB : ENC == QMM_Q5_K ? Q5_K_BPB : Q4_K_BPB;
    constexpr int STRIDE = (BPB + 3) / 4 * 4;  // 212 for Q6_K
    constexpr int NPL = ENC == QMM_Q6_K ? 2 : 1;
    constexpr int COLS = TN / 4;
    __shared__ __attribute__((aligned(16))) uint16_t stage[COLS * STRIDE / 2];
    const int tid = (int)threadIdx.x, col0 = quarter * COLS;
    // Rows that are whole 16-byte pieces (every row of Q4_K and Q5_K; Q6_K where K is a multiple of 2048) in a 16-byte aligned
    // tensor: the blocks come as aligned 16-byte loads (a Q6_K block starts 0, 2, .. 14 bytes into its first piece and ends with
    // its row at the latest) and are spread into the stage two bytes at a time.  Timing of the Q6_K conversion of 14336 x 4096
    // with two-byte loads: 75 us, of which 30 were the loads.
    const bool wide = ((uintptr_t)w & 15) == 0 && ((int64_t)nblk * BPB) % 16 == 0;
    if (wide) {
        constexpr int NP = (14 + BPB + 15) / 16;  // pieces that cover a block wherever it starts
        for (int i = tid; i < COLS * NP; i += 256) {
            const int c = i / NP, pc = i - c * NP;
            const int64_t src_col = min(tile_n * TN + col0 + c, n - 1);
            const int64_t addr = (src_col * nblk + rb) * BPB;
            const int off = (int)(addr & 15);
            if (16 * pc < off + BPB) {
                const uint4 v = *(const uint4*)(w + addr - off + 16 * pc);
                const uint32_t dw[4] = {v.x, v.y, v.z, v.w};
                const int b0 = 16 * pc - off;  // block byte of the piece's first byte (even)
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int b = b0 + 2 * j;
                    if (b >= 0 && b < BPB) stage[c * (STRIDE / 2) + (b >> 1)] = (uint16_t)(dw[j >> 1] >> (16 * (j & 1)));
                }
            }
        }
    } else {
        for (int i = tid; i < COLS * (BPB / 2); i += 256) {
            const int c = i / (BPB / 2), e = i - c * (BPB / 2);
            const int64_t src_col = min(tile_n * TN + col0 + c, n - 1);
            stage[c * (STRIDE / 2) + e] = ((const uint16_t*)(w + (src_col * nblk + rb) * BPB))[e];
        }
    }
    __syncthreads();
    const int piece = tid & 7, g = piece & 1, f = piece >> 1;
    const int64_t steps_row = (int64_t)nblk_tile * 4;
    {
        const int col = col0 + (tid >> 3), ncol = tile_n * TN + col;
        const uint8_t* blk = (const uint8_t*)stage + (tid >> 3) * STRIDE;
        const uint16_t dbits = *(const uint16_t*)(blk + (ENC == QMM_Q6_K ? 208 : 0));
        const bool in_n = ncol < n, live = in_n && (dbits & 0x7fffu) != 0;  // live: the column exists and its block has a scale
        const uint32_t dst_in_tile = (uint32_t)(col * 128 + ((piece ^ ((col >> 1) & 7)) << 4));
        // Q4_K / Q5_K header fields of this column's block
        uint32_t sc5[8], mn5[8];
        uint2 fifth = make_uint2(0, 0);
        if constexpr (ENC != QMM_Q6_K) {
            const uint32_t s3[3] = {*(const uint32_t*)(blk + 4), *(const uint32_t*)(blk + 8), *(const uint32_t*)(blk + 12)};
#pragma unroll
            for (int q = 0; q < 8; q++) q4k_scale_min(q, s3, sc5[q], mn5[q]);
            if constexpr (ENC == QMM_Q5_K) fifth = *(const uint2*)(blk + 16 + 8 * f);  // fifth bits of elements 8 f .. 8 f + 7 of every sub-block
        }
        // Codes to fp16 without a conversion instruction: the nibble byte (nibble in its high half) under a byte that holds the
        // remaining code bits below 0x54 reads as 0x5400 + (code << 4) = 64 + code; two byte permutes per dword put the eight
        // codes in the piece's element order (0, 2, 1, 3, 4, 6, 5, 7), a packed subtraction takes the 64 (and Q6_K's 32) off and
        // a packed multiplication by the scale gives the plane values, all exact small integers.
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        auto pair = [](uint32_t x) __attribute__((always_inline)) { return __builtin_bit_cast(half2v, x); };
        auto bits = [](half2v x) __attribute__((always_inline)) { return __builtin_bit_cast(uint32_t, x); };
        auto both = [](float x) __attribute__((always_inline)) {
            half2v r = {(_Float16)x, (_Float16)x};
            return r;
        };
#pragma unroll
        for (int c = 0; c < 4; c++) {
            // the eight weights 64 c + 32 g + 8 f + (0..7) of the super-block: their code bytes are eight neighbours
            uint2 lo4, hi4;
            half2v off, s0, s1 = both(0.0f);
            if constexpr (ENC == QMM_Q6_K) {
                const int h = c >> 1, quad = (2 * c + g) & 3;
                // (columns are 212 bytes apart in the stage: four-byte reads)
                const uint32_t* qlp = (const uint32_t*)(blk + 64 * h + (quad & 1) * 32 + 8 * f);
                const uint32_t* qhp = (const uint32_t*)(blk + 128 + 32 * h + 8 * f);
                const uint2 ql = make_uint2(qlp[0], qlp[1]), qh = make_uint2(qhp[0], qhp[1]);
                const int sc = (int)(int8_t)blk[192 + 8 * h + 2 * quad + (f >> 1)];
                s0 = both(live ? (float)((sc >> 4) * 16) : 0.0f);  // sc = 16 hi + lo
                s1 = both(live ? (float)(sc & 15) : 0.0f);
                lo4 = (quad & 2) ? make_uint2(ql.x & 0xF0F0F0F0u, ql.y & 0xF0F0F0F0u) : make_uint2((ql.x << 4) & 0xF0F0F0F0u, (ql.y << 4) & 0xF0F0F0F0u);
                hi4 = make_uint2(((qh.x >> (2 * quad)) & 0x03030303u) | 0x54545454u, ((qh.y >> (2 * quad)) & 0x03030303u) | 0x54545454u);
                off = both(96.0f);
            } else {
                const int sb = 2 * c + g;
                const uint2 qs = *(const uint2*)(blk + (ENC == QMM_Q5_K ? 48 : 16) + 32 * c + 8 * f);
                s0 = both(live ? (float)sc5[sb] : 0.0f);
                lo4 = g ? make_uint2(qs.x & 0xF0F0F0F0u, qs.y & 0xF0F0F0F0u) : make_uint2((qs.x << 4) & 0xF0F0F0F0u, (qs.y << 4) & 0xF0F0F0F0u);
                if constexpr (ENC == QMM_Q5_K) hi4 = make_uint2(((fifth.x >> sb) & 0x01010101u) | 0x54545454u, ((fifth.y >> sb) & 0x01010101u) | 0x54545454u);
                else hi4 = make_uint2(0x54545454u, 0x54545454u);
                off = both(64.0f);
            }
            // elements (0, 2), (1, 3) of the first dword, (4, 6), (5, 7) of the second
            const half2v q0 = pair(__builtin_amdgcn_perm(hi4.x, lo4.x, 0x06020400u)) - off, q1 = pair(__builtin_amdgcn_perm(hi4.x, lo4.x, 0x07030501u)) - off;
            const half2v q2 = pair(__builtin_amdgcn_perm(hi4.y, lo4.y, 0x06020400u)) - off, q3 = pair(__builtin_amdgcn_perm(hi4.y, lo4.y, 0x07030501u)) - off;
            const int64_t step = (int64_t)rb * 4 + c;
#pragma unroll
            for (int pl = 0; pl < NPL; pl++) {
                const half2v sp = pl == 0 ? s0 : s1;
                uint8_t* tile = planes + (((int64_t)tile_n * NPL + pl) * steps_row + step) * kBBuf;
                *(uint4*)(tile + dst_in_tile) = make_uint4(bits(q0 * sp), bits(q1 * sp), bits(q2 * sp), bits(q3 * sp));
            }
        }
        // tables: one thread per column
        if (piece == 0) {
            const int64_t tb = (int64_t)tile_n * nblk_tile + rb;
            dtab[tb * TN + col] = in_n ? h2f(dbits) : 0.0f;
            if constexpr (ENC != QMM_Q6_K) {
                const uint32_t ndm = ((uint32_t)(*(const uint16_t*)(blk + 2)) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
                uint32_t hi[4], lo[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t mp = in_n ? pack_half2((float)mn5[2 * q], (float)mn5[2 * q + 1]) : 0u;
                    hi[q] = pk_mul(ndm, mp);
                    lo[q] = pk_fma(ndm, mp, hi[q] ^ 0x80008000u);
                }
                if (nblk_tile > nblk) {
                    // pieces 4 (rb % 2) + (0, 1, 2, 3) of step (rb % 8) / 2 of the extension block rb / 8
                    const int xb = rb >> 3;
                    uint8_t* tile = planes + ((int64_t)tile_n * steps_row + (nblk + xb) * 4 + ((rb & 7) >> 1)) * kBBuf + col * 128;
                    const int sw = (col >> 1) & 7, p0 = (rb & 1) * 4;
                    const uint4 vh = make_uint4(hi[0], hi[1], hi[2], hi[3]), vl = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                    *(uint4*)(tile + (((p0 + 0) ^ sw) << 4)) = vh;
                    *(uint4*)(tile + (((p0 + 1) ^ sw) << 4)) = vh;
                    *(uint4*)(tile + (((p0 + 2) ^ sw) << 4)) = vl;
                    *(uint4*)(tile + (((p0 + 3) ^ sw) << 4)) = vl;
                    if ((rb & 7) == 0) dtab[((int64_t)tile_n * nblk_tile + nblk + xb) * TN + col] = 1.0f;
                    if (rb == nblk - 1) {  // the rest of the last extension block
                        for (int b2 = rb + 1; b2 < (xb + 1) * 8; b2++) {
                            uint8_t* t2 = planes + ((int64_t)tile_n * steps_row + (nblk + xb) * 4 + ((b2 & 7) >> 1)) * kBBuf + col * 128;
                            for (int q = 0; q < 4; q++) *(uint4*)(t2 + ((((b2 & 1) * 4 + q) ^ sw) << 4)) = make_uint4(0, 0, 0, 0);
                        }
                    }
                }
                if (mtab) {  // (planes kept across calls carry both forms of the min operands)
                    uint8_t* mt = mtab + (((int64_t)tile_n * nblk + rb) * TN + col) * 32;
                    *(uint4*)mt = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                    *(uint4*)(mt + 16) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                }
            }
        }
    }
}

// Everything the GEMM needs done first, in one launch of 256-thread workgroups: [0, conv) convert weights (the long part,
// so it starts first), the next m narrow one lhs row each, the rest zero the output tiles that the GEMM fills with atomic adds.
template <int ENC, typename AT>
__global__ __launch_bounds__(256) void planes_prologue_kernel(const uint8_t* __restrict__ w, int nblk, int nblk_tile, int tiles_n128,
                                                              uint8_t* __restrict__ planes, float* __restrict__ dtab,
                                                              uint8_t* __restrict__ mtab, int conv, const AT* __restrict__ a, int k,
                                                              int lhs_ext, int lhs_rows, LhsPlanes p, SplitTiles z, int twin_rows) {
    const int b = (int)blockIdx.x;
    if (b < conv) {
        const int t = b >> 2, rb = t / tiles_n128;
        planes_from_kquant<ENC>(t - rb * tiles_n128, rb, b & 3, w, z.n, nblk, nblk_tile, planes, dtab, mtab);
    } else if (b < conv + lhs_rows) {
        // (lhs_ext: extension blocks behind each lhs row, as many as the planes have when the wide GEMM follows, else none)
        prep_lhs_row<AT, kLhsOrderTile>(b - conv, a, k, p.a16, p.a16_lo, p.asum, p.inv, (int64_t)k + lhs_ext * 256, lhs_ext, twin_rows);
    } else {
        const int e = b - conv - lhs_rows;
        if (z.part) zero_flat(z.out, z.part, (int64_t)z.m * z.n, e);
        else zero_split_tile_part(z, e >> 6, (e >> 3) & 7, e & 7);
    }
}

// out += part (the second pair of K quarters of gemm_planes_kernel's quarter mode)
__global__ __launch_bounds__(256) void add_part_kernel(float* __restrict__ out, const float* __restrict__ part, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) out[i] += part[i];
}

// The GEMM over the planes.  Structure, buffers and schedule are those of gemm_q4_k_tile_kernel (see there); what differs:
// the weight operands of a step arrive ready-made (16 KB per tile and step, global -> LDS directly, two steps ahead in a
// ring of three buffers like the lhs) and the tables of a super-block come from memory.  One plane with a min term (Q5_K, Q4_K).
__global__ __launch_bounds__(512, 1) void gemm_planes_kernel(const uint8_t* __restrict__ planes, const float* __restrict__ dtab,
                                                            const uint8_t* __restrict__ mtab, const _Float16* __restrict__ a16,
                                                            const _Float16* __restrict__ asum, const float* __restrict__ inv,
                                                            float* __restrict__ out, int m, int n, int k, int tiles_m,
                                                            int tiles_n, int nblk_tile, int with_min, int accumulate, int allow_split,
                                                            float* __restrict__ part) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int nl = lane & 31, g = lane >> 5;
    const int nblk_row = k >> 8;
    const uint32_t fb0 = (uint32_t)(kOffB + (wn * 64 + nl) * 128 + ((g ^ ((nl >> 1) & 7)) << 4));
    const int a_minus_b = (kOffA + wm * 64 * 128) - (kOffB + wn * 64 * 128);
    const float16v zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8, wgs_per_xcd = (int)(gridDim.x >> 3);
    const int xcd_base = (int)(blockIdx.x & 7) * per_xcd, n_x = max(0, min(per_xcd, total - xcd_base));
    // part != null: every tile in four K quarters, one unit each.  Quarters 0 and 1 meet in `out`, 2 and 3 in `part` (both zeroed
    // beforehand; two terms per element each, so neither sum depends on the order), and a launch behind this one adds `part` to `out`.
    int full;
    const int units = part ? 4 * n_x : xcd_units(n_x, wgs_per_xcd, nblk_row, allow_split, full);
    for (int u = (int)(blockIdx.x >> 3); u < units; u += wgs_per_xcd) {
        TileUnit unit;
        if (part) {
            const int q = u & 3, b0 = q * nblk_row / 4, b1 = (q + 1) * nblk_row / 4;
            unit.tile = xcd_base + (u >> 2); unit.kb0 = b0; unit.nb = b1 - b0; unit.half = 1;
        } else {
            unit = xcd_unit(u, xcd_base, full, nblk_row);
        }
        float* __restrict__ dst = part && (u & 2) ? part : out;
        // (uniform values that come out of integer divisions live in vector registers unless told otherwise; everything
        // below that is derived from them, the base pointers above all, would follow them there)
        const int nblk = __builtin_amdgcn_readfirstlane(unit.nb), ns = nblk * 4;  // this unit's share of K
        const int kb0 = __builtin_amdgcn_readfirstlane(unit.kb0), unit_half = __builtin_amdgcn_readfirstlane(unit.half);
        int tile_m, tile_n;
        tile_order(unit.tile, tiles_m, tiles_n, kTileGm, tile_m, tile_n);
        tile_m = __builtin_amdgcn_readfirstlane(tile_m);
        tile_n = __builtin_amdgcn_readfirstlane(tile_n);
        const int m0 = tile_m * TM, n0 = tile_n * TN;
        const uint32_t lane16 = (uint32_t)(lane * 16);

        uint32_t a_off[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
            a_off[i] = (uint32_t)((lane >> 3) * (k * 2) + (((lane & 7) ^ ((4 * i + (lane >> 4)) & 7)) << 4));
        const uint8_t* a_base = (const uint8_t*)a16 + (int64_t)(m0 + wave * 32) * k * 2;
        const uint32_t s_off = (uint32_t)((wave * 32 + (lane >> 1)) * (nblk_row * 32) + (lane & 1) * 16);
        const uint8_t* s_base = (const uint8_t*)asum + (int64_t)m0 * nblk_row * 32;
        // (nblk_tile: blocks of four steps a tile holds in planes and dtab; more than the super-blocks where the planes also
        // carry the wide GEMM's extension blocks)
        const uint8_t* b_base = planes + ((int64_t)tile_n * nblk_tile + kb0) * 4 * kBBuf;
        const uint8_t* d_base = (const uint8_t*)dtab + (int64_t)tile_n * nblk_tile * kDBuf;
        const uint8_t* m_base = mtab + (int64_t)tile_n * nblk_row * kMBuf;
        auto real_blk = [&](int blk) __attribute__((always_inline)) { return kb0 + min(blk, nblk - 1); };  // super-block of the row

        auto issue_A1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const int sr = kb0 * 4 + min(step, ns - 1);
            const uint32_t dst = lds0 + kOffA + buf * kABuf + wave * 4096;
            load16_to_lds(a_off[i & 1], a_base + (int64_t)sr * 128 + (int64_t)i * 16 * k,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(dst + i * 1024)));
        };
        // the i-th (0, 1) of this wavefront's two 1 KB pieces of the weight tile of step `step`
        auto issue_B1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const int piece = (wave * 2 + i) * 1024;
            load16_to_lds(lane16, b_base + (int64_t)min(step, ns - 1) * kBBuf + piece,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffB + buf * kBBuf + piece)));
        };
        // tables and lhs sums of super-block `blk` (of this unit): every wavefront brings an eighth of each
        auto issue_tables = [&](int blk) __attribute__((always_inline)) {
            const int rb = real_blk(blk);
            if (lane < 4)
                load16_to_lds(lane16, d_base + (int64_t)rb * kDBuf + wave * 64,
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffD + wave * 64)));
            if (lane < 32)
                load16_to_lds(lane16, m_base + (int64_t)rb * kMBuf + wave * 512,
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffM + wave * 512)));
            load16_to_lds(s_off, s_base + (int64_t)rb * 32, (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffS + wave * 1024)));
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
        float dcur[2] = {0.f, 0.f};

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
        if (tid < TM) *(float*)(smem + kOffInv + tid * 4) = inv[min(m0 + tid, m - 1)];
        wait_vmcnt<0>();
        int abuf = 0;  // buffer of the current step (step % 3), lhs and weights alike
        __syncthreads();

        // Operand addresses of the current step: recomputed every phase from the buffer index behind an empty asm statement.
        // (Left to itself the compiler keeps the addresses of all three buffers in registers and rotates them, some twenty
        // registers that push accumulators out to scratch memory.)
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
        auto mfma_slice = [&](int slot, bool fresh, auto&& between) __attribute__((always_inline)) {
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    if (fresh) P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[slot][mi], bfr[slot][ni], zero16, 0, 0, 0);
                    else P[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[slot][mi], bfr[slot][ni], P[mi][ni], 0, 0, 0);
                    between(mi * 2 + ni);
                    __builtin_amdgcn_sched_barrier(0);
                }
        };
        auto rescale_tile = [&](int t) __attribute__((always_inline)) {
            const int mi = t >> 1, ni = t & 1;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[mi][ni][r] = fmaf(dcur[ni], P[mi][ni][r], acc[mi][ni][r]);
        };

        // One phase = from the barrier inside step s - 1 to the barrier inside step s (see gemm_q4_k_tile_kernel).
        auto phase = [&](int blk, auto CC) __attribute__((always_inline)) {
            constexpr int c = decltype(CC)::value;
            const int s = blk * 4 + c;
            step_bases(abuf);
            read_frags(0, 0);
            __builtin_amdgcn_sched_barrier(0);
            const int ab2 = abuf == 0 ? 2 : abuf - 1;  // (step + 2) % 3
            if (s > 0) mfma_slice(1, false, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 0); });
            else issue_A1(s + 2, ab2, 0);
            issue_B1(s + 2, ab2, 0);
            // tables of super-block blk + 1: the current ones were last read in phase 1 (d in phase 0)
            if constexpr (c == 2) issue_tables(blk + 1);
            __builtin_amdgcn_sched_barrier(0);
            half8 sfr[2], mh, ml;
            const bool min_now = c == 1 && with_min;
            if (min_now) {
#pragma unroll
                for (int mi = 0; mi < 2; mi++) sfr[mi] = *(const half8*)(smem + kOffS + (wm * 64 + mi * 32 + nl) * 32 + g * 16);
                mh = *(const half8*)(smem + kOffM + (wn * 64 + nl) * 32);
                ml = *(const half8*)(smem + kOffM + (wn * 64 + nl) * 32 + 16);
            }
            read_frags(1, 1);
            __builtin_amdgcn_sched_barrier(0);
            if (c == 0 && s > 0) {
                // the finished super-block's rescale, sub-tile by sub-tile, in front of the instruction that restarts its P
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    rescale_tile(t);
                    __builtin_amdgcn_sched_barrier(0);
                    P[t >> 1][t & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t >> 1], bfr[0][t & 1], zero16, 0, 0, 0);
                    if (t == 3) issue_A1(s + 2, ab2, 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                mfma_slice(0, c == 0, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 1); });
            }
            if (c == 0) {
#pragma unroll
                for (int ni = 0; ni < 2; ni++) dcur[ni] = *(const float*)(smem + kOffD + (wn * 64 + ni * 32 + nl) * 4);
            }
            if (min_now) {
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
#pragma unroll
                    for (int mi = 0; mi < 2; mi++) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sfr[mi], mh, acc[mi][ni], 0, 0, 0);
#pragma unroll
                    for (int mi = 0; mi < 2; mi++) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sfr[mi], ml, acc[mi][ni], 0, 0, 0);
                    if (ni == 0) {
                        __builtin_amdgcn_sched_barrier(0);
                        mh = *(const half8*)(smem + kOffM + (wn * 64 + 32 + nl) * 32);
                        ml = *(const half8*)(smem + kOffM + (wn * 64 + 32 + nl) * 32 + 16);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            read_frags(2, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(1, false, [&](int i) __attribute__((always_inline)) {
                if (i == 1) issue_B1(s + 2, ab2, 1);
                if (i == 3) issue_A1(s + 2, ab2, 2);
            });
            read_frags(3, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(0, false, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 3); });
            // everything issued before this phase has landed: lhs and weights of step s + 1 (and, after phase 3, the tables)
            if constexpr (c == 2) wait_vmcnt<9>();
            else wait_vmcnt<6>();
            __syncthreads();
            abuf = abuf == 2 ? 0 : abuf + 1;
        };
        for (int blk = 0; blk < nblk; blk++) {
            phase(blk, std::integral_constant<int, 0>{});
            phase(blk, std::integral_constant<int, 1>{});
            phase(blk, std::integral_constant<int, 2>{});
            phase(blk, std::integral_constant<int, 3>{});
        }
        mfma_slice(1, false, [](int) __attribute__((always_inline)) {});  // last slice of the last step
#pragma unroll
        for (int t = 0; t < 4; t++) rescale_tile(t);

        // ---- tile epilogue: undo the row scale, store
        {
            const int col0 = n0 + wn * 64 + nl, col1 = col0 + 32;
            const bool c0_ok = col0 < n, c1_ok = col1 < n;
#pragma unroll
            for (int mi = 0; mi < 2; mi++) {
                float4 iv[4];
#pragma unroll
                for (int j = 0; j < 4; j++) iv[j] = *(const float4*)(smem + kOffInv + (wm * 64 + mi * 32 + 8 * j + 4 * g) * 4);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                    const float4 q = iv[r >> 2];
                    const float is = (r & 3) == 0 ? q.x : (r & 3) == 1 ? q.y : (r & 3) == 2 ? q.z : q.w;
                    if (row < m) {
                        float* o_ = dst + (int64_t)row * n;
                        const float v0 = acc[mi][0][r] * is, v1 = acc[mi][1][r] * is;
                        if (unit_half) {  // one of the two K parts of this tile that meet here: zero or the other part is there
                            if (c0_ok) unsafeAtomicAdd(o_ + col0, v0);
                            if (c1_ok) unsafeAtomicAdd(o_ + col1, v1);
                        } else if (accumulate) {
                            if (c0_ok) o_[col0] += v0;
                            if (c1_ok) o_[col1] += v1;
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

// The GEMM over TWO planes of one encoding (Q6_K: (16 hi) * q and lo * q, same super-block scale d): both planes of a step are
// multiplied with the same lhs operands, so the lhs tile travels to LDS and into registers once for both, and a step holds 32
// matrix-core instructions per wavefront instead of 16.  That lengthens the lead of every operand read (eight instructions instead of
// four) and lets two buffers per operand do (a step ahead is as long as two steps of the one-plane kernel): lhs 2 x 32 KB, weights
// 2 x (2 planes x 16 KB).  No min term (Q6_K has none).
namespace {
constexpr int k2OffA = 0, k2OffB = 2 * kABuf, k2OffD = k2OffB + 4 * kBBuf, k2OffInv = k2OffD + kDBuf, kPlanes2Lds = k2OffInv + TM * 4;
static_assert(kPlanes2Lds <= kLdsPerCu, "two-plane kernel LDS");
}  // namespace

__global__ __launch_bounds__(512, 1) void gemm_planes2_kernel(const uint8_t* __restrict__ planes, const float* __restrict__ dtab,
                                                             const _Float16* __restrict__ a16, const float* __restrict__ inv,
                                                             float* __restrict__ out, int m, int n, int k, int tiles_m, int tiles_n,
                                                             int accumulate, int allow_split, float* __restrict__ part) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int nl = lane & 31, g = lane >> 5;
    const int nblk_row = k >> 8;
    // operand reads: row (column) nl of the wavefront's 32-row groups, piece 2 f + g, swizzled; slice f: the address xor f << 5
    const uint32_t fa0 = (uint32_t)(k2OffA + (wm * 64 + nl) * 128 + ((g ^ ((nl >> 1) & 7)) << 4));
    const uint32_t fb0 = (uint32_t)(k2OffB + (wn * 64 + nl) * 128 + ((g ^ ((nl >> 1) & 7)) << 4));
    const uint32_t lane16 = (uint32_t)(lane * 16);
    uint32_t fax[4], fbx[4];
#pragma unroll
    for (int f = 0; f < 4; f++) {
        fax[f] = fa0 ^ (uint32_t)(f << 5);
        fbx[f] = fb0 ^ (uint32_t)(f << 5);
    }

    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8, wgs_per_xcd = (int)(gridDim.x >> 3);
    const int xcd_base = (int)(blockIdx.x & 7) * per_xcd, n_x = max(0, min(per_xcd, total - xcd_base));
    // (part != null: every tile in four K quarters that meet pairwise in `out` and `part`, as in gemm_planes_kernel)
    int full;
    const int units = part ? 4 * n_x : xcd_units(n_x, wgs_per_xcd, nblk_row, allow_split, full);
    for (int u = (int)(blockIdx.x >> 3); u < units; u += wgs_per_xcd) {
        TileUnit unit;
        if (part) {
            const int q = u & 3, b0 = q * nblk_row / 4, b1 = (q + 1) * nblk_row / 4;
            unit.tile = xcd_base + (u >> 2); unit.kb0 = b0; unit.nb = b1 - b0; unit.half = 1;
        } else {
            unit = xcd_unit(u, xcd_base, full, nblk_row);
        }
        float* __restrict__ dst = part && (u & 2) ? part : out;
        const int nblk = __builtin_amdgcn_readfirstlane(unit.nb), ns = nblk * 4;  // this unit's share of K
        const int kb0 = __builtin_amdgcn_readfirstlane(unit.kb0), unit_half = __builtin_amdgcn_readfirstlane(unit.half);
        int tile_m, tile_n;
        tile_order(unit.tile, tiles_m, tiles_n, kTileGm, tile_m, tile_n);
        tile_m = __builtin_amdgcn_readfirstlane(tile_m);
        tile_n = __builtin_amdgcn_readfirstlane(tile_n);
        const int m0 = tile_m * TM, n0 = tile_n * TN;

        const uint8_t* a_base = (const uint8_t*)a16 + ((int64_t)(m0 + wave * 32) * k + (int64_t)kb0 * 256) * 2;
        const int64_t plane_bytes = (int64_t)nblk_row * 4 * kBBuf;  // one plane of one column tile
        const uint8_t* b_base = planes + (int64_t)tile_n * 2 * plane_bytes + (int64_t)kb0 * 4 * kBBuf;
        const uint8_t* d_base = (const uint8_t*)dtab + ((int64_t)tile_n * nblk_row + kb0) * kDBuf;

        // the i-th of the four loads that bring this wavefront's 32 rows of the lhs of step `step` into buffer `buf`
        // lhs rows wave * 32 + 8 i + lane / 8; LDS position lane % 8 of a row holds piece (lane % 8) ^ ((row / 2) % 8)
        uint32_t a_offs[2];
#pragma unroll
        for (int i = 0; i < 2; i++) a_offs[i] = (uint32_t)((lane >> 3) * (k * 2) + (((lane & 7) ^ ((4 * i + (lane >> 4)) & 7)) << 4));
        auto issue_A1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const uint32_t a_off = a_offs[i & 1];
            const uint32_t dst = lds0 + k2OffA + buf * kABuf + wave * 4096;
            load16_to_lds(a_off, a_base + (int64_t)min(step, ns - 1) * 128 + (int64_t)i * 16 * k,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(dst + i * 1024)));
        };
        // the i-th (0..3) of this wavefront's four 1 KB pieces of the two weight tiles of step `step`: plane i / 2, piece 2 wave + i % 2
        auto issue_B1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const int pl = i >> 1, piece = (wave * 2 + (i & 1)) * 1024;
            load16_to_lds(lane16, b_base + pl * plane_bytes + (int64_t)min(step, ns - 1) * kBBuf + piece,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + k2OffB + (buf * 2 + pl) * kBBuf + piece)));
        };
        auto issue_D = [&](int blk) __attribute__((always_inline)) {
            if (lane < 4)
                load16_to_lds(lane16, d_base + (int64_t)min(blk, nblk - 1) * kDBuf + wave * 64,
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + k2OffD + wave * 64)));
        };

        // The accumulators are kept in units of the current super-block's scale (see gemm_planes_wide_kernel below): no second
        // set for the running super-block.
        float16v acc[2][2];
#pragma unroll
        for (int mi = 0; mi < 2; mi++)
#pragma unroll
            for (int ni = 0; ni < 2; ni++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[mi][ni][r] = 0.0f;
        half8 afr[2][2], bfr[2][2][2];  // [slot][row group], [slot][plane][column group]
        float unit_d[2] = {1.f, 1.f}, ratio[2] = {1.f, 1.f};

        // ---- tile prologue
        __syncthreads();  // every wavefront is done with the previous tile's LDS contents
        issue_D(0);
#pragma unroll
        for (int i = 0; i < 4; i++) issue_A1(0, 0, i);
#pragma unroll
        for (int i = 0; i < 4; i++) issue_B1(0, 0, i);
        if (tid < TM) *(float*)(smem + k2OffInv + tid * 4) = inv[min(m0 + tid, m - 1)];
        wait_vmcnt<0>();
        __syncthreads();

        // operand addresses of the four slices (the slice index is xor-ed into the swizzled piece index), buffer 0: eight registers;
        // buffer, row group, plane and column group are immediate offsets of the reads
        auto read_frags = [&](int buf, int f, int slot) __attribute__((always_inline)) {
#pragma unroll
            for (int mi = 0; mi < 2; mi++) afr[slot][mi] = *(const half8*)(smem + fax[f] + (buf * kABuf + mi * 4096));
#pragma unroll
            for (int pl = 0; pl < 2; pl++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++) bfr[slot][pl][ni] = *(const half8*)(smem + fbx[f] + (buf * 2 * kBBuf + pl * kBBuf + ni * 4096));
        };
        // the eight matrix-core instructions of one slice (both planes); `between(i)` is placed after the i-th of them
        auto mfma_slice = [&](int slot, auto&& between) __attribute__((always_inline)) {
#pragma unroll
            for (int pl = 0; pl < 2; pl++)
#pragma unroll
                for (int mi = 0; mi < 2; mi++)
#pragma unroll
                    for (int ni = 0; ni < 2; ni++) {
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[slot][mi], bfr[slot][pl][ni], acc[mi][ni], 0, 0, 0);
                        between(pl * 4 + mi * 2 + ni);
                        __builtin_amdgcn_sched_barrier(0);
                    }
        };

        // One phase = from the barrier inside step s - 1 to the barrier inside step s; the buffers of step s are those of index s % 2 = c % 2.
        // All loads of step s + 1 are issued in the first half of the phase, into the buffers that step s - 1 used.
        // FIRST: the first step of the unit, a variant of its own (see gemm_planes_wide_kernel)
        auto phase = [&](int blk, auto CC, auto FF) __attribute__((always_inline)) {
            constexpr int c = decltype(CC)::value, cur = c & 1, nxt = cur ^ 1;
            constexpr bool FIRST = decltype(FF)::value;
            const int s = blk * 4 + c;
            read_frags(cur, 0, 0);
            if (c == 0) {
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    const float dn = *(const float*)(smem + k2OffD + (wn * 64 + ni * 32 + nl) * 4), un = dn != 0.0f ? dn : unit_d[ni];
                    ratio[ni] = unit_d[ni] * __builtin_amdgcn_rcpf(un);  // (one ulp off at most: 2e-7 relative per super-block)
                    unit_d[ni] = un;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!FIRST) {
                mfma_slice(1, [&](int i) __attribute__((always_inline)) {  // last slice of step s - 1
                    if (i & 1) issue_A1(s + 1, nxt, i >> 1);
                });
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++) issue_A1(s + 1, nxt, i);
            }
            if constexpr (c == 2) issue_D(blk + 1);  // (the current scales were read in phase 0)
            __builtin_amdgcn_sched_barrier(0);
            read_frags(cur, 1, 1);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (c == 0 && !FIRST) {
                // the accumulators change unit, sub-tile by sub-tile, in front of the new super-block's first instruction on each
#pragma unroll
                for (int t = 0; t < 4; t++) {
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[t >> 1][t & 1][r] *= ratio[t & 1];
                    __builtin_amdgcn_sched_barrier(0);
                    acc[t >> 1][t & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t >> 1], bfr[0][0][t & 1], acc[t >> 1][t & 1], 0, 0, 0);
                    issue_B1(s + 1, nxt, t);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    acc[t >> 1][t & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t >> 1], bfr[0][1][t & 1], acc[t >> 1][t & 1], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                mfma_slice(0, [&](int i) __attribute__((always_inline)) { if (i < 4) issue_B1(s + 1, nxt, i); });
            }
            read_frags(cur, 2, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(1, [](int) __attribute__((always_inline)) {});
            read_frags(cur, 3, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(0, [](int) __attribute__((always_inline)) {});
            wait_vmcnt<0>();  // lhs and weights of step s + 1 (and, in phase 2, the next scales) have landed
            __syncthreads();
        };
        phase(0, std::integral_constant<int, 0>{}, std::true_type{});
        phase(0, std::integral_constant<int, 1>{}, std::false_type{});
        phase(0, std::integral_constant<int, 2>{}, std::false_type{});
        phase(0, std::integral_constant<int, 3>{}, std::false_type{});
        for (int blk = 1; blk < nblk; blk++) {
            phase(blk, std::integral_constant<int, 0>{}, std::false_type{});
            phase(blk, std::integral_constant<int, 1>{}, std::false_type{});
            phase(blk, std::integral_constant<int, 2>{}, std::false_type{});
            phase(blk, std::integral_constant<int, 3>{}, std::false_type{});
        }
        mfma_slice(1, [](int) __attribute__((always_inline)) {});  // last slice of the last step

        // ---- tile epilogue: undo the row scale, store
        {
            const int col0 = n0 + wn * 64 + nl, col1 = col0 + 32;
            const bool c0_ok = col0 < n, c1_ok = col1 < n;
#pragma unroll
            for (int mi = 0; mi < 2; mi++) {
                float4 iv[4];
#pragma unroll
                for (int j = 0; j < 4; j++) iv[j] = *(const float4*)(smem + k2OffInv + (wm * 64 + mi * 32 + 8 * j + 4 * g) * 4);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                    const float4 q = iv[r >> 2];
                    const float is = (r & 3) == 0 ? q.x : (r & 3) == 1 ? q.y : (r & 3) == 2 ? q.z : q.w;
                    if (row < m) {
                        float* o_ = dst + (int64_t)row * n;
                        const float v0 = acc[mi][0][r] * unit_d[0] * is, v1 = acc[mi][1][r] * unit_d[1] * is;
                        if (unit_half) {  // one of the two K halves of this tile: out holds zero or the other half
                            if (c0_ok) unsafeAtomicAdd(o_ + col0, v0);
                            if (c1_ok) unsafeAtomicAdd(o_ + col1, v1);
                        } else if (accumulate) {
                            if (c0_ok) o_[col0] += v0;
                            if (c1_ok) o_[col1] += v1;
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

// The GEMM over one plane on 256 x 256 output tiles: the two-plane kernel's structure (32 KB of lhs and 2 x 16 KB of weights per
// step, two buffers each, 32 matrix-core instructions per wavefront and step, six operand reads for eight of them), with the second
// 16 KB being the neighbouring 128-column tile instead of a second plane, and one set of 128 accumulators per lane and no second
// set for the running super-block: the accumulators are kept in units of the current super-block's scale,
//     acc <- acc * (d_prev / d_cur)   at each super-block boundary,   acc <- acc * d_last   at the end,
// so that the matrix cores add each super-block's exact integer products directly onto them.  A zero scale keeps the unit of the
// block before it (its plane holds zeros, see the conversion).
namespace {
constexpr int kwOffA = 0, kwOffB = 2 * kABuf, kwOffD = kwOffB + 4 * kBBuf, kwOffInv = kwOffD + 2 * kDBuf, kPlanesWLds = kwOffInv + TM * 4;
static_assert(kPlanesWLds <= kLdsPerCu, "wide kernel LDS");
}  // namespace

// SPB: steps (of 64 k) per scale block: 4 for the K-quants, 2 for GPTQ groups of 128.  NG: 32-column groups per wavefront: 4 for
// the 256 x 256 tile, 3 for a 256 x 192 tile (a launch of those finishes a problem whose last round of 256 x 256 tiles would
// leave a quarter or more of the compute units idle).  The launch covers the columns from n_begin (a multiple of 64) on.
template <int SPB, int NG>
__global__ __launch_bounds__(512, 1) void gemm_planes_wide_kernel(const uint8_t* __restrict__ planes, const float* __restrict__ dtab,
                                                                 const _Float16* __restrict__ a16, const float* __restrict__ inv,
                                                                 float* __restrict__ out, int m, int n, int lda, int nblk_walk,
                                                                 int nblk_tile, int tiles_m, int tiles_n, int tiles_n128, int n_begin,
                                                                 int accumulate, int allow_split) {
    constexpr int TW = NG * 64;  // columns of a tile
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int nl = lane & 31, g = lane >> 5;
    const int nblk_row = nblk_walk;  // blocks of a full unit; nblk_tile: blocks per 128-column tile in the planes and tables
    // operand reads: row (column) nl of the wavefront's 32-row groups, piece 2 f + g, swizzled; slice f: the address xor f << 5.
    // The weight tile sits in LDS as TW rows of 128 bytes; the wavefront's columns are wn * 32 NG + 32 j + nl.
    const uint32_t fa0 = (uint32_t)(kwOffA + (wm * 64 + nl) * 128 + ((g ^ ((nl >> 1) & 7)) << 4));
    const uint32_t fb0 = (uint32_t)(kwOffB + (wn * NG * 32 + nl) * 128 + ((g ^ ((nl >> 1) & 7)) << 4));
    const uint32_t lane16 = (uint32_t)(lane * 16);
    uint32_t fax[4], fbx[4];
#pragma unroll
    for (int f = 0; f < 4; f++) {
        fax[f] = fa0 ^ (uint32_t)(f << 5);
        fbx[f] = fb0 ^ (uint32_t)(f << 5);
    }
    const int64_t plane_bytes = (int64_t)nblk_tile * SPB * kBBuf;  // the plane of one 128-column tile
    const int64_t dtile = (int64_t)nblk_tile * kDBuf;             // its scales

    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8, wgs_per_xcd = (int)(gridDim.x >> 3);
    const int xcd_base = (int)(blockIdx.x & 7) * per_xcd, n_x = max(0, min(per_xcd, total - xcd_base));
    int full;
    const int units = xcd_units(n_x, wgs_per_xcd, nblk_row, allow_split, full);
    for (int u = (int)(blockIdx.x >> 3); u < units; u += wgs_per_xcd) {
        const TileUnit unit = xcd_unit(u, xcd_base, full, nblk_row);
        const int nblk = __builtin_amdgcn_readfirstlane(unit.nb), ns = nblk * SPB;  // this unit's share of K
        const int kb0 = __builtin_amdgcn_readfirstlane(unit.kb0), unit_half = __builtin_amdgcn_readfirstlane(unit.half);
        int tile_m, tile_n;
        tile_order(unit.tile, tiles_m, tiles_n, kTileGm, tile_m, tile_n);
        tile_m = __builtin_amdgcn_readfirstlane(tile_m);
        tile_n = __builtin_amdgcn_readfirstlane(tile_n);
        const int m0 = tile_m * TM, n0 = n_begin + tile_n * TW;

        const uint8_t* a_base = (const uint8_t*)a16 + ((int64_t)(m0 + wave * 32) * lda + (int64_t)kb0 * (SPB * 64)) * 2;
        uint32_t a_offs[2];
#pragma unroll
        for (int i = 0; i < 2; i++) a_offs[i] = (uint32_t)((lane >> 3) * (lda * 2) + (((lane & 7) ^ ((4 * i + (lane >> 4)) & 7)) << 4));
        auto issue_A1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const uint32_t a_off = a_offs[i & 1];
            const uint32_t dst = lds0 + kwOffA + buf * kABuf + wave * 4096;
            load16_to_lds(a_off, a_base + (int64_t)min(step, ns - 1) * 128 + (int64_t)i * 16 * lda,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(dst + i * 1024)));
        };
        // This wavefront's NG pieces of 1 KB (eight columns) of the weight tile: piece NG wave + i.  A piece lies inside one
        // 128-column tile of the planes (at a ragged edge the last one again: those columns lie beyond n and are not stored).
        const uint8_t* b_src[NG];
#pragma unroll
        for (int i = 0; i < NG; i++) {
            const int c = n0 + (wave * NG + i) * 8;
            b_src[i] = planes + (int64_t)min(c >> 7, tiles_n128 - 1) * plane_bytes + (int64_t)kb0 * SPB * kBBuf + (c & 127) * 128;
        }
        auto issue_B1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            load16_to_lds(lane16, b_src[i] + (int64_t)min(step, ns - 1) * kBBuf,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kwOffB + buf * 2 * kBBuf + (wave * NG + i) * 1024)));
        };
        // the TW scales of block blk, in column order: lanes 0..7 of the first 2 NG wavefronts bring 32 each
        const uint32_t d_voff = [&] {
            const int c = n0 + wave * 32 + (lane & 7) * 4;
            return (uint32_t)min(c >> 7, tiles_n128 - 1) * (uint32_t)dtile + (uint32_t)((c & 127) * 4);
        }();
        const uint8_t* d_base = (const uint8_t*)dtab + (int64_t)kb0 * kDBuf;
        auto issue_D = [&](int blk) __attribute__((always_inline)) {
            if (wave < 2 * NG && lane < 8)
                load16_to_lds(d_voff, d_base + (int64_t)min(blk, nblk - 1) * kDBuf,
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kwOffD + wave * 128)));
        };
        auto d_at = [&](int j) __attribute__((always_inline)) { return *(const float*)(smem + kwOffD + (wn * NG * 32 + j * 32 + nl) * 4); };

        float16v acc[NG][2];  // [column group][row group]
#pragma unroll
        for (int t = 0; t < 2 * NG; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t >> 1][t & 1][r] = 0.0f;
        half8 afr[2][2], bfr[2][NG];  // [slot][row group], [slot][column group]
        float unit_d[NG], ratio[NG];
#pragma unroll
        for (int j = 0; j < NG; j++) unit_d[j] = ratio[j] = 1.0f;

        // ---- tile prologue
        __syncthreads();  // every wavefront is done with the previous tile's LDS contents
        issue_D(0);
#pragma unroll
        for (int i = 0; i < 4; i++) issue_A1(0, 0, i);
#pragma unroll
        for (int i = 0; i < NG; i++) issue_B1(0, 0, i);
        if (tid < TM) *(float*)(smem + kwOffInv + tid * 4) = inv[min(m0 + tid, m - 1)];
        wait_vmcnt<0>();
        __syncthreads();

        // operand addresses of the four slices (the slice index is xor-ed into the swizzled piece index), buffer 0: eight registers;
        // buffer, row group and column group are immediate offsets of the reads
        auto read_frags = [&](int buf, int f, int slot) __attribute__((always_inline)) {
#pragma unroll
            for (int mi = 0; mi < 2; mi++) afr[slot][mi] = *(const half8*)(smem + fax[f] + (buf * kABuf + mi * 4096));
#pragma unroll
            for (int j = 0; j < NG; j++) bfr[slot][j] = *(const half8*)(smem + fbx[f] + (buf * 2 * kBBuf + j * 4096));
        };
        // the 2 NG matrix-core instructions of one slice; `between(i)` is placed after the i-th of them
        auto mfma_slice = [&](int slot, auto&& between) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < NG; j++)
#pragma unroll
                for (int mi = 0; mi < 2; mi++) {
                    acc[j][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[slot][mi], bfr[slot][j], acc[j][mi], 0, 0, 0);
                    between(j * 2 + mi);
                    __builtin_amdgcn_sched_barrier(0);
                }
        };

        // One phase = from the barrier inside step s - 1 to the barrier inside step s; the buffers of step s are those of index s % 2.
        // All loads of step s + 1 are issued in the first half of the phase, into the buffers that step s - 1 used.
        // FIRST: the first step of the unit (nothing to finish, nothing to rescale), a variant of its own so that the loop body
        // has no branches around matrix-core instructions (the compiler copies accumulators where they meet).
        auto phase = [&](int blk, auto CC, auto FF) __attribute__((always_inline)) {
            constexpr int c = decltype(CC)::value, cur = c & 1, nxt = cur ^ 1;
            constexpr bool FIRST = decltype(FF)::value;
            const int s = blk * SPB + c;
            read_frags(cur, 0, 0);
            if (c == 0) {
                // the new block's unit: its scale, or the previous unit where the scale is zero
#pragma unroll
                for (int j = 0; j < NG; j++) {
                    const float dn = d_at(j), un = dn != 0.0f ? dn : unit_d[j];
                    ratio[j] = unit_d[j] * __builtin_amdgcn_rcpf(un);  // (one ulp off at most: 2e-7 relative per block)
                    unit_d[j] = un;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!FIRST) {
                mfma_slice(1, [&](int i) __attribute__((always_inline)) {  // last slice of step s - 1
                    if constexpr (NG == 4) {
                        if (i & 1) issue_A1(s + 1, nxt, i >> 1);
                    } else {
                        if (i == 0) issue_A1(s + 1, nxt, 0);
                        if (i == 2) issue_A1(s + 1, nxt, 1);
                        if (i == 3) issue_A1(s + 1, nxt, 2);
                        if (i == 5) issue_A1(s + 1, nxt, 3);
                    }
                });
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++) issue_A1(s + 1, nxt, i);
            }
            if constexpr (c == 1) issue_D(blk + 1);  // (the current scales were read in phase 0)
            __builtin_amdgcn_sched_barrier(0);
            read_frags(cur, 1, 1);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (c == 0 && !FIRST) {
                // the accumulators change unit, sub-tile by sub-tile, in front of the new block's first instruction on each
#pragma unroll
                for (int t = 0; t < 2 * NG; t++) {
                    const int j = t >> 1, mi = t & 1;
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[j][mi][r] *= ratio[j];
                    __builtin_amdgcn_sched_barrier(0);
                    acc[j][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][mi], bfr[0][j], acc[j][mi], 0, 0, 0);
                    if (t < NG) issue_B1(s + 1, nxt, t);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                mfma_slice(0, [&](int i) __attribute__((always_inline)) { if (i < NG) issue_B1(s + 1, nxt, i); });
            }
            read_frags(cur, 2, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(1, [](int) __attribute__((always_inline)) {});
            read_frags(cur, 3, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(0, [](int) __attribute__((always_inline)) {});
            wait_vmcnt<0>();  // lhs and weights of step s + 1 (and, in phase 1, the next scales) have landed
            __syncthreads();
        };
        // (the first block apart from the loop: see FIRST)
        phase(0, std::integral_constant<int, 0>{}, std::true_type{});
        phase(0, std::integral_constant<int, 1>{}, std::false_type{});
        if constexpr (SPB == 4) {
            phase(0, std::integral_constant<int, 2>{}, std::false_type{});
            phase(0, std::integral_constant<int, 3>{}, std::false_type{});
        }
        for (int blk = 1; blk < nblk; blk++) {
            phase(blk, std::integral_constant<int, 0>{}, std::false_type{});
            phase(blk, std::integral_constant<int, 1>{}, std::false_type{});
            if constexpr (SPB == 4) {
                phase(blk, std::integral_constant<int, 2>{}, std::false_type{});
                phase(blk, std::integral_constant<int, 3>{}, std::false_type{});
            }
        }
        mfma_slice(1, [](int) __attribute__((always_inline)) {});  // last slice of the last step

        // ---- tile epilogue: back to true units (last block's scale, row scale), store
#pragma unroll
        for (int mi = 0; mi < 2; mi++) {
            float4 iv[4];
#pragma unroll
            for (int q = 0; q < 4; q++) iv[q] = *(const float4*)(smem + kwOffInv + (wm * 64 + mi * 32 + 8 * q + 4 * g) * 4);
#pragma unroll
            for (int j = 0; j < NG; j++) {
                const int col = n0 + wn * NG * 32 + j * 32 + nl;
                const bool col_ok = col < n;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                    const float4 q = iv[r >> 2];
                    const float is = (r & 3) == 0 ? q.x : (r & 3) == 1 ? q.y : (r & 3) == 2 ? q.z : q.w;
                    if (row < m && col_ok) {
                        float* o_ = out + (int64_t)row * n + col;
                        const float v = acc[j][mi][r] * unit_d[j] * is;
                        if (unit_half) unsafeAtomicAdd(o_, v);  // one of the two K parts of this tile: out holds zero or the other part
                        else if (accumulate) *o_ += v;
                        else __builtin_nontemporal_store(v, o_);
                    }
                }
            }
        }
    }
}

// How a problem is cut into launches of the wide kernel.  All 256 x 256 tiles, unless the last round of those would leave
// a quarter or more of the compute units idle while 256 x 192 tiles over the remaining columns fit one round: then the
// first launch takes whole rounds of 256 x 256 tiles (`wide_strips` column strips), the second the rest as 256 x 192 tiles.
struct WidePlan {
    int wide_strips;    // 256-column strips of the first launch
    int narrow_strips;  // 192-column strips of the second launch (0: one launch)
};
WidePlan wide_plan(int64_t m, int64_t n, int cus) {
    const int tiles_m = (int)((m + TM - 1) / TM), strips = (int)((n + 2 * TN - 1) / (2 * TN));
    const int total = tiles_m * strips, rounds = total / cus, rem = total - rounds * cus;
    WidePlan p{strips, 0};
    if (rounds == 0 || rem == 0 || 4 * rem > 3 * cus || (rounds * cus) % tiles_m != 0 || kernel_disabled("planes_192")) return p;
    const int first = rounds * cus / tiles_m;
    const int64_t rest = n - (int64_t)first * 2 * TN;
    const int narrow = (int)((rest + 191) / 192);
    if (rest <= 0 || tiles_m * narrow > cus) return p;
    p.wide_strips = first;
    p.narrow_strips = narrow;
    return p;
}

int compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    return cus;
}

// The launches of the wide kernel for one lhs plane.  `z` is what the preparation launch zeroes (split tiles of a single launch;
// a problem cut into two launches splits none).
struct WideLaunch {
    WidePlan plan;
    int tiles_m, tiles_n128, wg;
    SplitTiles z;
};
WideLaunch wide_launch(float* out, int64_t m, int64_t n, int blocks_walked) {
    WideLaunch L;
    const int cus = compute_units();
    L.plan = wide_plan(m, n, cus);
    L.tiles_m = (int)((m + TM - 1) / TM);
    L.tiles_n128 = (int)((n + TN - 1) / TN);
    const int total = L.tiles_m * L.plan.wide_strips, per_xcd = (total + 7) / 8, per_xcd_cus = std::max(1, cus / 8);
    L.wg = 8 * std::min(per_xcd, per_xcd_cus);
    L.z = split_tiles(out, m, n, L.tiles_m, L.plan.wide_strips, blocks_walked, L.wg, 2 * TN);
    if (L.plan.narrow_strips) L.z.max_split = 0;
    return L;
}
template <int SPB>
hipError_t run_wide(const WideLaunch& L, const uint8_t* planes, const float* dtab, const _Float16* a, const float* inv, float* out, int64_t m,
                    int64_t n, int64_t lda, int nblk_walk, int nblk_tile, int pass, hipStream_t s) {
    hipError_t e = allow_full_lds<gemm_planes_wide_kernel<SPB, 4>>();
    if (e == hipSuccess && L.plan.narrow_strips) e = allow_full_lds<gemm_planes_wide_kernel<SPB, 3>>();
    if (e != hipSuccess) return e;
    const int split = pass == 0 && L.z.max_split > 0 ? 1 : 0;
    gemm_planes_wide_kernel<SPB, 4><<<dim3((unsigned)L.wg), dim3(512), kPlanesWLds, s>>>(planes, dtab, a, inv, out, (int)m, (int)n, (int)lda, nblk_walk,
                                                                                        nblk_tile, L.tiles_m, L.plan.wide_strips, L.tiles_n128, 0,
                                                                                        pass, split);
    if (L.plan.narrow_strips) {
        const int total = L.tiles_m * L.plan.narrow_strips;
        const int wg = 8 * std::min((total + 7) / 8, std::max(1, compute_units() / 8));
        gemm_planes_wide_kernel<SPB, 3><<<dim3((unsigned)wg), dim3(512), kPlanesWLds, s>>>(planes, dtab, a, inv, out, (int)m, (int)n, (int)lda, nblk_walk,
                                                                                          nblk_tile, L.tiles_m, L.plan.narrow_strips, L.tiles_n128,
                                                                                          L.plan.wide_strips * 2 * TN, pass, 0);
    }
    return hipGetLastError();
}

// GPTQ (4-bit, [K/8, N] int32 words of eight consecutive k, zero point = stored + 1) to one plane of q - zero in [-16, 14],
// the scale blocks being the groups: one workgroup per (128-column tile, 256 k).  The 32 x 128 words come in coalesced,
// through LDS, and leave as 16-byte pieces, eight neighbouring threads writing one 128-byte row of the tile; a word is exactly
// one piece (k = 64 step + 32 g + 8 f + 0..7).  Nibble n under the byte 0x64 reads as fp16 1024 + n; the packed subtraction of
// 1024 + zero leaves the exact difference.
__device__ __forceinline__ void planes_from_gptq(int tile_n, int rb, const uint32_t* __restrict__ qweight, const uint16_t* __restrict__ scales,
                                                 const uint32_t* __restrict__ qzeros, int n, int k, int group, uint8_t* __restrict__ planes,
                                                 float* __restrict__ dtab) {
    __shared__ uint32_t stage[32 * 129];
    const int tid = (int)threadIdx.x, n0 = tile_n * TN;
    for (int i = tid; i < 32 * 128; i += 256) {
        const int row = i >> 7, col = i & 127;
        stage[row * 129 + col] = n0 + col < n ? qweight[(int64_t)(rb * 32 + row) * n + n0 + col] : 0u;
    }
    __syncthreads();
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    auto pair = [](uint32_t x) __attribute__((always_inline)) { return __builtin_bit_cast(half2v, x); };
    auto bits = [](half2v x) __attribute__((always_inline)) { return __builtin_bit_cast(uint32_t, x); };
    const int piece = tid & 7, g = piece & 1, f = piece >> 1;
    const int64_t steps_tile = k / 64, groups = k / group;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int col = j * 32 + (tid >> 3), ncol = min(n0 + col, n - 1);
        const bool in_n = n0 + col < n;
        const uint32_t dst = (uint32_t)(col * 128 + ((piece ^ ((col >> 1) & 7)) << 4));
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int64_t gi = ((int64_t)rb * 256 + c * 64) / group;
            const uint32_t zero = ((qzeros[gi * (n >> 3) + (ncol >> 3)] >> (4 * (ncol & 7))) & 0xFu) + 1u;
            const uint16_t sbits = scales[gi * n + ncol];
            const bool live = in_n && (sbits & 0x7fffu) != 0;
            const uint32_t x = stage[(8 * c + 4 * g + f) * 129 + col];
            const uint32_t y = x & 0x0F0F0F0Fu, z = (x >> 4) & 0x0F0F0F0Fu;  // nibbles 0, 2, 4, 6 and 1, 3, 5, 7
            const _Float16 o = (_Float16)(float)(1024u + zero);
            const half2v off = {o, o};
            uint4 v;
            v.x = bits(pair(__builtin_amdgcn_perm(0x64646464u, y, 0x04010400u)) - off);  // k 0, 2
            v.y = bits(pair(__builtin_amdgcn_perm(0x64646464u, z, 0x04010400u)) - off);  // k 1, 3
            v.z = bits(pair(__builtin_amdgcn_perm(0x64646464u, y, 0x04030402u)) - off);  // k 4, 6
            v.w = bits(pair(__builtin_amdgcn_perm(0x64646464u, z, 0x04030402u)) - off);  // k 5, 7
            if (!live) v = make_uint4(0u, 0u, 0u, 0u);
            *(uint4*)(planes + ((int64_t)tile_n * steps_tile + rb * 4 + c) * kBBuf + dst) = v;
            if (piece == 0 && ((rb * 256 + c * 64) % group) == 0) dtab[((int64_t)tile_n * groups + gi) * TN + col] = in_n ? h2f(sbits) : 0.0f;
        }
    }
}

template <typename AT>
__global__ __launch_bounds__(256) void gptq_planes_prologue_kernel(const uint32_t* __restrict__ qweight, const uint16_t* __restrict__ scales,
                                                                   const uint32_t* __restrict__ qzeros, int group, int tiles_n128,
                                                                   uint8_t* __restrict__ planes, float* __restrict__ dtab, int conv,
                                                                   const AT* __restrict__ a, int k, int lhs_rows, LhsPlanes p, SplitTiles z) {
    const int b = (int)blockIdx.x;
    if (b < conv) {
        const int rb = b / tiles_n128;
        planes_from_gptq(b - rb * tiles_n128, rb, qweight, scales, qzeros, z.n, k, group, planes, dtab);
    } else if (b < conv + lhs_rows) {
        prep_lhs_row<AT, kLhsOrderTile>(b - conv, a, k, p.a16, p.a16_lo, p.asum, p.inv);
    } else {
        const int e = b - conv - lhs_rows;
        zero_split_tile_part(z, e >> 6, (e >> 3) & 7, e & 7);
    }
}

bool gemm_planes_wanted(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    if (kernel_disabled("kquant_planes") || k % 256 || k < 256) return false;
    if (encoding == QMM_Q4_K) {
        // From three row tiles on (and 160 tiles of 256 x 256) the conversion pass costs less than the plane GEMM gains on the
        // tile kernel that unpacks as it goes (14336 x 4096 with 2048 rows: 226 + 34 us against 285 + 11 us; 768 rows: 126
        // against 132 us, GPTQ 113 against 137 us; 512 rows: 119 against 88 us).  QMM_Q4K_PLANES=1 (read
        // once) sends every Q4_K prefill shape here, for tests and comparisons.
        static const bool force = getenv("QMM_Q4K_PLANES") != nullptr && atoi(getenv("QMM_Q4K_PLANES")) == 1;
        return m > 16 && (force || (m >= kOptionalPlanesMinRows && wide_tiles(encoding, m, n) && !kernel_disabled("q4k_planes")));
    }
    if (encoding != QMM_Q5_K && encoding != QMM_Q6_K) return false;
    // Up to these row counts the passes of the small-batch kernels (16 lhs rows a pass) cost less than the conversion pass plus
    // a GEMM whose 256-row tiles are mostly empty (14336 x 4096, Q5_K: 48 rows 52 us, 64 rows 69 us, the planes 65 us; Q6_K:
    // 64 rows 88 us, the planes 118 us; beyond 64 rows neither encoding has a kernel that takes more than four rows a pass).
    // Where the small-batch kernel does not take the K (Q5_K: a multiple of 512 up to 32768; Q6_K: of 2048 up to 32768), the
    // alternative is the decode kernel once per one or two lhs rows, at about the cost of a one-row call each time (us, W in
    // millions of weights: 5 + 0.2 W): 4096 x 11008 with 16 / 32 rows 198 / 401 us (Q5_K), 195 / 398 (Q6_K), the planes 88 /
    // 152; 8192 x 28672, Q6_K, 64 rows 3810 against 500.
    const bool mm_takes_k = encoding == QMM_Q5_K ? (k % 512 == 0 && k <= 32768 && !kernel_disabled("q5k_mm"))
                                                 : (k % 2048 == 0 && k <= 32768 && !kernel_disabled("q6k_mm"));
    if (!mm_takes_k) {
        const double W = (double)n * (double)k * 1e-6, row_us = 5.0 + 0.2 * W;
        const double planes_us = (encoding == QMM_Q5_K ? 12.0 + 1.15 * W : 25.0 + 1.85 * W) +
                                 (k > 4096 ? std::min(encoding == QMM_Q5_K ? 45.0 : 60.0, (encoding == QMM_Q5_K ? 9.0 : 11.0) * (double)k / (double)n) : 0.0);
        return m > 4 && 0.9 * (double)m * row_us > planes_us;
    }
    // The small-batch kernels take 16 bf16 or 8 fp32 rows a pass (up to 64 rows), the planes any number in one (an fp32 lhs as
    // twice the rows) behind a conversion.  Both sides in microseconds, fitted to this part (W: millions of weights; a K beyond
    // 4096 costs the small-batch kernels a launch that adds the rounds of 4096 columns, and the planes the K shares of few
    // tiles).  Measured, one pass / the planes at 65 rows, bf16 and fp32 lhs: Q5_K 4096 x 4096 9.6, 13.5 / 35, 46;
    // 14336 x 4096 16.9, 20.4 / 85, 94; 4096 x 14336 20.2, 24.0 / 116, 118; Q6_K 12.5, 12.9 / 55, 69; 21.6, 20.8 / 134, 142;
    // 24.4, 24.5 / 175, 175.
    const bool f32 = lhs_dtype == QMM_F32, long_k = k > 4096;
    const double W = (double)n * (double)k * 1e-6;
    const int64_t me = f32 ? 2 * m : m;  // rows of the plane GEMM (more than 128: two wavefront rows of a tile at work)
    // (a long K: the planes pay for K shares, the more the fewer column tiles there are: at 65 bf16 rows, Q5_K / Q6_K,
    // 4096 x 8192 65 / 100 us, 2048 x 16384 94 / 146, 4096 x 14336 116 / 175, 8192 x 14336 162 / 250)
    const double k_over_n = (double)k / (double)n;
    double pass_us, planes_us;
    if (encoding == QMM_Q5_K) {
        pass_us = (f32 ? 9.0 : 6.0) + W * (f32 ? 0.20 : 0.18) + (long_k ? 3.5 : 0.0);
        planes_us = 12.0 + 1.15 * W + (f32 ? 4.0 : 0.0) + (me > 128 ? 8.0 : 0.0) + (long_k ? std::min(45.0, 9.0 * k_over_n) : 0.0);
    } else {
        pass_us = (f32 ? 9.5 : 8.5) + W * (f32 ? 0.20 : 0.225) + (long_k ? 3.0 : 0.0);
        planes_us = 25.0 + 1.85 * W + (f32 ? 2.0 : 0.0) + (me > 128 ? 14.0 : 0.0) + (long_k ? std::min(60.0, 11.0 * k_over_n) : 0.0);
    }
    const int64_t passes = (m + (f32 ? 8 : 16) - 1) / (f32 ? 8 : 16);
    return m > 64 || (double)passes * pass_us > planes_us;
}

// Very few tiles, or few on a long K: the 256 x 128 plane kernels (one plane, and Q6_K's two) cut every tile in four K quarters (bf16 lhs: one pass), which
// takes a second m x n buffer behind everything else in the workspace, zeroing of both and a launch that adds them.  Against K halves,
// over kept planes: 4096 x 4096 with 65 rows (16 tiles) 36 -> 27 us, 1024 x 4096 with 512 rows 40 -> 35 us, 4096 x 14336 with 256 / 512
// rows (32 / 64 tiles) 104 -> 74 / 113 -> 103 us; but 4096 x 4096 with 256 rows (32 tiles) 41 -> 41 us, with 512 rows (64 tiles) 49 -> 60 us.
bool few_tiles_for_quarters(int64_t m, int64_t n, int64_t k) {
    const int64_t tiles = ((m + TM - 1) / TM) * ((n + TN - 1) / TN), nblk = k / 256;
    // (up to 128 lhs rows half of a tile's wavefront rows have no work, and the quarters pay up to 64 tiles: 4096 x 4096, 65 rows)
    const bool few = tiles <= std::min<int64_t>(64, nblk + nblk / 4) || (m <= 128 && tiles <= 64);
    return few && nblk >= 8 && 4 * ((tiles + 7) / 8) <= std::max(1, compute_units() / 8);
}
hipError_t launch_add_part(float* out, const float* part, int64_t count, hipStream_t s) {
    add_part_kernel<<<dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s>>>(out, part, count);
    return hipGetLastError();
}
bool quarter_mode(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    if (lhs_dtype != QMM_BF16 || wide_tiles(encoding, m, n) || kernel_disabled("planes_quarters")) return false;
    return few_tiles_for_quarters(m, n, k);
}
int64_t quarter_part_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    return quarter_mode(encoding, lhs_dtype, m, n, k) ? (m * n * 4 + 255) / 256 * 256 : 0;
}

// An fp32 lhs of up to 256 rows goes through the GEMM as ONE lhs of twice the rows, hi plane on top of residual plane, like a
// bf16 lhs (one pass, every way of cutting few tiles along K open to it); the GEMM writes into the workspace and the pass
// that adds K quarters adds the two halves of the rows as well.  Two passes, the second one over whole tiles onto the
// first one's result, had cost 4096 x 4096 with 65 fp32 rows 110 us (Q5_K) and 176 us (Q6_K) against 31 and 56 us for bf16 rows.
bool planes_twin(int lhs_dtype, int64_t m) { return lhs_dtype == QMM_F32 && m <= 256 && twin_rows_allowed() && !kernel_disabled("planes_twin_rows"); }
// rows and type that the GEMM sees
int64_t gemm_rows(int lhs_dtype, int64_t m) { return planes_twin(lhs_dtype, m) ? 2 * m : m; }
int gemm_dtype(int lhs_dtype, int64_t m) { return planes_twin(lhs_dtype, m) ? QMM_BF16 : lhs_dtype; }
// what follows the lhs planes (and, inside qmm_matmul, the weight planes) in the workspace: the second buffer of the quarter
// mode, or, for twin rows, the GEMM's result (2 m x n, whole) and that second buffer right behind it
int64_t planes_tail_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    if (!planes_twin(lhs_dtype, m)) return quarter_part_bytes(encoding, lhs_dtype, m, n, k);
    return (2 * m * n * 4 * (quarter_mode(encoding, QMM_BF16, 2 * m, n, k) ? 2 : 1) + 255) / 256 * 256;
}

int64_t gemm_planes_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    const int64_t me = gemm_rows(lhs_dtype, m);
    const int dte = gemm_dtype(lhs_dtype, m);
    const bool q6 = encoding == QMM_Q6_K, wide = wide_tiles(encoding, me, n);
    const int64_t nblk_tile = blocks_per_tile(encoding, me, n, k);
    const int64_t lhs = (lhs_planes(nullptr, dte, me, k, TM, nblk_tile * 256).bytes + 255) / 256 * 256;
    return lhs + plane_space(nullptr, n, k, q6 ? 2 : 1, !q6 && !wide, nblk_tile).bytes + planes_tail_bytes(encoding, lhs_dtype, m, n, k);
}

namespace {

// One launch of the preparation kernel and the GEMM launches behind it.  `ps` holds the planes, nblk_tile blocks of four steps
// per tile (the super-blocks, then extension blocks if any); convert: they are made from `w` in the preparation launch,
// otherwise they were made earlier.  wide (not Q6_K): the 256 x 256 tiles, which walk the extension blocks for the min term;
// the 256 x 128 kernel reads the min operands from ps.mtab and skips the extension blocks if the planes have them.
// `tail`: the workspace behind the planes (planes_tail_bytes).  m, lhs_dtype: as the caller gave them; nblk_tile and wide: for
// the rows the GEMM sees (gemm_rows).
hipError_t run_kquant_planes(int encoding, const void* lhs, int lhs_dtype, const uint8_t* w, bool convert, int64_t m, int64_t n, int64_t k,
                             float* out, void* lhs_space, const PlaneSpace& ps, int nblk_tile, bool wide, float* tail, hipStream_t s) {
    const bool q6 = encoding == QMM_Q6_K;
    const bool twin = planes_twin(lhs_dtype, m);
    const int64_t m_given = m;
    float* const out_given = out;
    const int prep_dtype = lhs_dtype;  // (the narrowing reads the caller's values)
    if (twin) {
        m *= 2;
        lhs_dtype = QMM_BF16;
        out = tail;
        tail += m * n;
    }
    float* part = quarter_mode(encoding, lhs_dtype, m, n, k) ? tail : nullptr;
    const int nblk = (int)(k / 256), lhs_ext = wide ? nblk_tile - nblk : 0;
    const int64_t lda = (int64_t)(nblk + lhs_ext) * 256;
    LhsPlanes p = lhs_planes(lhs_space, lhs_dtype, m, k, TM, lda);
    LhsPlanes pp = p;  // as the narrowing launch sees them
    if (twin) pp.a16_lo = p.a16 + m_given * lda;
    hipError_t e = q6 ? allow_full_lds<gemm_planes2_kernel>() : wide ? hipSuccess : allow_full_lds<gemm_planes_kernel>();
    if (e != hipSuccess) return e;
    const int tiles_m = (int)((m + TM - 1) / TM), tiles_n128 = (int)((n + TN - 1) / TN);
    const int tiles_n = tiles_n128;  // the column tiles of the 256 x 128 kernels
    const int total = tiles_m * tiles_n, per_xcd = (total + 7) / 8;
    // Tiles for no more than half of the compute units: the launch still takes a workgroup per compute unit, and the unit
    // arithmetic then cuts every tile in two K halves.  A tile's time is set by K, so up to 96 tiles this takes a quarter to
    // a third off the call (14336 x 4096 Q6_K, 65 lhs rows: 160 -> 118 us; 4096 x 4096 Q5_K, 256 rows: 66 -> 48 us); from 112
    // tiles on the zeroing and the atomic adds cost what the halves gain (4096 x 4096, 1024 rows: 63 -> 72 us), unless K is long
    // (4096 x 14336, 1024 rows: 188 -> 159 us).
    const int per_xcd_cus = std::max(1, compute_units() / 8);
    // (A single row tile with at most 192 rows leaves a wavefront row without work, and the halves pay up to 128 tiles:
    // 14336 x 4096 with 65 rows, Q6_K 160 -> 118 us; with 256 rows 60 -> 62 us.)
    const bool halve_all = 2 * per_xcd <= per_xcd_cus && nblk >= 2 && (total <= 96 || nblk >= 32 || m <= 192);
    const int wg = 8 * (halve_all || part ? per_xcd_cus : std::min(per_xcd, per_xcd_cus));
    const WideLaunch L = wide ? wide_launch(out, m, n, nblk_tile) : WideLaunch{};
    SplitTiles z = wide ? L.z : split_tiles(out, m, n, tiles_m, tiles_n, nblk, wg, TN);
    if (part) {  // quarter mode: no halves, the whole of out and part zeroed
        z.max_split = 0;
        z.part = part;
    }
    const int max_split = z.max_split;
    const int64_t zero_blocks = part ? (m * n + kZeroFlatFloats - 1) / kZeroFlatFloats : (int64_t)max_split * 64;
    const int64_t conv = convert ? (int64_t)tiles_n128 * nblk * 4 : 0, blocks = conv + m_given + zero_blocks;
    if (blocks > INT32_MAX || lda * 2 * 8 > INT32_MAX) return hipErrorInvalidValue;
    const dim3 pgrid((unsigned)blocks);
    auto prologue = [&](auto enc_c) {
        constexpr int ENC = decltype(enc_c)::value;
        if (prep_dtype == QMM_F32)
            planes_prologue_kernel<ENC, float><<<pgrid, dim3(256), 0, s>>>(w, nblk, nblk_tile, tiles_n128, ps.planes, ps.dtab, ps.mtab, (int)conv,
                                                                          (const float*)lhs, (int)k, lhs_ext, (int)m_given, pp, z,
                                                                          twin ? (int)m_given : 0);
        else
            planes_prologue_kernel<ENC, uint16_t><<<pgrid, dim3(256), 0, s>>>(w, nblk, nblk_tile, tiles_n128, ps.planes, ps.dtab, ps.mtab, (int)conv,
                                                                             (const uint16_t*)lhs, (int)k, lhs_ext, (int)m_given, pp, z, 0);
    };
    if (q6) prologue(std::integral_constant<int, QMM_Q6_K>{});
    else if (encoding == QMM_Q4_K) prologue(std::integral_constant<int, QMM_Q4_K>{});
    else prologue(std::integral_constant<int, QMM_Q5_K>{});
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    for (int pass = 0; pass < (p.a16_lo ? 2 : 1); pass++) {
        // fp32 lhs: the residual plane of the lhs in a second launch, added on top (whole tiles only, no min term)
        const _Float16* a = pass == 0 ? p.a16 : p.a16_lo;
        const int split = pass == 0 && max_split > 0 ? 1 : 0;
        if (q6)
            gemm_planes2_kernel<<<dim3((unsigned)wg), dim3(512), kPlanes2Lds, s>>>(ps.planes, ps.dtab, a, p.inv, out, (int)m, (int)n, (int)k,
                                                                                 tiles_m, tiles_n, pass, split, part);
        else if (wide) {
            e = run_wide<4>(L, ps.planes, ps.dtab, a, p.inv, out, m, n, lda, pass == 0 ? nblk_tile : nblk, nblk_tile, pass, s);
            if (e != hipSuccess) return e;
        } else
            gemm_planes_kernel<<<dim3((unsigned)wg), dim3(512), kPlanesLds, s>>>(ps.planes, ps.dtab, ps.mtab, a, p.asum, p.inv, out, (int)m, (int)n,
                                                                               (int)k, tiles_m, tiles_n, nblk_tile, pass == 0, pass, split, part);
    }
    // twin rows: the row halves (and the quarter mode's second buffer right behind them: four terms) into the caller's tensor
    if (twin) return launch_sum_shares(out, out_given, m_given * n, part ? 4 : 2, s);
    if (part) add_part_kernel<<<dim3((unsigned)((m * n + 255) / 256)), dim3(256), 0, s>>>(out, part, m * n);
    return hipGetLastError();
}

// Planes that outlive a call serve every row count, so Q4_K / Q5_K carry the min operands in both forms: extension blocks for
// the wide GEMM and the table for the 256 x 128 kernel.
int repacked_blocks_per_tile(int encoding, int64_t k) {
    const int nblk = (int)(k / 256);
    return encoding == QMM_Q6_K ? nblk : nblk + (nblk + 7) / 8;
}
PlaneSpace repacked_space(int encoding, void* base, int64_t n, int64_t k) {
    const bool q6 = encoding == QMM_Q6_K;
    return plane_space(base, n, k, q6 ? 2 : 1, !q6, repacked_blocks_per_tile(encoding, k));
}

}  // namespace

hipError_t launch_gemm_planes(int encoding, const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                              float* out, void* workspace, hipStream_t s) {
    const int64_t me = gemm_rows(lhs_dtype, m);
    const bool q6 = encoding == QMM_Q6_K, wide = wide_tiles(encoding, me, n);
    const int nblk_tile = (int)blocks_per_tile(encoding, me, n, k);
    const int64_t lhs_bytes = (lhs_planes(nullptr, gemm_dtype(lhs_dtype, m), me, k, TM, (int64_t)nblk_tile * 256).bytes + 255) / 256 * 256;
    const PlaneSpace ps = plane_space((uint8_t*)workspace + lhs_bytes, n, k, q6 ? 2 : 1, !q6 && !wide, nblk_tile);
    float* tail = (float*)((uint8_t*)workspace + lhs_bytes + ps.bytes);
    return run_kquant_planes(encoding, lhs, lhs_dtype, w, true, m, n, k, out, workspace, ps, nblk_tile, wide, tail, s);
}

// Weight planes kept across calls (the weights of a model are converted once, at load time): the conversion alone, and the
// GEMM over planes made by it.
int64_t repacked_planes_bytes(int encoding, int64_t n, int64_t k) { return repacked_space(encoding, nullptr, n, k).bytes; }

hipError_t launch_repack_planes(int encoding, const uint8_t* w, int64_t n, int64_t k, void* packed, hipStream_t s) {
    const int nblk = (int)(k / 256), nblk_tile = repacked_blocks_per_tile(encoding, k);
    const PlaneSpace ps = repacked_space(encoding, packed, n, k);
    const int tiles_n128 = (int)((n + TN - 1) / TN);
    const int64_t conv = (int64_t)tiles_n128 * nblk * 4;
    if (conv > INT32_MAX) return hipErrorInvalidValue;
    SplitTiles z{};
    z.n = (int)n;
    const LhsPlanes none{};
    const dim3 grid((unsigned)conv);
    if (encoding == QMM_Q6_K)
        planes_prologue_kernel<QMM_Q6_K, uint16_t><<<grid, dim3(256), 0, s>>>(w, nblk, nblk_tile, tiles_n128, ps.planes, ps.dtab, ps.mtab, (int)conv, nullptr, (int)k, 0, 0, none, z, 0);
    else if (encoding == QMM_Q4_K)
        planes_prologue_kernel<QMM_Q4_K, uint16_t><<<grid, dim3(256), 0, s>>>(w, nblk, nblk_tile, tiles_n128, ps.planes, ps.dtab, ps.mtab, (int)conv, nullptr, (int)k, 0, 0, none, z, 0);
    else
        planes_prologue_kernel<QMM_Q5_K, uint16_t><<<grid, dim3(256), 0, s>>>(w, nblk, nblk_tile, tiles_n128, ps.planes, ps.dtab, ps.mtab, (int)conv, nullptr, (int)k, 0, 0, none, z, 0);
    return hipGetLastError();
}

// With the conversion out of the way the plane GEMMs pay from fewer rows on than inside qmm_matmul.
// 14336 x 4096: Q5_K 40 lhs rows 39.5 us against 52 us for three passes of the small-batch kernel, Q6_K 53 us against 44 / 66 us
// for two / three passes of its decode kernel; 4096 x 4096: Q5_K 36 us against 30 us (48 rows) / 40 us (64), Q6_K 45 against 38 / 53.
// (Q4_K: below.)
bool repacked_planes_wanted(int encoding, int64_t m, int64_t n, int64_t k) {
    if (k % 256 || k < 256) return false;
    if (encoding == QMM_Q6_K || encoding == QMM_Q5_K) return m > 48 || (m > 32 && n * k >= ((int64_t)48 << 20));
    if (encoding != QMM_Q4_K) return false;
    // Against qmm_matmul's kernels that unpack as they go, bf16 lhs, microseconds (those / the planes): 4096 x 4096 with 384 / 1024 /
    // 2048 rows (64 / 128 / 256 tiles) 37 / 47, 59 / 64, 92 / 86; 14336 x 4096 with 256 / 384 rows (112 / 224 tiles) 59 / 62, 79 / 76;
    // 4096 x 14336 with 512 / 768 rows (64 / 96 tiles) 102 / 108, 153 / 134; 1024 x 4096 with 2048 rows (64 tiles) 45 / 54.
    // Those are replays of one matrix, whose planes then come from the last-level cache.  Inside a layer's step (seven matrices,
    // 0.5 GB of planes against 0.12 GB of packed weights) the planes come from memory, 2 bytes a weight whatever the row count:
    // with 512 rows the kept planes of gate and up cost the step 386 -> 408 us, with 768 rows they save it 633 -> 569.
    const int64_t tiles = ((m + TM - 1) / TM) * ((n + TN - 1) / TN);
    return m > 512 && (tiles >= 200 || (k >= 8192 && tiles >= 96));
}
static int64_t repacked_lhs_bytes(int encoding, int lhs_dtype, int64_t m, int64_t k) {
    return (lhs_planes(nullptr, lhs_dtype, m, k, TM, (int64_t)repacked_blocks_per_tile(encoding, k) * 256).bytes + 255) / 256 * 256;
}
int64_t repacked_planes_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    return repacked_lhs_bytes(encoding, gemm_dtype(lhs_dtype, m), gemm_rows(lhs_dtype, m), k) + planes_tail_bytes(encoding, lhs_dtype, m, n, k);
}
hipError_t launch_gemm_planes_repacked(int encoding, const void* lhs, int lhs_dtype, const void* packed, int64_t m, int64_t n, int64_t k,
                                       float* out, void* workspace, hipStream_t s) {
    const PlaneSpace ps = repacked_space(encoding, const_cast<void*>(packed), n, k);
    const int64_t me = gemm_rows(lhs_dtype, m);
    float* tail = (float*)((uint8_t*)workspace + repacked_lhs_bytes(encoding, gemm_dtype(lhs_dtype, m), me, k));
    return run_kquant_planes(encoding, lhs, lhs_dtype, nullptr, false, m, n, k, out, workspace, ps, repacked_blocks_per_tile(encoding, k),
                             wide_tiles(encoding, me, n), tail, s);
}

// GPTQ through the plane GEMM: groups of 128 or 256 (a scale block is two or four steps), plain groups (no act-order), and
// enough 256 x 256 tiles that the conversion pass (the weights once) costs less than the GEMM gains.
bool gemm_gptq_planes_wanted(int64_t m, int64_t n, int64_t k, int group) {
    if (kernel_disabled("gptq_planes") || (group != 128 && group != 256) || k % 256 || n % 8) return false;
    return m >= kOptionalPlanesMinRows && wide_tiles(QMM_GPTQ, m, n);
}

int64_t gemm_gptq_planes_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    const int64_t lhs = (lhs_planes(nullptr, lhs_dtype, m, k, TM).bytes + 255) / 256 * 256;
    return lhs + plane_space(nullptr, n, k, 1, false, k / 256, k / 128).bytes;  // (tables sized for the smaller group)
}

namespace {
// convert: the planes in `ps` are made from the checkpoint tensors in the preparation launch; otherwise they were made earlier.
hipError_t run_gptq_planes(const void* lhs, int lhs_dtype, const uint32_t* qweight, const uint16_t* scales, const uint32_t* qzeros, bool convert,
                           int64_t m, int64_t n, int64_t k, int group, float* out, void* lhs_space, const PlaneSpace& ps, hipStream_t s) {
    const int groups = (int)(k / group), nblk256 = (int)(k / 256);
    const LhsPlanes p = lhs_planes(lhs_space, lhs_dtype, m, k, TM);
    const WideLaunch L = wide_launch(out, m, n, groups);
    const SplitTiles& z = L.z;
    const int tiles_n128 = L.tiles_n128;
    hipError_t e = hipSuccess;
    const int64_t conv = convert ? (int64_t)tiles_n128 * nblk256 : 0, blocks = conv + m + (int64_t)z.max_split * 64;
    if (blocks > INT32_MAX || k * 2 * 8 > INT32_MAX) return hipErrorInvalidValue;
    if (lhs_dtype == QMM_F32)
        gptq_planes_prologue_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(qweight, scales, qzeros, group, tiles_n128, ps.planes, ps.dtab,
                                                                                       (int)conv, (const float*)lhs, (int)k, (int)m, p, z);
    else
        gptq_planes_prologue_kernel<uint16_t><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(qweight, scales, qzeros, group, tiles_n128, ps.planes, ps.dtab,
                                                                                          (int)conv, (const uint16_t*)lhs, (int)k, (int)m, p, z);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    for (int pass = 0; pass < (p.a16_lo ? 2 : 1); pass++) {
        const _Float16* a = pass == 0 ? p.a16 : p.a16_lo;
        e = group == 128 ? run_wide<2>(L, ps.planes, ps.dtab, a, p.inv, out, m, n, k, groups, groups, pass, s)
                         : run_wide<4>(L, ps.planes, ps.dtab, a, p.inv, out, m, n, k, groups, groups, pass, s);
        if (e != hipSuccess) return e;
    }
    return hipGetLastError();
}
// (steps per tile k / 64 = 4 blocks of 256: the plane array is sized in those; the tables in groups of 128, the smaller size)
PlaneSpace gptq_space(void* base, int64_t n, int64_t k) { return plane_space(base, n, k, 1, false, k / 256, k / 128); }
}  // namespace

hipError_t launch_gemm_gptq_planes(const void* lhs, int lhs_dtype, const uint32_t* qweight, const uint16_t* scales, const uint32_t* qzeros,
                                   int64_t m, int64_t n, int64_t k, int group, float* out, void* workspace, hipStream_t s) {
    const int64_t lhs_bytes = (lhs_planes(nullptr, lhs_dtype, m, k, TM).bytes + 255) / 256 * 256;
    return run_gptq_planes(lhs, lhs_dtype, qweight, scales, qzeros, true, m, n, k, group, out, workspace,
                           gptq_space((uint8_t*)workspace + lhs_bytes, n, k), s);
}

// GPTQ planes kept across calls.
bool gptq_planes_supported(int64_t n, int64_t k, int group) { return (group == 128 || group == 256) && k % 256 == 0 && k >= 256 && n % 8 == 0; }
int64_t repacked_gptq_bytes(int64_t n, int64_t k) { return gptq_space(nullptr, n, k).bytes; }
hipError_t launch_repack_gptq(const uint32_t* qweight, const uint16_t* scales, const uint32_t* qzeros, int64_t n, int64_t k, int group, void* packed,
                              hipStream_t s) {
    const PlaneSpace ps = gptq_space(packed, n, k);
    const int tiles_n128 = (int)((n + TN - 1) / TN);
    const int64_t conv = (int64_t)tiles_n128 * (k / 256);
    if (conv > INT32_MAX) return hipErrorInvalidValue;
    SplitTiles z{};
    z.n = (int)n;
    gptq_planes_prologue_kernel<uint16_t><<<dim3((unsigned)conv), dim3(256), 0, s>>>(qweight, scales, qzeros, group, tiles_n128, ps.planes, ps.dtab, (int)conv,
                                                                                    nullptr, (int)k, 0, LhsPlanes{}, z);
    return hipGetLastError();
}
// Against the GEMM that unpacks as it goes, whose few tiles are cut into K shares (bf16 lhs, microseconds, that GEMM / the planes):
// 14336 x 4096 with 512 / 1024 / 2048 rows 74 / 74, 129 / 107, 228 / 205; 4096 x 4096 with 256 / 1024 / 2048 rows 31 / 55, 57 / 76,
// 83 / 83; 4096 x 14336 with 256 / 2048 rows 55 / 149, 263 / 262: the planes serve the problems with enough 256 x 256 tiles.
bool repacked_gptq_wanted(int64_t m, int64_t n) {
    return m > 256 && wide_tiles(QMM_GPTQ, m, n);
}
int64_t repacked_gptq_workspace_bytes(int lhs_dtype, int64_t m, int64_t k) { return (lhs_planes(nullptr, lhs_dtype, m, k, TM).bytes + 255) / 256 * 256; }
hipError_t launch_gemm_gptq_repacked(const void* lhs, int lhs_dtype, const void* packed, int64_t m, int64_t n, int64_t k, int group, float* out,
                                     void* workspace, hipStream_t s) {
    return run_gptq_planes(lhs, lhs_dtype, nullptr, nullptr, nullptr, false, m, n, k, group, out, workspace, gptq_space(const_cast<void*>(packed), n, k), s);
}

}  // namespace qmm
