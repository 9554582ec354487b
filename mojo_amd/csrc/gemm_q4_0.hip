// Q4_0 weights x Q8_0-quantised activations on the int8 matrix cores, for m >= 5 lhs rows.
//
// The reference CPU kernel quantises the lhs to Q8_0 (32-wide blocks, fp16 scale) and forms, per
// (lhs row, weight row, block), the integer dot of the codes times the product of the two block
// scales.  Here one v_mfma_i32_16x16x32_i8 produces the 16 x 16 integer block dots of 16 lhs rows
// against 16 weight rows for one block (K = 32 is exactly a block, so the integer sums are the
// reference's, bit for bit), and the lanes apply  acc += float(isum - 8 asum) * (d_w * d_a)  as the
// decode kernel does.
//
// lhs side: a pre-pass writes the Q8_0 codes in matrix-core operand order (for every 16-row tile and
// block, 64 lanes x 8 bytes, so a wavefront's operand load is 512 contiguous bytes), and the block
// scales and code sums transposed to [tile][block][16 rows] so that the four rows a lane scales are
// one 16-byte load.  Rows beyond m are zero.
//
// Weight side: 18-byte blocks are only 2-byte aligned.  A wavefront owns 16 weight rows and a
// share of K; it copies runs of 16 blocks of its 16 rows into private LDS with aligned 16-byte
// loads (19 pieces per row and run), and each lane reads its 8 code bytes and the block scale as
// aligned dwords joined by v_alignbyte_b32.  The nibbles stay unsigned (0..15); the -8 goes through
// the activation code sums.  The 4 or 8 wavefronts of a workgroup add their K shares through LDS.
// For m > 16 the grid's second dimension walks groups of four 16-row tiles, each group streaming the
// weights again (this path is bound by the per-block fp32 scaling in the vector ALUs, not by the
// matrix cores: 4 instructions per (lhs row, weight row, block)).
//
// Up to 16 lhs rows with K a multiple of 256 take gemm_q4_0_small_kernel instead (described at the kernel): 16
// wavefronts per workgroup, a ring of 16-row items in LDS shared by the workgroup and loaded row by row, the lhs
// operands of a wavefront's 8 blocks per 4096 columns in registers.  Inside a wavefront's 144 bytes of a row the block
// offsets 18 j are compile-time, so the byte alignment of every field is too.
#include <stdlib.h>

#include <algorithm>

#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {

typedef int int4v __attribute__((ext_vector_type(4)));

namespace {

constexpr int kRun = 16;                 // blocks per staged run
constexpr int kRowPieces = 19;           // 16-byte pieces per row and run: 288 bytes + lead-in
constexpr int kRowLds = kRowPieces * 16; // 304
constexpr int kWaveLds = 16 * kRowLds + 16;  // one dword of read-ahead past the last row

struct LhsQ8T {
    int8_t* codes;   // [tiles][k/32][64][8]
    float* scale;    // [tiles][k/32][16]
    int32_t* sum;    // [tiles][k/32][16]
    int64_t bytes;
};
inline LhsQ8T lhs_q8t(void* ws, int64_t m, int64_t k) {
    auto up = [](int64_t v) { return (v + 255) / 256 * 256; };
    const int64_t tiles = (m + 15) / 16, nkb = k / 32;
    LhsQ8T p;
    char* b = (char*)ws;
    p.codes = (int8_t*)b;
    int64_t off = up(tiles * nkb * 512);
    p.scale = (float*)(b + off);
    off += up(tiles * nkb * 64);
    p.sum = (int32_t*)(b + off);
    off += up(tiles * nkb * 64);
    p.bytes = off;
    return p;
}

}  // namespace

// One 32-lane group per (padded lhs row, block); same rounding rule as the Q8_0 quantiser:
// d = amax / 127 stored as fp16, codes = round-half-away(x / d) with the fp32 d.
// WORDS: the K order of gemm_q4_0_small_kernel inside a block: k-group g holds the elements whose weight nibbles share
// dword g of the block's 16 code bytes (4 g .. 4 g + 3, then 16 + 4 g .. 16 + 4 g + 3) instead of 8 g .. 8 g + 7.
template <typename InT, bool WORDS>
__global__ __launch_bounds__(256) void quantize_q8_0_operand_kernel(const InT* __restrict__ x, int m, int k, int64_t ngroups,
                                                                    int8_t* __restrict__ codes, float* __restrict__ dscale,
                                                                    int32_t* __restrict__ csum) {
    const int64_t grp = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    const int l = threadIdx.x & 31;
    if (grp >= ngroups) return;
    const int nkb = k >> 5;
    const int64_t row = grp / nkb;
    const int kb = (int)(grp - row * nkb);
    const float v = row < m ? load_f32(x, row * (int64_t)k + kb * 32 + l) : 0.0f;
    float amax = fabsf(v);
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 32));
    uint16_t dh;
    const float id = q8_0_block_rule(amax, dh);
    const int q = q8_0_code(v, id);
    int sum = q;
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 32);
    const int64_t tile = row >> 4;
    const int mm = (int)(row & 15);
    const int g = WORDS ? (l & 15) >> 2 : l >> 3, pos = WORDS ? (l & 3) + 4 * (l >> 4) : l & 7;
    const int64_t tb = tile * nkb + kb;
    codes[(tb * 64 + g * 16 + mm) * 8 + pos] = (int8_t)q;
    if (l == 0) {
        if (WORDS) {
            // one 64-byte record per block: 16 scales as fp16, then 16 times -8 * code sum as int16 (|sum| <= 32 * 127)
            uint16_t* rec = (uint16_t*)dscale + tb * 32;
            rec[mm] = dh;
            rec[16 + mm] = (uint16_t)(int16_t)(-8 * sum);
        } else {
            dscale[tb * 16 + mm] = h2f(dh);
            csum[tb * 16 + mm] = sum;
        }
    }
}

template <int MG>
__global__ __launch_bounds__(512) void gemm_q4_0_kernel(const uint8_t* __restrict__ w, const int8_t* __restrict__ codes,
                                                        const float* __restrict__ dscale, const int32_t* __restrict__ csum,
                                                        float* __restrict__ out, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nkb = k >> 5;
    const int64_t row_bytes = (int64_t)nkb * Q4_0_BPB;
    const int n0 = (int)blockIdx.x * 16;
    const int tile0 = (int)blockIdx.y * MG;           // first 16-row lhs tile of this pass
    const int tiles = (m + 15) >> 4;
    const int nn = lane & 15, g = lane >> 4;
    uint8_t* wbuf = smem + wave * kWaveLds;
    const uint32_t* lds32 = (const uint32_t*)wbuf;

    // this wavefront's share of K (4 or 8 wavefronts per workgroup)
    const int nw = (int)(blockDim.x >> 6);
    const int kb0 = wave * nkb / nw, kb1 = (wave + 1) * nkb / nw;

    float acc[MG][4];
#pragma unroll
    for (int t = 0; t < MG; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;

    // piece p = lane + 64 i of the run: row p / 19, 16-byte piece p % 19 of that row's run
    int prow[5], pidx[5];
#pragma unroll
    for (int i = 0; i < 5; i++) {
        const int p = min(lane + 64 * i, 16 * kRowPieces - 1);  // pieces 0..303; the last load is partial
        prow[i] = p / kRowPieces;
        pidx[i] = p - prow[i] * kRowPieces;
    }
    const uint8_t* my_row = w + (int64_t)min(n0 + nn, n - 1) * row_bytes;  // the row this lane decodes

    for (int kb = kb0; kb < kb1; kb += kRun) {
        const int nb = min(kRun, kb1 - kb);
        // stage: aligned 16-byte pieces covering blocks kb .. kb + nb - 1 of each of the 16 rows
        uint4 r0, r1, r2, r3, r4;
#define QMM_STAGE_LOAD(I, R)                                                                                          \
    do {                                                                                                              \
        const uintptr_t ad_ = (uintptr_t)(w + (int64_t)min(n0 + prow[I], n - 1) * row_bytes + (int64_t)kb * Q4_0_BPB); \
        const int dl_ = (int)(ad_ & 15);                                                                              \
        const int last_ = (dl_ + nb * Q4_0_BPB + 15) / 16 - 1;                                                        \
        R = ((const uint4*)(ad_ - (uintptr_t)dl_))[min(pidx[I], last_)];                                              \
    } while (0)
        QMM_STAGE_LOAD(0, r0);
        QMM_STAGE_LOAD(1, r1);
        QMM_STAGE_LOAD(2, r2);
        QMM_STAGE_LOAD(3, r3);
        QMM_STAGE_LOAD(4, r4);
#undef QMM_STAGE_LOAD
        __builtin_amdgcn_wave_barrier();  // the previous run's LDS reads are issued (LDS is in order per wavefront)
        *(uint4*)(wbuf + prow[0] * kRowLds + pidx[0] * 16) = r0;
        *(uint4*)(wbuf + prow[1] * kRowLds + pidx[1] * 16) = r1;
        *(uint4*)(wbuf + prow[2] * kRowLds + pidx[2] * 16) = r2;
        *(uint4*)(wbuf + prow[3] * kRowLds + pidx[3] * 16) = r3;
        if (lane + 256 < 16 * kRowPieces) *(uint4*)(wbuf + prow[4] * kRowLds + pidx[4] * 16) = r4;
        __builtin_amdgcn_wave_barrier();

        const int delta = (int)((uintptr_t)(my_row + (int64_t)kb * Q4_0_BPB) & 15);
        for (int b = 0; b < nb; b++) {
            // weight operand: 8 code bytes of k-group g (low nibbles of bytes 8(g&1).., or their high nibbles)
            const int boff = nn * kRowLds + delta + Q4_0_BPB * b;
            const int qoff = boff + 2 + 8 * (g & 1);
            const int wi = qoff >> 2;
            const uint32_t sh = (uint32_t)(qoff & 3);
            const uint32_t w0 = lds32[wi], w1 = lds32[wi + 1], w2 = lds32[wi + 2];
            uint32_t lo = __builtin_amdgcn_alignbyte(w1, w0, sh), hi = __builtin_amdgcn_alignbyte(w2, w1, sh);
            if (g & 2) {
                lo >>= 4;
                hi >>= 4;
            }
            lo &= 0x0F0F0F0Fu;
            hi &= 0x0F0F0F0Fu;
            const long bop = (long)(((uint64_t)hi << 32) | lo);
            const uint32_t dw32 = lds32[boff >> 2] >> (8 * (boff & 3));
            const float dw = h2f((uint16_t)(dw32 & 0xffffu));
#pragma unroll
            for (int t = 0; t < MG; t++) {
                const int tile = min(tile0 + t, tiles - 1);
                const int64_t tb = (int64_t)tile * nkb + kb + b;
                const long aop = *(const long*)(codes + (tb * 64 + lane) * 8);
                const float4 da = *(const float4*)(dscale + tb * 16 + 4 * g);
                const int4v as = *(const int4v*)(csum + tb * 16 + 4 * g);
                int4v z = {0, 0, 0, 0};
                const int4v dot = __builtin_amdgcn_mfma_i32_16x16x32_i8(aop, bop, z, 0, 0, 0);
                acc[t][0] = fmaf((float)(dot[0] - 8 * as[0]), dw * da.x, acc[t][0]);
                acc[t][1] = fmaf((float)(dot[1] - 8 * as[1]), dw * da.y, acc[t][1]);
                acc[t][2] = fmaf((float)(dot[2] - 8 * as[2]), dw * da.z, acc[t][2]);
                acc[t][3] = fmaf((float)(dot[3] - 8 * as[3]), dw * da.w, acc[t][3]);
            }
        }
    }

    // add the K shares: red[wave][MG*4][64]
    __syncthreads();
    float* red = (float*)smem;
#pragma unroll
    for (int t = 0; t < MG; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) red[(wave * MG * 4 + t * 4 + r) * 64 + lane] = acc[t][r];
    __syncthreads();
    if (wave == 0 && n0 + nn < n) {
#pragma unroll
        for (int t = 0; t < MG; t++) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = (tile0 + t) * 16 + 4 * g + r;
                if (row < m) {
                    const int i = (t * 4 + r) * 64 + lane;
                    float v = (red[i] + red[MG * 4 * 64 + i]) + (red[2 * MG * 4 * 64 + i] + red[3 * MG * 4 * 64 + i]);
                    if (nw == 8)
                        v += (red[4 * MG * 4 * 64 + i] + red[5 * MG * 4 * 64 + i]) +
                             (red[6 * MG * 4 * 64 + i] + red[7 * MG * 4 * 64 + i]);
                    out[(int64_t)row * n + n0 + nn] = v;
                }
            }
        }
    }
}

namespace {
constexpr int kSWaves = 16;                          // wavefronts per workgroup
constexpr int kSGroup = 128;                         // blocks per group: 4096 columns, 2304 bytes of a row
constexpr int kSBlk = kSGroup / kSWaves;             // 8 blocks per wavefront and group
constexpr int kSParts = 1;                           // an item is 1 / kSParts of a group's columns of a tile's 16 rows
constexpr int kSPartBlk = kSBlk / kSParts;           // blocks per wavefront and item
constexpr int kSItemBlk = kSGroup / kSParts;         // blocks of an item
constexpr int kSItemRow = kSItemBlk * Q4_0_BPB;      // bytes of a row of an item: 2304 / kSParts
constexpr int kSPieces = kSItemRow / 16;             // 16-byte pieces of that
constexpr int kSLoads = (kSPieces + 63) / 64;        // load instructions per wavefront and item
constexpr int kSRowLds = kSItemRow + 16;             // rows an odd multiple of 4 dwords apart: 16 rows on 16 bank groups
constexpr int kSSlot = 16 * kSRowLds;                // one item, 16 rows
// Items in flight beyond the one being used.  Measured at 16 x 14336 x 4096 (the call with its lhs quantiser, us):
// whole groups as items, 1 / 2 / 3 in flight: 13.9 / 14.4 / 15.1; half groups, 4 / 6 in flight: 15.0 / 15.8.  Every compute
// unit asks for its data in the same microsecond, and more requests per compute unit make the first item later.
constexpr int kSAhead = 1 * kSParts;
constexpr int kSSlots = kSAhead + kSParts;
constexpr int kSMaxTiles = 4;
constexpr int kSRing = kSSlots * kSSlot;
constexpr int kSSums = kSWaves * kSMaxTiles * 4 * 64 * 4;     // 65536: the final sums reuse the ring's memory
constexpr int kSScales = kSBlk * 64;                          // per wavefront: scale / code-sum records of its 8 blocks
constexpr int kSLds = (kSRing > kSSums ? kSRing : kSSums) + kSWaves * kSScales;
static_assert(kSItemRow % 16 == 0 && (kSRowLds / 4) % 8 == 4, "whole pieces; row stride an odd multiple of 4 dwords");
static_assert(kSAhead * kSLoads < 64, "the waits count load instructions in six bits");
static_assert(kSLds <= 160 * 1024, "LDS of a compute unit");

typedef _Float16 q40_half2 __attribute__((ext_vector_type(2)));

// wait until at most `items` items (kSLoads load instructions each) are outstanding
__device__ __forceinline__ void q40_wait(int items) {
    switch (items < kSAhead ? items : kSAhead) {
        case 0: wait_vmcnt<0>(); break;
        case 1: wait_vmcnt<kSLoads>(); break;
        case 2: wait_vmcnt<2 * kSLoads>(); break;
        case 3: wait_vmcnt<3 * kSLoads>(); break;
        case 4: wait_vmcnt<4 * kSLoads>(); break;
        case 5: wait_vmcnt<5 * kSLoads>(); break;
        case 6: wait_vmcnt<6 * kSLoads>(); break;
        case 7: wait_vmcnt<7 * kSLoads>(); break;
        default: wait_vmcnt<kSAhead * kSLoads>(); break;
    }
}
}  // namespace

// A workgroup of 16 wavefronts walks up to 4 tiles of 16 weight rows, in groups of 4096 columns (128 blocks, 2304 bytes
// of a row).  An item is a tile's 16 rows x one part of a group (the whole group as built).  Loading and arithmetic are
// cut differently: wavefront w LOADS row w of an item, contiguous bytes, global -> LDS directly into a ring of items
// shared by the workgroup (whole DRAM pages per instruction), and it COMPUTES a fixed set of 8 blocks per group of all
// 16 rows, 8 / parts in each part, whose lhs operands it keeps in registers for all tiles; one barrier per item.  Per
// block: one dword of nibbles per lane (two operand dwords by mask and shift), one matrix-core instruction whose
// accumulator input is -8 * (code sum), so that it returns isum - 8 asum, and acc += float(that) * (d_w * d_a), the
// scale product formed from the two fp16 values.
__global__ __launch_bounds__(64 * kSWaves) void gemm_q4_0_small_kernel(const uint8_t* __restrict__ w,
                                                                      const int8_t* __restrict__ codes,
                                                                      const float* __restrict__ records,
                                                                      float* __restrict__ out, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nkb = k >> 5;                       // a multiple of 8
    const int64_t row_bytes = (int64_t)nkb * Q4_0_BPB;
    const int nn = lane & 15, g = lane >> 4;
    uint8_t* ring = smem;
    const uint32_t ring_lds = lds_address(ring);
    const int ntiles = (n + 15) >> 4;
    const int my_tiles = min(kSMaxTiles, (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x);
    const int ngrp = (nkb + kSGroup - 1) / kSGroup;
    const int total = ngrp * my_tiles * kSParts;
    // This wavefront's blocks of group gi, part p: [128 gi + (128 / parts) p + (8 / parts) wave, + 8 / parts) when they
    // exist (K is a multiple of 256, so every run of 8 / parts <= 8 blocks is whole or absent).
    auto first_block = [&](int gi, int p) { return kSGroup * gi + kSItemBlk * p + kSPartBlk * wave; };

    // lhs operands of the wavefront's 8 blocks of the current group (one 16-row lhs tile).  The codes are a lane's own 8
    // bytes per block; the scales and code sums are shared by 16 lanes each, and a vector load costs the compute unit's
    // memory path 64 lanes x its width whatever the lanes ask for, so the 8 records (1 KB) go global -> LDS in one
    // instruction and are read from there.
    u32x2 xa[kSBlk];
    const uint8_t* recs = smem + (kSLds - kSWaves * kSScales) + wave * kSScales;
    const uint32_t recs_lds = lds_address(recs);
    auto load_lhs = [&](int gi) {
#pragma unroll
        for (int j = 0; j < kSBlk; j++) {
            const int kb = min(first_block(gi, j / kSPartBlk) + j % kSPartBlk, nkb - 1);  // (absent: a valid address)
            hidden_load(xa[j], codes + ((int64_t)kb * 64 + lane) * 8);
        }
        // record j of the wavefront (64 bytes) is lanes 4 j .. 4 j + 3 of the load (lanes 0..31)
        const int j = (lane >> 2) & 7;
        const int kb = min(first_block(gi, j / kSPartBlk) + j % kSPartBlk, nkb - 1);
        if (lane < 32) load16_to_lds((const uint8_t*)records + (int64_t)kb * 64 + 16 * (lane & 3), recs_lds);
    };
    long aop[kSBlk];
    q40_half2 dah[kSBlk][2];  // block scales of lhs rows 4 g .. 4 g + 3 (they are fp16 values: the narrowing is exact)
    int4v c8[kSBlk];          // -8 * code sum of those rows
    auto take_lhs = [&]() {
#pragma unroll
        for (int j = 0; j < kSBlk; j++) {
            tie(xa[j]);
            aop[j] = (long)(((uint64_t)xa[j].y << 32) | xa[j].x);
            const uint2 d = *(const uint2*)(recs + 64 * j + 8 * g), c = *(const uint2*)(recs + 64 * j + 32 + 8 * g);
            dah[j][0] = __builtin_bit_cast(q40_half2, d.x);
            dah[j][1] = __builtin_bit_cast(q40_half2, d.y);
            c8[j][0] = (int)(c.x << 16) >> 16;
            c8[j][1] = (int)c.x >> 16;
            c8[j][2] = (int)(c.y << 16) >> 16;
            c8[j][3] = (int)c.y >> 16;
        }
    };

    // this wavefront's row of item (group gi, tile index t, part p) -> ring slot `slot`, row `wave`
    auto issue = [&](int gi, int t, int p, int slot) {
        const int n0 = ((int)blockIdx.x + t * (int)gridDim.x) * 16;
        const int kb = min(kSGroup * gi + kSItemBlk * p, nkb - 8);  // (a part past the end of K: a valid address, not used)
        const int pieces = min(kSItemBlk, nkb - kb) * Q4_0_BPB / 16;  // 9 per 8 blocks
        const uint8_t* src = w + (int64_t)min(n0 + wave, n - 1) * row_bytes + (int64_t)kb * Q4_0_BPB;
        const uint32_t dst = ring_lds + slot * kSSlot + wave * kSRowLds;
#pragma unroll
        for (int i = 0; i < kSLoads; i++) {
            // (lanes past a short last part read its last piece again, into row bytes nobody uses)
            if (i < kSLoads - 1 || lane < kSPieces - 64 * (kSLoads - 1))
                load16_to_lds_once(src + 16 * min(lane + 64 * i, pieces - 1), dst + i * 1024);
        }
    };
    int last_issued = -1, ig = 0, it_t = 0, ip = 0, islot = 0;
    auto issue_next = [&]() {
        issue(ig, it_t, ip, islot);
        last_issued++;
        islot = islot == kSSlots - 1 ? 0 : islot + 1;
        if (++ip == kSParts) {
            ip = 0;
            if (++it_t == my_tiles) { it_t = 0; ig++; }
        }
    };
    // Every wavefront's lhs loads (hits in the L2, 72 KB per workgroup) are in the compute unit's memory path before
    // anybody's weight loads (asking for the first item before them measured 0.1 us slower).
    if (total > 0) {
        load_lhs(0);
        asm volatile("s_barrier" ::: "memory");
        while (last_issued < min(kSAhead - 1, total - 1)) issue_next();
        q40_wait(last_issued + 1);  // the lhs operands; the items issued after them stay in flight
        take_lhs();
    }

    float acc[kSMaxTiles][4];
#pragma unroll
    for (int t = 0; t < kSMaxTiles; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;

    int it = 0, slot = 0;
    for (int grp = 0; grp < ngrp; grp++) {
        if (grp > 0) {
            load_lhs(grp);
            wait_vmcnt<0>();  // (also the items in flight: once per group of 4096 columns)
            take_lhs();
        }
#pragma unroll
        for (int ti = 0; ti < kSMaxTiles; ti++) {
            if (ti >= my_tiles) break;
#pragma unroll
            for (int part = 0; part < kSParts; part++) {
                q40_wait(last_issued - it);  // this wavefront's row of item `it` has landed
                // every row of the item has landed, and everybody has used item it - 1, whose slot the next load overwrites
                asm volatile("s_barrier" ::: "memory");
                while (last_issued < min(it + kSAhead, total - 1)) issue_next();
                const uint32_t* l32 =
                    (const uint32_t*)(ring + slot * kSSlot + nn * kSRowLds + wave * (kSPartBlk * Q4_0_BPB));
                if (first_block(grp, part) < nkb) {
#pragma unroll
                    for (int jj = 0; jj < kSPartBlk; jj++) {
                        // block jj of the wavefront's run at byte 18 jj of it (the run starts on a dword): d, then 16 nibble
                        // bytes; this lane's operand is dword g of them
                        const int j = part * kSPartBlk + jj;
                        const int wi = ((Q4_0_BPB * jj + 2) >> 2) + g;
                        uint32_t raw;
                        if (((Q4_0_BPB * jj + 2) & 3) == 0) raw = l32[wi];
                        else raw = __builtin_amdgcn_alignbyte(l32[wi + 1], l32[wi], 2);
                        const uint32_t lo = raw & 0x0F0F0F0Fu, hi = (raw >> 4) & 0x0F0F0F0Fu;
                        const long bop = (long)(((uint64_t)hi << 32) | lo);
                        const q40_half2 dpair = __builtin_bit_cast(q40_half2, l32[(Q4_0_BPB * jj) >> 2]);
                        const _Float16 dw = ((Q4_0_BPB * jj) & 2) ? dpair.y : dpair.x;
                        const int4v dot = __builtin_amdgcn_mfma_i32_16x16x32_i8(aop[j], bop, c8[j], 0, 0, 0);
                        // (d_w * d_a is exact in fp32; written as a fused multiply-add with 0 so that both fp16 operands
                        // are taken as they are, v_fma_mix_f32)
                        acc[ti][0] = fmaf((float)dot[0], fmaf((float)dw, (float)dah[j][0].x, 0.0f), acc[ti][0]);
                        acc[ti][1] = fmaf((float)dot[1], fmaf((float)dw, (float)dah[j][0].y, 0.0f), acc[ti][1]);
                        acc[ti][2] = fmaf((float)dot[2], fmaf((float)dw, (float)dah[j][1].x, 0.0f), acc[ti][2]);
                        acc[ti][3] = fmaf((float)dot[3], fmaf((float)dw, (float)dah[j][1].y, 0.0f), acc[ti][3]);
                    }
                }
                slot = slot == kSSlots - 1 ? 0 : slot + 1;
                it++;
            }
        }
    }
    // add the 16 K shares: the ring's memory is free once every wavefront has read its last item
    __syncthreads();
    float* sums = (float*)smem;  // [kSWaves][kSMaxTiles][4][64]
#pragma unroll
    for (int t = 0; t < kSMaxTiles; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) sums[((wave * kSMaxTiles + t) * 4 + r) * 64 + lane] = acc[t][r];
    __syncthreads();
    {
        const int t = wave >> 2, r = wave & 3;  // 16 (tile, register) pairs, one per wavefront
        const int col = ((int)blockIdx.x + t * (int)gridDim.x) * 16 + nn, row = 4 * g + r;
        float v = 0.0f;
#pragma unroll
        for (int ww = 0; ww < kSWaves; ww++) v += sums[((ww * kSMaxTiles + t) * 4 + r) * 64 + lane];
        if (t < my_tiles && row < m && col < n) out[(int64_t)row * n + col] = v;
    }
}

// Many lhs rows (prefill).  Same operands and the same staging of the weight rows as gemm_q4_0_kernel, with the
// work cut so that the vector cache is not the bound: the weights are the A operand of the matrix-core
// instruction, so a lane holds the block dots of four weight rows (4 g + r) against ONE lhs row (lane % 16) and
// needs one activation scale and one code sum per instruction (16 bytes per lane with the codes, against 40 the
// other way round); a wavefront owns 32 weight rows for all of K and 8 lhs tiles per pass, so an activation
// operand serves two matrix-core instructions and a weight operand eight; the 8 wavefronts of a workgroup take
// neighbouring weight rows (no sum across wavefronts) and read the same activation operands (vector-cache hits).
// Per (lhs row, weight row, block):  acc += d_w * (float(dot) * d_a - 8 asum d_a)  (convert, two fused
// multiply-adds).
namespace {
constexpr int kWNT = 2;      // 16-row weight tiles per wavefront
constexpr int kWMG = 8;      // 16-row lhs tiles per pass
constexpr int kWWaves = 8;   // wavefronts per workgroup
}  // namespace

__global__ __launch_bounds__(64 * kWWaves) void gemm_q4_0_wide_kernel(const uint8_t* __restrict__ w, const int8_t* __restrict__ codes,
                                                                     const float* __restrict__ dscale, const int32_t* __restrict__ csum,
                                                                     float* __restrict__ out, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nkb = k >> 5;
    const int64_t row_bytes = (int64_t)nkb * Q4_0_BPB;
    const int n0 = ((int)blockIdx.x * kWWaves + wave) * 16 * kWNT;  // first weight row of this wavefront
    if (n0 >= n) return;                                            // (no workgroup-wide barrier below)
    const int tile0 = (int)blockIdx.y * kWMG;
    const int tiles = (m + 15) >> 4;
    const int nn = lane & 15, g = lane >> 4;
    uint8_t* wbuf = smem + wave * (kWNT * kWaveLds);

    float acc[kWNT][kWMG][4];
#pragma unroll
    for (int nt = 0; nt < kWNT; nt++)
#pragma unroll
        for (int t = 0; t < kWMG; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[nt][t][r] = 0.0f;

    // piece p = lane + 64 i of a tile's run: row p / 19, 16-byte piece p % 19 of that row's run
    int prow[5], pidx[5];
#pragma unroll
    for (int i = 0; i < 5; i++) {
        const int p = min(lane + 64 * i, 16 * kRowPieces - 1);
        prow[i] = p / kRowPieces;
        pidx[i] = p - prow[i] * kRowPieces;
    }
    const uint32_t lane8 = 8u * (uint32_t)lane, nn4 = 4u * (uint32_t)nn;
    const uint8_t* my_row[kWNT];  // the row whose codes this lane turns into operands
#pragma unroll
    for (int nt = 0; nt < kWNT; nt++) my_row[nt] = w + (int64_t)min(n0 + 16 * nt + nn, n - 1) * row_bytes;

    for (int kb = 0; kb < nkb; kb += kRun) {
        const int nb = min(kRun, nkb - kb);
        __builtin_amdgcn_wave_barrier();  // the previous run's LDS reads are issued (LDS is in order per wavefront)
#pragma unroll
        for (int nt = 0; nt < kWNT; nt++) {
            uint4 rr[5];
#pragma unroll
            for (int i = 0; i < 5; i++) {
                const uintptr_t ad = (uintptr_t)(w + (int64_t)min(n0 + 16 * nt + prow[i], n - 1) * row_bytes + (int64_t)kb * Q4_0_BPB);
                const int dl = (int)(ad & 15);
                const int last = (dl + nb * Q4_0_BPB + 15) / 16 - 1;
                rr[i] = ((const uint4*)(ad - (uintptr_t)dl))[min(pidx[i], last)];
            }
            uint8_t* dst = wbuf + nt * kWaveLds;
#pragma unroll
            for (int i = 0; i < 4; i++) *(uint4*)(dst + prow[i] * kRowLds + pidx[i] * 16) = rr[i];
            if (lane + 256 < 16 * kRowPieces) *(uint4*)(dst + prow[4] * kRowLds + pidx[4] * 16) = rr[4];
        }
        __builtin_amdgcn_wave_barrier();

        int delta[kWNT];
#pragma unroll
        for (int nt = 0; nt < kWNT; nt++) delta[nt] = (int)((uintptr_t)(my_row[nt] + (int64_t)kb * Q4_0_BPB) & 15);
        for (int b = 0; b < nb; b++) {
            long wop[kWNT];
            float dw4[kWNT][4];
#pragma unroll
            for (int nt = 0; nt < kWNT; nt++) {
                const uint32_t* lds32 = (const uint32_t*)(wbuf + nt * kWaveLds);
                // 8 code bytes of k-group g (low nibbles of bytes 8 (g & 1) .., or their high nibbles)
                const int boff = nn * kRowLds + delta[nt] + Q4_0_BPB * b;
                const int qoff = boff + 2 + 8 * (g & 1);
                const int wi = qoff >> 2;
                const uint32_t sh = (uint32_t)(qoff & 3);
                const uint32_t w0 = lds32[wi], w1 = lds32[wi + 1], w2 = lds32[wi + 2];
                uint32_t lo = __builtin_amdgcn_alignbyte(w1, w0, sh), hi = __builtin_amdgcn_alignbyte(w2, w1, sh);
                if (g & 2) {
                    lo >>= 4;
                    hi >>= 4;
                }
                lo &= 0x0F0F0F0Fu;
                hi &= 0x0F0F0F0Fu;
                wop[nt] = (long)(((uint64_t)hi << 32) | lo);
                const uint32_t dw32 = lds32[boff >> 2] >> (8 * (boff & 3));
                const float dw = h2f((uint16_t)(dw32 & 0xffffu));  // scale of row nn; the lane needs rows 4 g + r
#pragma unroll
                for (int r = 0; r < 4; r++) dw4[nt][r] = __shfl(dw, 4 * g + r, 64);
            }
#pragma unroll
            for (int t = 0; t < kWMG; t++) {
                const int tile = min(tile0 + t, tiles - 1);
                const int64_t tb = (int64_t)tile * nkb + kb + b;
                const long aop = *(const long*)((const char*)(codes + tb * 512) + lane8);
                const float da = *(const float*)((const char*)(dscale + tb * 16) + nn4);
                const float ts = -8.0f * (float)*(const int32_t*)((const char*)(csum + tb * 16) + nn4) * da;
#pragma unroll
                for (int nt = 0; nt < kWNT; nt++) {
                    int4v z = {0, 0, 0, 0};
                    const int4v dot = __builtin_amdgcn_mfma_i32_16x16x32_i8(wop[nt], aop, z, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[nt][t][r] = fmaf(dw4[nt][r], fmaf((float)dot[r], da, ts), acc[nt][t][r]);
                }
            }
        }
    }

    // lane holds out[16 (tile0 + t) + nn][n0 + 16 nt + 4 g + r]
    const bool vec = (n & 3) == 0;
#pragma unroll
    for (int t = 0; t < kWMG; t++) {
        const int row = (tile0 + t) * 16 + nn;
        if (tile0 + t >= tiles || row >= m) continue;
#pragma unroll
        for (int nt = 0; nt < kWNT; nt++) {
            const int col = n0 + 16 * nt + 4 * g;
            float* o = out + (int64_t)row * n + col;
            if (vec && col + 3 < n) {
                *(float4*)o = make_float4(acc[nt][t][0], acc[nt][t][1], acc[nt][t][2], acc[nt][t][3]);
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (col + r < n) o[r] = acc[nt][t][r];
            }
        }
    }
}

int64_t gemm_q4_0_workspace_bytes(int64_t m, int64_t k) { return lhs_q8t(nullptr, m, k).bytes; }

hipError_t launch_gemm_q4_0(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                            float* out, void* workspace, hipStream_t s) {
    const LhsQ8T p = lhs_q8t(workspace, m, k);
    const int64_t tiles = (m + 15) / 16, ngroups = tiles * 16 * (k / 32);
    // Up to 16 lhs rows a pass: the weights are read once per pass and the kernel lives on HBM latency (gemm_q4_0_small_kernel).
    // More rows go in passes of 16 (the plane GEMM takes over where it is faster, see gemm_q4_0_planes_wanted): a pass costs 10.6 /
    // 12.8 / 16.0 us on 4096 x 4096 / 14336 x 4096 / 4096 x 14336, the 17..64-row kernel below 20 / 33 / 57 us up to 32 rows
    // and 49 / 56 / 165 up to 64.
    const bool small = k % 256 == 0 && !kernel_disabled("q4_0_small") && (tiles == 1 || !kernel_disabled("q4_0_small_passes"));
    dim3 qgrid((unsigned)((ngroups * 32 + 255) / 256)), qblock(256);
#define QMM_Q8_OPERAND(T_, W_)                                                                                        \
    quantize_q8_0_operand_kernel<T_, W_><<<qgrid, qblock, 0, s>>>((const T_*)lhs, (int)m, (int)k, ngroups, p.codes, p.scale, p.sum)
    if (lhs_dtype == QMM_F32) {
        if (small) QMM_Q8_OPERAND(float, true);
        else QMM_Q8_OPERAND(float, false);
    } else {
        if (small) QMM_Q8_OPERAND(uint16_t, true);
        else QMM_Q8_OPERAND(uint16_t, false);
    }
#undef QMM_Q8_OPERAND
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (small) {
        static int cus = 0;
        if (!cus) {
            int dev = 0;
            if (hipGetDevice(&dev) != hipSuccess ||
                hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
                cus = 256;
        }
        static bool lds_set = false;
        if (!lds_set) {
            hipError_t e = hipFuncSetAttribute((const void*)gemm_q4_0_small_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kSLds);
            if (e != hipSuccess) return e;
            lds_set = true;
        }
        // tiles are dealt round robin: one workgroup per compute unit until that means more than kSMaxTiles each
        const int64_t ntiles = (n + 15) / 16;
        const int64_t wgs = std::min<int64_t>(ntiles, std::max<int64_t>(cus, (ntiles + kSMaxTiles - 1) / kSMaxTiles));
        const int64_t nkb = k / 32;
        for (int64_t t = 0; t < tiles; t++) {  // (codes 512 bytes, records 64 bytes per lhs tile and block)
            gemm_q4_0_small_kernel<<<dim3((unsigned)wgs), dim3(64 * kSWaves), kSLds, s>>>(
                w, p.codes + t * nkb * 512, (const float*)((const char*)p.scale + t * nkb * 64), out + t * 16 * n,
                (int)std::min<int64_t>(16, m - 16 * t), (int)n, (int)k);
        }
        return hipGetLastError();
    }
    if (tiles > 4 && !kernel_disabled("q4_0_wide")) {
        const size_t wlds = (size_t)kWWaves * kWNT * kWaveLds;
        if (hipError_t e2 = allow_full_lds<gemm_q4_0_wide_kernel>(); e2 != hipSuccess) return e2;
        dim3 grid((unsigned)((n + 16 * kWNT * kWWaves - 1) / (16 * kWNT * kWWaves)), (unsigned)((tiles + kWMG - 1) / kWMG));
        gemm_q4_0_wide_kernel<<<grid, dim3(64 * kWWaves), wlds, s>>>(w, p.codes, p.scale, p.sum, out, (int)m, (int)n, (int)k);
        return hipGetLastError();
    }
    const int nw = (tiles <= 2 && k >= 2048) ? 8 : 4;
    const size_t lds = (size_t)nw * kWaveLds;  // also holds the nw x MG*4 x 64 floats of the final reduction
    dim3 block(64 * nw);
    if (tiles == 1) {
        dim3 grid((unsigned)((n + 15) / 16), 1);
        gemm_q4_0_kernel<1><<<grid, block, lds, s>>>(w, p.codes, p.scale, p.sum, out, (int)m, (int)n, (int)k);
    } else if (tiles == 2) {
        dim3 grid((unsigned)((n + 15) / 16), 1);
        gemm_q4_0_kernel<2><<<grid, block, lds, s>>>(w, p.codes, p.scale, p.sum, out, (int)m, (int)n, (int)k);
    } else {
        dim3 grid((unsigned)((n + 15) / 16), (unsigned)((tiles + 3) / 4));
        gemm_q4_0_kernel<4><<<grid, block, lds, s>>>(w, p.codes, p.scale, p.sum, out, (int)m, (int)n, (int)k);
    }
    return hipGetLastError();
}

}  // namespace qmm
