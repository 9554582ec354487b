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
// Up to 16 lhs rows with K a multiple of 256 take gemm_q4_0_small_kernel instead: the schedule of the
// Q4_K small-batch kernel (gemv_q4k_mm.hip).  A workgroup of 8 wavefronts walks up to 4 tiles of 16
// weight rows; wavefront w owns 8 blocks (144 bytes of every row, 16-byte aligned) of each group of 64
// blocks and keeps the lhs operands of those 8 blocks in registers for all the tiles; the 16 x 144
// bytes of a (group, tile) item go global -> LDS directly into a private 3-slot ring, two items
// ahead.  Inside the 144 bytes the block offsets 18 j are compile-time, so the byte alignment of
// every field is too.
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
template <typename InT>
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
    const int mm = (int)(row & 15), g = l >> 3;
    const int64_t tb = tile * nkb + kb;
    codes[(tb * 64 + g * 16 + mm) * 8 + (l & 7)] = (int8_t)q;
    if (l == 0) {
        dscale[tb * 16 + mm] = h2f(dh);
        csum[tb * 16 + mm] = sum;
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
constexpr int kSWaves = 8;                          // wavefronts per workgroup
constexpr int kSBlk = 8;                            // blocks per wavefront and group: 144 bytes of a row
constexpr int kSRow = kSBlk * Q4_0_BPB;             // 144
constexpr int kSPieces = 16 * kSRow / 16;           // 144 pieces of 16 bytes per item
constexpr int kSLoads = (kSPieces + 63) / 64;       // 3 load instructions per item, the last one by 16 lanes
constexpr int kSSlot = kSPieces * 16 + 16;          // 2320: one dword of read-ahead past the last row
constexpr int kSSlots = 3;
constexpr int kSMaxTiles = 4;
constexpr int kSRing = kSWaves * kSSlots * kSSlot;
constexpr int kSLds = kSRing + kSWaves * kSMaxTiles * 4 * 64 * 4;
}  // namespace

__global__ __launch_bounds__(64 * kSWaves) void gemm_q4_0_small_kernel(const uint8_t* __restrict__ w,
                                                                      const int8_t* __restrict__ codes,
                                                                      const float* __restrict__ dscale,
                                                                      const int32_t* __restrict__ csum,
                                                                      float* __restrict__ out, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nkb = k >> 5;                       // a multiple of 8
    const int64_t row_bytes = (int64_t)nkb * Q4_0_BPB;
    const int nn = lane & 15, g = lane >> 4;
    uint8_t* ring = smem + wave * (kSSlots * kSSlot);
    const uint32_t ring_lds = lds_address(ring);
    float* accs = (float*)(smem + kSRing);        // [kSWaves][kSMaxTiles][4][64]
    const int ntiles = (n + 15) >> 4;
    const int my_tiles = min(kSMaxTiles, (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x);
    const int ngrp = (nkb + kSWaves * kSBlk - 1) / (kSWaves * kSBlk);
    const int total = ngrp * my_tiles;
    // group gi: blocks [64 gi + 8 wave, + 8) when they exist (K is a multiple of 256, so a share is whole or absent)
    auto share = [&](int gi, int& first, bool& have) {
        first = kSWaves * kSBlk * gi + kSBlk * wave;
        have = first < nkb;
        first = min(first, nkb - kSBlk);  // (absent: a valid address, the data is not used)
    };
    int prow[kSLoads], pidx[kSLoads];
#pragma unroll
    for (int i = 0; i < kSLoads; i++) {
        const int p = min(lane + 64 * i, kSPieces - 1);
        prow[i] = p / 9;
        pidx[i] = p - prow[i] * 9;
    }
    auto issue = [&](int gi, int t, int slot) {
        const int n0 = ((int)blockIdx.x + t * (int)gridDim.x) * 16;
        int kb;
        bool have;
        share(gi, kb, have);
        const uint8_t* base = w + (int64_t)kb * Q4_0_BPB;
#pragma unroll
        for (int i = 0; i < kSLoads; i++) {
            const uint8_t* src = base + (int64_t)min(n0 + prow[i], n - 1) * row_bytes + 16 * pidx[i];
            if (i < kSLoads - 1 || lane < kSPieces - 64 * (kSLoads - 1))
                load16_to_lds_once(src, ring_lds + slot * kSSlot + i * 1024);
        }
    };
    int last_issued = -1, ig = 0, it_t = 0, islot = 0;
    auto issue_next = [&]() {
        issue(ig, it_t, islot);
        last_issued++;
        islot = islot == kSSlots - 1 ? 0 : islot + 1;
        if (++it_t == my_tiles) { it_t = 0; ig++; }
    };

    // lhs operands of the wavefront's 8 blocks of the current group
    long aop[kSBlk];
    float4 da[kSBlk], da8[kSBlk];  // block scales of lhs rows 4 g .. 4 g + 3, and -8 * code sum * scale

    int grp = 0, ti = 0, slot = 0;
    for (int it = 0; it < total; it++) {
        int kb0;
        bool have;
        share(grp, kb0, have);
        if (ti == 0) {
            // (ordinary loads: the compiler's waits for them also wait for the items in flight, once per group)
#pragma unroll
            for (int j = 0; j < kSBlk; j++) {
                const int64_t tb = kb0 + j;  // one 16-row lhs tile
                aop[j] = *(const long*)(codes + (tb * 64 + lane) * 8);
                da[j] = *(const float4*)(dscale + tb * 16 + 4 * g);
                const int4v as = *(const int4v*)(csum + tb * 16 + 4 * g);
                da8[j] = make_float4(-8.0f * (float)as[0] * da[j].x, -8.0f * (float)as[1] * da[j].y,
                                     -8.0f * (float)as[2] * da[j].z, -8.0f * (float)as[3] * da[j].w);
            }
        }
        while (last_issued < min(it + 2, total - 1)) issue_next();
        wait_items<kSLoads, 0>(last_issued - it, false);
        const uint8_t* wrow = ring + slot * kSSlot + nn * kSRow;
        const uint32_t* l32 = (const uint32_t*)wrow;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        if (have) {
#pragma unroll
            for (int j = 0; j < kSBlk; j++) {
                // block j at byte 18 j of the row's 144: d, then 16 nibble bytes; this lane's 8 code bytes are the low
                // nibbles of bytes 8 (g & 1) .. + 7 (g < 2) or their high nibbles
                constexpr int kUnused = 0;
                (void)kUnused;
                const int qoff = Q4_0_BPB * j + 2 + 8 * (g & 1);
                const int wi = qoff >> 2;                                  // (18 j + 2) / 4 + 2 (g & 1)
                const uint32_t sh = (uint32_t)((Q4_0_BPB * j + 2) & 3);    // compile-time: 2, 0, 2, 0, ...
                uint32_t lo, hi;
                if (sh == 0) {
                    lo = l32[wi];
                    hi = l32[wi + 1];
                } else {
                    const uint32_t w0 = l32[wi], w1 = l32[wi + 1], w2 = l32[wi + 2];
                    lo = __builtin_amdgcn_alignbyte(w1, w0, sh);
                    hi = __builtin_amdgcn_alignbyte(w2, w1, sh);
                }
                if (g & 2) {
                    lo >>= 4;
                    hi >>= 4;
                }
                lo &= 0x0F0F0F0Fu;
                hi &= 0x0F0F0F0Fu;
                const long bop = (long)(((uint64_t)hi << 32) | lo);
                const uint32_t dwv = l32[(Q4_0_BPB * j) >> 2] >> (8 * ((Q4_0_BPB * j) & 3));
                const float dw = h2f((uint16_t)(dwv & 0xffffu));
                int4v z = {0, 0, 0, 0};
                const int4v dot = __builtin_amdgcn_mfma_i32_16x16x32_i8(aop[j], bop, z, 0, 0, 0);
                // float(dot - 8 asum) * (dw * da), with the -8 asum da part formed once per group
                acc[0] = fmaf(dw, fmaf((float)dot[0], da[j].x, da8[j].x), acc[0]);
                acc[1] = fmaf(dw, fmaf((float)dot[1], da[j].y, da8[j].y), acc[1]);
                acc[2] = fmaf(dw, fmaf((float)dot[2], da[j].z, da8[j].z), acc[2]);
                acc[3] = fmaf(dw, fmaf((float)dot[3], da[j].w, da8[j].w), acc[3]);
            }
        }
        float* mine = accs + ((wave * kSMaxTiles + ti) * 4) * 64 + lane;
#pragma unroll
        for (int r = 0; r < 4; r++) mine[r * 64] = grp == 0 ? acc[r] : mine[r * 64] + acc[r];
        slot = slot == kSSlots - 1 ? 0 : slot + 1;
        if (++ti == my_tiles) { ti = 0; grp++; }
    }
    __syncthreads();
    for (int pr = wave; pr < my_tiles * 4; pr += kSWaves) {
        const int t = pr >> 2, r = pr & 3;
        const int col = ((int)blockIdx.x + t * (int)gridDim.x) * 16 + nn, row = 4 * g + r;
        float v = 0.0f;
#pragma unroll
        for (int ww = 0; ww < kSWaves; ww++) v += accs[((ww * kSMaxTiles + t) * 4 + r) * 64 + lane];
        if (row < m && col < n) out[(int64_t)row * n + col] = v;
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
    dim3 qgrid((unsigned)((ngroups * 32 + 255) / 256)), qblock(256);
    if (lhs_dtype == QMM_F32)
        quantize_q8_0_operand_kernel<float><<<qgrid, qblock, 0, s>>>((const float*)lhs, (int)m, (int)k, ngroups, p.codes,
                                                                     p.scale, p.sum);
    else
        quantize_q8_0_operand_kernel<uint16_t><<<qgrid, qblock, 0, s>>>((const uint16_t*)lhs, (int)m, (int)k, ngroups,
                                                                        p.codes, p.scale, p.sum);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    // Few lhs rows: the weights are read once and the kernel lives on HBM latency, so K is cut eight
    // ways for more wavefronts in flight; otherwise four.
    if (tiles == 1 && k % 256 == 0 && !kernel_disabled("q4_0_small")) {
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
        const int64_t ntiles = (n + 15) / 16;
        const int64_t per_wg = std::min<int64_t>(kSMaxTiles, (ntiles + cus - 1) / cus);
        const int64_t wgs = (ntiles + per_wg - 1) / per_wg;
        gemm_q4_0_small_kernel<<<dim3((unsigned)wgs), dim3(64 * kSWaves), kSLds, s>>>(w, p.codes, p.scale, p.sum, out, (int)m, (int)n,
                                                                                   (int)k);
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
