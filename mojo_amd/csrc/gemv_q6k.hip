// Q6_K decode kernel for m <= 4 lhs rows: weights streamed through LDS, decoded 16 per lane.
//
// A Q6_K super-block is 210 bytes (128 B low nibbles, 64 B high bit pairs, 16 int8 scales, fp16 d),
// so blocks are only 2-byte aligned and no field can be loaded as an aligned vector straight from
// memory.  A wavefront therefore copies a run of up to 16 blocks of its row into a private LDS
// buffer with aligned 16-byte loads (the run starts at the 16-byte boundary below its first byte),
// and the lanes pick their fields out of LDS as two aligned dwords joined by a byte alignment
// (every field sits at a multiple of 4 from its block's start, so one shift per block suffices).
//
// Lane t of a 16-lane group owns, in half h = t / 8 of a block, the four ql bytes 4j..4j+3
// (j = t % 8), the four bytes 32 further and the four qh bytes 4j..4j+3: sixteen weights, four
// each at columns 128h + 4j + {0, 32, 64, 96}, each quartet with its own scale.  Four groups work
// on four blocks at a time.  The -32 offset of the codes is applied through per-16-column sums of
// the activations, computed once per workgroup:  sum_k a_k sc (q_k - 32) = sc (sum a_k q_k) -
// 32 sc asum16, one 16-column group per lane.  Activations come through the vector cache (a
// 16 KB row stays resident), which keeps the LDS pipe for the weights.
//
// The vocabulary projection and other matrices with many rows (K a multiple of 2048, a 16-byte aligned tensor) take
// gemv_q6_k_lanes_kernel instead: a row of 8 n super-blocks is a multiple of 16 bytes, so rows (or, beyond 16
// super-blocks, their 2 or 4 parts, one wavefront each) go global -> LDS directly into a private ring, two ahead; the super-blocks of a row are dealt four to a
// 16-lane group (block = 4 group + round), which makes the 2-byte misalignment of every field a compile-time
// constant per round; a lane keeps the 64 activations of its four blocks in registers for the whole kernel.
#include <stdlib.h>

#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {


namespace {

constexpr int kRunBlocks = 16;                                   // blocks per staged run
constexpr int kRunBytes = (kRunBlocks * Q6_K_BPB + 14 + 4 + 15) / 16 * 16;  // 3392: lead-in + run + one dword of read-ahead, in 16-byte pieces

template <typename AT>
__device__ __forceinline__ float4 load4(const AT* __restrict__ a, int64_t i);
template <>
__device__ __forceinline__ float4 load4<float>(const float* __restrict__ a, int64_t i) {
    return *(const float4*)(a + i);
}
template <>
__device__ __forceinline__ float4 load4<uint16_t>(const uint16_t* __restrict__ a, int64_t i) {
    const uint2 v = *(const uint2*)(a + i);
    return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                       __uint_as_float(v.y & 0xffff0000u));
}

__device__ __forceinline__ float ubf0(uint32_t x) { float r; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float ubf1(uint32_t x) { float r; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float ubf2(uint32_t x) { float r; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float ubf3(uint32_t x) { float r; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(x)); return r; }
__device__ __forceinline__ float dot4u(float4 x, uint32_t q) {
    return fmaf(x.w, ubf3(q), fmaf(x.z, ubf2(q), fmaf(x.y, ubf1(q), x.x * ubf0(q))));
}
// The same dot with the four bytes spread into fp16 lanes first: a byte value q under a zero byte IS the fp16 subnormal
// q * 2^-24, and v_fma_mix_f32 multiplies it with an fp32 operand exactly: two byte permutes and four mixed fused
// multiply-adds instead of four conversions and four multiply-adds.  The result is 2^-24 times dot4u's.
typedef _Float16 q6_half2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot4h(float4 x, uint32_t q) {
    const q6_half2 p01 = __builtin_bit_cast(q6_half2, __builtin_amdgcn_perm(q, q, 0x0c010c00u));
    const q6_half2 p23 = __builtin_bit_cast(q6_half2, __builtin_amdgcn_perm(q, q, 0x0c030c02u));
    float u = fmaf((float)p01.x, x.x, 0.0f);  // (a fused multiply-add with 0: the mixed instruction has no plain multiply)
    u = fmaf((float)p01.y, x.y, u);
    u = fmaf((float)p23.x, x.z, u);
    return fmaf((float)p23.y, x.w, u);
}
__device__ __forceinline__ float sbyte(uint32_t x, int shift) { return (float)((int)(x << (24 - shift)) >> 24); }

}  // namespace

template <int MT, typename AT>
__global__ __launch_bounds__(256) void gemv_q6_k_rows_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                             float* __restrict__ out, int m, int n, int k, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk = k >> 8, ngrp = k >> 4;
    float* asum16 = (float*)smem;  // [MT][k/16]
    uint8_t* wbuf = smem + ((MT * ngrp * 4 + 15) & ~15) + wave * kRunBytes;

    // per-16-column activation sums
    for (int gidx = tid; gidx < MT * ngrp; gidx += 256) {
        const int mi = gidx / ngrp, gi = gidx - mi * ngrp;
        float s = 0.0f;
        if (mi < m) {
            const AT* ar = a + (int64_t)mi * k + gi * 16;
            const float4 x0 = load4(ar, 0), x1 = load4(ar, 4), x2 = load4(ar, 8), x3 = load4(ar, 12);
            s = ((x0.x + x0.y) + (x0.z + x0.w)) + ((x1.x + x1.y) + (x1.z + x1.w)) + ((x2.x + x2.y) + (x2.z + x2.w)) +
                ((x3.x + x3.y) + (x3.z + x3.w));
        }
        asum16[gidx] = s;
    }
    __syncthreads();

    const int total_waves = (int)gridDim.x * 4, gw = (int)blockIdx.x * 4 + wave;
    const int nrun = (nblk + kRunBlocks - 1) / kRunBlocks;
    const int64_t row_bytes = (int64_t)nblk * Q6_K_BPB;
    const int bq = lane >> 4, t = lane & 15, h = t >> 3, j = t & 7;
    const int f_ql = 64 * h + 4 * j, f_qh = 128 + 32 * h + 4 * j, f_sc = 192 + 8 * h;
    const int sc_shift = 8 * (j >> 2);          // this lane's quartet scales: bytes jj, jj + 2 of each scale dword
    const uint32_t* lds32 = (const uint32_t*)wbuf;

    uint4 r0, r1, r2, r3;
    int delta = 0;  // offset of the run's first byte inside its first 16-byte piece
    // aligned 16-byte pieces covering run `c` of row `row`; pieces past the end repeat the last one
    auto issue = [&](int row, int c, int& dl) {
        const int nb = min(kRunBlocks, nblk - c * kRunBlocks);
        const uint8_t* p = w + (int64_t)row * row_bytes + (int64_t)c * kRunBlocks * Q6_K_BPB;
        const uintptr_t ad = (uintptr_t)p;
        dl = (int)(ad & 15);
        const uint4* base = (const uint4*)(ad - (uintptr_t)dl);
        const int last = (dl + nb * Q6_K_BPB + 15) / 16 - 1;
        r0 = base[min(lane, last)];
        r1 = base[min(lane + 64, last)];
        r2 = base[min(lane + 128, last)];
        r3 = base[min(lane + 192, last)];
    };

    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;

    int row = gw, c = 0;
    if (row < n) issue(row, 0, delta);
    while (row < n) {
        // registers -> LDS (the previous run's reads were issued before this point: LDS is in order per wavefront)
        uint4* wb = (uint4*)wbuf;
        wb[lane] = r0;
        wb[lane + 64] = r1;
        wb[lane + 128] = r2;
        if (lane + 192 < kRunBytes / 16) wb[lane + 192] = r3;
        const int cur_delta = delta, cur_c = c, cur_row = row;
        // next run of this row, or the first run of this wavefront's next row
        int nrow = row, nc = c + 1;
        if (nc == nrun) {
            nc = 0;
            nrow = row + total_waves;
        }
        int ndelta = delta;
        issue(min(nrow, n - 1), nrow < n ? nc : 0, ndelta);  // past the end: a harmless repeat, never used
        __builtin_amdgcn_wave_barrier();

        const int nb = min(kRunBlocks, nblk - cur_c * kRunBlocks);
#pragma unroll
        for (int it = 0; it < kRunBlocks / 4; it++) {
            const int bl = 4 * it + bq;
            const bool live = bl < nb;
            const int boff = cur_delta + Q6_K_BPB * min(bl, nb - 1);
            const int sh = boff & 3, w0 = boff >> 2;  // byte shift (0 or 2), first aligned dword
            auto rd = [&](int field) {
                const int i = w0 + (field >> 2);
                return __builtin_amdgcn_alignbyte(lds32[i + 1], lds32[i], (uint32_t)sh);
            };
            const uint32_t A = rd(f_ql), B = rd(f_ql + 32), H = rd(f_qh);
            const uint32_t s0 = rd(f_sc), s1 = rd(f_sc + 4);
            const float d = live ? h2f((uint16_t)(rd(208) & 0xffffu)) : 0.0f;
            const uint32_t q1 = (A & 0x0F0F0F0Fu) | ((H << 4) & 0x30303030u);
            const uint32_t q2 = (B & 0x0F0F0F0Fu) | ((H << 2) & 0x30303030u);
            const uint32_t q3 = ((A >> 4) & 0x0F0F0F0Fu) | (H & 0x30303030u);
            const uint32_t q4 = ((B >> 4) & 0x0F0F0F0Fu) | ((H >> 2) & 0x30303030u);
            const float e1 = d * sbyte(s0, sc_shift), e2 = d * sbyte(s0, sc_shift + 16);
            const float e3 = d * sbyte(s1, sc_shift), e4 = d * sbyte(s1, sc_shift + 16);
            // this lane's 16-column group for the offset term: scale byte t % 8 of half h
            const float eo = -32.0f * d * sbyte(j < 4 ? s0 : s1, 8 * (j & 3));
            const int blk = cur_c * kRunBlocks + min(bl, nb - 1);
            const int kb = blk * 256 + 128 * h + 4 * j;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                if (mi < m) {
                    const AT* ar = a + (int64_t)mi * k + kb;
                    const float4 x1 = load4(ar, 0), x2 = load4(ar, 32), x3 = load4(ar, 64), x4 = load4(ar, 96);
                    float v = acc[mi];
                    v = fmaf(e1, dot4u(x1, q1), v);
                    v = fmaf(e2, dot4u(x2, q2), v);
                    v = fmaf(e3, dot4u(x3, q3), v);
                    v = fmaf(e4, dot4u(x4, q4), v);
                    acc[mi] = fmaf(eo, asum16[mi * ngrp + blk * 16 + t], v);
                }
            }
        }
        if (cur_c == nrun - 1) {
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const float v = wave_sum(acc[mi]);
                if (lane == 0 && mi < m) out[(int64_t)mi * ldo + cur_row] = v;
                acc[mi] = 0.0f;
            }
        }
        __builtin_amdgcn_wave_barrier();
        row = nrow;
        c = nc;
        delta = ndelta;
    }
}


// Variant for one lhs row with the loops interchanged: the run index is the outer loop and the
// wavefront's rows the inner one, so a lane's activations (64 floats per lhs row for its four
// block slots of the run) and offset sums are loaded once per run and stay in registers while
// the weights of all its rows stream through.  Per-row partial sums wait in LDS until the last
// run (one slot per row of the wavefront, kParkRows at most).
constexpr int kParkRows = 128;
constexpr int kLanesSlot = (12 + 16 * Q6_K_BPB + 15) / 16 * 16 + 16;  // 3392: LDS slot of the vocabulary kernel

template <int MT, typename AT>
__global__ __launch_bounds__(256) void gemv_q6_k_slab_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                             float* __restrict__ out, int m, int n, int k, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk = k >> 8;
    uint8_t* wbuf = smem + wave * kRunBytes;
    float* park = (float*)(smem + 4 * kRunBytes) + wave * MT * kParkRows;  // [MT][kParkRows]
    const int total_waves = (int)gridDim.x * 4, gw = (int)blockIdx.x * 4 + wave;
    const int nrows_w = gw < n ? (n - gw + total_waves - 1) / total_waves : 0;
    const int nrun = (nblk + kRunBlocks - 1) / kRunBlocks;
    const int64_t row_bytes = (int64_t)nblk * Q6_K_BPB;
    const int bq = lane >> 4, t = lane & 15, h = t >> 3, j = t & 7;
    const int f_ql = 64 * h + 4 * j, f_qh = 128 + 32 * h + 4 * j, f_sc = 192 + 8 * h;
    const int sc_shift = 8 * (j >> 2);
    const uint32_t* lds32 = (const uint32_t*)wbuf;
    for (int i = lane; i < MT * kParkRows; i += 64) park[i] = 0.0f;

    // two register sets: the loads of rows i + 1 and i + 2 are in flight while row i is decoded
    uint4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3;
    int delta_a = 0, delta_b = 0;
#define QMM_Q6K_ISSUE(SET, ROW, C, DL)                                                               \
    do {                                                                                             \
        const int nb_ = min(kRunBlocks, nblk - (C) * kRunBlocks);                                    \
        const uintptr_t ad_ = (uintptr_t)(w + (int64_t)(ROW) * row_bytes + (int64_t)(C) * kRunBlocks * Q6_K_BPB); \
        DL = (int)(ad_ & 15);                                                                        \
        const uint4* base_ = (const uint4*)(ad_ - (uintptr_t)(DL));                                  \
        const int last_ = ((DL) + nb_ * Q6_K_BPB + 15) / 16 - 1;                                     \
        SET##0 = base_[min(lane, last_)];                                                            \
        SET##1 = base_[min(lane + 64, last_)];                                                       \
        SET##2 = base_[min(lane + 128, last_)];                                                      \
        SET##3 = base_[min(lane + 192, last_)];                                                      \
    } while (0)
#define QMM_Q6K_STAGE(SET)                                              \
    do {                                                                \
        uint4* wb_ = (uint4*)wbuf;                                      \
        wb_[lane] = SET##0;                                             \
        wb_[lane + 64] = SET##1;                                        \
        wb_[lane + 128] = SET##2;                                       \
        if (lane + 192 < kRunBytes / 16) wb_[lane + 192] = SET##3;      \
    } while (0)

    for (int c = 0; c < nrun; c++) {
        const int nb = min(kRunBlocks, nblk - c * kRunBlocks);
        // this lane's activations for the run: per block slot, four quartets; and its offset sums
        float4 x[MT][4][4];
        float os[MT][4], lv[4];
        int boff0[4];
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int bl = 4 * it + bq;
            lv[it] = bl < nb ? 1.0f : 0.0f;
            const int blc = min(bl, nb - 1);
            boff0[it] = Q6_K_BPB * blc;
            const int blk = c * kRunBlocks + blc;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                if (mi < m) {
                    const AT* ar = a + (int64_t)mi * k + blk * 256;
                    const AT* aq = ar + 128 * h + 4 * j;
                    x[mi][it][0] = load4(aq, 0);
                    x[mi][it][1] = load4(aq, 32);
                    x[mi][it][2] = load4(aq, 64);
                    x[mi][it][3] = load4(aq, 96);
                    const AT* ag = ar + 16 * t;
                    const float4 y0 = load4(ag, 0), y1 = load4(ag, 4), y2 = load4(ag, 8), y3 = load4(ag, 12);
                    os[mi][it] = -32.0f * (((y0.x + y0.y) + (y0.z + y0.w)) + ((y1.x + y1.y) + (y1.z + y1.w)) +
                                           ((y2.x + y2.y) + (y2.z + y2.w)) + ((y3.x + y3.y) + (y3.z + y3.w)));
                } else {
                    x[mi][it][0] = x[mi][it][1] = x[mi][it][2] = x[mi][it][3] = make_float4(0.f, 0.f, 0.f, 0.f);
                    os[mi][it] = 0.0f;
                }
            }
        }
        auto row_of = [&](int i) { return min(gw + i * total_waves, n - 1); };  // past the last row: a harmless repeat
        auto decode_row = [&](int i, int cur_delta) {
            float v[MT];
#pragma unroll
            for (int mi = 0; mi < MT; mi++) v[mi] = 0.0f;
#pragma unroll
            for (int it = 0; it < 4; it++) {
                const int boff = cur_delta + boff0[it];
                const int sh = boff & 3, w0 = boff >> 2;
                auto rd = [&](int field) {
                    const int q = w0 + (field >> 2);
                    return __builtin_amdgcn_alignbyte(lds32[q + 1], lds32[q], (uint32_t)sh);
                };
                const uint32_t A = rd(f_ql), B = rd(f_ql + 32), H = rd(f_qh);
                const uint32_t s0 = rd(f_sc), s1 = rd(f_sc + 4);
                const float d = h2f((uint16_t)(rd(208) & 0xffffu)) * lv[it];
                const uint32_t q1 = (A & 0x0F0F0F0Fu) | ((H << 4) & 0x30303030u);
                const uint32_t q2 = (B & 0x0F0F0F0Fu) | ((H << 2) & 0x30303030u);
                const uint32_t q3 = ((A >> 4) & 0x0F0F0F0Fu) | (H & 0x30303030u);
                const uint32_t q4 = ((B >> 4) & 0x0F0F0F0Fu) | ((H >> 2) & 0x30303030u);
                const float e1 = d * sbyte(s0, sc_shift), e2 = d * sbyte(s0, sc_shift + 16);
                const float e3 = d * sbyte(s1, sc_shift), e4 = d * sbyte(s1, sc_shift + 16);
                const float eo = d * sbyte(j < 4 ? s0 : s1, 8 * (j & 3));
#pragma unroll
                for (int mi = 0; mi < MT; mi++) {
                    float u = v[mi];
                    u = fmaf(e1, dot4u(x[mi][it][0], q1), u);
                    u = fmaf(e2, dot4u(x[mi][it][1], q2), u);
                    u = fmaf(e3, dot4u(x[mi][it][2], q3), u);
                    u = fmaf(e4, dot4u(x[mi][it][3], q4), u);
                    v[mi] = fmaf(eo, os[mi][it], u);
                }
            }
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const float sum = wave_sum(v[mi]);
                if (lane == 0) park[mi * kParkRows + i] += sum;
            }
        };
        if (nrows_w > 0) {
            QMM_Q6K_ISSUE(ra, row_of(0), c, delta_a);
            QMM_Q6K_ISSUE(rb, row_of(1), c, delta_b);
        }
        for (int i = 0; i < nrows_w; i += 2) {
            QMM_Q6K_STAGE(ra);
            const int da = delta_a;
            QMM_Q6K_ISSUE(ra, row_of(i + 2), c, delta_a);
            __builtin_amdgcn_wave_barrier();
            decode_row(i, da);
            __builtin_amdgcn_wave_barrier();
            if (i + 1 < nrows_w) {
                QMM_Q6K_STAGE(rb);
                const int db = delta_b;
                QMM_Q6K_ISSUE(rb, row_of(i + 3), c, delta_b);
                __builtin_amdgcn_wave_barrier();
                decode_row(i + 1, db);
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
#undef QMM_Q6K_ISSUE
#undef QMM_Q6K_STAGE
    __builtin_amdgcn_wave_barrier();
    for (int i = lane; i < nrows_w; i += 64) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++)
            if (mi < m) out[(int64_t)mi * ldo + gw + (int64_t)i * total_waves] = park[mi * kParkRows + i];
    }
}

// LDS bytes of one workgroup; 0 if the shape does not fit (the caller then uses the generic kernel).
static size_t q6k_rows_lds(int mt, int64_t k) {
    const size_t b = ((size_t)mt * (k / 16) * 4 + 15) / 16 * 16 + 4 * (size_t)kRunBytes;
    return b <= 96 * 1024 ? b : 0;
}

// One lhs row, rows of 8 or 16 super-blocks (K = 2048 or 4096: then every row is 16-byte aligned): the
// decode of the slab kernel above with the alignment worked out at compile time and the rows delivered
// global -> LDS directly.  Group bq = lane / 16 takes super-blocks 4 bq + it, it = 0..3, so a super-block
// starts at 840 bq + 210 it bytes of the row: 4-byte aligned for even `it` (fields are plain dword reads),
// 2 bytes off for odd `it` (two dwords joined at a fixed byte offset).  A wavefront walks its rows
// (persistent) with a private ring of three LDS slots, two rows in flight (global_load_lds_dwordx4, hidden
// from the compiler, exact vmcnt waits: lds_stream.h); no registers are spent on staging.
// L: load instructions per row (64 pieces of 16 bytes each): 4 for 16 super-blocks, 2 for 8.
// MT: lhs rows (1 or 2; the decode of a weight row is shared, the activations of both rows stay in registers).
template <int MT, int L, typename AT>
__global__ __launch_bounds__(256) void gemv_q6_k_lanes_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                              float* __restrict__ out, int n, int k, int ring_slots,
                                                              int64_t ldo, int wpr, int bpw) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk = k >> 8;                       // a multiple of 8: rows are whole 16-byte pieces
    const int64_t row_bytes = (int64_t)nblk * Q6_K_BPB;
    // Rows longer than 16 super-blocks are cut into wpr (2 or 4) parts of bpw (even) super-blocks, one wavefront
    // each; a part starts 4, 8 or 12 bytes after a 16-byte boundary at most (bpw * 210 is a multiple of 4), so the
    // pieces are taken from the boundary below it and every field keeps its dword parity.
    const int part = wave % wpr, blk0 = part * bpw;
    const int nbp = max(0, min(bpw, nblk - blk0));                    // super-blocks of this part
    const int lead = (blk0 * Q6_K_BPB) & 15;                          // bytes before the part in its first piece
    const int pieces = (12 + bpw * Q6_K_BPB + 15) / 16;               // per slot: the longest lead-in and a full part
    const int last_piece = (lead + max(nbp, 1) * Q6_K_BPB + 15) / 16 - 1;  // of this part (nothing past it is read)
    const int kSlot = kLanesSlot;                  // room for 16 super-blocks whatever bpw is: lanes of a last,
                                                   // partial group of four read (and discard) what lies behind the part
    uint8_t* ring = smem + wave * (ring_slots * kSlot);
    const uint32_t ring_lds = lds_address(ring);
    float* park = (float*)(smem + 4 * ring_slots * kSlot) + wave * MT * kParkRows;  // [row][MT]
    const int spw = 4 / wpr;                                          // row streams per workgroup
    const int total_waves = (int)gridDim.x * spw, gw = (int)blockIdx.x * spw + wave / wpr;
    const int my_rows = gw < n ? (n - gw + total_waves - 1) / total_waves : 0;
    const int bq = lane >> 4, t = lane & 15, h = t >> 3, j = t & 7;
    const int sc_shift = 8 * (j >> 2);

    // the first rows are requested before the activations, so that their latencies overlap
    // (the mask follows the slot size, the same for every part, so each of the L instructions has a live lane in
    // every wavefront and the wait counts stay exact; a shorter part repeats its last piece)
    auto issue = [&](int ri, int slot) {
        const uint8_t* base = w + (int64_t)(gw + (int64_t)ri * total_waves) * row_bytes + (int64_t)blk0 * Q6_K_BPB - lead;
#pragma unroll
        for (int i = 0; i < L; i++)
            if (lane + 64 * i < pieces)
                load16_to_lds_once(base + 16 * min(lane + 64 * i, last_piece), ring_lds + slot * kSlot + i * 1024);
    };
    int issued = 0, islot = 0, cslot = 0;
    for (; issued < min(ring_slots - 1, my_rows); issued++) {
        issue(issued, islot);
        islot = islot + 1 == ring_slots ? 0 : islot + 1;
    }
    // this lane's activations: per super-block slot `it`, four quartets at columns 128 h + 4 j + {0, 32, 64, 96};
    // and -32 times the sum of one 16-column group per lane (group t of the super-block)
    float4 x[MT][4][4];
    float os[MT][4];
    bool lv[4];  // the lane's super-block `it` exists in this part
    float keep = 0.0f;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int bl = 4 * bq + it;                 // super-block of the part
        lv[it] = bl < nbp;
        const int blc = min(blk0 + bl, nblk - 1);   // of the row
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const AT* ar = a + (int64_t)mi * k + blc * 256;
            const AT* aq = ar + 128 * h + 4 * j;
            x[mi][it][0] = load4(aq, 0);
            x[mi][it][1] = load4(aq, 32);
            x[mi][it][2] = load4(aq, 64);
            x[mi][it][3] = load4(aq, 96);
            // The sum of group t = 8 h + j (columns 128 h + 16 j .. + 15) from the quartets already loaded, not from loads of its
            // own (a wavefront's lhs loads are half of its start-up: 32 KB through the compute unit's load path for 16 KB of
            // values): those 16 columns are quartet j / 2 of the four lanes 4 (j % 2) .. + 3 of this half row.  Quartet sums,
            // added over each aligned group of four lanes; the other group of the eight is a mirror away.
            float qs[4], qo[4];
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++) {
                const float4 q = x[mi][it][c4];
                qs[c4] = (q.x + q.y) + (q.z + q.w);
                qs[c4] += dpp_move<0xB1>(qs[c4]);
                qs[c4] += dpp_move<0x4E>(qs[c4]);
                qo[c4] = dpp_move<0x141>(qs[c4]);
            }
            const int cj = j >> 1;
            const float mine = cj == 0 ? qs[0] : cj == 1 ? qs[1] : cj == 2 ? qs[2] : qs[3];
            const float othr = cj == 0 ? qo[0] : cj == 1 ? qo[1] : cj == 2 ? qo[2] : qo[3];
            // (in units of 2^-24 like the dots below: -32 * 2^-24 = -2^-19; the row's sum is scaled back at its end)
            os[mi][it] = -0x1p-19f * ((j & 1) == (j >> 2) ? mine : othr);
            keep += os[mi][it];
        }
    }
    // (ordinary loads, younger than the rows requested above: the wait for them also covers those rows, and it
    // is forced here, before the loop, so that no wait of the compiler's lands between the counted ones)
    asm volatile("" : "+v"(keep));

    // dword offsets of this lane's fields inside a super-block
    const int o_ql = 16 * h + j, o_qh = 32 + 8 * h + j, o_sc = 48 + 2 * h;
    for (int ri = 0; ri < my_rows; ri++) {
        if (issued < my_rows) {
            issue(issued, islot);
            islot = islot + 1 == ring_slots ? 0 : islot + 1;
            issued++;
        }
        wait_items<L, 0>(issued - 1 - ri, false);
        // super-block 4 bq of the part: byte lead + 840 bq (groups past the part read its last group again; discarded)
        const uint32_t* l32 = (const uint32_t*)(ring + cslot * kSlot) + (lead >> 2) + 210 * min(bq, (max(nbp, 1) - 1) / 4);
        cslot = cslot + 1 == ring_slots ? 0 : cslot + 1;
        float v[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) v[mi] = 0.0f;
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int q0 = (Q6_K_BPB * it) >> 2;              // dword of the super-block's first (aligned) byte
            const bool odd = ((Q6_K_BPB * it) & 3) != 0;      // compile-time: it = 1, 3 start 2 bytes into that dword
            auto rd = [&](int dw) {
                return odd ? __builtin_amdgcn_alignbyte(l32[q0 + dw + 1], l32[q0 + dw], 2u) : l32[q0 + dw];
            };
            const uint32_t A = rd(o_ql), B = rd(o_ql + 8), H = rd(o_qh);
            const uint32_t s0 = rd(o_sc), s1 = rd(o_sc + 1);
            const uint32_t dv = odd ? l32[q0 + 52] >> 16 : l32[q0 + 52] & 0xffffu;
            const float d = h2f((uint16_t)dv);
            const uint32_t q1 = (A & 0x0F0F0F0Fu) | ((H << 4) & 0x30303030u);
            const uint32_t q2 = (B & 0x0F0F0F0Fu) | ((H << 2) & 0x30303030u);
            const uint32_t q3 = ((A >> 4) & 0x0F0F0F0Fu) | (H & 0x30303030u);
            const uint32_t q4 = ((B >> 4) & 0x0F0F0F0Fu) | ((H >> 2) & 0x30303030u);
            // the int8 scales of the four quartets and of this lane's 16-column group; d once at the end
            // (one shift per dword, then sign-extending byte selects: a conversion instruction each)
            const uint32_t t0 = s0 >> sc_shift, t1 = s1 >> sc_shift, tg = (j < 4 ? s0 : s1) >> (8 * (j & 3));
            const float c1 = (float)(signed char)(t0 & 0xffu), c2 = (float)(signed char)((t0 >> 16) & 0xffu);
            const float c3 = (float)(signed char)(t1 & 0xffu), c4 = (float)(signed char)((t1 >> 16) & 0xffu);
            const float cg = (float)(signed char)(tg & 0xffu);
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                float u = c1 * dot4h(x[mi][it][0], q1);
                u = fmaf(c2, dot4h(x[mi][it][1], q2), u);
                u = fmaf(c3, dot4h(x[mi][it][2], q3), u);
                u = fmaf(c4, dot4h(x[mi][it][3], q4), u);
                u = fmaf(cg, os[mi][it], u);
                v[mi] = lv[it] ? fmaf(d, u, v[mi]) : v[mi];  // (a select: what a missing super-block's lanes read is arbitrary)
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const float sum = wave_sum_dpp_lane63(v[mi]);
            if (lane == 63) park[ri * MT + mi] = sum * 0x1p24f;
        }
    }
    if (wpr > 1) __syncthreads();  // (every wavefront gets here: no early exit above)
    else __builtin_amdgcn_wave_barrier();
    if (part == 0) {
        for (int i = lane; i < my_rows * MT; i += 64) {
            const int r = i / MT, mi = i - r * MT;
            float v = park[i];
            for (int q = 1; q < wpr; q++) v += park[q * MT * kParkRows + i];  // the other parts of the row
            out[(int64_t)mi * ldo + gw + (int64_t)r * total_waves] = v;
        }
    }
}

hipError_t launch_gemv_q6_k_rows(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                                 float* out, int64_t ldo, hipStream_t s, bool* handled) {
    *handled = false;
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    if (m < 1 || m > 16 || ((uintptr_t)w & 1)) return hipSuccess;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    const int pc_env = 0, pc = 3;  // (workgroups per compute unit of the kernels below the vocabulary one)
    const bool lanes_off = kernel_disabled("q6k_lanes");
    // Rows of whole 16-byte pieces (K a multiple of 2048, up to 16384) and enough of them: the kernel with the rows
    // global -> LDS and the activations in registers, one or two lhs rows per pass over the weights (up to 16 rows:
    // passes of two).  Rows longer than 16 super-blocks are cut into 2 or 4 parts, one wavefront each.
    const int nblk = (int)(k / 256);
    const int wpr = nblk <= 16 ? 1 : nblk <= 32 ? 2 : 4;
    const int64_t need_parts = (int64_t)cus * 4 * 8;  // below 8 row parts per wavefront of a one-workgroup-per-CU grid the row-at-a-time kernel is faster
    if (k % 2048 == 0 && nblk <= 64 && !((uintptr_t)w & 15) && n * wpr >= need_parts && !lanes_off) {
        // Ring slots and workgroups per compute unit, 128256 x 4096 with one lhs row (us): 3 / 3: 77.9, 2 / 3: 77.8, 2 / 4: 76.9,
        // 3 / 2: 81.9, 4 / 2: 81.5: the wavefronts per SIMD count (the decode of a row is a chain of LDS reads), a second row
        // in flight does not.
        const int ring = m == 1 ? 2 : 3, pc = m == 1 ? 4 : 3;
        const int bpw = nblk / wpr;                                  // 8 .. 16, even
        const int pieces = (12 + bpw * Q6_K_BPB + 15) / 16;
        const int l = (pieces + 63) / 64;                            // 2 .. 4 load instructions per row part
        const int spw = 4 / wpr;
        const int64_t esz = a_dtype == QMM_F32 ? 4 : 2;
        for (int m0 = 0; m0 < m; m0 += 2) {
            const int rows = min(2, m - m0);
            const int pcl = rows == 1 ? pc : min(pc, 2);  // two lhs rows: twice the registers, two wavefronts per SIMD
            const size_t lds3 = 4 * ring * (size_t)kLanesSlot + 4 * (size_t)rows * kParkRows * 4;
            const int64_t wgs = max((int64_t)cus * pcl, (n + (int64_t)spw * kParkRows - 1) / ((int64_t)spw * kParkRows));
            dim3 grid3((unsigned)min(wgs, (n + spw - 1) / spw)), block3(256);
            const void* am = (const char*)a + (int64_t)m0 * k * esz;
            float* om = out + (int64_t)m0 * ldo;
#define QMM_Q6K_LANES(MT_, L_)                                                                                        \
    do {                                                                                                              \
        if (a_dtype == QMM_F32)                                                                                       \
            gemv_q6_k_lanes_kernel<MT_, L_, float><<<grid3, block3, lds3, s>>>(w, (const float*)am, om, (int)n, (int)k, ring, ldo, wpr, bpw); \
        else                                                                                                          \
            gemv_q6_k_lanes_kernel<MT_, L_, uint16_t><<<grid3, block3, lds3, s>>>(w, (const uint16_t*)am, om, (int)n, (int)k, ring, ldo, wpr, bpw); \
    } while (0)
#define QMM_Q6K_LANES_L(MT_)               \
    do {                                   \
        if (l == 2) QMM_Q6K_LANES(MT_, 2); \
        else if (l == 3) QMM_Q6K_LANES(MT_, 3); \
        else QMM_Q6K_LANES(MT_, 4);        \
    } while (0)
            if (rows == 1) QMM_Q6K_LANES_L(1);
            else QMM_Q6K_LANES_L(2);
#undef QMM_Q6K_LANES_L
#undef QMM_Q6K_LANES
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
        }
        *handled = true;
        return hipSuccess;
    }
    if (m > 4) return hipSuccess;
    if (mt == 1 && n >= (int64_t)cus * pc * 4 * 4 && !kernel_disabled("q6k_slab")) {
        const size_t lds2 = 4 * (size_t)kRunBytes + 4 * (size_t)kParkRows * 4;
        // enough wavefronts that none has more rows than its LDS parking slots
        const int64_t wgs = max((int64_t)cus * pc, (n + 4 * kParkRows - 1) / (4 * kParkRows));
        dim3 grid2((unsigned)min(wgs, (n + 3) / 4)), block2(256);
        if (a_dtype == QMM_F32)
            gemv_q6_k_slab_kernel<1, float><<<grid2, block2, lds2, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo);
        else
            gemv_q6_k_slab_kernel<1, uint16_t><<<grid2, block2, lds2, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo);
        *handled = true;
        return hipGetLastError();
    }
    const size_t lds = q6k_rows_lds(mt, k);
    if (!lds) return hipSuccess;
    int per_cu = pc_env > 0 ? pc_env : (int)min((size_t)4, (size_t)(128 * 1024) / lds);
    per_cu = max(per_cu, 1);
    const int64_t wg_needed = (n + 3) / 4;
    dim3 grid((unsigned)min((int64_t)cus * per_cu, wg_needed)), block(256);
#define QMM_Q6K_GO(MT_)                                                                                              \
    do {                                                                                                             \
        if (a_dtype == QMM_F32) {                                                                                    \
            if (lds > 64 * 1024) (void)allow_full_lds<gemv_q6_k_rows_kernel<MT_, float>>();                          \
            gemv_q6_k_rows_kernel<MT_, float><<<grid, block, lds, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo); \
        } else {                                                                                                     \
            if (lds > 64 * 1024) (void)allow_full_lds<gemv_q6_k_rows_kernel<MT_, uint16_t>>();                       \
            gemv_q6_k_rows_kernel<MT_, uint16_t><<<grid, block, lds, s>>>(w, (const uint16_t*)a, out, m, (int)n,     \
                                                                         (int)k, ldo);                               \
        }                                                                                                            \
    } while (0)
    if (mt == 1) QMM_Q6K_GO(1);
    else if (mt == 2) QMM_Q6K_GO(2);
    else QMM_Q6K_GO(4);
#undef QMM_Q6K_GO
    *handled = true;
    return hipGetLastError();
}

}  // namespace qmm
