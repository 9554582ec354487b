// Q5_K with up to 16 lhs rows a pass on the matrix cores, K a multiple of 512: the small-batch kernel of Q6_K
// (gemv_q6k_mm.hip: persistent workgroups over 16-row tiles, a wavefront owns two super-blocks of every row and keeps the
// lhs operands of its 512 columns in registers, rows global -> LDS directly into a private ring, partial tiles added
// through LDS) with Q5_K's arithmetic.
//
// A Q5_K weight is d * sc_j * q - dmin * m_j with q = nibble | fifth bit << 4 in 0..31 and a 6-bit scale and min per
// 32-weight sub-block j.  The matrix-core operand of a weight is q as fp16: a byte permute interleaves the nibble bytes
// with bytes that hold the fifth bit under 0x54, which reads as 0x5400 + (q << 4) = 64 + q, and a packed subtraction of
// 64 (exact) leaves q.  One v_mfma_f32_16x16x32_f16 per sub-block gives P = sum x * q for 16 weight rows at once
// (products exact, fp32 sums; hi parts and residuals of the lhs in operand rows 0..7 and 8..15); u += sc_j * P in the
// lanes.  The min term of a super-block is one more instruction: (sub-block sums of the lhs, hi and residual) x (the eight
// m_j as fp16 integers); acc += d * u - dmin * that.
//
// A super-block is 176 bytes = 11 pieces of 16, so a wavefront's 352 bytes of a row start on a 16-byte boundary and every
// field is dword-aligned; the rows sit 368 bytes apart in LDS (one padding piece, a repeat of the last), which spreads the
// 16 rows of a tile over all banks.
#include <stdlib.h>

#include <algorithm>

#include "lds_stream.h"
#include "qmm_device.h"
#include "qmm_internal.h"

namespace qmm {

typedef _Float16 v_half4 __attribute__((ext_vector_type(4)));
typedef _Float16 v_half8 __attribute__((ext_vector_type(8)));
typedef float v_float4 __attribute__((ext_vector_type(4)));
typedef __fp16 v_fp16x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int kVWaves = 8;
constexpr int kVRowPieces = 23;                 // 22 pieces of data and one of padding
constexpr int kVRowLds = kVRowPieces * 16;      // 368
constexpr int kVPieces = 16 * kVRowPieces;      // 368 pieces per item
constexpr int kVLoads = (kVPieces + 63) / 64;   // 6 load instructions, the last one by 48 lanes
constexpr int kVSlot = kVLoads * 1024;
constexpr int kVSlots = 2;
constexpr int kVRing = kVWaves * kVSlots * kVSlot;
constexpr int kVRed = 2 * kVWaves * 2 * 1024;   // two buffers of two 16 x 16 partial results (4 floats a lane each) per wavefront
constexpr int kVInv = kVWaves * 16 * 4;         // inverse lhs scales: 16 lhs rows per wavefront
constexpr int kVLds = kVRing + kVRed + kVInv;
static_assert(kVLds <= kLdsPerCu, "Q5_K small-batch kernel LDS");
static_assert((16 * 16 * 4) * 4 <= kVSlot, "the staged sub-block sums fit a ring slot");

__device__ __forceinline__ v_half4 v_as_half4(uint32_t lo, uint32_t hi) {
    const uint2 v = make_uint2(lo, hi);
    return __builtin_bit_cast(v_half4, v);
}
__device__ __forceinline__ uint32_t v_pkrtz(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}

template <typename AT>
__device__ __forceinline__ float4 v_lhs4(const AT* __restrict__ a);
template <>
__device__ __forceinline__ float4 v_lhs4<float>(const float* __restrict__ a) {
    return *(const float4*)a;
}
template <>
__device__ __forceinline__ float4 v_lhs4<uint16_t>(const uint16_t* __restrict__ a) {
    const uint2 v = *(const uint2*)a;
    return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                       __uint_as_float(v.y & 0xffff0000u));
}

// 16 bytes per lane, non-temporal, global (uniform base + lane offset) -> LDS at lds_base + 16 * lane
__device__ __forceinline__ void v_stream16_to_lds(uint32_t lane_offset, const void* uniform_base, uint32_t lds_base) {
    uint32_t keep;
    const uint64_t b = (uint64_t)(uintptr_t)uniform_base;
    const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) |
                        (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(lane_offset), "s"(sb), "s"(lds_base)
                 : "memory");
}

}  // namespace

// MROWS: lhs rows of the pass, 2, 4, 8 or 16 (>= m; rows past m are zero operands and their results are dropped).  Sixteen
// bf16 rows need no residual rows and are one set (sixteen fp32 rows would be two sets of eight, each with its own operands
// and sums; the launcher does not use that: it spills).  A lane holds rows 4 (lane / 16) + r of a set; accumulator registers
// that hold no wanted lhs row are not computed.
// ROUNDS: K other than 4096 in rounds of 16 super-blocks; 0: a single whole round, everything about rounds is constant; 1: the
// workgroup walks the rounds one after the other and adds to its own output; 2: round blockIdx.y only, its result stored as
// part blockIdx.y of [rounds][m][ldo] at `out` (the caller adds the parts in round order).
template <int MROWS, typename AT, int ROUNDS>
__global__ __launch_bounds__(64 * kVWaves) void gemv_q5_k_mm_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                                   float* __restrict__ out, int m, int n, int k, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nn = lane & 15, kg = lane >> 4;
    constexpr bool HI16 = MROWS == 16 && sizeof(AT) == 2;
    constexpr int SETS = MROWS > 8 && !HI16 ? 2 : 1, MR1 = MROWS > 8 ? 8 : MROWS;  // sets of lhs rows, rows of a set
    constexpr int RN = MR1 < 4 ? MR1 : 4;  // accumulator registers in use per set
    const int nblk = k >> 8;  // even
    const int64_t row_bytes = (int64_t)nblk * Q5_K_BPB;
    uint8_t* ring = smem + wave * (kVSlots * kVSlot);
    const uint32_t ring_lds = lds_address(ring);
    float* red = (float*)(smem + kVRing);  // [2][kVWaves][2 sets][4][64]
    const int ntiles = (n + 15) >> 4;
    const int my_tiles = (int)blockIdx.x < ntiles ? (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;

    // piece p = lane + 64 i of an item: row p / 23, piece min(p % 23, 21) of the wavefront's 352 bytes of the row
    uint32_t full[kVLoads];  // byte offset of the piece in a tile that lies inside the matrix
#pragma unroll
    for (int i = 0; i < kVLoads; i++) {
        const int p = min(lane + 64 * i, kVPieces - 1), pr = p / kVRowPieces;
        full[i] = (uint32_t)pr * (uint32_t)row_bytes + (uint32_t)(min(p - pr * kVRowPieces, kVRowPieces - 2) * 16);
    }
    auto issue = [&](int round, int ti, int slot) {
        const int n0 = ((int)blockIdx.x + ti * (int)gridDim.x) * 16;
        const uint8_t* base = w + (int64_t)n0 * row_bytes + (16 * round + 2 * wave) * Q5_K_BPB;
        const int last = n - 1 - n0;  // rows past the matrix repeat its last row (their results are dropped)
#pragma unroll
        for (int i = 0; i < kVLoads; i++) {
            uint32_t off = full[i];
            if (last < 15) {  // (the last tile of a ragged matrix only)
                const uint32_t pr = off / (uint32_t)row_bytes;
                off -= (pr - (uint32_t)min((int)pr, last)) * (uint32_t)row_bytes;
            }
            if (i < kVLoads - 1 || lane < kVPieces - 64 * (kVLoads - 1)) v_stream16_to_lds(off, base, ring_lds + slot * kVSlot + i * 1024);
        }
    };
    // (constants of the unpack in vector registers: an and-or in one instruction takes no literal and one scalar at most)
    uint32_t m01 = 0x01010101u, c54 = 0x54545454u;
    asm volatile("" : "+v"(m01), "+v"(c54));
    const v_float4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const v_half8 off64 = {(_Float16)64.0f, (_Float16)64.0f, (_Float16)64.0f, (_Float16)64.0f,
                           (_Float16)64.0f, (_Float16)64.0f, (_Float16)64.0f, (_Float16)64.0f};
    float* stg = (float*)(smem + kVRing + kVRed) + 16 * wave;  // this wavefront's inverse lhs scales
    float* sums = (float*)(ring + kVSlot);                     // staged sub-block sums: the second ring slot, free in the prologue
    int it = 0;  // tiles done, over all rounds: its parity picks the buffer of the partial results

    const int rounds = ROUNDS ? (nblk + 15) >> 4 : 1;
    const int round0 = ROUNDS == 2 ? (int)blockIdx.y : 0, round1 = ROUNDS == 2 ? round0 + 1 : rounds;
    for (int round = round0; round < round1; round++) {
    const bool have = ROUNDS ? 16 * round + 2 * wave < nblk : true;            // this wavefront has super-blocks in the round
    const int nw = ROUNDS ? min(kVWaves, (nblk - 16 * round) >> 1) : kVWaves;  // wavefronts that have
    if (have && my_tiles > 0) issue(round, 0, 0);

    // ---- the lhs operands of this wavefront's 512 columns.  Operand row nn of set st: lhs row 8 st + nn % 8, hi part (nn < 8)
    // or residual (sixteen bf16 rows: lhs row nn, hi part).  Per sub-block of 32 columns a lane holds columns 8 kg .. 8 kg + 7.
    v_half8 fa[SETS][2][8];
    v_half4 fo[SETS][2], fo2[2];  // (fo2: the residuals of the sums where all sixteen operand rows are hi parts)
#pragma unroll
    for (int st = 0; st < SETS; st++) {
        const int lrow = HI16 ? nn : 8 * st + (nn & 7);
        const bool live = lrow < m;
        const bool hi_lane = HI16 || nn < 8;
        const AT* ar = a + (int64_t)min(lrow, m - 1) * k + min(4096 * round + 512 * wave, k - 512) + 8 * kg;
        constexpr int CH = SETS == 1 ? 16 : 8;  // sub-blocks loaded together
        float4 xs[CH][2];
        float mx = 0.0f;
#pragma unroll
        for (int c0 = 0; c0 < 16; c0 += CH) {
#pragma unroll
            for (int j = 0; j < CH; j++) {
                xs[j][0] = v_lhs4<AT>(ar + 32 * (c0 + j));
                xs[j][1] = v_lhs4<AT>(ar + 32 * (c0 + j) + 4);
            }
#pragma unroll
            for (int j = 0; j < CH; j++)
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    const float4 x = xs[j][q];
                    mx = fmaxf(fmaxf(mx, fmaxf(fabsf(x.x), fabsf(x.y))), fmaxf(fabsf(x.z), fabsf(x.w)));
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        int e = (int)((__float_as_uint(mx) >> 23) & 0xffu) - 127;
        if (e < -100 || e > 127) e = 9;  // zero, denormal or non-finite: leave unscaled
        const float sc = live ? __uint_as_float((uint32_t)(127 + 9 - e) << 23) : 0.0f, isc = __uint_as_float((uint32_t)(127 - 9 + e) << 23);
        __builtin_amdgcn_wave_barrier();  // (a second set: the first one's staged sums have been read)
#pragma unroll
        for (int c0 = 0; c0 < 16; c0 += CH) {
            if constexpr (SETS > 1) {
#pragma unroll
                for (int j = 0; j < CH; j++) {
                    xs[j][0] = v_lhs4<AT>(ar + 32 * (c0 + j));
                    xs[j][1] = v_lhs4<AT>(ar + 32 * (c0 + j) + 4);
                }
            }
#pragma unroll
            for (int jj = 0; jj < CH; jj++) {
                const int j = c0 + jj;  // sub-block of the wavefront's two super-blocks
                uint32_t hw[4], lw[4];
                float ssum = 0.0f;
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    float4 x = xs[jj][q];
                    x.x *= sc; x.y *= sc; x.z *= sc; x.w *= sc;
                    // hi: the value cut to fp16 (toward zero); the residual x - hi is exact in fp32 and is cut the same way
                    const v_fp16x2 h01 = __builtin_amdgcn_cvt_pkrtz(x.x, x.y), h23 = __builtin_amdgcn_cvt_pkrtz(x.z, x.w);
                    hw[2 * q] = __builtin_bit_cast(uint32_t, h01);
                    hw[2 * q + 1] = __builtin_bit_cast(uint32_t, h23);
                    lw[2 * q] = v_pkrtz(x.x - (float)h01.x, x.y - (float)h01.y);
                    lw[2 * q + 1] = v_pkrtz(x.z - (float)h23.x, x.w - (float)h23.y);
                    ssum += (x.x + x.y) + (x.z + x.w);
                }
                const uint4 pick = hi_lane ? make_uint4(hw[0], hw[1], hw[2], hw[3]) : make_uint4(lw[0], lw[1], lw[2], lw[3]);
                fa[st][j >> 3][j & 7] = __builtin_bit_cast(v_half8, pick);
                sums[(j * 16 + nn) * 4 + kg] = ssum;
            }
        }
        if (kg == 0 && hi_lane) stg[8 * st + nn] = isc;
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // operand of the min term: row nn, column j = sub-block j of the super-block (lanes kg = 0, 1 hold 4 kg .. 4 kg + 3):
        // hi part or residual of the sub-block's lhs sum
#pragma unroll
        for (int bb = 0; bb < 2; bb++) {
            float sg[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float4 q = *(const float4*)(sums + ((8 * bb + 4 * (kg & 1) + i) * 16 + nn) * 4);
                sg[i] = kg < 2 ? (q.x + q.y) + (q.z + q.w) : 0.0f;
            }
            const v_fp16x2 h01 = __builtin_amdgcn_cvt_pkrtz(sg[0], sg[1]), h23 = __builtin_amdgcn_cvt_pkrtz(sg[2], sg[3]);
            const v_half4 shi = v_as_half4(__builtin_bit_cast(uint32_t, h01), __builtin_bit_cast(uint32_t, h23));
            const v_half4 slo = v_as_half4(v_pkrtz(sg[0] - (float)h01.x, sg[1] - (float)h01.y), v_pkrtz(sg[2] - (float)h23.x, sg[3] - (float)h23.y));
            fo[st][bb] = hi_lane ? shi : slo;
            if constexpr (HI16) fo2[bb] = slo;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_wave_barrier();

    for (int ti = 0; ti < my_tiles; ti++, it++) {
        const int slot = ti & 1;
        if (have && ti + 1 < my_tiles) {
            issue(round, ti + 1, slot ^ 1);
            wait_vmcnt<kVLoads>();
        } else {
            wait_vmcnt<0>();
        }
        const uint32_t* l32 = (const uint32_t*)(ring + slot * kVSlot + nn * kVRowLds);
        float acc[SETS][RN];
#pragma unroll
        for (int st = 0; st < SETS; st++)
#pragma unroll
            for (int r = 0; r < RN; r++) acc[st][r] = 0.0f;
        if (have) {
#pragma unroll
        for (int bb = 0; bb < 2; bb++) {
            const uint32_t* b32 = l32 + bb * (Q5_K_BPB >> 2);  // d, dmin | 12 scale bytes | qh[32] at dword 4 | qs[128] at dword 12
            const uint32_t dd = b32[0];
            const float d = h2f((uint16_t)(dd & 0xffffu)), dmin = h2f((uint16_t)(dd >> 16));
            const uint32_t s[3] = {b32[1], b32[2], b32[3]};
            const uint32_t QH0 = b32[4 + 2 * kg], QH1 = b32[5 + 2 * kg];  // fifth bits of columns 8 kg .. 8 kg + 7, bit j for sub-block j
            float u[SETS][RN];
#pragma unroll
            for (int st = 0; st < SETS; st++)
#pragma unroll
                for (int r = 0; r < RN; r++) u[st][r] = 0.0f;
            uint32_t mn[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                uint32_t scj;
                q4k_scale_min(j, s, scj, mn[j]);
                const uint32_t Q0 = b32[12 + 8 * (j >> 1) + 2 * kg], Q1 = b32[13 + 8 * (j >> 1) + 2 * kg];
                // (64 + q) as fp16 = 0x5400 + (q << 4): the nibble in the high half of the low byte, the fifth bit under 0x54 in
                // the high byte; minus 64 (exact) leaves q
                const uint32_t l0 = (j & 1) ? Q0 & 0xF0F0F0F0u : (Q0 << 4) & 0xF0F0F0F0u;
                const uint32_t l1 = (j & 1) ? Q1 & 0xF0F0F0F0u : (Q1 << 4) & 0xF0F0F0F0u;
                const uint32_t h0 = ((QH0 >> j) & m01) | c54, h1 = ((QH1 >> j) & m01) | c54;
                const uint4 bq = make_uint4(__builtin_amdgcn_perm(h0, l0, 0x05010400u), __builtin_amdgcn_perm(h0, l0, 0x07030602u),
                                            __builtin_amdgcn_perm(h1, l1, 0x05010400u), __builtin_amdgcn_perm(h1, l1, 0x07030602u));
                const v_half8 bw = __builtin_bit_cast(v_half8, bq) - off64;
                const float cs = (float)scj;
#pragma unroll
                for (int st = 0; st < SETS; st++) {
                    const v_float4 P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[st][bb][j], bw, zero4, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < RN; r++) u[st][r] = fmaf(cs, P[r], u[st][r]);
                }
            }
            // the min term: (sub-block sums of the lhs) x (m_j as fp16 integers, this lane's four columns of that operand)
            const uint32_t ma = kg == 0 ? mn[0] : mn[4], mb = kg == 0 ? mn[1] : mn[5], mc = kg == 0 ? mn[2] : mn[6], md = kg == 0 ? mn[3] : mn[7];
            const v_half4 bm = kg < 2 ? v_as_half4(v_pkrtz((float)ma, (float)mb), v_pkrtz((float)mc, (float)md)) : v_as_half4(0u, 0u);
#pragma unroll
            for (int st = 0; st < SETS; st++) {
                v_float4 O = __builtin_amdgcn_mfma_f32_16x16x16f16(fo[st][bb], bm, zero4, 0, 0, 0);
                if constexpr (HI16) O = __builtin_amdgcn_mfma_f32_16x16x16f16(fo2[bb], bm, O, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < RN; r++) acc[st][r] = fmaf(d, u[st][r], fmaf(-dmin, O[r], acc[st][r]));
            }
        }
        }
        // partial result of the tile: lane (column nn, operand rows 4 kg + r), lhs scale undone
        const int buf = it & 1;
        float* mine = red + ((buf * kVWaves + wave) * 8) * 64 + lane;
#pragma unroll
        for (int st = 0; st < SETS; st++)
#pragma unroll
            for (int r = 0; r < RN; r++) mine[(4 * st + r) * 64] = acc[st][r] * stg[HI16 ? 4 * kg + r : 8 * st + ((4 * kg + r) & 7)];
        __syncthreads();
        if (tid < MROWS * 16) {
            const int row = tid >> 4, col = tid & 15;  // lhs row, column of the tile
            const int n0 = ((int)blockIdx.x + ti * (int)gridDim.x) * 16;
            const float* src = HI16 ? red + (buf * kVWaves * 8 + (row & 3)) * 64 + col + 16 * (row >> 2)
                                    : red + (buf * kVWaves * 8 + 4 * (row >> 3) + (row & 3)) * 64 + col + 16 * ((row & 7) >> 2);
            float v = 0.0f;
#pragma unroll
            for (int ww = 0; ww < kVWaves; ww++)
                if (ww < nw) v += HI16 ? src[ww * 512] : src[ww * 512 + 0] + src[ww * 512 + 32];  // hi rows, residual rows (8 further)
            if (row < m && n0 + col < n) {
                float* o = out + (ROUNDS == 2 ? (int64_t)round * m * ldo : 0) + (int64_t)row * ldo + n0 + col;
                *o = ROUNDS == 1 && round ? *o + v : v;
            }
        }
    }
    }
}

bool gemv_q5_k_mm_supported(const void* w, int64_t m, int64_t n, int64_t k) {
    return !kernel_disabled("q5k_mm") && m >= 1 && m <= 64 && k >= 512 && k % 512 == 0 && k <= 32768 && n >= 1 && n <= 0x7fffffff &&
           ((uintptr_t)w & 15) == 0;
}

// Any number of lhs rows in passes of 16 (bf16) or 8 (fp32); out is fp32 [m, ldo].  The caller checks
// gemv_q5_k_mm_supported.  workspace: gemv_kquant_mm_workspace_bytes(m, n, k) bytes, or null (the rounds of a long K then
// run one after the other in each workgroup).
hipError_t launch_gemv_q5_k_mm(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out, int64_t ldo,
                               void* workspace, hipStream_t s) {
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const int64_t ntiles = (n + 15) / 16;
    // A long K: a workgroup per (share of the tiles, round), so that it converts its lhs operands once and streams several
    // tiles behind them; the rounds' results go to the workspace and are added in round order by a launch of their own.
    const int rounds = (int)(((k >> 8) + 15) / 16);
    const bool side_by_side = rounds > 1 && workspace && ldo == n && !kernel_disabled("kquant_mm_rounds_grid");
    const dim3 grid((unsigned)std::min<int64_t>(ntiles, side_by_side ? std::max(1, cus / rounds) : cus), side_by_side ? rounds : 1), block(64 * kVWaves);
    const size_t esz = a_dtype == QMM_F32 ? 4 : 2;
    // (sixteen fp32 rows would be two operand sets of 64 registers each: the compiler spills 700 bytes; two passes of eight)
    const int pass = a_dtype != QMM_F32 ? 16 : 8;
    for (int m0 = 0; m0 < m; m0 += pass) {
        const int rows = std::min(pass, m - m0);
        const void* am = (const char*)a + (size_t)m0 * k * esz;
        float* om = out + (int64_t)m0 * ldo;
#define QMM_Q5MM(MR_, AT_)                                                                                              \
    do {                                                                                                                \
        if (k == 4096) {                                                                                                \
            hipError_t e_ = allow_full_lds<gemv_q5_k_mm_kernel<MR_, AT_, 0>>();                                         \
            if (e_ != hipSuccess) return e_;                                                                            \
            gemv_q5_k_mm_kernel<MR_, AT_, 0><<<grid, block, kVLds, s>>>(w, (const AT_*)am, om, rows, (int)n, (int)k, ldo); \
        } else if (side_by_side) {                                                                                      \
            hipError_t e_ = allow_full_lds<gemv_q5_k_mm_kernel<MR_, AT_, 2>>();                                         \
            if (e_ != hipSuccess) return e_;                                                                            \
            gemv_q5_k_mm_kernel<MR_, AT_, 2><<<grid, block, kVLds, s>>>(w, (const AT_*)am, (float*)workspace, rows, (int)n, (int)k, ldo); \
        } else {                                                                                                        \
            hipError_t e_ = allow_full_lds<gemv_q5_k_mm_kernel<MR_, AT_, 1>>();                                         \
            if (e_ != hipSuccess) return e_;                                                                            \
            gemv_q5_k_mm_kernel<MR_, AT_, 1><<<grid, block, kVLds, s>>>(w, (const AT_*)am, om, rows, (int)n, (int)k, ldo); \
        }                                                                                                               \
    } while (0)
#define QMM_Q5MM_AT(MR_)                               \
    do {                                               \
        if (a_dtype == QMM_F32) QMM_Q5MM(MR_, float);  \
        else QMM_Q5MM(MR_, uint16_t);                  \
    } while (0)
        if (rows <= 2) QMM_Q5MM_AT(2);
        else if (rows <= 4) QMM_Q5MM_AT(4);
        else if (rows <= 8) QMM_Q5MM_AT(8);
        else QMM_Q5MM(16, uint16_t);
#undef QMM_Q5MM_AT
#undef QMM_Q5MM
        hipError_t e = hipGetLastError();
        if (e == hipSuccess && side_by_side) e = launch_sum_shares((const float*)workspace, om, (int64_t)rows * n, rounds, s);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace qmm
