// Q6_K with up to 16 lhs rows a pass on the matrix cores, K a multiple of 2048 up to 32768: the weight rows are decoded
// once for all lhs rows of a pass, and the per-16 int8 scales are applied to a 16 x 16 block of results at a time.
//
// Arithmetic.  A Q6_K weight is d * sc * q with q = (ql nibble | qh bits << 4) - 32 and sc an int8 per 16 weights.  The
// matrix-core operand of a weight is q itself as fp16: a byte permute interleaves the nibble bytes with bytes that hold
// the two qh bits under 0x54, which reads as 0x5400 + (code << 4) = 64 + code, and a packed subtraction of 96 (exact)
// leaves q.  The lhs is narrowed to fp16 after an exact power-of-two scaling per (lhs row, wavefront share of K) as hi
// part plus residual, which sit in operand rows 0..7 and 8..15 of the same instruction.  One v_mfma_f32_16x16x16_f16
// per scale group gives P = sum x * q for 16 weight rows at once (products exact, fp32 sums); u += sc * P in the lanes,
// acc += d * u per super-block.  (Leaving the 96 in the operand and taking 96 * sum x out through the lhs group sums
// saves the subtraction, but the sums then carry a term three to five times the wanted one: results a thousand times
// smaller than their row's typical one missed the tolerance.)
//
// Shape of the work.  A workgroup of 8 wavefronts owns 16-row tiles t = block, block + grid, ...; wavefront w owns
// super-blocks 2 w and 2 w + 1 of every row (K = 4096: 16 super-blocks) and keeps the lhs operands of those 512 columns
// in registers for all its tiles.  Longer rows go in rounds of 16 super-blocks: operands converted again, all tiles
// again, results added to the output of the round before (the same thread stored it).  The 420 bytes of its super-blocks of each of the 16 rows travel global -> LDS
// directly as 27 aligned 16-byte pieces per row (a row of 3360 bytes and 420 w both are multiples of 4 past a 16-byte
// boundary, so fields keep a compile-time byte parity and the row stride of 432 bytes spreads 16 rows over all banks)
// into a private ring of two slots, one tile ahead.  Per tile the wavefronts' partial results meet in LDS (two
// buffers, one barrier per tile) and are added in wavefront order.
#include <stdlib.h>

#include <algorithm>

#include "lds_stream.h"
#include "qmm_device.h"
#include "qmm_internal.h"

namespace qmm {

typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef __fp16 fp16x2v __attribute__((ext_vector_type(2)));

namespace {

constexpr int kQWaves = 8;
constexpr int kQRowPieces = 27;                 // 16-byte pieces per row and item: up to 12 bytes of lead-in + 420
constexpr int kQRowLds = kQRowPieces * 16;      // 432
constexpr int kQPieces = 16 * kQRowPieces;      // 432 pieces per item
constexpr int kQLoads = (kQPieces + 63) / 64;   // 7 load instructions, the last one by 48 lanes
constexpr int kQSlot = kQLoads * 1024;
constexpr int kQSlots = 2;
constexpr int kQRing = kQWaves * kQSlots * kQSlot;
constexpr int kQRed = 2 * kQWaves * 2 * 1024;   // two buffers of two 16 x 16 partial results (4 floats a lane each) per wavefront
constexpr int kQInv = kQWaves * 16 * 4;         // inverse lhs scales: 16 lhs rows per wavefront
constexpr int kQLds = kQRing + kQRed + kQInv;
static_assert(kQLds <= kLdsPerCu, "Q6_K small-batch kernel LDS");

__device__ __forceinline__ half4v as_half4(uint32_t lo, uint32_t hi) {
    const uint2 v = make_uint2(lo, hi);
    return __builtin_bit_cast(half4v, v);
}
__device__ __forceinline__ uint32_t pkrtz(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
__device__ __forceinline__ float s8(uint32_t x, int shift) { return (float)((int)(x << (24 - shift)) >> 24); }

template <typename AT>
__device__ __forceinline__ float4 lhs4(const AT* __restrict__ a);
template <>
__device__ __forceinline__ float4 lhs4<float>(const float* __restrict__ a) {
    return *(const float4*)a;
}
template <>
__device__ __forceinline__ float4 lhs4<uint16_t>(const uint16_t* __restrict__ a) {
    const uint2 v = *(const uint2*)a;
    return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                       __uint_as_float(v.y & 0xffff0000u));
}

// 16 bytes per lane, non-temporal, global (uniform base + lane offset) -> LDS at lds_base + 16 * lane
__device__ __forceinline__ void stream16_to_lds(uint32_t lane_offset, const void* uniform_base, uint32_t lds_base) {
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

// MROWS: lhs rows of the pass, 1, 2, 4, 8 or 16 (>= m; rows past m are zero operands and their results are dropped).  Sixteen
// rows are two sets of eight, each with its own operands and sums, multiplied with the same decoded weights.
// Accumulator registers that hold no wanted lhs row are not computed: a lane holds rows 4 (lane / 16) + r of a set.
// ROUNDS: K beyond 4096 (or 2048) in rounds of 16 super-blocks; 0: a single round, everything about rounds is constant; 1: the
// workgroup walks the rounds one after the other and adds to its own output; 2: round blockIdx.y only, its result stored as
// part blockIdx.y of [rounds][m][ldo] at `out` (the caller adds the parts in round order).
template <int MROWS, typename AT, int ROUNDS>
__global__ __launch_bounds__(64 * kQWaves) void gemv_q6_k_mm_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                                   float* __restrict__ out, int m, int n, int k, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nn = lane & 15, kg = lane >> 4;
    // Sixteen bf16 lhs rows need no residual rows (a bf16 value scaled by a power of two is an fp16 number, down to what is
    // 2^-26 of its row's largest: far below the fp32 sums' resolution): all sixteen operand rows carry hi parts, one set.
    constexpr bool HI16 = MROWS == 16 && sizeof(AT) == 2;
    constexpr int SETS = MROWS > 8 && !HI16 ? 2 : 1, MR1 = MROWS > 8 ? 8 : MROWS;  // sets of lhs rows, rows of a set
    constexpr int RN = MR1 < 4 ? MR1 : 4;  // accumulator registers in use per set
    const int nblk = k >> 8;                                  // a multiple of 8: rows are whole 16-byte pieces
    const int64_t row_bytes = (int64_t)nblk * Q6_K_BPB;
    uint8_t* ring = smem + wave * (kQSlots * kQSlot);
    const uint32_t ring_lds = lds_address(ring);
    float* red = (float*)(smem + kQRing);  // [2][kQWaves][2 sets][4][64]
    const int ntiles = (n + 15) >> 4;
    const int my_tiles = (int)blockIdx.x < ntiles ? (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const int lead = (2 * wave * Q6_K_BPB) & 15;  // of this wavefront's super-blocks past a 16-byte boundary: 0, 4, 8 or 12
                                                  // (the same in every round: 16 super-blocks are 3360 bytes)

    // piece p = lane + 64 i of an item: row p / 27, piece p % 27 of the row's aligned range
    uint32_t full[kQLoads];  // byte offset of the piece in a tile that lies inside the matrix
#pragma unroll
    for (int i = 0; i < kQLoads; i++) {
        const int p = min(lane + 64 * i, kQPieces - 1), pr = p / kQRowPieces;
        full[i] = (uint32_t)pr * (uint32_t)row_bytes + (uint32_t)((p - pr * kQRowPieces) * 16);
    }
    auto issue = [&](int round, int ti, int slot) {
        const int n0 = ((int)blockIdx.x + ti * (int)gridDim.x) * 16;
        const uint8_t* base = w + (int64_t)n0 * row_bytes + ((16 * round + 2 * wave) * Q6_K_BPB - lead);
        const int last = n - 1 - n0;  // rows past the matrix repeat its last row (their results are dropped)
#pragma unroll
        for (int i = 0; i < kQLoads; i++) {
            uint32_t off = full[i];
            if (last < 15) {  // (the last tile of a ragged matrix only)
                const uint32_t pr = off / (uint32_t)row_bytes;
                off -= (pr - (uint32_t)min((int)pr, last)) * (uint32_t)row_bytes;
            }
            if (i < kQLoads - 1 || lane < kQPieces - 64 * (kQLoads - 1)) stream16_to_lds(off, base, ring_lds + slot * kQSlot + i * 1024);
        }
    };
    // (constants of the unpack in vector registers: an and-or in one instruction takes no literal and one scalar at most)
    uint32_t m03 = 0x03030303u, c54 = 0x54545454u;
    asm volatile("" : "+v"(m03), "+v"(c54));
    const float4v zero4 = {0.f, 0.f, 0.f, 0.f};
    const half4v off96 = {(_Float16)96.0f, (_Float16)96.0f, (_Float16)96.0f, (_Float16)96.0f};
    float* stg = (float*)(smem + kQRing + kQRed) + 16 * wave;  // this wavefront's inverse lhs scales
    int it = 0;  // tiles done, over all rounds: its parity picks the buffer of the partial results

    // K in rounds of 16 super-blocks (4096 columns); a last round of 8 keeps wavefronts 0..3 busy.  Results of the rounds
    // after the first are added to what the same thread stored before.
    const int rounds = ROUNDS ? (nblk + 15) >> 4 : 1;
    const int round0 = ROUNDS == 2 ? (int)blockIdx.y : 0, round1 = ROUNDS == 2 ? round0 + 1 : rounds;
    for (int round = round0; round < round1; round++) {
    const bool have = ROUNDS ? 16 * round + 2 * wave < nblk : true;            // this wavefront has super-blocks in the round
    const int nw = ROUNDS ? min(kQWaves, (nblk - 16 * round) >> 1) : kQWaves;  // wavefronts that have
    if (have && my_tiles > 0) issue(round, 0, 0);

    // ---- the lhs operands of this wavefront's 512 columns.  Operand row nn of set st: lhs row 8 st + nn % 8, hi part (nn < 8)
    // or residual.  The inverse scales go to LDS and are read back where a tile's sums are finished.
    half4v fa[SETS][2][16];
#pragma unroll
    for (int st = 0; st < SETS; st++) {
        const int lrow = HI16 ? nn : 8 * st + (nn & 7);
        const bool live = lrow < m;
        const AT* ar = a + (int64_t)min(lrow, m - 1) * k + min(4096 * round + 512 * wave, k - 512) + 4 * kg;
        // One set: all 32 loads of the lane go out together (one round trip) and the values stay in registers for the
        // conversion.  Two sets: 16 at a time, and a second round of loads for the conversion (the first set's operands
        // take 64 registers already).
        constexpr int CH = SETS == 1 ? 32 : 16;
        float4 xs[CH];
        float mx = 0.0f;
#pragma unroll
        for (int c0 = 0; c0 < 32; c0 += CH) {
#pragma unroll
            for (int g = 0; g < CH; g++) xs[g] = lhs4<AT>(ar + 16 * (c0 + g));
#pragma unroll
            for (int g = 0; g < CH; g++) {
                const float4 x = xs[g];
                mx = fmaxf(fmaxf(mx, fmaxf(fabsf(x.x), fabsf(x.y))), fmaxf(fabsf(x.z), fabsf(x.w)));
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        int e = (int)((__float_as_uint(mx) >> 23) & 0xffu) - 127;
        if (e < -100 || e > 127) e = 9;  // zero, denormal or non-finite: leave unscaled
        const float sc = live ? __uint_as_float((uint32_t)(127 + 9 - e) << 23) : 0.0f, isc = __uint_as_float((uint32_t)(127 - 9 + e) << 23);
#pragma unroll
        for (int c0 = 0; c0 < 32; c0 += CH) {
            if constexpr (SETS > 1) {
#pragma unroll
                for (int g = 0; g < CH; g++) xs[g] = lhs4<AT>(ar + 16 * (c0 + g));
            }
#pragma unroll
            for (int gg = 0; gg < CH; gg++) {
                const int g = c0 + gg;
                float4 x = xs[gg];
                x.x *= sc; x.y *= sc; x.z *= sc; x.w *= sc;
                // hi: the value cut to fp16 (toward zero); the residual x - hi is exact in fp32 and is cut the same way
                const fp16x2v h01 = __builtin_amdgcn_cvt_pkrtz(x.x, x.y), h23 = __builtin_amdgcn_cvt_pkrtz(x.z, x.w);
                const uint32_t r01 = pkrtz(x.x - (float)h01.x, x.y - (float)h01.y), r23 = pkrtz(x.z - (float)h23.x, x.w - (float)h23.y);
                fa[st][g >> 4][g & 15] = HI16 || nn < 8 ? as_half4(__builtin_bit_cast(uint32_t, h01), __builtin_bit_cast(uint32_t, h23)) : as_half4(r01, r23);
            }
        }
        if (kg == 0 && (HI16 || nn < 8)) stg[8 * st + nn] = isc;
    }
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    for (int ti = 0; ti < my_tiles; ti++, it++) {
        const int slot = ti & 1;
        if (have && ti + 1 < my_tiles) {
            issue(round, ti + 1, slot ^ 1);
            wait_vmcnt<kQLoads>();
        } else {
            wait_vmcnt<0>();
        }
        const uint32_t* l32 = (const uint32_t*)(ring + slot * kQSlot + nn * kQRowLds) + (lead >> 2);
        float acc[SETS][RN];
#pragma unroll
        for (int st = 0; st < SETS; st++)
#pragma unroll
            for (int r = 0; r < RN; r++) acc[st][r] = 0.0f;
        if (have) {
#pragma unroll
        for (int bb = 0; bb < 2; bb++) {
            constexpr int kBlockDw[2] = {0, (Q6_K_BPB) >> 2};  // dword of the super-block's first aligned byte: 0, 52
            const int q0 = kBlockDw[bb];
            const bool odd = bb == 1;  // the second super-block starts 2 bytes into that dword
            auto rd = [&](int dw) __attribute__((always_inline)) {
                return odd ? __builtin_amdgcn_alignbyte(l32[q0 + dw + 1], l32[q0 + dw], 2u) : l32[q0 + dw];
            };
            const uint32_t s0 = rd(48), s1 = rd(49), s2 = rd(50), s3 = rd(51);
            const uint32_t dv = odd ? l32[q0 + 52] >> 16 : l32[q0 + 52] & 0xffffu;
            const float d = h2f((uint16_t)dv);
            const uint32_t sd[4] = {s0, s1, s2, s3};
            float u[SETS][RN];
#pragma unroll
            for (int st = 0; st < SETS; st++)
#pragma unroll
                for (int r = 0; r < RN; r++) u[st][r] = 0.0f;
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int e2 = 0; e2 < 2; e2++) {
                    const uint32_t QH = rd(32 + 8 * h + 4 * e2 + kg);
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const int g = 8 * h + 2 * c + e2;  // scale group: weights 128 h + 32 c + 16 e2 + (0..15)
                        const uint32_t QL = rd(16 * h + 8 * (c & 1) + 4 * e2 + kg);
                        // (64 + code) as fp16 = 0x5400 + (code << 4): the nibble in the high half of the low byte, the two qh bits
                        // under 0x54 in the high byte; minus 96 (exact) leaves q = code - 32
                        const uint32_t lo = (c >> 1) ? QL & 0xF0F0F0F0u : (QL << 4) & 0xF0F0F0F0u;
                        const uint32_t hi = ((QH >> (2 * c)) & m03) | c54;
                        const half4v bw = as_half4(__builtin_amdgcn_perm(hi, lo, 0x05010400u), __builtin_amdgcn_perm(hi, lo, 0x07030602u)) - off96;
                        const float cs = s8(sd[g >> 2], 8 * (g & 3));
#pragma unroll
                        for (int st = 0; st < SETS; st++) {
                            const float4v P = __builtin_amdgcn_mfma_f32_16x16x16f16(fa[st][bb][g], bw, zero4, 0, 0, 0);
#pragma unroll
                            for (int r = 0; r < RN; r++) u[st][r] = fmaf(cs, P[r], u[st][r]);
                        }
                    }
                }
#pragma unroll
            for (int st = 0; st < SETS; st++)
#pragma unroll
                for (int r = 0; r < RN; r++) acc[st][r] = fmaf(d, u[st][r], acc[st][r]);
        }
        }
        // partial result of the tile: lane (column nn, operand rows 4 kg + r), lhs scale undone
        const int buf = it & 1;
        float* mine = red + ((buf * kQWaves + wave) * 8) * 64 + lane;
#pragma unroll
        for (int st = 0; st < SETS; st++)
#pragma unroll
            for (int r = 0; r < RN; r++) mine[(4 * st + r) * 64] = acc[st][r] * stg[HI16 ? 4 * kg + r : 8 * st + ((4 * kg + r) & 7)];
        __syncthreads();
        if (tid < MROWS * 16) {
            const int row = tid >> 4, col = tid & 15;  // lhs row, column of the tile
            const int n0 = ((int)blockIdx.x + ti * (int)gridDim.x) * 16;
            const float* src = HI16 ? red + (buf * kQWaves * 8 + (row & 3)) * 64 + col + 16 * (row >> 2)
                                    : red + (buf * kQWaves * 8 + 4 * (row >> 3) + (row & 3)) * 64 + col + 16 * ((row & 7) >> 2);
            float v = 0.0f;
#pragma unroll
            for (int ww = 0; ww < kQWaves; ww++)
                if (ww < nw) v += HI16 ? src[ww * 512] : src[ww * 512 + 0] + src[ww * 512 + 32];  // hi rows, residual rows (8 further)
            if (row < m && n0 + col < n) {
                float* o = out + (ROUNDS == 2 ? (int64_t)round * m * ldo : 0) + (int64_t)row * ldo + n0 + col;
                *o = ROUNDS == 1 && round ? *o + v : v;
            }
        }
    }
    }
}

bool gemv_q6_k_mm_supported(const void* w, int64_t m, int64_t n, int64_t k) {
    return !kernel_disabled("q6k_mm") && m >= 1 && m <= 64 && k >= 2048 && k % 2048 == 0 && k <= 32768 && n >= 1 && n <= 0x7fffffff && ((uintptr_t)w & 15) == 0;
}

// K beyond 4096 with the rounds side by side in the grid (this kernel and the Q5_K one): room for the rounds' results of one
// pass of up to 16 lhs rows.
int64_t gemv_kquant_mm_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    if (k <= 4096 || k % 512 || k > 32768 || m < 1 || m > 64) return 0;
    return ((k >> 8) + 15) / 16 * std::min<int64_t>(m, 16) * n * 4;
}

// Any number of lhs rows in passes of 16 (K = 4096) or 8; out is fp32 [m, ldo].  The caller checks gemv_q6_k_mm_supported.
// workspace: gemv_kquant_mm_workspace_bytes(m, n, k) bytes, or null (the rounds of a long K then run one after the other
// in each workgroup).
hipError_t launch_gemv_q6_k_mm(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out, int64_t ldo,
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
    const dim3 grid((unsigned)std::min<int64_t>(ntiles, side_by_side ? std::max(1, cus / rounds) : cus), side_by_side ? rounds : 1), block(64 * kQWaves);
    const size_t esz = a_dtype == QMM_F32 ? 4 : 2;
    // Sixteen bf16 rows are one operand set and go as one pass everywhere.  Sixteen fp32 rows are two sets (hi parts and
    // residuals of eight rows each) and the kernel spills registers in its loop: two passes of eight rows are faster unless a
    // workgroup has many tiles to stream (K = 4096, 16 rows: 4096 rows of weights 26.9 against 36.1 us, 14336: 42.7 against 46.7,
    // 32000: 64.5 against 60.2, 128256: 192 against 144; K in rounds, 4096 x 14336: 98 against 112 us).
    const int pass = a_dtype != QMM_F32 || (k == 4096 && ntiles >= 6 * (int64_t)cus) ? 16 : 8;
    for (int m0 = 0; m0 < m; m0 += pass) {
        const int rows = std::min(pass, m - m0);
        const void* am = (const char*)a + (size_t)m0 * k * esz;
        float* om = out + (int64_t)m0 * ldo;
#define QMM_Q6MM(MR_, AT_)                                                                                          \
    do {                                                                                                            \
        if (k == 4096) {                                                                                            \
            hipError_t e_ = allow_full_lds<gemv_q6_k_mm_kernel<MR_, AT_, 0>>();                                     \
            if (e_ != hipSuccess) return e_;                                                                        \
            gemv_q6_k_mm_kernel<MR_, AT_, 0><<<grid, block, kQLds, s>>>(w, (const AT_*)am, om, rows, (int)n, (int)k, ldo); \
        } else if (side_by_side) {                                                                                  \
            hipError_t e_ = allow_full_lds<gemv_q6_k_mm_kernel<MR_, AT_, 2>>();                                     \
            if (e_ != hipSuccess) return e_;                                                                        \
            gemv_q6_k_mm_kernel<MR_, AT_, 2><<<grid, block, kQLds, s>>>(w, (const AT_*)am, (float*)workspace, rows, (int)n, (int)k, ldo); \
        } else {                                                                                                    \
            hipError_t e_ = allow_full_lds<gemv_q6_k_mm_kernel<MR_, AT_, 1>>();                                     \
            if (e_ != hipSuccess) return e_;                                                                        \
            gemv_q6_k_mm_kernel<MR_, AT_, 1><<<grid, block, kQLds, s>>>(w, (const AT_*)am, om, rows, (int)n, (int)k, ldo); \
        }                                                                                                           \
    } while (0)
#define QMM_Q6MM_AT(MR_)                               \
    do {                                               \
        if (a_dtype == QMM_F32) QMM_Q6MM(MR_, float);  \
        else QMM_Q6MM(MR_, uint16_t);                  \
    } while (0)
        if (rows == 1) QMM_Q6MM_AT(1);
        else if (rows == 2) QMM_Q6MM_AT(2);
        else if (rows <= 4) QMM_Q6MM_AT(4);
        else if (rows <= 8) QMM_Q6MM_AT(8);
        else QMM_Q6MM_AT(16);
#undef QMM_Q6MM_AT
#undef QMM_Q6MM
        hipError_t e = hipGetLastError();
        if (e == hipSuccess && side_by_side) e = launch_sum_shares((const float*)workspace, om, (int64_t)rows * n, rounds, s);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace qmm
