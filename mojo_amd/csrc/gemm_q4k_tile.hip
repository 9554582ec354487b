// Q4_K prefill kernel for large problems (hundreds of lhs rows, enough 256 x 128 output tiles to fill the
// device): every weight tile is unpacked ONCE per workgroup into LDS, in matrix-core operand order, and all
// eight wavefronts of the workgroup take their operands from there.
//
// Arithmetic: that of gemm_q4k.hip.  A masked nibble is the fp16 subnormal q * 2^-24 and one packed fp16
// multiply folds the 6-bit sub-block scale in (sc * q * 2^-18, exact); the lhs is scaled per row by a power
// of two and narrowed to fp16, so every product inside v_mfma_f32_32x32x16_f16 is exact and the sums are
// fp32.  Per super-block b the matrix cores produce P_b = sum_k a * (sc * q); the lanes apply
// acc += d[n, b] * P_b.  The min term is two extra matrix-core products per super-block over the eight
// sub-block sums of the lhs (hi + lo) with -(dmin * mn) split exactly into two fp16 values.
//
// Shape.  One workgroup of 8 wavefronts per compute unit, persistent over 256 x 128 output tiles; wavefront
// (wm, wn) owns the 64 x 64 sub-tile at (64 wm, 64 wn).  K advances in steps of 64 (one 32-byte code chunk
// per weight column: sub-block 2c in the low nibbles, 2c + 1 in the high ones):
//   * lhs: 256 rows x 128 bytes per step go global -> LDS directly (global_load_lds_dwordx4, two steps
//     ahead, three buffers).  The 16-byte pieces of a row are stored at piece index p ^ ((row / 2) % 8), so
//     that the operand reads of 32 rows at one piece index spread over all banks without padding (an
//     LDS-direct load writes 1 KB contiguously, which rules padding out; rows are 128 bytes, half the width
//     of the banks, so the key has to tell 16 rows apart: with row % 8 the reads run at 170 B per clock, with
//     (row / 2) % 8 at 265, as fast as rows padded to 144 bytes).
//   * weights: the 32 code bytes per column of a step also go global -> LDS directly (three steps ahead, a
//     ring of three 4 KB stages; wavefront w fetches the columns 16 w .. 16 w + 15 that its own threads
//     unpack).  Thread (column t / 4, part t % 4) reads 8 of them one step before they are needed and turns
//     them into 8 + 8 operand values: four masks, two shifts and eight packed multiplies for 16 weights,
//     about 1.5 vector instructions per matrix-core instruction of the workgroup (the kernel that unpacks per
//     wavefront needs 5).  They go to LDS as the two 16-byte pieces (slice f = part: low-nibble piece,
//     high-nibble piece) of the column's row, same swizzle.  The scale pair of chunk c is decoded by the
//     thread with part = c once per super-block and handed to the other three threads of the column's quad
//     by a DPP move.
//   * per super-block, the 16-byte block headers arrive the same way (two stages); the threads write
//     d * 2^18 and the split min operands of their column to small LDS tables, and the lhs sub-block sums of
//     the tile rows go global -> LDS directly.  The rescale of a finished super-block is interleaved, sub-tile
//     by sub-tile, with the first matrix-core instructions of the next one (no pipeline drain); the min term
//     follows one step later.
//   No load of the main loop has a register destination: nothing the compiler allocates is written
//   asynchronously (a register that is in flight across a loop back-edge is not safe: where the compiler
//   copies the variable, the data lands in a register that by then holds something else).
//   * one barrier per step, placed before the last of the four 16-wide slices: by then every operand read
//     of the step has been issued, so the buffers can be refilled, and the first operands of the next step
//     are read under the last slice's matrix-core instructions.
// All global loads are issued from inline asm and waited for with exact vmcnt counts (lds_stream.h): at the
// end of a step a wavefront waits for everything it issued before that step, which gives every load at
// least one full step (about 0.5 us) in flight and most of them two.
//
// LDS operand reads are 16 bytes per lane: 2 lhs + 2 weight fragments per slice and wavefront against 4
// matrix-core instructions, 1 KB per instruction, i.e. about 130 B per clock per compute unit at full
// matrix-core rate; the LDS of this part delivers about 290 B per clock for conflict-free 16-byte reads
// (measured with 16 wavefronts reading; a single wavefront that waits for each read sees 64).
#include <stdlib.h>

#include <type_traits>

#include "gemm_lhs.h"
#include "gemm_tile.h"
#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int TM = 256, TN = 128;
constexpr int kABuf = TM * 128;  // bytes of one lhs step buffer: 256 rows x 64 halfs
constexpr int kBBuf = TN * 128;  // bytes of one unpacked weight step buffer: 128 columns x 64 halfs
constexpr int kSBuf = TM * 32;   // lhs sub-block sums of a super-block: 256 rows x (8 hi + 8 lo) halfs
constexpr int kMBuf = TN * 32;   // min operands of a super-block: 128 columns x (8 hi + 8 lo) halfs
constexpr int kDBuf = TN * 4;    // d * 2^18 of a super-block: 128 columns, fp32
constexpr int kQBuf = TN * 32;   // code bytes of a step: 128 columns x 32 bytes
constexpr int kHBuf = TN * 16;   // block headers of a super-block: 128 columns x 16 bytes
constexpr int kOffA = 0, kOffB = kOffA + 3 * kABuf, kOffS = kOffB + 2 * kBBuf, kOffM = kOffS + kSBuf;
constexpr int kOffD = kOffM + kMBuf, kOffInv = kOffD + kDBuf, kOffQ = kOffInv + TM * 4, kOffH = kOffQ + 3 * kQBuf;
constexpr int kTileLds = kOffH + 2 * kHBuf;
static_assert(kTileLds <= kLdsPerCu, "tile kernel LDS");
constexpr float kTwo18f = 262144.0f;

// the value of lane (lane & ~3) + Q of every quad, in all four of its lanes
template <int Q>
__device__ __forceinline__ uint32_t quad_bcast(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, Q | (Q << 2) | (Q << 4) | (Q << 6), 0xf, 0xf, true);
}

__device__ __forceinline__ float cvt_ubyte0(uint32_t v) { float f; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float cvt_ubyte1(uint32_t v) { float f; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v)); return f; }

}  // namespace

__global__ __launch_bounds__(512, 1) void gemm_q4_k_tile_kernel(const uint8_t* __restrict__ w, const _Float16* __restrict__ a16,
                                                                 const _Float16* __restrict__ asum, const float* __restrict__ inv,
                                                                 float* __restrict__ out, int m, int n, int k, int tiles_m,
                                                                 int tiles_n, int with_min, int accumulate, int allow_split) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int nl = lane & 31, g = lane >> 5;
    const int nblk_row = k >> 8;  // super-blocks of a whole row
    const int64_t row_bytes = (int64_t)nblk_row * Q4_K_BPB;
    const int ucol = tid >> 2, upart = tid & 3;  // unpack role: weight column of the tile, 8-byte part of its chunk

    // operand reads: row (or column) nl of the wavefront's 32-row groups, piece 2 f + g, swizzled
    // (piece (2 f + g) ^ key = (2 f) ^ (g ^ key): the address of slice f is that of slice 0 with f << 5 xor-ed in; the bases are multiples of 128)
    const uint32_t fb0 = (uint32_t)(kOffB + (wn * 64 + nl) * 128 + ((g ^ ((nl >> 1) & 7)) << 4));
    static_assert(kOffB % 128 == 0 && kABuf % 128 == 0 && kBBuf % 128 == 0, "operand rows must start on 128-byte boundaries");
    const int a_minus_b = (kOffA + wm * 64 * 128) - (kOffB + wn * 64 * 128);
    // unpack writes: pieces 2 part (low nibbles) and 2 part + 1 (high nibbles) of column ucol
    const uint32_t bw_lo = (uint32_t)(kOffB + ucol * 128 + (((2 * upart) ^ ((ucol >> 1) & 7)) << 4));  // (the high-nibble piece: this ^ 16)
    const uint32_t M1 = 0x000F000Fu, M2 = 0x00F000F0u;

    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8, wgs_per_xcd = (int)(gridDim.x >> 3);
    const int xcd_base = (int)(blockIdx.x & 7) * per_xcd, n_x = max(0, min(per_xcd, total - xcd_base));
    int full;
    const int units = xcd_units(n_x, wgs_per_xcd, nblk_row, allow_split, full);
    for (int u = (int)(blockIdx.x >> 3); u < units; u += wgs_per_xcd) {
        const TileUnit unit = xcd_unit(u, xcd_base, full, nblk_row);
        const int nblk = unit.nb, ns = nblk * 4, kb0 = unit.kb0;  // this unit's share of K
        int tile_m, tile_n;
        tile_order(unit.tile, tiles_m, tiles_n, kTileGm, tile_m, tile_n);
        const int m0 = tile_m * TM, n0 = tile_n * TN;

        // ---- this thread's sources: a fixed 32-bit byte offset per lane, added to a wave-uniform base that moves with the step
        // lhs rows wave * 32 + 8 i + lane / 8 (i = 0..3); LDS position lane % 8 of a row holds piece (lane % 8) ^ key(row),
        // key(row) = (row / 2) % 8 = (4 i + lane / 16) % 8
        // (the 8-row group i goes into the uniform base; the lane offset only depends on the parity of i, through the key)
        uint32_t a_off[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
            a_off[i] = (uint32_t)((lane >> 3) * (k * 2) + (((lane & 7) ^ ((4 * i + (lane >> 4)) & 7)) << 4));
        const uint8_t* a_base = (const uint8_t*)a16 + ((int64_t)(m0 + wave * 32) * k + kb0 * 256) * 2;
        const uint32_t s_off = (uint32_t)((wave * 32 + (lane >> 1)) * (nblk_row * 32) + (lane & 1) * 16);
        const uint8_t* s_base = (const uint8_t*)asum + ((int64_t)m0 * nblk_row + kb0) * 32;
        // weight columns this lane fetches: codes (lanes 0..31: column 16 wave + lane / 2, half lane % 2), headers (lanes 0..15)
        const uint32_t q_off = (uint32_t)((min(n0 + wave * 16 + ((lane & 31) >> 1), n - 1) - n0) * (int)row_bytes + (lane & 1) * 16);
        const uint32_t h_off = (uint32_t)((min(n0 + wave * 16 + (lane & 15), n - 1) - n0) * (int)row_bytes);
        const uint8_t* w_base = w + (int64_t)n0 * row_bytes + kb0 * Q4_K_BPB;

        // the i-th of the four loads that bring this wavefront's 32 rows of the lhs of step `step` into buffer `buf`
        auto issue_A1 = [&](int step, int buf, int i) __attribute__((always_inline)) {
            const uint8_t* src = a_base + (int64_t)min(step, ns - 1) * 128;
            const uint32_t dst = lds0 + kOffA + buf * kABuf + wave * 4096;
            load16_to_lds(a_off[i & 1], src + (int64_t)i * 16 * k, (uint32_t)__builtin_amdgcn_readfirstlane((int)(dst + i * 1024)));
        };
        auto issue_A = [&](int step, int buf) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 4; i++) issue_A1(step, buf, i);
        };
        auto issue_S = [&](int blk) __attribute__((always_inline)) {
            load16_to_lds(s_off, s_base + (int64_t)min(blk, nblk - 1) * 32,
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffS + wave * 1024)));
        };
        // code bytes of step `step`, columns 16 wave + lane / 2, half lane % 2 (lanes 0..31), into stage `stage`
        auto issue_Q = [&](int step, int stage) __attribute__((always_inline)) {
            const int st = min(step, ns - 1);
            if (lane < 32)
                load16_to_lds(q_off, w_base + (st >> 2) * Q4_K_BPB + 16 + 32 * (st & 3),
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffQ + stage * kQBuf + wave * 512)));
        };
        // block headers of super-block `blk`, columns 16 wave + lane (lanes 0..15), into stage blk % 2
        auto issue_H = [&](int blk) __attribute__((always_inline)) {
            if (lane < 16)
                load16_to_lds(h_off, w_base + min(blk, nblk - 1) * Q4_K_BPB,
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + kOffH + (blk & 1) * kHBuf + wave * 256)));
        };

        uint32_t cur_lo = 0, cur_hi = 0;
        // Header stage -> this thread's share of the column's table entries (decode_tables) and its scale pair, that of
        // chunk `upart`, in cur_lo / cur_hi (decode_scales).  Two parts, run in different phases: together they hold a
        // dozen registers at once, more than the phase that does the rest of the bookkeeping has to spare.
        // (Both recompute what they need of the thread's role from its index, behind an empty asm statement that keeps the
        // compiler from hoisting those values out of the loop into registers of their own: they are needed once in four steps.)
        auto role = [&](int& col, int& part) __attribute__((always_inline)) {
            int t = tid;
            asm volatile("" : "+v"(t));
            col = t >> 2;
            part = t & 3;
        };
        auto decode_tables = [&](int hstage) __attribute__((always_inline)) {
            int ucol, upart;
            role(ucol, upart);
            const int sh = 16 * (upart & 1);
            const bool upper = upart >= 2;
            const uint2 hdr = *(const uint2*)(smem + kOffH + hstage * kHBuf + ucol * 16);              // d, dmin, scale bytes 0..3
            const uint2 hdr2 = *(const uint2*)(smem + kOffH + hstage * kHBuf + ucol * 16 + 8);         // scale bytes 4..11
            const uint32_t p1 = (hdr2.x >> sh) & 0xffffu, p2 = (hdr2.y >> sh) & 0xffffu;
            const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
            const uint32_t ndm = ((hdr.x >> 16) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
            const uint32_t mp = pack_half2(cvt_ubyte0(mn_pair), cvt_ubyte1(mn_pair));
            const uint32_t hi = pk_mul(ndm, mp), lo = pk_fma(ndm, mp, hi ^ 0x80008000u);
            uint8_t* mt = smem + kOffM + ucol * 32 + upart * 4;
            *(uint32_t*)mt = hi;
            *(uint32_t*)(mt + 16) = lo;
            if (upart == 0) *(float*)(smem + kOffD + ucol * 4) = h2f((uint16_t)(hdr.x & 0xffffu)) * kTwo18f;
        };
        auto decode_scales = [&](int hstage) __attribute__((always_inline)) {
            int ucol, upart;
            role(ucol, upart);
            const int sh = 16 * (upart & 1);
            const bool upper = upart >= 2;
            const uint32_t s0 = *(const uint32_t*)(smem + kOffH + hstage * kHBuf + ucol * 16 + 4);     // scale bytes 0..3
            const uint32_t s2 = *(const uint32_t*)(smem + kOffH + hstage * kHBuf + ucol * 16 + 12);    // scale bytes 8..11
            const uint32_t p0 = (s0 >> sh) & 0xffffu, p2 = (s2 >> sh) & 0xffffu;
            const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
            // 64 sc for the low nibbles (q * 2^-24), 4 sc for the high ones (16 q * 2^-24): operand sc * q * 2^-18
            const float e0 = 64.0f * cvt_ubyte0(sc_pair), e1 = 4.0f * cvt_ubyte1(sc_pair);
            cur_lo = pack_half2(e0, e0);
            cur_hi = pack_half2(e1, e1);
        };
        auto decode = [&](int hstage) __attribute__((always_inline)) {
            decode_tables(hstage);
            decode_scales(hstage);
        };
        // 8 code bytes -> the low-nibble and the high-nibble piece of slice `upart`, in three parts that the phase
        // spreads between its matrix-core instructions: fetch (the bytes from their LDS stage, the scale pair of
        // chunk CN from quad lane CN), four quarters of arithmetic (two codes pairs each), store.
        uint2 uq = make_uint2(0, 0);
        uint32_t u_slo = 0, u_shi = 0;
        uint2 u_lo = make_uint2(0, 0), u_hi = make_uint2(0, 0);  // two quarters' worth: stored as 8-byte halves of the pieces
        auto unpack_fetch = [&](int qstage, uint32_t own_lo, uint32_t own_hi, auto CN) __attribute__((always_inline)) {
            constexpr int cn = decltype(CN)::value;
            uq = *(const uint2*)(smem + kOffQ + qstage * kQBuf + tid * 8);
            u_slo = quad_bcast<cn>(own_lo);
            u_shi = quad_bcast<cn>(own_hi);
        };
        auto unpack_quarter = [&](int i, int bbuf) __attribute__((always_inline)) {
            const uint32_t x = (i & 2) ? uq.y : uq.x;
            const uint32_t v = (i & 1) ? x >> 8 : x;
            const uint32_t lo = pk_mul(v & M1, u_slo), hi = pk_mul(v & M2, u_shi);
            if (i & 1) {
                u_lo.y = lo;
                u_hi.y = hi;
                *(uint2*)(smem + bw_lo + bbuf * kBBuf + (i >> 1) * 8) = u_lo;
                *(uint2*)(smem + ((bw_lo + bbuf * kBBuf) ^ 16u) + (i >> 1) * 8) = u_hi;
            } else {
                u_lo.x = lo;
                u_hi.x = hi;
            }
        };
        auto unpack = [&](int qstage, uint32_t own_lo, uint32_t own_hi, auto CN, int bbuf) __attribute__((always_inline)) {
            unpack_fetch(qstage, own_lo, own_hi, CN);
#pragma unroll
            for (int i = 0; i < 4; i++) unpack_quarter(i, bbuf);
        };

        float16v acc[2][2], P[2][2];
        const float16v zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};  // (an inline constant)
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
        issue_H(0);
        issue_S(0);
        issue_A(0, 0);
        issue_A(1, 1);
        issue_Q(0, 0);
        issue_Q(1, 1);
        issue_Q(2, 2);
        if (tid < TM) *(float*)(smem + kOffInv + tid * 4) = inv[min(m0 + tid, m - 1)];
        wait_vmcnt<0>();
        decode(0);  // (a wavefront decodes and unpacks only what it fetched itself: no barrier needed in between)
        issue_H(1);
        unpack(0, cur_lo, cur_hi, std::integral_constant<int, 0>{}, 0);
        int abuf = 0;  // lhs buffer of the current step (step % 3); also the stage its code bytes were in
        __syncthreads();

        auto read_frags = [&](int f, int slot, int ab, int bb) __attribute__((always_inline)) {
            const uint32_t ao = (uint32_t)(a_minus_b + ab * kABuf), bo = (uint32_t)(bb * kBBuf);
#pragma unroll
            for (int mi = 0; mi < 2; mi++) afr[slot][mi] = *(const half8*)(smem + (uint32_t)(((fb0 + ao) ^ (uint32_t)(f << 5)) + mi * 4096));
#pragma unroll
            for (int ni = 0; ni < 2; ni++) bfr[slot][ni] = *(const half8*)(smem + (uint32_t)(((fb0 + bo) ^ (uint32_t)(f << 5)) + ni * 4096));
        };
        // four matrix-core instructions of one slice; `between(i)` is placed after the i-th of them
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
        auto nothing = [](int) __attribute__((always_inline)) {};
        // acc += d * P for sub-tile t = 2 mi + ni
        auto rescale_tile = [&](int t, const float (&d)[2]) __attribute__((always_inline)) {
            const int mi = t >> 1, ni = t & 1;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[mi][ni][r] = fmaf(d[ni], P[mi][ni][r], acc[mi][ni][r]);
        };

        // One phase = from the barrier inside step s - 1 to the barrier inside step s.  The order of its parts is
        // pinned (sched_barrier): left to itself the compiler moves every operand read down to the instruction that
        // uses it, and the matrix cores then wait for the LDS once per slice.
        auto phase = [&](int blk, auto CC) __attribute__((always_inline)) {
            constexpr int c = decltype(CC)::value;
            const int s = blk * 4 + c;
            // first operands of step s, read under the last slice of step s - 1
            read_frags(0, 0, abuf, c & 1);
            __builtin_amdgcn_sched_barrier(0);
            // Refills: the buffers of step s - 1 are free (all their reads were issued before the barrier).  The
            // loads are spread over the phase, one behind each group of matrix-core instructions: a wavefront
            // waits at a load until the memory pipeline takes it (1 KB per instruction, about 16 cycles each, all
            // eight wavefronts at once), and with its matrix-core instructions already queued that wait costs nothing.
            const int ab2 = abuf == 0 ? 2 : abuf - 1;  // (step + 2) % 3
            const int ab1 = abuf == 2 ? 0 : abuf + 1;  // (step + 1) % 3
            if (s > 0) mfma_slice(1, false, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 0); });
            else issue_A1(s + 2, ab2, 0);
            issue_Q(s + 3, abuf);  // (the stage of step s: its bytes were unpacked one phase ago)
            // Header of super-block blk + 1 (fetched one super-block ago).  Phase 2: its tables (the current ones were last
            // read in phase 1; the sums likewise).  Phase 3: this thread's scale pair (that of the current super-block was
            // last used in phase 2, for chunk 3; the unpack of phase 3 makes chunk 0 of the next super-block).
            if constexpr (c == 2) {
                issue_S(blk + 1);
                decode_tables((blk + 1) & 1);
            }
            if constexpr (c == 3) {
                decode_scales((blk + 1) & 1);
                issue_H(blk + 2);
            }
            __builtin_amdgcn_sched_barrier(0);
            // The tables and sums of this super-block were written during the last one; they are rewritten in phase 2
            // (behind the barrier that ends phase 1).  Phase 0 takes d, phase 1 the min term.
            half8 sfr[2], mh, ml;
            if (c == 1 && with_min) {
#pragma unroll
                for (int mi = 0; mi < 2; mi++) sfr[mi] = *(const half8*)(smem + kOffS + (wm * 64 + mi * 32 + nl) * 32 + g * 16);
                mh = *(const half8*)(smem + kOffM + (wn * 64 + nl) * 32);
                ml = *(const half8*)(smem + kOffM + (wn * 64 + nl) * 32 + 16);
            }
            // next step's code bytes and scales
            if constexpr (c == 0) unpack_fetch(ab1, cur_lo, cur_hi, std::integral_constant<int, 1>{});
            else if constexpr (c == 1) unpack_fetch(ab1, cur_lo, cur_hi, std::integral_constant<int, 2>{});
            else if constexpr (c == 2) unpack_fetch(ab1, cur_lo, cur_hi, std::integral_constant<int, 3>{});
            else unpack_fetch(ab1, cur_lo, cur_hi, std::integral_constant<int, 0>{});
            __builtin_amdgcn_sched_barrier(0);
            // slice 0 (operands read at the top), while the operands of slice 1 arrive
            read_frags(1, 1, abuf, c & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (c == 0 && s > 0) {
                // Super-block blk - 1 is complete.  Its rescale runs sub-tile by sub-tile in front of the first
                // matrix-core instruction of the new super-block on the same sub-tile (which restarts P from zero):
                // the product that a rescale reads was finished four matrix-core instructions ago, so nothing drains.
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    rescale_tile(t, dcur);
                    __builtin_amdgcn_sched_barrier(0);
                    P[t >> 1][t & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t >> 1], bfr[0][t & 1], zero16, 0, 0, 0);
                    if (t == 3) issue_A1(s + 2, ab2, 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                mfma_slice(0, c == 0, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 1); });
            }
            if (c == 0) {  // d of the new super-block, for the rescale that ends it
#pragma unroll
                for (int ni = 0; ni < 2; ni++) dcur[ni] = *(const float*)(smem + kOffD + (wn * 64 + ni * 32 + nl) * 4);
            }
            if (c == 1 && with_min) {
                // min term: the hi products of the four sub-tiles first, then the lo ones (each pair is a dependent chain)
                // (the operands of the second column group are read while the first group's four products run)
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
            // slice 1, with the arithmetic of the unpack between its matrix-core instructions
            read_frags(2, 0, abuf, c & 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(1, false, [&](int i) __attribute__((always_inline)) {
                unpack_quarter(i, (c + 1) & 1);  // (the unpacked operands go to the other weight buffer)
                if (i == 3) issue_A1(s + 2, ab2, 2);
            });
            // slice 2
            read_frags(3, 1, abuf, c & 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_slice(0, false, [&](int i) __attribute__((always_inline)) { if (i == 3) issue_A1(s + 2, ab2, 3); });
            // everything issued before this phase has landed: the lhs of step s + 1, the code bytes of step s + 2
            if constexpr (c >= 2) wait_vmcnt<6>();
            else wait_vmcnt<5>();
            __syncthreads();
            abuf = abuf == 2 ? 0 : abuf + 1;
        };
        for (int blk = 0; blk < nblk; blk++) {
            phase(blk, std::integral_constant<int, 0>{});
            phase(blk, std::integral_constant<int, 1>{});
            phase(blk, std::integral_constant<int, 2>{});
            phase(blk, std::integral_constant<int, 3>{});
        }
        mfma_slice(1, false, nothing);  // last slice of the last step
#pragma unroll
        for (int t = 0; t < 4; t++) rescale_tile(t, dcur);

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
                        float* o_ = out + (int64_t)row * n;
                        const float v0 = acc[mi][0][r] * is, v1 = acc[mi][1][r] * is;
                        if (unit.half) {  // one of the two K halves of this tile: out holds zero or the other half
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

// Everything the GEMM needs done first, in one launch: workgroups [0, m) narrow one lhs row each; the rest zero the
// output tiles that the GEMM will fill with atomic adds of two K halves.
template <typename AT>
__global__ __launch_bounds__(256) void tile_prologue_kernel(const AT* __restrict__ a, int k, LhsPlanes p, SplitTiles z) {
    const int b = (int)blockIdx.x;
    if (b < z.m) {
        prep_lhs_row<AT, kLhsOrderTile>(b, a, k, p.a16, p.a16_lo, p.asum, p.inv);
    } else {
        const int e = b - z.m;
        zero_split_tile_part(z, e >> 6, (e >> 3) & 7, e & 7);
    }
}

bool gemm_q4_k_tile_wanted(int64_t m, int64_t n, int64_t k) {
    // QMM_Q4K_TILE=1 (read once) sends every prefill shape here, for tests of the kernel on small problems
    static const bool force = getenv("QMM_Q4K_TILE") != nullptr && atoi(getenv("QMM_Q4K_TILE")) == 1;
    if (k % 256 || k < 256 || kernel_disabled("q4k_tile")) return false;
    if (force) return m > 16;
    // (one round of tiles takes 72 .. 78 us at K = 4096 however many there are; the GEMM with 64-row tiles, microseconds
    // against this kernel's: 512 x 14336, 224 tiles, 86.5 / 78.5; 512 x 11008, 172 tiles, 80.5 / 72.5; 768 x 8192, 192 tiles,
    // 80.5 / 73.8; 512 x 8192, 128 tiles, 57.8 / 71.9)
    const int64_t tiles = ((m + TM - 1) / TM) * ((n + TN - 1) / TN);
    return m > 128 && tiles >= 160;
}

int64_t gemm_q4_k_tile_workspace_bytes(int lhs_dtype, int64_t m, int64_t k) { return lhs_planes(nullptr, lhs_dtype, m, k, TM).bytes; }

hipError_t launch_gemm_q4_k_tile(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out,
                                 void* workspace, hipStream_t s) {
    const LhsPlanes p = lhs_planes(workspace, lhs_dtype, m, k, TM);
    hipError_t e = allow_full_lds<gemm_q4_k_tile_kernel>();
    if (e != hipSuccess) return e;
    const int tiles_m = (int)((m + TM - 1) / TM), tiles_n = (int)((n + TN - 1) / TN);
    const int total = tiles_m * tiles_n, per_xcd = (total + 7) / 8;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const int wg = 8 * std::min(per_xcd, std::max(1, cus / 8));  // persistent: one workgroup per compute unit
    // the tiles of a last, at most half-full round are cut in two along K (see TileUnit): their outputs start from zero
    const SplitTiles z = split_tiles(out, m, n, tiles_m, tiles_n, (int)(k / 256), wg);
    const int max_split = z.max_split;
    const dim3 pgrid((unsigned)(m + (int64_t)max_split * 64));
    if (lhs_dtype == QMM_F32) tile_prologue_kernel<float><<<pgrid, dim3(256), 0, s>>>((const float*)lhs, (int)k, p, z);
    else tile_prologue_kernel<uint16_t><<<pgrid, dim3(256), 0, s>>>((const uint16_t*)lhs, (int)k, p, z);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    gemm_q4_k_tile_kernel<<<dim3((unsigned)wg), dim3(512), kTileLds, s>>>(w, p.a16, p.asum, p.inv, out, (int)m, (int)n, (int)k, tiles_m,
                                                                          tiles_n, 1, 0, max_split > 0 ? 1 : 0);
    if (p.a16_lo)  // fp32 lhs: the residual plane, added on top (whole tiles only: every element gets one more term, in a fixed order)
        gemm_q4_k_tile_kernel<<<dim3((unsigned)wg), dim3(512), kTileLds, s>>>(w, p.a16_lo, p.asum, p.inv, out, (int)m, (int)n, (int)k,
                                                                              tiles_m, tiles_n, 0, 1, 0);
    return hipGetLastError();
}

}  // namespace qmm
