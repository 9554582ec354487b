// Q4_K decode kernel for one or two lhs rows: every lane owns one fixed 64-column chunk of K, so its
// activations never leave its registers; weight rows travel global -> LDS directly.
//
// A wavefront covers up to 16 super-blocks of a row (4096 columns): lane l owns chunk l % 4 of
// super-block l / 4, i.e. 32 code bytes whose low nibbles are sub-block 2c and whose high nibbles are
// sub-block 2c + 1, and needs only those two scales and mins.  Longer rows are cut into 2 or 4
// parts, one wavefront each (K = 14336: 4 parts of 14 super-blocks), and the partial sums of a row
// are added through LDS at the end.  The 64 activations of the lane's chunk (and their two sums, for
// the min term) are read once, from a copy of the lhs that the workgroup stages in LDS at the start.
//
// A wavefront walks its rows (persistent); a row part goes as 16-byte pieces straight into a
// private ring of three LDS slots (global_load_lds_dwordx4, two rows ahead, hidden from the
// compiler and waited for with exact vmcnt counts: lds_stream.h).  Per row a lane issues three
// 16-byte LDS reads (header, 32 code bytes), masks the nibbles in place into fp16 subnormals
// (q * 2^-24, or 16 q * 2^-24 for the high ones) and multiplies them by its fp32 activations with
// v_fma_mix_f32; d * sc and dmin * mn are applied once per chunk.  Against the streaming kernel
// (8 lanes per super-block, activations from LDS) this is about 150 instead of 235 vector
// instructions per 2304-byte row, which is what bounds both.
//
// Up to four matrices that share the lhs go through one launch (rows numbered through the matrices).  In
// the gated-pair mode (two matrices of equal size: gate, up) a row stream walks gate row r, up row r, gate
// row r + GS, ... and the epilogue stores silu(gate) * up, one output row per pair.
#include <stdlib.h>

#include <algorithm>

#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int kWaves = 8;     // wavefronts per workgroup
constexpr int kMaxRows = 64;  // rows a wavefront may own (LDS result slots)

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ half2v as_half2(uint32_t u) { return __builtin_bit_cast(half2v, u); }

__device__ __forceinline__ float ubyte0(uint32_t v) { float f; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ubyte1(uint32_t v) { float f; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v)); return f; }

}  // namespace

// WPR: wavefronts (parts of K) per row.  L: load instructions per row part (64 pieces of 16 bytes each).
// ring: LDS slots per wavefront (2..4): one row part being decoded, the others in flight.
// mats: up to kLanesMaxMats weight matrices that share the lhs and K; their rows are numbered through
// (matrix j owns rows [end[j - 1], end[j])), so one launch serves q|k|v or gate|up.
// HALF: a lane owns one 32-column sub-block instead of a 64-column chunk (lane l: super-block l / 8, chunk (l / 2) % 4, low nibbles
// for even l, high nibbles for odd l), which halves the activations a lane keeps per lhs row and so makes room for four lhs
// rows; a wavefront then covers 8 super-blocks, a row of 4096 columns takes two wavefronts (WPR up to 8, parts of up to 8).
// PLAIN: one matrix, one lhs row, no pairing, two ring slots, all known at compile time: the row-to-matrix lookup, the
// pair walk and the run-time slot arithmetic fall away, which shortens the scalar code in front of the first loads (a
// launch spends its first microsecond there; the weights of a short launch arrive that much later).
template <int MT, int WPR, int L, typename AT, bool HALF, bool PLAIN>
__device__ __forceinline__ void lanes_body(const LanesMats& mats, const AT* __restrict__ a, int m, int k, int64_t ldo, int ring_slots,
                                           int streams, int rows_each, int rows_extra) {
    // One matrix (the plain call) needs nothing from the argument block per row.  With several, the row's matrix is
    // looked up in the block: a dependent scalar load per row, a round trip to memory while the scalar cache is
    // cold, which a short launch cannot hide; the grouped launches are long enough.
    const bool single = PLAIN || mats.count == 1;
    const uint8_t* const w0 = mats.w[0];
    float* const o0 = mats.out[0];
    const int e0 = mats.end[0];
    const int n = mats.end[kLanesMaxMats - 1];  // (entries past count repeat the last one)
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int part = wave % WPR;
    const int bpw = (nblk + WPR - 1) / WPR;                       // super-blocks per part (<= 16)
    const int blk0 = min(part * bpw, nblk - 1);
    const int nb = max(0, min(bpw, nblk - part * bpw));           // super-blocks of this part
    const int kRing = PLAIN ? 2 : ring_slots;
    const int pieces = bpw * 9;       // 16-byte pieces of a full row part
    const int kSlot = pieces * 16;    // bytes of a slot
    uint8_t* ring = smem + wave * (kRing * kSlot);
    const uint32_t ring_lds = lds_address(ring);
    float* res = (float*)(smem + kWaves * kRing * kSlot) + wave * kMaxRows * MT;
    const int gs = (int)blockIdx.x * (kWaves / WPR) + wave / WPR, GS = streams;  // streams = workgroups * kWaves / WPR
    // Rows of this row stream.  Plain: gs, gs + GS, ...  Gated pair (mats.swiglu): the stream owns the row PAIRS
    // gs, gs + GS, ... and walks gate row, up row, gate row, ...: both results of a pair end up in its own slots.
    const bool paired = !PLAIN && mats.swiglu != 0;
    const int np = paired ? e0 : n;
    // rows (or pairs) of this stream: np / GS, one more for the first np % GS streams (the host did the division)
    const int my_rows = (rows_each + (gs < rows_extra ? 1 : 0)) * (paired ? 2 : 1);
    auto row_of = [&](int ri) __attribute__((always_inline)) { return paired ? (ri & 1) * np + gs + (ri >> 1) * GS : gs + ri * GS; };

    // a row part into a slot.  Every one of the L instructions has a live lane in every wavefront (the mask
    // follows the full part length, a shorter last part repeats its last piece), so the wait counts stay exact.
    const int last_piece = max(nb, 1) * 9 - 1;
    auto issue = [&](int ri, int slot) __attribute__((always_inline)) {
        const int row = row_of(ri);
        const uint8_t* wp = w0;
        int local = row;
        if (!single) {
            int j = 0;
            while (j + 1 < mats.count && row >= mats.end[j]) j++;  // (uniform: a few scalar compares)
            local = row - (j ? mats.end[j - 1] : 0);
            wp = mats.w[j];
        }
        const uint8_t* base = wp + (int64_t)local * row_bytes + (int64_t)blk0 * Q4_K_BPB;
#pragma unroll
        for (int i = 0; i < L; i++)
            if (lane + 64 * i < pieces)
                load16_to_lds_once(base + 16 * min(lane + 64 * i, last_piece),
                              (uint32_t)__builtin_amdgcn_readfirstlane((int)(ring_lds + slot * kSlot + i * 1024)));  // (uniform; says so)
    };

    // --- the lane's chunk: super-block blk0 + lane / 4 (clamped: lanes past the part repeat its last super-block; their sum is dropped),
    //     chunk c = lane % 4.  The lhs rows are staged once per workgroup: coalesced 16-byte pieces straight
    //     into LDS, laid out as one record per 64-column chunk (its pieces plus one piece of padding, so that
    //     the lanes' 16-byte reads of their own records spread over the banks), issued before the first weight
    //     rows and waited for together with them.
    const int lsb = HALF ? lane >> 3 : lane >> 2;  // this lane's super-block of the part
    const int lb = min(lsb, max(nb, 1) - 1), c = HALF ? (lane >> 1) & 3 : lane & 3;
    const int hn = lane & 1;  // (HALF) 0: the low nibbles, sub-block 2 c; 1: the high nibbles, sub-block 2 c + 1
    const bool live = lsb < nb;
    constexpr int kCp = sizeof(AT) == 4 ? 16 : 8;  // 16-byte pieces of a chunk's 64 activations
    uint8_t* act = smem + kWaves * kRing * kSlot + kWaves * kMaxRows * MT * 4;
    const int nchunk = k >> 6, npos = nchunk * (kCp + 1);  // records, and their pieces (padding included)
    const int nposp = (npos + 63) & ~63;                   // per lhs row, rounded up to whole load instructions
    {
        const uint32_t act_lds = lds_address(act);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const uint8_t* ar = (const uint8_t*)(a + (int64_t)min(mi, m - 1) * k);
            for (int q0 = wave * 64; q0 < npos; q0 += 64 * kWaves) {
                const int q = min(q0 + lane, npos - 1);
                const int owner = q / (kCp + 1), slot = q - owner * (kCp + 1);
                load16_to_lds(ar + 16 * (owner * kCp + min(slot, kCp - 1)), act_lds + (mi * nposp + q0) * 16);
            }
        }
    }
    int issued = 0;
    int islot = 0;  // slot of the next row to issue
    for (; issued < min(kRing - 1, my_rows); issued++) {
        issue(issued, islot);
        islot = islot + 1 == kRing ? 0 : islot + 1;
    }
    wait_items<L, 0>(issued, false);  // the activation loads are older than these rows
    __syncthreads();                  // every wavefront's share of the activations has landed
    constexpr int kAh = HALF ? 1 : 32;  // (HALF keeps one 32-value set per lhs row, in alo)
    float alo[MT][32], ahi[MT][kAh], slo_a[MT], shi_a[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        float v[64];
        const uint4* rec = (const uint4*)(act + ((size_t)mi * nposp + (size_t)((blk0 + lb) * 4 + c) * (kCp + 1)) * 16);
        if constexpr (HALF) {
            // this lane's half of the record: pieces [hn * kCp / 2, (hn + 1) * kCp / 2)
            constexpr int kHp = kCp / 2;
#pragma unroll
            for (int i = 0; i < kHp; i++) {
                const uint4 r = rec[hn * kHp + i];
                if constexpr (sizeof(AT) == 4) {
                    v[4 * i] = __uint_as_float(r.x); v[4 * i + 1] = __uint_as_float(r.y);
                    v[4 * i + 2] = __uint_as_float(r.z); v[4 * i + 3] = __uint_as_float(r.w);
                } else {
                    v[8 * i] = __uint_as_float(r.x << 16); v[8 * i + 1] = __uint_as_float(r.x & 0xffff0000u);
                    v[8 * i + 2] = __uint_as_float(r.y << 16); v[8 * i + 3] = __uint_as_float(r.y & 0xffff0000u);
                    v[8 * i + 4] = __uint_as_float(r.z << 16); v[8 * i + 5] = __uint_as_float(r.z & 0xffff0000u);
                    v[8 * i + 6] = __uint_as_float(r.w << 16); v[8 * i + 7] = __uint_as_float(r.w & 0xffff0000u);
                }
            }
            float s0 = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; i++) alo[mi][i] = v[i];
#pragma unroll
            for (int i = 0; i < 32; i += 4) s0 += (alo[mi][i] + alo[mi][i + 1]) + (alo[mi][i + 2] + alo[mi][i + 3]);
            slo_a[mi] = s0;
            shi_a[mi] = 0.0f;
            ahi[mi][0] = 0.0f;
            continue;
        }
#pragma unroll
        for (int i = 0; i < kCp; i++) {
            const uint4 r = rec[i];
            if constexpr (sizeof(AT) == 4) {
                v[4 * i] = __uint_as_float(r.x); v[4 * i + 1] = __uint_as_float(r.y);
                v[4 * i + 2] = __uint_as_float(r.z); v[4 * i + 3] = __uint_as_float(r.w);
            } else {
                v[8 * i] = __uint_as_float(r.x << 16); v[8 * i + 1] = __uint_as_float(r.x & 0xffff0000u);
                v[8 * i + 2] = __uint_as_float(r.y << 16); v[8 * i + 3] = __uint_as_float(r.y & 0xffff0000u);
                v[8 * i + 4] = __uint_as_float(r.z << 16); v[8 * i + 5] = __uint_as_float(r.z & 0xffff0000u);
                v[8 * i + 6] = __uint_as_float(r.w << 16); v[8 * i + 7] = __uint_as_float(r.w & 0xffff0000u);
            }
        }
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; i++) {
            alo[mi][i] = v[i];
            ahi[mi][i] = v[32 + i];
        }
#pragma unroll
        for (int i = 0; i < 32; i += 4) {
            s0 += (alo[mi][i] + alo[mi][i + 1]) + (alo[mi][i + 2] + alo[mi][i + 3]);
            s1 += (ahi[mi][i] + ahi[mi][i + 1]) + (ahi[mi][i + 2] + ahi[mi][i + 3]);
        }
        slo_a[mi] = s0;
        shi_a[mi] = s1;
    }
    const int sh = 16 * (c & 1);  // byte pair (2c, 2c + 1) mod 4 inside a dword of the 6-bit fields
    const bool upper = c >= 2;    // sub-blocks 4..7 use the split encoding

    int cslot = 0;  // slot of the row being decoded
    for (int ri = 0; ri < my_rows; ri++) {
        // the slot of row ri - 1 is free (its reads fed the sum that was parked): refill it
        if (issued < my_rows) {
            issue(issued, islot);
            islot = islot + 1 == kRing ? 0 : islot + 1;
            issued++;
        }
        wait_items<L, 0>(issued - 1 - ri, false);
        const uint8_t* blk = ring + cslot * kSlot + lb * Q4_K_BPB;
        cslot = cslot + 1 == kRing ? 0 : cslot + 1;
        const uint4 hdr = *(const uint4*)blk;
        const uint4 q0 = *(const uint4*)(blk + 16 + 32 * c), q1 = *(const uint4*)(blk + 32 + 32 * c);
        const uint32_t qd[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        float slo[MT], shi[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) slo[mi] = shi[mi] = 0.0f;
        if constexpr (HALF) {
            const int nsh = 4 * hn;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                // this lane's nibbles moved to the low position: q * 2^-24 as fp16 subnormals, as below
                const uint32_t x = qd[i] >> nsh;
                const half2v l02 = as_half2(x & 0x000F000Fu), l13 = as_half2((x >> 8) & 0x000F000Fu);
                const float w0 = (float)l02.x, w1 = (float)l13.x, w2 = (float)l02.y, w3 = (float)l13.y;
#pragma unroll
                for (int mi = 0; mi < MT; mi++) {
                    float t = slo[mi];
                    t = fmaf(alo[mi][4 * i], w0, t);
                    t = fmaf(alo[mi][4 * i + 1], w1, t);
                    t = fmaf(alo[mi][4 * i + 2], w2, t);
                    slo[mi] = fmaf(alo[mi][4 * i + 3], w3, t);
                }
            }
        } else
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // a masked nibble in a 16-bit half is the fp16 subnormal q * 2^-24 (low nibbles) or 16 q * 2^-24 (high
            // nibbles, left in place); the fused multiply-add widens the half itself
            const uint32_t y = qd[i] >> 8;
            const half2v l02 = as_half2(qd[i] & 0x000F000Fu), l13 = as_half2(y & 0x000F000Fu);
            const half2v h02 = as_half2(qd[i] & 0x00F000F0u), h13 = as_half2(y & 0x00F000F0u);
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                float t = slo[mi];
                t = fmaf(alo[mi][4 * i], (float)l02.x, t);
                t = fmaf(alo[mi][4 * i + 1], (float)l13.x, t);
                t = fmaf(alo[mi][4 * i + 2], (float)l02.y, t);
                slo[mi] = fmaf(alo[mi][4 * i + 3], (float)l13.y, t);
                t = shi[mi];
                t = fmaf(ahi[mi][4 * i], (float)h02.x, t);
                t = fmaf(ahi[mi][4 * i + 1], (float)h13.x, t);
                t = fmaf(ahi[mi][4 * i + 2], (float)h02.y, t);
                shi[mi] = fmaf(ahi[mi][4 * i + 3], (float)h13.y, t);
            }
        }
        const float d = h2f((uint16_t)(hdr.x & 0xffffu)), dmin = h2f((uint16_t)(hdr.x >> 16));
        const uint32_t p0 = (hdr.y >> sh) & 0xffffu, p1 = (hdr.z >> sh) & 0xffffu, p2 = (hdr.w >> sh) & 0xffffu;
        const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
        const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
        float d1 = d * ubyte0(sc_pair) * 16777216.0f, d2 = d * ubyte1(sc_pair) * 1048576.0f;  // 2^24, 2^24 / 16
        float m1 = dmin * ubyte0(mn_pair), m2 = dmin * ubyte1(mn_pair);
        if constexpr (HALF) {  // one sub-block per lane: its scale and min; nibbles sit in the low position either way
            d1 = hn ? d * ubyte1(sc_pair) * 16777216.0f : d1;
            m1 = hn ? m2 : m1;
            d2 = 0.0f;
            m2 = 0.0f;
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            float t = d1 * slo[mi];
            t = fmaf(-m1, slo_a[mi], t);
            t = fmaf(d2, shi[mi], t);
            t = fmaf(-m2, shi_a[mi], t);
            t = live ? t : 0.0f;  // lanes past the part decoded its last super-block again (valid data): dropped here
            const float v = wave_sum_dpp_lane63(t);
            if (lane == 63) res[ri * MT + mi] = v;
        }
    }
    auto store_row = [&](int mi, int row, float v) __attribute__((always_inline)) {
        float* op = o0;
        int local = row, nj = e0;
        if (!single) {
            int j = 0;
            while (j + 1 < mats.count && row >= mats.end[j]) j++;
            local = row - (j ? mats.end[j - 1] : 0);
            nj = mats.end[j] - (j ? mats.end[j - 1] : 0);
            op = mats.out[j];
        }
        const int64_t at = (int64_t)mi * (ldo ? ldo : nj) + local;
        if (mats.out_bf16) ((uint16_t*)op)[at] = f2bf(v);
        else op[at] = v;
    };
    // result slot idx of this stream, the K parts added
    auto result = [&](int idx) __attribute__((always_inline)) {
        float v = res[idx];
#pragma unroll
        for (int q = 1; q < WPR; q++) v += res[q * kMaxRows * MT + idx];
        return v;
    };
    if constexpr (WPR > 1) __syncthreads();
    if (WPR == 1 || part == 0) {
        if (paired) {
            // (one lhs row) out[pair] = silu(gate) * up, silu(x) = x / (1 + exp(-x))
            for (int idx = lane; idx < my_rows / 2; idx += 64) {
                const float g = result(2 * idx), u = result(2 * idx + 1);
                const float v = g / (1.0f + expf(-g)) * u;
                if (mats.out_bf16) ((uint16_t*)o0)[gs + idx * GS] = f2bf(v);
                else o0[gs + idx * GS] = v;
            }
        } else {
            for (int idx = lane; idx < my_rows * MT; idx += 64) {
                const int r = idx / MT, mi = idx - r * MT;
                if (mi < m) store_row(mi, gs + r * GS, result(idx));
            }
        }
    }
}

template <int MT, int WPR, int L, typename AT, bool HALF>
__global__ __launch_bounds__(64 * kWaves, MT == 1 ? 4 : 2) void gemv_q4_k_lanes_kernel(const LanesMats mats, const AT* __restrict__ a,
                                                                        int m, int k, int64_t ldo, int ring_slots,
                                                                        int streams, int rows_each, int rows_extra) {
    lanes_body<MT, WPR, L, AT, HALF, false>(mats, a, m, k, ldo, ring_slots, streams, rows_each, rows_extra);
}

// The plain call: one matrix [n, k], one lhs row, dense fp32 or bf16 output.  Twelve dwords of arguments.
template <int WPR, int L, typename AT>
__global__ __launch_bounds__(64 * kWaves, 4) void gemv_q4_k_lanes_plain_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                                               float* __restrict__ out, int n, int k, int out_bf16,
                                                                               int streams, int rows_each, int rows_extra) {
    // every argument is fetched in the first batch of scalar loads (left alone, the compiler fetches a pointer where it is first
    // used: another round trip in front of the loads that need it)
    asm volatile("" ::"s"(w), "s"(a), "s"(out), "s"(k), "s"(streams), "s"(rows_each), "s"(rows_extra));
    LanesMats mats;
#pragma unroll
    for (int j = 0; j < kLanesMaxMats; j++) {
        mats.w[j] = w;
        mats.out[j] = out;
        mats.end[j] = n;
    }
    mats.count = 1;
    mats.swiglu = 0;
    mats.out_bf16 = out_bf16;
    lanes_body<1, WPR, L, AT, false, true>(mats, a, 1, k, 0, 2, streams, rows_each, rows_extra);
}

// Takes K <= 16384 and m = 1 (reports other shapes through *handled = false).  count matrices [n[j], k] share the
// lhs; out[j] is fp32 [m, n[j]] (ldo = 0: dense; a single matrix may give its own leading dimension).
hipError_t launch_gemv_q4_k_lanes_grouped(const void* a, int a_dtype, int count, const uint8_t* const* ws, const int64_t* ns,
                                          float* const* outs, int m, int64_t k, int64_t ldo, hipStream_t s, bool* handled,
                                          bool swiglu, bool out_bf16) {
    *handled = false;
    if (swiglu && (count != 2 || ns[0] != ns[1] || m != 1)) return hipSuccess;
    const bool off = kernel_disabled("q4k_lanes");
    const int nblk = (int)(k / 256);
    if (off || m > 1 || nblk > 128 || count < 1 || count > kLanesMaxMats) return hipSuccess;  // (two lhs rows: the small-batch matrix-core kernel is faster)
    LanesMats mats;
    int64_t n = 0;
    for (int j = 0; j < kLanesMaxMats; j++) {
        const int jj = j < count ? j : count - 1;
        if (j < count) n += ns[j];
        mats.w[j] = ws[jj];
        mats.out[j] = outs[jj];
        mats.end[j] = (int)n;
    }
    mats.count = count;
    mats.swiglu = swiglu ? 1 : 0;
    mats.out_bf16 = out_bf16 ? 1 : 0;
    if (n > 0x7fffffff) return hipSuccess;
    const int wpr = nblk <= 16 ? 1 : nblk <= 32 ? 2 : nblk <= 64 ? 4 : 8;  // (8: the whole workgroup on one row at a time, K up to 32768)
    const int bpw = (nblk + wpr - 1) / wpr;
    const int l = (bpw * 9 + 63) / 64;  // 1..3
    const int mt = m <= 1 ? 1 : 2;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const size_t esz = a_dtype == QMM_F32 ? 4 : 2;
    // staged lhs rows: one padded record per chunk, each row rounded up to whole load instructions (1 KB)
    const size_t act_bytes = (size_t)mt * (((size_t)(k / 64) * (64 * esz + 16) + 1023) / 1024 * 1024);
    const size_t fixed = (size_t)kWaves * kMaxRows * mt * 4 + act_bytes, slot = (size_t)bpw * Q4_K_BPB;
    // Two slots (one row part in flight per wavefront while it decodes the other) and one workgroup per compute
    // unit; two workgroups per compute unit where a row stream is long (16 rows or more) and both fit the LDS.
    // Measured over (2..4 slots) x (1, 2 workgroups per compute unit), weight loads non-temporal: more slots
    // never help (14336 x 4096: 7.9 / 8.1 / 8.4 us with 2 / 3 / 4; 196608 x 4096: 85 / 91 / 93 us), the second
    // workgroup takes the 453 MB tensor from 85 to 75 us (6.05 TB/s) and costs the short launches up to 20 %.
    const int ring = 2;
    const size_t lds = (size_t)kWaves * ring * slot + fixed;
    if (lds > (size_t)kLdsPerCu) return hipSuccess;
    const int streams = kWaves / wpr;  // rows in progress per workgroup
    const int64_t units = swiglu ? n / 2 : n;  // rows, or gate / up row pairs, to deal to the streams
    const int per_cu = (units >= (int64_t)16 * cus * streams && 2 * lds + 2048 <= (size_t)kLdsPerCu ? 2 : 1);
    int64_t wgs = (int64_t)cus * per_cu;
    if (wgs * streams > units) wgs = (units + streams - 1) / streams;
    const int64_t min_wgs = (n + (int64_t)streams * kMaxRows - 1) / ((int64_t)streams * kMaxRows);
    if (wgs < min_wgs) wgs = min_wgs;  // no wavefront owns more rows than it has result slots
    dim3 grid((unsigned)wgs), block(64 * kWaves);
    const int total_streams = (int)wgs * streams;
    const bool plain = count == 1 && !swiglu && (ldo == 0 || ldo == ns[0]) && !kernel_disabled("q4k_lanes_plain");
#define QMM_GO3(MT_, WPR_, L_, AT_)                                                                                   \
    do {                                                                                                              \
        if (plain) {                                                                                                  \
            hipError_t e_ = allow_full_lds<gemv_q4_k_lanes_plain_kernel<WPR_, L_, AT_>>();                            \
            if (e_ != hipSuccess) return e_;                                                                          \
            gemv_q4_k_lanes_plain_kernel<WPR_, L_, AT_><<<grid, block, lds, s>>>(ws[0], (const AT_*)a, outs[0], (int)n, (int)k,  \
                                                                                 out_bf16 ? 1 : 0, total_streams,     \
                                                                                 (int)(units / total_streams),       \
                                                                                 (int)(units % total_streams));      \
            break;                                                                                                    \
        }                                                                                                             \
        hipError_t e_ = allow_full_lds<gemv_q4_k_lanes_kernel<MT_, WPR_, L_, AT_, false>>();                         \
        if (e_ != hipSuccess) return e_;                                                                              \
        gemv_q4_k_lanes_kernel<MT_, WPR_, L_, AT_, false><<<grid, block, lds, s>>>(mats, (const AT_*)a, m, (int)k, ldo, ring, \
                                                                            total_streams, (int)(units / total_streams), \
                                                                            (int)(units % total_streams));           \
    } while (0)
#define QMM_GO2(MT_, WPR_, L_)                            \
    do {                                                  \
        if (a_dtype == QMM_F32) QMM_GO3(MT_, WPR_, L_, float); \
        else QMM_GO3(MT_, WPR_, L_, uint16_t);            \
    } while (0)
#define QMM_GO1(WPR_, L_) QMM_GO2(1, WPR_, L_)
#define QMM_GO0(WPR_)               \
    do {                            \
        if (l == 1) QMM_GO1(WPR_, 1); \
        else if (l == 2) QMM_GO1(WPR_, 2); \
        else QMM_GO1(WPR_, 3);      \
    } while (0)
    if (wpr == 1) QMM_GO0(1);
    else if (wpr == 2) QMM_GO0(2);
    else if (wpr == 4) QMM_GO0(4);
    else QMM_GO0(8);
#undef QMM_GO0
#undef QMM_GO1
#undef QMM_GO2
#undef QMM_GO3
    *handled = true;
    return hipGetLastError();
}

// Two to four lhs rows with the sub-block-per-lane mapping (HALF): count matrices that share the lhs, K <= 16384; out[j] is
// fp32 [m, n[j]] (ldo = 0: dense).  Four rows need their activations staged in LDS four times over; where that does not
// fit (K > 8192 with an fp32 lhs) the rows go in two passes of two.
hipError_t launch_gemv_q4_k_lanes_rows_grouped(const void* a, int a_dtype, int count, const uint8_t* const* ws, const int64_t* ns,
                                               float* const* outs, int m, int64_t k, int64_t ldo, hipStream_t s, bool* handled) {
    *handled = false;
    const int nblk = (int)(k / 256);
    if (kernel_disabled("q4k_lanes_rows") || m < 2 || m > 4 || k % 256 || nblk > 64 || count < 1 || count > kLanesMaxMats) return hipSuccess;
    int64_t n = 0;
    for (int j = 0; j < count; j++) n += ns[j];
    if (n > 0x7fffffff) return hipSuccess;
    const size_t esz = a_dtype == QMM_F32 ? 4 : 2;
    const int wpr = nblk <= 8 ? 1 : nblk <= 16 ? 2 : nblk <= 32 ? 4 : 8;
    const int bpw = (nblk + wpr - 1) / wpr;  // <= 8
    const int l = (bpw * 9 + 63) / 64;       // 1 or 2
    const int ring = 2;
    const size_t slot = (size_t)bpw * Q4_K_BPB;
    auto lds_for = [&](int mt) {
        const size_t act_bytes = (size_t)mt * (((size_t)(k / 64) * (64 * esz + 16) + 1023) / 1024 * 1024);
        return (size_t)kWaves * ring * slot + (size_t)kWaves * kMaxRows * mt * 4 + act_bytes;
    };
    int mt = m <= 2 ? 2 : 4;
    if (lds_for(mt) > (size_t)kLdsPerCu) mt = 2;
    if (lds_for(mt) > (size_t)kLdsPerCu) return hipSuccess;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const size_t lds = lds_for(mt);
    const int streams = kWaves / wpr;
    int64_t wgs = cus;
    if (wgs * streams > n) wgs = (n + streams - 1) / streams;
    const int64_t min_wgs = (n + (int64_t)streams * kMaxRows - 1) / ((int64_t)streams * kMaxRows);
    if (wgs < min_wgs) wgs = min_wgs;  // no wavefront owns more rows than it has result slots
    const dim3 grid((unsigned)wgs), block(64 * kWaves);
    const int total_streams = (int)wgs * streams;
    for (int m0 = 0; m0 < m; m0 += mt) {
        const int rows = std::min(mt, m - m0);
        LanesMats mats;
        int64_t end = 0;
        for (int j = 0; j < kLanesMaxMats; j++) {
            const int jj = j < count ? j : count - 1;
            if (j < count) end += ns[j];
            mats.w[j] = ws[jj];
            mats.out[j] = outs[jj] + (int64_t)m0 * (ldo ? ldo : ns[jj]);
            mats.end[j] = (int)end;
        }
        mats.count = count;
        mats.swiglu = 0;
        mats.out_bf16 = 0;
        const void* am = (const char*)a + (size_t)m0 * k * esz;
#define QMM_H3(MT_, WPR_, L_, AT_)                                                                                                  \
    do {                                                                                                                            \
        hipError_t e_ = allow_full_lds<gemv_q4_k_lanes_kernel<MT_, WPR_, L_, AT_, true>>();                                         \
        if (e_ != hipSuccess) return e_;                                                                                            \
        gemv_q4_k_lanes_kernel<MT_, WPR_, L_, AT_, true><<<grid, block, lds, s>>>(mats, (const AT_*)am, rows, (int)k, ldo, ring,    \
                                                                                  total_streams, (int)(n / total_streams),         \
                                                                                  (int)(n % total_streams));                       \
    } while (0)
#define QMM_H2(MT_, WPR_, L_)                               \
    do {                                                    \
        if (a_dtype == QMM_F32) QMM_H3(MT_, WPR_, L_, float); \
        else QMM_H3(MT_, WPR_, L_, uint16_t);               \
    } while (0)
#define QMM_H1(MT_, WPR_)              \
    do {                               \
        if (l == 1) QMM_H2(MT_, WPR_, 1); \
        else QMM_H2(MT_, WPR_, 2);     \
    } while (0)
#define QMM_H0(MT_)                    \
    do {                               \
        if (wpr == 1) QMM_H1(MT_, 1);  \
        else if (wpr == 2) QMM_H1(MT_, 2); \
        else if (wpr == 4) QMM_H1(MT_, 4); \
        else QMM_H1(MT_, 8);           \
    } while (0)
        if (mt == 2) QMM_H0(2);
        else QMM_H0(4);
#undef QMM_H0
#undef QMM_H1
#undef QMM_H2
#undef QMM_H3
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    *handled = true;
    return hipSuccess;
}

// The gated-MLP combination as a kernel of its own, for the shapes the fused epilogue above does not take.
__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                     float* __restrict__ out, int64_t count) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const float g = gate[i];
        out[i] = g / (1.0f + expf(-g)) * up[i];
    }
}

hipError_t launch_swiglu(const float* gate, const float* up, float* out, int64_t count, hipStream_t s) {
    const int64_t blocks = std::min<int64_t>((count + 255) / 256, 4096);
    swiglu_kernel<<<dim3((unsigned)std::max<int64_t>(blocks, 1)), dim3(256), 0, s>>>(gate, up, out, count);
    return hipGetLastError();
}

hipError_t launch_gemv_q4_k_lanes_rows(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                       int64_t ldo, hipStream_t s, bool* handled) {
    return launch_gemv_q4_k_lanes_rows_grouped(a, a_dtype, 1, &w, &n, &out, m, k, ldo, s, handled);
}

hipError_t launch_gemv_q4_k_lanes(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                  int64_t ldo, hipStream_t s, bool* handled, bool out_bf16) {
    return launch_gemv_q4_k_lanes_grouped(a, a_dtype, 1, &w, &n, &out, m, k, ldo, s, handled, false, out_bf16);
}

}  // namespace qmm
