// Q4_0 decode kernel (m <= 4 lhs rows, K <= 8192; one lhs row: K up to 14528): weight rows streamed global -> LDS with 16-byte loads, the
// Q8_0 quantisation of the lhs done in the kernel, v_dot4_i32_i8 block dots.
//
// A Q4_0 block is 18 bytes (fp16 d, 16 bytes of nibbles), so blocks are only 2-byte aligned.  A
// wavefront owns whole weight rows (persistent: rows gw, gw + GW, ...).  A row travels as aligned
// 16-byte pieces straight into a wavefront-private ring of LDS slots (global_load_lds_dwordx4, up
// to three rows ahead of the one being decoded; the loads are hidden from the compiler and waited
// for with exact vmcnt counts, see gemv_q4k_mm.hip).  Lane l decodes blocks l, l + 64, ... of the
// row: five dwords from LDS joined by v_alignbyte_b32, low / high nibbles masked into two int8x4
// operands per dword, eight v_dot4_i32_i8 per block.
//
// The lhs is quantised to Q8_0 once per workgroup at the start (four threads per block, codes to LDS);
// the codes a lane needs are those of its own blocks, the same for every row, and it keeps them, their
// scales and code sums in registers.  The arithmetic is that of quantize_q8_0_kernel
// (d = amax / 127 rounded to fp16, q = roundf(x / d)) and of the block dot
//   acc += float(sum q4 q8 - 8 sum q8) * (d4 * d8),
// so the int32 block dots are the ones qmm_block_dots_q4_0 returns.
#include <stdlib.h>

#include <algorithm>

#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int kWaves = 8;        // wavefronts per workgroup
constexpr int kMaxRows = 64;     // rows a wavefront may own (LDS result slots)

// wait until at most `rows` rows (L load instructions each) are outstanding
template <int L>
__device__ __forceinline__ void wait_rows(int rows) {
    if (rows >= 3) wait_vmcnt<3 * L>();
    else if (rows == 2) wait_vmcnt<2 * L>();
    else if (rows == 1) wait_vmcnt<L>();
    else wait_vmcnt<0>();
}

}  // namespace

// BPL: blocks per lane (k <= 2048 * BPL).  L = load instructions per row = pieces of 16 bytes / 64, for the
// longest row BPL allows plus one piece of misalignment (LROW: given instead, for the rows of a K beyond 8192, whose slots
// would not fit the LDS at the full length BPL allows).  RING: LDS slots per wavefront.  Six and eight blocks per lane hold
// one workgroup per compute unit (LDS) and are built for it.
// NORM: the lhs rows are RMS-normalised first, y = x * rsqrt(mean(x^2) + eps) * gamma in fp32 (rounded to bf16 when the
// lhs is bf16: what a bf16 normalisation node would hand over), and y is what gets quantised.
template <int MT, int BPL, int RING, typename AT, bool NORM, int LROW = 0>
__global__ __launch_bounds__(64 * kWaves, BPL > 4 ? 1 : 2) void gemv_q4_0_stream_kernel(const uint8_t* __restrict__ w,
                                                                         const AT* __restrict__ a,
                                                                         float* __restrict__ out, int m, int n, int k,
                                                                         int64_t ldo, const float* __restrict__ gamma, float eps) {
    constexpr int L = LROW ? LROW : (72 * BPL + 1 + 63) / 64;
    constexpr int kSlot = L * 1024;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nblk = k >> 5;
    const int64_t row_bytes = (int64_t)nblk * Q4_0_BPB;
    uint8_t* ring = smem + wave * (RING * kSlot);
    const uint32_t ring_lds = lds_address(ring);
    float* res = (float*)(smem + kWaves * RING * kSlot) + wave * kMaxRows * MT;
    const int gw = (int)blockIdx.x * kWaves + wave, GW = (int)gridDim.x * kWaves;
    const int my_rows = gw < n ? (n - gw + GW - 1) / GW : 0;

    // a row into a slot: aligned 16-byte pieces from the row's first byte rounded down; lanes past the row's
    // last piece repeat it (their bytes land in the unused tail of the slot), so every instruction is issued
    // by all lanes and the wait counts stay exact
    auto issue = [&](int ri, int slot) {
        const uintptr_t ad = (uintptr_t)(w + (int64_t)(gw + (int64_t)ri * GW) * row_bytes);
        const int dl = (int)(ad & 15);
        const int last = (int)((dl + row_bytes + 15) / 16) - 1;
        const uint8_t* base = (const uint8_t*)(ad - (uintptr_t)dl);
#pragma unroll
        for (int i = 0; i < L; i++)
            load16_to_lds_once(base + 16 * (int64_t)min(lane + 64 * i, last), ring_lds + slot * kSlot + i * 1024);
    };

    // --- the lhs, quantised to Q8_0 once per workgroup: thread t takes values 8 t .. 8 t + 7 of every 4096
    //     (four threads per block).  Raw values first, as hidden loads, so that they arrive while the first
    //     weight rows, issued right after them, are in flight.
    constexpr int P = BPL / 2;                       // passes of 4096 values
    constexpr int kPieces = sizeof(AT) == 4 ? 2 : 1;  // 16-byte pieces of 8 lhs values
    uint8_t* qbase = smem + kWaves * RING * kSlot + kWaves * kMaxRows * MT * 4;
    uint32_t* lds_codes = (uint32_t*)qbase;                      // [MT][nblk][8]
    float* lds_scale = (float*)(qbase + (size_t)MT * nblk * 32);  // [MT][nblk]
    int* lds_sum = (int*)(lds_scale + MT * nblk);                // [MT][nblk]
    const int t = (int)threadIdx.x;
    u32x4 raw[MT][P][kPieces];
#pragma unroll
    for (int mi = 0; mi < MT; mi++)
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t v0 = min((int64_t)p * 4096 + 8 * t, (int64_t)k - 8);
            const AT* ar = a + (int64_t)min(mi, m - 1) * k + v0;
#pragma unroll
            for (int i = 0; i < kPieces; i++) hidden_load(raw[mi][p][i], (const uint8_t*)ar + 16 * i);
        }
    u32x4 graw[NORM ? P : 1][2];
    if constexpr (NORM) {
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t v0 = min((int64_t)p * 4096 + 8 * t, (int64_t)k - 8);
            hidden_load(graw[p][0], (const uint8_t*)(gamma + v0));
            hidden_load(graw[p][1], (const uint8_t*)(gamma + v0) + 16);
        }
    }
    int issued = 0;
    for (; issued < min(RING - 1, my_rows); issued++) issue(issued, issued % RING);
    wait_rows<L>(issued);  // the lhs loads are older than these rows
    // the eight lhs values of (row mi, pass p) that this thread holds
    auto values = [&](int mi, int p, float (&v)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kPieces; i++) {
            tie(raw[mi][p][i]);
            const u32x4 r = raw[mi][p][i];
            if constexpr (sizeof(AT) == 4) {
                v[4 * i] = __uint_as_float(r.x); v[4 * i + 1] = __uint_as_float(r.y);
                v[4 * i + 2] = __uint_as_float(r.z); v[4 * i + 3] = __uint_as_float(r.w);
            } else {
                v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
                v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
                v[4] = __uint_as_float(r.z << 16); v[5] = __uint_as_float(r.z & 0xffff0000u);
                v[6] = __uint_as_float(r.w << 16); v[7] = __uint_as_float(r.w & 0xffff0000u);
            }
        }
    };
    float rs[MT];
    if constexpr (NORM) {
        // sum of squares of every lhs row over the workgroup: per thread, per wavefront (DPP), then over the 8 wavefronts in order
        float* red = (float*)(qbase + (size_t)MT * nblk * 40);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            float ss = 0.0f;
#pragma unroll
            for (int p = 0; p < P; p++) {
                float v[8];
                values(mi, p, v);
                const float part = ((v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3])) + ((v[4] * v[4] + v[5] * v[5]) + (v[6] * v[6] + v[7] * v[7]));
                ss += (int64_t)p * 4096 + 8 * t < k ? part : 0.0f;
            }
            ss = wave_sum_dpp(ss);
            if (lane == 0) red[wave * MT + mi] = ss;
        }
        __syncthreads();
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            float tot = 0.0f;
#pragma unroll
            for (int q = 0; q < kWaves; q++) tot += red[q * MT + mi];
            rs[mi] = 1.0f / sqrtf(tot / (float)k + eps);
        }
    }
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
#pragma unroll
        for (int p = 0; p < P; p++) {
            float v[8];
            values(mi, p, v);
            if constexpr (NORM) {
                tie(graw[p][0]);
                tie(graw[p][1]);
                const u32x4 g0 = graw[p][0], g1 = graw[p][1];
                const float g[8] = {__uint_as_float(g0.x), __uint_as_float(g0.y), __uint_as_float(g0.z), __uint_as_float(g0.w),
                                    __uint_as_float(g1.x), __uint_as_float(g1.y), __uint_as_float(g1.z), __uint_as_float(g1.w)};
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    v[i] = (v[i] * rs[mi]) * g[i];
                    if constexpr (sizeof(AT) == 2) v[i] = bf2f(f2bf(v[i]));
                }
            }
            float amax = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                               fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
            amax = fmaxf(amax, dpp_move<0xB1>(amax));
            amax = fmaxf(amax, dpp_move<0x4E>(amax));  // the four threads of a block hold its amax
            uint16_t dh;
            const float id = q8_0_block_rule(amax, dh);
            int q[8];
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = q8_0_code(v[i], id);
            int sum = ((q[0] + q[1]) + (q[2] + q[3])) + ((q[4] + q[5]) + (q[6] + q[7]));
            sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xf, 0xf, true);
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xf, 0xf, true);
            const int blk = p * 128 + (t >> 2);
            if ((int64_t)p * 4096 + 8 * t < k) {
                const uint32_t c0 = (uint32_t)(q[0] & 0xff) | ((uint32_t)(q[1] & 0xff) << 8) | ((uint32_t)(q[2] & 0xff) << 16) |
                                    ((uint32_t)q[3] << 24);
                const uint32_t c1 = (uint32_t)(q[4] & 0xff) | ((uint32_t)(q[5] & 0xff) << 8) | ((uint32_t)(q[6] & 0xff) << 16) |
                                    ((uint32_t)q[7] << 24);
                *(uint2*)(lds_codes + ((size_t)mi * nblk + blk) * 8 + 2 * (t & 3)) = make_uint2(c0, c1);
                if ((t & 3) == 0) {
                    lds_scale[mi * nblk + blk] = h2f(dh);
                    lds_sum[mi * nblk + blk] = sum;
                }
            }
        }
    }
    __syncthreads();
    // the codes, scales and code sums of this lane's own blocks: registers for the whole kernel
    uint32_t acode[MT][BPL][8];
    float ascale[MT][BPL];
    int asum[MT][BPL];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
#pragma unroll
        for (int j = 0; j < BPL; j++) {
            const int b = min(lane + 64 * j, nblk - 1);
            const uint4 c0 = *(const uint4*)(lds_codes + ((size_t)mi * nblk + b) * 8);
            const uint4 c1 = *(const uint4*)(lds_codes + ((size_t)mi * nblk + b) * 8 + 4);
            acode[mi][j][0] = c0.x; acode[mi][j][1] = c0.y; acode[mi][j][2] = c0.z; acode[mi][j][3] = c0.w;
            acode[mi][j][4] = c1.x; acode[mi][j][5] = c1.y; acode[mi][j][6] = c1.z; acode[mi][j][7] = c1.w;
            ascale[mi][j] = lane + 64 * j < nblk ? lds_scale[mi * nblk + b] : 0.0f;  // blocks past the row contribute nothing
            asum[mi][j] = lds_sum[mi * nblk + b];
        }
    }

    for (int ri = 0; ri < my_rows; ri++) {
        // the slot of row ri - 1 is free (its reads fed the sums that were parked): refill it
        if (issued < my_rows) {
            issue(issued, issued % RING);
            issued++;
        }
        wait_rows<L>(issued - 1 - ri);
        const uint8_t* slot = ring + (ri % RING) * kSlot;
        const uint32_t* lds32 = (const uint32_t*)slot;
        const int dl = (int)((uintptr_t)(w + (int64_t)(gw + (int64_t)ri * GW) * row_bytes) & 15);
        float acc[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;
#pragma unroll
        for (int j = 0; j < BPL; j++) {
            const int b = min(lane + 64 * j, nblk - 1);
            const int boff = dl + Q4_0_BPB * b;  // 2-byte aligned: the fp16 d lies inside one dword
            const float dw = h2f((uint16_t)((lds32[boff >> 2] >> (8 * (boff & 3))) & 0xffffu));
            // the 16 nibble bytes start 2 bytes further: five dwords from there, joined at the byte offset
            const int wq = (boff + 2) >> 2;
            const uint32_t sq = (uint32_t)((boff + 2) & 3);
            const uint32_t w0 = lds32[wq], w1 = lds32[wq + 1], w2 = lds32[wq + 2], w3 = lds32[wq + 3], w4 = lds32[wq + 4];
            const uint32_t q[4] = {__builtin_amdgcn_alignbyte(w1, w0, sq), __builtin_amdgcn_alignbyte(w2, w1, sq),
                                   __builtin_amdgcn_alignbyte(w3, w2, sq), __builtin_amdgcn_alignbyte(w4, w3, sq)};
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                int s = 0;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int lo = (int)(q[i] & 0x0F0F0F0Fu), hi = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
                    s = __builtin_amdgcn_sdot4(lo, (int)acode[mi][j][i], s, false);
                    s = __builtin_amdgcn_sdot4(hi, (int)acode[mi][j][4 + i], s, false);
                }
                acc[mi] = fmaf((float)(s - 8 * asum[mi][j]), dw * ascale[mi][j], acc[mi]);
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const float v = wave_sum_dpp(acc[mi]);
            if (lane == 0) res[ri * MT + mi] = v;
        }
    }
    for (int idx = lane; idx < my_rows * MT; idx += 64) {
        const int r = idx / MT, mi = idx - r * MT;
        if (mi < m) out[(int64_t)mi * ldo + gw + (int64_t)r * GW] = res[idx];
    }
}

// Takes the shapes the kernel is built for (reports the others through *handled = false).
hipError_t launch_gemv_q4_0_stream(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                   int64_t ldo, hipStream_t s, bool* handled, const float* gamma, float eps) {
    *handled = false;
    if (kernel_disabled("q4_0_stream") || m > 4 || k < 8) return hipSuccess;
    if (gamma && ((uintptr_t)gamma & 15)) return hipSuccess;  // (the kernel reads gamma in 16-byte pieces)
    const int nblk = (int)(k / 32);
    const int mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    // one lhs row on a K beyond 8192: six or eight blocks per lane, rows of up to seven / eight KB (K <= 12288 / 14528)
    const int64_t row_pieces = ((int64_t)nblk * Q4_0_BPB + 15 + 15) / 16;  // with the worst misalignment
    const int bpl = nblk <= 128 ? 2 : nblk <= 256 ? 4 : (mt == 1 && !gamma && nblk <= 384 && row_pieces <= 7 * 64) ? 6
                  : (mt == 1 && !gamma && nblk <= 512 && row_pieces <= 8 * 64) ? 8 : 0;
    if (!bpl || mt * bpl > 8) return hipSuccess;  // the codes of the lane's blocks must fit its registers
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const int L = bpl == 6 ? 7 : bpl == 8 ? 8 : (72 * bpl + 1 + 63) / 64;
    const int ring = bpl == 2 ? 4 : bpl == 4 ? 3 : 2;  // LDS: 8 wavefronts x ring x L KB
    const size_t lds = (size_t)kWaves * ring * L * 1024 + (size_t)kWaves * kMaxRows * mt * 4 + (size_t)mt * nblk * 40 + 128;  // (the last 128 bytes: the row norms' partial sums)
    int64_t wgs = cus;  // one workgroup of 8 wavefronts per compute unit
    if (wgs * kWaves > n) wgs = (n + kWaves - 1) / kWaves;
    const int64_t min_wgs = (n + (int64_t)kWaves * kMaxRows - 1) / ((int64_t)kWaves * kMaxRows);
    if (wgs < min_wgs) wgs = min_wgs;  // no wavefront owns more rows than it has result slots
    dim3 grid((unsigned)wgs), block(64 * kWaves);
#define QMM_GO2(MT_, BPL_, RING_, AT_, NORM_)                                                                         \
    do {                                                                                                              \
        hipError_t e_ = allow_full_lds<gemv_q4_0_stream_kernel<MT_, BPL_, RING_, AT_, NORM_>>();                      \
        if (e_ != hipSuccess) return e_;                                                                              \
        gemv_q4_0_stream_kernel<MT_, BPL_, RING_, AT_, NORM_><<<grid, block, lds, s>>>(w, (const AT_*)a, out, m, (int)n,  \
                                                                                      (int)k, ldo, gamma, eps);      \
    } while (0)
#define QMM_GO(MT_, BPL_, RING_)                                          \
    do {                                                                  \
        if (a_dtype == QMM_F32) {                                         \
            if (gamma) QMM_GO2(MT_, BPL_, RING_, float, true);            \
            else QMM_GO2(MT_, BPL_, RING_, float, false);                 \
        } else {                                                          \
            if (gamma) QMM_GO2(MT_, BPL_, RING_, uint16_t, true);         \
            else QMM_GO2(MT_, BPL_, RING_, uint16_t, false);              \
        }                                                                 \
    } while (0)
    if (bpl > 4) {
#define QMM_GO_LONG(BPL_, L_)                                                                                         \
    do {                                                                                                              \
        if (a_dtype == QMM_F32) {                                                                                     \
            hipError_t e_ = allow_full_lds<gemv_q4_0_stream_kernel<1, BPL_, 2, float, false, L_>>();                  \
            if (e_ != hipSuccess) return e_;                                                                          \
            gemv_q4_0_stream_kernel<1, BPL_, 2, float, false, L_><<<grid, block, lds, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo, nullptr, 0.0f); \
        } else {                                                                                                      \
            hipError_t e_ = allow_full_lds<gemv_q4_0_stream_kernel<1, BPL_, 2, uint16_t, false, L_>>();               \
            if (e_ != hipSuccess) return e_;                                                                          \
            gemv_q4_0_stream_kernel<1, BPL_, 2, uint16_t, false, L_><<<grid, block, lds, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo, nullptr, 0.0f); \
        }                                                                                                             \
    } while (0)
        if (bpl == 6) QMM_GO_LONG(6, 7);
        else QMM_GO_LONG(8, 8);
#undef QMM_GO_LONG
    } else if (bpl == 2) {
        if (mt == 1) QMM_GO(1, 2, 4);
        else if (mt == 2) QMM_GO(2, 2, 4);
        else QMM_GO(4, 2, 4);
    } else {
        if (mt == 1) QMM_GO(1, 4, 3);
        else QMM_GO(2, 4, 3);
    }
#undef QMM_GO
#undef QMM_GO2
    *handled = true;
    return hipGetLastError();
}

}  // namespace qmm
