// Q5_K and Q6_K decode with Q8_K-quantised activations: integer sub-block dots (v_dot4_i32_i8), the treatment of the
// ggml-lineage CPU kernels.  Selected by QMM_FLAG_ACT_Q8K for up to 16 lhs rows (passes of four); Q4_K has its own
// kernel (gemv_q4k_q8k.hip), which quantises the lhs inside the kernel.
//
// Per (lhs row, weight row, super-block) the kernels form the integers
//   Q5_K:  isum = sum_sub sc_sub * sum_32 q5 * q8,   msum = sum_sub mn_sub * (sum of the sub-block's 32 q8)
//   Q6_K:  isum = sum_16-groups sc_g * sum_16 (q6 - 32) * q8
// exactly (int32, added over the lanes that share a super-block with integer DPP steps), then
//   out += (d8 * d) * float(isum)   [Q5_K:  out -= (d8 * dmin) * float(msum)]
// in fp32.  The integers are those of the CPU path; only the order of the fp32 additions over the super-blocks differs.
//
// The lhs is quantised once per call by quantize_q8_k_planes_kernel (the Q8_K rule of the stand-alone quantiser:
// d8 = -max / 127 for the first element of largest magnitude, codes rounded to nearest even) into three planes in the
// workspace: int8 codes [m, k], fp32 d8 [m, k / 256], int32 sums of 32 codes [m, k / 32].
#include <stdlib.h>

#include <algorithm>

#include "qmm_internal.h"

namespace qmm {

namespace {

constexpr int kWavesI = 4;  // wavefronts per workgroup

// integer sum over aligned groups of 4 / 16 lanes; every lane of the group gets it
__device__ __forceinline__ int isum4(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true);
    return v;
}
__device__ __forceinline__ int isum16(int v) {
    v = isum4(v);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, true);
    return v;
}

// round to nearest, ties to even, through the fp32 adder
__device__ __forceinline__ int nearest_int_rne(float f) {
    const float v = __fadd_rn(f, 12582912.f);
    return (__float_as_int(v) & 0x007fffff) - 0x00400000;
}

}  // namespace

// x [rows, k] -> Q8_K codes, scales and 32-code sums as planes.  32 consecutive threads per 256-wide block, 8 values each.
template <typename AT>
__global__ __launch_bounds__(256) void quantize_q8_k_planes_kernel(const AT* __restrict__ x, int64_t nblocks, int8_t* __restrict__ codes,
                                                                   float* __restrict__ d8s, int32_t* __restrict__ sums) {
    const int64_t blk = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    const int l = threadIdx.x & 31;
    const int64_t bc = min(blk, nblocks - 1);  // whole 32-thread groups stay together for the cross-lane steps
    const AT* xp = x + bc * 256 + 8 * l;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = load_f32(xp, i);
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v[i]));
    amax = fmaxf(amax, dpp_move<0xB1>(amax));
    amax = fmaxf(amax, dpp_move<0x4E>(amax));
    amax = fmaxf(amax, dpp_move<0x141>(amax));
    amax = fmaxf(amax, dpp_move<0x140>(amax));
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    // the first element of that magnitude decides the sign of the scale: smallest (index << 1 | sign bit)
    int key = 0x7fffffff;
#pragma unroll
    for (int i = 7; i >= 0; i--)
        if (fabsf(v[i]) == amax) key = ((8 * l + i) << 1) | (int)(__float_as_uint(v[i]) >> 31);
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0xB1, 0xf, 0xf, false));
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0x4E, 0xf, 0xf, false));
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0x141, 0xf, 0xf, false));
    key = min(key, __builtin_amdgcn_update_dpp(0x7fffffff, key, 0x140, 0xf, 0xf, false));
    key = min(key, __shfl_xor(key, 16, 64));
    const float mx = (key & 1) ? -amax : amax;
    int q[8];
    float d8 = 0.0f;
    if (amax == 0.0f) {
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = 0;
    } else {
        const float iscale = -127.f / mx;
        d8 = 1.0f / iscale;
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = min(127, nearest_int_rne(__fmul_rn(iscale, v[i])));
    }
    int s = ((q[0] + q[1]) + (q[2] + q[3])) + ((q[4] + q[5]) + (q[6] + q[7]));
    s = isum4(s);  // 32 codes: four threads
    if (blk >= nblocks) return;
    const uint32_t c0 = (uint32_t)(q[0] & 0xff) | ((uint32_t)(q[1] & 0xff) << 8) | ((uint32_t)(q[2] & 0xff) << 16) | ((uint32_t)q[3] << 24);
    const uint32_t c1 = (uint32_t)(q[4] & 0xff) | ((uint32_t)(q[5] & 0xff) << 8) | ((uint32_t)(q[6] & 0xff) << 16) | ((uint32_t)q[7] << 24);
    *(uint2*)(codes + blk * 256 + 8 * l) = make_uint2(c0, c1);
    if (l == 0) d8s[blk] = d8;
    if ((l & 3) == 0) sums[blk * 8 + (l >> 2)] = s;
}

int64_t q8k_planes_bytes(int64_t m, int64_t k) {
    const int64_t codes = (m * k + 255) / 256 * 256, d8 = (m * (k / 256) * 4 + 255) / 256 * 256, sums = (m * (k / 32) * 4 + 255) / 256 * 256;
    return codes + d8 + sums;
}

Q8KPlanes q8k_planes(void* ws, int64_t m, int64_t k) {
    Q8KPlanes p;
    const int64_t codes = (m * k + 255) / 256 * 256, d8 = (m * (k / 256) * 4 + 255) / 256 * 256;
    p.codes = (int8_t*)ws;
    p.d8 = (float*)((char*)ws + codes);
    p.sums = (int32_t*)((char*)ws + codes + d8);
    return p;
}

hipError_t launch_quantize_q8_k_planes(const void* x, int x_dtype, int64_t rows, int64_t k, const Q8KPlanes& p, hipStream_t s) {
    const int64_t nblocks = rows * (k / 256);
    const dim3 grid((unsigned)((nblocks * 32 + 255) / 256)), block(256);
    if (x_dtype == QMM_F32) quantize_q8_k_planes_kernel<float><<<grid, block, 0, s>>>((const float*)x, nblocks, p.codes, p.d8, p.sums);
    else quantize_q8_k_planes_kernel<uint16_t><<<grid, block, 0, s>>>((const uint16_t*)x, nblocks, p.codes, p.d8, p.sums);
    return hipGetLastError();
}

// Q5_K: a wavefront owns whole weight rows and walks them 16 super-blocks at a time; lane (block lb = lane / 4, chunk c = lane % 4)
// holds the 64 weights of sub-blocks 2c and 2c + 1 of its block (32 code bytes, bits 2c and 2c + 1 of the 32 fifth-bit bytes).
// The four lanes of a block add their integers; lane c = 0 applies the scales.  MT lhs rows (1, 2 or 4).
template <int MT>
__global__ __launch_bounds__(64 * kWavesI) void gemv_q5_k_q8k_kernel(const uint8_t* __restrict__ w, const int8_t* __restrict__ codes,
                                                                    const float* __restrict__ d8s, const int32_t* __restrict__ sums,
                                                                    float* __restrict__ out, int m, int n, int k, int64_t ldo) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int nblk = k >> 8;
    const int ngroups = (nblk + 15) >> 4;
    const int64_t row_bytes = (int64_t)nblk * Q5_K_BPB;
    const int lb = lane >> 2, c = lane & 3;
    const int total_waves = (int)gridDim.x * kWavesI, gw = (int)blockIdx.x * kWavesI + wave;
    const int sh = 16 * (c & 1);  // byte pair (2c, 2c + 1) mod 4 inside a dword of the 6-bit fields
    const bool upper = c >= 2;    // sub-blocks 4..7 use the split encoding
    for (int row = gw; row < n; row += total_waves) {
        float acc[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;
        for (int g = 0; g < ngroups; g++) {
            const bool live = 16 * g + lb < nblk;
            const int blk = min(16 * g + lb, nblk - 1);
            const uint8_t* b = w + (int64_t)row * row_bytes + (int64_t)blk * Q5_K_BPB;
            const uint4 hdr = *(const uint4*)b, qh0 = *(const uint4*)(b + 16), qh1 = *(const uint4*)(b + 32);
            const uint4 qs0 = *(const uint4*)(b + 48 + 32 * c), qs1 = *(const uint4*)(b + 64 + 32 * c);
            const float d = h2f((uint16_t)(hdr.x & 0xffffu)), dmin = h2f((uint16_t)(hdr.x >> 16));
            const uint32_t p0 = (hdr.y >> sh) & 0xffffu, p1 = (hdr.z >> sh) & 0xffffu, p2 = (hdr.w >> sh) & 0xffffu;
            const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
            const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
            const int sc0 = (int)(sc_pair & 0xffu), sc1 = (int)(sc_pair >> 8), mn0 = (int)(mn_pair & 0xffu), mn1 = (int)(mn_pair >> 8);
            const uint32_t qs[8] = {qs0.x, qs0.y, qs0.z, qs0.w, qs1.x, qs1.y, qs1.z, qs1.w};
            const uint32_t qh[8] = {qh0.x, qh0.y, qh0.z, qh0.w, qh1.x, qh1.y, qh1.z, qh1.w};
            uint32_t lo[8], hi[8];  // four 5-bit codes per dword: low nibbles + fifth bit 2c, high nibbles + fifth bit 2c + 1
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t hb = qh[i] >> (2 * c);
                lo[i] = (qs[i] & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
                hi[i] = ((qs[i] >> 4) & 0x0F0F0F0Fu) | ((hb << 3) & 0x10101010u);
            }
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const int r = min(mi, m - 1);
                const uint4* cp = (const uint4*)(codes + (int64_t)r * k + (int64_t)blk * 256 + 64 * c);
                const uint4 a0 = cp[0], a1 = cp[1], a2 = cp[2], a3 = cp[3];
                const uint32_t alo[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                const uint32_t ahi[8] = {a2.x, a2.y, a2.z, a2.w, a3.x, a3.y, a3.z, a3.w};
                int il = 0, ih = 0;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    il = __builtin_amdgcn_sdot4((int)lo[i], (int)alo[i], il, false);
                    ih = __builtin_amdgcn_sdot4((int)hi[i], (int)ahi[i], ih, false);
                }
                const int32_t* sp = sums + ((int64_t)r * nblk + blk) * 8 + 2 * c;
                // |il| <= 32 * 31 * 127 < 2^17, times a 6-bit scale, twice, over four lanes: below 2^26
                const int is = isum4(sc0 * il + sc1 * ih);
                const int ms = isum4(mn0 * sp[0] + mn1 * sp[1]);
                const float d8 = d8s[(int64_t)r * nblk + blk];
                if (live && c == 0) {
                    acc[mi] = acc[mi] + (d8 * d) * (float)is;
                    acc[mi] = acc[mi] - (d8 * dmin) * (float)ms;
                }
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const float v = wave_sum_dpp(acc[mi]);
            if (lane == 0 && mi < m) out[(int64_t)mi * ldo + row] = v;
        }
    }
}

// Q6_K: super-blocks are only 2-byte aligned, so a lane reads every field as two aligned dwords joined at the byte offset.  A
// wavefront owns whole rows and walks them 4 super-blocks at a time; lane t of a 16-lane group owns, in half h = t / 8 of its
// block, the four ql bytes 4j .. 4j + 3 (j = t % 8), the four bytes 32 further and the four qh bytes 4j .. 4j + 3: sixteen
// weights, four each at columns 128 h + 4 j + {0, 32, 64, 96}, each quartet under its own int8 scale.  The sixteen lanes of a
// block add their integers; lane t = 0 applies d8 * d.
template <int MT>
__global__ __launch_bounds__(64 * kWavesI) void gemv_q6_k_q8k_kernel(const uint8_t* __restrict__ w, const int8_t* __restrict__ codes,
                                                                    const float* __restrict__ d8s, float* __restrict__ out, int m, int n,
                                                                    int k, int64_t ldo) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q6_K_BPB;
    const int bq = lane >> 4, t = lane & 15, h = t >> 3, j = t & 7;
    const int f_ql = 64 * h + 4 * j, f_qh = 128 + 32 * h + 4 * j, f_sc = 192 + 8 * h;
    const int sc_shift = 8 * (j >> 2);  // this lane's quartet scales: bytes jj, jj + 2 of each of the half's two scale dwords
    const int total_waves = (int)gridDim.x * kWavesI, gw = (int)blockIdx.x * kWavesI + wave;
    const uint8_t* const w_end = w + (int64_t)n * row_bytes;
    for (int row = gw; row < n; row += total_waves) {
        float acc[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;
        for (int b0 = 0; b0 < nblk; b0 += 4) {
            const bool live = b0 + bq < nblk;
            const int blk = min(b0 + bq, nblk - 1);
            const uint8_t* bp = w + (int64_t)row * row_bytes + (int64_t)blk * Q6_K_BPB;
            const uint32_t shift = (uint32_t)((uintptr_t)bp & 3);  // 0 or 2
            const uint32_t* base = (const uint32_t*)(bp - shift);
            // (the dword behind the tensor's last byte is not read: the last field of the last block is joined with itself)
            auto rd = [&](int field) {
                const uint32_t* p = base + (field >> 2);
                const uint32_t lo = p[0], hi = (const uint8_t*)(p + 1) < w_end ? p[1] : lo;
                return __builtin_amdgcn_alignbyte(hi, lo, shift);
            };
            const uint32_t A = rd(f_ql), B = rd(f_ql + 32), H = rd(f_qh);
            const uint32_t s0 = rd(f_sc), s1 = rd(f_sc + 4);
            const float d = h2f((uint16_t)(rd(208) & 0xffffu));
            // four 6-bit codes per dword, then minus 32 in every byte: (q | 0x80) - 0x20 borrows from no neighbour, xor 0x80 restores the sign
            auto centred = [](uint32_t q) { return (((q | 0x80808080u) - 0x20202020u) ^ 0x80808080u); };
            const uint32_t q1 = centred((A & 0x0F0F0F0Fu) | ((H << 4) & 0x30303030u));
            const uint32_t q2 = centred((B & 0x0F0F0F0Fu) | ((H << 2) & 0x30303030u));
            const uint32_t q3 = centred(((A >> 4) & 0x0F0F0F0Fu) | (H & 0x30303030u));
            const uint32_t q4 = centred(((B >> 4) & 0x0F0F0F0Fu) | ((H >> 2) & 0x30303030u));
            const int e1 = (int)(s0 << (24 - sc_shift)) >> 24, e2 = (int)(s0 << (8 - sc_shift)) >> 24;
            const int e3 = (int)(s1 << (24 - sc_shift)) >> 24, e4 = (int)(s1 << (8 - sc_shift)) >> 24;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const int r = min(mi, m - 1);
                const uint32_t* ap = (const uint32_t*)(codes + (int64_t)r * k + (int64_t)blk * 256 + 128 * h + 4 * j);
                const int p1 = __builtin_amdgcn_sdot4((int)q1, (int)ap[0], 0, false), p2 = __builtin_amdgcn_sdot4((int)q2, (int)ap[8], 0, false);
                const int p3 = __builtin_amdgcn_sdot4((int)q3, (int)ap[16], 0, false), p4 = __builtin_amdgcn_sdot4((int)q4, (int)ap[24], 0, false);
                // |p| <= 4 * 32 * 127, times an int8 scale, four times, over sixteen lanes: below 2^27
                const int is = isum16(e1 * p1 + e2 * p2 + e3 * p3 + e4 * p4);
                const float d8 = d8s[(int64_t)r * nblk + blk];
                if (live && t == 0) acc[mi] = acc[mi] + (d8 * d) * (float)is;
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const float v = wave_sum_dpp(acc[mi]);
            if (lane == 0 && mi < m) out[(int64_t)mi * ldo + row] = v;
        }
    }
}

// One pass: up to four lhs rows (rows m0 .. of the planes), all weight rows.
hipError_t launch_gemv_kquant_q8k(int encoding, const Q8KPlanes& p, int64_t m0, int rows, const uint8_t* w, int64_t n, int64_t k, float* out,
                                  int64_t ldo, hipStream_t s) {
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const int mt = rows <= 1 ? 1 : rows <= 2 ? 2 : 4;
    const int64_t nblk = k / 256;
    const int8_t* codes = p.codes + m0 * k;
    const float* d8 = p.d8 + m0 * nblk;
    const int32_t* sums = p.sums + m0 * nblk * 8;
    const dim3 grid((unsigned)std::min<int64_t>((n + kWavesI - 1) / kWavesI, (int64_t)cus * 8)), block(64 * kWavesI);
    if (encoding == QMM_Q5_K) {
        if (mt == 1) gemv_q5_k_q8k_kernel<1><<<grid, block, 0, s>>>(w, codes, d8, sums, out, rows, (int)n, (int)k, ldo);
        else if (mt == 2) gemv_q5_k_q8k_kernel<2><<<grid, block, 0, s>>>(w, codes, d8, sums, out, rows, (int)n, (int)k, ldo);
        else gemv_q5_k_q8k_kernel<4><<<grid, block, 0, s>>>(w, codes, d8, sums, out, rows, (int)n, (int)k, ldo);
    } else {
        if (mt == 1) gemv_q6_k_q8k_kernel<1><<<grid, block, 0, s>>>(w, codes, d8, out, rows, (int)n, (int)k, ldo);
        else if (mt == 2) gemv_q6_k_q8k_kernel<2><<<grid, block, 0, s>>>(w, codes, d8, out, rows, (int)n, (int)k, ldo);
        else gemv_q6_k_q8k_kernel<4><<<grid, block, 0, s>>>(w, codes, d8, out, rows, (int)n, (int)k, ldo);
    }
    return hipGetLastError();
}

}  // namespace qmm
