// Q4_K decode kernel for one or two lhs rows on the vector ALUs.
//
// A wavefront owns R consecutive weight rows.  Eight lanes share a 144-byte
// super-block: lane u of the group loads the 16-byte header and the 16-byte code
// unit u (consecutive lanes, consecutive addresses), i.e. 16 weights of sub-block
// 2c in its low nibbles and 16 weights of sub-block 2c+1 in its high nibbles
// (c = u/2).  The 32 activations a lane needs for a super-block position are
// loaded once and reused for all R rows; the loads of all R rows are issued
// before any of them is consumed.  With w = (d*sc)*q - dmin*m the row dot is
//   sum_sub (d*sc) * sum(q*a) - (dmin*m) * sum(a),
// so the per-weight work is one byte-to-float conversion and one fp32 FMA.
#include <stdlib.h>

#include "qmm_internal.h"

namespace qmm {


namespace {

template <typename AT>
__device__ __forceinline__ float4 load_a4(const AT* __restrict__ a, int64_t i) {
    if constexpr (sizeof(AT) == 4) {
        return *(const float4*)(a + i);
    } else {
        uint2 v = *(const uint2*)(a + i);
        return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                           __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
    }
}

// Byte i of a dword as fp32 in one instruction.  Written as asm so that the nibble mask applied
// to the whole dword is not re-fused into a per-byte bit-field extract plus conversion.
__device__ __forceinline__ float ub0(uint32_t v) { float f; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ub1(uint32_t v) { float f; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ub2(uint32_t v) { float f; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ub3(uint32_t v) { float f; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v)); return f; }

}  // namespace

// LDSA: the lhs rows are staged once per workgroup in LDS, 16-byte pieces stored in the order the
// lanes consume them (piece index = iteration*512 + j*64 + lane), so that the main loop reads
// them with conflict-free ds_read_b128 instead of scattered global loads.
template <int R, int MT, typename AT, bool LDSA>
__global__ __launch_bounds__(512, 4) void gemv_q4_k_rows_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                             float* __restrict__ out, int m, int n, int k,
                                                             int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) float4 lds_act[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int nblk = k >> 8;
    const int iters = (nblk + 7) >> 3;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int sb = lane >> 3, u = lane & 7, c = u >> 1, h = u & 1;

    if constexpr (LDSA) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const AT* ar = a + (int64_t)min(mi, m - 1) * k;
            for (int pk = threadIdx.x; pk < nblk * 64; pk += blockDim.x) {
                const int b = pk >> 6, p = pk & 63;
                const int pc = p >> 4, r16 = p & 15;
                const int pu = 2 * pc + ((r16 >> 2) & 1), pj = 4 * (r16 >> 3) + (r16 & 3);
                lds_act[(size_t)mi * iters * 512 + (b >> 3) * 512 + pj * 64 + (b & 7) * 8 + pu] = load_a4(ar, 4 * pk);
            }
        }
        __syncthreads();
    }

    // branch-free selection of this lane's two sub-blocks (2c, 2c+1) out of the 6-bit fields
    const int sh = 16 * (c & 1);   // byte pair (2c, 2c+1) mod 4 inside a dword
    const bool upper = c >= 2;     // sub-blocks 4..7 use the split encoding

    const int ngroups = (n + R - 1) / R;
    for (int grp = blockIdx.x * nwaves + wave; grp < ngroups; grp += gridDim.x * nwaves) {
    const int row0 = grp * R;
    const uint8_t* wrow[R];
#pragma unroll
    for (int r = 0; r < R; r++) wrow[r] = w + (int64_t)min(row0 + r, n - 1) * row_bytes;

    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int i = 0; i < MT; i++) acc[r][i] = 0.0f;

    // one super-block position: packed bytes of the R rows, activations of the MT lhs rows
    struct Pos {
        uint4 hdr[R], qs[R];
        float4 x[MT][4], y[MT][4];
    };
    auto load_pos = [&](Pos& p, int blk_i) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint4* blk = (const uint4*)(wrow[r] + (int64_t)blk_i * Q4_K_BPB);
            p.hdr[r] = blk[0];
            p.qs[r] = blk[1 + u];
        }
        const int kbase = blk_i * 256 + 64 * c + 16 * h;
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            if constexpr (LDSA) {
                const float4* la = lds_act + (size_t)mi * iters * 512 + (blk_i >> 3) * 512 + lane;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    p.x[mi][i] = la[i * 64];
                    p.y[mi][i] = la[(4 + i) * 64];
                }
            } else {
                const AT* ar = a + (int64_t)min(mi, m - 1) * k + kbase;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    p.x[mi][i] = load_a4(ar, 4 * i);
                    p.y[mi][i] = load_a4(ar, 32 + 4 * i);
                }
            }
        }
    };
    auto compute = [&](const Pos& p) {
        float alo[MT], ahi[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            alo[mi] = 0.0f;
            ahi[mi] = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                alo[mi] += (p.x[mi][i].x + p.x[mi][i].y) + (p.x[mi][i].z + p.x[mi][i].w);
                ahi[mi] += (p.y[mi][i].x + p.y[mi][i].y) + (p.y[mi][i].z + p.y[mi][i].w);
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float d = h2f((uint16_t)(p.hdr[r].x & 0xffffu)), dmin = h2f((uint16_t)(p.hdr[r].x >> 16));
            // bytes (2c, 2c+1) mod 4 of the three scale dwords, as 16-bit pairs
            const uint32_t p0 = (p.hdr[r].y >> sh) & 0xffffu, p1 = (p.hdr[r].z >> sh) & 0xffffu,
                           p2 = (p.hdr[r].w >> sh) & 0xffffu;
            const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
            const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
            const float d1 = d * ub0(sc_pair), d2 = d * ub1(sc_pair);
            const float m1 = dmin * ub0(mn_pair), m2 = dmin * ub1(mn_pair);
            const uint32_t qw[4] = {p.qs[r].x, p.qs[r].y, p.qs[r].z, p.qs[r].w};
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                float slo = 0.0f, shi = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t lo = qw[i] & 0x0F0F0F0Fu, hi = (qw[i] >> 4) & 0x0F0F0F0Fu;
                    slo = fmaf(p.x[mi][i].x, ub0(lo), slo);
                    slo = fmaf(p.x[mi][i].y, ub1(lo), slo);
                    slo = fmaf(p.x[mi][i].z, ub2(lo), slo);
                    slo = fmaf(p.x[mi][i].w, ub3(lo), slo);
                    shi = fmaf(p.y[mi][i].x, ub0(hi), shi);
                    shi = fmaf(p.y[mi][i].y, ub1(hi), shi);
                    shi = fmaf(p.y[mi][i].z, ub2(hi), shi);
                    shi = fmaf(p.y[mi][i].w, ub3(hi), shi);
                }
                float t = fmaf(d1, slo, acc[r][mi]);
                t = fmaf(-m1, alo[mi], t);
                t = fmaf(d2, shi, t);
                acc[r][mi] = fmaf(-m2, ahi[mi], t);
            }
        }
    };

    if constexpr (LDSA) {
        // Activations stay in LDS and are read one 16-byte piece at a time, so that registers hold
        // little more than the R rows of packed bytes in flight.
        for (int b = sb; b < nblk; b += 8) {
            uint4 hdr[R], qs[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint4* blk = (const uint4*)(wrow[r] + (int64_t)b * Q4_K_BPB);
                hdr[r] = blk[0];
                qs[r] = blk[1 + u];
            }
            float slo[R][MT], shi[R][MT], alo[MT], ahi[MT];
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                alo[mi] = 0.0f;
                ahi[mi] = 0.0f;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    slo[r][mi] = 0.0f;
                    shi[r][mi] = 0.0f;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
#pragma unroll
                for (int mi = 0; mi < MT; mi++) {
                    const float4* la = lds_act + (size_t)mi * iters * 512 + (b >> 3) * 512 + lane;
                    const float4 x = la[i * 64], y = la[(4 + i) * 64];
                    alo[mi] += (x.x + x.y) + (x.z + x.w);
                    ahi[mi] += (y.x + y.y) + (y.z + y.w);
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const uint32_t qd = i == 0 ? qs[r].x : (i == 1 ? qs[r].y : (i == 2 ? qs[r].z : qs[r].w));
                        const uint32_t lo = qd & 0x0F0F0F0Fu, hi = (qd >> 4) & 0x0F0F0F0Fu;
                        float t = slo[r][mi];
                        t = fmaf(x.x, ub0(lo), t);
                        t = fmaf(x.y, ub1(lo), t);
                        t = fmaf(x.z, ub2(lo), t);
                        slo[r][mi] = fmaf(x.w, ub3(lo), t);
                        t = shi[r][mi];
                        t = fmaf(y.x, ub0(hi), t);
                        t = fmaf(y.y, ub1(hi), t);
                        t = fmaf(y.z, ub2(hi), t);
                        shi[r][mi] = fmaf(y.w, ub3(hi), t);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float d = h2f((uint16_t)(hdr[r].x & 0xffffu)), dmin = h2f((uint16_t)(hdr[r].x >> 16));
                const uint32_t p0 = (hdr[r].y >> sh) & 0xffffu, p1 = (hdr[r].z >> sh) & 0xffffu,
                               p2 = (hdr[r].w >> sh) & 0xffffu;
                const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
                const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
                const float d1 = d * ub0(sc_pair), d2 = d * ub1(sc_pair);
                const float m1 = dmin * ub0(mn_pair), m2 = dmin * ub1(mn_pair);
#pragma unroll
                for (int mi = 0; mi < MT; mi++) {
                    float t = fmaf(d1, slo[r][mi], acc[r][mi]);
                    t = fmaf(-m1, alo[mi], t);
                    t = fmaf(d2, shi[r][mi], t);
                    acc[r][mi] = fmaf(-m2, ahi[mi], t);
                }
            }
        }
    } else {
        Pos p;
        for (int b = sb; b < nblk; b += 8) {
            load_pos(p, b);
            compute(p);
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const float v = wave_sum_dpp(acc[r][mi]);
            if (lane == 0 && mi < m && row0 + r < n) out[(int64_t)mi * ldo + row0 + r] = v;
        }
    }
    }  // row groups
}

// Streaming variant: one weight row per wavefront at a time, workgroups persistent.  A wavefront
// walks its (row, 8-super-block step) units with a ring of four units of loads in flight, so the
// loads of later units overlap the arithmetic of the current one; activations are read from LDS
// (staged once per workgroup in lane order) one 16-byte piece at a time.
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ half2v as_half2(uint32_t u) { return __builtin_bit_cast(half2v, u); }

constexpr int kStreamMaxRows = 64;  // rows a wavefront may own in the streaming kernel (LDS result slots)

template <int MT, typename AT>
__global__ __launch_bounds__(512, MT == 1 ? 4 : 2) void gemv_q4_k_stream_kernel(const uint8_t* __restrict__ w,
                                                                  const AT* __restrict__ a, float* __restrict__ out,
                                                                  int m, int n, int k, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) float4 lds_act[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int nblk = k >> 8;
    const int iters = (nblk + 7) >> 3;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int sb = lane >> 3, u = lane & 7, c = u >> 1;

    const int sh = 16 * (c & 1);
    const bool upper = c >= 2;
    const int gw = blockIdx.x * nwaves + wave, GW = gridDim.x * nwaves;
    const int my_rows = gw < n ? (n - gw + GW - 1) / GW : 0;  // rows gw, gw + GW, ...
    const int total = my_rows * iters;

    struct Unit {
        uint4 hdr, qs;
    };
    auto load_unit = [&](Unit& x, int unit) {
        const int ri = unit / iters, it = unit - ri * iters;
        // unconditional (clamped) loads: no control flow around them, so the waits in the ring stay exact
        const int b = min(it * 8 + sb, nblk - 1);
        const uint4* blk = (const uint4*)(w + (int64_t)(gw + ri * GW) * row_bytes + (int64_t)b * Q4_K_BPB);
        x.hdr = blk[0];
        x.qs = blk[1 + u];
    };
    Unit ring[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        ring[s].hdr = make_uint4(0, 0, 0, 0);
        ring[s].qs = make_uint4(0, 0, 0, 0);
        if (s < total) load_unit(ring[s], s);
    }
    // The first ring of weight loads is already in flight: stage the activations under its latency.
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        const AT* ar = a + (int64_t)min(mi, m - 1) * k;
        for (int pk = threadIdx.x; pk < nblk * 64; pk += blockDim.x) {
            const int b = pk >> 6, p = pk & 63;
            const int pc = p >> 4, r16 = p & 15;
            const int pu = 2 * pc + ((r16 >> 2) & 1), pj = 4 * (r16 >> 3) + (r16 & 3);
            lds_act[(size_t)mi * iters * 512 + (b >> 3) * 512 + pj * 64 + (b & 7) * 8 + pu] = load_a4(ar, 4 * pk);
        }
    }

    __syncthreads();  // staged activations visible
    // per (step, lane) sums of the 16 + 16 activations a lane multiplies: the same for every row
    float2* lds_asum = (float2*)(lds_act + (size_t)MT * iters * 512);
    for (int e = threadIdx.x; e < MT * iters * 64; e += blockDim.x) {
        const float4* la = lds_act + (size_t)(e >> 6) * 512 + (e & 63);
        float lo = 0.0f, hi = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float4 xa = la[i * 64], ya = la[(4 + i) * 64];
            lo += (xa.x + xa.y) + (xa.z + xa.w);
            hi += (ya.x + ya.y) + (ya.z + ya.w);
        }
        lds_asum[e] = make_float2(lo, hi);
    }
    __syncthreads();

    float acc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) acc[i] = 0.0f;

    auto process = [&](const Unit& x, int it) {
        if (it * 8 + sb >= nblk) return;
        float slo[MT], shi[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) slo[mi] = shi[mi] = 0.0f;
        const uint32_t qd[4] = {x.qs.x, x.qs.y, x.qs.z, x.qs.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // A masked nibble in a 16-bit half is the fp16 subnormal q * 2^-24 (low nibbles) or 16 q * 2^-24
            // (high nibbles, left in place); the fused multiply-add widens the half itself, so no
            // conversion instruction is spent per code.  The powers of two go into d1 / d2 below.
            const uint32_t y = qd[i] >> 8;
            const half2v l02 = as_half2(qd[i] & 0x000F000Fu), l13 = as_half2(y & 0x000F000Fu);
            const half2v h02 = as_half2(qd[i] & 0x00F000F0u), h13 = as_half2(y & 0x00F000F0u);
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const float4* la = lds_act + (size_t)mi * iters * 512 + it * 512 + lane;
                const float4 xa = la[i * 64], ya = la[(4 + i) * 64];
                float t = slo[mi];
                t = fmaf(xa.x, (float)l02.x, t);
                t = fmaf(xa.y, (float)l13.x, t);
                t = fmaf(xa.z, (float)l02.y, t);
                slo[mi] = fmaf(xa.w, (float)l13.y, t);
                t = shi[mi];
                t = fmaf(ya.x, (float)h02.x, t);
                t = fmaf(ya.y, (float)h13.x, t);
                t = fmaf(ya.z, (float)h02.y, t);
                shi[mi] = fmaf(ya.w, (float)h13.y, t);
            }
        }
        const float d = h2f((uint16_t)(x.hdr.x & 0xffffu)), dmin = h2f((uint16_t)(x.hdr.x >> 16));
        const uint32_t p0 = (x.hdr.y >> sh) & 0xffffu, p1 = (x.hdr.z >> sh) & 0xffffu, p2 = (x.hdr.w >> sh) & 0xffffu;
        const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
        const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
        const float d1 = d * ub0(sc_pair) * 16777216.0f, d2 = d * ub1(sc_pair) * 1048576.0f;  // 2^24, 2^24 / 16
        const float m1 = dmin * ub0(mn_pair), m2 = dmin * ub1(mn_pair);
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const float2 as = lds_asum[(mi * iters + it) * 64 + lane];
            float t = fmaf(d1, slo[mi], acc[mi]);
            t = fmaf(-m1, as.x, t);
            t = fmaf(d2, shi[mi], t);
            acc[mi] = fmaf(-m2, as.y, t);
        }
    };

    // The ring is walked with a statically unrolled body so that every wait names exactly the loads
    // it needs (three younger units stay in flight); a remainder loop handles the last < 4 units.
    // Row results are parked in LDS and written out after the loop: a global store inside the loop
    // would force every wait on the ring down to "all loads returned".
    float* res = (float*)(lds_asum + (size_t)MT * iters * 64) + (size_t)wave * kStreamMaxRows * MT;
    int it = 0, ri = 0;
    auto finish_row = [&]() {
        if (++it == iters) {
            it = 0;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const float v = wave_sum_dpp(acc[mi]);
                if (lane == 0) res[ri * MT + mi] = v;
                acc[mi] = 0.0f;
            }
            ri++;
        }
    };
    int unit = 0;
    if (total >= 8) {
        // first round peeled: the loop is then entered with the same loads in flight as at its back edge
#pragma unroll
        for (int s = 0; s < 4; s++) {
            process(ring[s], it);
            load_unit(ring[s], s + 4);
            finish_row();
        }
        for (unit = 4; unit + 8 <= total; unit += 4) {
#pragma unroll
            for (int s = 0; s < 4; s++) {
                process(ring[s], it);
                load_unit(ring[s], unit + s + 4);
                finish_row();
            }
        }
    }
#pragma unroll
    for (int s = 0; s < 4; s++) {  // units unit .. unit+3: the last ones that still have a successor to load
        if (unit + s < total) {
            process(ring[s], it);
            if (unit + s + 4 < total) load_unit(ring[s], unit + s + 4);
            finish_row();
        }
    }
#pragma unroll
    for (int s = 0; s < 4; s++) {
        if (unit + 4 + s < total) {
            process(ring[s], it);
            finish_row();
        }
    }
    for (int idx = lane; idx < my_rows * MT; idx += 64) {
        const int r = idx / MT, mi = idx - r * MT;
        if (mi < m) out[(int64_t)mi * ldo + gw + (int64_t)r * GW] = res[idx];
    }
}

hipError_t launch_gemv_q4_k_rows(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                                 float* out, int64_t ldo, hipStream_t s) {
    const int r_env = 0, g_env = 0, w_env = 0;  // (launch-shape overrides of earlier tuning runs: none)
    const int mt = m <= 1 ? 1 : 2;
    // rows per wavefront: as many as keep at least ~2000 wavefronts in the grid
    const int r = r_env > 0 ? r_env : (n >= 8192 ? 4 : (n >= 4096 ? 2 : 1));
    const int nblk = (int)(k >> 8);
    // staged lhs rows, padded to 8 super-blocks, plus 512 bytes of lane sums per step, plus result slots
    const int wv_stream = (w_env == 4 || w_env == 8) ? w_env : 8;  // wavefronts per workgroup of the streaming kernel
    const size_t lds = (size_t)mt * ((nblk + 7) / 8) * (8192 + 512) + (size_t)wv_stream * kStreamMaxRows * mt * 4;
    const bool ldsa = lds <= 64 * 1024;
    const int waves = w_env > 0 ? w_env : (lds > 32 * 1024 ? 8 : 4);
    const int g = g_env > 0 ? g_env : 1;  // row groups per wavefront
    if (ldsa && !kernel_disabled("q4k_stream")) {
        // streaming kernel: persistent workgroups, as many as fill the machine at 4 wavefronts per SIMD
        static const int num_cu = [] {
            int dev = 0, cu = 256;
            if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev);
            return cu > 0 ? cu : 256;
        }();
        const int wv = wv_stream;
        int64_t wgs = (int64_t)num_cu * (16 / wv) * (g_env > 0 ? g_env : 1);
        size_t per_cu = (size_t)160 * 1024 / lds;  // workgroups per CU that the staged activations allow
        if (per_cu < 1) per_cu = 1;
        if (wgs > (int64_t)num_cu * (int64_t)per_cu) wgs = (int64_t)num_cu * (int64_t)per_cu;
        if (wgs * wv > n) wgs = (n + wv - 1) / wv;
        const int64_t min_wgs = (n + (int64_t)wv * kStreamMaxRows - 1) / ((int64_t)wv * kStreamMaxRows);
        if (wgs < min_wgs) wgs = min_wgs;  // no wavefront owns more rows than it has result slots
        dim3 sgrid((unsigned)wgs), sblock(wv * 64);
        if (mt == 1) {
            if (a_dtype == QMM_F32) gemv_q4_k_stream_kernel<1, float><<<sgrid, sblock, lds, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo);
            else gemv_q4_k_stream_kernel<1, uint16_t><<<sgrid, sblock, lds, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo);
        } else {
            if (a_dtype == QMM_F32) gemv_q4_k_stream_kernel<2, float><<<sgrid, sblock, lds, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo);
            else gemv_q4_k_stream_kernel<2, uint16_t><<<sgrid, sblock, lds, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo);
        }
        return hipGetLastError();
    }
    const int64_t groups = (n + r - 1) / r;
    dim3 grid((unsigned)((groups + (int64_t)waves * g - 1) / ((int64_t)waves * g))), block(waves * 64);
#define QMM_CALL2(R, MT, L)                                                                                          \
    do {                                                                                                             \
        const size_t sm = L ? lds : 0;                                                                               \
        if (a_dtype == QMM_F32)                                                                                      \
            gemv_q4_k_rows_kernel<R, MT, float, L><<<grid, block, sm, s>>>(w, (const float*)a, out, m, (int)n, (int)k, ldo); \
        else                                                                                                         \
            gemv_q4_k_rows_kernel<R, MT, uint16_t, L><<<grid, block, sm, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, ldo); \
    } while (0)
#define QMM_CALL(R, MT)               \
    do {                              \
        if (ldsa) QMM_CALL2(R, MT, true); \
        else QMM_CALL2(R, MT, false); \
    } while (0)
    if (mt == 1) {
        if (r >= 4) QMM_CALL(4, 1);
        else if (r == 2) QMM_CALL(2, 1);
        else QMM_CALL(1, 1);
    } else {
        if (r >= 4) QMM_CALL(4, 2);
        else if (r == 2) QMM_CALL(2, 2);
        else QMM_CALL(1, 2);
    }
#undef QMM_CALL
#undef QMM_CALL2
    return hipGetLastError();
}

}  // namespace qmm
