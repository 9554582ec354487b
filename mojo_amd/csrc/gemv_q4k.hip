// Q4_K decode kernel for m <= 16 lhs rows: packed weights streamed once with
// fully coalesced 128-bit loads, nibbles used directly as fp16 operands of the
// matrix cores.
//
// Arithmetic.  A 4-bit code q, masked in place, is the fp16 subnormal q*2^-24
// (low nibble) or q*2^-20 (high nibble, still inside its byte), so unpacking is
// one AND per two weights.  One packed fp16 multiply per two weights folds the
// 6-bit sub-block scale in: q*sc <= 945 is exact in fp16.  Activations are split
// into fp16 hi + lo parts (22 significant bits) after an exact power-of-two
// scaling per (lhs row, 256-wide super-block); all products are exact in the
// fp32 accumulators of the matrix core.  Per super-block
//   P[m]  = sum_k a[m][k] * (sc_j(k) * q[k])            16 products, one chain
//   Pm[m] = sum_j mn_j * (sum_{k in j} a[m][k])          1 product
//   out[m][n] += d * P - dmin * Pm                        fp32, in the lanes.
//
// Mapping.  One v_mfma_f32_32x32x16_f16 column is one super-block: a wavefront
// step covers RT weight rows x S consecutive super-blocks (RT * S = 32 columns,
// S * MT <= 16), i.e. RT runs of S*144 contiguous bytes, loaded with consecutive
// lanes on consecutive 16-byte units and turned into the per-column operand
// order through a wavefront-private LDS buffer.  Column j = r*S + s is block
// S*t + s of row r; lane (j, g = lane/32) takes the 16 bytes [32c+16g, +16) of
// chunk c: low nibbles are weights 64c+16g+i of sub-block 2c, high nibbles the
// same offsets of sub-block 2c+1.  The A operand rows carry the activations of
// the S super-blocks: row 8*(v/4) + (v%4) holds the hi part and that row + 4 the
// lo part of virtual lhs row v = s*MT + m; only the diagonal (column's own s) of
// the product is used.
//
// Schedule.  Workgroups are persistent and stage the activations in LDS once
// per K slice.  Every wavefront owns whole weight rows, so no partial sums cross
// wavefronts; it keeps three steps of loads in flight, the first issued before
// the activations are touched.
#include <stdlib.h>

#include "qmm_internal.h"

namespace qmm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

namespace {

union HalfPack {
    uint32_t u[4];
    half8 h;
};

__device__ __forceinline__ half8 pack4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    HalfPack p;
    p.u[0] = a;
    p.u[1] = b;
    p.u[2] = c;
    p.u[3] = d;
    return p.h;
}

__device__ __forceinline__ uint32_t pack_half2(float x, float y) {
    return (uint32_t)f2h(x) | ((uint32_t)f2h(y) << 16);
}

// (x.lo * s.lo, x.hi * s.hi) on packed fp16 pairs held in dwords.
__device__ __forceinline__ uint32_t pk_mul(uint32_t x, uint32_t s) {
    union { uint32_t u; half2v h; } a, b, r;
    a.u = x;
    b.u = s;
    r.h = a.h * b.h;
    return r.u;
}

constexpr float kTwo24 = 16777216.0f;
constexpr int kRing = 3;            // wavefront steps of loads in flight
constexpr int kStepBytes = 32 * 144;  // one step: 32 super-blocks

// (lhs row, super-block) units a wavefront stages per slice
constexpr int stage_units(int) { return 16; }
// bytes of the inverse-scale table, padded so that what follows stays 16-byte aligned
__host__ __device__ constexpr size_t inv_bytes(int bs, int mt) { return ((size_t)bs * mt * 4 + 15) & ~(size_t)15; }
__host__ __device__ constexpr size_t lds_bytes(int bs, int mt, int waves) {
    return (size_t)bs * 1056 * mt + inv_bytes(bs, mt) + 16 + (size_t)waves * kStepBytes;
}
// super-blocks per weight row in one step
constexpr int blocks_per_step(int mt) { return mt <= 2 ? 8 : 16 / mt; }

struct StepRegs {
    uint4 v[5];  // 4.5 wavefront loads of 64 x 16 bytes
};

// Walks a wavefront's (slice, tile, step) units in processing order.
struct UnitIter {
    int b0, tile, t;
    __device__ __forceinline__ void advance(int steps, int t0, int t1, int BS) {
        if (++t == steps) {
            t = 0;
            if (++tile == t1) {
                tile = t0;
                b0 += BS;
            }
        }
    }
};

}  // namespace

// LDS layout (bytes), BS = super-blocks per K slice, MT = lhs row capacity:
//   act   [BS][4 chunks][4 mfma][2 g][2*MT rows][8 halfs]   = BS * 1024 * MT
//   asum  [BS][2 g][MT rows][8 halfs]                       = BS * 32 * MT
//   inv   [BS][MT] floats: inverse of the power-of-two activation scale
//   zero  16 bytes read by lanes whose A-operand row holds no lhs row
//   wbuf  [waves][4608]: one step of packed weights per wavefront
template <int MT, typename AT>
__global__ __launch_bounds__(512) void gemv_q4_k_mfma_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                             float* __restrict__ out, int m, int n, int k,
                                                             int slice_blocks, int64_t ldo) {
    constexpr int S = blocks_per_step(MT);  // super-blocks per row and step
    constexpr int RT = 32 / S;              // weight rows per step
    constexpr int U = 9 * S;                // 16-byte units per row and step
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int nwaves = blockDim.x >> 6;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps index math scalar
    const int nl = lane & 31, g = lane >> 5;
    const int nblk = k >> 8;
    const int BS = slice_blocks;  // a multiple of S unless it covers all of K
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;

    _Float16* act = (_Float16*)smem;
    _Float16* asum = (_Float16*)(smem + (size_t)BS * 1024 * MT);
    float* inv = (float*)(smem + (size_t)BS * 1056 * MT);
    _Float16* zero16 = (_Float16*)(smem + (size_t)BS * 1056 * MT + inv_bytes(BS, MT));
    uint8_t* wbuf = (uint8_t*)(zero16 + 8) + (size_t)wave * kStepBytes;

    // this wavefront's row tiles (RT rows each)
    const int ntiles = (n + RT - 1) / RT;
    const int gw = blockIdx.x * nwaves + wave, GW = gridDim.x * nwaves;
    // balanced contiguous split without 64-bit division: the first (ntiles % GW) wavefronts take one more
    const int tq = ntiles / GW, tr = ntiles - tq * GW;
    const int t0 = gw * tq + min(gw, tr);
    const int t1 = t0 + tq + (gw < tr ? 1 : 0);
    const bool has_work = t0 < t1;
    const int steps = (min(BS, nblk) + S - 1) / S;  // steps per (slice, tile)

    // ---- first slice's activation loads go out first, then the weight ring
    constexpr int kStageUnits = stage_units(MT);
    float4 sreg[kStageUnits];
    auto stage_load = [&](int b0, int bs) {
        int mi = wave / bs, bb = wave - mi * bs;
#pragma unroll
        for (int j = 0; j < kStageUnits; j++) {
            if (j > 0) {
                bb += nwaves;
                while (bb >= bs) {
                    bb -= bs;
                    mi++;
                }
            }
            sreg[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (mi < m) {
                const int64_t gk = (int64_t)mi * k + (int64_t)(b0 + bb) * 256 + lane * 4;
                if constexpr (sizeof(AT) == 4) {
                    sreg[j] = *(const float4*)(a + gk);
                } else {
                    uint2 v = *(const uint2*)(a + gk);
                    sreg[j] = make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                                          __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
                }
            }
        }
    };
    stage_load(0, min(BS, nblk));

    // One step of loads: unit u = it*64 + lane is 16-byte unit (u % U) of row (u / U) of the
    // tile, starting at super-block b_first.  Out-of-range rows and blocks are clamped to
    // valid addresses here and masked when used.
    auto load_step = [&](StepRegs& r, int tile, int b_first) {
#pragma unroll
        for (int it = 0; it < 5; it++) {
            const int u = it * 64 + lane;
            if (it < 4 || lane < 32) {
                int row = tile * RT + u / U;
                const int unit = u % U;
                int blk = b_first + unit / 9;
                if (row >= n) row = n - 1;
                if (blk >= nblk) blk = nblk - 1;
                r.v[it] = *(const uint4*)(w + (int64_t)row * row_bytes + (int64_t)blk * Q4_K_BPB + (unit % 9) * 16);
            }
        }
    };

    StepRegs ring[kRing];
    UnitIter pref = {0, t0, 0};
#pragma unroll
    for (int s = 0; s < kRing; s++) {
#pragma unroll
        for (int it = 0; it < 5; it++) ring[s].v[it] = make_uint4(0, 0, 0, 0);
        if (has_work && pref.b0 < nblk) {
            load_step(ring[s], pref.tile, pref.b0 + pref.t * S);
            pref.advance(steps, t0, t1, BS);
        }
    }

    // this lane's column: weight row r_col of the tile, super-block s_col of the step
    const int r_col = nl / S, s_col = nl % S;
    // this lane's A-operand row: part v_a (0 hi, 1 lo) of virtual lhs row -> (s_a, m_a)
    const int vrow = 4 * (nl >> 3) + (nl & 3), v_a = (nl >> 2) & 1;
    const int s_a = vrow / MT, m_a = vrow % MT;
    const bool a_row_ok = s_a < S && m_a < m;
    if (tid < 8) zero16[tid] = (_Float16)0.0f;

    float acc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) acc[i] = 0.0f;

    // One step: bb0 = first super-block of the step relative to the slice, bs = blocks in the slice.
    auto process = [&](const StepRegs& sr, int tile, int bb0, int bs) {
        // packed bytes -> LDS in load order, back in column order
#pragma unroll
        for (int it = 0; it < 5; it++)
            if (it < 4 || lane < 32) *(uint4*)(wbuf + (size_t)(it * 64 + lane) * 16) = sr.v[it];
        const uint8_t* col = wbuf + (size_t)nl * Q4_K_BPB;
        uint4 hdr = *(const uint4*)col;
        uint4 q[4];
#pragma unroll
        for (int c = 0; c < 4; c++) q[c] = *(const uint4*)(col + 16 + 32 * c + 16 * g);
        const int bb_col = bb0 + s_col;
        const bool col_ok = bb_col < bs && tile * RT + r_col < n;
        if (!col_ok) hdr = make_uint4(0, 0, 0, 0);  // d = dmin = 0, scales 0: the column contributes nothing
        const int bb_inv = col_ok ? bb_col : 0;

        const float d = h2f((uint16_t)(hdr.x & 0xffffu)) * kTwo24;
        const float dmin = h2f((uint16_t)(hdr.x >> 16)) * kTwo24;
        const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
        const uint32_t sc_lo = s0 & 0x3F3F3F3Fu, sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
        const uint32_t mn_lo = s1 & 0x3F3F3F3Fu, mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
        // packed (sc, sc) per sub-block; odd sub-blocks sit in the high nibbles and take sc/16
        uint32_t sp[8];
        {
            const float e0 = (float)(sc_lo & 0xffu), e1 = 0.0625f * (float)((sc_lo >> 8) & 0xffu);
            const float e2 = (float)((sc_lo >> 16) & 0xffu), e3 = 0.0625f * (float)(sc_lo >> 24);
            const float e4 = (float)(sc_hi & 0xffu), e5 = 0.0625f * (float)((sc_hi >> 8) & 0xffu);
            const float e6 = (float)((sc_hi >> 16) & 0xffu), e7 = 0.0625f * (float)(sc_hi >> 24);
            sp[0] = pack_half2(e0, e0); sp[1] = pack_half2(e1, e1); sp[2] = pack_half2(e2, e2); sp[3] = pack_half2(e3, e3);
            sp[4] = pack_half2(e4, e4); sp[5] = pack_half2(e5, e5); sp[6] = pack_half2(e6, e6); sp[7] = pack_half2(e7, e7);
        }
        // this lane's A-operand row reads the activations of super-block bb0 + s_a
        const int bb_a = bb0 + s_a;
        const bool a_ok = a_row_ok && bb_a < bs;
        float16v P = {0}, Pm = {0};
        {
            const _Float16* sp_ptr = (a_ok && v_a == 0) ? asum + ((size_t)(bb_a * 2 + g) * MT + m_a) * 8 : zero16;
            const half8 av = *(const half8*)sp_ptr;
            const half8 bv = pack4(mn_lo & 0x00FF00FFu, (mn_lo >> 8) & 0x00FF00FFu, mn_hi & 0x00FF00FFu,
                                   (mn_hi >> 8) & 0x00FF00FFu);
            Pm = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, Pm, 0, 0, 0);
        }
        const size_t fstride = a_ok ? (size_t)2 * (2 * MT) * 8 : 0;  // halfs between consecutive mfma operands
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint4 x = q[c];
            const _Float16* ap =
                a_ok ? act + ((((size_t)(bb_a * 4 + c) * 4) * 2 + g) * (2 * MT) + v_a * MT + m_a) * 8 : zero16;
            const half8 a0 = *(const half8*)(ap);
            const half8 a1 = *(const half8*)(ap + fstride);
            const half8 a2 = *(const half8*)(ap + 2 * fstride);
            const half8 a3 = *(const half8*)(ap + 3 * fstride);
            const uint32_t xs = x.x >> 8, ys = x.y >> 8, zs = x.z >> 8, ws = x.w >> 8;
            const uint32_t M1 = 0x000F000Fu, M2 = 0x00F000F0u;
            const uint32_t se = sp[2 * c], so = sp[2 * c + 1];
            P = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                a0, pack4(pk_mul(x.x & M1, se), pk_mul(xs & M1, se), pk_mul(x.y & M1, se), pk_mul(ys & M1, se)), P, 0, 0, 0);
            P = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                a1, pack4(pk_mul(x.z & M1, se), pk_mul(zs & M1, se), pk_mul(x.w & M1, se), pk_mul(ws & M1, se)), P, 0, 0, 0);
            P = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                a2, pack4(pk_mul(x.x & M2, so), pk_mul(xs & M2, so), pk_mul(x.y & M2, so), pk_mul(ys & M2, so)), P, 0, 0, 0);
            P = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                a3, pack4(pk_mul(x.z & M2, so), pk_mul(zs & M2, so), pk_mul(x.w & M2, so), pk_mul(ws & M2, so)), P, 0, 0, 0);
        }
        // diagonal of the product: this column's own super-block rows
        float vP[MT], vM[MT];
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            vP[mi] = P[mi];
            vM[mi] = Pm[mi];
        }
#pragma unroll
        for (int ss = 1; ss < S; ss++) {
            const bool hit = s_col == ss;
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                vP[mi] = hit ? P[ss * MT + mi] : vP[mi];
                vM[mi] = hit ? Pm[ss * MT + mi] : vM[mi];
            }
        }
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const float t = fmaf(d, vP[mi], -dmin * vM[mi]);
            acc[mi] = fmaf(inv[bb_inv * MT + mi], t, acc[mi]);
        }
    };

    int slot = 0;
    for (int b0 = 0; b0 < nblk; b0 += BS) {
        const int bs = min(BS, nblk - b0);
        if (b0 > 0) {
            __syncthreads();  // previous slice fully consumed
            stage_load(b0, bs);
        }
        // ---- stage this slice's activations as fp16 hi/lo in A-operand order:
        //      one wavefront per (lhs row, super-block), four consecutive k per lane
        int mi = wave / bs, bb = wave - mi * bs;
#pragma unroll
        for (int j = 0; j < kStageUnits; j++) {
            if (j > 0) {
                bb += nwaves;
                while (bb >= bs) {
                    bb -= bs;
                    mi++;
                }
            }
            if (mi < m) {
                const int kb = lane * 4;
                float x0 = sreg[j].x, x1 = sreg[j].y, x2 = sreg[j].z, x3 = sreg[j].w;
                // power-of-two scale bringing the super-block's largest magnitude into [2^9, 2^10)
                const float mx4 = fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3)));
                const uint32_t mxb = wave_max_nonneg_bits(mx4);
                int e = (int)((mxb >> 23) & 0xffu) - 127;
                if (e < -100 || e > 127) e = 9;  // zero, denormal or non-finite: leave unscaled
                const float s = __uint_as_float((uint32_t)(127 + 9 - e) << 23);
                x0 *= s; x1 *= s; x2 *= s; x3 *= s;
                const float h0 = h2f(f2h(x0)), h1 = h2f(f2h(x1)), h2 = h2f(f2h(x2)), h3 = h2f(f2h(x3));
                const int c = kb >> 6, hin = (kb >> 5) & 1, gg = (kb >> 4) & 1, t = kb & 15;
                const int f = 2 * hin + (t >> 3);
                // 8-half operand row; bytes t..t+3 sit at slots (0,2,1,3) of the half selected by t&4
                const size_t base = ((((size_t)(bb * 4 + c) * 4 + f) * 2 + gg) * (2 * MT)) * 8 + (t & 4);
                *(uint2*)(act + base + (size_t)mi * 8) = make_uint2(pack_half2(h0, h2), pack_half2(h1, h3));
                *(uint2*)(act + base + (size_t)(MT + mi) * 8) =
                    make_uint2(pack_half2(x0 - h0, x2 - h2), pack_half2(x1 - h1, x3 - h3));
                // sub-block activation sum over 8 consecutive lanes (32 k)
                const float sum = sum8((x0 + x1) + (x2 + x3));
                if ((lane & 7) == 0) {
                    const int jj = lane >> 3;  // sub-block 0..7 -> operand slot order (0,2,1,3,4,6,5,7)
                    const int pos = (jj & 4) | ((jj & 1) << 1) | ((jj >> 1) & 1);
                    const float sh = h2f(f2h(sum));
                    asum[((size_t)(bb * 2 + 0) * MT + mi) * 8 + pos] = (_Float16)sh;
                    asum[((size_t)(bb * 2 + 1) * MT + mi) * 8 + pos] = (_Float16)(sum - sh);
                }
                if (lane == 0) inv[bb * MT + mi] = __uint_as_float((uint32_t)(127 - 9 + e) << 23);
            }
        }
        __syncthreads();

        // ---- stream this wavefront's row tiles over the slice; the ring slot follows the
        //      wavefront's running step count, so it carries across tiles and slices
        const int steps_here = (bs + S - 1) / S;
        for (int tile = t0; tile < t1; tile++) {
            for (int t = 0; t < steps; t++) {
                int ptile = -1, pblk = 0;
                if (pref.b0 < nblk) {
                    ptile = pref.tile;
                    pblk = pref.b0 + pref.t * S;
                    pref.advance(steps, t0, t1, BS);
                }
#define QMM_STEP(R)                                                   \
    do {                                                              \
        if (t < steps_here) process(ring[R], tile, t * S, bs);        \
        if (ptile >= 0) load_step(ring[R], ptile, pblk);              \
    } while (0)
                switch (slot) {
                    case 0: QMM_STEP(0); break;
                    case 1: QMM_STEP(1); break;
                    default: QMM_STEP(2); break;
                }
#undef QMM_STEP
                slot = slot == kRing - 1 ? 0 : slot + 1;
            }
            // sum the S columns of each weight row and the hi/lo halves
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                float v = acc[mi];
                if (S >= 2) v += dpp_move<0xB1>(v);
                if (S >= 4) v += dpp_move<0x4E>(v);
                if (S >= 8) v += dpp_move<0x141>(v);
                v += __shfl_xor(v, 32, 64);
                const int row = tile * RT + r_col;
                if (s_col == 0 && g == 0 && mi < m && row < n) {
                    float* o = out + (int64_t)mi * ldo + row;
                    *o = (b0 == 0) ? v : *o + v;
                }
                acc[mi] = 0.0f;
            }
        }
    }
}

// QMM_GEMV_WAVES=<n> / QMM_GEMV_GRID=<n> override the launch shape (tuning aids).
static int env_int(const char* name) {
    const char* e = getenv(name);
    return e ? atoi(e) : 0;
}

hipError_t launch_gemv_q4_k_mfma(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                                 float* out, int64_t ldo, hipStream_t s) {
    static const int waves_env = env_int("QMM_GEMV_WAVES"), grid_env = env_int("QMM_GEMV_GRID");
    static const int num_cu = [] {
        int dev = 0, cu = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev);
        return cu > 0 ? cu : 256;
    }();
    const int nblk = (int)(k >> 8);
    const int mt = m <= 1 ? 1 : (m <= 2 ? 2 : (m <= 4 ? 4 : (m <= 8 ? 8 : 16)));
    const int S = blocks_per_step(mt), RT = 32 / S;
    const int kStageUnits = stage_units(mt);
    const size_t lds_budget = 112 * 1024;
    const int ntiles = (int)((n + RT - 1) / RT);
    int grid_x = grid_env > 0 ? grid_env : num_cu;
    // Wavefronts per workgroup: enough to give every wavefront a row tile, at most 8.
    // Super-blocks per K slice: a wavefront stages at most kStageUnits (lhs row, super-block)
    // units per slice, a slice holds a multiple of S super-blocks (or all of K), and
    // everything fits the LDS budget.
    int waves = waves_env > 0 ? waves_env : (ntiles + grid_x - 1) / grid_x;
    if (waves > 8) waves = 8;
    if (waves < 1) waves = 1;
    int bs = kStageUnits * waves / mt;
    if (bs >= nblk) bs = nblk;
    else bs = bs / S * S;
    while (bs > S && lds_bytes(bs, mt, waves) > lds_budget) bs -= S;
    if (bs < 1) bs = nblk < S ? nblk : S;
    const int max_grid = (ntiles + waves - 1) / waves;
    if (grid_x > max_grid) grid_x = max_grid;
    size_t smem = lds_bytes(bs, mt, waves);
    dim3 grid((unsigned)grid_x), block(waves * 64);
#define QMM_LAUNCH(MT)                                                                                         \
    do {                                                                                                       \
        static const bool attr_set = [] {                                                                      \
            (void)hipFuncSetAttribute((const void*)gemv_q4_k_mfma_kernel<MT, float>,                           \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);                 \
            (void)hipFuncSetAttribute((const void*)gemv_q4_k_mfma_kernel<MT, uint16_t>,                        \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);                 \
            return true;                                                                                       \
        }();                                                                                                   \
        (void)attr_set;                                                                                        \
        if (a_dtype == QMM_F32)                                                                                \
            gemv_q4_k_mfma_kernel<MT, float><<<grid, block, smem, s>>>(w, (const float*)a, out, m, (int)n, (int)k, bs, ldo); \
        else                                                                                                   \
            gemv_q4_k_mfma_kernel<MT, uint16_t><<<grid, block, smem, s>>>(w, (const uint16_t*)a, out, m, (int)n, (int)k, bs, ldo); \
    } while (0)
    switch (mt) {
        case 1: QMM_LAUNCH(1); break;
        case 2: QMM_LAUNCH(2); break;
        case 4: QMM_LAUNCH(4); break;
        case 8: QMM_LAUNCH(8); break;
        default: QMM_LAUNCH(16); break;
    }
#undef QMM_LAUNCH
    return hipGetLastError();
}

}  // namespace qmm
