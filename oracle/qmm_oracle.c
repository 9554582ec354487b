/*
 * qmm_oracle.c -- CPU restatement of the quantized-weight matmul path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the timed CPU baseline; it is never linked into, loaded
 * by or called from the shipped library or its Python host layer.
 *
 * What it restates.  The reference snapshot (modularml/mojo, Mojo v24.6) does
 * not contain MAX's qmatmul kernels: MAX is an un-vendored binary dependency
 * (pixi.toml:12-15, magic.lock:135-137, max 24.6.0).  The arithmetic below
 * therefore follows the published GGUF (ggml-common.h / ggml-quants.c) and
 * AutoGPTQ block formats, and, from the reference tree, only its numeric
 * substrate:
 *   - bf16 narrowing = round-to-nearest-even with canonical NaN
 *     (stdlib/src/builtin/simd.mojo:3279-3300),
 *   - half types accumulate in fp32 (stdlib/src/utils/numerics.mojo:1031-1048),
 *   - little-endian lane order of packed fields
 *     (stdlib/test/memory/test_bitcast.mojo:19-28),
 *   - the symmetric isclose tolerance used by the tests
 *     (stdlib/src/math/math.mojo:1023-1030),
 *   - rows of N split across host cores (examples/matmul.mojo:126-141).
 *
 * Pinning status of each function (what the unit tests check it against):
 *   qo_f16_to_f32 / qo_f32_to_f16     pinned: exhaustive vs IEEE binary16 (numpy)
 *   qo_f32_to_bf16                    pinned: reference rule above + torch
 *   qo_unpack_scales_q4_k             pinned: pack/unpack round trip over all
 *                                     8 positions x 64 x 64 values + hand KAT
 *   qo_dequantize (Q4_0/Q4_K/Q5_K/Q6_K), qo_dequantize_gptq
 *                                     pinned: hand-worked known-answer blocks,
 *                                     exactness lemma brute force, independent
 *                                     vectorised restatement; the g_idx (act-
 *                                     order) route: identity with k / group,
 *                                     and equality with the sorted-order weight
 *                                     whose columns are put back
 *   qo_block_dots_q4_0_q8_0           pinned: integer arithmetic, brute force vs
 *                                     int64, extreme vectors
 *   qo_matmul_* outputs               pinned: fp64 truth, closed-form special
 *                                     cases (one-hot, constant-code blocks)
 *   qo_baseline_matmul_q4_k           timed baseline only, never a checker: held
 *                                     to the matmul tolerance against
 *                                     qo_matmul_f32 and the fp64 truth
 *   qo_quantize_q4_0 / qo_quantize_q8_0
 *                                     closed form pinned by properties (argmax
 *                                     -> code 0 / +-127, error bound, ties);
 *                                     the choice of rounding rule itself
 *                                     (roundf, fp16 scale) is PARITY UNPINNED:
 *                                     nothing in the reference fixes it.
 *   qo_quantize_q4_k / qo_quantize_q5_k / qo_quantize_q6_k / qo_quantize_gptq
 *                                     PARITY UNPINNED: these are this build's
 *                                     own simple packers (ggml's iterative
 *                                     search is not restated); they exist to
 *                                     make valid packed bytes, and the same
 *                                     bytes feed oracle and GPU.
 *   activation treatment for Q4_K/Q6_K (fp32 activations, no Q8_K step)
 *                                     PARITY UNPINNED: taken from the workload
 *                                     description, not from reference source.
 *   qo_quantize_q8_k, qo_block_sums_q4_k_q8_k, qo_matmul_q4_k_q8_k
 *                                     the alternative ggml-lineage CPU kernels
 *                                     compute (activations -> Q8_K, integer
 *                                     sub-block dots): integer sums pinned by
 *                                     brute force vs int64 and by the identity
 *                                     with the fp32 path on exactly
 *                                     representable activations; the quantiser
 *                                     by its properties (largest element ->
 *                                     -127, round-half-even, bsums).  Which of
 *                                     the two treatments the reference uses is
 *                                     PARITY UNPINNED (see the line above).
 *   qo_block_sums_kquant_q8_k, qo_matmul_kquant_act_q8_k
 *                                     the same treatment for Q5_K and Q6_K
 *                                     weights: integer sums pinned by brute
 *                                     force vs int64 over an independent
 *                                     unpack of the blocks, the matmul by the
 *                                     identity with the fp64 product on
 *                                     activations that Q8_K represents exactly,
 *                                     and by equality with the Q4_K functions
 *                                     above for enc = Q4_K.
 *   qo_rmsnorm                        the normalisation in front of the op in a
 *                                     Llama block, y = x * rsqrt(mean(x^2) + eps)
 *                                     * gamma: pinned by closed forms (constant
 *                                     rows, sum of squares of y / gamma = K at
 *                                     eps = 0, invariance under scaling of x)
 *                                     and an independent fp64 restatement.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define QO_Q4_0 0
#define QO_Q4_K 1
#define QO_Q6_K 2
#define QO_GPTQ 3
#define QO_Q5_K 4

/* ------------------------------------------------------------------ */
/* scalar conversions                                                  */
/* ------------------------------------------------------------------ */

float qo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t qo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) { /* inf / nan */
        if (x == 0x7f800000u) return sign | 0x7c00u;
        uint16_t r = (uint16_t)(0x7c00u + ((x & 0x7fffffu) >> 13));
        if (r == 0x7c00u) r++;
        return sign | r;
    }
    uint32_t e = x >> 23;
    if (e >= 113) { /* normal half (or overflow) */
        uint32_t man = x & 0x7fffffu;
        uint32_t h = ((e - 112u) << 10) | (man >> 13);
        uint32_t rem = man & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
        if (h >= 0x7c00u) h = 0x7c00u;
        return sign | (uint16_t)h;
    }
    if (e < 102) return sign; /* below half of the smallest subnormal */
    uint32_t man = (x & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e; /* 14..24 */
    uint32_t h = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (h & 1u))) h++;
    return sign | (uint16_t)h;
}

/* Reference rule: stdlib/src/builtin/simd.mojo:3279-3300. */
uint16_t qo_f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(((x >> 16) & 0x8000u) | 0x7fc0u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

float qo_bf16_to_f32(uint16_t h) {
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void qo_f16_to_f32_n(const uint16_t* h, int64_t n, float* out) {
    for (int64_t i = 0; i < n; i++) out[i] = qo_f16_to_f32(h[i]);
}
void qo_f32_to_f16_n(const float* f, int64_t n, uint16_t* out) {
    for (int64_t i = 0; i < n; i++) out[i] = qo_f32_to_f16(f[i]);
}
void qo_f32_to_bf16_n(const float* f, int64_t n, uint16_t* out) {
    for (int64_t i = 0; i < n; i++) out[i] = qo_f32_to_bf16(f[i]);
}

/*
 * RMS normalisation of each row: y = (x * rs) * gamma with rs = 1 / sqrt(mean(x^2) + eps) as a float, the mean summed in
 * double; to_bf16 != 0 rounds y to bf16 (the value a bf16 normalisation node hands on) and returns it widened again.
 */
void qo_rmsnorm(const float* x, const float* gamma, float eps, int64_t rows, int64_t k, int to_bf16, float* y) {
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * k;
        double ss = 0.0;
        for (int64_t i = 0; i < k; i++) ss += (double)xr[i] * (double)xr[i];
        const float rs = (float)(1.0 / sqrt(ss / (double)k + (double)eps));
        for (int64_t i = 0; i < k; i++) {
            float v = (xr[i] * rs) * gamma[i];
            if (to_bf16) {
                uint32_t u = (uint32_t)qo_f32_to_bf16(v) << 16;
                memcpy(&v, &u, 4);
            }
            y[r * k + i] = v;
        }
    }
}

static inline float rd_f16(const uint8_t* p) {
    return qo_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
}
static inline void wr_f16(uint8_t* p, float f) {
    uint16_t h = qo_f32_to_f16(f);
    p[0] = (uint8_t)(h & 0xff);
    p[1] = (uint8_t)(h >> 8);
}

int qo_block_params(int enc, int64_t* epb, int64_t* bpb) {
    switch (enc) {
        case QO_Q4_0: *epb = 32; *bpb = 18; return 0;
        case QO_Q4_K: *epb = 256; *bpb = 144; return 0;
        case QO_Q6_K: *epb = 256; *bpb = 210; return 0;
        case QO_Q5_K: *epb = 256; *bpb = 176; return 0;
        default: return -1;
    }
}

/* ------------------------------------------------------------------ */
/* Q4_0 / Q8_0 quantisers (ggml quantize_row_q4_0_ref / q8_0_ref form) */
/* ------------------------------------------------------------------ */

void qo_quantize_q4_0(const float* x, int64_t rows, int64_t k, uint8_t* out) {
    int64_t nb = k / 32;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t b = 0; b < nb; b++) {
            const float* xb = x + r * k + b * 32;
            uint8_t* ob = out + (r * nb + b) * 18;
            float amax = 0.0f, mx = 0.0f;
            for (int j = 0; j < 32; j++) {
                float v = xb[j];
                if (amax < fabsf(v)) {
                    amax = fabsf(v);
                    mx = v;
                }
            }
            float d = mx / -8.0f;
            float id = d != 0.0f ? 1.0f / d : 0.0f;
            wr_f16(ob, d);
            for (int j = 0; j < 16; j++) {
                float x0 = xb[j] * id;
                float x1 = xb[j + 16] * id;
                int q0 = (int)(int8_t)(x0 + 8.5f);
                int q1 = (int)(int8_t)(x1 + 8.5f);
                if (q0 > 15) q0 = 15;
                if (q1 > 15) q1 = 15;
                ob[2 + j] = (uint8_t)(q0 | (q1 << 4));
            }
        }
    }
}

void qo_quantize_q8_0(const float* x, int64_t rows, int64_t k, uint8_t* out) {
    int64_t nb = k / 32;
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t b = 0; b < nb; b++) {
            const float* xb = x + r * k + b * 32;
            uint8_t* ob = out + (r * nb + b) * 34;
            float amax = 0.0f;
            for (int j = 0; j < 32; j++) {
                float v = fabsf(xb[j]);
                if (amax < v) amax = v;
            }
            float d = amax / 127.0f;
            float id = d != 0.0f ? 1.0f / d : 0.0f;
            wr_f16(ob, d);
            for (int j = 0; j < 32; j++) {
                ob[2 + j] = (uint8_t)(int8_t)roundf(xb[j] * id);
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* K-quant and GPTQ packers (this build's own; see header)             */
/* ------------------------------------------------------------------ */

static inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* 12 bytes <- 8 x (6-bit scale, 6-bit min); inverse of qo_unpack_scales_q4_k. */
void qo_pack_scales_q4_k(const uint8_t* sc, const uint8_t* mn, uint8_t* s) {
    memset(s, 0, 12);
    for (int j = 0; j < 8; j++) {
        if (j < 4) {
            s[j] |= sc[j] & 63;
            s[j + 4] |= mn[j] & 63;
        } else {
            s[j + 4] = (uint8_t)((sc[j] & 0xF) | ((mn[j] & 0xF) << 4));
            s[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
            s[j] |= (uint8_t)((mn[j] >> 4) << 6);
        }
    }
}

void qo_unpack_scales_q4_k(const uint8_t* s, uint8_t* sc, uint8_t* mn) {
    for (int j = 0; j < 8; j++) {
        if (j < 4) {
            sc[j] = s[j] & 63;
            mn[j] = s[j + 4] & 63;
        } else {
            sc[j] = (uint8_t)((s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4));
            mn[j] = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
        }
    }
}

void qo_quantize_q4_k(const float* x, int64_t rows, int64_t k, uint8_t* out) {
    int64_t nb = k / 256;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t b = 0; b < nb; b++) {
            const float* xb = x + r * k + b * 256;
            uint8_t* ob = out + (r * nb + b) * 144;
            float scale[8], minv[8];
            float max_scale = 0.0f, max_min = 0.0f;
            for (int j = 0; j < 8; j++) {
                float lo = 0.0f, hi = 0.0f; /* lo <= 0 <= hi: offsets stay non-negative */
                for (int l = 0; l < 32; l++) {
                    float v = xb[j * 32 + l];
                    if (v < lo) lo = v;
                    if (v > hi) hi = v;
                }
                scale[j] = (hi - lo) / 15.0f;
                minv[j] = -lo;
                if (scale[j] > max_scale) max_scale = scale[j];
                if (minv[j] > max_min) max_min = minv[j];
            }
            float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
            float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
            uint8_t sc[8], mn[8];
            for (int j = 0; j < 8; j++) {
                sc[j] = (uint8_t)clampi((int)rintf(inv_scale * scale[j]), 0, 63);
                mn[j] = (uint8_t)clampi((int)rintf(inv_min * minv[j]), 0, 63);
            }
            wr_f16(ob, max_scale / 63.0f);
            wr_f16(ob + 2, max_min / 63.0f);
            qo_pack_scales_q4_k(sc, mn, ob + 4);
            float d = rd_f16(ob), dmin = rd_f16(ob + 2);
            uint8_t q[256];
            for (int j = 0; j < 8; j++) {
                float dl = d * (float)sc[j];
                float ml = dmin * (float)mn[j];
                for (int l = 0; l < 32; l++) {
                    int v = 0;
                    if (dl != 0.0f) v = clampi((int)rintf((xb[j * 32 + l] + ml) / dl), 0, 15);
                    q[j * 32 + l] = (uint8_t)v;
                }
            }
            for (int c = 0; c < 4; c++)
                for (int l = 0; l < 32; l++)
                    ob[16 + c * 32 + l] = (uint8_t)(q[c * 64 + l] | (q[c * 64 + 32 + l] << 4));
        }
    }
}

/* Q5_K: the Q4_K fit with 5-bit codes.  Block: f16 d, f16 dmin, 12 B scales (as Q4_K), qh[32], qs[128];
 * code j of chunk c (64 weights) has its low four bits in the low (j < 32) or high (j >= 32) nibble of
 * qs[32 c + j % 32] and its fifth bit in bit 2 c + j / 32 of qh[j % 32]. */
void qo_quantize_q5_k(const float* x, int64_t rows, int64_t k, uint8_t* out) {
    int64_t nb = k / 256;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t b = 0; b < nb; b++) {
            const float* xb = x + r * k + b * 256;
            uint8_t* ob = out + (r * nb + b) * 176;
            float scale[8], minv[8];
            float max_scale = 0.0f, max_min = 0.0f;
            for (int j = 0; j < 8; j++) {
                float lo = 0.0f, hi = 0.0f;
                for (int l = 0; l < 32; l++) {
                    float v = xb[j * 32 + l];
                    if (v < lo) lo = v;
                    if (v > hi) hi = v;
                }
                scale[j] = (hi - lo) / 31.0f;
                minv[j] = -lo;
                if (scale[j] > max_scale) max_scale = scale[j];
                if (minv[j] > max_min) max_min = minv[j];
            }
            float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
            float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
            uint8_t sc[8], mn[8];
            for (int j = 0; j < 8; j++) {
                sc[j] = (uint8_t)clampi((int)rintf(inv_scale * scale[j]), 0, 63);
                mn[j] = (uint8_t)clampi((int)rintf(inv_min * minv[j]), 0, 63);
            }
            wr_f16(ob, max_scale / 63.0f);
            wr_f16(ob + 2, max_min / 63.0f);
            qo_pack_scales_q4_k(sc, mn, ob + 4);
            float d = rd_f16(ob), dmin = rd_f16(ob + 2);
            uint8_t q[256];
            for (int j = 0; j < 8; j++) {
                float dl = d * (float)sc[j];
                float ml = dmin * (float)mn[j];
                for (int l = 0; l < 32; l++) {
                    int v = 0;
                    if (dl != 0.0f) v = clampi((int)rintf((xb[j * 32 + l] + ml) / dl), 0, 31);
                    q[j * 32 + l] = (uint8_t)v;
                }
            }
            uint8_t* qh = ob + 16;
            uint8_t* qs = ob + 48;
            memset(qh, 0, 32);
            for (int c = 0; c < 4; c++)
                for (int l = 0; l < 32; l++) {
                    uint8_t a = q[c * 64 + l], bb = q[c * 64 + 32 + l];
                    qs[c * 32 + l] = (uint8_t)((a & 0xF) | ((bb & 0xF) << 4));
                    qh[l] |= (uint8_t)(((a >> 4) << (2 * c)) | ((bb >> 4) << (2 * c + 1)));
                }
        }
    }
}

void qo_quantize_q6_k(const float* x, int64_t rows, int64_t k, uint8_t* out) {
    int64_t nb = k / 256;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t b = 0; b < nb; b++) {
            const float* xb = x + r * k + b * 256;
            uint8_t* ob = out + (r * nb + b) * 210;
            float scale[16];
            float amax_scale = 0.0f, max_scale = 0.0f;
            for (int j = 0; j < 16; j++) {
                float amax = 0.0f, mx = 0.0f;
                for (int l = 0; l < 16; l++) {
                    float v = xb[j * 16 + l];
                    if (amax < fabsf(v)) {
                        amax = fabsf(v);
                        mx = v;
                    }
                }
                scale[j] = mx / -32.0f;
                if (amax_scale < fabsf(scale[j])) {
                    amax_scale = fabsf(scale[j]);
                    max_scale = scale[j];
                }
            }
            int8_t* sc8 = (int8_t*)(ob + 192);
            if (amax_scale == 0.0f) {
                memset(ob, 0, 210);
                /* code 32 == value 0 */
                for (int i = 0; i < 128; i++) ob[i] = 0;
                for (int i = 0; i < 64; i++) ob[128 + i] = 0xAA;
                continue;
            }
            float iscale = -128.0f / max_scale;
            wr_f16(ob + 208, 1.0f / iscale);
            float d = rd_f16(ob + 208);
            uint8_t q[256];
            for (int j = 0; j < 16; j++) {
                int s = (int)rintf(iscale * scale[j]);
                if (s > 127) s = 127;
                if (s < -128) s = -128;
                sc8[j] = (int8_t)s;
                float dl = d * (float)s;
                for (int l = 0; l < 16; l++) {
                    int v = 0;
                    if (dl != 0.0f) v = clampi((int)rintf(xb[j * 16 + l] / dl), -32, 31);
                    q[j * 16 + l] = (uint8_t)(v + 32);
                }
            }
            for (int h = 0; h < 2; h++) {
                uint8_t* ql = ob + 64 * h;
                uint8_t* qh = ob + 128 + 32 * h;
                const uint8_t* qq = q + 128 * h;
                for (int l = 0; l < 32; l++) {
                    ql[l] = (uint8_t)((qq[l] & 0xF) | ((qq[l + 64] & 0xF) << 4));
                    ql[l + 32] = (uint8_t)((qq[l + 32] & 0xF) | ((qq[l + 96] & 0xF) << 4));
                    qh[l] = (uint8_t)((qq[l] >> 4) | ((qq[l + 32] >> 4) << 2) |
                                      ((qq[l + 64] >> 4) << 4) | ((qq[l + 96] >> 4) << 6));
                }
            }
        }
    }
}

/* AutoGPTQ v1 tensors, symmetric 4-bit.  w is [N, K] row-major (the transposed
 * weight, like the GGUF rhs); qweight int32[K/8, N], scales f16[K/group, N],
 * qzeros int32[K/group, N/8] (stored zero = 7), g_idx int32[K]. */
void qo_quantize_gptq(const float* w, int64_t n, int64_t k, int64_t group, int32_t* qweight,
                      uint16_t* scales, int32_t* qzeros, int32_t* g_idx) {
    int64_t ng = k / group;
    memset(qweight, 0, sizeof(int32_t) * (size_t)(k / 8 * n));
    memset(qzeros, 0, sizeof(int32_t) * (size_t)(ng * (n / 8)));
    for (int64_t kk = 0; kk < k; kk++) g_idx[kk] = (int32_t)(kk / group);
#pragma omp parallel for schedule(static)
    for (int64_t c8 = 0; c8 < n / 8; c8++) {
        for (int64_t col = c8 * 8; col < c8 * 8 + 8; col++) {
            for (int64_t g = 0; g < ng; g++) {
                float amax = 0.0f;
                for (int64_t kk = g * group; kk < (g + 1) * group; kk++) {
                    float v = fabsf(w[col * k + kk]);
                    if (amax < v) amax = v;
                }
                float scale = 2.0f * amax / 15.0f;
                scales[g * n + col] = qo_f32_to_f16(scale);
                qzeros[g * (n / 8) + col / 8] |= (int32_t)(7u << (4 * (col % 8)));
                for (int64_t kk = g * group; kk < (g + 1) * group; kk++) {
                    int q = 8;
                    if (scale != 0.0f) q = clampi((int)rintf(w[col * k + kk] / scale) + 8, 0, 15);
                    uint32_t* p = (uint32_t*)&qweight[(kk / 8) * n + col];
                    *p |= (uint32_t)q << (4 * (kk % 8));
                }
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* dequantisers                                                        */
/* ------------------------------------------------------------------ */

static void dequant_block_q4_0(const uint8_t* b, float* y) {
    float d = rd_f16(b);
    for (int j = 0; j < 16; j++) {
        y[j] = (float)((int)(b[2 + j] & 0xF) - 8) * d;
        y[j + 16] = (float)((int)(b[2 + j] >> 4) - 8) * d;
    }
}

static void dequant_block_q4_k(const uint8_t* b, float* y) {
    float d = rd_f16(b), dmin = rd_f16(b + 2);
    uint8_t sc[8], mn[8];
    qo_unpack_scales_q4_k(b + 4, sc, mn);
    const uint8_t* qs = b + 16;
    for (int c = 0; c < 4; c++) {
        float d1 = d * (float)sc[2 * c], m1 = dmin * (float)mn[2 * c];
        float d2 = d * (float)sc[2 * c + 1], m2 = dmin * (float)mn[2 * c + 1];
        for (int l = 0; l < 32; l++) {
            y[64 * c + l] = d1 * (float)(qs[32 * c + l] & 0xF) - m1;
            y[64 * c + 32 + l] = d2 * (float)(qs[32 * c + l] >> 4) - m2;
        }
    }
}

static void dequant_block_q5_k(const uint8_t* b, float* y) {
    float d = rd_f16(b), dmin = rd_f16(b + 2);
    uint8_t sc[8], mn[8];
    qo_unpack_scales_q4_k(b + 4, sc, mn);
    const uint8_t* qh = b + 16;
    const uint8_t* qs = b + 48;
    for (int c = 0; c < 4; c++) {
        float d1 = d * (float)sc[2 * c], m1 = dmin * (float)mn[2 * c];
        float d2 = d * (float)sc[2 * c + 1], m2 = dmin * (float)mn[2 * c + 1];
        for (int l = 0; l < 32; l++) {
            int q1 = (qs[32 * c + l] & 0xF) + (((qh[l] >> (2 * c)) & 1) << 4);
            int q2 = (qs[32 * c + l] >> 4) + (((qh[l] >> (2 * c + 1)) & 1) << 4);
            y[64 * c + l] = d1 * (float)q1 - m1;
            y[64 * c + 32 + l] = d2 * (float)q2 - m2;
        }
    }
}

static void dequant_block_q6_k(const uint8_t* b, float* y) {
    float d = rd_f16(b + 208);
    for (int h = 0; h < 2; h++) {
        const uint8_t* ql = b + 64 * h;
        const uint8_t* qh = b + 128 + 32 * h;
        const int8_t* sc = (const int8_t*)(b + 192 + 8 * h);
        float* yy = y + 128 * h;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
            int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            yy[l] = d * (float)sc[is + 0] * (float)q1;
            yy[l + 32] = d * (float)sc[is + 2] * (float)q2;
            yy[l + 64] = d * (float)sc[is + 4] * (float)q3;
            yy[l + 96] = d * (float)sc[is + 6] * (float)q4;
        }
    }
}

static void dequant_block(int enc, const uint8_t* b, float* y) {
    if (enc == QO_Q4_0) dequant_block_q4_0(b, y);
    else if (enc == QO_Q4_K) dequant_block_q4_k(b, y);
    else if (enc == QO_Q5_K) dequant_block_q5_k(b, y);
    else dequant_block_q6_k(b, y);
}

/* w: uint8[rows, k/epb*bpb] -> out fp32[rows, k] */
int qo_dequantize(int enc, const uint8_t* w, int64_t rows, int64_t k, float* out) {
    int64_t epb, bpb;
    if (qo_block_params(enc, &epb, &bpb) || k % epb) return -1;
    int64_t nb = k / epb;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++)
        for (int64_t b = 0; b < nb; b++)
            dequant_block(enc, w + (r * nb + b) * bpb, out + r * k + b * epb);
    return 0;
}

/* out fp32[N, K] (transposed orientation, like the GGUF rhs after dequant) */
void qo_dequantize_gptq(const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                        const int32_t* g_idx, int64_t n, int64_t k, int64_t group, float* out) {
#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < n; col++) {
        for (int64_t kk = 0; kk < k; kk++) {
            int64_t g = g_idx ? g_idx[kk] : kk / group; /* act-order checkpoints: any group per k */
            int q = (int)(((uint32_t)qweight[(kk / 8) * n + col] >> (4 * (kk % 8))) & 0xF);
            int z = (int)(((uint32_t)qzeros[g * (n / 8) + col / 8] >> (4 * (col % 8))) & 0xF) + 1;
            out[col * k + kk] = qo_f16_to_f32(scales[g * n + col]) * (float)(q - z);
        }
    }
}

/* ------------------------------------------------------------------ */
/* Q8_0 x Q4_0 integer block dots and the Q4_0 matmul                  */
/* ------------------------------------------------------------------ */

static inline int32_t block_dot_q4_0_q8_0(const uint8_t* wb, const uint8_t* ab) {
    const int8_t* a = (const int8_t*)(ab + 2);
    int32_t s = 0;
    for (int j = 0; j < 16; j++) {
        s += ((int)(wb[2 + j] & 0xF) - 8) * (int)a[j];
        s += ((int)(wb[2 + j] >> 4) - 8) * (int)a[j + 16];
    }
    return s;
}

/* out int32[M, N, K/32] */
void qo_block_dots_q4_0_q8_0(const uint8_t* a_q8, const uint8_t* w_q4, int64_t m, int64_t n,
                             int64_t k, int32_t* out) {
    int64_t nb = k / 32;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; j++)
        for (int64_t i = 0; i < m; i++)
            for (int64_t b = 0; b < nb; b++)
                out[(i * n + j) * nb + b] =
                    block_dot_q4_0_q8_0(w_q4 + (j * nb + b) * 18, a_q8 + (i * nb + b) * 34);
}

/* out[m, n] = sum_b isum(m,n,b) * (f32(d_w) * f32(d_a)), blocks in ascending order. */
void qo_matmul_q4_0_q8_0(const uint8_t* a_q8, const uint8_t* w_q4, int64_t m, int64_t n, int64_t k,
                         float* out) {
    int64_t nb = k / 32;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; j++) {
        for (int64_t i = 0; i < m; i++) {
            float acc = 0.0f;
            for (int64_t b = 0; b < nb; b++) {
                const uint8_t* wb = w_q4 + (j * nb + b) * 18;
                const uint8_t* ab = a_q8 + (i * nb + b) * 34;
                acc += (float)block_dot_q4_0_q8_0(wb, ab) * (rd_f16(wb) * rd_f16(ab));
            }
            out[i * n + j] = acc;
        }
    }
}

void qo_matmul_q4_0(const float* a, const uint8_t* w_q4, int64_t m, int64_t n, int64_t k,
                    float* out) {
    uint8_t* aq = (uint8_t*)malloc((size_t)(m * (k / 32) * 34));
    qo_quantize_q8_0(a, m, k, aq);
    qo_matmul_q4_0_q8_0(aq, w_q4, m, n, k, out);
    free(aq);
}

/* ------------------------------------------------------------------ */
/* Q8_K activations and the integer Q4_K dot (ggml block_q8_K:         */
/* float d; int8 qs[256]; int16 bsums[16]: 292 bytes)                  */
/* ------------------------------------------------------------------ */

/* round to nearest, ties to even, through the fp32 adder (ggml nearest_int) */
static inline int nearest_int(float f) {
    float v = f + 12582912.f;
    int i;
    memcpy(&i, &v, 4);
    return (i & 0x007fffff) - 0x00400000;
}

/* ggml quantize_row_q8_K_ref: max = the first element of largest magnitude (signed), iscale = -127 / max,
 * q = min(127, nearest_int(iscale * x)), d = 1 / iscale, bsums = sums of 16 codes.  An all-zero block has
 * d = 0, codes 0, bsums 0. */
void qo_quantize_q8_k(const float* x, int64_t rows, int64_t k, uint8_t* out) {
    int64_t nb = k / 256;
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t b = 0; b < nb; b++) {
            const float* xb = x + r * k + b * 256;
            uint8_t* ob = out + (r * nb + b) * 292;
            int8_t* qs = (int8_t*)(ob + 4);
            float max = 0.0f, amax = 0.0f;
            for (int j = 0; j < 256; j++) {
                float ax = fabsf(xb[j]);
                if (ax > amax) {
                    amax = ax;
                    max = xb[j];
                }
            }
            float d = 0.0f;
            if (amax == 0.0f) {
                memset(qs, 0, 256);
            } else {
                const float iscale = -127.f / max;
                for (int j = 0; j < 256; j++) {
                    int v = nearest_int(iscale * xb[j]);
                    qs[j] = (int8_t)(v > 127 ? 127 : v);
                }
                d = 1.0f / iscale;
            }
            memcpy(ob, &d, 4);
            for (int j = 0; j < 16; j++) {
                int sum = 0;
                for (int i = 0; i < 16; i++) sum += qs[j * 16 + i];
                int16_t s16 = (int16_t)sum;
                memcpy(ob + 260 + 2 * j, &s16, 2);
            }
        }
    }
}

/* integer sums of one Q4_K block against one Q8_K block:
 *   isum = sum_sub sc_sub * sum_32 q4 * q8,   msum = sum_sub mn_sub * (bsums[2 sub] + bsums[2 sub + 1]) */
static void block_sums_q4_k_q8_k(const uint8_t* wb, const uint8_t* ab, int32_t* isum, int32_t* msum) {
    uint8_t sc[8], mn[8];
    qo_unpack_scales_q4_k(wb + 4, sc, mn);
    const int8_t* q8 = (const int8_t*)(ab + 4);
    const uint8_t* qs = wb + 16;
    int32_t is = 0, ms = 0;
    for (int c = 0; c < 4; c++) {
        int32_t lo = 0, hi = 0;
        for (int t = 0; t < 32; t++) {
            lo += (int)(qs[32 * c + t] & 0xF) * (int)q8[64 * c + t];
            hi += (int)(qs[32 * c + t] >> 4) * (int)q8[64 * c + 32 + t];
        }
        is += (int32_t)sc[2 * c] * lo + (int32_t)sc[2 * c + 1] * hi;
    }
    for (int sub = 0; sub < 8; sub++) {
        int16_t b0, b1;
        memcpy(&b0, ab + 260 + 4 * sub, 2);
        memcpy(&b1, ab + 262 + 4 * sub, 2);
        ms += (int32_t)mn[sub] * ((int32_t)b0 + (int32_t)b1);
    }
    *isum = is;
    *msum = ms;
}

/* out int32[M, N, K/256] each */
void qo_block_sums_q4_k_q8_k(const uint8_t* a_q8k, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                             int32_t* isum, int32_t* msum) {
    int64_t nb = k / 256;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; j++)
        for (int64_t i = 0; i < m; i++)
            for (int64_t b = 0; b < nb; b++)
                block_sums_q4_k_q8_k(w + (j * nb + b) * 144, a_q8k + (i * nb + b) * 292,
                                     isum + (i * n + j) * nb + b, msum + (i * n + j) * nb + b);
}

/* out[m, n] = sum_b (d8 * f32(d)) * isum - (d8 * f32(dmin)) * msum, blocks in ascending order */
void qo_matmul_q4_k_q8_k(const uint8_t* a_q8k, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out) {
    int64_t nb = k / 256;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; j++) {
        for (int64_t i = 0; i < m; i++) {
            float acc = 0.0f;
            for (int64_t b = 0; b < nb; b++) {
                const uint8_t* wb = w + (j * nb + b) * 144;
                const uint8_t* ab = a_q8k + (i * nb + b) * 292;
                int32_t is, ms;
                block_sums_q4_k_q8_k(wb, ab, &is, &ms);
                float d8;
                memcpy(&d8, ab, 4);
                acc += (d8 * rd_f16(wb)) * (float)is;
                acc -= (d8 * rd_f16(wb + 2)) * (float)ms;
            }
            out[i * n + j] = acc;
        }
    }
}

/* The same for Q5_K (codes 0..31 with the fifth bit from qh) and for Q6_K (codes -32..31, an int8 scale per 16 weights, no
 * min term): integer sums of one weight block against one Q8_K block. */
static void block_sums_q5_k_q8_k(const uint8_t* wb, const uint8_t* ab, int32_t* isum, int32_t* msum) {
    uint8_t sc[8], mn[8];
    qo_unpack_scales_q4_k(wb + 4, sc, mn);
    const int8_t* q8 = (const int8_t*)(ab + 4);
    const uint8_t* qh = wb + 16;
    const uint8_t* qs = wb + 48;
    int32_t is = 0, ms = 0;
    for (int c = 0; c < 4; c++) {
        int32_t lo = 0, hi = 0;
        for (int t = 0; t < 32; t++) {
            lo += (int)((qs[32 * c + t] & 0xF) + (((qh[t] >> (2 * c)) & 1) << 4)) * (int)q8[64 * c + t];
            hi += (int)((qs[32 * c + t] >> 4) + (((qh[t] >> (2 * c + 1)) & 1) << 4)) * (int)q8[64 * c + 32 + t];
        }
        is += (int32_t)sc[2 * c] * lo + (int32_t)sc[2 * c + 1] * hi;
    }
    for (int sub = 0; sub < 8; sub++) {
        int16_t b0, b1;
        memcpy(&b0, ab + 260 + 4 * sub, 2);
        memcpy(&b1, ab + 262 + 4 * sub, 2);
        ms += (int32_t)mn[sub] * ((int32_t)b0 + (int32_t)b1);
    }
    *isum = is;
    *msum = ms;
}
static int32_t block_sum_q6_k_q8_k(const uint8_t* wb, const uint8_t* ab) {
    const int8_t* q8 = (const int8_t*)(ab + 4);
    int32_t is = 0;
    for (int h = 0; h < 2; h++) {
        const uint8_t* ql = wb + 64 * h;
        const uint8_t* qh = wb + 128 + 32 * h;
        const int8_t* sc = (const int8_t*)(wb + 192 + 8 * h);
        const int8_t* a = q8 + 128 * h;
        int32_t part[8] = {0, 0, 0, 0, 0, 0, 0, 0};  /* the eight 16-weight groups of this half, in scale order */
        for (int l = 0; l < 32; l++) {
            int g = l / 16;
            part[g + 0] += ((int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32) * (int)a[l];
            part[g + 2] += ((int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32) * (int)a[l + 32];
            part[g + 4] += ((int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32) * (int)a[l + 64];
            part[g + 6] += ((int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32) * (int)a[l + 96];
        }
        for (int g = 0; g < 8; g++) is += (int32_t)sc[g] * part[g];
    }
    return is;
}

/* out int32[M, N, K/256]: isum (and msum, zero for Q6_K) of every block pair, enc = Q4_K, Q5_K or Q6_K */
int qo_block_sums_kquant_q8_k(int enc, const uint8_t* a_q8k, const uint8_t* w, int64_t m, int64_t n, int64_t k, int32_t* isum, int32_t* msum) {
    int64_t epb, bpb;
    if ((enc != QO_Q4_K && enc != QO_Q5_K && enc != QO_Q6_K) || qo_block_params(enc, &epb, &bpb) || k % 256) return -1;
    int64_t nb = k / 256;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; j++)
        for (int64_t i = 0; i < m; i++)
            for (int64_t b = 0; b < nb; b++) {
                const uint8_t* wb = w + (j * nb + b) * bpb;
                const uint8_t* ab = a_q8k + (i * nb + b) * 292;
                int32_t* is = isum + (i * n + j) * nb + b;
                int32_t* ms = msum + (i * n + j) * nb + b;
                if (enc == QO_Q4_K) block_sums_q4_k_q8_k(wb, ab, is, ms);
                else if (enc == QO_Q5_K) block_sums_q5_k_q8_k(wb, ab, is, ms);
                else { *is = block_sum_q6_k_q8_k(wb, ab); *ms = 0; }
            }
    return 0;
}

/* fp32 activations in, quantised to Q8_K on the way: out[m, n] = sum_b (d8 * f32(d)) * isum - (d8 * f32(dmin)) * msum, blocks
 * in ascending order (Q6_K: d at byte 208, no min term) */
int qo_matmul_kquant_act_q8_k(int enc, const float* a, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out) {
    int64_t epb, bpb;
    if ((enc != QO_Q4_K && enc != QO_Q5_K && enc != QO_Q6_K) || qo_block_params(enc, &epb, &bpb) || k % 256) return -1;
    int64_t nb = k / 256;
    uint8_t* aq = (uint8_t*)malloc((size_t)(m * nb * 292));
    qo_quantize_q8_k(a, m, k, aq);
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; j++) {
        for (int64_t i = 0; i < m; i++) {
            float acc = 0.0f;
            for (int64_t b = 0; b < nb; b++) {
                const uint8_t* wb = w + (j * nb + b) * bpb;
                const uint8_t* ab = aq + (i * nb + b) * 292;
                float d8;
                memcpy(&d8, ab, 4);
                if (enc == QO_Q6_K) {
                    acc += (d8 * rd_f16(wb + 208)) * (float)block_sum_q6_k_q8_k(wb, ab);
                } else {
                    int32_t is, ms;
                    if (enc == QO_Q4_K) block_sums_q4_k_q8_k(wb, ab, &is, &ms);
                    else block_sums_q5_k_q8_k(wb, ab, &is, &ms);
                    acc += (d8 * rd_f16(wb)) * (float)is;
                    acc -= (d8 * rd_f16(wb + 2)) * (float)ms;
                }
            }
            out[i * n + j] = acc;
        }
    }
    free(aq);
    return 0;
}

/* fp32 activations in, quantised to Q8_K on the way */
void qo_matmul_q4_k_act_q8_k(const float* a, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out) {
    uint8_t* aq = (uint8_t*)malloc((size_t)(m * (k / 256) * 292));
    qo_quantize_q8_k(a, m, k, aq);
    qo_matmul_q4_k_q8_k(aq, w, m, n, k, out);
    free(aq);
}

/* ------------------------------------------------------------------ */
/* fp32-activation matmuls (Q4_K, Q6_K, GPTQ, and Q4_0 without Q8_0)   */
/* ------------------------------------------------------------------ */

static inline float maybe_bf16(float v, int w_bf16) {
    return w_bf16 ? qo_bf16_to_f32(qo_f32_to_bf16(v)) : v;
}

/* out[m, n] = sum_k a[m,k] * dequant(w)[n,k]; fp32 products and accumulation
 * in 8 strided partial sums combined as a balanced tree, the shape of an
 * 8-lane SIMD kernel.  w_bf16 != 0 rounds every dequantised weight to bf16
 * first (the prefill kernels' "fast" operand mode). */
int qo_matmul_f32(int enc, const float* a, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                  int w_bf16, float* out) {
    int64_t epb, bpb;
    if (qo_block_params(enc, &epb, &bpb) || k % epb) return -1;
    int64_t nb = k / epb;
#pragma omp parallel
    {
        float* wrow = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
        for (int64_t j = 0; j < n; j++) {
            for (int64_t b = 0; b < nb; b++) dequant_block(enc, w + (j * nb + b) * bpb, wrow + b * epb);
            if (w_bf16)
                for (int64_t kk = 0; kk < k; kk++) wrow[kk] = maybe_bf16(wrow[kk], 1);
            for (int64_t i = 0; i < m; i++) {
                const float* ar = a + i * k;
                float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int64_t kk = 0; kk < k; kk += 8)
                    for (int l = 0; l < 8; l++) acc[l] += ar[kk + l] * wrow[kk + l];
                out[i * n + j] = ((acc[0] + acc[4]) + (acc[2] + acc[6])) +
                                 ((acc[1] + acc[5]) + (acc[3] + acc[7]));
            }
        }
        free(wrow);
    }
    return 0;
}

/* The timed CPU baseline for Q4_K with fp32 activations, hand-vectorised (AVX2 + FMA, the ISA class an x86 host of
 * the reference dispatches on: stdlib/src/sys/info.mojo:97-162), rows of N split across threads
 * (examples/matmul.mojo:126-141).  NOT a checker: it sums in a different order from qo_matmul_f32
 * (sum_k a*q per sub-block first, then (d*sc) * that - (dmin*mn) * sum_k a), so it agrees with it to rounding only;
 * the unit tests hold it to the matmul tolerance against qo_matmul_f32.  Returns -1 where the host lacks AVX2. */
#if defined(__AVX2__) && defined(__FMA__)
#include <immintrin.h>
static inline float hsum8(__m256 v) {
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    s = _mm_add_ps(s, _mm_movehl_ps(s, s));
    s = _mm_add_ss(s, _mm_movehdup_ps(s));
    return _mm_cvtss_f32(s);
}
int qo_baseline_matmul_q4_k(const float* a, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out) {
    if (k % 256) return -1;
    const int64_t nb = k / 256, nsub = k / 32;
    float* asum = (float*)malloc(sizeof(float) * (size_t)(m * nsub));
    for (int64_t i = 0; i < m; i++)
        for (int64_t sb = 0; sb < nsub; sb++) {
            const float* p = a + i * k + sb * 32;
            __m256 t = _mm256_add_ps(_mm256_add_ps(_mm256_loadu_ps(p), _mm256_loadu_ps(p + 8)),
                                     _mm256_add_ps(_mm256_loadu_ps(p + 16), _mm256_loadu_ps(p + 24)));
            asum[i * nsub + sb] = hsum8(t);
        }
    const __m256i lo4 = _mm256_set1_epi32(0xF);
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; j++) {
        for (int64_t i = 0; i < m; i++) {
            const float* ar = a + i * k;
            const float* as = asum + i * nsub;
            __m256 acc = _mm256_setzero_ps();
            float macc = 0.0f;
            for (int64_t b = 0; b < nb; b++) {
                const uint8_t* blk = w + (j * nb + b) * 144;
                const float d = rd_f16(blk), dmin = rd_f16(blk + 2);
                uint8_t sc[8], mn[8];
                qo_unpack_scales_q4_k(blk + 4, sc, mn);
                for (int c = 0; c < 4; c++) {
                    const uint8_t* qs = blk + 16 + 32 * c;
                    const float* x = ar + b * 256 + 64 * c;
                    __m256 tl = _mm256_setzero_ps(), th = _mm256_setzero_ps();
                    for (int g = 0; g < 4; g++) {  /* 8 code bytes: 8 weights of sub-block 2c (low nibbles), 8 of 2c + 1 */
                        const __m256i q = _mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i*)(qs + 8 * g)));
                        tl = _mm256_fmadd_ps(_mm256_cvtepi32_ps(_mm256_and_si256(q, lo4)), _mm256_loadu_ps(x + 8 * g), tl);
                        th = _mm256_fmadd_ps(_mm256_cvtepi32_ps(_mm256_srli_epi32(q, 4)), _mm256_loadu_ps(x + 32 + 8 * g), th);
                    }
                    acc = _mm256_fmadd_ps(_mm256_set1_ps(d * (float)sc[2 * c]), tl, acc);
                    acc = _mm256_fmadd_ps(_mm256_set1_ps(d * (float)sc[2 * c + 1]), th, acc);
                    macc += dmin * (float)mn[2 * c] * as[b * 8 + 2 * c] + dmin * (float)mn[2 * c + 1] * as[b * 8 + 2 * c + 1];
                }
            }
            out[i * n + j] = hsum8(acc) - macc;
        }
    }
    free(asum);
    return 0;
}
#else
int qo_baseline_matmul_q4_k(const float* a, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out) {
    (void)a; (void)w; (void)m; (void)n; (void)k; (void)out;
    return -1;
}
#endif

int qo_matmul_f64(int enc, const float* a, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                  int w_bf16, double* out) {
    int64_t epb, bpb;
    if (qo_block_params(enc, &epb, &bpb) || k % epb) return -1;
    int64_t nb = k / epb;
#pragma omp parallel
    {
        float* wrow = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
        for (int64_t j = 0; j < n; j++) {
            for (int64_t b = 0; b < nb; b++) dequant_block(enc, w + (j * nb + b) * bpb, wrow + b * epb);
            for (int64_t i = 0; i < m; i++) {
                const float* ar = a + i * k;
                double acc = 0.0;
                for (int64_t kk = 0; kk < k; kk++)
                    acc += (double)ar[kk] * (double)maybe_bf16(wrow[kk], w_bf16);
                out[i * n + j] = acc;
            }
        }
        free(wrow);
    }
    return 0;
}

/* GPTQ: weights dequantised to fp32[N, K] per output column on the fly. */
void qo_matmul_gptq_f32(const float* a, const int32_t* qweight, const uint16_t* scales,
                        const int32_t* qzeros, const int32_t* g_idx, int64_t m, int64_t n, int64_t k,
                        int64_t group, int w_bf16, float* out, double* out64) {
#pragma omp parallel
    {
        float* wrow = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
        for (int64_t col = 0; col < n; col++) {
            for (int64_t kk = 0; kk < k; kk++) {
                int64_t g = g_idx ? g_idx[kk] : kk / group;
                int q = (int)(((uint32_t)qweight[(kk / 8) * n + col] >> (4 * (kk % 8))) & 0xF);
                int z = (int)(((uint32_t)qzeros[g * (n / 8) + col / 8] >> (4 * (col % 8))) & 0xF) + 1;
                wrow[kk] = maybe_bf16(qo_f16_to_f32(scales[g * n + col]) * (float)(q - z), w_bf16);
            }
            for (int64_t i = 0; i < m; i++) {
                const float* ar = a + i * k;
                if (out) {
                    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                    for (int64_t kk = 0; kk < k; kk += 8)
                        for (int l = 0; l < 8; l++) acc[l] += ar[kk + l] * wrow[kk + l];
                    out[i * n + col] = ((acc[0] + acc[4]) + (acc[2] + acc[6])) +
                                       ((acc[1] + acc[5]) + (acc[3] + acc[7]));
                }
                if (out64) {
                    double acc = 0.0;
                    for (int64_t kk = 0; kk < k; kk++) acc += (double)ar[kk] * (double)wrow[kk];
                    out64[i * n + col] = acc;
                }
            }
        }
        free(wrow);
    }
}

/* ------------------------------------------------------------------ */
/* helpers for the timed CPU baseline                                  */
/* ------------------------------------------------------------------ */

int qo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void qo_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* CLOCK_MONOTONIC seconds, the clock the reference's timers use
 * (stdlib/src/time/time.mojo:108-118). */
double qo_now(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}
