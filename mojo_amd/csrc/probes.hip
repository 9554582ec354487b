// Device-side yardsticks for the matrix-core roofline: what the matrix cores sustain with no memory traffic at all.
//
// Every wavefront runs `iters` rounds of sixteen v_mfma_f32_32x32x16_f16 (four independent accumulator chains, operands
// and accumulators in registers for the whole kernel), eight wavefronts per compute unit.  The operand data decides
// how much the part draws, and with it the clock it sustains:
//   kind 0  zeros
//   kind 1  1.0 everywhere
//   kind 2  random values in +-[1, 4) on both sides (dense activations x dense weights)
//   kind 3  random values in +-[1, 4) x random integers 0..945 (what the plane GEMMs multiply: narrowed activations x sc * q)
// Kinds 4 and 5 are kinds 0 and 2 with v_mfma_f32_16x16x32_f16 (the small-batch kernels' instruction: half the products
// per instruction), sixteen independent-enough instructions a round on four accumulator chains as well.
#include "qmm_internal.h"

namespace qmm {

namespace {

typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef float probe_float16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

}  // namespace

__global__ __launch_bounds__(512, 1) void mfma_probe_kernel(float* __restrict__ out, int kind, int iters) {
    union {
        uint32_t u[4];
        probe_half8 h;
    } a[4], b[4];
    const uint32_t t = blockIdx.x * 512 + threadIdx.x;
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 4; i++) {
            const uint32_t ra = probe_hash(t * 64 + j * 8 + i), rb = probe_hash(t * 64 + j * 8 + i + 4);
            uint32_t va = 0, vb = 0;
            if (kind == 1) va = vb = 0x3C003C00u;
            if (kind >= 2) {
                va = (ra & 0x87ff87ffu) | 0x3C003C00u;  // +-[1, 4)
                if (kind == 2) {
                    vb = (rb & 0x87ff87ffu) | 0x3C003C00u;
                } else {
                    union {
                        _Float16 h[2];
                        uint32_t u;
                    } p;
                    p.h[0] = (_Float16)(float)(rb % 946u);
                    p.h[1] = (_Float16)(float)((rb >> 16) % 946u);
                    vb = p.u;
                }
            }
            a[j].u[i] = va;
            b[j].u[i] = vb;
        }
    probe_float16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j].h, b[j].h, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j].h, b[(j + 1) & 3].h, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(j + 1) & 3].h, b[j].h, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(j + 2) & 3].h, b[(j + 3) & 3].h, c3, 0, 0, 0);
        }
        if ((i & 63) == 63) {  // keep the sums finite
#pragma unroll
            for (int r = 0; r < 16; r++) {
                c0[r] *= 1e-6f;
                c1[r] *= 1e-6f;
                c2[r] *= 1e-6f;
                c3[r] *= 1e-6f;
            }
        }
    }
    out[t] = c0[0] + c1[1] + c2[2] + c3[3];
}

__global__ __launch_bounds__(512, 1) void mfma_probe16_kernel(float* __restrict__ out, int kind, int iters) {
    typedef float probe_float4 __attribute__((ext_vector_type(4)));
    union {
        uint32_t u[4];
        probe_half8 h;
    } a[4], b[4];
    const uint32_t t = blockIdx.x * 512 + threadIdx.x;
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 4; i++) {
            const uint32_t ra = probe_hash(t * 64 + j * 8 + i), rb = probe_hash(t * 64 + j * 8 + i + 4);
            a[j].u[i] = kind == 5 ? (ra & 0x87ff87ffu) | 0x3C003C00u : 0u;
            b[j].u[i] = kind == 5 ? (rb & 0x87ff87ffu) | 0x3C003C00u : 0u;
        }
    probe_float4 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j].h, b[j].h, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j].h, b[(j + 1) & 3].h, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(j + 1) & 3].h, b[j].h, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(j + 2) & 3].h, b[(j + 3) & 3].h, c3, 0, 0, 0);
        }
        if ((i & 63) == 63) {  // keep the sums finite
#pragma unroll
            for (int r = 0; r < 4; r++) {
                c0[r] *= 1e-6f;
                c1[r] *= 1e-6f;
                c2[r] *= 1e-6f;
                c3[r] *= 1e-6f;
            }
        }
    }
    out[t] = c0[0] + c1[1] + c2[2] + c3[3];
}

// kind 6: v_mfma_f32_32x32x16_bf16 on dense random bf16 values in +-[1, 4)
__global__ __launch_bounds__(512, 1) void mfma_probe_bf16_kernel(float* __restrict__ out, int iters) {
    typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
    union {
        uint32_t u[4];
        probe_bf16x8 h;
    } a[4], b[4];
    const uint32_t t = blockIdx.x * 512 + threadIdx.x;
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 4; i++) {
            const uint32_t ra = probe_hash(t * 64 + j * 8 + i), rb = probe_hash(t * 64 + j * 8 + i + 4);
            a[j].u[i] = (ra & 0x80ff80ffu) | 0x3F803F80u;
            b[j].u[i] = (rb & 0x80ff80ffu) | 0x3F803F80u;
        }
    probe_float16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j].h, b[j].h, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j].h, b[(j + 1) & 3].h, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + 1) & 3].h, b[j].h, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + 2) & 3].h, b[(j + 3) & 3].h, c3, 0, 0, 0);
        }
        if ((i & 63) == 63) {  // keep the sums finite
#pragma unroll
            for (int r = 0; r < 16; r++) {
                c0[r] *= 1e-6f;
                c1[r] *= 1e-6f;
                c2[r] *= 1e-6f;
                c3[r] *= 1e-6f;
            }
        }
    }
    out[t] = c0[0] + c1[1] + c2[2] + c3[3];
}

hipError_t launch_mfma_probe(float* out, int workgroups, int kind, int iters, hipStream_t s) {
    if (kind == 6) mfma_probe_bf16_kernel<<<dim3((unsigned)workgroups), dim3(512), 0, s>>>(out, iters);
    else if (kind >= 4) mfma_probe16_kernel<<<dim3((unsigned)workgroups), dim3(512), 0, s>>>(out, kind, iters);
    else mfma_probe_kernel<<<dim3((unsigned)workgroups), dim3(512), 0, s>>>(out, kind, iters);
    return hipGetLastError();
}

}  // namespace qmm
