// Host-side launch functions shared between the kernel translation units and
// the C ABI in qmm_api.hip.  Each returns the hipError_t of its launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qmm.h"
#include "qmm_device.h"

namespace qmm {

// Kernel families switched off by the environment variable QMM_DISABLE (a comma-separated list of names, read once
// per process), for tests and triage: a disabled family reports that it does not take a shape, and the next kernel
// in the dispatch order serves it.  Names: q4k_lanes, q4k_lanes_rows, q4k_stream, q4k_mm, q4k_kc, q4k_tile, q4k_gemm64, q4k_twin_rows, q4k_rows_v2,
// q4_0_stream, q4_0_mfma, q4_0_small, q4_0_small_passes, q4_0_wide, q4_0_planes, q6k_lanes, q6k_slab, q6k_staged, kquant_planes, planes_wide, planes_192, planes_quarters, planes_twin_rows, gptq_twin_rows, gptq_k_shares, gptq_long_k_mm, kquant_mm_rounds_grid, q4k_mm_k_parts, q4k_planes, gptq_planes, gptq_mm, gptq_cols, gptq_cols16.
// Nothing is disabled by default.
bool kernel_disabled(const char* family);
// False while qmm_matmul_static serves a problem whose one-pass treatment of an fp32 lhs (the lhs as twice the rows, the
// result in the workspace) does not fit its scratch: the GEMMs then take their two passes.  Per thread.
bool twin_rows_allowed();

hipError_t launch_read_probe(const void* buf, int64_t bytes, hipStream_t s);
// register-resident matrix-core loop (probes.hip): `workgroups` workgroups of 8 wavefronts, out fp32 [workgroups * 512]
hipError_t launch_mfma_probe(float* out, int workgroups, int kind, int iters, hipStream_t s);
hipError_t launch_dequant(int enc, const void* rhs, int64_t n, int64_t k, void* out, int out_dtype,
                          hipStream_t s);
hipError_t launch_dequant_gptq(const void* qweight, const void* scales, const void* qzeros,
                               const void* g_idx, int64_t n, int64_t k, int group, void* out,
                               int out_dtype, hipStream_t s);
hipError_t launch_quantize(int enc, const float* x, int64_t rows, int64_t k, void* out, hipStream_t s);
hipError_t launch_quantize_q8_0(const void* x, int x_dtype, int64_t rows, int64_t k, void* blocks,
                                void* codes, void* dscale, void* csum, hipStream_t s);
hipError_t launch_quantize_q8_k(const void* x, int x_dtype, int64_t rows, int64_t k, void* out, hipStream_t s);
// y fp32[rows, k] = d8 * code of the Q8_K quantisation of x (k a multiple of 256)
// Q8_K activations as planes (codes [m, k], d8 [m, k / 256], sums of 32 codes [m, k / 32]) and the integer-dot decode kernels
// for Q5_K and Q6_K weights over them (gemv_kquant_q8k.hip): one pass takes up to four lhs rows.
struct Q8KPlanes {
    int8_t* codes;
    float* d8;
    int32_t* sums;
};
int64_t q8k_planes_bytes(int64_t m, int64_t k);
Q8KPlanes q8k_planes(void* ws, int64_t m, int64_t k);
hipError_t launch_quantize_q8_k_planes(const void* x, int x_dtype, int64_t rows, int64_t k, const Q8KPlanes& p, hipStream_t s);
hipError_t launch_gemv_kquant_q8k(int encoding, const Q8KPlanes& p, int64_t m0, int rows, const uint8_t* w, int64_t n, int64_t k, float* out,
                                  int64_t ldo, hipStream_t s);
hipError_t launch_q8k_round_trip(const void* x, int x_dtype, int64_t rows, int64_t k, float* y, hipStream_t s);
hipError_t launch_quantize_gptq(const float* w, int64_t n, int64_t k, int group, void* qweight,
                                void* scales, void* qzeros, void* g_idx, hipStream_t s);

// Decode-shape kernels (m <= 16 rows of lhs per launch).
// gamma != nullptr: the lhs rows are RMS-normalised in the kernel before they are quantised (y = x * rsqrt(mean(x^2) + eps) * gamma)
hipError_t launch_gemv_q4_0_stream(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                   int64_t ldo, hipStream_t s, bool* handled, const float* gamma = nullptr, float eps = 0.0f);
// y[rows, k] = x * rsqrt(mean(x^2) + eps) * gamma, computed in fp32; y has the dtype of x (bf16: rounded to nearest even)
hipError_t launch_rmsnorm(const void* x, int x_dtype, const float* gamma, float eps, int64_t rows, int64_t k, void* y, hipStream_t s);
hipError_t launch_gemv_q4_0(const int8_t* a_codes, const float* a_scale, const int32_t* a_sum,
                            const uint8_t* w, int m, int64_t n, int64_t k, float* out, int64_t ldo,
                            hipStream_t s);
hipError_t launch_gemv_q4_k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                            float* out, int64_t ldo, hipStream_t s);
// Kernels that use more than 64 KB of dynamic LDS must say so once before their first launch: this raises the
// kernel's limit to the 160 KB of a gfx950 compute unit, the first time it is called for the kernel.
constexpr int kLdsPerCu = 160 * 1024;
template <auto Kernel>
inline hipError_t allow_full_lds() {
    static const hipError_t st = hipFuncSetAttribute((const void*)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsPerCu);
    return st;
}

// Q5_K decode kernel, m <= 4 (fewer when K is long: the lhs copy in LDS takes 16 KB per row and 4096 columns).
hipError_t launch_gemv_q5_k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                            int64_t ldo, hipStream_t s, bool* handled);

// Q4_K with Q8_K-quantised activations (integer dots), m <= 4.
hipError_t launch_gemv_q4_k_q8k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                int64_t ldo, hipStream_t s, bool* handled);

// Weight matrices that share one lhs, for the grouped decode launch.
constexpr int kLanesMaxMats = 4;
struct LanesMats {
    const uint8_t* w[kLanesMaxMats];
    float* out[kLanesMaxMats];
    int end[kLanesMaxMats];  // running row count: matrix j owns rows [end[j - 1], end[j])
    int count;
    int swiglu;              // 1: two matrices (gate, up) of equal size; out[0][r] = silu(gate row r) * (up row r)
    int out_bf16;            // 1: the out pointers are bf16 arrays (round to nearest even, canonical NaN)
};
// The same for the small-batch matrix-core kernel: 16-row tiles are numbered through the matrices.
struct MmMats {
    const uint8_t* w[kLanesMaxMats];
    float* out[kLanesMaxMats];
    int tile_end[kLanesMaxMats];  // running tile count: matrix j owns tiles [tile_end[j - 1], tile_end[j])
    int n[kLanesMaxMats];
    int count;
};
hipError_t launch_gemv_q4_k_mm_grouped(const void* lhs, int lhs_dtype, int count, const uint8_t* const* ws, const int64_t* ns,
                                       float* const* outs, int64_t m, int64_t k, void* workspace, hipStream_t s, bool k_parts = false);
hipError_t launch_gemv_q4_k_lanes_grouped(const void* a, int a_dtype, int count, const uint8_t* const* ws, const int64_t* ns,
                                          float* const* outs, int m, int64_t k, int64_t ldo, hipStream_t s, bool* handled,
                                          bool swiglu = false, bool out_bf16 = false);
// out[i] = silu(gate[i]) * up[i], i < count (fp32)
hipError_t launch_swiglu(const float* gate, const float* up, float* out, int64_t count, hipStream_t s);
hipError_t launch_gemv_q4_k_lanes(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                  int64_t ldo, hipStream_t s, bool* handled, bool out_bf16 = false);
// out[i] = bf16(x[i]), i < count: round to nearest even, NaN to the canonical quiet NaN
hipError_t launch_f32_to_bf16(const float* x, uint16_t* out, int64_t count, hipStream_t s);
// Two to four lhs rows through the decode kernel with one 32-column sub-block per lane (K <= 16384).
hipError_t launch_gemv_q4_k_lanes_rows(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                                       int64_t ldo, hipStream_t s, bool* handled);
hipError_t launch_gemv_q4_k_lanes_rows_grouped(const void* a, int a_dtype, int count, const uint8_t* const* ws, const int64_t* ns,
                                               float* const* outs, int m, int64_t k, int64_t ldo, hipStream_t s, bool* handled);
hipError_t launch_gemv_q4_k_rows(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                                 float* out, int64_t ldo, hipStream_t s);
hipError_t launch_gemv_q6_k(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                            float* out, int64_t ldo, hipStream_t s);
// Q5_K, up to 64 lhs rows (passes of 16 or 8), K a multiple of 512 up to 32768, 16-byte aligned weights: the small-batch
// matrix-core kernel (gemv_q5k_mm.hip).
bool gemv_q5_k_mm_supported(const void* w, int64_t m, int64_t n, int64_t k);
hipError_t launch_gemv_q5_k_mm(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out, int64_t ldo,
                               void* workspace, hipStream_t s);
// Both small-batch K-quant kernels on a K beyond 4096: bytes for the results of the rounds of K, which then run side by side.
int64_t gemv_kquant_mm_workspace_bytes(int64_t m, int64_t n, int64_t k);
// Q6_K, up to 64 lhs rows (passes of 16 or 8), K a multiple of 2048 up to 32768, 16-byte aligned weights: the small-batch
// matrix-core kernel (gemv_q6k_mm.hip).
bool gemv_q6_k_mm_supported(const void* w, int64_t m, int64_t n, int64_t k);
hipError_t launch_gemv_q6_k_mm(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out, int64_t ldo,
                               void* workspace, hipStream_t s);
hipError_t launch_gemv_q6_k_rows(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k,
                                 float* out, int64_t ldo, hipStream_t s, bool* handled);
int64_t gemm_q4_0_workspace_bytes(int64_t m, int64_t k);
// Q4_0 prefill on the fp16 matrix cores with exact integer operands (weights as a plane of q - 8, lhs as Q8_0 codes, the
// per-block scale products made by the matrix cores too): taken where gemm_q4_0_planes_wanted says so.
bool gemm_q4_0_planes_wanted(int64_t m, int64_t n, int64_t k);
int64_t gemm_q4_0_planes_workspace_bytes(int64_t m, int64_t n, int64_t k);
hipError_t launch_gemm_q4_0_planes(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k, float* out,
                                   void* workspace, hipStream_t s);
hipError_t launch_gemm_q4_0(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                            float* out, void* workspace, hipStream_t s);
bool gemv_gptq_cols16_wanted(int64_t n, int group);  // the decode kernel with 16 columns per workgroup serves this matrix
hipError_t launch_gemv_gptq_cols(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                                 const uint32_t* qzeros, int m, int64_t n, int64_t k, int group, float* out,
                                 int64_t ldo, hipStream_t s, bool* handled);
bool gemv_gptq_mm_supported(const void* qweight, int64_t n, int64_t k, int group);
int64_t gemv_gptq_mm_workspace_bytes(int64_t m, int64_t n, int64_t k);
hipError_t launch_gemv_gptq_mm(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                               const uint32_t* qzeros, int m, int64_t n, int64_t k, int group, float* out, int64_t ldo,
                               void* workspace, hipStream_t s, bool* handled);
hipError_t launch_gemv_gptq_act_order(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                                      const uint32_t* qzeros, const int32_t* g_idx, int m, int64_t n, int64_t k, int group,
                                      float* out, int64_t ldo, hipStream_t s);
bool gemv_q4_k_kc_supported(const void* w, int64_t k);
int64_t gemv_q4_k_kc_workspace_bytes(int64_t m, int64_t n, int64_t k);
hipError_t launch_gemv_q4_k_kc(const void* a, int a_dtype, const uint8_t* w, int m, int64_t n, int64_t k, float* out,
                               int64_t ldo, void* workspace, hipStream_t s, bool* handled);
int64_t gemv_q4_k_mm_workspace_bytes(int lhs_dtype, int64_t m, int64_t k);
int64_t gemv_q4_k_mm_plain_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k);  // launch_gemv_q4_k_mm
hipError_t launch_gemv_q4_k_mm(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                               float* out, void* workspace, hipStream_t s);
bool gemm_gptq_supported(int64_t k, int group);
int64_t gemm_gptq_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k);
bool gemm_gptq_twin(int lhs_dtype, int64_t m);  // an fp32 lhs goes through the GEMM as one lhs of twice the rows
int gemm_gptq_k_shares(int64_t m, int64_t n, int64_t k);  // K shares per tile of the GEMM (m: the rows it sees)
hipError_t launch_gemm_gptq(const void* lhs, int lhs_dtype, const uint32_t* qweight, const uint16_t* scales,
                            const uint32_t* qzeros, int64_t m, int64_t n, int64_t k, int group, float* out,
                            void* workspace, hipStream_t s);
hipError_t launch_gemv_gptq(const void* a, int a_dtype, const uint32_t* qweight, const uint16_t* scales,
                            const uint32_t* qzeros, int m, int64_t n, int64_t k, int group, float* out,
                            int64_t ldo, hipStream_t s);
// Prefill-shape kernels (m > 16).
int64_t gemm_q4_k_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k);
hipError_t launch_gemm_q4_k(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                            float* out, void* workspace, hipStream_t s);
// The kernel that unpacks each weight tile once per workgroup into LDS (256 x 128 output tiles): taken by
// launch_gemm_q4_k where gemm_q4_k_tile_wanted says so.
bool gemm_q4_k_tile_wanted(int64_t m, int64_t n, int64_t k);
int64_t gemm_q4_k_tile_workspace_bytes(int lhs_dtype, int64_t m, int64_t k);
hipError_t launch_gemm_q4_k_tile(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                                 float* out, void* workspace, hipStream_t s);
// Q5_K and Q6_K (Q4_K on request) on the matrix cores: a pass that turns the weights into fp16 integer planes in the
// workspace, then a tile GEMM over them.
// out[i] = part[i] + part[count + i] + ... (`shares` terms, in that order)
hipError_t launch_sum_shares(const float* part, float* out, int64_t count, int shares, hipStream_t s);
bool gemm_planes_wanted(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k);
// GPTQ through the same GEMM (plain groups of 128 or 256 and large problems only)
bool gemm_gptq_planes_wanted(int64_t m, int64_t n, int64_t k, int group);
int64_t gemm_gptq_planes_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k);
hipError_t launch_gemm_gptq_planes(const void* lhs, int lhs_dtype, const uint32_t* qweight, const uint16_t* scales, const uint32_t* qzeros,
                                   int64_t m, int64_t n, int64_t k, int group, float* out, void* workspace, hipStream_t s);
int64_t gemm_planes_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k);
hipError_t launch_gemm_planes(int encoding, const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                              float* out, void* workspace, hipStream_t s);
int compute_units();  // of the current device, read once (gemm_planes.hip)
// The 256 x 128 plane kernels' quarter mode (gemm_planes.hip): the shapes with few enough tiles, and out += part behind the GEMM.
bool few_tiles_for_quarters(int64_t m, int64_t n, int64_t k);
hipError_t launch_add_part(float* out, const float* part, int64_t count, hipStream_t s);
// The Q4_0 weight plane kept across calls (gemm_q4_0_planes.hip)
int64_t repacked_q4_0_bytes(int64_t n, int64_t k);
hipError_t launch_repack_q4_0(const uint8_t* w, int64_t n, int64_t k, void* packed, hipStream_t s);
int64_t repacked_q4_0_workspace_bytes(int64_t m, int64_t n, int64_t k);
hipError_t launch_gemm_q4_0_repacked(const void* lhs, int lhs_dtype, const void* packed, int64_t m, int64_t n, int64_t k, float* out,
                                     void* workspace, hipStream_t s);
// Weight planes kept across calls: the conversion alone into a buffer of *_bytes, and the plane GEMMs over such a buffer (workspace:
// the lhs planes only).  *_wanted: the row counts from which the planes beat the kernels that read the packed weights, the
// conversion no longer counting.  The K-quant layout serves both plane GEMMs (Q4_K / Q5_K: min operands in both forms).
int64_t repacked_planes_bytes(int encoding, int64_t n, int64_t k);
hipError_t launch_repack_planes(int encoding, const uint8_t* w, int64_t n, int64_t k, void* packed, hipStream_t s);
bool repacked_planes_wanted(int encoding, int64_t m, int64_t n, int64_t k);
int64_t repacked_planes_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k);
hipError_t launch_gemm_planes_repacked(int encoding, const void* lhs, int lhs_dtype, const void* packed, int64_t m, int64_t n, int64_t k,
                                       float* out, void* workspace, hipStream_t s);
bool gptq_planes_supported(int64_t n, int64_t k, int group);
int64_t repacked_gptq_bytes(int64_t n, int64_t k);
hipError_t launch_repack_gptq(const uint32_t* qweight, const uint16_t* scales, const uint32_t* qzeros, int64_t n, int64_t k, int group, void* packed,
                              hipStream_t s);
bool repacked_gptq_wanted(int64_t m, int64_t n);
int64_t repacked_gptq_workspace_bytes(int lhs_dtype, int64_t m, int64_t k);
hipError_t launch_gemm_gptq_repacked(const void* lhs, int lhs_dtype, const void* packed, int64_t m, int64_t n, int64_t k, int group, float* out,
                                     void* workspace, hipStream_t s);

hipError_t launch_block_dots_q4_0(const uint8_t* a_q8, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                                  int32_t* out, hipStream_t s);

}  // namespace qmm
