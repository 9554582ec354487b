/*
 * qmm.h -- C ABI of libqmm.so: quantized-weight matmul for AMD MI355X (gfx950).
 *
 * This is the boundary a host runtime binds to replace MAX's
 * `max.graph.ops.qmatmul(encoding, config, lhs, *rhs)` and the
 * `QuantizationEncoding` block parameters.  MAX itself is not part of the
 * reference snapshot (it is the binary dependency pinned at
 * magic.lock:135-137), so each entry point cites the in-tree interface whose
 * conventions it follows:
 *   - plain C symbols resolved with dlopen/dlsym, POD arguments only
 *     (stdlib/src/sys/ffi.mojo:118-367, external_call at :471-502,
 *     C scalar aliases at :29-60);
 *   - the callee borrows every buffer and never frees or reallocates one
 *     (stdlib/src/python/_bindings.mojo:222-243,252-260);
 *   - errors come back as a status plus a message, never as an abort
 *     (stdlib/src/python/_bindings.mojo:285-291).
 *
 * All pointers are device pointers on the current HIP device unless a
 * parameter is documented as host memory.  Kernels are enqueued on `stream`
 * (a hipStream_t passed as void*; NULL = the default stream) and the calls
 * return without synchronising.  The library allocates no device memory:
 * scratch space is passed in as `workspace`.
 *
 * Every function returns QMM_OK (0) or a negative qmm_status;
 * qmm_last_error() then holds a thread-local description.
 */
#ifndef QMM_H
#define QMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* QuantizationEncoding values (GGUF block encodings + GPTQ). */
enum qmm_encoding {
    QMM_Q4_0 = 0, /* 32 weights / 18 bytes : f16 d, 16 B nibbles            */
    QMM_Q4_K = 1, /* 256 weights / 144 bytes: f16 d, dmin, 12 B 6-bit, 128 B */
    QMM_Q6_K = 2, /* 256 weights / 210 bytes: ql[128] qh[64] i8 sc[16] f16 d */
    QMM_GPTQ = 3, /* AutoGPTQ v1 tensors: qweight, scales, qzeros[, g_idx]   */
    QMM_Q5_K = 4, /* 256 weights / 176 bytes: the Q4_K header, qh[32] fifth bits, 128 B nibbles */
    QMM_Q8_0 = 8, /* 32 values / 34 bytes  : f16 d, 32 x i8 (activations)    */
    QMM_Q8_K = 9  /* 256 values / 292 bytes: f32 d, 256 x i8, 16 x i16 sums (activations) */
};

enum qmm_dtype { QMM_F32 = 0, QMM_BF16 = 1, QMM_F16 = 2 };

enum qmm_status {
    QMM_OK = 0,
    QMM_ERR_INVALID = -1,     /* bad argument: shape, alignment, null, enum */
    QMM_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for */
    QMM_ERR_HIP = -3,         /* HIP runtime error at launch                */
    QMM_ERR_WORKSPACE = -4    /* workspace missing or too small             */
};

/* QuantizationConfig of the reference API (GPTQ only). */
typedef struct qmm_gptq_config {
    int32_t bits;       /* 4                                      */
    int32_t group_size; /* 128 (any multiple of 32 dividing K)    */
    int32_t desc_act;   /* 0: the group of k is k / group_size (g_idx is not read); 1: act-order checkpoint, the
                           group of k is g_idx[k] (required; any order, values in [0, K / group_size))       */
    int32_t sym;        /* 1: stored zero-point 7 (true zero 8); 0: any stored zero-point (true zero = stored + 1) */
} qmm_gptq_config;

int qmm_version(void);
const char* qmm_last_error(void);

/* QuantizationEncoding.block_parameters: elements and bytes per block. */
int qmm_block_params(int encoding, int64_t* elements_per_block, int64_t* bytes_per_block);

/* Number of compute units and peak engine clock (kHz) of the current device,
 * for roofline reports (the role of the reference's
 * stdlib/src/sys/info.mojo:789-818 core-count queries). */
int qmm_device_info(int32_t* compute_units, int32_t* clock_khz);

/*
 * Roofline calibration: a plain read of `bytes` bytes (16-byte coalesced loads, grid-stride,
 * nothing written) on `stream`.  Timing it gives the read bandwidth this device sustains at a
 * given footprint, and profiling it gives the FETCH_SIZE a known number of bytes produces.  The
 * reference times its kernels with its own benchmark harness (stdlib/docs/bencher/Bench.md);
 * this is the device-side yardstick for the same purpose.  `buf` must be 16-byte aligned.
 */
int qmm_read_probe(const void* buf, int64_t bytes, void* stream);

/*
 * Roofline calibration for the matrix cores: a loop of v_mfma_f32_32x32x16_f16 on operands and accumulators that stay in
 * registers (no memory traffic), one workgroup of 8 wavefronts on every compute unit, `iters` rounds of 16 instructions per
 * wavefront.  `kind` selects the operand data: 0 zeros, 1 ones, 2 random values in +-[1, 4) on both sides, 3 such values
 * against random integers 0..945 (what the plane GEMMs multiply); 4 and 5 are kinds 0 and 2 with v_mfma_f32_16x16x32_f16,
 * the instruction of the small-batch kernels; 6 is kind 2 with v_mfma_f32_32x32x16_bf16 on bf16 values.  Timing it gives the
 * matrix-core rate this part sustains
 * on that kind of data, which for dense random data is well below the published peak (the part settles at a lower clock).
 * `out` receives 512 floats per compute unit (checksums; qmm_device_info gives the count), *flops the operations of the
 * launch.  No counterpart in the reference, whose harness times whole kernels (stdlib/docs/bencher/Bench.md).
 */
int qmm_mfma_probe(void* out, int64_t out_bytes, int kind, int iters, int64_t* flops, void* stream);

/*
 * Block unpack / dequantise: rhs uint8[n, k/epb*bpb] -> out[n, k] in
 * out_dtype (QMM_F32 or QMM_BF16, bf16 by round-to-nearest-even as
 * stdlib/src/builtin/simd.mojo:3279-3300).  Q4_0, Q4_K, Q6_K.
 */
int qmm_dequantize(int encoding, const void* rhs, int64_t n, int64_t k, void* out, int out_dtype,
                   void* stream);

/* GPTQ tensors -> out[n, k] (the transposed, GGUF-like orientation).  g_idx may be null when cfg->desc_act is 0. */
int qmm_dequantize_gptq(const qmm_gptq_config* cfg, const void* qweight, const void* scales,
                        const void* qzeros, const void* g_idx, int64_t n, int64_t k, void* out,
                        int out_dtype, void* stream);

/*
 * Quantisers.  x fp32[rows, k] -> packed blocks uint8[rows, k/epb*bpb].
 * QMM_Q4_0, QMM_Q8_0 and QMM_Q8_K follow the GGUF reference quantisers; QMM_Q4_K and
 * QMM_Q6_K use a direct (non-iterative) min/max fit.
 */
int qmm_quantize(int encoding, const float* x, int64_t rows, int64_t k, void* out, void* stream);

/* w fp32[n, k] -> AutoGPTQ tensors (symmetric 4-bit, desc_act = 0). */
int qmm_quantize_gptq(const qmm_gptq_config* cfg, const float* w, int64_t n, int64_t k,
                      void* qweight, void* scales, void* qzeros, void* g_idx, void* stream);

/* Bytes of device scratch qmm_matmul needs for this problem (may be 0); the second form for a call with `flags`
 * (QMM_FLAG_OUT_BF16 adds room for an fp32 result wherever the kernel does not store bf16 itself).  For large
 * Q4_K / GPTQ prefill problems (more than 512 lhs rows) the figure includes fp16 planes of the weights (2 bytes per
 * weight) for the faster of two kernels; qmm_matmul given less than that, but enough for the lhs planes, runs the other one. */
int64_t qmm_matmul_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k);
int64_t qmm_matmul_workspace_bytes_flags(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k, int flags);

/*
 * ops.qmatmul: out fp32[m, n] = lhs[m, k] . dequant(rhs)^T.
 *   encoding Q4_0/Q4_K/Q6_K: n_rhs = 1, rhs[0] = uint8[n, k/epb*bpb];
 *   encoding GPTQ: cfg required, n_rhs = 3 or 4,
 *     rhs = {qweight i32[k/8, n], scales f16[k/g, n], qzeros i32[k/g, n/8], g_idx i32[k]}.
 *     cfg->desc_act = 1 (n_rhs = 4) goes through a decode-shaped kernel for every m, four lhs rows per
 *     pass over the weights; the matrix-core kernel takes plain groups only.
 *   lhs_dtype QMM_F32 or QMM_BF16.  Q4_0 quantises lhs rows to Q8_0 and takes
 *   integer block dots (the reference CPU path); the others keep lhs as given.
 *   flags: bit 0 (QMM_FLAG_W_BF16) is reserved for a mode that rounds the dequantised
 *   weights to bf16 before the product; no kernel implements it and a call that sets
 *   it returns QMM_ERR_UNSUPPORTED.  Bit 1 (QMM_FLAG_ACT_Q8K), Q4_K / Q5_K / Q6_K: the
 *   lhs is quantised to Q8_K blocks (256 wide, fp32 scale) and the products are those of the
 *   integer sub-block dots of the ggml-lineage CPU kernels instead of the default
 *   floating-point ones.  Up to 16 lhs rows go through kernels that form the integer sub-block sums
 *   themselves (v_dot4_i32_i8, int32 sums per super-block, then (d8 * d) * isum - (d8 * dmin) * msum in fp32),
 *   in passes of four rows: Q4_K (K <= 16384) quantises the lhs inside the kernel, Q5_K and Q6_K read Q8_K
 *   codes, scales and 32-code sums that one launch per call writes into the workspace.  The integer sums equal
 *   the CPU path's bit for bit.  No integer kernel exists beyond 16 rows (or for Q4_K with K > 16384): those
 *   problems write d8 * code as fp32 rows into the workspace and run the floating-point kernels on them (the
 *   same products, summed in fp32, not in int32).  Workspace from qmm_matmul_workspace_bytes_flags.
 *   Bit 2 (QMM_FLAG_OUT_BF16): `out`
 *   points to bf16[m, n] instead of fp32 (the caller's next op takes bf16 activations): the fp32 result is
 *   rounded to nearest even with NaN mapped to the canonical quiet NaN, the reference's narrowing rule
 *   (stdlib/src/builtin/simd.mojo:3279-3300).  The Q4_K decode kernel (m = 1, K <= 16384) stores bf16 itself;
 *   every other problem computes fp32 into the workspace and narrows in a second launch, which takes
 *   qmm_matmul_workspace_bytes_flags bytes of workspace.
 * rhs is a host array of device pointers.
 */
#define QMM_FLAG_W_BF16 1
#define QMM_FLAG_ACT_Q8K 2
#define QMM_FLAG_OUT_BF16 4
int qmm_matmul(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m,
               int64_t k, const void* const* rhs, int n_rhs, int64_t n, float* out,
               void* workspace, int64_t workspace_bytes, int flags, void* stream);

/*
 * qmm_matmul for callers that cannot allocate or pass device memory of their own for scratch: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments and results as qmm_matmul without the workspace pair: the kernels' scratch
 * (the planes and partial sums qmm_matmul_workspace_bytes sizes) lives in a buffer of
 * QMM_STATIC_SCRATCH_BYTES that is part of the loaded library, one copy per GPU, held until the process
 * ends.  The call allocates and frees nothing.  A problem that needs more scratch than that returns
 * QMM_ERR_WORKSPACE (use qmm_matmul with a workspace).  All calls on one GPU share the buffer: calls that
 * can overlap there (different streams, different host threads) race and must be ordered by the caller.
 * Nothing in the buffer is expected to be zero or to survive from one call to the next.
  * The first call on a device looks the buffer's address up and sets kernel attributes: make it outside graph capture.
 */
#define QMM_STATIC_SCRATCH_BYTES (64 * 1024 * 1024)
int qmm_matmul_static(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m,
                      int64_t k, const void* const* rhs, int n_rhs, int64_t n, float* out, int flags,
                      void* stream);

/*
 * Several GGUF weight matrices applied to one lhs, as the callers of ops.qmatmul in a transformer
 * block do (q | k | v, and gate | up, take the same activations):
 *   out[j] fp32[m, n[j]] = lhs[m, k] . dequant(rhs[j])^T,  j < count, all rhs of `encoding` and of row length k.
 * Where a kernel takes the whole group (Q4_K, count <= 4: m = 1 with k <= 16384, or 2 <= m <= 16) this is one
 * launch that numbers the rows of the matrices through (the lhs is staged or narrowed once for all of them); otherwise it is one qmm_matmul per matrix, in order
 * (workspace: the largest any of them needs).  The reference exposes the per-matrix op only; fusing
 * its calls is its graph compiler's job, for which this is the kernel-side counterpart.
 * rhs, n and out are host arrays.
 */
int qmm_matmul_grouped(int encoding, const void* lhs, int lhs_dtype, int64_t m, int64_t k, int count,
                       const void* const* rhs, const int64_t* n, float* const* out, void* workspace,
                       int64_t workspace_bytes, void* stream);

/*
 * Weight planes kept across calls.  (External knowledge, not verifiable from the reference snapshot, which holds no
 * MAX code: MAX is understood to fold a weight repack step ahead of its quantized matmul kernels into model load; the
 * packed layout is contractual on disk only.)  These calls are an explicit form of such a step for the prefill GEMMs
 * here; nothing in the reference's op interface corresponds to them.
 *   qmm_repack converts the packed weights of one matrix, once, into the fp16 integer planes and scale tables
 *   that the matrix-core GEMMs read: 2 bytes per weight (Q6_K 4) plus tables, qmm_repack_bytes in all, into a
 *   256-byte aligned buffer the caller owns.  The buffer depends on the weights only.  Encodings: Q4_K, Q5_K,
 *   Q6_K; GPTQ with plain groups of 128 or 256; Q4_0 (the plane of q - 8 and its block scales: the lhs is still
 *   quantised to Q8_0 in every call).  K must be a multiple of 256.  qmm_repack_bytes returns 0, and qmm_repack
 *   QMM_ERR_UNSUPPORTED, for anything else (act-order GPTQ, other groups, other K).
 *   qmm_matmul_repacked is qmm_matmul with that buffer at hand.  Row counts for which the plane GEMMs are the
 *   faster route skip the conversion that qmm_matmul repeats per call: Q5_K / Q6_K from 49 rows (33 on matrices
 *   of 48 Mi weights or more), Q4_0 from 49, Q4_K from 129 with at least 64 tiles of 256 x 128, GPTQ from 257
 *   with at least 160 tiles of 256 x 256 or from 97 with at most 64.  Same kernels, same planes: where qmm_matmul
 *   takes the planes too, the results are equal bit for bit.  Other row counts are handed to qmm_matmul with
 *   `rhs`.  rhs = NULL (a caller that dropped the packed tensors): every row count goes through the planes.
 *   flags must be 0.  Workspace: qmm_matmul_repacked_workspace_bytes (the lhs planes, or what qmm_matmul needs
 *   for the kernels that read the packed tensors).
 *   The price is memory: the buffer is 4.25 x the packed tensor for Q4_K / Q5_K (2 bytes per weight plus one extension
 *   block per eight super-blocks and the tables: 140 MB for 14336 x 4096), 3.9 x for GPTQ, 4.9 x for Q6_K (two planes),
 *   3.6 x for Q4_0.  A host that keeps planes for every matrix holds an fp16-sized model; a host that does not pays the
 *   conversion in every qmm_matmul call that takes the plane GEMM, inside a workspace of that size.
 *   The buffer begins with a 256-byte record (encoding, N, K, GPTQ group, layout version) that qmm_repack writes.  Every
 *   qmm_matmul_repacked call that reads the planes compares the record with its own arguments on the device, behind its
 *   kernels: on a mismatch the whole result is set to NaN (planes of equal size made for another matrix shape, encoding
 *   or group would otherwise give plausible garbage).  qmm_repack_check does the same comparison on the host (it copies
 *   the record back and synchronises the stream: for load time, not for the hot path) and returns QMM_ERR_INVALID with
 *   both descriptions in qmm_last_error.  Neither can tell two matrices of the same encoding and shape apart.
 */
int64_t qmm_repack_bytes(int encoding, const qmm_gptq_config* cfg, int64_t n, int64_t k);
int qmm_repack(int encoding, const qmm_gptq_config* cfg, const void* const* rhs, int n_rhs, int64_t n, int64_t k,
               void* packed, int64_t packed_bytes, void* stream);
int qmm_repack_check(int encoding, const qmm_gptq_config* cfg, int64_t n, int64_t k, const void* packed, int64_t packed_bytes,
                     void* stream);
int64_t qmm_matmul_repacked_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k);
int qmm_matmul_repacked(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m, int64_t k,
                        const void* const* rhs, int n_rhs, const void* packed, int64_t packed_bytes, int64_t n, float* out,
                        void* workspace, int64_t workspace_bytes, int flags, void* stream);

/*
 * The gated-MLP step either side of ops.qmatmul in a Llama block (no counterpart in the reference's op set: there the
 * graph holds two qmatmul nodes, a SiLU and a multiply):
 *     out fp32[m, n] = silu(lhs . dequant(gate)^T) * (lhs . dequant(up)^T),   silu(x) = x / (1 + exp(-x)).
 * gate and up are two tensors of one GGUF encoding, uint8[n, k/epb*bpb] each.  Q4_K with one lhs row (K <= 16384) runs
 * as ONE launch of the decode kernel with the combination as its epilogue and needs no workspace; every other shape is
 * two qmm_matmul launches into the workspace and a combining launch.
 */
int64_t qmm_matmul_swiglu_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k);
int qmm_matmul_swiglu(int encoding, const void* lhs, int lhs_dtype, int64_t m, int64_t k, const void* gate, const void* up,
                      int64_t n, float* out, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * The normalisation in front of ops.qmatmul in a Llama block, fused into the call (no counterpart in the reference's op
 * set: there the graph holds an rms_norm node and a qmatmul node):
 *     y[m, k] = x * rsqrt(mean_k(x^2) + eps) * gamma,   out = qmatmul(encoding, y, rhs)
 * with the normalisation in fp32 and y rounded to bf16 when x is bf16 (what a bf16 rms_norm node hands to qmatmul).
 * x fp32 or bf16 [m, k], gamma fp32 [k], eps >= 0.  Q4_0 with m <= 4 and K <= 8192 (flags = 0) is ONE launch: the decode
 * kernel, which quantises its lhs rows to Q8_0 itself, normalises them first (gamma must then be 16-byte aligned, else the
 * general route is taken).  Every other problem is a normalisation launch into the workspace and qmm_matmul on the result.
 * flags, rhs, cfg, out as for qmm_matmul.
 */
int64_t qmm_matmul_rmsnorm_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k, int flags);
int qmm_matmul_rmsnorm(int encoding, const qmm_gptq_config* cfg, const void* x, int x_dtype, const float* gamma, float eps,
                       int64_t m, int64_t k, const void* const* rhs, int n_rhs, int64_t n, float* out, void* workspace,
                       int64_t workspace_bytes, int flags, void* stream);

/*
 * Test hook for the bit-exact integer check: raw int32 block sums
 * out[m, n, k/32] = sum_32 (q4 - 8) * q8 of Q8_0 lhs blocks (uint8[m, k/32*34])
 * against Q4_0 rhs blocks.
 */
int qmm_block_dots_q4_0(const void* lhs_q8_0, const void* rhs_q4_0, int64_t m, int64_t n,
                        int64_t k, int32_t* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QMM_H */
