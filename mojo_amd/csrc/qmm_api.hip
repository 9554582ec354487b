// C ABI of libqmm.so: argument validation and dispatch by encoding and shape.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <string>

#include "qmm_internal.h"

namespace qmm {

bool kernel_disabled(const char* family) {
    // (parsed on first use; a C++11 static initialiser runs once, also when two host threads get here together)
    static const std::string list = [] {
        const char* e = getenv("QMM_DISABLE");
        return std::string(",") + (e ? e : "") + ",";
    }();
    return list.size() > 2 && list.find(std::string(",") + family + ",") != std::string::npos;
}

}  // namespace qmm

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_status(hipError_t e, const char* what) {
    if (e == hipSuccess) return QMM_OK;
    return fail(QMM_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

bool aligned(const void* p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// GPTQ with more than 16 lhs rows: do passes of the small-batch kernel (16 rows each, bound by the bytes of the weights)
// beat the GEMM (128 x 256 output tiles, one workgroup each, bound by K per round of 256 tiles)?  Times in
// microseconds as measured on 14336 x 4096, 4096 x 14336 and 4096 x 4096 with 64 to 128 rows: a GEMM round costs
// 64 us per 4096 of K (bf16 lhs; 2.1 x that for an fp32 lhs, which runs two launches) whatever N is, so few column tiles
// (N = 4096: 16 of 256 compute units) and long K favour the passes: 4096 x 14336 with 128 bf16 rows 126 against 209 us.
// Q4_K with 2..16 lhs rows: the kernel that cuts K across workgroups, or the one that gives a workgroup whole rows?
bool q4k_kc_wins(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    // measured, 4096 x 14336, this kernel against the row kernel: 16 rows 29.5 / 49.9 us (fp32 lhs), 22.2 / 35.0 us (bf16);
    // 8 rows 27.1 / 26.9 us (fp32), 21.1 / 26.4 us (bf16); 4 rows 26.6 / 18.8 us, 20.9 / 18.7 us.  On 14336 x 4096 and on
    // K = 4096 the row kernel wins at every row count.
    return m >= (lhs_dtype == QMM_F32 ? 9 : 5) && n <= 4096 && k > 4096;
}

static bool q4k_gemm_from_9_rows(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    return encoding == QMM_Q4_K && lhs_dtype == QMM_F32 && m > 8 && m <= 16 && k > 4096 && k % 256 == 0 && n * k >= ((int64_t)128 << 20) &&
           !q4k_kc_wins(lhs_dtype, m, n, k);
}

// Q4_K with 2..4 lhs rows: the decode kernel with one sub-block per lane, or the small-batch matrix-core kernel?
bool q4k_lanes_rows_wins(int64_t n, int64_t k) {
    // The decode kernel pays per weight (its decode runs on the vector units once per row group), the matrix-core kernel
    // per K step and per launch.  Measured, 4 fp32 rows, decode kernel / matrix-core kernel: 512 x 4096 5.1 / 6.7 us,
    // 1024 x 4096 5.2 / 6.7, 2048 x 4096 6.3 / 6.8, 3072 x 4096 7.7 / 6.9, 4096 x 4096 8.9 / 7.0, 14336 x 4096 20.8 / 12.3,
    // 1024 x 8192 9.9 / 10.6, 1024 x 14336 16.2 / 17.5 (bf16 rows: 10.1 / 17.9), 4096 x 14336 42.9 / 18.0.
    static const bool forced = [] {
        const char* e = getenv("QMM_Q4K_LANES_ROWS");
        return e && e[0] == '1';
    }();
    return forced || n <= 1024 || n * k <= ((int64_t)8 << 20);
}

// Q6_K (K a multiple of 2048 up to 32768): the small-batch matrix-core kernel, or passes of the decode kernel (one or two
// lhs rows each)?
bool q6k_mm_wanted(int64_t m, int64_t n, int64_t k) {
    // Measured, small-batch kernel / decode-kernel passes, fp32 lhs: 128256 rows: 1 lhs row 87 / 78 us, 2 87 / 113, 4 95 / 225,
    // 8 98 / 449, 16 144 / 895; 14336 rows: 1 17.0 / 14.8, 2 17.5 / 20.6, 4 19.5 / 40.8, 8 21.6 / 81.7, 16 46.7 / 162;
    // 4096 rows: 2 10.3 / 9.6, 4 11.7 / 15.2, 8 13.8 / 32.9, 16 36 / 52; 1024 rows: 2 9.8 / 6.1, 4 11.2 / 7.7, 8 13.2 / 21.9,
    // 16 29 / 38; 4096 x 14336 (four rounds over K, side by side): 1 19.2 / 16.1, 2 20.0 / 22.4, 4 22.1 / 47.  (Its fixed cost is
    // the conversion of the lhs in every workgroup and round.)  QMM_Q6K_MM=1 sends every shape there.
    static const bool forced = [] {
        const char* e = getenv("QMM_Q6K_MM");
        return e && e[0] == '1';
    }();
    // (a K beyond 16384, which the decode kernel with the rows global -> LDS does not take: from one bf16 row on)
    return forced || m >= 5 || (m >= 3 && n >= 2048) || (m == 2 && (n >= 8192 || (k > 8192 && n >= 2048))) || (k > 16384 && n >= 2048);
}

// Q5_K: the small-batch matrix-core kernel, or passes of the decode kernel (up to four lhs rows each)?
bool q5k_mm_wanted(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    // Measured, small-batch kernel / decode-kernel passes, fp32 lhs (bf16 lhs: the small-batch kernel is 10-20 % faster, and
    // sixteen bf16 rows cost what eight do): 14336 x 4096: 2 lhs rows 17.5 / 17.5 us, 4 19.2 / 27.2, 8 20.9 / 53.6, 16 41.5 / 106;
    // 4096 x 4096: 4 11.9 / 11.4, 8 14.3 / 22.1; 1024 x 4096: 4 11.6 / 7.8, 8 13.9 / 15.3; 4096 x 14336: 2 34.4 / 33.1, 4 40.4 / 65.4,
    // 8 50.2 / 130; with the rounds of a long K side by side: 2 19.9 / 32.1, 4 21.6 / 65.  QMM_Q5K_MM=1 sends every shape the kernel
    // takes there.
    static const bool forced = [] {
        const char* e = getenv("QMM_Q5K_MM");
        return e && e[0] == '1';
    }();
    // Other shapes: 5120 x 5120 with 4 rows 21 / 29.8; 32000 x 4096 with 2 rows 28 / 32.2; 8192 x 28672 with one row 50 / 61.
    // (three and four bf16 rows from 16 Mi weights on: 4096 x 4096 8.8 / 9.1 against 10.6 / 10.8)
    const int64_t min3 = lhs_dtype == QMM_BF16 ? ((int64_t)16 << 20) : ((int64_t)32 << 20);
    return forced || m >= 5 || (m >= 3 && (n * k >= min3 || (k > 4096 && n >= 2048))) ||
           (m >= 2 && ((k > 8192 && n >= 2048) || n * k >= ((int64_t)96 << 20))) || (k > 16384 && n >= 2048);
}

bool gptq_small_batch_wins(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    // Passes of the small-batch kernel (16 rows each) against the GEMM (128 x 256 tiles, cut into K shares when they are few, an
    // fp32 lhs of up to 256 rows as twice the rows), in microseconds as measured on this part: 4096 x 4096, bf16 / fp32 lhs: a
    // pass 10.2 / 15.9, the GEMM at 65 .. 256 rows 24 .. 28 / 23 .. 35; 14336 x 4096: a pass 13.0 / 19.6, the GEMM 30 .. 48 / 43 .. 77.
    const bool f32 = lhs_dtype == QMM_F32, twin = qmm::gemm_gptq_twin(lhs_dtype, m);
    const int64_t me = twin ? 2 * m : m;
    const int ks = qmm::gemm_gptq_k_shares(me, n, k);
    const double tiles = (double)((me + 127) / 128) * (double)((n + 255) / 256);
    const double rounds = (double)(int64_t)((tiles * ks + 255.0) / 256.0);
    const double gemm_us = rounds * ((double)k / 4096.0) * 64.0 / ks * (f32 && !twin ? 2.1 : 1.0) + (twin || ks > 1 ? 14.0 : 0.0);
    const double pass_us = (f32 ? 12.0 : 8.0) + (double)n * (double)k * 0.52 / (f32 ? 3.8e6 : 6.0e6) + (k > 4096 ? 2.0 : 0.0);
    return (double)((m + 15) / 16) * pass_us < gemm_us;
}

bool block_params(int enc, int64_t& epb, int64_t& bpb) {
    switch (enc) {
        case QMM_Q4_0: epb = 32; bpb = 18; return true;
        case QMM_Q8_0: epb = 32; bpb = 34; return true;
        case QMM_Q8_K: epb = 256; bpb = 292; return true;
        case QMM_Q4_K: epb = 256; bpb = 144; return true;
        case QMM_Q6_K: epb = 256; bpb = 210; return true;
        case QMM_Q5_K: epb = 256; bpb = 176; return true;
        default: return false;
    }
}

int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// sym = 0 (asymmetric checkpoints: zero points other than 8) is read like sym = 1: every kernel takes the zero
// point from qzeros (stored value + 1, the AutoGPTQ v1 convention); only the quantiser here is symmetric.
int check_gptq(const qmm_gptq_config* cfg, int64_t n, int64_t k, bool quantiser = false) {
    if (!cfg) return fail(QMM_ERR_INVALID, "GPTQ requires a config");
    if (cfg->bits != 4) return fail(QMM_ERR_UNSUPPORTED, "GPTQ bits=%d: only 4-bit is supported", cfg->bits);
    if (cfg->desc_act && quantiser) return fail(QMM_ERR_UNSUPPORTED, "GPTQ desc_act=True: the quantiser here writes plain groups only");
    if (!cfg->sym && quantiser) return fail(QMM_ERR_UNSUPPORTED, "GPTQ sym=False: the quantiser here is symmetric only");
    if (cfg->group_size <= 0 || cfg->group_size % 32 || k % cfg->group_size)
        return fail(QMM_ERR_INVALID, "GPTQ group_size=%d must be a multiple of 32 dividing K=%lld", cfg->group_size,
                    (long long)k);
    if (n % 8) return fail(QMM_ERR_INVALID, "GPTQ needs N %% 8 == 0 (N=%lld)", (long long)n);
    return QMM_OK;
}

// Workspace layout of the Q4_0 path: int8 codes [m,k], fp32 scales [m,k/32], int32 sums [m,k/32].
struct Q8Planes {
    int8_t* codes;
    float* scale;
    int32_t* sum;
    int64_t bytes;
};
Q8Planes q8_planes(void* ws, int64_t m, int64_t k) {
    Q8Planes p;
    int64_t codes = align_up(m * k, 256), sc = align_up(m * (k / 32) * 4, 256);
    p.codes = (int8_t*)ws;
    p.scale = (float*)((char*)ws + codes);
    p.sum = (int32_t*)((char*)ws + codes + sc);
    p.bytes = codes + 2 * sc;
    return p;
}

}  // namespace

// Scratch memory of qmm_matmul_static: device memory that belongs to the loaded library, one copy per GPU, held
// until the process ends.  In host code the array's name is only a handle for the runtime, not a device
// address; the address on each GPU comes from hipGetSymbolAddress with that GPU current, once, and only that
// pointer is ever handed to a kernel.  (No kernel names the array, so it is the host use in static_scratch() that
// makes the compiler emit it, with a symbol the runtime can look up; marking it `used` instead keeps that
// symbol local to the code object and the lookup then fails.)
static __device__ __align__(256) unsigned char scratch[QMM_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int static_scratch(void** ws) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul_static: device ordinal %d out of range", dev);
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        // (two threads that get here together read the same address for this device)
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_status(e, "hipGetSymbolAddress(scratch)");
        if (!p || !aligned(p, 256)) return fail(QMM_ERR_HIP, "qmm_matmul_static: the static scratch buffer has no usable device address");
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *ws = p;
    return QMM_OK;
}

}  // namespace

extern "C" {

int qmm_version(void) { return 105; }

const char* qmm_last_error(void) { return g_err; }

int qmm_block_params(int encoding, int64_t* elements_per_block, int64_t* bytes_per_block) {
    int64_t e, b;
    if (!elements_per_block || !bytes_per_block) return fail(QMM_ERR_INVALID, "null output pointer");
    if (!block_params(encoding, e, b)) return fail(QMM_ERR_INVALID, "encoding %d has no block layout", encoding);
    *elements_per_block = e;
    *bytes_per_block = b;
    return QMM_OK;
}

int qmm_device_info(int32_t* compute_units, int32_t* clock_khz) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e, "hipGetDevice");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return hip_status(e, "hipGetDeviceProperties");
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    return QMM_OK;
}

int qmm_read_probe(const void* buf, int64_t bytes, void* stream) {
    if (!buf || bytes < 16) return fail(QMM_ERR_INVALID, "qmm_read_probe: needs a buffer of at least 16 bytes");
    if (!aligned(buf, 16)) return fail(QMM_ERR_INVALID, "qmm_read_probe: buffer must be 16-byte aligned");
    return hip_status(qmm::launch_read_probe(buf, bytes, (hipStream_t)stream), "qmm_read_probe");
}

int qmm_mfma_probe(void* out, int64_t out_bytes, int kind, int iters, int64_t* flops, void* stream) {
    if (!out || !flops) return fail(QMM_ERR_INVALID, "qmm_mfma_probe: null pointer");
    if (kind < 0 || kind > 6 || iters < 1 || iters > (1 << 24)) return fail(QMM_ERR_INVALID, "qmm_mfma_probe: kind 0..6, iters 1..2^24");
    int32_t cus = 0;
    if (int rc = qmm_device_info(&cus, nullptr)) return rc;
    if (!aligned(out, 4) || out_bytes < (int64_t)cus * 512 * 4)
        return fail(QMM_ERR_INVALID, "qmm_mfma_probe: out must hold 512 floats per compute unit (%lld bytes)", (long long)cus * 512 * 4);
    *flops = (int64_t)cus * 8 * iters * 16 * (kind == 4 || kind == 5 ? 2ll * 16 * 16 * 32 : 2ll * 32 * 32 * 16);
    return hip_status(qmm::launch_mfma_probe((float*)out, cus, kind, iters, (hipStream_t)stream), "qmm_mfma_probe");
}

int qmm_dequantize(int encoding, const void* rhs, int64_t n, int64_t k, void* out, int out_dtype, void* stream) {
    int64_t epb, bpb;
    if (encoding == QMM_Q8_0 || encoding == QMM_Q8_K || !block_params(encoding, epb, bpb))
        return fail(QMM_ERR_INVALID, "qmm_dequantize: encoding %d is not a GGUF weight encoding", encoding);
    if (!rhs || !out) return fail(QMM_ERR_INVALID, "qmm_dequantize: null pointer");
    if (n <= 0 || k <= 0 || k % epb)
        return fail(QMM_ERR_INVALID, "qmm_dequantize: N=%lld, K=%lld; K must be a positive multiple of %lld",
                    (long long)n, (long long)k, (long long)epb);
    if (out_dtype != QMM_F32 && out_dtype != QMM_BF16)
        return fail(QMM_ERR_INVALID, "qmm_dequantize: out_dtype must be f32 or bf16");
    if ((encoding == QMM_Q4_K || encoding == QMM_Q5_K) && !aligned(rhs, 16))
        return fail(QMM_ERR_INVALID, "qmm_dequantize: Q4_K / Q5_K rhs must be 16-byte aligned");
    return hip_status(qmm::launch_dequant(encoding, rhs, n, k, out, out_dtype, (hipStream_t)stream),
                      "qmm_dequantize");
}

int qmm_dequantize_gptq(const qmm_gptq_config* cfg, const void* qweight, const void* scales, const void* qzeros,
                        const void* g_idx, int64_t n, int64_t k, void* out, int out_dtype, void* stream) {
    if (!qweight || !scales || !qzeros || !out) return fail(QMM_ERR_INVALID, "qmm_dequantize_gptq: null pointer");
    if (n <= 0 || k <= 0) return fail(QMM_ERR_INVALID, "qmm_dequantize_gptq: empty shape");
    if (int rc = check_gptq(cfg, n, k)) return rc;
    if (cfg->desc_act && !g_idx) return fail(QMM_ERR_INVALID, "qmm_dequantize_gptq: desc_act=True needs g_idx");
    if (out_dtype != QMM_F32 && out_dtype != QMM_BF16)
        return fail(QMM_ERR_INVALID, "qmm_dequantize_gptq: out_dtype must be f32 or bf16");
    // desc_act = 0: the groups are k / group_size whatever g_idx says (it is not read)
    return hip_status(qmm::launch_dequant_gptq(qweight, scales, qzeros, cfg->desc_act ? g_idx : nullptr, n, k, cfg->group_size, out, out_dtype,
                                               (hipStream_t)stream),
                      "qmm_dequantize_gptq");
}

int qmm_quantize(int encoding, const float* x, int64_t rows, int64_t k, void* out, void* stream) {
    int64_t epb, bpb;
    if (!block_params(encoding, epb, bpb)) return fail(QMM_ERR_INVALID, "qmm_quantize: unknown encoding %d", encoding);
    if (!x || !out) return fail(QMM_ERR_INVALID, "qmm_quantize: null pointer");
    if (rows <= 0 || k <= 0 || k % epb)
        return fail(QMM_ERR_INVALID, "qmm_quantize: rows=%lld, K=%lld; K must be a positive multiple of %lld",
                    (long long)rows, (long long)k, (long long)epb);
    if (encoding == QMM_Q8_K)
        return hip_status(qmm::launch_quantize_q8_k(x, QMM_F32, rows, k, out, (hipStream_t)stream), "qmm_quantize(Q8_K)");
    return hip_status(qmm::launch_quantize(encoding, x, rows, k, out, (hipStream_t)stream), "qmm_quantize");
}

int qmm_quantize_gptq(const qmm_gptq_config* cfg, const float* w, int64_t n, int64_t k, void* qweight, void* scales,
                      void* qzeros, void* g_idx, void* stream) {
    if (!w || !qweight || !scales || !qzeros || !g_idx) return fail(QMM_ERR_INVALID, "qmm_quantize_gptq: null pointer");
    if (n <= 0 || k <= 0) return fail(QMM_ERR_INVALID, "qmm_quantize_gptq: empty shape");
    if (int rc = check_gptq(cfg, n, k, true)) return rc;
    return hip_status(
        qmm::launch_quantize_gptq(w, n, k, cfg->group_size, qweight, scales, qzeros, g_idx, (hipStream_t)stream),
        "qmm_quantize_gptq");
}

// Q4_K and GPTQ have prefill kernels that need no weight planes: the plane GEMM serves them only when the caller's
// workspace holds the planes (what qmm_matmul_workspace_bytes reports); a smaller workspace gets the other kernel.  The
// switch is per call and thread: set at the top of qmm_matmul, read by the dispatch and by the size queries under it.
static thread_local bool g_skip_twin_rows = false;
struct TwinRowsScope {
    bool prev;
    explicit TwinRowsScope(bool skip) : prev(g_skip_twin_rows) { g_skip_twin_rows = skip; }
    ~TwinRowsScope() { g_skip_twin_rows = prev; }
};
extern "C++" {
namespace qmm {
bool twin_rows_allowed() { return !g_skip_twin_rows; }
}  // namespace qmm
}
static thread_local bool g_skip_optional_planes = false;
struct OptionalPlanesScope {
    bool prev;
    explicit OptionalPlanesScope(bool skip) : prev(g_skip_optional_planes) { g_skip_optional_planes = skip; }
    ~OptionalPlanesScope() { g_skip_optional_planes = prev; }
};
static bool kquant_planes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    return qmm::gemm_planes_wanted(encoding, lhs_dtype, m, n, k) && !(encoding == QMM_Q4_K && g_skip_optional_planes);
}
static bool gptq_planes(int64_t m, int64_t n, int64_t k, int group) {
    return !g_skip_optional_planes && qmm::gemm_gptq_planes_wanted(m, n, k, group);
}

int64_t qmm_matmul_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || k <= 0) return 0;
    if (kquant_planes(encoding, lhs_dtype, m, n, k)) return qmm::gemm_planes_workspace_bytes(encoding, lhs_dtype, m, n, k);
    if (encoding == QMM_Q4_0) {
        const int64_t a = q8_planes(nullptr, m, k).bytes, b = (m >= 5 || k > 4096) && k % 32 == 0 ? qmm::gemm_q4_0_workspace_bytes(m, k) : 0;
        const int64_t c = qmm::gemm_q4_0_planes_wanted(m, n, k) ? qmm::gemm_q4_0_planes_workspace_bytes(m, n, k) : 0;
        return std::max(std::max(a, b), c);
    }
    if (encoding == QMM_Q4_K && m <= 16 && k % 256 == 0) {  // lhs planes from 9 rows on; partial sums of K chunks
        const int64_t a = qmm::gemv_q4_k_mm_plain_workspace_bytes(lhs_dtype, m, n, k), b = m >= 2 ? qmm::gemv_q4_k_kc_workspace_bytes(m, n, k) : 0;
        const int64_t c = q4k_gemm_from_9_rows(encoding, lhs_dtype, m, n, k) ? qmm::gemm_q4_k_workspace_bytes(lhs_dtype, m, n, k) : 0;
        return std::max(std::max(a, b), c);
    }
    if (encoding == QMM_Q4_K && m > 16 && k % 256 == 0) return qmm::gemm_q4_k_workspace_bytes(lhs_dtype, m, n, k);
    // (the small-batch kernels with the rounds of a long K side by side; the decode kernels need nothing)
    if (encoding == QMM_Q5_K) return q5k_mm_wanted(lhs_dtype, m, n, k) && k % 512 == 0 ? qmm::gemv_kquant_mm_workspace_bytes(m, n, k) : 0;
    if (encoding == QMM_Q6_K) return q6k_mm_wanted(m, n, k) && k % 2048 == 0 ? qmm::gemv_kquant_mm_workspace_bytes(m, n, k) : 0;
    if (encoding == QMM_GPTQ && k % 256 == 0) {  // small-batch kernel: partial sums of the K chunks; GEMM: lhs planes
        const int64_t a = qmm::gemv_gptq_mm_workspace_bytes(m, n, k), b = m > 16 ? qmm::gemm_gptq_workspace_bytes(lhs_dtype, m, n, k) : 0;
        const int64_t c = gptq_planes(m, n, k, 128) ? qmm::gemm_gptq_planes_workspace_bytes(lhs_dtype, m, n, k) : 0;  // (the group size is not known here)
        return std::max(std::max(a, b), c);
    }
    return 0;
}

static int64_t up256(int64_t v) { return (v + 255) / 256 * 256; }

// Does the kernel that serves this problem store bf16 itself?  (The Q4_K decode kernel does; everything else goes
// through an fp32 result in the workspace and a narrowing pass.)
static bool stores_bf16_itself(int encoding, int64_t m, int64_t k, int flags) {
    return encoding == QMM_Q4_K && m == 1 && k % 256 == 0 && k <= 16384 && !(flags & QMM_FLAG_ACT_Q8K) && !qmm::kernel_disabled("q4k_lanes");
}

// Q8_K activations: up to 16 lhs rows go through kernels that take the integer sub-block dots themselves, in passes of four
// rows (Q4_K: the lhs quantised inside the kernel, K <= 16384; Q5_K and Q6_K: quantised once per call into planes in the
// workspace).  More rows: the lhs is quantised, d8 * code written as fp32 rows into the workspace, and the floating-point
// path runs on those (the products of the integer treatment, summed in fp32).
constexpr int64_t kQ8kIntegerMaxRows = 16;
static bool q8k_integer_kernel(int encoding, int64_t m, int64_t k) {
    if (m > kQ8kIntegerMaxRows || k % 256) return false;
    return encoding == QMM_Q4_K ? k <= 16384 : (encoding == QMM_Q5_K || encoding == QMM_Q6_K);
}
static int64_t q8k_integer_workspace(int encoding, int64_t m, int64_t k) { return encoding == QMM_Q4_K ? 0 : qmm::q8k_planes_bytes(m, k); }

int64_t qmm_matmul_workspace_bytes_flags(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k, int flags) {
    int64_t base = qmm_matmul_workspace_bytes(encoding, lhs_dtype, m, n, k);
    if ((flags & QMM_FLAG_ACT_Q8K) && m > 0 && k > 0)
        base = q8k_integer_kernel(encoding, m, k) ? q8k_integer_workspace(encoding, m, k)
                                                  : up256(m * k * 4) + qmm_matmul_workspace_bytes(encoding, QMM_F32, m, n, k);
    if (!(flags & QMM_FLAG_OUT_BF16) || m <= 0 || n <= 0 || stores_bf16_itself(encoding, m, k, flags)) return base;
    return up256(base) + up256(m * n * 4);
}

static int matmul_f32(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m, int64_t k,
                      const void* const* rhs, int n_rhs, int64_t n, float* out, void* workspace, int64_t workspace_bytes,
                      int flags, void* stream);

int qmm_matmul(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m, int64_t k,
               const void* const* rhs, int n_rhs, int64_t n, float* out, void* workspace, int64_t workspace_bytes,
               int flags, void* stream) {
    // the plane GEMM for Q4_K / GPTQ only with a workspace that holds the planes
    const bool optional = (encoding == QMM_Q4_K || encoding == QMM_GPTQ) && m > 0 && n > 0 && k > 0 && !g_skip_optional_planes;
    const OptionalPlanesScope scope(g_skip_optional_planes ||
                                    (optional && (!workspace || workspace_bytes < qmm_matmul_workspace_bytes_flags(encoding, lhs_dtype, m, n, k, flags))));
    if (!(flags & QMM_FLAG_OUT_BF16) || (flags & ~(QMM_FLAG_W_BF16 | QMM_FLAG_ACT_Q8K | QMM_FLAG_OUT_BF16)))
        return matmul_f32(encoding, cfg, lhs, lhs_dtype, m, k, rhs, n_rhs, n, out, workspace, workspace_bytes, flags, stream);
    // bf16 output
    const int inner = flags & ~QMM_FLAG_OUT_BF16;
    if (!lhs || !rhs || !out) return fail(QMM_ERR_INVALID, "qmm_matmul: null pointer");
    if (!aligned(out, 2)) return fail(QMM_ERR_INVALID, "qmm_matmul: bf16 out must be 2-byte aligned");
    if (m > 0 && n > 0 && k > 0 && m <= INT32_MAX && n <= INT32_MAX && k <= INT32_MAX && n_rhs == 1 && rhs[0] &&
        (lhs_dtype == QMM_F32 || lhs_dtype == QMM_BF16) && aligned(lhs, 16) && aligned(rhs[0], 16) && !(inner & QMM_FLAG_W_BF16) &&
        stores_bf16_itself(encoding, m, k, inner)) {
        bool handled = false;
        hipError_t e = qmm::launch_gemv_q4_k_lanes(lhs, lhs_dtype, (const uint8_t*)rhs[0], (int)m, n, k, out, n, (hipStream_t)stream, &handled, true);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q4_K decode, bf16 out)");
        if (handled) return QMM_OK;
    }
    if (m <= 0 || n <= 0) return fail(QMM_ERR_INVALID, "qmm_matmul: M=%lld N=%lld must be positive", (long long)m, (long long)n);
    // (the fp32 result sits behind everything the inner call needs, the Q8_K round trip of the lhs included)
    const int64_t base = up256(qmm_matmul_workspace_bytes_flags(encoding, lhs_dtype, m, n, k, inner)), need = base + up256(m * n * 4);
    if (!workspace || workspace_bytes < need)
        return fail(QMM_ERR_WORKSPACE, "qmm_matmul: bf16 output of this problem goes through an fp32 result in the workspace: %lld bytes required "
                                       "(qmm_matmul_workspace_bytes_flags), %lld given", (long long)need, (long long)workspace_bytes);
    if (!aligned(workspace, 256)) return fail(QMM_ERR_INVALID, "qmm_matmul: workspace must be 256-byte aligned");
    float* tmp = (float*)((char*)workspace + base);
    if (int rc = matmul_f32(encoding, cfg, lhs, lhs_dtype, m, k, rhs, n_rhs, n, tmp, workspace, base, inner, stream)) return rc;
    return hip_status(qmm::launch_f32_to_bf16(tmp, (uint16_t*)out, m * n, (hipStream_t)stream), "qmm_matmul(narrow to bf16)");
}

static int matmul_f32(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m, int64_t k,
                      const void* const* rhs, int n_rhs, int64_t n, float* out, void* workspace, int64_t workspace_bytes,
                      int flags, void* stream) {
    hipStream_t s = (hipStream_t)stream;
    if (!lhs || !rhs || !out) return fail(QMM_ERR_INVALID, "qmm_matmul: null pointer");
    if (flags & ~(QMM_FLAG_W_BF16 | QMM_FLAG_ACT_Q8K)) return fail(QMM_ERR_INVALID, "qmm_matmul: unknown flag bits 0x%x", flags);
    if (flags & QMM_FLAG_W_BF16)
        return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul: QMM_FLAG_W_BF16 (weights rounded to bf16 before the product) has no kernel in this build");
    if (m <= 0 || n <= 0 || k <= 0)
        return fail(QMM_ERR_INVALID, "qmm_matmul: M=%lld N=%lld K=%lld must all be positive", (long long)m,
                    (long long)n, (long long)k);
    if (m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return fail(QMM_ERR_INVALID, "qmm_matmul: dimension too large");
    if (lhs_dtype != QMM_F32 && lhs_dtype != QMM_BF16)
        return fail(QMM_ERR_INVALID, "qmm_matmul: lhs dtype must be f32 or bf16");
    if (!aligned(lhs, 16) || !aligned(out, 4)) return fail(QMM_ERR_INVALID, "qmm_matmul: lhs must be 16-byte aligned");
    int64_t esz = lhs_dtype == QMM_F32 ? 4 : 2;
    int64_t need = qmm_matmul_workspace_bytes_flags(encoding, lhs_dtype, m, n, k, flags & QMM_FLAG_ACT_Q8K);
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(QMM_ERR_WORKSPACE, "qmm_matmul: workspace of %lld bytes required, %lld given", (long long)need,
                    (long long)workspace_bytes);
    if (need > 0 && !aligned(workspace, 256)) return fail(QMM_ERR_INVALID, "qmm_matmul: workspace must be 256-byte aligned");

    if (encoding == QMM_GPTQ) {
        if (n_rhs != 3 && n_rhs != 4)
            return fail(QMM_ERR_INVALID, "qmm_matmul: GPTQ takes rhs = (qweight, scales, qzeros[, g_idx]), got %d", n_rhs);
        if (int rc = check_gptq(cfg, n, k)) return rc;
        for (int i = 0; i < 3; i++)
            if (!rhs[i] || !aligned(rhs[i], 4)) return fail(QMM_ERR_INVALID, "qmm_matmul: GPTQ rhs[%d] null or misaligned", i);
        if (cfg->desc_act) {
            // act-order checkpoints: the decode kernel that looks the group of every k up, four lhs rows per pass
            if (n_rhs != 4 || !rhs[3] || !aligned(rhs[3], 4))
                return fail(QMM_ERR_INVALID, "qmm_matmul: GPTQ desc_act=True needs rhs[3] = g_idx int32[K]");
            for (int64_t m0 = 0; m0 < m; m0 += 4) {
                hipError_t e = qmm::launch_gemv_gptq_act_order((const char*)lhs + m0 * k * esz, lhs_dtype, (const uint32_t*)rhs[0],
                                                               (const uint16_t*)rhs[1], (const uint32_t*)rhs[2],
                                                               (const int32_t*)rhs[3], (int)std::min<int64_t>(4, m - m0), n, k,
                                                               cfg->group_size, out + m0 * n, n, s);
                if (e != hipSuccess) return hip_status(e, "qmm_matmul(GPTQ act-order)");
            }
            return QMM_OK;
        }
        // GEMM (128 x 256 tiles) or passes of the small-batch kernel (16 rows each)?
        if (gptq_planes(m, n, k, cfg->group_size))
            return hip_status(qmm::launch_gemm_gptq_planes(lhs, lhs_dtype, (const uint32_t*)rhs[0], (const uint16_t*)rhs[1], (const uint32_t*)rhs[2],
                                                           m, n, k, cfg->group_size, out, workspace, s),
                              "qmm_matmul(GPTQ planes GEMM)");
        const bool gemm_wins = !gptq_small_batch_wins(lhs_dtype, m, n, k);
        if (m > 16 && qmm::gemm_gptq_supported(k, cfg->group_size) &&
            (gemm_wins || !qmm::gemv_gptq_mm_supported(rhs[0], n, k, cfg->group_size)))
            return hip_status(qmm::launch_gemm_gptq(lhs, lhs_dtype, (const uint32_t*)rhs[0], (const uint16_t*)rhs[1],
                                                    (const uint32_t*)rhs[2], m, n, k, cfg->group_size, out, workspace, s),
                              "qmm_matmul(GPTQ GEMM)");
        // One pass of the matrix-core small-batch kernel per 16 lhs rows; the fewest rows go to the column kernels (weights from the
        // last-level cache, us).  More than 4096 columns, 64 per workgroup: one row, and two fp32 rows (14336 x 4096 with two rows:
        // 12.3 bf16 / 16 fp32 in the small-batch kernel, 16.5 in the column kernel); on a K past 8192 not even one (that kernel walks
        // K with one workgroup per 64 columns, the small-batch kernel splits it: 8192 x 28672 30 against 37).  Up to 4096 columns,
        // 16 per workgroup: one and two rows at any K (4096 x 4096: 4.2 / 5.9 against 6.7 / 8.0; 4096 x 14336: 9.0 / 14.2 against
        // 13.0 / 17.0), three and four fp32 rows up to K = 4096 (9.1 / 9.7 against 11.1 / 11.5).
        const bool long_k = k > 8192 && !qmm::kernel_disabled("gptq_long_k_mm");
        const bool cols16 = qmm::gemv_gptq_cols16_wanted(n, cfg->group_size) && !qmm::kernel_disabled("gptq_cols");
        const int mm_min = cols16 ? (lhs_dtype == QMM_F32 && k <= 4096 ? 5 : 3) : long_k ? 1 : (lhs_dtype == QMM_F32 ? 3 : 2);
        for (int64_t m0 = 0; m0 < m; m0 += 16) {
            int mt = (int)(m - m0 < 16 ? m - m0 : 16);
            bool handled = false;
            if (m >= mm_min) {
                hipError_t e = qmm::launch_gemv_gptq_mm((const char*)lhs + m0 * k * esz, lhs_dtype, (const uint32_t*)rhs[0],
                                                        (const uint16_t*)rhs[1], (const uint32_t*)rhs[2], mt, n, k,
                                                        cfg->group_size, out + m0 * n, n, workspace, s, &handled);
                if (e != hipSuccess) return hip_status(e, "qmm_matmul(GPTQ small batch)");
            }
            if (handled) continue;
            hipError_t e = qmm::launch_gemv_gptq((const char*)lhs + m0 * k * esz, lhs_dtype, (const uint32_t*)rhs[0],
                                                 (const uint16_t*)rhs[1], (const uint32_t*)rhs[2], mt, n, k,
                                                 cfg->group_size, out + m0 * n, n, s);
            if (e != hipSuccess) return hip_status(e, "qmm_matmul(GPTQ)");
        }
        return QMM_OK;
    }

    int64_t epb, bpb;
    if (encoding == QMM_Q8_0 || encoding == QMM_Q8_K || !block_params(encoding, epb, bpb))
        return fail(QMM_ERR_INVALID, "qmm_matmul: unknown encoding %d", encoding);
    if (n_rhs != 1 || !rhs[0]) return fail(QMM_ERR_INVALID, "qmm_matmul: GGUF encodings take exactly one rhs tensor");
    if (k % epb)
        return fail(QMM_ERR_INVALID, "qmm_matmul: K=%lld is not a multiple of the block size %lld", (long long)k,
                    (long long)epb);
    const uint8_t* w = (const uint8_t*)rhs[0];
    if ((encoding == QMM_Q4_K || encoding == QMM_Q5_K) && !aligned(w, 16))
        return fail(QMM_ERR_INVALID, "qmm_matmul: Q4_K / Q5_K rhs must be 16-byte aligned");
    if (!aligned(w, 2)) return fail(QMM_ERR_INVALID, "qmm_matmul: rhs must be 2-byte aligned");

    if (flags & QMM_FLAG_ACT_Q8K) {
        if (encoding != QMM_Q4_K && encoding != QMM_Q5_K && encoding != QMM_Q6_K)
            return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul: Q8_K activations go with Q4_K, Q5_K and Q6_K weights");
        if (q8k_integer_kernel(encoding, m, k) && encoding == QMM_Q4_K) {
            for (int64_t m0 = 0; m0 < m; m0 += 4) {
                bool handled = false;
                hipError_t e = qmm::launch_gemv_q4_k_q8k((const char*)lhs + m0 * k * esz, lhs_dtype, w, (int)std::min<int64_t>(4, m - m0), n, k,
                                                         out + m0 * n, n, s, &handled);
                if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q4_K x Q8_K)");
                if (!handled) return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul: Q4_K x Q8_K shape not taken (M=%lld K=%lld)", (long long)m, (long long)k);
            }
            return QMM_OK;
        }
        if (q8k_integer_kernel(encoding, m, k)) {
            if (encoding == QMM_Q5_K && !aligned(w, 16)) return fail(QMM_ERR_INVALID, "qmm_matmul: Q5_K rhs must be 16-byte aligned");
            const qmm::Q8KPlanes p = qmm::q8k_planes(workspace, m, k);
            hipError_t e = qmm::launch_quantize_q8_k_planes(lhs, lhs_dtype, m, k, p, s);
            if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q8_K planes)");
            for (int64_t m0 = 0; m0 < m; m0 += 4) {
                e = qmm::launch_gemv_kquant_q8k(encoding, p, m0, (int)std::min<int64_t>(4, m - m0), w, n, k, out + m0 * n, n, s);
                if (e != hipSuccess) return hip_status(e, "qmm_matmul(K-quant x Q8_K)");
            }
            return QMM_OK;
        }
        // the quantised activations as fp32 rows (d8 * code), then the floating-point path on them: the products are those of
        // the integer treatment, summed in fp32
        const int64_t ybytes = up256(m * k * 4);
        float* y = (float*)workspace;
        hipError_t e = qmm::launch_q8k_round_trip(lhs, lhs_dtype, m, k, y, s);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q8_K round trip)");
        return matmul_f32(encoding, cfg, y, QMM_F32, m, k, rhs, n_rhs, n, out, (char*)workspace + ybytes, workspace_bytes - ybytes, 0, stream);
    }
    // Q5_K and Q6_K with many lhs rows, Q4_K with more than 512 on large matrices: weights to fp16 integer planes in the workspace,
    // then the matrix cores
    if (kquant_planes(encoding, lhs_dtype, m, n, k))
        return hip_status(qmm::launch_gemm_planes(encoding, lhs, lhs_dtype, w, m, n, k, out, workspace, s), "qmm_matmul(K-quant planes GEMM)");
    // Q5_K with several lhs rows: the small-batch matrix-core kernel (passes of 16 or 8 rows)
    if (encoding == QMM_Q5_K && q5k_mm_wanted(lhs_dtype, m, n, k) && qmm::gemv_q5_k_mm_supported(w, m, n, k))
        return hip_status(qmm::launch_gemv_q5_k_mm(lhs, lhs_dtype, w, (int)m, n, k, out, n, workspace, s), "qmm_matmul(Q5_K small batch)");
    if (encoding == QMM_Q5_K) {
        // a decode-shaped kernel; a pass takes as many lhs rows as fit its LDS copy of the lhs
        const int64_t ngroups = (k / 256 + 15) / 16;
        const int64_t pass = ngroups <= 2 ? 4 : ngroups <= 4 ? 2 : 1;
        if (ngroups > 8) return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul: Q5_K takes K <= 32768 (K = %lld)", (long long)k);
        for (int64_t m0 = 0; m0 < m; m0 += pass) {
            bool handled = false;
            hipError_t e = qmm::launch_gemv_q5_k((const char*)lhs + m0 * k * esz, lhs_dtype, w, (int)std::min<int64_t>(pass, m - m0), n, k,
                                                 out + m0 * n, n, s, &handled);
            if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q5_K)");
            if (!handled) return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul: Q5_K shape not taken (M=%lld K=%lld)", (long long)m, (long long)k);
        }
        return QMM_OK;
    }
    if (encoding == QMM_Q4_0 && qmm::gemm_q4_0_planes_wanted(m, n, k))
        return hip_status(qmm::launch_gemm_q4_0_planes(lhs, lhs_dtype, w, m, n, k, out, workspace, s), "qmm_matmul(Q4_0 plane GEMM)");
    // (two rows and more on a K beyond what the decode kernel takes: the matrix-core kernel too, 4096 x 14336 with 4 rows 32 -> 16 us)
    // (three and four rows on a K beyond 4096 as well: 8192 x 8192 with 4 rows 34.8 -> 14.4 us, 5120 x 5120 18.1 -> 12.2)
    if (encoding == QMM_Q4_0 && (m >= 5 || (m >= 2 && k > 8192 && k % 256 == 0) || (m >= 3 && k > 4096 && k % 256 == 0)) && !qmm::kernel_disabled("q4_0_mfma"))
        return hip_status(qmm::launch_gemm_q4_0(lhs, lhs_dtype, w, m, n, k, out, workspace, s), "qmm_matmul(Q4_0 int8 MFMA)");
    if (encoding == QMM_Q4_0 && m <= 4) {
        // decode: the kernel that quantises the lhs itself (takes K <= 8192)
        bool handled = false;
        hipError_t e = qmm::launch_gemv_q4_0_stream(lhs, lhs_dtype, w, (int)m, n, k, out, n, s, &handled);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q4_0 decode)");
        if (handled) return QMM_OK;
    }
    if (encoding == QMM_Q4_0) {
        Q8Planes p = q8_planes(workspace, m, k);
        hipError_t e = qmm::launch_quantize_q8_0(lhs, lhs_dtype, m, k, nullptr, p.codes, p.scale, p.sum, s);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q8_0 quantise)");
        for (int64_t m0 = 0; m0 < m; m0 += 16) {
            int mt = (int)(m - m0 < 16 ? m - m0 : 16);
            e = qmm::launch_gemv_q4_0(p.codes + m0 * k, p.scale + m0 * (k / 32), p.sum + m0 * (k / 32), w, mt, n, k,
                                      out + m0 * n, n, s);
            if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q4_0)");
        }
        return QMM_OK;
    }

    // 2..4 lhs rows on a small matrix: the decode kernel with one sub-block per lane (the activations of four rows fit a
    // lane's registers)
    // (not with 3 or 4 rows where the matrix-core kernel cuts a long K over the grid: 1024 x 14336 with 4 fp32 rows 23.4 -> 10.5 us,
    // bf16 rows 13.6 -> 10.0)
    const bool q4k_mm_cuts_k = encoding == QMM_Q4_K && m >= 2 && m <= 8 && !qmm::kernel_disabled("q4k_mm") &&
                               qmm::gemv_q4_k_mm_plain_workspace_bytes(lhs_dtype, m, n, k) > 0;
    if (encoding == QMM_Q4_K && m >= 2 && m <= 4 && q4k_lanes_rows_wins(n, k) && !(m >= 3 && q4k_mm_cuts_k)) {
        bool handled = false;
        hipError_t e = qmm::launch_gemv_q4_k_lanes_rows(lhs, lhs_dtype, w, (int)m, n, k, out, n, s, &handled);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q4_K decode, 2..4 rows)");
        if (handled) return QMM_OK;
    }
    // 2..16 lhs rows on few weight rows and long K: the small-batch kernel that cuts K across workgroups (up to 8 rows the
    // matrix-core kernel below does so itself where its grid then fills the part: 4096 x 14336 with 8 bf16 rows 20.6 -> 15.6 us)
    if (encoding == QMM_Q4_K && m >= 2 && m <= 16 && q4k_kc_wins(lhs_dtype, m, n, k) && !q4k_mm_cuts_k && qmm::gemv_q4_k_kc_supported(w, k)) {
        bool handled = false;
        hipError_t e = qmm::launch_gemv_q4_k_kc(lhs, lhs_dtype, w, (int)m, n, k, out, n, workspace, s, &handled);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul(Q4_K small batch, K chunks)");
        if (handled) return QMM_OK;
    }
    // 3..16 lhs rows: the small-batch matrix-core kernel; more: the prefill kernel (which also takes 9..16 fp32 rows on a large
    // matrix with a long K, where the small-batch kernel works through two planes of a prepared lhs: 28672 x 8192 with 16 rows
    // 70 us against 61 for 32 rows, 8192 x 28672 94 against 76)
    if (q4k_gemm_from_9_rows(encoding, lhs_dtype, m, n, k))
        return hip_status(qmm::launch_gemm_q4_k(lhs, lhs_dtype, w, m, n, k, out, workspace, s), "qmm_matmul(Q4_K GEMM)");
    if (encoding == QMM_Q4_K && m >= 2 && m <= 16 && !qmm::kernel_disabled("q4k_mm"))
        return hip_status(qmm::launch_gemv_q4_k_mm(lhs, lhs_dtype, w, m, n, k, out, workspace, s), "qmm_matmul(Q4_K small batch)");
    if (encoding == QMM_Q4_K && m > 16)
        return hip_status(qmm::launch_gemm_q4_k(lhs, lhs_dtype, w, m, n, k, out, workspace, s), "qmm_matmul(Q4_K GEMM)");

    // Q6_K with 2..64 lhs rows: the small-batch matrix-core kernel (passes of 16 or 8 rows)
    if (encoding == QMM_Q6_K && q6k_mm_wanted(m, n, k) && qmm::gemv_q6_k_mm_supported(w, m, n, k))
        return hip_status(qmm::launch_gemv_q6_k_mm(lhs, lhs_dtype, w, (int)m, n, k, out, n, workspace, s), "qmm_matmul(Q6_K small batch)");

    // (Q6_K with more than four rows on a long K that is no multiple of 2048: passes of four rows through the kernel that stages
    // the lhs, not the first-version kernel on all of them: 4096 x 11008 with 8 rows 102 -> 73 us)
    const int64_t pass = encoding == QMM_Q6_K && m > 4 && k % 2048 != 0 && k > 8192 ? 4 : 16;
    for (int64_t m0 = 0; m0 < m; m0 += pass) {
        int mt = (int)(m - m0 < pass ? m - m0 : pass);
        const void* a = (const char*)lhs + m0 * k * esz;
        hipError_t e = encoding == QMM_Q4_K ? qmm::launch_gemv_q4_k(a, lhs_dtype, w, mt, n, k, out + m0 * n, n, s)
                                            : qmm::launch_gemv_q6_k(a, lhs_dtype, w, mt, n, k, out + m0 * n, n, s);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul");
    }
    return QMM_OK;
}

int64_t qmm_matmul_rmsnorm_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k, int flags) {
    if (m <= 0 || k <= 0) return 0;
    return up256(m * k * (lhs_dtype == QMM_F32 ? 4 : 2)) + qmm_matmul_workspace_bytes_flags(encoding, lhs_dtype, m, n, k, flags);
}

int qmm_matmul_rmsnorm(int encoding, const qmm_gptq_config* cfg, const void* x, int x_dtype, const float* gamma, float eps, int64_t m,
                       int64_t k, const void* const* rhs, int n_rhs, int64_t n, float* out, void* workspace, int64_t workspace_bytes,
                       int flags, void* stream) {
    hipStream_t s = (hipStream_t)stream;
    if (!x || !gamma || !rhs || !out) return fail(QMM_ERR_INVALID, "qmm_matmul_rmsnorm: null pointer");
    if (m <= 0 || n <= 0 || k <= 0 || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX)
        return fail(QMM_ERR_INVALID, "qmm_matmul_rmsnorm: M=%lld N=%lld K=%lld out of range", (long long)m, (long long)n, (long long)k);
    if (x_dtype != QMM_F32 && x_dtype != QMM_BF16) return fail(QMM_ERR_INVALID, "qmm_matmul_rmsnorm: x dtype must be f32 or bf16");
    if (!aligned(x, 16) || !aligned(gamma, 4)) return fail(QMM_ERR_INVALID, "qmm_matmul_rmsnorm: x must be 16-byte aligned, gamma 4-byte aligned");
    if (!(eps >= 0.0f)) return fail(QMM_ERR_INVALID, "qmm_matmul_rmsnorm: eps must be non-negative");
    // One launch: the Q4_0 decode kernel normalises the rows it quantises anyway.
    if (encoding == QMM_Q4_0 && m <= 4 && flags == 0 && n_rhs == 1 && rhs[0] && k % 32 == 0 && aligned(rhs[0], 2)) {
        bool handled = false;
        hipError_t e = qmm::launch_gemv_q4_0_stream(x, x_dtype, (const uint8_t*)rhs[0], (int)m, n, k, out, n, s, &handled, gamma, eps);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul_rmsnorm(Q4_0 decode)");
        if (handled) return QMM_OK;
    }
    // Otherwise: normalised rows into the workspace, then the matmul on them.
    const int64_t ybytes = up256(m * k * (x_dtype == QMM_F32 ? 4 : 2));
    const int64_t need = ybytes + qmm_matmul_workspace_bytes_flags(encoding, x_dtype, m, n, k, flags);
    if (!workspace || workspace_bytes < need)
        return fail(QMM_ERR_WORKSPACE, "qmm_matmul_rmsnorm: workspace of %lld bytes required (qmm_matmul_rmsnorm_workspace_bytes), %lld given",
                    (long long)need, (long long)workspace_bytes);
    if (!aligned(workspace, 256)) return fail(QMM_ERR_INVALID, "qmm_matmul_rmsnorm: workspace must be 256-byte aligned");
    hipError_t e = qmm::launch_rmsnorm(x, x_dtype, gamma, eps, m, k, workspace, s);
    if (e != hipSuccess) return hip_status(e, "qmm_matmul_rmsnorm(normalise)");
    return qmm_matmul(encoding, cfg, workspace, x_dtype, m, k, rhs, n_rhs, n, out, (char*)workspace + ybytes, workspace_bytes - ybytes, flags, stream);
}

int qmm_matmul_static(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m, int64_t k,
                      const void* const* rhs, int n_rhs, int64_t n, float* out, int flags, void* stream) {
    int64_t need = qmm_matmul_workspace_bytes_flags(encoding, lhs_dtype, m, n, k, flags);
    const TwinRowsScope twin(need > (int64_t)QMM_STATIC_SCRATCH_BYTES);  // (the two-pass treatment of an fp32 lhs needs less)
    if (need > (int64_t)QMM_STATIC_SCRATCH_BYTES) need = qmm_matmul_workspace_bytes_flags(encoding, lhs_dtype, m, n, k, flags);
    if (need > (int64_t)QMM_STATIC_SCRATCH_BYTES && (encoding == QMM_Q4_K || encoding == QMM_GPTQ)) {
        const OptionalPlanesScope no_planes(true);  // the kernels that need no weight planes
        need = qmm_matmul_workspace_bytes_flags(encoding, lhs_dtype, m, n, k, flags);
    }
    if (need > (int64_t)QMM_STATIC_SCRATCH_BYTES)
        return fail(QMM_ERR_WORKSPACE,
                    "qmm_matmul_static: this problem needs %lld bytes of scratch and the static buffer holds %lld; "
                    "use qmm_matmul with a workspace of the caller's",
                    (long long)need, (long long)QMM_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return qmm_matmul(encoding, cfg, lhs, lhs_dtype, m, k, rhs, n_rhs, n, out, ws, (int64_t)QMM_STATIC_SCRATCH_BYTES, flags, stream);
}

// Weight planes kept across calls.  The buffer starts with a 256-byte record of what it was made for; the planes follow.
namespace {
constexpr int64_t kPackHeaderBytes = 256;
constexpr uint32_t kPackMagic = 0x504D4D51u;  // "QMMP"
constexpr uint32_t kPackLayout = 1;           // bumped whenever the plane layouts change
struct PackHeader {
    uint32_t magic, layout;
    int32_t encoding, group;
    int64_t n, k, bytes;
};
static_assert(sizeof(PackHeader) <= kPackHeaderBytes, "header fits its 256 bytes");
__host__ __device__ inline bool same_header(const PackHeader& a, const PackHeader& b) {
    return a.magic == b.magic && a.layout == b.layout && a.encoding == b.encoding && a.group == b.group && a.n == b.n && a.k == b.k &&
           a.bytes == b.bytes;
}
PackHeader make_header(int encoding, const qmm_gptq_config* cfg, int64_t n, int64_t k, int64_t bytes) {
    PackHeader h;
    h.magic = kPackMagic;
    h.layout = kPackLayout;
    h.encoding = encoding;
    h.group = encoding == QMM_GPTQ && cfg ? cfg->group_size : 0;
    h.n = n;
    h.k = k;
    h.bytes = bytes;
    return h;
}
__global__ void pack_header_write_kernel(PackHeader* at, const PackHeader h) {
    if (blockIdx.x == 0 && threadIdx.x == 0) *at = h;
}
// Runs behind the kernels of a qmm_matmul_repacked call.  A buffer whose record says another encoding, shape or group than the
// call (planes of the same size made for something else pass every host-side check) turns the whole result into NaN: a
// wrong buffer cannot pass for a right one.
__global__ __launch_bounds__(256) void pack_header_check_kernel(const PackHeader* at, const PackHeader want, float* out, int64_t count) {
    const PackHeader have = *at;
    if (same_header(have, want)) return;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) out[i] = __uint_as_float(0x7fc00000u);
}
}  // namespace

static bool repackable(int encoding, const qmm_gptq_config* cfg, int64_t n, int64_t k) {
    if (n <= 0 || k < 256 || k % 256 || n > INT32_MAX || k > INT32_MAX) return false;
    if (encoding == QMM_GPTQ) return cfg && cfg->bits == 4 && !cfg->desc_act && qmm::gptq_planes_supported(n, k, cfg->group_size);
    return encoding == QMM_Q4_K || encoding == QMM_Q5_K || encoding == QMM_Q6_K || encoding == QMM_Q4_0;
}

static int64_t repack_plane_bytes(int encoding, int64_t n, int64_t k) {
    if (encoding == QMM_Q4_0) return qmm::repacked_q4_0_bytes(n, k);
    return encoding == QMM_GPTQ ? qmm::repacked_gptq_bytes(n, k) : qmm::repacked_planes_bytes(encoding, n, k);
}

int64_t qmm_repack_bytes(int encoding, const qmm_gptq_config* cfg, int64_t n, int64_t k) {
    if (!repackable(encoding, cfg, n, k)) return 0;
    return kPackHeaderBytes + repack_plane_bytes(encoding, n, k);
}

int qmm_repack_check(int encoding, const qmm_gptq_config* cfg, int64_t n, int64_t k, const void* packed, int64_t packed_bytes,
                     void* stream) {
    if (!packed) return fail(QMM_ERR_INVALID, "qmm_repack_check: null pointer");
    if (!repackable(encoding, cfg, n, k))
        return fail(QMM_ERR_UNSUPPORTED, "qmm_repack_check: no weight planes for encoding %d with N=%lld K=%lld", encoding, (long long)n, (long long)k);
    const int64_t need = qmm_repack_bytes(encoding, cfg, n, k);
    if (packed_bytes < need || !aligned(packed, 256))
        return fail(QMM_ERR_INVALID, "qmm_repack_check: the packed buffer must be 256-byte aligned and hold qmm_repack_bytes = %lld bytes (%lld given)",
                    (long long)need, (long long)packed_bytes);
    PackHeader have;
    hipError_t e = hipMemcpyAsync(&have, packed, sizeof(have), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return hip_status(e, "qmm_repack_check");
    const PackHeader want = make_header(encoding, cfg, n, k, need);
    if (have.magic != kPackMagic) return fail(QMM_ERR_INVALID, "qmm_repack_check: the buffer does not start with the record qmm_repack writes");
    if (!same_header(have, want))
        return fail(QMM_ERR_INVALID, "qmm_repack_check: the buffer holds planes of encoding %d, N=%lld, K=%lld, group %d, layout %u; the call names "
                                     "encoding %d, N=%lld, K=%lld, group %d, layout %u", have.encoding, (long long)have.n, (long long)have.k, have.group,
                    have.layout, want.encoding, (long long)want.n, (long long)want.k, want.group, want.layout);
    return QMM_OK;
}

int qmm_repack(int encoding, const qmm_gptq_config* cfg, const void* const* rhs, int n_rhs, int64_t n, int64_t k, void* packed,
               int64_t packed_bytes, void* stream) {
    if (!rhs || !packed) return fail(QMM_ERR_INVALID, "qmm_repack: null pointer");
    if (!repackable(encoding, cfg, n, k))
        return fail(QMM_ERR_UNSUPPORTED, "qmm_repack: no weight planes for encoding %d with N=%lld K=%lld (Q4_0, Q4_K, Q5_K, Q6_K, and 4-bit GPTQ with "
                                         "plain groups of 128 or 256; K a multiple of 256)", encoding, (long long)n, (long long)k);
    const int64_t need = qmm_repack_bytes(encoding, cfg, n, k);
    if (packed_bytes < need) return fail(QMM_ERR_WORKSPACE, "qmm_repack: %lld bytes required (qmm_repack_bytes), %lld given", (long long)need, (long long)packed_bytes);
    if (!aligned(packed, 256)) return fail(QMM_ERR_INVALID, "qmm_repack: the buffer must be 256-byte aligned");
    void* const planes = (char*)packed + kPackHeaderBytes;
    auto finish = [&](hipError_t e, const char* what) {
        if (e != hipSuccess) return hip_status(e, what);
        pack_header_write_kernel<<<dim3(1), dim3(64), 0, (hipStream_t)stream>>>((PackHeader*)packed, make_header(encoding, cfg, n, k, need));
        return hip_status(hipGetLastError(), "qmm_repack(record)");
    };
    if (encoding == QMM_GPTQ) {
        if (n_rhs != 3 && n_rhs != 4) return fail(QMM_ERR_INVALID, "qmm_repack: GPTQ takes rhs = (qweight, scales, qzeros[, g_idx]), got %d", n_rhs);
        if (int rc = check_gptq(cfg, n, k)) return rc;
        for (int i = 0; i < 3; i++)
            if (!rhs[i] || !aligned(rhs[i], 4)) return fail(QMM_ERR_INVALID, "qmm_repack: GPTQ rhs[%d] null or misaligned", i);
        return finish(qmm::launch_repack_gptq((const uint32_t*)rhs[0], (const uint16_t*)rhs[1], (const uint32_t*)rhs[2], n, k, cfg->group_size,
                                              planes, (hipStream_t)stream), "qmm_repack(GPTQ)");
    }
    if (n_rhs != 1 || !rhs[0]) return fail(QMM_ERR_INVALID, "qmm_repack: GGUF encodings take exactly one rhs tensor");
    if (!aligned(rhs[0], encoding == QMM_Q6_K || encoding == QMM_Q4_0 ? 2 : 16))
        return fail(QMM_ERR_INVALID, "qmm_repack: rhs misaligned (Q4_K / Q5_K 16 bytes, Q4_0 / Q6_K 2)");
    if (encoding == QMM_Q4_0)
        return finish(qmm::launch_repack_q4_0((const uint8_t*)rhs[0], n, k, planes, (hipStream_t)stream), "qmm_repack(Q4_0)");
    return finish(qmm::launch_repack_planes(encoding, (const uint8_t*)rhs[0], n, k, planes, (hipStream_t)stream), "qmm_repack");
}

// Does a call with these rows go through the planes?  Without the packed tensors every row count does.
// Q4_0: passes of the 16-row int8 kernel against the kept planes.  4096 x 4096: 28 us against 35 at 64 rows, 41 against 37 at 96;
// 4096 x 14336: 57 against 83 at 64 rows, 84 against 84 at 96.
static int64_t q4_0_repacked_min_rows(int64_t k) { return k > 4096 ? 96 : 80; }
static bool repacked_path(int encoding, int64_t m, int64_t n, int64_t k, bool have_rhs) {
    if (!have_rhs) return true;
    if (encoding == QMM_Q4_0) return m > q4_0_repacked_min_rows(k);
    return encoding == QMM_GPTQ ? qmm::repacked_gptq_wanted(m, n) : qmm::repacked_planes_wanted(encoding, m, n, k);
}

int64_t qmm_matmul_repacked_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || n <= 0 || k < 256 || k % 256) return 0;
    const int64_t planes = encoding == QMM_Q4_0 ? qmm::repacked_q4_0_workspace_bytes(m, n, k)
                           : encoding == QMM_GPTQ ? qmm::repacked_gptq_workspace_bytes(lhs_dtype, m, k)
                                                  : qmm::repacked_planes_workspace_bytes(encoding, lhs_dtype, m, n, k);
    if (repacked_path(encoding, m, n, k, true)) return planes;
    const OptionalPlanesScope no_planes(true);  // the other route: qmm_matmul's kernels on the packed tensors (or, without those, the planes)
    return std::max(planes, qmm_matmul_workspace_bytes(encoding, lhs_dtype, m, n, k));
}

int qmm_matmul_repacked(int encoding, const qmm_gptq_config* cfg, const void* lhs, int lhs_dtype, int64_t m, int64_t k,
                        const void* const* rhs, int n_rhs, const void* packed, int64_t packed_bytes, int64_t n, float* out,
                        void* workspace, int64_t workspace_bytes, int flags, void* stream) {
    if (!lhs || !packed || !out) return fail(QMM_ERR_INVALID, "qmm_matmul_repacked: null pointer");
    if (flags) return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul_repacked: flags must be 0 (0x%x given)", flags);
    if (m <= 0 || m > INT32_MAX) return fail(QMM_ERR_INVALID, "qmm_matmul_repacked: M=%lld", (long long)m);
    if (!repackable(encoding, cfg, n, k))
        return fail(QMM_ERR_UNSUPPORTED, "qmm_matmul_repacked: no weight planes for encoding %d with N=%lld K=%lld", encoding, (long long)n, (long long)k);
    if (packed_bytes < qmm_repack_bytes(encoding, cfg, n, k) || !aligned(packed, 256))
        return fail(QMM_ERR_INVALID, "qmm_matmul_repacked: the packed buffer must be 256-byte aligned and hold qmm_repack_bytes = %lld bytes (%lld given)",
                    (long long)qmm_repack_bytes(encoding, cfg, n, k), (long long)packed_bytes);
    if (!repacked_path(encoding, m, n, k, rhs != nullptr)) {
        const OptionalPlanesScope no_planes(true);
        return qmm_matmul(encoding, cfg, lhs, lhs_dtype, m, k, rhs, n_rhs, n, out, workspace, workspace_bytes, 0, stream);
    }
    if (lhs_dtype != QMM_F32 && lhs_dtype != QMM_BF16) return fail(QMM_ERR_INVALID, "qmm_matmul_repacked: lhs dtype must be f32 or bf16");
    if (!aligned(lhs, 16) || !aligned(out, 4)) return fail(QMM_ERR_INVALID, "qmm_matmul_repacked: lhs must be 16-byte aligned");
    const int64_t need = encoding == QMM_Q4_0 ? qmm::repacked_q4_0_workspace_bytes(m, n, k)
                         : encoding == QMM_GPTQ ? qmm::repacked_gptq_workspace_bytes(lhs_dtype, m, k)
                                                : qmm::repacked_planes_workspace_bytes(encoding, lhs_dtype, m, n, k);
    if (!workspace || workspace_bytes < need)
        return fail(QMM_ERR_WORKSPACE, "qmm_matmul_repacked: workspace of %lld bytes required, %lld given", (long long)need, (long long)workspace_bytes);
    if (!aligned(workspace, 256)) return fail(QMM_ERR_INVALID, "qmm_matmul_repacked: workspace must be 256-byte aligned");
    const void* const planes = (const char*)packed + kPackHeaderBytes;
    hipError_t e;
    if (encoding == QMM_Q4_0) e = qmm::launch_gemm_q4_0_repacked(lhs, lhs_dtype, planes, m, n, k, out, workspace, (hipStream_t)stream);
    else if (encoding == QMM_GPTQ) e = qmm::launch_gemm_gptq_repacked(lhs, lhs_dtype, planes, m, n, k, cfg->group_size, out, workspace, (hipStream_t)stream);
    else e = qmm::launch_gemm_planes_repacked(encoding, lhs, lhs_dtype, planes, m, n, k, out, workspace, (hipStream_t)stream);
    if (e != hipSuccess) return hip_status(e, "qmm_matmul_repacked");
    // the record at the head of the buffer against this call, on the device (the host never reads the buffer here)
    const int64_t count = m * n;
    pack_header_check_kernel<<<dim3((unsigned)std::min<int64_t>((count + 255) / 256, 1024)), dim3(256), 0, (hipStream_t)stream>>>(
        (const PackHeader*)packed, make_header(encoding, cfg, n, k, qmm_repack_bytes(encoding, cfg, n, k)), out, count);
    return hip_status(hipGetLastError(), "qmm_matmul_repacked(record check)");
}

int qmm_matmul_grouped(int encoding, const void* lhs, int lhs_dtype, int64_t m, int64_t k, int count,
                       const void* const* rhs, const int64_t* n, float* const* out, void* workspace,
                       int64_t workspace_bytes, void* stream) {
    if (!lhs || !rhs || !n || !out) return fail(QMM_ERR_INVALID, "qmm_matmul_grouped: null pointer");
    if (count < 1 || count > 64) return fail(QMM_ERR_INVALID, "qmm_matmul_grouped: count %d out of range (1..64)", count);
    int64_t epb, bpb;
    if (encoding == QMM_Q8_0 || encoding == QMM_Q8_K || encoding == QMM_GPTQ || !block_params(encoding, epb, bpb))
        return fail(QMM_ERR_INVALID, "qmm_matmul_grouped: encoding %d is not a GGUF weight encoding", encoding);
    for (int j = 0; j < count; j++)
        if (!rhs[j] || !out[j] || n[j] <= 0) return fail(QMM_ERR_INVALID, "qmm_matmul_grouped: matrix %d: null pointer or N <= 0", j);
    if (encoding == QMM_Q4_K && m >= 1 && m <= 16 && k > 0 && k % 256 == 0 && count <= qmm::kLanesMaxMats &&
        (lhs_dtype == QMM_F32 || lhs_dtype == QMM_BF16) && aligned(lhs, 16)) {
        bool ok = true;
        int64_t total = 0;
        const uint8_t* ws[qmm::kLanesMaxMats];
        for (int j = 0; j < count; j++) {
            ok = ok && aligned(rhs[j], 16) && aligned(out[j], 4);
            total += n[j];
            ws[j] = (const uint8_t*)rhs[j];
        }
        if (ok && total <= INT32_MAX && m == 1) {
            bool handled = false;
            hipError_t e = qmm::launch_gemv_q4_k_lanes_grouped(lhs, lhs_dtype, count, ws, n, out, 1, k, 0, (hipStream_t)stream, &handled);
            if (e != hipSuccess) return hip_status(e, "qmm_matmul_grouped(Q4_K decode)");
            if (handled) return QMM_OK;
        }
        if (ok && total <= INT32_MAX && m >= 2 && m <= 4) {
            // Each matrix goes to the kernel qmm_matmul would give it, so a group and separate calls agree bit for bit:
            // the small ones as one launch of the decode kernel, the others (below) as one of the matrix-core kernel.
            const uint8_t* small_w[qmm::kLanesMaxMats];
            int64_t small_n[qmm::kLanesMaxMats];
            float* small_out[qmm::kLanesMaxMats];
            int small = 0;
            for (int j = 0; j < count; j++)
                if (q4k_lanes_rows_wins(n[j], k)) small_w[small] = ws[j], small_n[small] = n[j], small_out[small++] = out[j];
            bool handled = false;
            if (small > 0) {
                hipError_t e = qmm::launch_gemv_q4_k_lanes_rows_grouped(lhs, lhs_dtype, small, small_w, small_n, small_out, (int)m, k, 0,
                                                                        (hipStream_t)stream, &handled);
                if (e != hipSuccess) return hip_status(e, "qmm_matmul_grouped(Q4_K decode, 2..4 rows)");
            }
            if (handled) {
                if (small == count) return QMM_OK;
                int rest = 0;
                const void* rest_w[qmm::kLanesMaxMats];
                int64_t rest_n[qmm::kLanesMaxMats];
                float* rest_out[qmm::kLanesMaxMats];
                for (int j = 0; j < count; j++)
                    if (!q4k_lanes_rows_wins(n[j], k)) rest_w[rest] = rhs[j], rest_n[rest] = n[j], rest_out[rest++] = out[j];
                return qmm_matmul_grouped(encoding, lhs, lhs_dtype, m, k, rest, rest_w, rest_n, rest_out, workspace, workspace_bytes, stream);
            }
        }
        if (ok && total <= INT32_MAX && m >= 2 && !qmm::kernel_disabled("q4k_mm")) {
            // the lhs is narrowed once (in the kernel up to 8 rows, by the separate pass beyond) for all the matrices
            const int64_t need = qmm::gemv_q4_k_mm_workspace_bytes(lhs_dtype, m, k);
            if (need > 0 && (!workspace || workspace_bytes < need))
                return fail(QMM_ERR_WORKSPACE, "qmm_matmul_grouped: workspace of %lld bytes required, %lld given", (long long)need,
                            (long long)workspace_bytes);
            if (need > 0 && !aligned(workspace, 256)) return fail(QMM_ERR_INVALID, "qmm_matmul_grouped: workspace must be 256-byte aligned");
            return hip_status(qmm::launch_gemv_q4_k_mm_grouped(lhs, lhs_dtype, count, ws, n, out, m, k, workspace, (hipStream_t)stream),
                              "qmm_matmul_grouped(Q4_K small batch)");
        }
    }
    for (int j = 0; j < count; j++) {
        const void* one[1] = {rhs[j]};
        if (int rc = qmm_matmul(encoding, nullptr, lhs, lhs_dtype, m, k, one, 1, n[j], out[j], workspace, workspace_bytes, 0, stream))
            return rc;
    }
    return QMM_OK;
}

int64_t qmm_matmul_swiglu_workspace_bytes(int encoding, int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    // one lhs row of Q4_K goes through the decode kernel with the combination as its epilogue: nothing to keep
    if (encoding == QMM_Q4_K && m == 1 && k % 256 == 0 && k <= 16384) return 0;
    return align_up(qmm_matmul_workspace_bytes(encoding, lhs_dtype, m, n, k), 256) + 2 * align_up(m * n * 4, 256);
}

int qmm_matmul_swiglu(int encoding, const void* lhs, int lhs_dtype, int64_t m, int64_t k, const void* gate, const void* up,
                      int64_t n, float* out, void* workspace, int64_t workspace_bytes, void* stream) {
    if (!lhs || !gate || !up || !out) return fail(QMM_ERR_INVALID, "qmm_matmul_swiglu: null pointer");
    int64_t epb, bpb;
    if (encoding == QMM_Q8_0 || encoding == QMM_Q8_K || encoding == QMM_GPTQ || !block_params(encoding, epb, bpb))
        return fail(QMM_ERR_INVALID, "qmm_matmul_swiglu: encoding %d is not a GGUF weight encoding", encoding);
    if (m <= 0 || n <= 0 || k <= 0 || k % epb || m > INT32_MAX || n > INT32_MAX / 2 || k > INT32_MAX)
        return fail(QMM_ERR_INVALID, "qmm_matmul_swiglu: M=%lld N=%lld K=%lld (K a positive multiple of %lld)", (long long)m,
                    (long long)n, (long long)k, (long long)epb);
    if (lhs_dtype != QMM_F32 && lhs_dtype != QMM_BF16) return fail(QMM_ERR_INVALID, "qmm_matmul_swiglu: lhs dtype must be f32 or bf16");
    if (!aligned(lhs, 16) || !aligned(out, 4)) return fail(QMM_ERR_INVALID, "qmm_matmul_swiglu: lhs must be 16-byte aligned");
    if (encoding == QMM_Q4_K && m == 1 && k % 256 == 0 && aligned(gate, 16) && aligned(up, 16)) {
        const uint8_t* ws[2] = {(const uint8_t*)gate, (const uint8_t*)up};
        const int64_t ns[2] = {n, n};
        float* outs[2] = {out, out};
        bool handled = false;
        hipError_t e = qmm::launch_gemv_q4_k_lanes_grouped(lhs, lhs_dtype, 2, ws, ns, outs, 1, k, 0, (hipStream_t)stream, &handled, true);
        if (e != hipSuccess) return hip_status(e, "qmm_matmul_swiglu(Q4_K decode)");
        if (handled) return QMM_OK;
    }
    // two products into the workspace, then the combination
    const int64_t mm_ws = align_up(qmm_matmul_workspace_bytes(encoding, lhs_dtype, m, n, k), 256), plane = align_up(m * n * 4, 256);
    if (!workspace || workspace_bytes < mm_ws + 2 * plane)
        return fail(QMM_ERR_WORKSPACE, "qmm_matmul_swiglu: workspace of %lld bytes required, %lld given", (long long)(mm_ws + 2 * plane),
                    (long long)workspace_bytes);
    if (!aligned(workspace, 256)) return fail(QMM_ERR_INVALID, "qmm_matmul_swiglu: workspace must be 256-byte aligned");
    float* g = (float*)((char*)workspace + mm_ws);
    float* u = (float*)((char*)workspace + mm_ws + plane);
    // (one launch for both products where a kernel takes matrices that share their lhs: Q4_K with 2..16 rows)
    const void* both[2] = {gate, up};
    const int64_t ns[2] = {n, n};
    float* outs[2] = {g, u};
    if (int rc = qmm_matmul_grouped(encoding, lhs, lhs_dtype, m, k, 2, both, ns, outs, workspace, mm_ws, stream)) return rc;
    return hip_status(qmm::launch_swiglu(g, u, out, m * n, (hipStream_t)stream), "qmm_matmul_swiglu(combine)");
}

int qmm_block_dots_q4_0(const void* lhs_q8_0, const void* rhs_q4_0, int64_t m, int64_t n, int64_t k, int32_t* out,
                        void* stream) {
    if (!lhs_q8_0 || !rhs_q4_0 || !out) return fail(QMM_ERR_INVALID, "qmm_block_dots_q4_0: null pointer");
    if (m <= 0 || n <= 0 || k <= 0 || k % 32) return fail(QMM_ERR_INVALID, "qmm_block_dots_q4_0: bad shape");
    return hip_status(qmm::launch_block_dots_q4_0((const uint8_t*)lhs_q8_0, (const uint8_t*)rhs_q4_0, m, n, k, out,
                                                  (hipStream_t)stream),
                      "qmm_block_dots_q4_0");
}

}  // extern "C"
