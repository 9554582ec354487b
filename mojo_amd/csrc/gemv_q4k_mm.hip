// Q4_K small-batch kernel (3 <= m <= 16 lhs rows): weight rows streamed through LDS, 16 x 16 x 32
// matrix-core products over exact integer codes.
//
// Arithmetic is that of the prefill kernel (gemm_q4k.hip): a masked nibble is the fp16 subnormal
// q*2^-24, one packed fp16 multiply folds the 6-bit sub-block scale in, the lhs is narrowed to fp16
// (hi, plus a residual plane for fp32 input) after an exact per-row power-of-two scaling, the fp32
// super-block scale is applied in the lanes and the min term is one extra matrix product per
// super-block (K = 32 slots hold  asum_hi x dmn_hi,  asum_lo x dmn_hi,  asum_hi x dmn_lo).
//
// Shape of the work: a workgroup of 8 wavefronts walks a list of up to 4 weight tiles of 16 rows.
// Wavefront w owns the super-blocks [w nblk / 8, (w + 1) nblk / 8) of every row and goes through
// them two at a time ("groups"); its lhs fragments for the two super-blocks of a group (16 lhs rows,
// hi and residual planes) are loaded into registers once per group and reused for every tile of the
// workgroup (loading them per tile made the lhs planes, not the weights, the bulk of the traffic).
// The weights of a (group, tile) item, 288 contiguous bytes of each of the 16 rows, travel from
// global memory straight into a wavefront-private ring of three LDS slots (global_load_lds_dwordx4:
// no registers are held while they are in flight), two items ahead of the one being decoded; the
// wavefront waits with a vmcnt that leaves the younger items in flight.  Each lane (row n =
// lane % 16, k-group lane / 16) reads its 8 code bytes of a 64-wide chunk with one ds_read_b64 and
// they serve two matrix-core instructions, the low nibbles (sub-block 2c) and the high nibbles
// (sub-block 2c + 1).  A wavefront accumulates its partial result of a tile over the groups in a
// private LDS slot; one barrier at the end, then the 8 partial results of a tile are added in a
// fixed order.
#include <stdlib.h>

#include <algorithm>

#include "gemm_lhs.h"
#include "qmm_internal.h"

namespace qmm {

typedef float float4v __attribute__((ext_vector_type(4)));

namespace {

constexpr int kRunBlk = 2;                      // super-blocks per item
constexpr int kRowBytes = kRunBlk * Q4_K_BPB;   // 288: bytes of a row in an item (18 pieces of 16 bytes)
constexpr int kPieces = 16 * kRowBytes / 16;    // 288 pieces per item, piece p at LDS offset 16 p
constexpr int kLoads = (kPieces + 63) / 64;     // 5 load instructions per item
constexpr int kSlotBytes = kLoads * 1024;       // 5120: the last instruction's upper lanes land in the slot's unused tail
constexpr int kSlots = 3;                       // ring: one item being decoded, two in flight
constexpr float kTwo24f = 16777216.0f;
constexpr int kWaves = 8;                       // wavefronts per workgroup
constexpr int kMaxTiles = 4;                    // tiles per workgroup (private LDS accumulators per wavefront)
constexpr int kRingBytes = kWaves * kSlots * kSlotBytes;
constexpr int kLdsBytes = kRingBytes + kWaves * kMaxTiles * 4 * 64 * 4;

typedef __attribute__((address_space(3))) void* lds_space_ptr;

// 16 bytes per lane from global memory to LDS at lds_base + 16 * lane (lds_base uniform).  The
// compiler is not told that this is a load: it keeps no count of it, and the caller waits with
// wait_vmcnt before reading the slot.  (The builtin for this instruction makes the compiler wait
// for all of them before every LDS read, which would leave nothing in flight.)  m0 is put back.
__device__ __forceinline__ void load16_to_lds(const void* g, uint32_t lds_base) {
    uint32_t keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(g), "s"(lds_base)
                 : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

}  // namespace

// NPART: matrix products per weight operand (2: hi and residual lhs planes).  STACK (with NPART 1, m <= 8):
// the residual plane of lhs row r rides in operand row r + 8 and the two results are added at the end.
template <int NPART, bool STACK>
__global__ __launch_bounds__(512) void gemv_q4_k_mm_kernel(const uint8_t* __restrict__ w, const _Float16* __restrict__ a16,
                                                           const _Float16* __restrict__ a16_lo,
                                                           const _Float16* __restrict__ asum, const float* __restrict__ inv,
                                                           float* __restrict__ out, int m, int n, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int nn = lane & 15, kg = lane >> 4;
    uint8_t* ring = smem + wave * (kSlots * kSlotBytes);
    const uint32_t ring_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_space_ptr)ring);
    float* accs = (float*)(smem + kRingBytes);  // [kWaves][kMaxTiles][4][64]
    const int ntiles = (n + 15) >> 4;
    const int my_tiles = min(kMaxTiles, (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x);
    // group g is super-blocks [16 g, 16 g + 16): two per wavefront, or, when 8 or fewer are left, one
    const int ngrp = (nblk + kRunBlk * kWaves - 1) / (kRunBlk * kWaves);
    const int total = ngrp * my_tiles;
    auto group_share = [&](int g, int& first, int& cnt) {
        const int left = nblk - kRunBlk * kWaves * g;  // > 0
        const int per = left > kWaves ? kRunBlk : 1;
        first = kRunBlk * kWaves * g + per * wave;
        cnt = max(0, min(per, nblk - first));
        first = min(first, nblk - 1);  // (no share: a valid address, the data is not used)
    };

    // piece p = lane + 64 i of an item: row p / 18, 16-byte piece p % 18
    int prow[kLoads], pidx[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
        const int p = min(lane + 64 * i, kPieces - 1);
        prow[i] = p / 18;
        pidx[i] = p - prow[i] * 18;
    }
    // item (group g, tile index t) -> ring slot `slot`
    auto issue = [&](int g, int t, int slot) {
        const int n0 = ((int)blockIdx.x + t * (int)gridDim.x) * 16;
        int bc, cnt;
        group_share(g, bc, cnt);
        const int last_piece = max(cnt, 1) * 9 - 1;
        const uint8_t* base = w + (int64_t)bc * Q4_K_BPB;
#pragma unroll
        for (int i = 0; i < kLoads; i++)
            load16_to_lds(base + (int64_t)min(n0 + prow[i], n - 1) * row_bytes + 16 * min(pidx[i], last_piece),
                          ring_lds + slot * kSlotBytes + i * 1024);
    };

    // lhs row whose fragments this lane holds (rows >= m repeat the last one)
    const int mrow = min(STACK ? (nn & 7) : nn, m - 1);
    const _Float16* a_hi = (STACK && nn >= 8 ? a16_lo : a16) + (int64_t)mrow * k + 8 * kg;
    const _Float16* a_lo = NPART == 2 ? a16_lo + (int64_t)mrow * k + 8 * kg : nullptr;
    const _Float16* as_row = asum + (int64_t)mrow * nblk * 16 + (kg & 1) * 8;
    const uint32_t M1 = 0x000F000Fu, M2 = 0x00F000F0u;

    // items in flight: it + 1 and it + 2
    int ig = 0, it_t = 0, islot = 0;  // next item to issue
    auto issue_next = [&]() {
        issue(ig, it_t, islot);
        islot = islot == kSlots - 1 ? 0 : islot + 1;
        if (++it_t == my_tiles) { it_t = 0; ig++; }
    };
    if (total > 0) issue_next();
    if (total > 1) issue_next();

    half8 fa[kRunBlk][8][NPART], fs[kRunBlk];
    int grp = 0, ti = 0, slot = 0;
    for (int it = 0; it < total; it++) {
        int gb0, nb;
        group_share(grp, gb0, nb);
        if (ti == 0) {
            // lhs fragments and sub-block sums of the group's super-blocks: registers, reused for every tile
#pragma unroll
            for (int bb = 0; bb < kRunBlk; bb++) {
                const int blk = min(gb0 + bb, nblk - 1);
                fs[bb] = *(const half8*)(as_row + (int64_t)blk * 16);
                if (STACK && nn >= 8) fs[bb] = half8{0, 0, 0, 0, 0, 0, 0, 0};  // the min term belongs to the hi rows
#pragma unroll
                for (int sl = 0; sl < 8; sl++) {
                    fa[bb][sl][0] = *(const half8*)(a_hi + (int64_t)blk * 256 + 32 * sl);
                    if constexpr (NPART == 2) fa[bb][sl][1] = *(const half8*)(a_lo + (int64_t)blk * 256 + 32 * sl);
                }
            }
        }
        // the slot of item it - 1 is free: its reads fed matrix products whose results are already stored
        if (it + 2 < total) {
            issue_next();
            wait_vmcnt<2 * kLoads>();
        } else if (it + 1 < total) {
            wait_vmcnt<kLoads>();
        } else {
            wait_vmcnt<0>();
        }
        const uint8_t* wbuf = ring + slot * kSlotBytes;

        float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int bb = 0; bb < kRunBlk; bb++) {
            if (bb >= nb) break;
            const uint8_t* lb = wbuf + nn * kRowBytes + bb * Q4_K_BPB;
            const uint4 hdr = *(const uint4*)lb;
            // 6-bit scales and mins of the 8 sub-blocks
            const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
            const uint32_t sc_lo = s0 & 0x3F3F3F3Fu, sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
            const uint32_t mn_lo = s1 & 0x3F3F3F3Fu, mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
            uint32_t sp[8];
            {
                const float e0 = (float)(sc_lo & 0xffu), e1 = 0.0625f * (float)((sc_lo >> 8) & 0xffu);
                const float e2 = (float)((sc_lo >> 16) & 0xffu), e3 = 0.0625f * (float)(sc_lo >> 24);
                const float e4 = (float)(sc_hi & 0xffu), e5 = 0.0625f * (float)((sc_hi >> 8) & 0xffu);
                const float e6 = (float)((sc_hi >> 16) & 0xffu), e7 = 0.0625f * (float)(sc_hi >> 24);
                sp[0] = pack_half2(e0, e0); sp[1] = pack_half2(e1, e1);
                sp[2] = pack_half2(e2, e2); sp[3] = pack_half2(e3, e3);
                sp[4] = pack_half2(e4, e4); sp[5] = pack_half2(e5, e5);
                sp[6] = pack_half2(e6, e6); sp[7] = pack_half2(e7, e7);
            }
            // min term: B slots (k-group 0,1: hi parts, 2: lo parts) of -(dmin*mn_j), A slots asum hi / lo
            {
                const uint32_t ndm = ((hdr.x >> 16) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
                const uint32_t mp[4] = {pack_half2((float)(mn_lo & 0xffu), (float)((mn_lo >> 8) & 0xffu)),
                                        pack_half2((float)((mn_lo >> 16) & 0xffu), (float)(mn_lo >> 24)),
                                        pack_half2((float)(mn_hi & 0xffu), (float)((mn_hi >> 8) & 0xffu)),
                                        pack_half2((float)((mn_hi >> 16) & 0xffu), (float)(mn_hi >> 24))};
                uint32_t v[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t hi = pk_mul(ndm, mp[i]);
                    const uint32_t lo = pk_fma(ndm, mp[i], hi ^ 0x80008000u);
                    v[i] = kg < 2 ? hi : (kg == 2 ? lo : 0u);  // slots 24..31 (asum_lo x dmn_lo) are dropped
                }
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(fs[bb], pack4(v[0], v[1], v[2], v[3]), acc, 0, 0, 0);
            }
            float4v P = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint2 q = *(const uint2*)(lb + 16 + 32 * c + 8 * kg);
                const uint32_t x0 = q.x, x1 = q.y, y0 = q.x >> 8, y1 = q.y >> 8;
                const half8 blo = pack4(pk_mul(x0 & M1, sp[2 * c]), pk_mul(y0 & M1, sp[2 * c]),
                                        pk_mul(x1 & M1, sp[2 * c]), pk_mul(y1 & M1, sp[2 * c]));
                const half8 bhi = pack4(pk_mul(x0 & M2, sp[2 * c + 1]), pk_mul(y0 & M2, sp[2 * c + 1]),
                                        pk_mul(x1 & M2, sp[2 * c + 1]), pk_mul(y1 & M2, sp[2 * c + 1]));
                P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c][0], blo, P, 0, 0, 0);
                P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c + 1][0], bhi, P, 0, 0, 0);
                if constexpr (NPART == 2) {
                    P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c][1], blo, P, 0, 0, 0);
                    P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][2 * c + 1][1], bhi, P, 0, 0, 0);
                }
            }
            const float dsc = h2f((uint16_t)(hdr.x & 0xffffu)) * kTwo24f;
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] = fmaf(dsc, P[r], acc[r]);
        }
        // this wavefront's running sum of the tile over its groups
        float* mine = accs + ((wave * kMaxTiles + ti) * 4) * 64 + lane;
#pragma unroll
        for (int r = 0; r < 4; r++) mine[r * 64] = grp == 0 ? acc[r] : mine[r * 64] + acc[r];

        slot = slot == kSlots - 1 ? 0 : slot + 1;
        if (++ti == my_tiles) { ti = 0; grp++; }
    }
    __syncthreads();
    // lane holds lhs rows 4 kg + r of weight row 16 tile + nn; (tile, r) pairs are dealt to the wavefronts
    for (int pr = wave; pr < my_tiles * 4; pr += kWaves) {
        const int t = pr >> 2, r = pr & 3;
        const int col = ((int)blockIdx.x + t * (int)gridDim.x) * 16 + nn, row = 4 * kg + r;
        float v = 0.0f;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) {
            const float* slot_r = accs + ((ww * kMaxTiles + t) * 4 + r) * 64;
            v += STACK ? slot_r[lane & 31] + slot_r[(lane & 31) + 32] : slot_r[lane];
        }
        if (row < m && col < n) out[(int64_t)row * n + col] = v * inv[row];
    }
}

int64_t gemv_q4_k_mm_workspace_bytes(int lhs_dtype, int64_t m, int64_t k) { return lhs_planes(nullptr, lhs_dtype, m, k).bytes; }

hipError_t launch_gemv_q4_k_mm(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                               float* out, void* workspace, hipStream_t s) {
    const LhsPlanes p = lhs_planes(workspace, lhs_dtype, m, k);
    hipError_t e = launch_prep_lhs<kLhsOrderQ4K16>(lhs, lhs_dtype, m, k, p, s);
    if (e != hipSuccess) return e;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    const int64_t ntiles = (n + 15) / 16;
    // every workgroup gets the same number of tiles (at most kMaxTiles), one workgroup per compute unit when that fits
    const int64_t per_wg = std::min<int64_t>(kMaxTiles, (ntiles + cus - 1) / cus);
    const int64_t wgs = (ntiles + per_wg - 1) / per_wg;
    static bool lds_set = false;
    if (!lds_set) {
        const void* fns[3] = {(const void*)gemv_q4_k_mm_kernel<1, false>, (const void*)gemv_q4_k_mm_kernel<1, true>,
                              (const void*)gemv_q4_k_mm_kernel<2, false>};
        for (const void* fn : fns) {
            e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
            if (e != hipSuccess) return e;
        }
        lds_set = true;
    }
    dim3 grid((unsigned)wgs), block(64 * kWaves);
    if (!p.a16_lo)
        gemv_q4_k_mm_kernel<1, false><<<grid, block, kLdsBytes, s>>>(w, p.a16, nullptr, p.asum, p.inv, out, (int)m, (int)n, (int)k);
    else if (m <= 8)
        gemv_q4_k_mm_kernel<1, true><<<grid, block, kLdsBytes, s>>>(w, p.a16, p.a16_lo, p.asum, p.inv, out, (int)m, (int)n, (int)k);
    else
        gemv_q4_k_mm_kernel<2, false><<<grid, block, kLdsBytes, s>>>(w, p.a16, p.a16_lo, p.asum, p.inv, out, (int)m, (int)n, (int)k);
    return hipGetLastError();
}

}  // namespace qmm
