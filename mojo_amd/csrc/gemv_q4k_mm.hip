// Q4_K small-batch kernel (up to 16 lhs rows): weight rows streamed through LDS, 16 x 16 x 32
// matrix-core products over exact integer codes.
//
// Arithmetic is that of the prefill kernel (gemm_q4k.hip): a masked nibble is the fp16 subnormal
// q*2^-24, one packed fp16 multiply folds the 6-bit sub-block scale in (times 64), the lhs is narrowed to fp16
// (hi, plus a residual plane) after an exact power-of-two scaling, the fp32 super-block scale is
// applied in the lanes and the min term is one extra matrix product per super-block.
//
// Shape of the work: a workgroup of 8 wavefronts walks a list of up to 4 weight tiles of 16 rows.
// The super-blocks of a row are dealt to the wavefronts in groups of 16, two per wavefront; a
// wavefront's lhs fragments for its two super-blocks of a group are held in registers and reused
// for every tile of the workgroup.  The weights of a (group, tile) item, 288 contiguous bytes of
// each of the 16 rows, travel from global memory straight into a wavefront-private ring of three
// LDS slots (global_load_lds_dwordx4: no registers are held while they are in flight), two items
// ahead of the one being decoded; the wavefront waits with a vmcnt that leaves the younger items
// in flight.  Lane (row n = lane % 16, chunk c = lane / 16) decodes the 32 code bytes of chunk c of
// its row: sub-block 2c in the low nibbles, 2c + 1 in the high ones, so it needs only those two
// scales and mins; 8 code bytes feed two matrix-core instructions.  A wavefront accumulates its
// partial result of a tile over the groups in a private LDS slot; one barrier at the end, then the
// 8 partial results of a tile are added in a fixed order.
//
// Two ways to the lhs fragments:
//   m <= 8  the wavefront converts its own two super-blocks of every lhs row itself (scaled by a
//           power of two per lhs row and super-block, hi part in operand rows 0..7, residual in
//           rows 8..15, added at the end): one launch, no workspace;
//   m > 8   a separate pass (gemm_lhs.h) has written fp16 planes scaled per lhs row; fp32 lhs costs
//           a second matrix product per operand.
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "gemm_lhs.h"
#include "lds_stream.h"
#include "qmm_internal.h"

namespace qmm {

typedef float float4v __attribute__((ext_vector_type(4)));

namespace {

constexpr int kRunBlk = 2;                      // super-blocks per item
constexpr int kRowBytes = kRunBlk * Q4_K_BPB;   // 288: bytes of a row in an item (18 pieces of 16 bytes)
constexpr int kPieces = 16 * kRowBytes / 16;    // 288 pieces per item, piece p at LDS offset 16 p
constexpr int kLoads = (kPieces + 63) / 64;     // 5 load instructions per item, the last one by 32 lanes
constexpr int kSlotBytes = kPieces * 16;        // 4608
constexpr int kSlots = 3;                       // ring: one item being decoded, two in flight
constexpr float kTwo18f = 262144.0f;
constexpr int kWaves = 8;                       // wavefronts per workgroup
constexpr int kMaxTiles = 4;                    // tiles per workgroup (private LDS accumulators per wavefront)
constexpr int kPlaneStride = 528;               // staged lhs plane of one super-block: 512 bytes + 16 (bank spread)
constexpr int kStageBytes = 2 * kPlaneStride + 32;  // hi plane, residual plane, 8 sub-block sums (hi, lo)
constexpr int kRingBytes = kWaves * kSlots * kSlotBytes;
constexpr int kAccBytes = kWaves * kMaxTiles * 4 * 64 * 4;
constexpr int kLdsBytes = kRingBytes + kAccBytes;
static_assert(4 * kStageBytes + 16 <= kSlotBytes, "four staged lhs rows and their scales fit the free ring slot");
static_assert(8 * kStageBytes + 32 <= 2 * kSlotBytes, "both super-blocks of four staged lhs rows fit two free ring slots");

typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));  // what the packed conversion builtin returns

__device__ __forceinline__ half8 zero_half8() { return pack4(0u, 0u, 0u, 0u); }

}  // namespace

// NPART: matrix products per weight operand (2: hi and residual planes from the workspace).
// INLINE: lhs converted in the kernel (m <= 8, AT = float or bf16 bits); otherwise a16 / a16_lo / asum /
// inv come from prep_lhs_kernel<.., kLhsOrderQ4K16>.
// MROWS (INLINE): lhs rows converted, 1, 2, 4 or 8 (>= m; rows past m repeat the last one and their results are dropped).
// PLAIN: one matrix, known at compile time: no matrix lookup per item, a short argument block.
// KPART (with PLAIN): the workgroup takes group blockIdx.y of K only and stores its result as part blockIdx.y of
// [groups][m][n] at the output pointer (the caller adds the parts in group order): few tiles on a long K then make one
// workgroup per (share of the tiles, group), which converts its lhs operands once for several tiles.
template <int NPART, bool INLINE, int MROWS, typename AT, bool PLAIN, bool KPART = false>
__device__ __forceinline__ void mm_body(const MmMats& mats, const AT* __restrict__ a, const _Float16* __restrict__ a16,
                                        const _Float16* __restrict__ a16_lo, const _Float16* __restrict__ asum,
                                        const float* __restrict__ inv, int m, int k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk = k >> 8;
    const int64_t row_bytes = (int64_t)nblk * Q4_K_BPB;
    const int nn = lane & 15, kg = lane >> 4;
    uint8_t* ring = smem + wave * (kSlots * kSlotBytes);
    const uint32_t ring_lds = lds_address(ring);
    float* accs = (float*)(smem + kRingBytes);  // [kWaves][kMaxTiles][4][64]
    const int ntiles = mats.tile_end[kLanesMaxMats - 1];  // 16-row tiles, numbered through the matrices (entries past count repeat the last)
    // One matrix (the plain call) needs nothing from the argument block per item; with several, the tile's matrix is
    // looked up there (dependent scalar loads per item).
    const bool single = PLAIN || mats.count == 1;
    const uint8_t* const w_first = mats.w[0];
    float* const out_first = mats.out[0];
    const int n_first = mats.n[0];
    const int my_tiles = min(kMaxTiles, (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x);
    // group g is super-blocks [16 g, 16 g + 16): two per wavefront, or, when 8 or fewer are left, one
    const int ngrp_all = (nblk + kRunBlk * kWaves - 1) / (kRunBlk * kWaves);
    const int grp0 = KPART ? (int)blockIdx.y : 0;          // first group of this workgroup
    const int ngrp = KPART ? grp0 + 1 : ngrp_all;          // one past its last
    const int total = (ngrp - grp0) * my_tiles;
    auto group_share = [&](int g, int& first, int& cnt) {
        const int left = nblk - kRunBlk * kWaves * g;  // > 0
        const int per = left > kWaves ? kRunBlk : 1;
        first = kRunBlk * kWaves * g + per * wave;
        cnt = max(0, min(per, nblk - first));
        first = min(first, nblk - 1);  // (no share: a valid address, the data is not used)
    };

    int last_issued = -1;  // newest item whose loads into LDS have been issued
    int x_after = -1;      // the item that was newest when the last load_x was issued
    // INLINE: raw lhs values of the wavefront's two super-blocks of the next group to convert; lane holds
    // columns 4 lane .. 4 lane + 3 of each.  Loaded a group ahead; the first ones are the first loads of the kernel
    // (the conversion waits for them while the first weights are on their way).
    constexpr int RP = MROWS < 4 ? MROWS : 4;  // rows converted together (they share the free ring slot as staging)
    constexpr int NX = INLINE ? kRunBlk * MROWS : 0;  // load instructions of one load_x
    typedef typename std::conditional<sizeof(AT) == 4, u32x4, u32x2>::type xraw_t;
    xraw_t xr[kRunBlk][MROWS];
    auto load_x = [&](int g) {
        int b0, cnt;
        group_share(g, b0, cnt);
#pragma unroll
        for (int bb = 0; bb < kRunBlk; bb++) {
            const int blk = min(b0 + bb, nblk - 1);
#pragma unroll
            for (int mi = 0; mi < MROWS; mi++)
                hidden_load(xr[bb][mi], a + (int64_t)min(mi, m - 1) * k + (int64_t)blk * 256 + 4 * lane);
        }
        x_after = last_issued;
    };
    if constexpr (INLINE) {
        if (total > 0) load_x(grp0);
    }
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
        const int tile = (int)blockIdx.x + t * (int)gridDim.x;
        int n0 = tile * 16, n = n_first;
        const uint8_t* wj = w_first;
        if (!single) {
            int j = 0;
            while (j + 1 < mats.count && tile >= mats.tile_end[j]) j++;  // (uniform: a few scalar compares)
            n0 = (tile - (j ? mats.tile_end[j - 1] : 0)) * 16;
            n = mats.n[j];
            wj = mats.w[j];
        }
        int bc, cnt;
        group_share(g, bc, cnt);
        const int last_piece = max(cnt, 1) * 9 - 1;
        const uint8_t* base = wj + (int64_t)bc * Q4_K_BPB;
#pragma unroll
        for (int i = 0; i < kLoads; i++) {
            const uint8_t* src = base + (int64_t)min(n0 + prow[i], n - 1) * row_bytes + 16 * min(pidx[i], last_piece);
            if (i < kLoads - 1 || lane < kPieces - 64 * (kLoads - 1))  // the last instruction: 32 lanes
                load16_to_lds_once(src, ring_lds + slot * kSlotBytes + i * 1024);
        }
    };

    // items in flight: it + 1 and it + 2
    int ig = grp0, it_t = 0, islot = 0;  // next item to issue
    auto issue_next = [&]() {
        issue(ig, it_t, islot);
        last_issued++;
        islot = islot == kSlots - 1 ? 0 : islot + 1;
        if (++it_t == my_tiles) { it_t = 0; ig++; }
    };
    // One item before the first conversion, whose staging area is the other two slots (more loads in front of it only delay
    // the raw lhs values it waits for); the kernel that reads ready-made lhs planes fills its ring.
    if (total > 0) issue_next();
    if (!INLINE && total > 1) issue_next();

    // lhs operand row of this lane: INLINE: row nn % 8, hi plane for nn < 8, residual for nn >= 8
    const int mrow = min(INLINE ? (nn & 7) : nn, m - 1);
    const uint32_t M1 = 0x000F000Fu, M2 = 0x00F000F0u;
    const int sh = 16 * (kg & 1);  // byte pair (2c, 2c + 1) mod 4 inside a dword of the 6-bit fields
    const bool upper = kg >= 2;    // sub-blocks 4..7 use the split encoding

    half8 fa[kRunBlk][4][2][NPART], fs[kRunBlk];
    float bs[kRunBlk][4];  // INLINE: inverse lhs scale of (super-block, accumulator register's lhs row)
#pragma unroll
    for (int bb = 0; bb < kRunBlk; bb++) {
        fs[bb] = zero_half8();
#pragma unroll
        for (int r = 0; r < 4; r++) bs[bb][r] = 0.0f;
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int q = 0; q < NPART; q++) fa[bb][p][h][q] = zero_half8();
    }

    int grp = grp0, ti = 0, slot = 0;
    for (int it = 0; it < total; it++) {
        int gb0, nb;
        group_share(grp, gb0, nb);
        if (ti == 0) {
            // lhs fragments of the group's super-blocks: registers, reused for every tile.
            // Fragment (p, h) of chunk kg holds lhs columns 64 kg + 32 h + 8 p + (0,2,1,3,4,6,5,7).
            if constexpr (INLINE) {
                // The slot the next item will be loaded into is free: RP staged rows fit it.
                uint8_t* stg = ring + islot * kSlotBytes;
                const int rr = nn & 7;
                // the raw lhs values: everything issued after them may stay in flight
                wait_items<kLoads, 0>(last_issued - x_after, false);
#pragma unroll
                for (int bb = 0; bb < kRunBlk; bb++)
#pragma unroll
                    for (int mi = 0; mi < MROWS; mi++) tie(xr[bb][mi]);
                x_after = -2;  // none outstanding
#pragma unroll
                for (int ps = 0; ps < MROWS / RP; ps++) {
                    uint32_t hp[kRunBlk][RP][2], lp[kRunBlk][RP][2], sp[kRunBlk][RP];
                    float isc[kRunBlk][RP];
                    auto widen = [&](const xraw_t raw, float& x0, float& x1, float& x2, float& x3) {
                        if constexpr (sizeof(AT) == 4) {
                            x0 = __uint_as_float(raw.x); x1 = __uint_as_float(raw.y);
                            x2 = __uint_as_float(raw.z); x3 = __uint_as_float(raw.w);
                        } else {
                            x0 = __uint_as_float(raw.x << 16); x1 = __uint_as_float(raw.x & 0xffff0000u);
                            x2 = __uint_as_float(raw.y << 16); x3 = __uint_as_float(raw.y & 0xffff0000u);
                        }
                    };
                    // largest magnitude of every (super-block, row), lane-local
                    uint32_t mxs[kRunBlk * RP];
                    uint32_t lane_max = 0;
                    bool floor_ok = true;
#pragma unroll
                    for (int bb = 0; bb < kRunBlk; bb++)
#pragma unroll
                        for (int j = 0; j < RP; j++) {
                            float x0, x1, x2, x3;
                            widen(xr[bb][ps * RP + j], x0, x1, x2, x3);
                            const uint32_t mx = max_abs_bits(x0, x1, x2, x3);
                            mxs[bb * RP + j] = mx;
                            lane_max = max(lane_max, mx);
                            floor_ok = floor_ok & (__builtin_amdgcn_ballot_w64(mx >= 0x3C800000u) != 0);  // some value of it reaches 2^-6
                        }
                    // Every one of them between 2^-6 and 2^15 (activations of ordinary size): the values go to fp16 as they are,
                    // hi + residual carry 22 bits of each, and what is below fp16's normal range (2^-14) is small against the
                    // largest value of its row and super-block.  Otherwise a power of two per row and super-block brings the
                    // largest value to 2^9 first (maxima over the wavefront, all of them in one go).
                    const bool as_is = floor_ok && __builtin_amdgcn_ballot_w64(lane_max >= 0x47000000u) == 0;
                    if (!as_is) wave_umax_many(mxs);
#pragma unroll
                    for (int bb = 0; bb < kRunBlk; bb++) {
#pragma unroll
                        for (int j = 0; j < RP; j++) {
                            float x0, x1, x2, x3;
                            widen(xr[bb][ps * RP + j], x0, x1, x2, x3);
                            isc[bb][j] = 1.0f;
                            if (!as_is) {
                                const uint32_t mxb = mxs[bb * RP + j];
                                int e = (int)((mxb >> 23) & 0xffu) - 127;
                                if (e < -100 || e > 127) e = 9;  // zero, denormal or non-finite: leave unscaled
                                const float sc = __uint_as_float((uint32_t)(127 + 9 - e) << 23);
                                isc[bb][j] = __uint_as_float((uint32_t)(127 - 9 + e) << 23);
                                x0 *= sc; x1 *= sc; x2 *= sc; x3 *= sc;
                            }
                            // hi part: the value cut to fp16 (toward zero: one instruction converts and packs two);
                            // the residual x - hi is exact in fp32 and is cut to fp16 the same way
                            const fp16x2 c02 = __builtin_amdgcn_cvt_pkrtz(x0, x2), c13 = __builtin_amdgcn_cvt_pkrtz(x1, x3);
                            const fp16x2 r02 = __builtin_amdgcn_cvt_pkrtz(x0 - (float)c02.x, x2 - (float)c02.y);
                            const fp16x2 r13 = __builtin_amdgcn_cvt_pkrtz(x1 - (float)c13.x, x3 - (float)c13.y);
                            const float sum = sum8((x0 + x1) + (x2 + x3));  // 8 consecutive lanes = one 32-wide sub-block
                            const fp16x2 sm = __builtin_amdgcn_cvt_pkrtz(sum, 0.0f);
                            hp[bb][j][0] = __builtin_bit_cast(uint32_t, c02); hp[bb][j][1] = __builtin_bit_cast(uint32_t, c13);
                            lp[bb][j][0] = __builtin_bit_cast(uint32_t, r02); lp[bb][j][1] = __builtin_bit_cast(uint32_t, r13);
                            sp[bb][j] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(sum, sum - (float)sm.x));
                        }
                    }
                    // The converted values change lanes through LDS: a lane wrote four columns of every row, it reads the
                    // fragments of one row and plane.  unit u = staged (super-block, row) record.
                    auto put = [&](uint8_t* area, int u, int bb, int j, float* scales) __attribute__((always_inline)) {
                        uint8_t* st = area + u * kStageBytes;
                        *(uint2*)(st + 8 * lane) = make_uint2(hp[bb][j][0], hp[bb][j][1]);
                        *(uint2*)(st + kPlaneStride + 8 * lane) = make_uint2(lp[bb][j][0], lp[bb][j][1]);
                        if ((lane & 7) == 0) *(uint32_t*)(st + 2 * kPlaneStride + 4 * (lane >> 3)) = sp[bb][j];
                        if (lane == 0) scales[u] = isc[bb][j];
                    };
                    auto get = [&](const uint8_t* area, int u0, int bb, const float* scales) __attribute__((always_inline)) {
                        if (rr >= ps * RP && rr < ps * RP + RP) {
                            const uint8_t* st = area + (u0 + rr - ps * RP) * kStageBytes;
                            const uint8_t* pl = st + (nn >= 8 ? kPlaneStride : 0) + 128 * kg;
#pragma unroll
                            for (int p = 0; p < 4; p++) {
                                fa[bb][p][0][0] = *(const half8*)(pl + 16 * p);
                                fa[bb][p][1][0] = *(const half8*)(pl + 64 + 16 * p);
                            }
                            if (nn < 8) {
                                // min-term operand: (ah0, al0, ah0, ah1, al1, ah1, 0, 0) for sub-blocks 2 kg, 2 kg + 1
                                const uint2 s2 = *(const uint2*)(st + 2 * kPlaneStride + 8 * kg);
                                fs[bb] = pack4(s2.x, (s2.x & 0xffffu) | (s2.y << 16), (s2.y >> 16) | (s2.y << 16), 0u);
                            }
                        }
                        // inverse scales of the lhs rows of this lane's accumulator registers: rows (4 kg + r) % 8
                        // (with fewer than 4 staged rows every lane takes them: rows past m are dropped at the end)
                        if (RP < 4 || (kg & 1) == ps) {
#pragma unroll
                            for (int r = 0; r < RP; r++) bs[bb][r] = scales[u0 + r];
                        }
                    };
                    // First group: only item 0 is in flight (slot 0), slots 1 and 2 take both super-blocks at once.  Later
                    // groups have one free slot (the next item's): one super-block at a time.
                    const bool both = grp == grp0;
                    uint8_t* area = both ? ring + kSlotBytes : stg;
                    float* scales = (float*)(area + (both ? kRunBlk : 1) * RP * kStageBytes);
                    static_assert(kRunBlk == 2, "the staging below is written for two super-blocks");
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int j = 0; j < RP; j++) put(area, j, 0, j, scales);
                    if (both) {
#pragma unroll
                        for (int j = 0; j < RP; j++) put(area, RP + j, 1, j, scales);
                    }
                    __builtin_amdgcn_wave_barrier();
                    get(area, 0, 0, scales);
                    if (!both) {
                        __builtin_amdgcn_wave_barrier();
#pragma unroll
                        for (int j = 0; j < RP; j++) put(area, j, 1, j, scales);
                        __builtin_amdgcn_wave_barrier();
                    }
                    get(area, both ? RP : 0, 1, scales);
                }
                // the staged rows are in registers before the next item's load may overwrite the slot
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (grp + 1 < ngrp) load_x(grp + 1);
            } else {
#pragma unroll
                for (int bb = 0; bb < kRunBlk; bb++) {
                    const int blk = min(gb0 + bb, nblk - 1);
                    const _Float16* ah = a16 + (int64_t)mrow * k + (int64_t)blk * 256 + 64 * kg;
#pragma unroll
                    for (int p = 0; p < 4; p++) {
                        fa[bb][p][0][0] = *(const half8*)(ah + 8 * p);
                        fa[bb][p][1][0] = *(const half8*)(ah + 32 + 8 * p);
                    }
                    if constexpr (NPART == 2) {
                        const _Float16* al = a16_lo + (int64_t)mrow * k + (int64_t)blk * 256 + 64 * kg;
#pragma unroll
                        for (int p = 0; p < 4; p++) {
                            fa[bb][p][0][1] = *(const half8*)(al + 8 * p);
                            fa[bb][p][1][1] = *(const half8*)(al + 32 + 8 * p);
                        }
                    }
                    // asum: 8 hi parts then 8 lo parts per super-block
                    const uint16_t* as = (const uint16_t*)asum + ((int64_t)mrow * nblk + blk) * 16 + 2 * kg;
                    const uint32_t hi = *(const uint32_t*)as, lo = *(const uint32_t*)(as + 8);  // (ah0, ah1), (al0, al1)
                    fs[bb] = pack4((hi & 0xffffu) | (lo << 16), hi, (lo >> 16) | (hi & 0xffff0000u), 0u);
                }
            }
        }
        // the slot of item it - 1 is free: its reads fed matrix products whose results are already stored
        // (items in flight beyond the one in use: with up to four lhs rows one measures faster than two, 62.2 against 63.3 us for
        // the seven projections, as in the other small-batch kernels; with eight rows two do, 86.0 against 86.6)
        constexpr int kAhead = INLINE && MROWS <= 4 ? 1 : 2;
        while (last_issued < min(it + kAhead, total - 1)) issue_next();
        // item `it` has landed when only the younger loads are outstanding: later items and, if it was
        // issued after this item, the next group's raw lhs
        wait_items<kLoads, NX>(last_issued - it, INLINE && x_after >= it);
        const uint8_t* wbuf = ring + slot * kSlotBytes;

        float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int bb = 0; bb < kRunBlk; bb++) {
            if (bb >= nb) break;
            const uint8_t* lb = wbuf + nn * kRowBytes + bb * Q4_K_BPB;
            const uint4 hdr = *(const uint4*)lb;
            const uint4 q0 = *(const uint4*)(lb + 16 + 32 * kg), q1 = *(const uint4*)(lb + 32 + 32 * kg);
            // 6-bit scales and mins of sub-blocks 2 kg, 2 kg + 1
            const uint32_t p0 = (hdr.y >> sh) & 0xffffu, p1 = (hdr.z >> sh) & 0xffffu, p2 = (hdr.w >> sh) & 0xffffu;
            const uint32_t sc_pair = upper ? ((p2 & 0x0F0Fu) | ((p0 >> 2) & 0x3030u)) : (p0 & 0x3F3Fu);
            const uint32_t mn_pair = upper ? (((p2 >> 4) & 0x0F0Fu) | ((p1 >> 2) & 0x3030u)) : (p1 & 0x3F3Fu);
            // 64 * sc for the low nibbles (q * 2^-24), 4 * sc for the high ones (16 q * 2^-24): the operand is
            // sc * q * 2^-18, a normal fp16 number from sc * q = 16 on (as sc * q * 2^-24, always a subnormal, the
            // matrix core drops low bits of the products of small sc * q towards minus infinity: a bias growing with K)
            const float e0 = 64.0f * (float)(sc_pair & 0xffu), e1 = 4.0f * (float)(sc_pair >> 8);
            const uint32_t sp_lo = pack_half2(e0, e0), sp_hi = pack_half2(e1, e1);
            // min term: weight slots (bh0, bh0, bl0, bh1, bh1, bl1, 0, 0) of -(dmin * mn_j), hi and residual parts
            float4v Bk = {0.f, 0.f, 0.f, 0.f};
            {
                const uint32_t ndm = ((hdr.x >> 16) ^ 0x8000u) * 0x00010001u;  // (-dmin, -dmin)
                const uint32_t mp = pack_half2((float)(mn_pair & 0xffu), (float)(mn_pair >> 8));
                const uint32_t hi = pk_mul(ndm, mp);
                const uint32_t lo = pk_fma(ndm, mp, hi ^ 0x80008000u);
                const half8 bmin = pack4((hi & 0xffffu) * 0x00010001u, (lo & 0xffffu) | (hi & 0xffff0000u),
                                         (hi >> 16) | (lo & 0xffff0000u), 0u);
                Bk = __builtin_amdgcn_mfma_f32_16x16x32_f16(fs[bb], bmin, Bk, 0, 0, 0);
            }
            float4v P = {0.f, 0.f, 0.f, 0.f}, Q = {0.f, 0.f, 0.f, 0.f};  // two chains: low and high nibbles
            const uint32_t qd[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const uint32_t x0 = qd[2 * p], x1 = qd[2 * p + 1], y0 = x0 >> 8, y1 = x1 >> 8;
                const half8 blo = pack4(pk_mul(x0 & M1, sp_lo), pk_mul(y0 & M1, sp_lo), pk_mul(x1 & M1, sp_lo),
                                        pk_mul(y1 & M1, sp_lo));
                const half8 bhi = pack4(pk_mul(x0 & M2, sp_hi), pk_mul(y0 & M2, sp_hi), pk_mul(x1 & M2, sp_hi),
                                        pk_mul(y1 & M2, sp_hi));
                P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][p][0][0], blo, P, 0, 0, 0);
                Q = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][p][1][0], bhi, Q, 0, 0, 0);
                if constexpr (NPART == 2) {
                    P = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][p][0][1], blo, P, 0, 0, 0);
                    Q = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[bb][p][1][1], bhi, Q, 0, 0, 0);
                }
            }
            const float dsc = h2f((uint16_t)(hdr.x & 0xffffu)) * kTwo18f;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float v = fmaf(dsc, P[r] + Q[r], Bk[r]);
                acc[r] = INLINE ? fmaf(bs[bb][r], v, acc[r]) : acc[r] + v;  // INLINE: undo the lhs scale of this super-block
            }
        }
        // this wavefront's running sum of the tile over its groups
        float* mine = accs + ((wave * kMaxTiles + ti) * 4) * 64 + lane;
#pragma unroll
        for (int r = 0; r < 4; r++) mine[r * 64] = grp == grp0 ? acc[r] : mine[r * 64] + acc[r];

        slot = slot == kSlots - 1 ? 0 : slot + 1;
        if (++ti == my_tiles) { ti = 0; grp++; }
    }
    __syncthreads();
    // lane holds lhs rows 4 kg + r of weight row 16 tile + nn; (tile, r) pairs are dealt to the wavefronts
    for (int pr = wave; pr < my_tiles * 4; pr += kWaves) {
        const int t = pr >> 2, r = pr & 3;
        const int tile = (int)blockIdx.x + t * (int)gridDim.x;
        int n = n_first, tile0 = 0;
        float* out = KPART ? out_first + (int64_t)grp0 * m * n_first : out_first;
        if (!single) {
            int j = 0;
            while (j + 1 < mats.count && tile >= mats.tile_end[j]) j++;
            n = mats.n[j];
            out = mats.out[j];
            tile0 = j ? mats.tile_end[j - 1] : 0;
        }
        const int col = (tile - tile0) * 16 + nn, row = 4 * kg + r;
        float v = 0.0f;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) {
            const float* slot_r = accs + ((ww * kMaxTiles + t) * 4 + r) * 64;
            v += INLINE ? slot_r[lane & 31] + slot_r[(lane & 31) + 32] : slot_r[lane];
        }
        if (row < m && col < n) out[(int64_t)row * n + col] = INLINE ? v : v * inv[row];
    }
}

template <int NPART, bool INLINE, int MROWS, typename AT>
__global__ __launch_bounds__(512) void gemv_q4_k_mm_kernel(const MmMats mats, const AT* __restrict__ a,
                                                           const _Float16* __restrict__ a16,
                                                           const _Float16* __restrict__ a16_lo,
                                                           const _Float16* __restrict__ asum, const float* __restrict__ inv,
                                                           int m, int k) {
    mm_body<NPART, INLINE, MROWS, AT, false>(mats, a, a16, a16_lo, asum, inv, m, k);
}

// The plain call with up to 8 lhs rows: one matrix [n, k], lhs converted in the kernel.  Nine dwords of arguments.
template <int MROWS, typename AT, bool KPART = false>
__global__ __launch_bounds__(512) void gemv_q4_k_mm_plain_kernel(const uint8_t* __restrict__ w, const AT* __restrict__ a,
                                                                 float* __restrict__ out, int n, int m, int k) {
    asm volatile("" ::"s"(w), "s"(a), "s"(out), "s"(n), "s"(m), "s"(k));  // (all arguments in the first batch of scalar loads)
    MmMats mats;
#pragma unroll
    for (int j = 0; j < kLanesMaxMats; j++) {
        mats.w[j] = w;
        mats.out[j] = out;
        mats.n[j] = n;
        mats.tile_end[j] = (n + 15) >> 4;
    }
    mats.count = 1;
    mm_body<1, true, MROWS, AT, true, KPART>(mats, a, nullptr, nullptr, nullptr, nullptr, m, k);
}

namespace {
// Up to 8 lhs rows, few tiles, a K beyond 4096: the groups of K side by side in the grid (KPART).  Measured, 4096 x 14336 with
// 4 fp32 rows: one workgroup per tile that walks the 3.5 groups and converts the lhs for each 16.3 us.
struct KParts {
    int groups;       // 1: not wanted
    int64_t per, gx;  // tiles per workgroup, workgroups across the tiles
};
KParts k_parts(int lhs_dtype, int64_t m, int64_t n, int64_t k, int cus) {
    const int64_t ntiles = (n + 15) / 16, groups = (k / 256 + kRunBlk * kWaves - 1) / (kRunBlk * kWaves);
    const KParts none = {1, 0, 0};
    if (m < 2 || m > 8 || groups < 2 || ntiles > cus || kernel_disabled("q4k_mm_k_parts")) return none;
    const bool heavy = m > 4 && lhs_dtype == QMM_F32;  // eight fp32 rows: the conversion is two thirds of a workgroup's time
    // two groups: the launch that adds the parts costs what one conversion of up to four rows saves (4096 x 8192, 4 rows: 10.4
    // against 9.8 us; 8 fp32 rows 13.0 against 14.0)
    if (groups == 2 && !heavy) return none;
    // One workgroup per compute unit at most (a few more would run behind all the others), and nearly all of them in use:
    // 4096 x 14336 (64 x 4 workgroups of 4 tiles) 4 rows 16.3 -> 13.5 us, 2048 x 16384 16.7 -> 10.0; but 4096 x 11008
    // (64 x 3 of 4 tiles) 13.1 -> 14.3, with 8 fp32 rows 19.3 -> 16.7.
    const int64_t across = std::max<int64_t>(1, cus / groups), per = (ntiles + across - 1) / across;
    if (per > kMaxTiles) return none;
    const int64_t gx = (ntiles + per - 1) / per;
    if (gx * groups * 10 < (int64_t)cus * (heavy ? 7 : 9)) return none;
    return {(int)groups, per, gx};
}
}  // namespace

int64_t gemv_q4_k_mm_workspace_bytes(int lhs_dtype, int64_t m, int64_t k) {
    return m <= 8 ? 0 : lhs_planes(nullptr, lhs_dtype, m, k).bytes;
}

// The plain call (launch_gemv_q4_k_mm): with up to 8 rows, the parts of K of a matrix of few tiles (on a part of 256 compute
// units; the launch does not cut K on any other).
int64_t gemv_q4_k_mm_plain_workspace_bytes(int lhs_dtype, int64_t m, int64_t n, int64_t k) {
    if (m > 8) return gemv_q4_k_mm_workspace_bytes(lhs_dtype, m, k);
    const int groups = k_parts(lhs_dtype, m, n, k, 256).groups;
    return groups > 1 ? (int64_t)groups * m * n * 4 : 0;
}

// count matrices [ns[j], k] that share the lhs (count = 1: the plain call); out[j] is fp32 [m, ns[j]], dense.
// k_parts_ok: the workspace holds gemv_q4_k_mm_plain_workspace_bytes (the plain call only).
hipError_t launch_gemv_q4_k_mm_grouped(const void* lhs, int lhs_dtype, int count, const uint8_t* const* ws, const int64_t* ns,
                                       float* const* outs, int64_t m, int64_t k, void* workspace, hipStream_t s, bool k_parts_ok) {
    if (count < 1 || count > kLanesMaxMats) return hipErrorInvalidValue;
    MmMats mats;
    int64_t ntiles = 0;
    for (int j = 0; j < kLanesMaxMats; j++) {
        const int jj = j < count ? j : count - 1;
        if (j < count) ntiles += (ns[j] + 15) / 16;
        mats.w[j] = ws[jj];
        mats.out[j] = outs[jj];
        mats.n[j] = (int)ns[jj];
        mats.tile_end[j] = (int)ntiles;
    }
    mats.count = count;
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipGetLastError();
        cus = prop.multiProcessorCount;
    }
    hipError_t e = hipSuccess;
    static bool lds_set = false;
    if (!lds_set) {
        const void* pfns[8] = {(const void*)gemv_q4_k_mm_plain_kernel<1, float>, (const void*)gemv_q4_k_mm_plain_kernel<2, float>,
                               (const void*)gemv_q4_k_mm_plain_kernel<4, float>, (const void*)gemv_q4_k_mm_plain_kernel<8, float>,
                               (const void*)gemv_q4_k_mm_plain_kernel<1, uint16_t>, (const void*)gemv_q4_k_mm_plain_kernel<2, uint16_t>,
                               (const void*)gemv_q4_k_mm_plain_kernel<4, uint16_t>, (const void*)gemv_q4_k_mm_plain_kernel<8, uint16_t>};
        for (const void* fn : pfns) {
            e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
            if (e != hipSuccess) return e;
        }
        const void* kfns[6] = {(const void*)gemv_q4_k_mm_plain_kernel<2, float, true>, (const void*)gemv_q4_k_mm_plain_kernel<4, float, true>,
                               (const void*)gemv_q4_k_mm_plain_kernel<8, float, true>, (const void*)gemv_q4_k_mm_plain_kernel<2, uint16_t, true>,
                               (const void*)gemv_q4_k_mm_plain_kernel<4, uint16_t, true>, (const void*)gemv_q4_k_mm_plain_kernel<8, uint16_t, true>};
        for (const void* fn : kfns) {
            e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
            if (e != hipSuccess) return e;
        }
        const void* fns[10] = {(const void*)gemv_q4_k_mm_kernel<1, true, 1, float>, (const void*)gemv_q4_k_mm_kernel<1, true, 2, float>,
                               (const void*)gemv_q4_k_mm_kernel<1, true, 4, float>, (const void*)gemv_q4_k_mm_kernel<1, true, 8, float>,
                               (const void*)gemv_q4_k_mm_kernel<1, true, 1, uint16_t>, (const void*)gemv_q4_k_mm_kernel<1, true, 2, uint16_t>,
                               (const void*)gemv_q4_k_mm_kernel<1, true, 4, uint16_t>, (const void*)gemv_q4_k_mm_kernel<1, true, 8, uint16_t>,
                               (const void*)gemv_q4_k_mm_kernel<1, false, 1, float>, (const void*)gemv_q4_k_mm_kernel<2, false, 1, float>};
        for (const void* fn : fns) {
            e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
            if (e != hipSuccess) return e;
        }
        lds_set = true;
    }
    // every workgroup gets the same number of tiles (at most kMaxTiles), one workgroup per compute unit when that fits
    // (more tiles on fewer workgroups is slower at every size: 4096 x 14336, 4 rows: 18.1 / 23.8 / 36.0 us with 1 / 2 / 4 tiles)
    const int64_t per_wg = std::min<int64_t>(kMaxTiles, (ntiles + cus - 1) / cus);
    const int64_t wgs = (ntiles + per_wg - 1) / per_wg;
    dim3 grid((unsigned)wgs), block(64 * kWaves);
    if (m <= 8) {
        const bool plain = count == 1 && !kernel_disabled("q4k_mm_plain");
        // few tiles on a long K: a workgroup per (share of the tiles, group of K), the groups' results added by a launch of
        // their own in group order
        const KParts kp = plain && k_parts_ok && workspace && cus == 256 ? k_parts(lhs_dtype, m, ns[0], k, cus) : KParts{1, 0, 0};
        const int groups = kp.groups;
        if (groups > 1) {
            const dim3 kgrid((unsigned)kp.gx, (unsigned)groups);
            float* part = (float*)workspace;
#define QMM_MM_KPART(MR_)                                                                                             \
    do {                                                                                                              \
        if (lhs_dtype == QMM_F32)                                                                                     \
            gemv_q4_k_mm_plain_kernel<MR_, float, true><<<kgrid, block, kLdsBytes, s>>>(ws[0], (const float*)lhs, part, (int)ns[0], (int)m, (int)k); \
        else                                                                                                          \
            gemv_q4_k_mm_plain_kernel<MR_, uint16_t, true><<<kgrid, block, kLdsBytes, s>>>(ws[0], (const uint16_t*)lhs, part, (int)ns[0], (int)m, (int)k); \
    } while (0)
            if (m == 2) QMM_MM_KPART(2);
            else if (m <= 4) QMM_MM_KPART(4);
            else QMM_MM_KPART(8);
#undef QMM_MM_KPART
            e = hipGetLastError();
            return e != hipSuccess ? e : launch_sum_shares(part, outs[0], m * ns[0], groups, s);
        }
#define QMM_MM_INLINE(MR_)                                                                                            \
    do {                                                                                                              \
        if (plain && lhs_dtype == QMM_F32)                                                                            \
            gemv_q4_k_mm_plain_kernel<MR_, float><<<grid, block, kLdsBytes, s>>>(ws[0], (const float*)lhs, outs[0], (int)ns[0], (int)m, (int)k); \
        else if (plain)                                                                                               \
            gemv_q4_k_mm_plain_kernel<MR_, uint16_t><<<grid, block, kLdsBytes, s>>>(ws[0], (const uint16_t*)lhs, outs[0], (int)ns[0], (int)m, (int)k); \
        else if (lhs_dtype == QMM_F32)                                                                                \
            gemv_q4_k_mm_kernel<1, true, MR_, float><<<grid, block, kLdsBytes, s>>>(                                  \
                mats, (const float*)lhs, nullptr, nullptr, nullptr, nullptr, (int)m, (int)k);                         \
        else                                                                                                          \
            gemv_q4_k_mm_kernel<1, true, MR_, uint16_t><<<grid, block, kLdsBytes, s>>>(                               \
                mats, (const uint16_t*)lhs, nullptr, nullptr, nullptr, nullptr, (int)m, (int)k);                      \
    } while (0)
        if (m == 1) QMM_MM_INLINE(1);
        else if (m == 2) QMM_MM_INLINE(2);
        else if (m <= 4) QMM_MM_INLINE(4);
        else QMM_MM_INLINE(8);
#undef QMM_MM_INLINE
        return hipGetLastError();
    }
    const LhsPlanes p = lhs_planes(workspace, lhs_dtype, m, k);
    e = launch_prep_lhs<kLhsOrderQ4K16>(lhs, lhs_dtype, m, k, p, s);
    if (e != hipSuccess) return e;
    if (!p.a16_lo)
        gemv_q4_k_mm_kernel<1, false, 1, float><<<grid, block, kLdsBytes, s>>>(mats, nullptr, p.a16, nullptr, p.asum, p.inv, (int)m, (int)k);
    else
        gemv_q4_k_mm_kernel<2, false, 1, float><<<grid, block, kLdsBytes, s>>>(mats, nullptr, p.a16, p.a16_lo, p.asum, p.inv, (int)m, (int)k);
    return hipGetLastError();
}

hipError_t launch_gemv_q4_k_mm(const void* lhs, int lhs_dtype, const uint8_t* w, int64_t m, int64_t n, int64_t k,
                               float* out, void* workspace, hipStream_t s) {
    return launch_gemv_q4_k_mm_grouped(lhs, lhs_dtype, 1, &w, &n, &out, m, k, workspace, s, true);
}

}  // namespace qmm
