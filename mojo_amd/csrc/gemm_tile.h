// Pieces shared by the prefill kernels that work on 256 x 128 (or 256 x 256) output tiles with one persistent workgroup per compute
// unit: the tile order inside an XCD, and the work units that balance a last, partly filled round of tiles.
#pragma once
#include <hip/hip_runtime.h>

namespace qmm {

constexpr int kTileGm = 8;  // lhs tile rows that stay fixed while the tile order of an XCD walks N

__device__ __host__ inline void tile_order(int o, int tiles_m, int tiles_n, int gm, int& tile_m, int& tile_n) {
    const int span = gm * tiles_n;
    const int grp = o / span, rem = o - grp * span;
    const int rows_here = gm < tiles_m - grp * gm ? gm : tiles_m - grp * gm;
    tile_n = rem / rows_here;
    tile_m = grp * gm + rem - tile_n * rows_here;
}

// Work units of one XCD.  The tiles are dealt to the 8 XCDs in contiguous ranges (workgroup ids congruent mod 8 share an
// XCD and its L2); inside a range the W persistent workgroups of the XCD take units u = slot, slot + W, ...  When the
// range is not a multiple of W, the last round would keep only `rem` of the W compute units busy for a whole tile; if
// rem <= W / 2, each of those last tiles is cut into two halves of K that go to different workgroups and are added in
// `out` with atomic adds (onto zeros written beforehand: exactly two terms per element, so the sum does not depend on
// their order).  That round then takes half a tile's time.
struct TileUnit {
    int tile;   // global tile index
    int kb0;    // first super-block
    int nb;     // super-blocks
    int half;   // 0: whole K, plain stores; 1: one of two halves, atomic adds
};
__device__ __host__ inline int xcd_units(int n_x, int wgs_per_xcd, int nblk, int allow_split, int& full) {
    const int rem = n_x % wgs_per_xcd;
    const bool split = allow_split && rem > 0 && 2 * rem <= wgs_per_xcd && nblk >= 2;
    full = split ? n_x - rem : n_x;
    return full + 2 * (n_x - full);
}
__device__ __host__ inline TileUnit xcd_unit(int u, int base, int full, int nblk) {
    TileUnit t;
    if (u < full) {
        t.tile = base + u; t.kb0 = 0; t.nb = nblk; t.half = 0;
    } else {
        const int j = u - full;
        t.tile = base + full + (j >> 1);
        t.kb0 = (j & 1) ? nblk / 2 : 0;
        t.nb = (j & 1) ? nblk - nblk / 2 : nblk / 2;
        t.half = 1;
    }
    return t;
}

// Zeroing of the output tiles that a tile kernel cuts in two along K and fills with atomic adds (same unit arithmetic as
// the kernel: `k_blocks` super-blocks a tile, `wgs_per_xcd` persistent workgroups per XCD).  One workgroup of 256 threads
// takes the eighth `part` of the rows of the j-th split tile of XCD x; a thread zeroes four columns of four rows.
struct SplitTiles {
    float* out;
    int m, n, tiles_m, tiles_n, k_blocks, wgs_per_xcd;
    int max_split;  // largest number of split tiles on any XCD: the zeroing takes max_split * 64 workgroups
    int tn;         // columns of a tile: 128 or 256
    float* part;    // not null: no tiles are split in halves; the whole of `out` and of this second m x n buffer is zeroed instead
};
constexpr int kZeroFlatFloats = 8192;  // per workgroup of 256 threads
__device__ __forceinline__ void zero_flat(float* a, float* b, int64_t count, int e) {
    const int64_t i0 = (int64_t)e * kZeroFlatFloats + threadIdx.x;
    for (int j = 0; j < kZeroFlatFloats / 256; j++) {
        const int64_t i = i0 + j * 256;
        if (i < count) {
            a[i] = 0.0f;
            b[i] = 0.0f;
        }
    }
}
__device__ __forceinline__ void zero_split_tile_part(const SplitTiles& z, int j, int x, int part) {
    constexpr int TM = 256;
    const int TN = z.tn;
    const int total = z.tiles_m * z.tiles_n, per_xcd = (total + 7) / 8;
    const int xcd_base = x * per_xcd, n_x = max(0, min(per_xcd, total - xcd_base));
    int full;
    xcd_units(n_x, z.wgs_per_xcd, z.k_blocks, 1, full);
    if (full + j >= n_x) return;
    int tile_m, tile_n;
    tile_order(xcd_base + full + j, z.tiles_m, z.tiles_n, kTileGm, tile_m, tile_n);
    const int m0 = tile_m * TM + part * (TM / 8), n0 = tile_n * TN;
    const int per_row = TN / 4;  // threads that cover a row of the tile: 32 or 64
    const int col = n0 + ((int)threadIdx.x & (per_row - 1)) * 4;
    const bool wide = (z.n & 3) == 0;  // rows start on 16-byte boundaries
    for (int r = (int)threadIdx.x / per_row; r < TM / 8; r += 256 / per_row) {
        const int row = m0 + r;
        if (row >= z.m) break;
        float* o = z.out + (int64_t)row * z.n + col;
        if (wide && col + 3 < z.n) {
            *(float4*)o = make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            for (int q = 0; q < 4; q++)
                if (col + q < z.n) o[q] = 0.0f;
        }
    }
}
// The split tiles of a launch with `wg` persistent workgroups (host side).
inline SplitTiles split_tiles(float* out, int64_t m, int64_t n, int tiles_m, int tiles_n, int k_blocks, int wg, int tn = 128) {
    SplitTiles z{out, (int)m, (int)n, tiles_m, tiles_n, k_blocks, wg / 8, 0, tn, nullptr};
    const int total = tiles_m * tiles_n, per_xcd = (total + 7) / 8;
    for (int x = 0; x < 8; x++) {
        const int n_x = per_xcd < total - x * per_xcd ? per_xcd : (total - x * per_xcd > 0 ? total - x * per_xcd : 0);
        int full;
        xcd_units(n_x, z.wgs_per_xcd, k_blocks, 1, full);
        if (n_x - full > z.max_split) z.max_split = n_x - full;
    }
    return z;
}

}  // namespace qmm
