// Pieces shared by the MFMA expert-FFN kernels (bf16: ffn_mfma.hip, fp8: ffn_fp8.hip): the 256 x 256 output tile,
// the two 64 KB LDS stages of 128-byte operand rows, the enumeration of tiles over variable-length expert segments
// with the XCD-aware block order, the LDS swizzle and the direct-to-LDS load.
#pragma once
#include "ffn.h"

namespace {

constexpr int BM = 256, BN = 256;
constexpr int kTileBytes = 256 * 128;  // one operand tile: 256 rows (K-major) or 64 k rows of 512 B (X-major), 32 KB
constexpr int kStageBytes = 2 * kTileBytes;
constexpr int kNumXcd = 8;

// K-major tiles: 16-byte chunk swizzle of tile row `row`.  A ds_read_b128 serves 16 lanes (16 consecutive rows, one
// chunk each) per cycle; rows are 128 B, half the 256 B bank span, so rows 2i and 2i+1 cover all banks between them
// and (row >> 1) & 7 puts the 8 row pairs on 8 different chunks: no bank conflicts (measured: 4 cycles per read).
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

__device__ __forceinline__ void load16_to_lds(const void* g, char* l) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)l, 16, 0, 0);
}


struct TileCoord {
    int e, n_tile, m_tile, rows;  // rows: valid M rows (M-grouped) or valid K rows (wgrad)
    int64_t row0;                 // first row of the tile (M-grouped) or of the expert segment (wgrad)
    // L2 prefetch shares: of the tiles one XCD runs at a time, a_sn share this tile's A slices and b_sn its B slices;
    // this tile touches lines a_si, a_si + a_sn, ... of an A slice and b_si, b_si + b_sn, ... of a B slice
    int a_si, a_sn, b_si, b_sn;
};


// M-grouped tiles come in two classes.  Heavy: full 256-row tiles and tails of more than 128 rows.  Light: tails
// of at most 128 rows, which cost about half (the wavefronts owning rows 128..255 skip their MFMAs).  Every XCD
// gets a contiguous run of the heavy tiles followed by a run of the light ones, so the light tiles fill the last,
// partly occupied round of blocks instead of a full-cost tile being left over there.
__device__ __forceinline__ bool locate_m_grouped(const int64_t* counts, int E, int n_tiles, TileCoord* tc) {
    int64_t heavy_m = 0, light_m = 0;
    for (int e = 0; e < E; ++e) {
        const int64_t c = counts[e], rem = c % BM;
        heavy_m += c / BM + (rem > BM / 2);
        light_m += (rem > 0 && rem <= BM / 2);
    }
    const int64_t heavy = heavy_m * n_tiles, light = light_m * n_tiles;
    const int64_t heavy_per_xcd = (heavy + kNumXcd - 1) / kNumXcd, light_per_xcd = (light + kNumXcd - 1) / kNumXcd;
    const int64_t xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    bool want_light;
    int64_t L;
    if (slot < heavy_per_xcd) {
        want_light = false;
        L = xcd * heavy_per_xcd + slot;
        if (L >= heavy) return false;
    } else if (slot - heavy_per_xcd < light_per_xcd) {
        want_light = true;
        L = xcd * light_per_xcd + (slot - heavy_per_xcd);
        if (L >= light) return false;
    } else {
        return false;
    }
    int64_t start = 0;
    for (int e = 0; e < E; ++e) {
        const int64_t c = counts[e], full = c / BM, rem = c % BM;
        const bool light_tail = rem > 0 && rem <= BM / 2;
        const int64_t me = want_light ? (int64_t)light_tail : full + (rem > BM / 2);
        const int64_t te = me * n_tiles;
        if (L < te) {
            const int m = want_light ? (int)full : (int)(L % me);
            tc->e = e;
            tc->m_tile = m;
            tc->n_tile = (int)(L / me);
            tc->row0 = start + (int64_t)m * BM;
            const int64_t left = c - (int64_t)m * BM;
            tc->rows = left < BM ? (int)left : BM;
            tc->a_sn = n_tiles < 4 ? n_tiles : 4;
            tc->a_si = tc->n_tile % tc->a_sn;
            tc->b_sn = me < 8 ? (int)me : 8;
            tc->b_si = m % tc->b_sn;
            return true;
        }
        L -= te;
        start += c;
    }
    return false;
}


inline unsigned round_up_xcd(int64_t g) { return (unsigned)(((g + kNumXcd - 1) / kNumXcd) * kNumXcd); }
// upper bound of 8 * (ceil(heavy / 8) + ceil(light / 8)) over every split of the rows among the experts
inline unsigned grid_m_grouped(const FfnShape& s, int n_tiles) {
    return round_up_xcd((s.n_rows / BM + s.E) * (int64_t)n_tiles) + 2 * kNumXcd;
}


}  // namespace
