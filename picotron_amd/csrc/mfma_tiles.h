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

// A 16-byte direct-to-LDS load as an instruction sequence the compiler does not look into: wave-uniform base pointer plus
// a 32-bit byte offset per lane, LDS destination (wave-uniform, lane l lands at +16*l) through M0.  Why: the compiler's
// wait-count pass knows a builtin direct-to-LDS load is in flight and puts "s_waitcnt vmcnt(0)" in front of every later
// LDS read it cannot prove disjoint from the destination -- it does so for the transpose reads
// (__builtin_amdgcn_ds_read_tr16_b64), which then wait for loads issued a moment ago.  A kernel that uses this form
// orders its LDS reads after the loads itself (explicit s_waitcnt vmcnt + barrier).  M0 is written here and is not in the
// clobber list (the compiler rejects it as reserved): nothing else in a kernel that uses this form may depend on M0 --
// no builtin direct-to-LDS load, no s_sendmsg, no GWS.
__device__ __forceinline__ void load16_to_lds_opaque(const char* base, uint32_t lane_offset, char* l) {
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)l;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr), "v"(lane_offset), "s"(base) : "memory");
}


__device__ __forceinline__ int uniform_i32(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

struct TileCoord {
    int e, n_tile, m_tile, rows;  // rows: valid M rows (M-grouped) or valid K rows (wgrad)
    int64_t row0;                 // first row of the tile (M-grouped) or of the expert segment (wgrad)
    // L2 prefetch shares: of the tiles one XCD runs at a time, a_sn share this tile's A slices and b_sn its B slices;
    // this tile touches lines a_si, a_si + a_sn, ... of an A slice and b_si, b_si + b_sn, ... of a B slice
    int a_si, a_sn, b_si, b_sn;
    // split last round (M-grouped kernels that are given a workspace): this block computes k range `piece` of `pieces`
    // and leaves its fp32 partial tile in workspace slot ws_slot
    int piece, pieces, ws_slot;
};


// M-grouped tiles come in two classes.  Heavy: full 256-row tiles and tails of more than 128 rows.  Light: tails
// of at most 128 rows, which cost about half (the wavefronts owning rows 128..255 skip their MFMAs).  Every XCD
// gets a contiguous run of the heavy tiles followed by a run of the light ones, so the light tiles fill the last,
// partly occupied round of blocks instead of a full-cost tile being left over there.
// Wave-wide helpers for the tile lookup: every lane holds one expert's numbers.
__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ int wave_scan_i32(int v, int lane) {  // inclusive prefix sum over the 64 lanes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int o = __shfl_up(v, off, 64);
        if (lane >= off) v += o;
    }
    return v;
}

constexpr int kCusPerXcd = 32;
constexpr int kMaxSplit = 4;
// fp32 partial tiles of the split last round: at most kCusPerXcd pieces per XCD
constexpr int64_t kSplitWorkspaceBytes = (int64_t)kNumXcd * kCusPerXcd * BM * BN * 4;

// How the M-grouped tiles of a launch are laid out over the XCDs: every XCD runs `heavy_per_xcd` heavy tiles and then
// `light_per_xcd` light ones (slots 0 .. per_xcd - 1).  With max_pieces > 1, the tiles left over after the full rounds of
// kCusPerXcd (`rem` of them, slots >= full) are cut into `pieces` ranges of K each, so that the last, partly filled round
// takes 1 / pieces of a tile instead of a whole one: slot full + t * pieces + p is piece p of tile slot full + t.
// Tile and row totals fit 32 bits (the grid does), and everything here is 32-bit unsigned arithmetic on purpose: every
// wavefront of every block runs this lookup on the CU's one scalar unit before its first load, and 64-bit divisions there
// (some hundred scalar instructions each) were 2 % of a tile's time.
struct GroupedLayout {
    uint32_t heavy, light, heavy_per_xcd, light_per_xcd, per_xcd;
    uint32_t full;  // slots of whole tiles that come first
    int rem, pieces;
    int c0;        // this lane's counts[lane] (0 past E): the lookup that follows reuses it instead of loading it again
};

// Runs in every wave, 64 experts at a time (lane = expert): one coalesced load of counts[] per pass instead of a chain
// of dependent scalar loads.
__device__ __forceinline__ GroupedLayout grouped_layout(const int64_t* counts, int E, int n_tiles, int max_pieces) {
    const int lane = threadIdx.x & 63;
    int heavy_m = 0, light_m = 0, c0 = 0;
    for (int base = 0; base < E; base += 64) {
        const uint32_t c = base + lane < E ? (uint32_t)counts[base + lane] : 0u, rem = c % BM;
        if (base == 0) c0 = (int)c;
        heavy_m += (int)(c / BM) + (rem > BM / 2);
        light_m += (rem > 0 && rem <= BM / 2);
    }
    heavy_m = uniform_i32(wave_sum_i32(heavy_m));  // the same in every lane: scalar from here on
    light_m = uniform_i32(wave_sum_i32(light_m));
    GroupedLayout g;
    g.c0 = c0;
    g.heavy = (uint32_t)heavy_m * (uint32_t)n_tiles;
    g.light = (uint32_t)light_m * (uint32_t)n_tiles;
    g.heavy_per_xcd = (g.heavy + kNumXcd - 1) / (uint32_t)kNumXcd;
    g.light_per_xcd = (g.light + kNumXcd - 1) / (uint32_t)kNumXcd;
    g.per_xcd = g.heavy_per_xcd + g.light_per_xcd;
    g.full = g.per_xcd;
    g.rem = 0;
    g.pieces = 1;
    if (max_pieces > 1) {
        static_assert(kCusPerXcd == 32 && kMaxSplit == 4, "the piece count below is kCusPerXcd / rem, capped at 4");
        const int rem = (int)(g.per_xcd % (uint32_t)kCusPerXcd);
        // as many pieces as keep rem * pieces within the XCD's 32 CUs: 4 up to 8 left-over tiles, 3 for 9 or 10, 2 up to 16
        int pieces = rem == 0 ? 1 : (rem <= 8 ? 4 : (rem <= 10 ? 3 : (rem <= 16 ? 2 : 1)));
        if (pieces > max_pieces) pieces = max_pieces;
        if (pieces > 1) {
            g.full = g.per_xcd - (uint32_t)rem;
            g.rem = rem;
            g.pieces = pieces;
        }
    }
    return g;
}

// Tile number `tile_slot` (0 .. per_xcd - 1) of XCD `xcd`.
__device__ __forceinline__ bool locate_tile_slot(const int64_t* counts, int E, int n_tiles, const GroupedLayout& g, uint32_t xcd,
                                                 uint32_t tile_slot, TileCoord* tc) {
    const int lane = threadIdx.x & 63;
    bool want_light;
    uint32_t L;
    if (tile_slot < g.heavy_per_xcd) {
        // Runs of kCusPerXcd heavy tiles are dealt to the XCDs in turn (run r to XCD r mod 8) while whole deals of eight runs
        // last, and what is left is split evenly, a contiguous eighth per XCD: every XCD still runs heavy_per_xcd tiles, but at
        // any time the eight of them work through neighbouring column ranges of the same expert, whose rows (the A operand,
        // re-read by every column range) then stay in the last-level cache -- with one expert per XCD the rows of eight
        // experts pass through it at once.
        want_light = false;
        const uint32_t deals = g.heavy_per_xcd / (uint32_t)kCusPerXcd, dealt = deals * (uint32_t)kCusPerXcd;
        if (tile_slot < dealt)
            L = ((tile_slot / (uint32_t)kCusPerXcd) * (uint32_t)kNumXcd + xcd) * (uint32_t)kCusPerXcd + tile_slot % (uint32_t)kCusPerXcd;
        else
            L = dealt * (uint32_t)kNumXcd + xcd * (g.heavy_per_xcd - dealt) + (tile_slot - dealt);
        if (L >= g.heavy) return false;
    } else if (tile_slot < g.per_xcd) {
        want_light = true;
        L = xcd * g.light_per_xcd + (tile_slot - g.heavy_per_xcd);
        if (L >= g.light) return false;
    } else {
        return false;
    }
    uint32_t tiles_before = 0, rows_before = 0;
    for (int base = 0; base < E; base += 64) {
        const uint32_t c = base == 0 ? (uint32_t)g.c0 : (base + lane < E ? (uint32_t)counts[base + lane] : 0u);
        const uint32_t full = c / BM, rem = c % BM;
        const int me = want_light ? (int)(rem > 0 && rem <= BM / 2) : (int)full + (rem > BM / 2);
        const int te = me * n_tiles;
        const int te_incl = wave_scan_i32(te, lane), rows_incl = wave_scan_i32((int)c, lane);
        const uint32_t te_total = (uint32_t)uniform_i32(__shfl(te_incl, 63, 64));
        if (L < tiles_before + te_total) {  // the tile belongs to an expert of this group of 64
            const uint64_t hit = __ballot(tiles_before + (uint32_t)te_incl > L);
            const int src = uniform_i32(__ffsll((unsigned long long)hit) - 1);
            const uint32_t c_e = (uint32_t)uniform_i32(__shfl((int)c, src, 64));
            const uint32_t me_e = (uint32_t)uniform_i32(__shfl(me, src, 64));
            const uint32_t Le = L - tiles_before - (uint32_t)uniform_i32(__shfl(te_incl, src, 64) - __shfl(te, src, 64));
            const uint32_t start = rows_before + (uint32_t)uniform_i32(__shfl(rows_incl, src, 64)) - c_e;
            // The expert's heavy tiles in groups of 8 tile rows: a group's tiles column by column, tile row fastest, then the
            // next group.  32 consecutive tiles -- what an XCD's CUs run at a time -- are then an 8 x 4 patch (8 + 4 operand
            // slices per k-step from the L2) however many rows the expert has; with all its tile rows in one column-major sweep
            // an expert of 64 tile rows (a shared expert over 16384 tokens) gave an XCD 32 x 1 patches, 33 slices per k-step.
            constexpr uint32_t GM = 8;
            const uint32_t grp = Le / (GM * (uint32_t)n_tiles), in_grp = Le - grp * (GM * (uint32_t)n_tiles);
            const uint32_t hm = want_light ? 1u : (me_e - grp * GM < GM ? me_e - grp * GM : GM);  // tile rows of this group
            const uint32_t nt = in_grp / hm, rm = in_grp - nt * hm;
            const uint32_t m = want_light ? c_e / BM : grp * GM + rm;
            tc->e = base + src;
            tc->m_tile = (int)m;
            tc->n_tile = (int)nt;
            tc->row0 = (int64_t)(start + m * BM);
            const uint32_t left = c_e - m * BM;
            tc->rows = (int)(left < (uint32_t)BM ? left : (uint32_t)BM);
            tc->a_sn = n_tiles < 4 ? n_tiles : 4;
            tc->a_si = tc->n_tile % tc->a_sn;
            tc->b_sn = (int)hm;
            tc->b_si = (int)rm;
            return true;
        }
        tiles_before += te_total;
        rows_before += (uint32_t)uniform_i32(__shfl(rows_incl, 63, 64));
    }
    return false;
}

// The tile (and, with max_pieces > 1, the piece of it) behind position `slot` of this block's XCD's run (blockIdx.x / 8).
__device__ __forceinline__ bool locate_m_grouped(const int64_t* counts, int E, int n_tiles, uint32_t slot, TileCoord* tc,
                                                 int max_pieces = 1) {
    const GroupedLayout g = grouped_layout(counts, E, n_tiles, max_pieces);
    uint32_t tile_slot = slot;
    tc->piece = 0;
    tc->pieces = 1;
    tc->ws_slot = 0;
    if (slot >= g.full && g.pieces > 1) {
        const uint32_t idx = slot - g.full;
        if (idx >= (uint32_t)(g.rem * g.pieces)) return false;
        const uint32_t tile = idx / (uint32_t)g.pieces;  // pieces is 2, 3 or 4
        tile_slot = g.full + tile;
        tc->piece = (int)(idx - tile * (uint32_t)g.pieces);
        tc->pieces = g.pieces;
        tc->ws_slot = (int)((blockIdx.x % kNumXcd) * kCusPerXcd + idx);
    }
    return locate_tile_slot(counts, E, n_tiles, g, blockIdx.x % kNumXcd, tile_slot, tc);
}

// first row of expert e's segment: the sum of the counts before it
__device__ __forceinline__ int64_t segment_start(const int64_t* counts, int e) {
    const int lane = threadIdx.x & 63;
    int64_t start = 0;
    for (int base = 0; base < e; base += 64) start += wave_sum_i32(base + lane < e ? (int)counts[base + lane] : 0);
    return uniform_i64(start);
}


inline unsigned round_up_xcd(int64_t g) { return (unsigned)(((g + kNumXcd - 1) / kNumXcd) * kNumXcd); }
// upper bound of 8 * (ceil(heavy / 8) + ceil(light / 8)) over every split of the rows among the experts
inline unsigned grid_m_grouped(const FfnShape& s, int n_tiles, bool split = false) {
    // a split last round adds at most kCusPerXcd slots per XCD
    return round_up_xcd((s.n_rows / BM + s.E) * (int64_t)n_tiles) + 2 * kNumXcd + (split ? kNumXcd * kCusPerXcd : 0);
}


}  // namespace
