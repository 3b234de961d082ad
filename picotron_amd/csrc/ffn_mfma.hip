// bf16 MFMA expert-FFN kernels for gfx950 (MI355X): grouped GEMMs over variable-length expert
// segments, forward + dgrad + wgrad, with the SwiGLU forward / backward fused into the epilogues.
//
// Block tile 256 x 256 x 64 (M x N x K), 8 wavefronts (two per SIMD), each owning a 128 x 64
// sub-tile as 8 x 4 v_mfma_f32_16x16x32_bf16 accumulators (128 fp32 per lane).  The 16 x 16 x 32 shape is a matter of
// power: an MFMA-only loop on random operands, where the chip's clock is set by the power it draws, runs 13-14 % faster
// with it than with 32 x 32 x 16 (1788 against 1577 and 2020 against 1773 TFLOP/s on two boxes; both reach 2460 on
// zeros) -- it reads and writes each accumulator once per 32 k values instead of once per 16.  (wgrad keeps
// 4 x 2 accumulators of 32 x 32 x 16: its loop waits for its strided operand loads, and the higher clock the narrow
// shape earns it only makes that wait longer in cycles -- 5 % slower in the layer.)  Operand
// tiles go HBM/L2 -> LDS with 16-byte direct-to-LDS loads (no staging registers), two LDS stages of
// 64 KB.  The k-loop is a ping-pong: the two waves of a SIMD alternate between a memory phase (fragment
// reads) and an MFMA phase (16 MFMAs with the operand loads of the next k-tile and the L2 prefetch issued
// between them), one phase apart.
//
// Two LDS tile layouts, chosen per operand by how it lies in memory:
//   K-major  (rows of the operand are contiguous along K: activations, forward weights)
//            LDS [256 rows][64 k] (128 B rows); fragments are plain ds_read_b128; the 16-byte chunk index
//            is XOR-swizzled with the row.
//   X-major  (contiguous along M or N, i.e. K is the slow index: weights in dgrad, both operands of wgrad)
//            LDS [64 k][256 cols] (512 B rows); fragments come from ds_read_b64_tr_b16, the LDS
//            transpose-read of gfx950, so no transposed copy of any tensor is ever made.
// A direct-to-LDS load always writes lane l at LDS base + 16*l, so every swizzle is applied on the
// global-address side (which 16-byte chunk a lane fetches).
//
// Tiles are enumerated on the device from counts[] (no host copy): expert by expert, N-tile by
// N-tile, M-tile fastest, and consecutive tiles are handed to the same XCD (block b runs on XCD
// b % 8) so that the blocks sharing an L2 share operand tiles.
#include <type_traits>

#include "ffn.h"
#include "mfma_tiles.h"

namespace {

constexpr int BK = 64;
constexpr int kWaves = 8;
// L2 prefetch distance in k-steps (2 for every mode: 1 cost the backward kernels 9 %, 3 and 4 nothing or 1 %)
constexpr int kPrefetchDist = 2;
// k-steps per trip of the k-loop.  The loop's back edge sits in front of a memory phase, whose fragment reads then start
// late and hold up the other group's MFMAs: four k-steps per trip gained 1.3 % on the forward and dgrad kernels; wgrad
// (the most scalar state, which then spills) gained nothing and stays at one.
constexpr int kKtUnroll = 4;
enum Mode { kGateUp = 0, kDown = 1, kDgradAct = 2, kDgradX = 3, kWgrad = 4 };

template <int MODE>
struct Traits {
    static constexpr bool kAKMajor = MODE != kWgrad;
    static constexpr bool kBKMajor = MODE == kGateUp || MODE == kDown;
};

struct MfmaParams {
    const int64_t* counts;
    int E;
    int64_t n_rows;
    int64_t K;          // contraction length for the M-grouped modes
    int64_t N;          // output columns (I for gate/up and dgrad_act, H for down and dgrad_x, Q for wgrad)
    int64_t M;          // wgrad only: output rows P
    int n_tiles;        // tiles along N
    int m_tiles;        // wgrad only: tiles along P
    const uint16_t* A;  // activations [n_rows, lda]; wgrad: lhs
    int64_t lda;
    const uint16_t* B0;  // gate_w / down_w; wgrad: rhs
    const uint16_t* B1;  // up_w or null
    int64_t ldb;         // row stride of B (elements)
    int64_t b_expert_stride;
    uint16_t* out;
    int64_t ldo;
    uint16_t* out2;       // gate/up: inter13 (optional); dgrad_act: act_out (optional)
    const uint16_t* aux;  // down: row_weight; dgrad_act: inter13
    float* ws;            // M-grouped modes: fp32 partial tiles of the split last round (kSplitWorkspaceBytes), or null
    int max_pieces;       // 1 = no split
};

// X-major tiles: 16-byte chunk swizzle of k row kr.  One transpose read takes 32 bytes from each of 16 k rows (rows
// 8g + j, g = 0..3, j = 0..3, plus a multiple of 4); rows are 512 B apart, i.e. on the same banks, and the swizzle puts the
// eight rows the first half of the lanes addresses (g = 0, 1) on the eight 32-byte slots of the 256 bytes of banks.
// With 32 x 32 MFMA blocks (wgrad) a read takes 64 bytes from each of 8 k rows (rows 8h + j, h = 0, 1), which the
// swizzle spreads over the four 64-byte slots twice.
template <bool WIDE>
__device__ __forceinline__ int swz_x(int kr) {
    return WIDE ? 4 * (kr & 3) + 16 * ((kr >> 3) & 1) : 2 * (kr & 3) + 8 * ((kr >> 3) & 1);
}

typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;

// wgrad tiles: expert by expert; inside an expert the P x Q tile grid is walked in bands of 4 tile columns and, inside
// a band, in groups of 8 tile rows (tile row fastest inside a group), so that any 32 consecutive tiles -- what one
// XCD's 32 CUs run at a time -- form an 8 x 4 patch that needs only 8 + 4 operand slices per k-step from its L2.
// The runs of 32 are dealt to the XCDs in turn (run r to XCD r mod 8), not as one contiguous eighth of the tiles each: a
// wgrad tile costs what its expert has rows, and with skewed counts a contiguous eighth is a few experts -- the XCD that
// drew the big ones ran 2.5 times as long as the mean at 64 experts under a Zipf load, and 5 % longer with eight experts
// of 1931 .. 2135 rows.  What is left after the last whole deal of eight runs is split evenly, a contiguous eighth per XCD
// (a launch of one or two rounds would otherwise give half the XCDs a whole run more than the others).
// (32-bit unsigned arithmetic throughout: see GroupedLayout.)
constexpr uint32_t kWgradRun = kCusPerXcd, kWgradDeal = kWgradRun * kNumXcd;
inline unsigned grid_wgrad(int64_t tiles) {
    const int64_t deals = tiles / kWgradDeal, left = tiles - deals * kWgradDeal;
    return (unsigned)((deals * kWgradRun + (left + kNumXcd - 1) / kNumXcd) * kNumXcd);
}
__device__ __forceinline__ bool locate_wgrad(const int64_t* counts, int E, int m_tiles, int n_tiles, uint32_t slot, TileCoord* tc) {
    const uint32_t per_e = (uint32_t)m_tiles * (uint32_t)n_tiles, total = per_e * (uint32_t)E;
    // logical tile id of this block: slot s of XCD x is tile s % 32 of run (s / 32) * 8 + x while whole deals last
    const uint32_t deals = total / kWgradDeal, xcd = blockIdx.x % kNumXcd;
    uint32_t L;
    if (slot < deals * kWgradRun) {
        L = ((slot / kWgradRun) * (uint32_t)kNumXcd + xcd) * kWgradRun + slot % kWgradRun;
    } else {
        const uint32_t left_per_xcd = (total - deals * kWgradDeal + kNumXcd - 1) / (uint32_t)kNumXcd, t = slot - deals * kWgradRun;
        if (t >= left_per_xcd) return false;
        L = deals * kWgradDeal + xcd * left_per_xcd + t;
    }
    if (L >= total) return false;
    const uint32_t e = L / per_e, rem = L - e * per_e;
    constexpr uint32_t GM = 8, GN = 4;
    const uint32_t um = (uint32_t)m_tiles, un = (uint32_t)n_tiles;
    const uint32_t band = rem / (um * GN), r = rem - band * (um * GN);
    const uint32_t wn = un - band * GN < GN ? un - band * GN : GN;
    const uint32_t g = r / (GM * wn), r2 = r - g * (GM * wn);
    const uint32_t hm = um - g * GM < GM ? um - g * GM : GM;
    const uint32_t q = r2 / hm, rm = r2 - q * hm;
    tc->e = (int)e;
    tc->m_tile = (int)(g * GM + rm);
    tc->n_tile = (int)(band * GN + q);
    tc->a_sn = (int)wn;
    tc->a_si = (int)q;
    tc->b_sn = (int)hm;
    tc->b_si = (int)rm;
    tc->row0 = segment_start(counts, (int)e);
    tc->rows = uniform_i32((int)counts[e]);
    return true;
}

// NW = 8 wavefronts per block, two per SIMD, wave tile 128 x 64: one wave's waits and memory instructions are covered by
// the other wave's MFMAs.
template <int MODE, int NW>
__global__ __launch_bounds__(NW * 64, 1) void ffn_mfma_kernel(MfmaParams p) {
    using T = Traits<MODE>;
    constexpr bool kWide = MODE == kWgrad;  // 32 x 32 x 16 MFMA blocks instead of 16 x 16 x 32
    constexpr int NI = 8;               // 16-row blocks per wave
    constexpr int NJ = 4;               // 16-column blocks per wave
    constexpr int WI = 4, WJ = 2;       // the same in 32 x 32 blocks
    constexpr int kWaveCols = NW / 2;   // wave grid: 2 rows x kWaveCols columns
    constexpr int CW = NJ * 16;         // columns per wave
    constexpr int QN = 32 / NW;         // direct-to-LDS load instructions per operand, wave and k-tile
    constexpr int RPW = QN * 8;         // K-major tile rows a wave fills
    constexpr int KPW = QN * 2;         // X-major k rows a wave fills
    __shared__ __attribute__((aligned(1024))) char lds[2 * kStageBytes];
    constexpr bool kCanSplit = MODE != kWgrad;  // the M-grouped modes can cut the tiles of a partly filled last round along K
    TileCoord tc;
    if (MODE == kWgrad) {
        if (!locate_wgrad(p.counts, p.E, p.m_tiles, p.n_tiles, blockIdx.x / kNumXcd, &tc)) return;
    } else {
        if (!locate_m_grouped(p.counts, p.E, p.n_tiles, blockIdx.x / kNumXcd, &tc, kCanSplit ? p.max_pieces : 1)) return;
    }

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: LDS bases and row ranges stay scalar
    const int wm = wave / kWaveCols, wn = wave % kWaveCols;
    const int l15 = lane & 15, g4 = lane >> 4;
    // k-tiles of this block: all of K, or this piece's share of it
    const int n_kt_all = MODE == kWgrad ? (int)((uint32_t)(tc.rows + BK - 1) / BK) : (int)((uint64_t)p.K / BK);
    // (pieces is 1 .. 4; two 32-bit divisions per block)
    const int kt_first = kCanSplit ? (int)((uint32_t)(tc.piece * n_kt_all) / (uint32_t)tc.pieces) : 0;
    const int n_kt = kCanSplit ? (int)((uint32_t)((tc.piece + 1) * n_kt_all) / (uint32_t)tc.pieces) - kt_first : n_kt_all;
    // a wavefront whose 128 rows all lie past the end of the expert's segment keeps loading and synchronising
    // but skips its fragment reads and MFMAs
    // 32-row blocks of this wave's 128 rows that hold rows of the expert's segment (wgrad: all four; its ragged dimension is K)
    const int rows_here = MODE == kWgrad ? 128 : (tc.rows - wm * 128 < 0 ? 0 : (tc.rows - wm * 128 > 128 ? 128 : tc.rows - wm * 128));
    const int active_blocks = (rows_here + 31) / 32;

    // ------------------------------------------------------------------------------------------
    // global -> LDS: a wave-uniform base pointer per operand plus, per lane, a 32-bit byte offset for each
    // of the wave's 8 load instructions (scalar base + vector offset addressing: no 64-bit vector adds)
    // ------------------------------------------------------------------------------------------
    uint32_t a_off[QN], b_off[QN];
    const char* a_base;
    const char* b_base;
    int64_t a_step, b_step;      // bytes per k-tile
    int64_t b_switch_delta = 0;  // dgrad_x: jump from gate_w to up_w half way through K
    int b_switch_kt = 0x7FFFFFFF;
    int64_t b_jump_now = 0;      // dgrad_x, a piece that starts in the up_w half: the same jump, taken from the start
    if (T::kAKMajor) {
        // wave w fills tile rows [RPW*w, RPW*(w+1)), 8 rows (128 B each) per instruction
        a_step = BK * 2;
        a_base = (const char*)(p.A + tc.row0 * p.lda);
#pragma unroll
        for (int q = 0; q < QN; ++q) {
            const int r = wave * RPW + q * 8 + (lane >> 3);
            const int ar = r < tc.rows ? r : tc.rows - 1;  // rows past the segment re-read its last row (never stored)
            a_off[q] = (uint32_t)(ar * (int)p.lda * 2 + ((lane & 7) ^ swz(r)) * 16);
        }
    } else {
        // wgrad lhs [k rows, P]: wave w fills k rows [KPW*w, KPW*(w+1)), 2 rows (512 B each) per instruction
        a_step = BK * p.lda * 2;
        a_base = (const char*)(p.A + tc.row0 * p.lda);
#pragma unroll
        for (int q = 0; q < QN; ++q) {
            const int kr = wave * KPW + q * 2 + (lane >> 5);
            const int chunk = (lane & 31) ^ swz_x<kWide>(kr);
            int64_t col = (int64_t)tc.m_tile * BM + chunk * 8;
            col = col + 8 <= p.M ? col : p.M - 8;
            a_off[q] = (uint32_t)(kr * (int)p.lda * 2 + (int)col * 2);
        }
    }
    if (T::kBKMajor) {
        b_step = BK * 2;
        int64_t brow0;
        const uint16_t* bmat;
        if (MODE == kGateUp) {
            // B tile rows: per wave column (CW rows), CW/2 gate rows then CW/2 up rows of the same I range.
            // RPW == CW/2, so even waves load gate rows and odd waves up rows.
            static_assert(RPW * 2 == CW, "gate/up interleave assumes one wave loads half a wave column");
            bmat = (wave & 1) ? p.B1 : p.B0;
            brow0 = (int64_t)tc.n_tile * 128 + (wave >> 1) * (CW / 2);
        } else {
            bmat = p.B0;
            brow0 = (int64_t)tc.n_tile * BN + wave * RPW;
        }
        // weight rows past the last output column (an N that is not a multiple of the tile) re-read the last row;
        // the columns they produce are never stored
        if (brow0 > p.N - 1) brow0 = p.N - 1;
        const int rel_max = (int)(p.N - 1 - brow0);
        b_base = (const char*)(bmat + (int64_t)tc.e * p.b_expert_stride + brow0 * p.ldb);
#pragma unroll
        for (int q = 0; q < QN; ++q) {
            const int r = wave * RPW + q * 8 + (lane >> 3);  // row of the LDS tile (fixes the swizzle)
            const int rel = q * 8 + (lane >> 3) < rel_max ? q * 8 + (lane >> 3) : rel_max;
            b_off[q] = (uint32_t)(rel * (int)p.ldb * 2 + ((lane & 7) ^ swz(r)) * 16);
        }
    } else {
        b_step = BK * p.ldb * 2;
        b_base = (const char*)(MODE == kWgrad ? p.B0 + tc.row0 * p.ldb : p.B0 + (int64_t)tc.e * p.b_expert_stride);
        if (MODE == kDgradX) {
            // B moves from gate_w to up_w at k-tile n_kt_all / 2 of the whole K; in this block's own numbering
            // (k-tile 0 = kt_first) that is either still ahead or already behind
            const int sw = n_kt_all / 2;
            const int64_t jump = ((const char*)p.B1 - (const char*)p.B0) - (int64_t)sw * b_step;
            if (kt_first >= sw) {
                b_jump_now = jump;
            } else if (sw - kt_first < n_kt) {  // a piece that ends at or before the switch never takes the jump
                b_switch_kt = sw - kt_first;
                b_switch_delta = jump;
            }
        }
#pragma unroll
        for (int q = 0; q < QN; ++q) {
            const int kr = wave * KPW + q * 2 + (lane >> 5);
            const int chunk = (lane & 31) ^ swz_x<kWide>(kr);
            int64_t col = (int64_t)tc.n_tile * BN + chunk * 8;
            col = col + 8 <= p.N ? col : p.N - 8;
            b_off[q] = (uint32_t)(kr * (int)p.ldb * 2 + (int)col * 2);
        }
    }
    // wgrad: k rows past the expert's last row are re-read from its last row and masked out of the fragments
    a_base += (int64_t)kt_first * a_step;
    b_base += (int64_t)kt_first * b_step + b_jump_now;
    // Only the last k-tile can reach past the segment, so its clamped lane offsets are worked out once, here, and a
    // load picks between the two precomputed offsets with one select (computing the clamp at every load put a dependent
    // chain of vector instructions, a 64-bit multiply-add among them, between the MFMAs of wgrad's load phases).
    uint32_t a_off_tail[T::kAKMajor ? 1 : QN], b_off_tail[T::kBKMajor ? 1 : QN];
    if (MODE == kWgrad) {
#pragma unroll
        for (int q = 0; q < QN; ++q) {
            const int kr = (n_kt - 1) * BK + wave * KPW + q * 2 + (lane >> 5);
            const int dk = kr < tc.rows ? 0 : tc.rows - 1 - kr;
            if (!T::kAKMajor) a_off_tail[q] = (uint32_t)((int)a_off[q] + dk * (int)p.lda * 2);
            if (!T::kBKMajor) b_off_tail[q] = (uint32_t)((int)b_off[q] + dk * (int)p.ldb * 2);
        }
    }
    // one load instruction (q of QN) of this wave for the A or the B tile of k-tile kt into a stage.  The loads are the
    // opaque form: every wait between a load and the LDS reads of its data is written out in this kernel (prologue,
    // sub-step 3 of the k-loop, the end of the loop), the compiler adds none.
    // ab / bb: the wave-uniform address of the operand's k-tile; last: it is the segment's last k-tile (wgrad's clamped offsets)
    auto a_tile = [&](int kt) { return a_base + (int64_t)kt * a_step; };
    auto b_tile = [&](int kt) { return b_base + (int64_t)kt * b_step + (kt >= b_switch_kt ? b_switch_delta : 0); };
    auto issue_a_at = [&](const char* ab, bool last, int stage, int q) {
        char* base = lds + stage * kStageBytes;
        if (T::kAKMajor)
            load16_to_lds_opaque(ab, a_off[q], base + (wave * RPW + q * 8) * 128);
        else
            load16_to_lds_opaque(ab, MODE == kWgrad && last ? a_off_tail[q] : a_off[q], base + (wave * KPW + q * 2) * 512);
    };
    auto issue_b_at = [&](const char* bb, bool last, int stage, int q) {
        char* base = lds + stage * kStageBytes + kTileBytes;
        if (T::kBKMajor)
            load16_to_lds_opaque(bb, b_off[q], base + (wave * RPW + q * 8) * 128);
        else
            load16_to_lds_opaque(bb, MODE == kWgrad && last ? b_off_tail[q] : b_off[q], base + (wave * KPW + q * 2) * 512);
    };
    auto issue_a = [&](int kt, int stage, int q) { issue_a_at(a_tile(kt), kt == n_kt - 1, stage, q); };
    auto issue_b = [&](int kt, int stage, int q) { issue_b_at(b_tile(kt), kt == n_kt - 1, stage, q); };
    // A wave whose 128 rows all lie past the segment (rows 128..255 of a tile of at most 128 rows) also fills tile rows
    // nobody reads: its A loads are left out, in the prologue here and in its copy of the k-loop (a quarter of the loads
    // of a light tile; 3 % of the gate/up launch at 64 skewed experts, nothing where light tiles are few).
    const bool skip_a = MODE != kWgrad && active_blocks == 0;
    auto issue_tile = [&](int kt, int stage) {
#pragma unroll
        for (int q = 0; q < QN; ++q) {
            if (!skip_a) issue_a(kt, stage, q);
            issue_b(kt, stage, q);
        }
    };

    // The first two k-tiles go out before anything else is set up (prefetch pointers, fragment addresses, the zeroed
    // accumulators): what follows runs under their latency.
    if (n_kt > 0) {
        issue_tile(0, 0);
        if (n_kt > 1) issue_tile(1, 1);
    }

    // ------------------------------------------------------------------------------------------
    // L2 prefetch.  The demand loads of the blocks that share an operand slice reach the L2 together, and when the
    // slice still has to come from HBM they all queue behind the same misses.  So every k-step each wave touches
    // (one 4-byte load per 64 bytes into a scratch register nobody reads) its share of the lines of a slice
    // kPrefetchDist k-steps ahead: the first half of the waves lines of the A slice, the second half lines of the B
    // slice.
    // ------------------------------------------------------------------------------------------
    const char* pf_ptr;   // this lane's line at k-tile 0
    int64_t pf_step;      // bytes per k-tile
    {
        const bool pf_b = wave >= NW / 2;
        const int q = (wave % (NW / 2)) * 64 + lane;
        const int si = pf_b ? tc.b_si : tc.a_si, sn = pf_b ? tc.b_sn : tc.a_sn;
        // two touches (one per 64 bytes) of every sn-th line; a tile that shares its slice with nobody (a light tail, an
        // expert of one row tile) touches every line once instead: at two touches per line its 256 lanes would only
        // reach lines 0..127 and leave the other half of the slice to the demand loads
        const int half = sn > 1 ? (q & 1) : 0;
        int j = sn > 1 ? si + sn * (q >> 1) : q;  // line of the 256-line slice
        if (j >= 256) j = si;
        // X-major slices: line j is 128 bytes of k row j / 4; a segment shorter than one k-tile clamps the row
        int kr = j >> 2;
        if (MODE == kWgrad && kr >= tc.rows) kr = tc.rows > 0 ? tc.rows - 1 : 0;
        if (!pf_b) {
            pf_step = a_step;
            if (T::kAKMajor) {
                const int r = j < tc.rows ? j : tc.rows - 1;
                pf_ptr = (const char*)(p.A + (tc.row0 + r) * p.lda) + half * 64;
            } else {
                int64_t col = (int64_t)tc.m_tile * BM + (j & 3) * 64 + half * 32;
                col = col + 8 <= p.M ? col : p.M - 8;
                pf_ptr = (const char*)(p.A + (tc.row0 + kr) * p.lda + col);
            }
        } else {
            pf_step = b_step;
            if (MODE == kGateUp) {
                const uint16_t* m = j < 128 ? p.B0 : p.B1;
                int64_t wr = (int64_t)tc.n_tile * 128 + (j & 127);
                wr = wr < p.N ? wr : p.N - 1;
                pf_ptr = (const char*)(m + (int64_t)tc.e * p.b_expert_stride + wr * p.ldb) + half * 64;
            } else if (MODE == kDown) {
                int64_t wr = (int64_t)tc.n_tile * BN + j;
                wr = wr < p.N ? wr : p.N - 1;
                pf_ptr = (const char*)(p.B0 + (int64_t)tc.e * p.b_expert_stride + wr * p.ldb) + half * 64;
            } else {
                int64_t col = (int64_t)tc.n_tile * BN + (j & 3) * 64 + half * 32;
                col = col + 8 <= p.N ? col : p.N - 8;
                const uint16_t* m = MODE == kWgrad ? p.B0 + tc.row0 * p.ldb : p.B0 + (int64_t)tc.e * p.b_expert_stride;
                pf_ptr = (const char*)(m + (int64_t)kr * p.ldb + col);
            }
        }
    }
    pf_ptr += (int64_t)kt_first * pf_step + (wave >= NW / 2 ? b_jump_now : 0);
    const int64_t pf_switch_delta = wave >= NW / 2 ? b_switch_delta : 0;
    // wgrad: only k-tiles that lie completely inside the expert's rows are prefetched
    const int pf_n_kt = MODE == kWgrad ? tc.rows / BK : n_kt;
    // the lane's pointer moves on by one k-tile per call until it reaches the last k-tile that may be touched
    const int pf_kt0 = kPrefetchDist < pf_n_kt ? kPrefetchDist : (pf_n_kt > 0 ? pf_n_kt - 1 : 0);
    const char* pf_cur = pf_ptr + (int64_t)pf_kt0 * pf_step + (pf_kt0 >= b_switch_kt ? pf_switch_delta : 0);
    auto prefetch_l2 = [&](int kt) {
        // Destination v255: a register the kernel never allocates (it needs fewer than 255; the build checks the
        // generated code for any other mention of v255), so a load still in flight cannot land on a live value.
        asm volatile("global_load_dword v255, %0, off" ::"v"(pf_cur) : "v255", "memory");
        const int kp = kt + kPrefetchDist + 1;  // the k-tile of the next call
        int64_t adv = kp < pf_n_kt ? pf_step : 0;
        if (MODE == kDgradX && kp == b_switch_kt) adv += pf_switch_delta;
        pf_cur += adv;
    };

    // ------------------------------------------------------------------------------------------
    // LDS -> fragments
    // ------------------------------------------------------------------------------------------
    // An MFMA takes 32 k values: a k-tile is two sub-steps.  Operand lane l holds row / column (l & 15) of a 16-wide block
    // and the 8 k values 8*(l >> 4) .. +7 of the sub-step.
    // K-major: lane reads row (l & 15) of a 16-row block, 16-byte k chunk 4*sub + (l >> 4).  The swizzle XORs the chunk
    //          index and depends on (row >> 1) & 7 only, which is the same in every 16-row block: one address register
    //          per operand, block b at + b * 2048 (an immediate), sub-step sub at XOR (sub << 6).
    // X-major: two transpose reads per fragment; lane addresses 8 bytes of k row 32*sub + 8*(l>>4) + 4t + ((l>>2)&3) at
    //          column 4*(l&3) of the 16-column block and receives k rows 32*sub + 8*(l>>4) + 4t..+3 of column (l & 15).
    //          sub and t are immediates (whole k rows), block b is XOR (b << 5): the block index sits in bits of the chunk
    //          index that the swizzle also flips, and XOR commutes where + does not.
    // One XOR per register and k-tile flips between the two stages.
    uint32_t a_ad, b_ad;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
    {
        const int kr = 8 * g4 + ((lane >> 2) & 3);  // X-major: the k row this lane addresses (sub-step 0, t = 0)
        const int h = (lane & 3) >> 1;              // which 16-byte chunk of the block's 32 bytes
        const int in_chunk = (4 * (lane & 1)) << 1; // byte offset of the lane's 4 columns inside the chunk
        if (T::kAKMajor) {
            const int ra = wm * 128 + l15;
            a_ad = lds0 + ra * 128 + ((g4 ^ swz(ra)) << 4);
        } else {
            a_ad = lds0 + kr * 512 + (((wm * 16 + h) ^ swz_x<kWide>(kr)) << 4) + in_chunk;
        }
        if (T::kBKMajor) {
            const int rb = wn * CW + l15;
            b_ad = lds0 + kTileBytes + rb * 128 + ((g4 ^ swz(rb)) << 4);
        } else {
            b_ad = lds0 + kTileBytes + kr * 512 + (((wn * 8 + h) ^ swz_x<kWide>(kr)) << 4) + in_chunk;
        }
    }
    // 32 x 32 blocks (wgrad, both operands X-major): one address register per block; lane addresses 8 bytes of k row
    // 16kk + 8*(l>>5) + 4t + ((l>>2)&3) at column 16*((l>>4)&1) + 4*(l&3) of the 32-column block and receives k rows
    // 16kk + 8*(l>>5) + 4t..+3 of column 16*((l>>4)&1) + (l&15).
    uint32_t a_adw[WI], b_adw[WJ];
    if (kWide) {
        const int hi = lane >> 5;
        const int xg = swz_x<true>(8 * hi + ((lane >> 2) & 3));
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            const int col = wm * 128 + i * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
            a_adw[i] = lds0 + (((col >> 3) ^ xg) << 4) + ((col & 7) << 1) + (8 * hi + ((lane >> 2) & 3)) * 512;
        }
#pragma unroll
        for (int j = 0; j < WJ; ++j) {
            const int col = wn * CW + j * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
            b_adw[j] = lds0 + kTileBytes + (((col >> 3) ^ xg) << 4) + ((col & 7) << 1) + (8 * hi + ((lane >> 2) & 3)) * 512;
        }
    }
    auto flip_stage = [&]() {
        if (kWide) {
#pragma unroll
            for (int i = 0; i < WI; ++i) a_adw[i] ^= (uint32_t)kStageBytes;
#pragma unroll
            for (int j = 0; j < WJ; ++j) b_adw[j] ^= (uint32_t)kStageBytes;
        } else {
            a_ad ^= (uint32_t)kStageBytes;
            b_ad ^= (uint32_t)kStageBytes;
        }
    };

    f32x4_t acc[NI][NJ];     // 16 x 16 blocks
    f32x16_t accw[WI][WJ];   // 32 x 32 blocks (wgrad); only the set the kernel uses exists in the compiled code
    if (kWide) {
#pragma unroll
        for (int i = 0; i < WI; ++i)
#pragma unroll
            for (int j = 0; j < WJ; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) accw[i][j][r] = 0.f;
    } else {
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    }

    // The 32 MFMAs of a sub-step are two phases of 16: rows 0..63 of the wave's 128 (blocks 0..3), then rows 64..127.
    // A phase holds its four A fragments and the sub-step's four B fragments, which the first phase of a sub-step reads.
    bf16x8_t af[4], bfr[NJ];
    auto read_b128 = [&](uint32_t ad) -> bf16x8_t { return *(__attribute__((address_space(3))) const bf16x8_t*)(uintptr_t)ad; };
    auto read_tr_frag = [&](uint32_t ad) -> bf16x8_t {
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(uintptr_t)ad);
        const s16x4_t hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(uintptr_t)(ad + 4 * 512));
        const s16x8_t v = {lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
        return __builtin_bit_cast(bf16x8_t, v);
    };
    auto read_a = [&](int ib, int sub) -> bf16x8_t {
        if (T::kAKMajor) return read_b128((a_ad ^ (uint32_t)(sub << 6)) + ib * 2048);
        return read_tr_frag((a_ad ^ (uint32_t)(ib << 5)) + sub * (32 * 512));
    };
    auto read_b = [&](int jb, int sub) -> bf16x8_t {
        if (T::kBKMajor) return read_b128((b_ad ^ (uint32_t)(sub << 6)) + jb * 2048);
        return read_tr_frag((b_ad ^ (uint32_t)(jb << 5)) + sub * (32 * 512));
    };
    // 16-row blocks of phase kk (sub-step kk >> 1, half kk & 1) that hold rows of the segment, given the wave's live
    // 32-row blocks
    auto live_blocks = [](int kk, int active32) {
        const int n = 2 * active32 - 4 * (kk & 1);
        return n < 0 ? 0 : (n > 4 ? 4 : n);
    };
    // reads the fragments of phase kk from the stage the address registers currently point at
    // (wide blocks: phase kk is the sub-step of 16 k values kk, 4 A and 2 B fragments, two transpose reads each)
    auto read_wide = [&](uint32_t ad, int kk) -> bf16x8_t { return read_tr_frag(ad + kk * (16 * 512)); };
    auto read_frags = [&](int kk, auto active) {
        constexpr int kActive32 = decltype(active)::value;
        if (kActive32 == 0) return;
        if (kWide) {
#pragma unroll
            for (int i = 0; i < kActive32; ++i) af[i] = read_wide(a_adw[i], kk);
#pragma unroll
            for (int j = 0; j < WJ; ++j) bfr[j] = read_wide(b_adw[j], kk);
            return;
        }
        const int sub = kk >> 1, half = kk & 1;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < live_blocks(kk, kActive32)) af[i] = read_a(4 * half + i, sub);
        if (half == 0) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) bfr[j] = read_b(j, sub);
        }
    };
    // wgrad, last k-tile: zero the fragment elements whose k row lies past the expert's last row
    auto mask_tail = [&](int kt, int kk) {
        if (MODE != kWgrad) return;
        // lane holds k = 8*(l >> 4) + 0..7 of its sub-step of 32 (wide blocks: 8*(l >> 5) + 0..7 of its sub-step of 16)
        const int valid = kWide ? tc.rows - kt * BK - kk * 16 - 8 * (lane >> 5) : tc.rows - kt * BK - (kk >> 1) * 32 - 8 * g4;
        if (valid >= 8) return;
        auto zero_tail = [&](bf16x8_t& f) {
            s16x8_t a = __builtin_bit_cast(s16x8_t, f);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (e >= valid) a[e] = 0;
            f = __builtin_bit_cast(bf16x8_t, a);
        };
#pragma unroll
        for (int i = 0; i < 4; ++i) zero_tail(af[i]);
        if (kWide || (kk & 1) == 0) {
#pragma unroll
            for (int j = 0; j < (kWide ? WJ : NJ); ++j) zero_tail(bfr[j]);
        }
    };
    // The 16 MFMAs of phase kk with side(n) run after MFMA n (n = 0 .. 15): the slots for this wave's loads.
    // The B fragment is the MFMA's first operand: the block comes out transposed, a lane holding four neighbouring
    // columns of one output row (what the epilogue wants to convert and stage together).
    // `active` carries the number of 32-row blocks the wave computes; a wave without rows runs the side jobs alone.
    auto mma_with = [&](int kk, auto active, auto side) {
        if (kWide) {  // 8 MFMAs of 32 x 32 x 16, side(n) after MFMA n (n = 0 .. 7)
#pragma unroll
            for (int i = 0; i < WI; ++i)
#pragma unroll
                for (int j = 0; j < WJ; ++j) {
                    if (i < decltype(active)::value)
                        accw[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], accw[i][j], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    side(i * WJ + j);
                    __builtin_amdgcn_sched_barrier(0);
                }
            return;
        }
        const int half = kk & 1;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                if (i < live_blocks(kk, decltype(active)::value))
                    acc[4 * half + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[j], af[i], acc[4 * half + i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                side(i * NJ + j);
                __builtin_amdgcn_sched_barrier(0);
            }
    };

    if (n_kt > 0) {
        if (n_kt > 1) {
            // vmcnt(2*QN): tile 0 has landed, tile 1 may still be in flight
            static_assert(QN == 4 || QN == 8, "wait counts below are written for 4 or 8 loads per operand, wave and k-tile");
            if (QN == 8) __builtin_amdgcn_s_waitcnt(0x4F70);
            else if (skip_a) __builtin_amdgcn_s_waitcnt(0x0F74);  // only the B loads were issued: QN per tile
            else __builtin_amdgcn_s_waitcnt(0x0F78);
        } else {
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        __syncthreads();
    }
    // The k-loop, a ping-pong between two groups of waves.  The eight waves form two groups, one wave of every SIMD in
    // each (waves 0-3 own tile rows 0..127, waves 4-7 rows 128..255).  A k-step is four pairs of phases (two sub-steps of
    // 32 k values, each in two halves of the wave's rows).  A pair is a memory phase -- the LDS reads of its fragments, in
    // the fourth also the wait for the next k-tile -- followed by an MFMA phase: its 16 MFMAs, and between them this
    // wave's direct-to-LDS loads of the next k-tile (pairs 0 and 1, one load after every fourth MFMA) and the L2 prefetch
    // (pair 2).  Every phase ends in a barrier and the second group runs one
    // phase behind the first, so while one wave of a SIMD reads LDS the other owns the MFMA pipe.
    // Where the loads sit matters.  A vector memory instruction holds its wave for some tens of cycles at issue.  In the
    // memory phase that time adds to the LDS reads, which alone take about as long as the other group's MFMAs (measured
    // with a cycle counter at every barrier: memory phases with loads ran 440-470 ticks against 341 for 8 MFMAs, the
    // ones without 364-400); between two MFMAs it is free, the matrix pipe being busy anyway (16 cycles per MFMA).
    // (History of the loop, each step measured side by side in one run: reads, loads and MFMAs interleaved finely in one
    // stream with two free-running waves per SIMD -- the older wave wins every MFMA slot and then idles a third of the
    // time at the k-step barrier; ping-pong with the loads in the memory phases, +8 %; loads in the MFMA phases, +4-7 %.)
    static_assert(NW == 8 && QN == 4, "the load slots of the MFMA phases are laid out for 8 waves (4 loads per operand tile and wave)");
    auto k_loop_pp = [&](auto active) {
        auto phase_end = [&]() {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        };
        if (wm == 1) phase_end();  // the phase offset of the second group
        // The k-tile the loads of a k-step fetch: kt + 1, or the last one again once kt + 1 runs past it (its stage was
        // last read one k-step ago).  Its operand addresses move on by one k-tile per k-step with two scalar adds;
        // working them out from kt (64-bit scalar multiplies by the run-time row pitch of an X-major operand) put some
        // twenty dependent scalar instructions in front of the first load of sub-step 0, between two MFMAs.
        const int kt_first_next = n_kt > 1 ? 1 : 0;
        // (readfirstlane: the loads take their base from scalar registers, and the compiler is free to evaluate even
        // wave-uniform selects like the one in b_tile on the vector unit)
        const char* a_next = (const char*)uniform_i64((int64_t)(uintptr_t)a_tile(kt_first_next));
        const char* b_next = (const char*)uniform_i64((int64_t)(uintptr_t)b_tile(kt_first_next));
        bool next_is_last = kt_first_next == n_kt - 1;
        // last_k_tile (compile time): wgrad's last k-tile, whose fragments are masked past the expert's last row.  It is a
        // copy of the k-step of its own, so that the other k-steps carry no test for it (a compare and a taken branch in
        // every memory phase, on the path the other group's MFMAs wait for).
        auto k_step = [&](int kt, auto last_k_tile) {
            const int stage = kt & 1;
            constexpr bool tail = MODE == kWgrad && decltype(last_k_tile)::value;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                // memory phase
                read_frags(kk, active);
                if (kk == 3) {
                    // this wave's operand loads of the next k-tile have landed (its prefetch load may stay in flight)
                    __builtin_amdgcn_s_waitcnt(0x0F71);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (tail) mask_tail(kt, kk);
                phase_end();
                // MFMA phase
                // load slots: every fourth of the 16 MFMAs (wide blocks: every second of the 8): one per 64 MFMA cycles
                constexpr int kSlotShift = kWide ? 1 : 2;
                mma_with(kk, active, [&](int n) {
                    if (kk < 2 && (n & ((1 << kSlotShift) - 1)) == 0) {
                        const int m = n >> kSlotShift;             // 0 .. 3
                        const int q = (QN / 2) * kk + (m >> 1);    // m = 0, 1: loads q of A and B; m = 2, 3: loads q + 1
                        constexpr bool kSkipA = MODE != kWgrad && decltype(active)::value == 0;
                        if ((m & 1) == 0) {
                            if (!kSkipA) issue_a_at(a_next, next_is_last, stage ^ 1, q);
                        } else {
                            issue_b_at(b_next, next_is_last, stage ^ 1, q);
                        }
                    }
                    if (kk == 2 && n == (kWide ? 1 : 2)) prefetch_l2(kt);
                });
                if (kk == 3) {
                    flip_stage();
                    if (kt + 2 < n_kt) {  // the next k-step fetches k-tile kt + 2
                        a_next += a_step;
                        b_next += b_step + (kt + 2 == b_switch_kt ? b_switch_delta : 0);
                    }
                    next_is_last = kt + 2 >= n_kt - 1;
                }
                phase_end();
            }
        };
        constexpr int kUnroll = MODE == kWgrad ? 1 : kKtUnroll;
        const int n_plain = MODE == kWgrad ? n_kt - 1 : n_kt;  // k-steps without the tail mask
        int kt_done = 0;
        for (; kt_done + kUnroll <= n_plain; kt_done += kUnroll) {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) k_step(kt_done + u, std::false_type{});
        }
        for (; kt_done < n_plain; ++kt_done) k_step(kt_done, std::false_type{});
        if (MODE == kWgrad && n_kt > 0) k_step(n_kt - 1, std::true_type{});
        if (wm == 0) phase_end();  // the first group finishes one phase early
    };
    // Five copies of the loop, picked per wave by the number of its 32-row blocks that hold rows of the segment: a wave
    // reads A fragments and issues MFMAs for those blocks only, and one whose 128 rows all lie past the end of a short tail
    // only loads and synchronises (same loads, waits and barriers, no reads, no MFMAs).  A tail tile then costs about what
    // its rows are worth instead of a half or a whole tile.
    switch (active_blocks) {
        case 4: k_loop_pp(std::integral_constant<int, 4>{}); break;
        case 3: k_loop_pp(std::integral_constant<int, 3>{}); break;
        case 2: k_loop_pp(std::integral_constant<int, 2>{}); break;
        case 1: k_loop_pp(std::integral_constant<int, 1>{}); break;
        default: k_loop_pp(std::integral_constant<int, 0>{}); break;
    }
    // the clamped refills of the last k-steps may still be landing in LDS, which the epilogue reuses
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    // ------------------------------------------------------------------------------------------
    // epilogue.  The MFMAs take the B fragment as their first operand, so an accumulator block is the transposed
    // product: a lane holds row (l & 15) of each 16-row block and the four neighbouring columns 4*(l >> 4) .. +3 of each
    // 16-column block (32 x 32 blocks: row (l & 31), columns 8q + 4*(l >> 5) .. +3, q = 0..3).  Four neighbours of an
    // output row convert to bf16 two at a time and go to LDS as one 8-byte write.  Each wave stages 32 rows at a time
    // through its own slice of LDS (the operand stages are free after the last barrier) and reads them back
    // row-contiguously, so HBM sees 16-byte lanes and 128..256-byte row segments, and the fused SwiGLU backward reads
    // g / u the same way.  The epilogues of gate/up and dgrad_act are bound by their vector instructions (some 130
    // VALU cycles per element before this form), so what counts here is instructions per element: packed conversions,
    // wave-uniform base pointers with one 32-bit lane offset, and a copy of every pass without bounds tests for the
    // passes whose 32 rows and whose tile columns all exist.
    // ------------------------------------------------------------------------------------------
    if (kCanSplit && tc.pieces > 1) {
        // a piece of a split tile: the fp32 accumulators go to the workspace as they are; ffn_mfma_fixup_kernel adds the
        // pieces up in a fixed order and applies the epilogue
        float* w = p.ws + (int64_t)tc.ws_slot * (BM * BN);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int row = wm * 128 + i * 16 + l15;
            if (row < tc.rows) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) *(f32x4_t*)(w + row * BN + wn * CW + j * 16 + 4 * g4) = acc[i][j];
            }
        }
        return;
    }
    int valid_rows = tc.rows;
    int64_t out_row0 = tc.row0;
    if (MODE == kWgrad) {
        const int64_t left = p.M - (int64_t)tc.m_tile * BM;
        valid_rows = left < BM ? (int)left : BM;
        out_row0 = (int64_t)tc.e * p.M + (int64_t)tc.m_tile * BM;
    }
    constexpr int kEpiCols = MODE == kGateUp ? CW / 2 : CW;  // output columns per wave and pass
    constexpr int kEpiStride = (kEpiCols + 8) * 2;        // bytes; the 16-byte pad rotates rows over the banks
    char* epi = lds + wave * (32 * kEpiStride);
    constexpr int kChunksPerRow = kEpiCols / 8;
    constexpr int kReadIters = 32 * kChunksPerRow / 64;
    static_assert(kReadIters >= 1, "a pass must cover at least one chunk per lane");
    constexpr int kRowsPerIt = 64 / kChunksPerRow;  // rows of a pass that one read-back iteration covers
    // the 16-byte chunk this lane reads back and stores: row c_row + it * kRowsPerIt of the pass, columns c_col .. +7 of the
    // wave's columns
    const int c_row = lane / kChunksPerRow;
    const int c_col = (lane % kChunksPerRow) * 8;
    auto lo16 = [](uint32_t v) { return __uint_as_float(v << 16); };
    auto hi16 = [](uint32_t v) { return __uint_as_float(v & 0xFFFF0000u); };
    auto pack4 = [](const f32x4_t& v) { return u32x2_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])}; };
    // packed(b, j) -> the four bf16 of 16-row block b (0, 1) of the pass and 16-column block j of the wave's pass columns
    auto stage_block = [&](auto packed) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // earlier read-backs of this slice are done
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int j = 0; j < kEpiCols / 16; ++j)
                *(u32x2_t*)(epi + (b * 16 + l15) * kEpiStride + (j * 16 + 4 * g4) * 2) = packed(b, j);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    // the same for a 32 x 32 block row; packed(j, q): 32-column block j, column group q
    auto stage_block_wide = [&](auto packed) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int j = 0; j < kEpiCols / 32; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *(u32x2_t*)(epi + (lane & 31) * kEpiStride + (j * 32 + 8 * q + 4 * (lane >> 5)) * 2) = packed(j, q);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    auto read_chunk = [&](int it) { return *(const u32x4_t*)(epi + (it * kRowsPerIt + c_row) * kEpiStride + c_col * 2); };
    // pass i (0..3) covers tile rows wm*128 + 32i .. +31
    auto pass_live = [&](int i) { return wm * 128 + i * 32 < valid_rows; };  // wave-uniform
    const bool cols_full = (int64_t)(tc.n_tile + 1) * (MODE == kGateUp ? BN / 2 : BN) <= p.N;
    // f(std::true_type) when every row of pass i and every column of the tile exists, f(std::false_type) otherwise
    auto with_fullness = [&](int i, auto f) {
        if (cols_full && wm * 128 + i * 32 + 32 <= valid_rows) f(std::true_type{});
        else f(std::false_type{});
    };
    auto row_ok = [&](int i, int it) { return wm * 128 + i * 32 + it * kRowsPerIt + c_row < valid_rows; };

    if (MODE == kGateUp) {
        const int64_t I = p.N;
        const int64_t col0 = (int64_t)tc.n_tile * 128 + wn * (CW / 2);
        // (I is a multiple of 8: a 16-byte chunk lies inside the row or past its end as a whole)
        const bool col_ok = col0 + c_col < I;
        const uint32_t off_act = (uint32_t)((c_row * (int)I + c_col) * 2);      // the lane's chunk in iteration 0, bytes
        const uint32_t off_gu = (uint32_t)((c_row * 2 * (int)I + c_col) * 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (!pass_live(i)) continue;  // wave-uniform: a block of rows past the segment has nothing to store
            // g and u rounded to bf16 (what the reference's two Linear outputs hold), kept as packed pairs: column blocks
            // 0, 1 of the wave hold g, blocks 2, 3 the u of the same output columns
            u32x2_t gb[2][NJ / 2], ub[2][NJ / 2];
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int j = 0; j < NJ / 2; ++j) {
                    gb[b][j] = pack4(acc[2 * i + b][j]);
                    ub[b][j] = pack4(acc[2 * i + b][j + NJ / 2]);
                }
            stage_block([&](int b, int j) {
                u32x2_t o;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float g0 = lo16(gb[b][j][h]), g1 = hi16(gb[b][j][h]);
                    const uint32_t s = pack_bf16x2(g0 * sigmoid_fast(g0), g1 * sigmoid_fast(g1));  // silu(g), rounded
                    o[h] = pack_bf16x2(lo16(s) * lo16(ub[b][j][h]), hi16(s) * hi16(ub[b][j][h]));
                }
                return o;
            });
            with_fullness(i, [&](auto full) {
                constexpr bool kFull = decltype(full)::value;
                const int64_t r0 = out_row0 + wm * 128 + i * 32;
                char* act_base = (char*)(p.out + r0 * I + col0);
#pragma unroll
                for (int it = 0; it < kReadIters; ++it)
                    if (kFull || (row_ok(i, it) && col_ok))
                        *(u32x4_t*)(act_base + (int64_t)it * kRowsPerIt * I * 2 + off_act) = read_chunk(it);
                if (p.out2) {
                    char* gu_base = (char*)(p.out2 + r0 * 2 * I + col0);
                    stage_block([&](int b, int j) { return gb[b][j]; });
#pragma unroll
                    for (int it = 0; it < kReadIters; ++it)
                        if (kFull || (row_ok(i, it) && col_ok))
                            *(u32x4_t*)(gu_base + (int64_t)it * kRowsPerIt * I * 4 + off_gu) = read_chunk(it);
                    stage_block([&](int b, int j) { return ub[b][j]; });
#pragma unroll
                    for (int it = 0; it < kReadIters; ++it)
                        if (kFull || (row_ok(i, it) && col_ok))
                            *(u32x4_t*)(gu_base + I * 2 + (int64_t)it * kRowsPerIt * I * 4 + off_gu) = read_chunk(it);
                }
            });
        }
    } else if (MODE == kDgradAct) {
        const int64_t I = p.N;
        const int64_t col0 = (int64_t)tc.n_tile * BN + wn * CW;
        const bool col_ok = col0 + c_col < I;
        const uint32_t off2 = (uint32_t)((c_row * 2 * (int)I + c_col) * 2);  // in the [.., 2I] tensors, bytes
        const uint32_t off1 = (uint32_t)((c_row * (int)I + c_col) * 2);      // in act_out
        const bool want_act = p.out2 != nullptr;  // the recomputed activation is only worked out when asked for
        // the [g | u] chunks of a pass are loaded one pass ahead, into two register sets
        u32x4_t gq[2][kReadIters], uq[2][kReadIters];
        auto load_gu = [&](int i) {
            with_fullness(i, [&](auto full) {
                constexpr bool kFull = decltype(full)::value;
                const char* base = (const char*)(p.aux + (out_row0 + wm * 128 + i * 32) * 2 * I + col0);
#pragma unroll
                for (int it = 0; it < kReadIters; ++it)
                    if (kFull || (row_ok(i, it) && col_ok)) {
                        gq[i & 1][it] = *(const u32x4_t*)(base + (int64_t)it * kRowsPerIt * I * 4 + off2);
                        uq[i & 1][it] = *(const u32x4_t*)(base + I * 2 + (int64_t)it * kRowsPerIt * I * 4 + off2);
                    }
            });
        };
        if (pass_live(0)) load_gu(0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (!pass_live(i)) continue;
            if (i + 1 < 4 && pass_live(i + 1)) load_gu(i + 1);
            stage_block([&](int b, int j) { return pack4(acc[2 * i + b][j]); });  // da, rounded to bf16
            with_fullness(i, [&](auto full) {
                constexpr bool kFull = decltype(full)::value;
                const int64_t r0 = out_row0 + wm * 128 + i * 32;
                char* out_base = (char*)(p.out + r0 * 2 * I + col0);
                char* act_base = (char*)(p.out2 + r0 * I + col0);
#pragma unroll
                for (int it = 0; it < kReadIters; ++it) {
                    if (!(kFull || (row_ok(i, it) && col_ok))) continue;
                    const u32x4_t v = read_chunk(it), gv = gq[i & 1][it], uv = uq[i & 1][it];
                    u32x4_t dgv, duv;
                    float gs8[8];  // silu(g), for the activation
#pragma unroll
                    for (int w2 = 0; w2 < 4; ++w2) {
                        float o_dg[2], o_du[2];
#pragma unroll
                        for (int h2 = 0; h2 < 2; ++h2) {
                            const float da = h2 ? hi16(v[w2]) : lo16(v[w2]);
                            const float g = h2 ? hi16(gv[w2]) : lo16(gv[w2]);
                            const float u = h2 ? hi16(uv[w2]) : lo16(uv[w2]);
                            const float sig = sigmoid_fast(g);
                            const float gs = g * sig;
                            o_dg[h2] = da * u * (sig + gs * (1.f - sig));
                            o_du[h2] = da * gs;
                            gs8[2 * w2 + h2] = gs;
                        }
                        dgv[w2] = pack_bf16x2(o_dg[0], o_dg[1]);
                        duv[w2] = pack_bf16x2(o_du[0], o_du[1]);
                    }
                    *(u32x4_t*)(out_base + (int64_t)it * kRowsPerIt * I * 4 + off2) = dgv;
                    *(u32x4_t*)(out_base + I * 2 + (int64_t)it * kRowsPerIt * I * 4 + off2) = duv;
                    if (want_act) {  // one branch per chunk, after its stores
                        u32x4_t av;
#pragma unroll
                        for (int w2 = 0; w2 < 4; ++w2) {
                            const uint32_t sl = pack_bf16x2(gs8[2 * w2], gs8[2 * w2 + 1]);  // silu(g), rounded
                            av[w2] = pack_bf16x2(lo16(sl) * lo16(uv[w2]), hi16(sl) * hi16(uv[w2]));
                        }
                        *(u32x4_t*)(act_base + (int64_t)it * kRowsPerIt * I * 2 + off1) = av;
                    }
                }
            });
        }
    } else {
        const int64_t col0 = (int64_t)tc.n_tile * BN + wn * CW;
        const bool col_ok = col0 + c_col < p.N;
        const uint32_t off = (uint32_t)((c_row * (int)p.ldo + c_col) * 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (!pass_live(i)) continue;
            if (kWide) {
                stage_block_wide([&](int j, int q) {
                    return u32x2_t{pack_bf16x2(accw[i][j][4 * q], accw[i][j][4 * q + 1]), pack_bf16x2(accw[i][j][4 * q + 2], accw[i][j][4 * q + 3])};
                });
            } else {
                stage_block([&](int b, int j) { return pack4(acc[2 * i + b][j]); });
            }
            with_fullness(i, [&](auto full) {
                constexpr bool kFull = decltype(full)::value;
                const int64_t r0 = out_row0 + wm * 128 + i * 32;
                char* out_base = (char*)(p.out + r0 * p.ldo + col0);
#pragma unroll
                for (int it = 0; it < kReadIters; ++it) {
                    if (!(kFull || (row_ok(i, it) && col_ok))) continue;
                    u32x4_t v = read_chunk(it);
                    if (MODE == kDown && p.aux) {
                        const float rw = bf16_bits_to_f32(p.aux[r0 + it * kRowsPerIt + c_row]);
#pragma unroll
                        for (int w2 = 0; w2 < 4; ++w2) v[w2] = pack_bf16x2(lo16(v[w2]) * rw, hi16(v[w2]) * rw);
                    }
                    *(u32x4_t*)(out_base + (int64_t)it * kRowsPerIt * p.ldo * 2 + off) = v;
                }
            });
        }
    }
}

// Second pass of a split last round: the blocks (b, y) add up the fp32 pieces of remainder tile b / 8 of XCD b % 8 (in
// piece order, so the result does not depend on timing) and apply the epilogue of the unsplit kernel to the sums:
//   down, dgrad_x: rounded to the output type; down: times the row weight, rounded again;
//   gate/up:       g and u rounded, act = silu(g) * u, [g | u] stored when asked for (the partial tile holds, per 64 columns
//                  of a wave, 32 gate columns and then the 32 up columns of the same FFN columns: lane l + 8 holds the u of lane l's g);
//   dgrad_act:     da rounded, then the SwiGLU backward at [g | u].
// Block (b, y) takes rows 32y .. 32y + 31 of the tile, eight per wavefront, four columns per lane, and issues the loads of all
// its rows and pieces before it adds: one block per tile walking its 256 rows took 20-75 us, the time of a load's latency per row.
constexpr int kFixupRows = 32;
template <int MODE>
__global__ __launch_bounds__(256) void ffn_mfma_fixup_kernel(MfmaParams p) {
    const GroupedLayout g = grouped_layout(p.counts, p.E, p.n_tiles, p.max_pieces);
    const int t = blockIdx.x / kNumXcd, xcd = blockIdx.x % kNumXcd;
    if (g.pieces <= 1 || t >= g.rem) return;
    TileCoord tc;
    if (!locate_tile_slot(p.counts, p.E, p.n_tiles, g, xcd, g.full + t, &tc)) return;
    const float* w = p.ws + (int64_t)(xcd * kCusPerXcd + t * g.pieces) * (BM * BN);
    const int lane = threadIdx.x & 63;
    const int c4 = lane * 4;  // column of the partial tile
    // output column of the lane's four values, and whether it exists (N is a multiple of 8)
    const int64_t out_col = MODE == kGateUp ? (int64_t)tc.n_tile * 128 + (lane >> 4) * 32 + (lane & 7) * 4 : (int64_t)tc.n_tile * BN + c4;
    const bool col_ok = out_col < p.N;
    if (MODE != kGateUp && !col_ok) return;  // (gate/up keeps every lane: the u values travel between lanes below)
    constexpr int kRowsPerWave = kFixupRows / 4;
    const int row0 = blockIdx.y * kFixupRows + (threadIdx.x >> 6) * kRowsPerWave;
    f32x4_t v[kRowsPerWave][kMaxSplit];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
        for (int pc = 0; pc < kMaxSplit; ++pc) {
            const bool live = row0 + r < tc.rows && pc < g.pieces;
            v[r][pc] = live ? *(const f32x4_t*)(w + (int64_t)pc * (BM * BN) + (row0 + r) * BN + c4) : f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
    auto round_bf16 = [](float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); };
    auto store4 = [](uint16_t* dst, const float (&x)[4]) {
        *(uint64_t*)dst = (uint64_t)pack_bf16x2(x[0], x[1]) | ((uint64_t)pack_bf16x2(x[2], x[3]) << 32);
    };
    auto load4 = [](const uint16_t* src, float (&x)[4]) {
        const uint64_t bits = *(const uint64_t*)src;
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] = bf16_bits_to_f32((uint32_t)(bits >> (16 * i)) & 0xFFFFu);
    };
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int row = row0 + r;
        if (row >= tc.rows) break;  // wave-uniform
        float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int pc = 0; pc < kMaxSplit; ++pc) {  // pieces past g.pieces hold zeros: x + 0 leaves every sum as it is
#pragma unroll
            for (int i = 0; i < 4; ++i) s[i] += v[r][pc][i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] = round_bf16(s[i]);
        const int64_t grow = tc.row0 + row;
        if (MODE == kGateUp) {
            const int64_t I = p.N;
            float u[4], a[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) u[i] = __shfl(s[i], (lane + 8) & 63, 64);
            if ((lane & 8) == 0 && col_ok) {  // the lanes that hold g
#pragma unroll
                for (int i = 0; i < 4; ++i) a[i] = round_bf16(s[i] * sigmoid_fast(s[i])) * u[i];
                store4(p.out + grow * I + out_col, a);
                if (p.out2) {
                    store4(p.out2 + grow * 2 * I + out_col, s);
                    store4(p.out2 + grow * 2 * I + I + out_col, u);
                }
            }
        } else if (MODE == kDgradAct) {
            const int64_t I = p.N;
            float gv[4], uv[4], dg[4], du[4], a[4];
            load4(p.aux + grow * 2 * I + out_col, gv);
            load4(p.aux + grow * 2 * I + I + out_col, uv);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float sig = sigmoid_fast(gv[i]);
                const float gs = gv[i] * sig;
                dg[i] = s[i] * uv[i] * (sig + gs * (1.f - sig));
                du[i] = s[i] * gs;
                a[i] = round_bf16(gs) * uv[i];
            }
            store4(p.out + grow * 2 * I + out_col, dg);
            store4(p.out + grow * 2 * I + I + out_col, du);
            if (p.out2) store4(p.out2 + grow * I + out_col, a);
        } else {
            if (MODE == kDown && p.aux) {
                const float rw = bf16_bits_to_f32(p.aux[grow]);
#pragma unroll
                for (int i = 0; i < 4; ++i) s[i] *= rw;
            }
            store4(p.out + grow * p.ldo + out_col, s);
        }
    }
}

// how many pieces the tiles of the last round may be cut into: none without the workspace, and none below 16 k-tiles a piece.
// `rich_epilogue`: gate/up and dgrad_act, whose second pass redoes a SwiGLU epilogue over three (two) outputs per element and whose
// pieces each park 256 KB of fp32 where the whole tile stores 192 KB of bf16: measured, the split pays for them from 64 k-tiles on
// (hidden 4096: -1...2 % on ragged counts) and costs up to 20 % at 32 (hidden 2048, two pieces of 16 k-steps), so they split only
// when four pieces are possible.
int split_pieces(const void* ws, int64_t ws_bytes, int64_t k_tiles, bool rich_epilogue = false) {
    if (!ws || ws_bytes < kSplitWorkspaceBytes) return 1;
    const int64_t by_k = k_tiles / 16;
    if (rich_epilogue) return by_k >= kMaxSplit ? kMaxSplit : 1;
    return by_k >= kMaxSplit ? kMaxSplit : (by_k >= 2 ? 2 : 1);
}

MfmaParams base_params(const FfnShape& s) {
    MfmaParams p{};
    p.counts = s.counts;
    p.E = s.E;
    p.n_rows = s.n_rows;
    p.max_pieces = 1;
    return p;
}

}  // namespace

int64_t ffn_mfma_workspace_bytes() { return kSplitWorkspaceBytes; }

bool ffn_mfma_supported(const FfnShape& s) {
    // Both H and I are a contraction length somewhere (k-tiles of 64, no K tail except wgrad's); as output widths they
    // only need whole 16-byte chunks, the tiles that reach past the last column clamp their loads and mask their stores.
    return s.dtype == PICOMOE_BF16 && s.H % 64 == 0 && s.I % 64 == 0 && s.H >= 128 && s.I >= 128;
}

int ffn_mfma_gate_up(const FfnShape& s, const void* x, const void* gate_w, const void* up_w, void* act, void* inter13,
                     void* ws, int64_t ws_bytes, hipStream_t st) {
    MfmaParams p = base_params(s);
    p.K = s.H; p.N = s.I; p.n_tiles = (int)((s.I + 127) / 128);
    p.A = (const uint16_t*)x; p.lda = s.H;
    p.B0 = (const uint16_t*)gate_w; p.B1 = (const uint16_t*)up_w; p.ldb = s.H; p.b_expert_stride = s.I * s.H;
    p.out = (uint16_t*)act; p.ldo = s.I; p.out2 = (uint16_t*)inter13;
    p.ws = (float*)ws; p.max_pieces = split_pieces(ws, ws_bytes, p.K / BK, true);
    hipLaunchKernelGGL((ffn_mfma_kernel<kGateUp, kWaves>), dim3(grid_m_grouped(s, p.n_tiles, p.max_pieces > 1)), dim3(kWaves * 64), 0, st, p);
    if (p.max_pieces > 1)
        hipLaunchKernelGGL((ffn_mfma_fixup_kernel<kGateUp>), dim3(kNumXcd * (kCusPerXcd / 2), BM / kFixupRows), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

int ffn_mfma_down(const FfnShape& s, const void* act, const void* down_w, const void* row_weight, void* y, void* ws,
                  int64_t ws_bytes, hipStream_t st) {
    MfmaParams p = base_params(s);
    p.K = s.I; p.N = s.H; p.n_tiles = (int)((s.H + BN - 1) / BN);
    p.A = (const uint16_t*)act; p.lda = s.I;
    p.B0 = (const uint16_t*)down_w; p.ldb = s.I; p.b_expert_stride = s.H * s.I;
    p.out = (uint16_t*)y; p.ldo = s.H; p.aux = (const uint16_t*)row_weight;
    p.ws = (float*)ws; p.max_pieces = split_pieces(ws, ws_bytes, p.K / BK);
    hipLaunchKernelGGL((ffn_mfma_kernel<kDown, kWaves>), dim3(grid_m_grouped(s, p.n_tiles, p.max_pieces > 1)), dim3(kWaves * 64), 0, st, p);
    if (p.max_pieces > 1)
        hipLaunchKernelGGL((ffn_mfma_fixup_kernel<kDown>), dim3(kNumXcd * (kCusPerXcd / 2), BM / kFixupRows), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

int ffn_mfma_dgrad_act(const FfnShape& s, const void* dy, const void* down_w, const void* inter13, void* d_inter13,
                       void* act_out, void* ws, int64_t ws_bytes, hipStream_t st) {
    MfmaParams p = base_params(s);
    p.K = s.H; p.N = s.I; p.n_tiles = (int)((s.I + BN - 1) / BN);
    p.A = (const uint16_t*)dy; p.lda = s.H;
    p.B0 = (const uint16_t*)down_w; p.ldb = s.I; p.b_expert_stride = s.H * s.I;  // down_w[e] read as [K = H][N = I]
    p.out = (uint16_t*)d_inter13; p.ldo = 2 * s.I; p.out2 = (uint16_t*)act_out; p.aux = (const uint16_t*)inter13;
    p.ws = (float*)ws; p.max_pieces = split_pieces(ws, ws_bytes, p.K / BK, true);
    hipLaunchKernelGGL((ffn_mfma_kernel<kDgradAct, kWaves>), dim3(grid_m_grouped(s, p.n_tiles, p.max_pieces > 1)), dim3(kWaves * 64), 0, st, p);
    if (p.max_pieces > 1)
        hipLaunchKernelGGL((ffn_mfma_fixup_kernel<kDgradAct>), dim3(kNumXcd * (kCusPerXcd / 2), BM / kFixupRows), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

int ffn_mfma_dgrad_x(const FfnShape& s, const void* d_inter13, const void* gate_w, const void* up_w, void* dx, void* ws,
                     int64_t ws_bytes, hipStream_t st) {
    MfmaParams p = base_params(s);
    p.K = 2 * s.I; p.N = s.H; p.n_tiles = (int)((s.H + BN - 1) / BN);
    p.A = (const uint16_t*)d_inter13; p.lda = 2 * s.I;
    p.B0 = (const uint16_t*)gate_w; p.B1 = (const uint16_t*)up_w; p.ldb = s.H; p.b_expert_stride = s.I * s.H;  // [K = I][N = H]
    p.out = (uint16_t*)dx; p.ldo = s.H;
    p.ws = (float*)ws; p.max_pieces = split_pieces(ws, ws_bytes, p.K / BK);
    hipLaunchKernelGGL((ffn_mfma_kernel<kDgradX, kWaves>), dim3(grid_m_grouped(s, p.n_tiles, p.max_pieces > 1)), dim3(kWaves * 64), 0, st, p);
    if (p.max_pieces > 1)
        hipLaunchKernelGGL((ffn_mfma_fixup_kernel<kDgradX>), dim3(kNumXcd * (kCusPerXcd / 2), BM / kFixupRows), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

bool ffn_mfma_wgrad_supported(int dtype, int64_t P, int64_t Q, int64_t ld_lhs, int64_t ld_rhs, const void* lhs,
                              const void* rhs) {
    return dtype == PICOMOE_BF16 && P % 8 == 0 && Q % 8 == 0 && P >= 128 && Q >= 128 && ld_lhs % 8 == 0 &&
           ld_rhs % 8 == 0 && (uintptr_t)lhs % 16 == 0 && (uintptr_t)rhs % 16 == 0;
}

int ffn_mfma_wgrad(const FfnShape& s, const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, int64_t P, int64_t Q,
                   void* out, hipStream_t st) {
    MfmaParams p = base_params(s);
    p.M = P; p.N = Q; p.m_tiles = (int)((P + BM - 1) / BM); p.n_tiles = (int)((Q + BN - 1) / BN);
    p.A = (const uint16_t*)lhs; p.lda = ld_lhs;
    p.B0 = (const uint16_t*)rhs; p.ldb = ld_rhs;
    p.out = (uint16_t*)out; p.ldo = Q;
    const int64_t tiles = (int64_t)s.E * p.m_tiles * p.n_tiles;
    hipLaunchKernelGGL((ffn_mfma_kernel<kWgrad, kWaves>), dim3(grid_wgrad(tiles)), dim3(kWaves * 64), 0, st, p);
    return picomoe_launch_status();
}
