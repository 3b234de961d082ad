// FP8 (E4M3) MFMA kernels for the forward projections of the expert FFN on gfx950 (MI355X): per-row quantised
// activations (codes + one fp32 scale per row: the FP8 dispatch's rows for gate/up, the quantised SwiGLU output for
// down) meet expert weights quantised the same way (one scale per output row) in v_mfma_f32_16x16x128_f8f6f4, fp32
// accumulation, and the two scales are applied to the accumulators in the epilogue -- fused with SwiGLU for gate/up,
// with the optional row weight for down.
//
// Same frame as the bf16 kernels: 256 x 256 block tile, 8 wavefronts (two per SIMD) of 128 x 64, two 64 KB LDS
// stages filled by 16-byte direct-to-LDS loads.  A 128-byte LDS row now holds 128 k values, which one MFMA consumes
// whole: a tile needs half as many k-steps, loads and barriers per FLOP.  A lane feeds an MFMA with 32 consecutive k
// bytes of its row (two ds_read_b128); which 32 of the 128 go to which lane group is free as long as both operands
// agree, because the instruction only sums over k.  (16 x 16 x 128 rather than 32 x 32 x 64: under the power cap a loop of
// nothing but MFMAs on random data runs 8 % faster with it.)
#include <type_traits>

#include "ffn.h"
#include "mfma_tiles.h"

namespace {

constexpr int kFp8Waves = 8;
constexpr int kFp8BK = 128;  // k values (bytes) per k-step
constexpr int kFp8PrefetchDist = 2;

typedef __attribute__((ext_vector_type(8))) int i32x8_t;

enum Fp8Mode { kFp8GateUp = 0, kFp8Down = 1 };

struct Fp8Params {
    const int64_t* counts;
    int E;
    int64_t n_rows;
    int64_t K;             // contraction length: H (gate/up) or I (down); row pitch in bytes of both operands
    int64_t N;             // output columns: I (gate/up) or H (down); weight rows per expert and matrix
    int n_tiles;
    const uint8_t* xq;     // [n_rows, K] e4m3 codes
    const float* x_scale;  // [n_rows]
    const uint8_t* gq;     // gate/up: gate_w codes [E, I, H]; down: down_w codes [E, H, I]
    const uint8_t* uq;     // gate/up: up_w codes; down: unused
    const float* g_scale;  // [E * N]
    const float* u_scale;
    uint16_t* act;         // gate/up: act [n_rows, I] bf16; down: y [n_rows, H] bf16
    uint16_t* inter13;     // gate/up: [n_rows, 2I] bf16 or null
    const uint16_t* row_weight;  // down: optional bf16 [n_rows], multiplied into the rounded output
};

template <int MODE>
__global__ __launch_bounds__(kFp8Waves * 64, 1) void ffn_fp8_kernel(Fp8Params p) {
    constexpr int NI = 8, NJ = 4, kWaveCols = 4, CW = 64, QN = 4, RPW = 32;
    __shared__ __attribute__((aligned(1024))) char lds[2 * kStageBytes];
    TileCoord tc;
    if (!locate_m_grouped(p.counts, p.E, p.n_tiles, blockIdx.x / kNumXcd, &tc)) return;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / kWaveCols, wn = wave % kWaveCols;
    const int l15 = lane & 15, g4 = lane >> 4;
    const int n_kt = (int)(p.K / kFp8BK);
    const bool wave_active = wm * 128 < tc.rows;

    // global -> LDS: wave w fills rows [32w, 32w + 32) of both tiles, 8 rows (128 B each) per instruction.  B tile,
    // gate/up: per wave column (64 rows) 32 gate rows then 32 up rows of the same FFN columns: even waves load gate rows;
    // down: 256 consecutive rows of down_w[e].
    uint32_t a_off[QN], b_off[QN];
    const char* a_base = (const char*)(p.xq + tc.row0 * p.K);
    const uint8_t* bmat = MODE == kFp8GateUp && (wave & 1) ? p.uq : p.gq;
    const int64_t brow0 = MODE == kFp8GateUp ? (int64_t)tc.n_tile * 128 + (wave >> 1) * 32 : (int64_t)tc.n_tile * BN + wave * RPW;
    const char* b_base = (const char*)(bmat + ((int64_t)tc.e * p.N + brow0) * p.K);
#pragma unroll
    for (int q = 0; q < QN; ++q) {
        const int r = wave * RPW + q * 8 + (lane >> 3);
        const int ar = r < tc.rows ? r : tc.rows - 1;  // rows past the segment re-read its last row (never stored)
        a_off[q] = (uint32_t)(ar * (int)p.K + ((lane & 7) ^ swz(r)) * 16);
        b_off[q] = (uint32_t)((q * 8 + (lane >> 3)) * (int)p.K + ((lane & 7) ^ swz(r)) * 16);
    }
    // one load instruction (q of QN) of this wave for the A or the B tile of k-tile kt.  Opaque loads: the waits between
    // a load and the LDS reads of its data are the explicit ones below (prologue, k-loop barrier, end of the loop).
    auto issue_a = [&](int kt, int stage, int q) {
        load16_to_lds_opaque(a_base + (int64_t)kt * kFp8BK, a_off[q], lds + stage * kStageBytes + (wave * RPW + q * 8) * 128);
    };
    auto issue_b = [&](int kt, int stage, int q) {
        load16_to_lds_opaque(b_base + (int64_t)kt * kFp8BK, b_off[q], lds + stage * kStageBytes + kTileBytes + (wave * RPW + q * 8) * 128);
    };
    auto issue_tile = [&](int kt, int stage) {
#pragma unroll
        for (int q = 0; q < QN; ++q) {
            issue_a(kt, stage, q);
            issue_b(kt, stage, q);
        }
    };

    // the first two k-tiles go out before the rest of the set-up (prefetch pointer, fragment addresses, zeroed accumulators)
    if (n_kt > 0) {
        issue_tile(0, 0);
        if (n_kt > 1) issue_tile(1, 1);
    }

    // L2 prefetch, as in the bf16 kernels: every k-step each wave touches (one 4-byte load per 128-byte line into a register
    // nobody reads) its share of the lines of an operand slice kFp8PrefetchDist k-steps ahead -- the first half of the waves lines
    // of the A slice, the second half lines of the B slice -- so that the demand loads of the tiles that share the slice do not
    // queue behind the same misses.
    const char* pf_cur;
    {
        const bool pf_b = wave >= kFp8Waves / 2;
        const int q = (wave % (kFp8Waves / 2)) * 64 + lane;
        const int si = pf_b ? tc.b_si : tc.a_si, sn = pf_b ? tc.b_sn : tc.a_sn;
        int j = sn > 1 ? si + sn * q : q;  // line of the 256-line slice (one line per row)
        if (j >= 256) j = si;
        if (!pf_b) {
            const int r = j < tc.rows ? j : tc.rows - 1;
            pf_cur = (const char*)(p.xq + (tc.row0 + r) * p.K);
        } else if (MODE == kFp8GateUp) {
            const uint8_t* m = j < 128 ? p.gq : p.uq;
            pf_cur = (const char*)(m + ((int64_t)tc.e * p.N + (int64_t)tc.n_tile * 128 + (j & 127)) * p.K);
        } else {
            pf_cur = (const char*)(p.gq + ((int64_t)tc.e * p.N + (int64_t)tc.n_tile * BN + j) * p.K);
        }
        const int kt0 = kFp8PrefetchDist < n_kt ? kFp8PrefetchDist : (n_kt > 0 ? n_kt - 1 : 0);
        pf_cur += (int64_t)kt0 * kFp8BK;
    }
    // the touch in front of the loop takes k-tile kFp8PrefetchDist, the one of k-step kt k-tile kt + kFp8PrefetchDist + 1 (its operand
    // loads go out a k-step later); past the last k-tile the pointer stays where it is
    int pf_kt = kFp8PrefetchDist;
    auto prefetch_l2 = [&]() {
        asm volatile("global_load_dword v255, %0, off" ::"v"(pf_cur) : "v255", "memory");
        ++pf_kt;
        if (pf_kt < n_kt) pf_cur += kFp8BK;
    };

    // LDS -> fragments.  An MFMA takes all 128 k values of a row: lane (row l & 15 of a 16-row block, k group l >> 4)
    // supplies the 32 bytes of k group l >> 4, the 16-byte chunks 2*(l >> 4) and 2*(l >> 4) + 1 of its row; with the XOR
    // swizzle the second is the address of the first XOR 16.  The swizzle depends on (row >> 1) & 7 only, which is the
    // same in every 16-row block: one address register per operand, block b at + b * 2048.
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
    const int ra = wm * 128 + l15, rb = wn * CW + l15;
    uint32_t a_ad = lds0 + ra * 128 + (((2 * g4) ^ swz(ra)) << 4);
    uint32_t b_ad = lds0 + kTileBytes + rb * 128 + (((2 * g4) ^ swz(rb)) << 4);
    auto flip_stage = [&]() {
        a_ad ^= (uint32_t)kStageBytes;
        b_ad ^= (uint32_t)kStageBytes;
    };
    auto read_frag = [&](uint32_t ad) -> i32x8_t {
        const u32x4_t lo = *(__attribute__((address_space(3))) const u32x4_t*)(uintptr_t)ad;
        const u32x4_t up = *(__attribute__((address_space(3))) const u32x4_t*)(uintptr_t)(ad ^ 16u);
        i32x8_t v;
        v[0] = (int)lo[0]; v[1] = (int)lo[1]; v[2] = (int)lo[2]; v[3] = (int)lo[3];
        v[4] = (int)up[0]; v[5] = (int)up[1]; v[6] = (int)up[2]; v[7] = (int)up[3];
        return v;
    };

    f32x4_t acc[NI][NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    // A k-step is two halves of 16 MFMAs: rows 0..63 of the wave's 128 (A blocks 0..3), then rows 64..127 (blocks 4..7),
    // each against the four B blocks.  af[h] holds the four A fragments of half h, bfr the B fragments of the k-tile.
    i32x8_t af[2][4], bfr[NJ];
    auto read_a = [&](int h, int i) { af[h][i] = read_frag(a_ad + (4 * h + i) * 2048); };
    auto read_b = [&](int j) { bfr[j] = read_frag(b_ad + j * 2048); };
    // the 16 MFMAs (32 cycles each) of half h, B block by B block (the B fragment first: the block comes out transposed,
    // four neighbouring columns of a row per lane, as the epilogue stages them), with side(n) run after MFMA n: the slots for LDS
    // reads and loads.  After MFMA 4j + 3 nothing in this k-step needs bfr[j] any more.
    auto mma_with = [&](int h, auto active, auto side) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (decltype(active)::value)
                    acc[4 * h + i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bfr[j], af[h][i], acc[4 * h + i][j], 0, 0, 0, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                side(j * 4 + i);
                __builtin_amdgcn_sched_barrier(0);
            }
    };

    if (n_kt > 0) {
        if (n_kt > 1) {
            prefetch_l2();  // from here on the youngest load in flight is always a prefetch touch
            __builtin_amdgcn_s_waitcnt(0x0F79);  // vmcnt(9): tile 0 has landed, tile 1 and the touch may still be in flight
        } else {
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        __syncthreads();
        if (wave_active) {
#pragma unroll
            for (int i = 0; i < 4; ++i) read_a(0, i);
#pragma unroll
            for (int j = 0; j < NJ; ++j) read_b(j);
        }
    }
    // One k-step.  First half: its MFMAs with the reads of the second half's A fragments between them; then every wave
    // holds its last fragments of this stage in registers, waits for its loads of the next k-tile (issued a whole k-step
    // ago) and meets the others at the barrier.  Second half: its MFMAs with all 8 loads of k-tile kt+2 into the stage just
    // vacated, one after each of the first eight MFMAs (issued right after the barrier they have the longest time to
    // land), and the fragment reads of k-tile kt+1 from the other stage: the first half's A fragments after MFMAs 8..11,
    // B block j after MFMA 4j + 3, the last MFMA of the k-step that multiplies by the old one.
    auto k_loop = [&](auto active) {
        constexpr bool kActive = decltype(active)::value;
        for (int kt = 0; kt < n_kt; ++kt) {
            const int stage = kt & 1;
            const int kt_load = kt + 2 < n_kt ? kt + 2 : n_kt - 1;  // clamped past the end: lands in a dead stage
            mma_with(0, active, [&](int n) {
                if (kActive && (n & 1) == 0 && n < 8) read_a(1, n >> 1);
            });
            __builtin_amdgcn_s_waitcnt(0x0F71);  // the operand loads of a k-step ago have landed; the prefetch touch issued after them may stay in flight
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            flip_stage();
            mma_with(1, active, [&](int n) {
                if (n < 8) {
                    if ((n & 1) == 0) issue_a(kt_load, stage, n >> 1);
                    else issue_b(kt_load, stage, n >> 1);
                }
                // past the last tile these read a stage that is not used any more
                if (kActive && (n & 3) == 3) read_b(n >> 2);
                if (kActive && n >= 8 && n < 12) read_a(0, n - 8);
                if (n == 13) prefetch_l2();
            });
        }
    };
    if (wave_active) k_loop(std::true_type{});
    else k_loop(std::false_type{});
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    // epilogue: the two scales, rounding to bf16, and 32 rows at a time through a wave-private slice of LDS so that the
    // stores are 16-byte lanes of contiguous rows.  The MFMAs take the B fragment as their first operand, so a lane holds
    // row (l & 15) of each 16-row block and the four neighbouring columns 4*(l >> 4) .. +3 of each 16-column block: one
    // row scale per block, four column scales per column block, two packed conversions and one 8-byte LDS write per
    // four values.  (Widths are whole tiles here -- ffn_fp8_supported -- so only rows need bounds.)
    float* row_scale = (float*)(lds + kStageBytes);  // 256 floats, past the staging slices
    if (tid < BM) row_scale[tid] = p.x_scale[tc.row0 + (tid < tc.rows ? tid : tc.rows - 1)];
    constexpr int kEpiCols = MODE == kFp8GateUp ? CW / 2 : CW;
    constexpr int kEpiStride = (kEpiCols + 8) * 2;
    char* epi = lds + wave * (32 * kEpiStride);
    constexpr int kChunksPerRow = kEpiCols / 8;
    constexpr int kReadIters = 32 * kChunksPerRow / 64;
    constexpr int kRowsPerIt = 64 / kChunksPerRow;
    const int c_row = lane / kChunksPerRow;        // the 16-byte chunk this lane reads back: row c_row + it * kRowsPerIt of the pass,
    const int c_col = (lane % kChunksPerRow) * 8;  // columns c_col .. +7 of the wave's columns
    auto lo16 = [](uint32_t v) { return __uint_as_float(v << 16); };
    auto hi16 = [](uint32_t v) { return __uint_as_float(v & 0xFFFF0000u); };
    auto pack4 = [](const f32x4_t& v) { return u32x2_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])}; };
    auto stage_block = [&](auto packed) {  // packed(b, j): the four bf16 of 16-row block b of the 32 rows and 16-column block j
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int j = 0; j < kEpiCols / 16; ++j)
                *(u32x2_t*)(epi + (b * 16 + l15) * kEpiStride + (j * 16 + 4 * g4) * 2) = packed(b, j);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    auto read_chunk = [&](int it) { return *(const u32x4_t*)(epi + (it * kRowsPerIt + c_row) * kEpiStride + c_col * 2); };
    auto pass_live = [&](int i) { return wm * 128 + i * 32 < tc.rows; };  // wave-uniform
    auto row_ok = [&](int i, int it) { return wm * 128 + i * 32 + it * kRowsPerIt + c_row < tc.rows; };
    // f(std::true_type) when all 32 rows of pass i exist: that copy of the pass carries no bounds tests
    auto with_fullness = [&](int i, auto f) {
        if (wm * 128 + i * 32 + 32 <= tc.rows) f(std::true_type{});
        else f(std::false_type{});
    };
    if (MODE == kFp8GateUp) {
        // g and u rounded to bf16 (what the two Linear outputs of the reference hold), then SwiGLU.  B blocks 0, 1 of the
        // wave are its 32 gate columns, blocks 2, 3 the up columns of the same FFN columns.
        const int64_t I = p.N;
        const int64_t col0 = (int64_t)tc.n_tile * 128 + wn * (CW / 2);
        f32x4_t gs[2], us[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            gs[j] = *(const f32x4_t*)(p.g_scale + (int64_t)tc.e * I + col0 + j * 16 + 4 * g4);
            us[j] = *(const f32x4_t*)(p.u_scale + (int64_t)tc.e * I + col0 + j * 16 + 4 * g4);
        }
        __syncthreads();
        const uint32_t off_act = (uint32_t)((c_row * (int)I + c_col) * 2);
        const uint32_t off_gu = (uint32_t)((c_row * 2 * (int)I + c_col) * 2);
#pragma unroll
        for (int i = 0; i < NI / 2; ++i) {
            if (!pass_live(i)) continue;
            u32x2_t gb[2][2], ub[2][2];
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const float sx = row_scale[wm * 128 + i * 32 + b * 16 + l15];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    f32x4_t g, u;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        g[r] = acc[2 * i + b][j][r] * sx * gs[j][r];
                        u[r] = acc[2 * i + b][2 + j][r] * sx * us[j][r];
                    }
                    gb[b][j] = pack4(g);
                    ub[b][j] = pack4(u);
                }
            }
            stage_block([&](int b, int j) {
                u32x2_t o;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float g0 = lo16(gb[b][j][h]), g1 = hi16(gb[b][j][h]);
                    const uint32_t sl = pack_bf16x2(g0 * sigmoid_fast(g0), g1 * sigmoid_fast(g1));  // silu(g), rounded
                    o[h] = pack_bf16x2(lo16(sl) * lo16(ub[b][j][h]), hi16(sl) * hi16(ub[b][j][h]));
                }
                return o;
            });
            with_fullness(i, [&](auto full) {
                constexpr bool kFull = decltype(full)::value;
                const int64_t r0 = tc.row0 + wm * 128 + i * 32;
                char* act_base = (char*)(p.act + r0 * I + col0);
#pragma unroll
                for (int it = 0; it < kReadIters; ++it)
                    if (kFull || row_ok(i, it)) *(u32x4_t*)(act_base + (int64_t)it * kRowsPerIt * I * 2 + off_act) = read_chunk(it);
                if (p.inter13) {
                    char* gu_base = (char*)(p.inter13 + r0 * 2 * I + col0);
                    stage_block([&](int b, int j) { return gb[b][j]; });
#pragma unroll
                    for (int it = 0; it < kReadIters; ++it)
                        if (kFull || row_ok(i, it)) *(u32x4_t*)(gu_base + (int64_t)it * kRowsPerIt * I * 4 + off_gu) = read_chunk(it);
                    stage_block([&](int b, int j) { return ub[b][j]; });
#pragma unroll
                    for (int it = 0; it < kReadIters; ++it)
                        if (kFull || row_ok(i, it))
                            *(u32x4_t*)(gu_base + I * 2 + (int64_t)it * kRowsPerIt * I * 4 + off_gu) = read_chunk(it);
                }
            });
        }
    } else {
        // y = bf16(acc * row scale * column scale), times the row weight (rounded again) when there is one
        const int64_t H = p.N;
        const int64_t col0 = (int64_t)tc.n_tile * BN + wn * CW;
        f32x4_t ws[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) ws[j] = *(const f32x4_t*)(p.g_scale + (int64_t)tc.e * H + col0 + j * 16 + 4 * g4);
        __syncthreads();
        const uint32_t off = (uint32_t)((c_row * (int)H + c_col) * 2);
#pragma unroll
        for (int i = 0; i < NI / 2; ++i) {
            if (!pass_live(i)) continue;
            stage_block([&](int b, int j) {
                const float sx = row_scale[wm * 128 + i * 32 + b * 16 + l15];
                f32x4_t v;
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = acc[2 * i + b][j][r] * sx * ws[j][r];
                return pack4(v);
            });
            with_fullness(i, [&](auto full) {
                constexpr bool kFull = decltype(full)::value;
                const int64_t r0 = tc.row0 + wm * 128 + i * 32;
                char* out_base = (char*)(p.act + r0 * H + col0);
#pragma unroll
                for (int it = 0; it < kReadIters; ++it) {
                    if (!(kFull || row_ok(i, it))) continue;
                    u32x4_t v = read_chunk(it);
                    if (p.row_weight) {
                        const float rw = bf16_bits_to_f32(p.row_weight[r0 + it * kRowsPerIt + c_row]);
#pragma unroll
                        for (int w2 = 0; w2 < 4; ++w2) v[w2] = pack_bf16x2(lo16(v[w2]) * rw, hi16(v[w2]) * rw);
                    }
                    *(u32x4_t*)(out_base + (int64_t)it * kRowsPerIt * H * 2 + off) = v;
                }
            });
        }
    }
}

}  // namespace

bool ffn_fp8_supported(const FfnShape& s) { return s.H % 256 == 0 && s.I % 128 == 0 && s.H >= 256 && s.I >= 128; }

int ffn_fp8_gate_up(const FfnShape& s, const void* xq, const float* x_scale, const void* gq, const void* uq,
                    const float* g_scale, const float* u_scale, void* act, void* inter13, hipStream_t st) {
    Fp8Params p{};
    p.counts = s.counts; p.E = s.E; p.n_rows = s.n_rows; p.K = s.H; p.N = s.I; p.n_tiles = (int)(s.I / 128);
    p.xq = (const uint8_t*)xq; p.x_scale = x_scale;
    p.gq = (const uint8_t*)gq; p.uq = (const uint8_t*)uq; p.g_scale = g_scale; p.u_scale = u_scale;
    p.act = (uint16_t*)act; p.inter13 = (uint16_t*)inter13;
    hipLaunchKernelGGL(ffn_fp8_kernel<kFp8GateUp>, dim3(grid_m_grouped(s, p.n_tiles)), dim3(kFp8Waves * 64), 0, st, p);
    return picomoe_launch_status();
}

int ffn_fp8_down(const FfnShape& s, const void* actq, const float* act_scale, const void* dq, const float* d_scale,
                 const void* row_weight, void* y, hipStream_t st) {
    Fp8Params p{};
    p.counts = s.counts; p.E = s.E; p.n_rows = s.n_rows; p.K = s.I; p.N = s.H; p.n_tiles = (int)(s.H / BN);
    p.xq = (const uint8_t*)actq; p.x_scale = act_scale;
    p.gq = (const uint8_t*)dq; p.g_scale = d_scale;
    p.act = (uint16_t*)y; p.row_weight = (const uint16_t*)row_weight;
    hipLaunchKernelGGL(ffn_fp8_kernel<kFp8Down>, dim3(grid_m_grouped(s, p.n_tiles)), dim3(kFp8Waves * 64), 0, st, p);
    return picomoe_launch_status();
}
