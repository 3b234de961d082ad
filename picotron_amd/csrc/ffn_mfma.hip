// bf16 MFMA expert-FFN kernels for gfx950 (MI355X): grouped GEMMs over variable-length expert
// segments with the SwiGLU forward / backward fused into the epilogues.
//
// Block tile 256 x 256 x 64 (M x N x K), 4 wavefronts (one per SIMD), each owning a 128 x 128
// sub-tile as 4 x 4 v_mfma_f32_32x32x16_bf16 accumulators (256 fp32 per lane).  Operand tiles go
// HBM -> LDS with 16-byte direct-to-LDS loads (no staging registers), two LDS stages of 64 KB.
// LDS rows are 128 B (64 bf16 of K); the 16-byte chunk index is XOR-swizzled with the row so the
// ds_read_b128 fragment reads of 32 consecutive rows spread over all banks.  The swizzle is applied
// on the global-address side because a direct-to-LDS load always writes lane l at LDS base + 16*l.
//
// Tiles are enumerated on the device from counts[] (no host copy): expert by expert, N-tile by
// N-tile, M-tile fastest, and consecutive tiles are handed to the same XCD (block b runs on XCD
// b % 8) so that the blocks sharing an L2 share weight tiles.
#include "ffn.h"

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kTileBytesA = BM * BK * 2;  // 32 KB
constexpr int kTileBytesB = BN * BK * 2;  // 32 KB
constexpr int kStageBytes = kTileBytesA + kTileBytesB;
constexpr int kNumXcd = 8;

enum Mode { kGateUp = 0, kDown = 1 };

struct MfmaParams {
    const int64_t* counts;
    int E;
    int64_t n_rows;
    int64_t K;         // contraction length (H for gate/up, I for down)
    int64_t n_cols;    // output columns the N tiles cover (I for gate/up: 128 per tile; H for down: 256 per tile)
    int n_tiles;
    const uint16_t* A;   // [n_rows, K]
    const uint16_t* B0;  // gate_w [E, I, H] or down_w [E, H, I]
    const uint16_t* B1;  // up_w or null
    uint16_t* out;       // act [n_rows, I] or y [n_rows, H]
    uint16_t* inter13;   // optional [n_rows, 2I]
    const uint16_t* row_weight;
};

__device__ __forceinline__ int swz(int row) { return (row + (row >> 3)) & 7; }

__device__ __forceinline__ void load16_to_lds(const void* g, char* l) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)l, 16, 0, 0);
}

struct TileCoord {
    int e, n_tile, rows;
    int64_t row0;
};

// Logical tile id -> (expert, N tile, M tile).  Returns false for ids past the last tile.
__device__ __forceinline__ bool locate(const int64_t* counts, int E, int n_tiles, TileCoord* tc) {
    int64_t total_m = 0;
    for (int e = 0; e < E; ++e) total_m += (counts[e] + BM - 1) / BM;
    const int64_t total = total_m * n_tiles;
    const int64_t per_xcd = (total + kNumXcd - 1) / kNumXcd;
    const int64_t slot = blockIdx.x / kNumXcd;
    if (slot >= per_xcd) return false;
    int64_t L = (int64_t)(blockIdx.x % kNumXcd) * per_xcd + slot;
    if (L >= total) return false;
    int64_t start = 0;
    for (int e = 0; e < E; ++e) {
        const int64_t c = counts[e];
        const int64_t me = (c + BM - 1) / BM;
        const int64_t te = me * n_tiles;
        if (L < te) {
            const int m = (int)(L % me);
            tc->e = e;
            tc->n_tile = (int)(L / me);
            tc->row0 = start + (int64_t)m * BM;
            const int64_t left = c - (int64_t)m * BM;
            tc->rows = left < BM ? (int)left : BM;
            return true;
        }
        L -= te;
        start += c;
    }
    return false;
}

template <int MODE>
__global__ __launch_bounds__(256, 1) void ffn_mfma_tn_kernel(MfmaParams p) {
    __shared__ __attribute__((aligned(1024))) char lds[2 * kStageBytes];
    TileCoord tc;
    if (!locate(p.counts, p.E, p.n_tiles, &tc)) return;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t K = p.K;

    // ---- global -> LDS assignment: wave w fills tile rows [64w, 64w+64) of A and of B, 8 rows per instruction
    const int lrow = lane >> 3, lchunk = lane & 7;
    const char* a_src[8];
    const char* b_src[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int r = wave * 64 + q * 8 + lrow;
        const int gchunk = lchunk ^ swz(r);
        const int ar = r < tc.rows ? r : tc.rows - 1;  // rows past the expert's last one re-read it (never stored)
        a_src[q] = (const char*)(p.A + (tc.row0 + ar) * K) + gchunk * 16;
        int64_t brow;
        const uint16_t* bmat;
        if (MODE == kGateUp) {
            bmat = ((r & 127) < 64) ? p.B0 : p.B1;
            brow = (int64_t)tc.e * p.n_cols + (int64_t)tc.n_tile * 128 + (r >> 7) * 64 + (r & 63);
        } else {
            bmat = p.B0;
            brow = (int64_t)tc.e * p.n_cols + (int64_t)tc.n_tile * BN + r;
        }
        b_src[q] = (const char*)(bmat + brow * K) + gchunk * 16;
    }
    auto issue_loads = [&](int kt, int stage) {
        char* base = lds + stage * kStageBytes + (wave * 64) * 128;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            load16_to_lds(a_src[q] + (int64_t)kt * (BK * 2), base + q * 1024);
            load16_to_lds(b_src[q] + (int64_t)kt * (BK * 2), base + kTileBytesA + q * 1024);
        }
    };

    // ---- fragment addressing: lane reads row (l & 31) of a 32-row block, k chunk (2*kk + (l >> 5))
    const int l31 = lane & 31, hi = lane >> 5;
    int a_rd[4], b_rd[4], a_f[4], b_f[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ra = wm * 128 + i * 32 + l31, rb = wn * 128 + i * 32 + l31;
        a_rd[i] = ra * 128;
        a_f[i] = swz(ra);
        b_rd[i] = kTileBytesA + rb * 128;
        b_f[i] = swz(rb);
    }

    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    bf16x8_t af[2][4], bfr[2][4];
    auto read_frags = [&](int stage, int kk, int buf) {
        const char* sb = lds + stage * kStageBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            af[buf][i] = *(const bf16x8_t*)(sb + a_rd[i] + (((kk * 2 + hi) ^ a_f[i]) << 4));
            bfr[buf][i] = *(const bf16x8_t*)(sb + b_rd[i] + (((kk * 2 + hi) ^ b_f[i]) << 4));
        }
    };
    auto mma = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[buf][i], bfr[buf][j], acc[i][j], 0, 0, 0);
    };

    const int n_kt = (int)(K / BK);
    issue_loads(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    read_frags(0, 0, 0);
    for (int kt = 0; kt < n_kt; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < n_kt) issue_loads(kt + 1, stage ^ 1);
        read_frags(stage, 1, 1);
        mma(0);
        read_frags(stage, 2, 0);
        mma(1);
        read_frags(stage, 3, 1);
        mma(0);
        // every wave has read its last fragments of this stage; the next tile must have landed
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (kt + 1 < n_kt) read_frags(stage ^ 1, 0, 0);
        mma(1);
    }

    // ---- epilogue: lane holds column (l & 31), rows 8*(r/4) + 4*(l >> 5) + (r % 4) of each 32 x 32 block
    if (MODE == kGateUp) {
        const int64_t I = p.n_cols;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int64_t col = (int64_t)tc.n_tile * 128 + wn * 64 + jj * 32 + l31;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = wm * 128 + i * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
                    if (row < tc.rows) {
                        const float g = bf16_bits_to_f32(f32_to_bf16_bits(acc[i][jj][r]));
                        const float u = bf16_bits_to_f32(f32_to_bf16_bits(acc[i][jj + 2][r]));
                        const float s = bf16_bits_to_f32(f32_to_bf16_bits(g * sigmoid_fast(g)));
                        const int64_t grow = tc.row0 + row;
                        p.out[grow * I + col] = (uint16_t)f32_to_bf16_bits(s * u);
                        if (p.inter13) {
                            p.inter13[grow * 2 * I + col] = (uint16_t)f32_to_bf16_bits(g);
                            p.inter13[grow * 2 * I + I + col] = (uint16_t)f32_to_bf16_bits(u);
                        }
                    }
                }
            }
        }
    } else {
        const int64_t H = p.n_cols;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t col = (int64_t)tc.n_tile * BN + wn * 128 + j * 32 + l31;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = wm * 128 + i * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
                    if (row < tc.rows) {
                        const int64_t grow = tc.row0 + row;
                        float v = acc[i][j][r];
                        if (p.row_weight)
                            v = bf16_bits_to_f32(f32_to_bf16_bits(v)) * bf16_bits_to_f32(p.row_weight[grow]);
                        p.out[grow * H + col] = (uint16_t)f32_to_bf16_bits(v);
                    }
                }
            }
        }
    }
}

inline unsigned grid_bound(const FfnShape& s, int n_tiles) {
    const int64_t m_bound = s.n_rows / BM + s.E;
    const int64_t g = m_bound * n_tiles;
    return (unsigned)(((g + kNumXcd - 1) / kNumXcd) * kNumXcd);
}

}  // namespace

bool ffn_mfma_supported(const FfnShape& s) {
    return s.dtype == PICOMOE_BF16 && s.H % 256 == 0 && s.I % 128 == 0 && s.H >= 256 && s.I >= 128;
}

int ffn_mfma_gate_up(const FfnShape& s, const void* x, const void* gate_w, const void* up_w, void* act, void* inter13,
                     hipStream_t st) {
    MfmaParams p{};
    p.counts = s.counts; p.E = s.E; p.n_rows = s.n_rows; p.K = s.H; p.n_cols = s.I; p.n_tiles = (int)(s.I / 128);
    p.A = (const uint16_t*)x; p.B0 = (const uint16_t*)gate_w; p.B1 = (const uint16_t*)up_w;
    p.out = (uint16_t*)act; p.inter13 = (uint16_t*)inter13; p.row_weight = nullptr;
    hipLaunchKernelGGL(ffn_mfma_tn_kernel<kGateUp>, dim3(grid_bound(s, p.n_tiles)), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

int ffn_mfma_down(const FfnShape& s, const void* act, const void* down_w, const void* row_weight, void* y, hipStream_t st) {
    MfmaParams p{};
    p.counts = s.counts; p.E = s.E; p.n_rows = s.n_rows; p.K = s.I; p.n_cols = s.H; p.n_tiles = (int)(s.H / BN);
    p.A = (const uint16_t*)act; p.B0 = (const uint16_t*)down_w; p.B1 = nullptr;
    p.out = (uint16_t*)y; p.inter13 = nullptr; p.row_weight = (const uint16_t*)row_weight;
    hipLaunchKernelGGL(ffn_mfma_tn_kernel<kDown>, dim3(grid_bound(s, p.n_tiles)), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

// The backward GEMMs still run on the generic kernels.
int ffn_mfma_dgrad_act(const FfnShape& s, const void* dy, const void* down_w, const void* inter13, void* d_inter13,
                       void* act_out, hipStream_t st) {
    return ffn_simple_dgrad_act(s, dy, down_w, inter13, d_inter13, act_out, st);
}
int ffn_mfma_dgrad_x(const FfnShape& s, const void* d_inter13, const void* gate_w, const void* up_w, void* dx,
                     hipStream_t st) {
    return ffn_simple_dgrad_x(s, d_inter13, gate_w, up_w, dx, st);
}
int ffn_mfma_wgrad(const FfnShape& s, const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, int64_t P, int64_t Q,
                   void* out, hipStream_t st) {
    return ffn_simple_wgrad(s, lhs, ld_lhs, rhs, ld_rhs, P, Q, out, st);
}
