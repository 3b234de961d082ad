// fp32 expert-FFN kernels on the matrix pipes of gfx950 (MI355X): the same five grouped GEMMs as the bf16 family
// (gate/up + SwiGLU, down, dgrad through down + SwiGLU backward, dgrad through gate/up, wgrad) for fp32 models, on
// v_mfma_f32_32x32x2_f32 -- full fp32 products and fp32 accumulation, so results stay within fp32 rounding of the
// scalar-FMA kernels (no TF32-style truncation of the operands).
//
// Block tile 128 x 128 x 16, 4 wavefronts (2 x 2), wave tile 64 x 64 = 2 x 2 accumulator blocks of 32 x 32.  Operand
// tiles go global -> registers -> LDS (float4 loads; the next k-tile is fetched into registers while the current one is
// multiplied), both stored k-major in LDS ([16 k][128 + 4 rows or columns]): an MFMA operand is one float per lane,
// lane l holding row / column (l & 31) at k = l >> 5, i.e. one ds_read_b32 of 32 consecutive floats from each of two k rows.
//   K-fast operands (activations, forward weights: contiguous along K) are transposed on the way into LDS,
//   X-fast operands (weights in dgrad, both operands of wgrad: K is the slow index) are stored as they come.
// Shapes: hidden and inter multiples of 4 (whole float4s), 16-byte aligned tensors; anything else stays on the generic kernels.
#include "ffn.h"

namespace {

constexpr int FM = 128, FN = 128, FK = 16;
constexpr int kPitch = FM + 4;  // floats per k row in LDS: 4 * kPitch = 528 = 16 (mod 64) spreads the transposing writes
enum Mode { kGateUp = 0, kDown = 1, kDgradAct = 2, kDgradX = 3, kWgrad = 4 };

struct F32Params {
    const int64_t* counts;
    int E;
    int64_t K;           // contraction length of the M-grouped modes
    int64_t N;           // output columns (gate/up, dgrad_act: I; down, dgrad_x: H; wgrad: Q)
    int64_t M;           // wgrad: output rows P
    const float* A;      // activations [n_rows, lda]; wgrad: lhs
    int64_t lda;
    const float* B0;     // gate_w / down_w; wgrad: rhs
    const float* B1;     // up_w or null
    int64_t ldb;
    int64_t b_expert_stride;
    float* out;
    int64_t ldo;
    float* out2;         // gate/up: inter13 (optional); dgrad_act: act_out (optional)
    const float* aux;    // down: row_weight; dgrad_act: inter13
    int64_t I;           // dgrad_x: where B moves from gate_w to up_w along K
};

typedef __attribute__((ext_vector_type(4))) float f32x4;

// Which expert and which rows does m-tile `tile` cover?  A tile never spans two experts.
__device__ __forceinline__ bool locate_rows(const int64_t* counts, int E, int tile, int* expert, int64_t* row0, int* rows) {
    int64_t start = 0;
    int t = tile;
    for (int e = 0; e < E; ++e) {
        const int64_t c = counts[e];
        const int nt = (int)((c + FM - 1) / FM);
        if (t < nt) {
            *expert = e;
            *row0 = start + (int64_t)t * FM;
            const int64_t left = c - (int64_t)t * FM;
            *rows = left < FM ? (int)left : FM;
            return true;
        }
        t -= nt;
        start += c;
    }
    return false;
}

template <int MODE>
__global__ __launch_bounds__(256) void ffn_f32_mfma_kernel(F32Params p) {
    constexpr bool kAKFast = MODE != kWgrad;
    constexpr bool kBKFast = MODE == kGateUp || MODE == kDown;
    __shared__ float As[FK * kPitch];
    __shared__ float Bs[FK * kPitch];

    int e, rows;       // M-grouped: valid rows of the tile; wgrad: rows of the expert (the contraction length)
    int64_t row0;      // first row of the tile (M-grouped) or of the expert's segment (wgrad)
    int64_t K;
    int64_t m0 = 0;    // wgrad: first output row (p) of the tile
    int64_t n0;        // first output column of the tile (gate/up: of its 64 gate and 64 up columns)
    if (MODE == kWgrad) {
        e = blockIdx.z;
        row0 = 0;
        for (int i = 0; i < e; ++i) row0 += p.counts[i];
        rows = (int)p.counts[e];
        K = rows;
        m0 = (int64_t)blockIdx.x * FM;
        n0 = (int64_t)blockIdx.y * FN;
    } else {
        if (!locate_rows(p.counts, p.E, blockIdx.x, &e, &row0, &rows)) return;
        K = p.K;
        n0 = (int64_t)blockIdx.y * (MODE == kGateUp ? FN / 2 : FN);
    }

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- global -> registers: two float4 per operand, thread and k-tile -------------------------------------------
    // K-fast tile: row (tid / 4) + 64 i, k quad tid % 4; X-fast tile: k row (tid / 32) + 8 i, column quad tid % 32
    const float* a_ptr[2];
    const float* b_ptr[2];
    bool a_ok[2], b_ok[2];
    const float* b_ptr_up[2] = {nullptr, nullptr};  // dgrad_x: the same address in up_w
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        if (kAKFast) {
            const int m = (tid >> 2) + 64 * i;
            a_ok[i] = m < rows;
            a_ptr[i] = p.A + (row0 + (a_ok[i] ? m : 0)) * p.lda + 4 * (tid & 3);
        } else {
            const int64_t col = m0 + 4 * (tid & 31);
            a_ok[i] = col < p.M;
            a_ptr[i] = p.A + (row0 + (tid >> 5) + 8 * i) * p.lda + (a_ok[i] ? col : 0);
        }
        if (kBKFast) {
            const int nb = (tid >> 2) + 64 * i;  // row of the B tile = output column of the block
            const float* mat = p.B0;
            int64_t wrow;
            if (MODE == kGateUp) {
                // tile columns: per wave column (64 wide) 32 gate rows then the 32 up rows of the same output columns
                const int half = (nb & 63) >> 5;
                mat = half ? p.B1 : p.B0;
                wrow = n0 + (nb >> 6) * 32 + (nb & 31);
            } else {
                wrow = n0 + nb;
            }
            b_ok[i] = wrow < p.N;
            b_ptr[i] = mat + (int64_t)e * p.b_expert_stride + (b_ok[i] ? wrow : 0) * p.ldb + 4 * (tid & 3);
        } else {
            const int64_t col = n0 + 4 * (tid & 31);
            b_ok[i] = col < p.N;
            const int64_t base = MODE == kWgrad ? row0 * p.ldb : (int64_t)e * p.b_expert_stride;
            b_ptr[i] = p.B0 + base + ((tid >> 5) + 8 * i) * p.ldb + (b_ok[i] ? col : 0);
            if (MODE == kDgradX) b_ptr_up[i] = p.B1 + base + ((tid >> 5) + 8 * i) * p.ldb + (b_ok[i] ? col : 0);
        }
    }
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int64_t k0, f32x4 (&ra)[2], f32x4 (&rb)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (kAKFast) {
                const bool ok = a_ok[i] && k0 + 4 * (tid & 3) < K;  // K is a multiple of 4: a float4 is inside or outside
                ra[i] = ok ? *(const f32x4*)(a_ptr[i] + k0) : zero4;
            } else {
                const bool ok = a_ok[i] && k0 + (tid >> 5) + 8 * i < K;
                ra[i] = ok ? *(const f32x4*)(a_ptr[i] + k0 * p.lda) : zero4;
            }
            if (kBKFast) {
                const bool ok = b_ok[i] && k0 + 4 * (tid & 3) < K;
                rb[i] = ok ? *(const f32x4*)(b_ptr[i] + k0) : zero4;
            } else {
                const int64_t k = k0 + (tid >> 5) + 8 * i;
                const bool ok = b_ok[i] && k < K;
                if (MODE == kDgradX)  // rows k < I of [gate_w; up_w] come from gate_w, the others from up_w
                    rb[i] = ok ? (k < p.I ? *(const f32x4*)(b_ptr[i] + k0 * p.ldb) : *(const f32x4*)(b_ptr_up[i] + (k0 - p.I) * p.ldb)) : zero4;
                else
                    rb[i] = ok ? *(const f32x4*)(b_ptr[i] + k0 * p.ldb) : zero4;
            }
        }
    };
    auto stash = [&](const f32x4 (&ra)[2], const f32x4 (&rb)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (kAKFast) {
                const int m = (tid >> 2) + 64 * i, kq = 4 * (tid & 3);
#pragma unroll
                for (int j = 0; j < 4; ++j) As[(kq + j) * kPitch + m] = ra[i][j];
            } else {
                *(f32x4*)(As + ((tid >> 5) + 8 * i) * kPitch + 4 * (tid & 31)) = ra[i];
            }
            if (kBKFast) {
                const int nb = (tid >> 2) + 64 * i, kq = 4 * (tid & 3);
#pragma unroll
                for (int j = 0; j < 4; ++j) Bs[(kq + j) * kPitch + nb] = rb[i][j];
            } else {
                *(f32x4*)(Bs + ((tid >> 5) + 8 * i) * kPitch + 4 * (tid & 31)) = rb[i];
            }
        }
    };

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    f32x4 ra[2], rb[2];
    if (K > 0) fetch(0, ra, rb);
    const float* a_frag = As + (lane >> 5) * kPitch + wm * 64 + (lane & 31);
    const float* b_frag = Bs + (lane >> 5) * kPitch + wn * 64 + (lane & 31);
    for (int64_t k0 = 0; k0 < K; k0 += FK) {
        stash(ra, rb);
        __syncthreads();
        if (k0 + FK < K) fetch(k0 + FK, ra, rb);  // in flight while this k-tile is multiplied
#pragma unroll
        for (int kk = 0; kk < FK; kk += 2) {
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i] = a_frag[kk * kPitch + i * 32];
                b[i] = b_frag[kk * kPitch + i * 32];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // ---- epilogue: lane holds column (l & 31) and rows 8 (r / 4) + 4 (l >> 5) + (r % 4) of every 32 x 32 block ------
    const int c32 = lane & 31, r4 = 4 * (lane >> 5);
    if (MODE == kGateUp) {
        const int64_t I = p.N;
        const int64_t col = n0 + wn * 32 + c32;  // block j = 0 holds g, j = 1 the u of the same column
        if (col >= I) return;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = wm * 64 + i * 32 + 8 * (r >> 2) + r4 + (r & 3);
                if (m >= rows) continue;
                const float g = acc[i][0][r], u = acc[i][1][r];
                p.out[(row0 + m) * I + col] = (g * sigmoid_f32(g)) * u;
                if (p.out2) {
                    p.out2[(row0 + m) * 2 * I + col] = g;
                    p.out2[(row0 + m) * 2 * I + I + col] = u;
                }
            }
        return;
    }
    const int valid_rows = MODE == kWgrad ? (int)(p.M - m0 < FM ? p.M - m0 : FM) : rows;
    const int64_t out_row0 = MODE == kWgrad ? (int64_t)e * p.M + m0 : row0;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t col = n0 + wn * 64 + j * 32 + c32;
            if (col >= p.N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = wm * 64 + i * 32 + 8 * (r >> 2) + r4 + (r & 3);
                if (m >= valid_rows) continue;
                const int64_t grow = out_row0 + m;
                const float v = acc[i][j][r];
                if (MODE == kDgradAct) {
                    const int64_t I = p.N;
                    const float g = p.aux[grow * 2 * I + col], u = p.aux[grow * 2 * I + I + col];
                    const float sig = sigmoid_f32(g);
                    p.out[grow * 2 * I + col] = v * u * (sig * (1.f + g * (1.f - sig)));
                    p.out[grow * 2 * I + I + col] = v * (g * sig);
                    if (p.out2) p.out2[grow * I + col] = (g * sig) * u;
                } else if (MODE == kDown && p.aux) {
                    p.out[grow * p.ldo + col] = v * p.aux[grow];
                } else {
                    p.out[grow * p.ldo + col] = v;
                }
            }
        }
}

inline unsigned cdiv_u(int64_t a, int64_t b) { return (unsigned)((a + b - 1) / b); }
inline unsigned m_tiles_bound(const FfnShape& s) { return (unsigned)(s.n_rows / FM + s.E); }
inline bool aligned16(const void* ptr) { return (uintptr_t)ptr % 16 == 0; }

F32Params base_params(const FfnShape& s) {
    F32Params p{};
    p.counts = s.counts;
    p.E = s.E;
    return p;
}

}  // namespace

bool ffn_f32_mfma_supported(const FfnShape& s) {
    return s.dtype == PICOMOE_F32 && s.H % 4 == 0 && s.I % 4 == 0 && s.H >= 32 && s.I >= 32;
}

int ffn_f32_mfma_gate_up(const FfnShape& s, const void* x, const void* gate_w, const void* up_w, void* act, void* inter13,
                         hipStream_t st) {
    if (!(aligned16(x) && aligned16(gate_w) && aligned16(up_w))) return ffn_simple_gate_up(s, x, gate_w, up_w, act, inter13, st);
    F32Params p = base_params(s);
    p.K = s.H; p.N = s.I;
    p.A = (const float*)x; p.lda = s.H;
    p.B0 = (const float*)gate_w; p.B1 = (const float*)up_w; p.ldb = s.H; p.b_expert_stride = s.I * s.H;
    p.out = (float*)act; p.ldo = s.I; p.out2 = (float*)inter13;
    hipLaunchKernelGGL((ffn_f32_mfma_kernel<kGateUp>), dim3(m_tiles_bound(s), cdiv_u(s.I, FN / 2)), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

int ffn_f32_mfma_down(const FfnShape& s, const void* act, const void* down_w, const void* row_weight, void* y, hipStream_t st) {
    if (!(aligned16(act) && aligned16(down_w))) return ffn_simple_down(s, act, down_w, row_weight, y, st);
    F32Params p = base_params(s);
    p.K = s.I; p.N = s.H;
    p.A = (const float*)act; p.lda = s.I;
    p.B0 = (const float*)down_w; p.ldb = s.I; p.b_expert_stride = s.H * s.I;
    p.out = (float*)y; p.ldo = s.H; p.aux = (const float*)row_weight;
    hipLaunchKernelGGL((ffn_f32_mfma_kernel<kDown>), dim3(m_tiles_bound(s), cdiv_u(s.H, FN)), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

int ffn_f32_mfma_dgrad_act(const FfnShape& s, const void* dy, const void* down_w, const void* inter13, void* d_inter13,
                           void* act_out, hipStream_t st) {
    if (!(aligned16(dy) && aligned16(down_w))) return ffn_simple_dgrad_act(s, dy, down_w, inter13, d_inter13, act_out, st);
    F32Params p = base_params(s);
    p.K = s.H; p.N = s.I;
    p.A = (const float*)dy; p.lda = s.H;
    p.B0 = (const float*)down_w; p.ldb = s.I; p.b_expert_stride = s.H * s.I;  // down_w[e] read as [K = H][N = I]
    p.out = (float*)d_inter13; p.ldo = 2 * s.I; p.out2 = (float*)act_out; p.aux = (const float*)inter13;
    hipLaunchKernelGGL((ffn_f32_mfma_kernel<kDgradAct>), dim3(m_tiles_bound(s), cdiv_u(s.I, FN)), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

int ffn_f32_mfma_dgrad_x(const FfnShape& s, const void* d_inter13, const void* gate_w, const void* up_w, void* dx,
                         hipStream_t st) {
    if (!(aligned16(d_inter13) && aligned16(gate_w) && aligned16(up_w))) return ffn_simple_dgrad_x(s, d_inter13, gate_w, up_w, dx, st);
    F32Params p = base_params(s);
    p.K = 2 * s.I; p.N = s.H; p.I = s.I;
    p.A = (const float*)d_inter13; p.lda = 2 * s.I;
    p.B0 = (const float*)gate_w; p.B1 = (const float*)up_w; p.ldb = s.H; p.b_expert_stride = s.I * s.H;  // [K = I][N = H]
    p.out = (float*)dx; p.ldo = s.H;
    hipLaunchKernelGGL((ffn_f32_mfma_kernel<kDgradX>), dim3(m_tiles_bound(s), cdiv_u(s.H, FN)), dim3(256), 0, st, p);
    return picomoe_launch_status();
}

bool ffn_f32_mfma_wgrad_supported(int dtype, int64_t P, int64_t Q, int64_t ld_lhs, int64_t ld_rhs, const void* lhs,
                                  const void* rhs) {
    return dtype == PICOMOE_F32 && P % 4 == 0 && Q % 4 == 0 && P >= 32 && Q >= 32 && ld_lhs % 4 == 0 && ld_rhs % 4 == 0 &&
           aligned16(lhs) && aligned16(rhs);
}

int ffn_f32_mfma_wgrad(const FfnShape& s, const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, int64_t P, int64_t Q,
                       void* out, hipStream_t st) {
    F32Params p = base_params(s);
    p.M = P; p.N = Q;
    p.A = (const float*)lhs; p.lda = ld_lhs;
    p.B0 = (const float*)rhs; p.ldb = ld_rhs;
    p.out = (float*)out; p.ldo = Q;
    hipLaunchKernelGGL((ffn_f32_mfma_kernel<kWgrad>), dim3(cdiv_u(P, FM), cdiv_u(Q, FN), (unsigned)s.E), dim3(256), 0, st, p);
    return picomoe_launch_status();
}
