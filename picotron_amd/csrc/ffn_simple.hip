// Generic expert-FFN kernels: any shape, fp32 or bf16 storage, fp32 FMA arithmetic.
// They serve fp32 models (where bf16 MFMA would lose precision) and shapes the MFMA kernels do not
// tile; speed is secondary here.  64x64 output tile, 256 threads, 4x4 outputs per thread, BK = 16.
#include "ffn.h"

namespace {

constexpr int TM = 64, TN = 64, TK = 16;

template <typename T>
__device__ __forceinline__ float ld(const T* p);
template <>
__device__ __forceinline__ float ld<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ld<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }
template <typename T>
__device__ __forceinline__ void st(T* p, float v);
template <>
__device__ __forceinline__ void st<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void st<uint16_t>(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
template <typename T>
__device__ __forceinline__ float rnd(float v);
template <>
__device__ __forceinline__ float rnd<float>(float v) { return v; }
template <>
__device__ __forceinline__ float rnd<uint16_t>(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// acc[i][j] += sum_k A(m0 + ty*4+i, k) * B(k, n0 + tx*4+j) for k in [0,K).
// a_elem(m_local, k) / b_elem(k, n_local) return 0 outside the valid range.
template <typename FA, typename FB>
__device__ __forceinline__ void tile_mac(float (&acc)[4][4], int64_t K, bool a_kfast, bool b_kfast, FA a_elem, FB b_elem) {
    __shared__ float As[TK][TM + 1];
    __shared__ float Bs[TK][TN + 1];
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    for (int64_t k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + 256 * i;
            const int am = a_kfast ? idx / TK : idx % TM, ak = a_kfast ? idx % TK : idx / TM;
            As[ak][am] = (k0 + ak < K) ? a_elem(am, k0 + ak) : 0.f;
            const int bn = b_kfast ? idx / TK : idx % TN, bk = b_kfast ? idx % TK : idx / TN;
            Bs[bk][bn] = (k0 + bk < K) ? b_elem(k0 + bk, bn) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; b[i] = Bs[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
}

// Which expert and which rows does m-tile `tile` cover?  Experts lie back to back; a tile never
// spans two experts.  Returns false when the tile index is past the last one.
__device__ __forceinline__ bool locate_tile(const int64_t* counts, int E, int tile, int* expert, int64_t* row0, int* rows) {
    int64_t start = 0;
    int t = tile;
    for (int e = 0; e < E; ++e) {
        const int64_t c = counts[e];
        const int nt = (int)((c + TM - 1) / TM);
        if (t < nt) {
            *expert = e;
            *row0 = start + (int64_t)t * TM;
            const int64_t left = c - (int64_t)t * TM;
            *rows = left < TM ? (int)left : TM;
            return true;
        }
        t -= nt;
        start += c;
    }
    return false;
}

template <typename T>
__global__ __launch_bounds__(256) void gate_up_kernel(FfnShape s, const T* __restrict__ x, const T* __restrict__ gate_w,
                                                      const T* __restrict__ up_w, T* __restrict__ act,
                                                      T* __restrict__ inter13) {
    int e, rows;
    int64_t row0;
    if (!locate_tile(s.counts, s.E, blockIdx.x, &e, &row0, &rows)) return;
    const int64_t n0 = (int64_t)blockIdx.y * TN, H = s.H, I = s.I;
    const T* wg = gate_w + (int64_t)e * I * H;
    const T* wu = up_w + (int64_t)e * I * H;
    float g[4][4] = {}, u[4][4] = {};
    auto a_elem = [&](int m, int64_t k) { return m < rows ? ld<T>(x + (row0 + m) * H + k) : 0.f; };
    tile_mac(g, H, true, true, a_elem, [&](int64_t k, int n) { return n0 + n < I ? ld<T>(wg + (n0 + n) * H + k) : 0.f; });
    tile_mac(u, H, true, true, a_elem, [&](int64_t k, int n) { return n0 + n < I ? ld<T>(wu + (n0 + n) * H + k) : 0.f; });
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = ty * 4 + i;
        if (m >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n >= I) continue;
            const float gr = rnd<T>(g[i][j]), ur = rnd<T>(u[i][j]);
            const float sl = rnd<T>(gr * sigmoid_f32(gr));
            st<T>(act + (row0 + m) * I + n, sl * ur);
            if (inter13) {
                st<T>(inter13 + (row0 + m) * 2 * I + n, gr);
                st<T>(inter13 + (row0 + m) * 2 * I + I + n, ur);
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void down_kernel(FfnShape s, const T* __restrict__ act, const T* __restrict__ down_w,
                                                   const T* __restrict__ row_weight, T* __restrict__ y) {
    int e, rows;
    int64_t row0;
    if (!locate_tile(s.counts, s.E, blockIdx.x, &e, &row0, &rows)) return;
    const int64_t n0 = (int64_t)blockIdx.y * TN, H = s.H, I = s.I;
    const T* wd = down_w + (int64_t)e * H * I;
    float acc[4][4] = {};
    tile_mac(acc, I, true, true, [&](int m, int64_t k) { return m < rows ? ld<T>(act + (row0 + m) * I + k) : 0.f; },
             [&](int64_t k, int n) { return n0 + n < H ? ld<T>(wd + (n0 + n) * I + k) : 0.f; });
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = ty * 4 + i;
        if (m >= rows) continue;
        const float rw = row_weight ? ld<T>(row_weight + row0 + m) : 1.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n < H) st<T>(y + (row0 + m) * H + n, row_weight ? rnd<T>(acc[i][j]) * rw : acc[i][j]);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void dgrad_act_kernel(FfnShape s, const T* __restrict__ dy, const T* __restrict__ down_w,
                                                        const T* __restrict__ inter13, T* __restrict__ d_inter13,
                                                        T* __restrict__ act_out) {
    int e, rows;
    int64_t row0;
    if (!locate_tile(s.counts, s.E, blockIdx.x, &e, &row0, &rows)) return;
    const int64_t n0 = (int64_t)blockIdx.y * TN, H = s.H, I = s.I;
    const T* wd = down_w + (int64_t)e * H * I;  // [H, I]: contraction index is the row
    float acc[4][4] = {};
    tile_mac(acc, H, true, false, [&](int m, int64_t k) { return m < rows ? ld<T>(dy + (row0 + m) * H + k) : 0.f; },
             [&](int64_t k, int n) { return n0 + n < I ? ld<T>(wd + k * I + n0 + n) : 0.f; });
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = ty * 4 + i;
        if (m >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n >= I) continue;
            const float da = rnd<T>(acc[i][j]);
            const float g = ld<T>(inter13 + (row0 + m) * 2 * I + n), u = ld<T>(inter13 + (row0 + m) * 2 * I + I + n);
            const float sig = sigmoid_f32(g);
            st<T>(d_inter13 + (row0 + m) * 2 * I + n, da * u * (sig * (1.f + g * (1.f - sig))));
            st<T>(d_inter13 + (row0 + m) * 2 * I + I + n, da * (g * sig));
            if (act_out) st<T>(act_out + (row0 + m) * I + n, rnd<T>(g * sig) * u);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void dgrad_x_kernel(FfnShape s, const T* __restrict__ d13, const T* __restrict__ gate_w,
                                                      const T* __restrict__ up_w, T* __restrict__ dx) {
    int e, rows;
    int64_t row0;
    if (!locate_tile(s.counts, s.E, blockIdx.x, &e, &row0, &rows)) return;
    const int64_t n0 = (int64_t)blockIdx.y * TN, H = s.H, I = s.I;
    const T* wg = gate_w + (int64_t)e * I * H;  // [I, H]: contraction index is the row
    const T* wu = up_w + (int64_t)e * I * H;
    float acc[4][4] = {};
    tile_mac(acc, I, true, false, [&](int m, int64_t k) { return m < rows ? ld<T>(d13 + (row0 + m) * 2 * I + k) : 0.f; },
             [&](int64_t k, int n) { return n0 + n < H ? ld<T>(wg + k * H + n0 + n) : 0.f; });
    tile_mac(acc, I, true, false, [&](int m, int64_t k) { return m < rows ? ld<T>(d13 + (row0 + m) * 2 * I + I + k) : 0.f; },
             [&](int64_t k, int n) { return n0 + n < H ? ld<T>(wu + k * H + n0 + n) : 0.f; });
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = ty * 4 + i;
        if (m >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n < H) st<T>(dx + (row0 + m) * H + n, acc[i][j]);
        }
    }
}

// grid (P tiles, Q tiles, E)
template <typename T>
__global__ __launch_bounds__(256) void wgrad_kernel(FfnShape s, const T* __restrict__ lhs, int64_t ld_lhs,
                                                    const T* __restrict__ rhs, int64_t ld_rhs, int64_t P, int64_t Q,
                                                    T* __restrict__ out) {
    const int e = blockIdx.z;
    int64_t start = 0;
    for (int i = 0; i < e; ++i) start += s.counts[i];
    const int64_t cnt = s.counts[e];
    const int64_t p0 = (int64_t)blockIdx.x * TM, q0 = (int64_t)blockIdx.y * TN;
    float acc[4][4] = {};
    tile_mac(acc, cnt, false, false, [&](int m, int64_t k) { return p0 + m < P ? ld<T>(lhs + (start + k) * ld_lhs + p0 + m) : 0.f; },
             [&](int64_t k, int n) { return q0 + n < Q ? ld<T>(rhs + (start + k) * ld_rhs + q0 + n) : 0.f; });
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    T* o = out + (int64_t)e * P * Q;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t p = p0 + ty * 4 + i;
        if (p >= P) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t q = q0 + tx * 4 + j;
            if (q < Q) st<T>(o + p * Q + q, acc[i][j]);
        }
    }
}

inline unsigned m_tiles_bound(const FfnShape& s) { return (unsigned)(s.n_rows / TM + s.E); }
inline unsigned cdiv(int64_t a, int64_t b) { return (unsigned)((a + b - 1) / b); }

}  // namespace

int ffn_simple_gate_up(const FfnShape& s, const void* x, const void* gate_w, const void* up_w, void* act, void* inter13,
                       hipStream_t st) {
    const dim3 grid(m_tiles_bound(s), cdiv(s.I, TN));
    if (s.dtype == PICOMOE_BF16)
        hipLaunchKernelGGL(gate_up_kernel<uint16_t>, grid, dim3(256), 0, st, s, (const uint16_t*)x, (const uint16_t*)gate_w, (const uint16_t*)up_w, (uint16_t*)act, (uint16_t*)inter13);
    else
        hipLaunchKernelGGL(gate_up_kernel<float>, grid, dim3(256), 0, st, s, (const float*)x, (const float*)gate_w, (const float*)up_w, (float*)act, (float*)inter13);
    return picomoe_launch_status();
}

int ffn_simple_down(const FfnShape& s, const void* act, const void* down_w, const void* row_weight, void* y,
                    hipStream_t st) {
    const dim3 grid(m_tiles_bound(s), cdiv(s.H, TN));
    if (s.dtype == PICOMOE_BF16)
        hipLaunchKernelGGL(down_kernel<uint16_t>, grid, dim3(256), 0, st, s, (const uint16_t*)act, (const uint16_t*)down_w, (const uint16_t*)row_weight, (uint16_t*)y);
    else
        hipLaunchKernelGGL(down_kernel<float>, grid, dim3(256), 0, st, s, (const float*)act, (const float*)down_w, (const float*)row_weight, (float*)y);
    return picomoe_launch_status();
}

int ffn_simple_dgrad_act(const FfnShape& s, const void* dy, const void* down_w, const void* inter13, void* d_inter13,
                         void* act_out, hipStream_t st) {
    const dim3 grid(m_tiles_bound(s), cdiv(s.I, TN));
    if (s.dtype == PICOMOE_BF16)
        hipLaunchKernelGGL(dgrad_act_kernel<uint16_t>, grid, dim3(256), 0, st, s, (const uint16_t*)dy, (const uint16_t*)down_w, (const uint16_t*)inter13, (uint16_t*)d_inter13, (uint16_t*)act_out);
    else
        hipLaunchKernelGGL(dgrad_act_kernel<float>, grid, dim3(256), 0, st, s, (const float*)dy, (const float*)down_w, (const float*)inter13, (float*)d_inter13, (float*)act_out);
    return picomoe_launch_status();
}

int ffn_simple_dgrad_x(const FfnShape& s, const void* d_inter13, const void* gate_w, const void* up_w, void* dx,
                       hipStream_t st) {
    const dim3 grid(m_tiles_bound(s), cdiv(s.H, TN));
    if (s.dtype == PICOMOE_BF16)
        hipLaunchKernelGGL(dgrad_x_kernel<uint16_t>, grid, dim3(256), 0, st, s, (const uint16_t*)d_inter13, (const uint16_t*)gate_w, (const uint16_t*)up_w, (uint16_t*)dx);
    else
        hipLaunchKernelGGL(dgrad_x_kernel<float>, grid, dim3(256), 0, st, s, (const float*)d_inter13, (const float*)gate_w, (const float*)up_w, (float*)dx);
    return picomoe_launch_status();
}

int ffn_simple_wgrad(const FfnShape& s, const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, int64_t P,
                     int64_t Q, void* out, hipStream_t st) {
    const dim3 grid(cdiv(P, TM), cdiv(Q, TN), (unsigned)s.E);
    if (s.dtype == PICOMOE_BF16)
        hipLaunchKernelGGL(wgrad_kernel<uint16_t>, grid, dim3(256), 0, st, s, (const uint16_t*)lhs, ld_lhs, (const uint16_t*)rhs, ld_rhs, P, Q, (uint16_t*)out);
    else
        hipLaunchKernelGGL(wgrad_kernel<float>, grid, dim3(256), 0, st, s, (const float*)lhs, ld_lhs, (const float*)rhs, ld_rhs, P, Q, (float*)out);
    return picomoe_launch_status();
}
