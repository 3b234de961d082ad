// Router for gfx950: fp32 softmax over the expert logits, top-k by wavefront-level argmax, gate
// weights, plus the pieces of load balancing that ride on the same pass (per-expert pick counts and
// column sums of the probabilities) and the backward through weights -> softmax -> logits.
//
// A group of G lanes (G = 8..64, a power of two >= E when E <= 64) owns one token; with more than
// 64 experts each lane holds EPL experts (e = lane + 64*i).  Selection rule: higher score first,
// on equal score the lower expert id.  Nothing here depends on atomics ordering: counts use integer
// atomics, probability column sums go through per-block partials reduced in a fixed order.
#include <math.h>

#include <type_traits>

#include "common.h"

namespace {

constexpr int kMaxTopK = 16;
constexpr int kRouteBlock = 256;
constexpr int kMaxExperts = 1024;  // the entry points refuse more

template <typename T>
__device__ __forceinline__ float to_f32(T v);
template <>
__device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float to_f32<uint16_t>(uint16_t v) { return bf16_bits_to_f32(v); }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ uint16_t from_f32<uint16_t>(float v) { return (uint16_t)f32_to_bf16_bits(v); }

template <int G>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

template <typename T, int G, int EPL>
__global__ __launch_bounds__(kRouteBlock) void route_fwd_kernel(const T* __restrict__ logits, int64_t n_tokens, int E,
                                                                int k, const float* __restrict__ bias, int norm,
                                                                int64_t* __restrict__ idx_out, T* __restrict__ w_out,
                                                                float* __restrict__ probs_out, int* __restrict__ counts,
                                                                float* __restrict__ colsum_partial) {
    constexpr int kGroupsPerBlock = kRouteBlock / G;
    const int gl = threadIdx.x % G;   // lane inside the token group
    const int grp = threadIdx.x / G;  // token group inside the block
    float colsum[EPL];
    int picked[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) { colsum[i] = 0.f; picked[i] = 0; }

    // every group of a wave runs the same trip count so the shuffles stay converged
    const int64_t n_iter = (n_tokens + (int64_t)gridDim.x * kGroupsPerBlock - 1) / ((int64_t)gridDim.x * kGroupsPerBlock);
    for (int64_t it = 0; it < n_iter; ++it) {
        const int64_t t = (it * gridDim.x + blockIdx.x) * kGroupsPerBlock + grp;
        const bool live = t < n_tokens;
        float x[EPL], p[EPL], sel[EPL];
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const int e = gl + G * i;
            x[i] = (live && e < E) ? to_f32<T>(logits[t * E + e]) : -INFINITY;
            m = fmaxf(m, x[i]);
        }
        m = group_max<G>(m);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            p[i] = (gl + G * i < E) ? expf(x[i] - m) : 0.f;
            s += p[i];
        }
        s = group_sum<G>(s);
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const int e = gl + G * i;
            p[i] = p[i] / s;
            sel[i] = (e < E) ? (bias ? p[i] + bias[e] : p[i]) : -INFINITY;
            if (live && e < E) {
                if (probs_out) probs_out[t * E + e] = p[i];
                colsum[i] += p[i];
            }
        }

        int win_e[kMaxTopK];
        float win_p[kMaxTopK];
        unsigned taken = 0u;  // bit i: this lane's i-th expert has been picked already
        constexpr int kNone = 0x7FFFFFFF;
#pragma unroll
        for (int j = 0; j < kMaxTopK; ++j) {
            if (j < k) {
                float bv = -INFINITY, bp = 0.f;
                int be = kNone;
#pragma unroll
                for (int i = 0; i < EPL; ++i) {  // ascending expert id: strict > keeps the lower id on ties
                    const int e = gl + G * i;
                    if (e < E && !((taken >> i) & 1u) && (be == kNone || sel[i] > bv)) { bv = sel[i]; be = e; bp = p[i]; }
                }
#pragma unroll
                for (int off = G / 2; off > 0; off >>= 1) {
                    const float ov = __shfl_xor(bv, off, kWave);
                    const int oe = __shfl_xor(be, off, kWave);
                    const float op = __shfl_xor(bp, off, kWave);
                    if (oe != kNone && (be == kNone || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; bp = op; }
                }
                win_e[j] = be;
                win_p[j] = bp;
#pragma unroll
                for (int i = 0; i < EPL; ++i)
                    if (gl + G * i == be) { taken |= 1u << i; if (live) picked[i] += 1; }
            }
        }

        if (live && gl == 0) {
            float denom = 1.f;
            if (norm && k > 1) {
                denom = 0.f;
#pragma unroll
                for (int j = 0; j < kMaxTopK; ++j)
                    if (j < k) denom += win_p[j];
            }
#pragma unroll
            for (int j = 0; j < kMaxTopK; ++j) {
                if (j < k) {
                    idx_out[t * k + j] = win_e[j];
                    const float w = (norm && k > 1) ? win_p[j] / denom : win_p[j];
                    w_out[t * k + j] = from_f32<T>(w);
                }
            }
        }
    }

    if (counts) {
        // per-block histogram in LDS first: one global atomic per expert and block instead of one per thread
        __shared__ int blk_counts[kMaxExperts];
        for (int e = threadIdx.x; e < E; e += kRouteBlock) blk_counts[e] = 0;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < EPL; ++i)
            if (picked[i] && gl + G * i < E) atomicAdd(blk_counts + gl + G * i, picked[i]);
        __syncthreads();
        for (int e = threadIdx.x; e < E; e += kRouteBlock)
            if (blk_counts[e]) atomicAdd(counts + e, blk_counts[e]);
    }
    if (colsum_partial) {
        __shared__ float acc[kRouteBlock * EPL];
#pragma unroll
        for (int i = 0; i < EPL; ++i) acc[threadIdx.x * EPL + i] = colsum[i];
        __syncthreads();
        for (int e = threadIdx.x; e < E; e += kRouteBlock) {
            const int lane_of_e = e % G, slot = e / G;
            float tot = 0.f;
            for (int g2 = 0; g2 < kGroupsPerBlock; ++g2) tot += acc[(g2 * G + lane_of_e) * EPL + slot];
            colsum_partial[(int64_t)blockIdx.x * E + e] = tot;
        }
    }
}

// d logits from d gate-weights (through the optional renormalisation), the aux-loss term and the
// softmax.  probs [T,E] fp32 and idx [T,k] come from the forward pass.
template <typename T, int G, int EPL>
__global__ __launch_bounds__(kRouteBlock) void route_bwd_kernel(const float* __restrict__ probs,
                                                                const int64_t* __restrict__ idx,
                                                                const T* __restrict__ d_w, int64_t n_tokens, int E, int k,
                                                                int norm, const float* __restrict__ d_aux,
                                                                const int* __restrict__ counts, float aux_coef,
                                                                T* __restrict__ d_logits) {
    constexpr int kGroupsPerBlock = kRouteBlock / G;
    const int gl = threadIdx.x % G;
    const int64_t t = (int64_t)blockIdx.x * kGroupsPerBlock + threadIdx.x / G;
    const bool live = t < n_tokens;
    const int64_t tt = live ? t : 0;

    float p[EPL], dp[EPL];
    const float aux_scale = (d_aux && counts) ? d_aux[0] * aux_coef : 0.f;
    const float f_scale = (float)((double)E / ((double)k * (double)n_tokens));
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        const int e = gl + G * i;
        p[i] = e < E ? probs[tt * E + e] : 0.f;
        dp[i] = (e < E && aux_scale != 0.f) ? aux_scale * ((float)counts[e] * f_scale) / (float)n_tokens : 0.f;
    }
    if (d_w) {
        float pj[kMaxTopK], dwj[kMaxTopK];
        int ej[kMaxTopK];
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < kMaxTopK; ++j) {
            if (j < k) {
                ej[j] = (int)idx[tt * k + j];
                pj[j] = probs[tt * E + ej[j]];
                dwj[j] = to_f32<T>(d_w[tt * k + j]);
                s += pj[j];
            }
        }
        const bool renorm = norm && k > 1;
        float dot = 0.f;
        if (renorm) {
#pragma unroll
            for (int j = 0; j < kMaxTopK; ++j)
                if (j < k) dot += dwj[j] * (pj[j] / s);
        }
#pragma unroll
        for (int j = 0; j < kMaxTopK; ++j) {
            if (j < k) {
                const float g = renorm ? (dwj[j] - dot) / s : dwj[j];
#pragma unroll
                for (int i = 0; i < EPL; ++i)
                    if (gl + G * i == ej[j]) dp[i] += g;
            }
        }
    }
    float inner = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) inner += dp[i] * p[i];
    inner = group_sum<G>(inner);
    if (live) {
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const int e = gl + G * i;
            if (e < E) d_logits[t * E + e] = from_f32<T>(p[i] * (dp[i] - inner));
        }
    }
}

// One block: finish the column sums in a fixed order, form the aux loss, step the loss-free bias.
__global__ __launch_bounds__(256) void balance_kernel(const int* __restrict__ counts,
                                                      const float* __restrict__ colsum_partial, int n_partials,
                                                      int64_t n_tokens, int E, int k, float aux_coef, float bias_rate,
                                                      float* __restrict__ aux_out, float* __restrict__ bias) {
    __shared__ float red[256];
    __shared__ float colsum[kMaxExperts];
    if (aux_out && colsum_partial) {
        // column sums of the probabilities: each expert's partials are split over kSplit threads (fixed split and a
        // fixed-order tree, so the result does not depend on timing), 256 / kSplit experts at a time
        constexpr int kSplit = 32;
        const int sub = threadIdx.x % kSplit;
        for (int e0 = 0; e0 < E; e0 += 256 / kSplit) {
            const int e = e0 + threadIdx.x / kSplit;
            float cs = 0.f;
            if (e < E)
                for (int b = sub; b < n_partials; b += kSplit) cs += colsum_partial[(int64_t)b * E + e];
#pragma unroll
            for (int off = kSplit / 2; off > 0; off >>= 1) cs += __shfl_xor(cs, off, kWave);
            if (e < E && sub == 0) colsum[e] = cs;
        }
        __syncthreads();
    }
    float local_fp = 0.f, local_load = 0.f;
    const float f_scale = (float)((double)E / ((double)k * (double)n_tokens));
    for (int e = threadIdx.x; e < E; e += 256) {
        const float load = (float)counts[e];
        local_load += load;
        if (aux_out && colsum_partial) local_fp += (load * f_scale) * (colsum[e] / (float)n_tokens);
    }
    red[threadIdx.x] = local_fp;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0 && aux_out) aux_out[0] = aux_coef * red[0];
    __syncthreads();
    red[threadIdx.x] = local_load;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (bias && bias_rate != 0.f) {
        const float mean = red[0] / (float)E;
        for (int e = threadIdx.x; e < E; e += 256) {
            const float d = mean - (float)counts[e];
            const float sgn = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
            bias[e] += bias_rate * sgn;
        }
    }
}

struct RouteShape {
    int G, EPL;
};
inline bool route_shape(int E, RouteShape* rs) {
    if (E < 1 || E > 1024) return false;
    if (E <= 16) {
        rs->G = E <= 8 ? 8 : 16;
        rs->EPL = 1;
    } else if (E <= 64) {
        // 16 lanes per token with 2 or 4 experts each: four tokens per wave and four shuffle steps per reduction
        // (one token per wave and six steps at 64 experts took 38 us for 16384 tokens)
        rs->G = 16;
        rs->EPL = E <= 32 ? 2 : 4;
    } else {
        int epl = 2;
        while (64 * epl < E) epl <<= 1;
        rs->G = 64;
        rs->EPL = epl;
    }
    return true;
}

}  // namespace

namespace {

// Calls f(integral_constant<G>, integral_constant<EPL>) for the (G, EPL) pair route_shape chose.
template <typename F>
void for_route_shape(const RouteShape& rs, F&& f) {
#define PICOMOE_RS(G_, EPL_) \
    if (rs.G == G_ && rs.EPL == EPL_) return f(std::integral_constant<int, G_>{}, std::integral_constant<int, EPL_>{});
    PICOMOE_RS(8, 1) PICOMOE_RS(16, 1) PICOMOE_RS(16, 2) PICOMOE_RS(16, 4)
    PICOMOE_RS(64, 2) PICOMOE_RS(64, 4) PICOMOE_RS(64, 8) PICOMOE_RS(64, 16)
#undef PICOMOE_RS
}

template <typename T>
void launch_route_fwd(const RouteShape& rs, int blocks, hipStream_t st, const void* logits, int64_t n_tokens, int E, int k,
                      const float* bias, int norm, int64_t* idx, void* w, float* probs, int* counts, float* partial) {
    for_route_shape(rs, [&](auto g, auto epl) {
        route_fwd_kernel<T, decltype(g)::value, decltype(epl)::value><<<dim3(blocks), dim3(kRouteBlock), 0, st>>>(
            (const T*)logits, n_tokens, E, k, bias, norm, idx, (T*)w, probs, counts, partial);
    });
}

template <typename T>
void launch_route_bwd(const RouteShape& rs, unsigned blocks, hipStream_t st, const float* probs, const int64_t* idx,
                      const void* d_w, int64_t n_tokens, int E, int k, int norm, const float* d_aux, const int* counts,
                      float aux_coef, void* d_logits) {
    for_route_shape(rs, [&](auto g, auto epl) {
        route_bwd_kernel<T, decltype(g)::value, decltype(epl)::value><<<dim3(blocks), dim3(kRouteBlock), 0, st>>>(
            probs, idx, (const T*)d_w, n_tokens, E, k, norm, d_aux, counts, aux_coef, (T*)d_logits);
    });
}

// ---- gradient of the gate Linear towards the tokens ---------------------------------------------------------------
// d_x[t, :] = addend[t, :] + d_logits[t, :] @ W,  W [E, hidden] with E <= 16: an [n_tokens, E] x [E, hidden] product is E
// multiply-adds per element written, so the pass is paid in bytes; done beside the sum of the tokens' two gradient paths
// (router and experts) it costs one read and one write of [n_tokens, hidden] where a GEMM followed by an add costs a
// write, two reads and a write.  A thread keeps its V columns of all E rows of W in registers and walks the tokens of its
// block; the E gradient logits of a token are loaded by the first E lanes and handed round as scalars.
// Rounding: the product is rounded to T, then the sum with the addend is rounded to T (a GEMM in T followed by an add in T).
template <typename T, int V>
struct Cols;
template <>
struct Cols<uint16_t, 8> {
    typedef u32x4_t raw_t;
    static __device__ __forceinline__ void widen(raw_t r, float (&f)[8]) {
        const uint32_t a[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(a[i] << 16);
            f[2 * i + 1] = __uint_as_float(a[i] & 0xFFFF0000u);
        }
    }
    static __device__ __forceinline__ raw_t narrow(const float (&f)[8]) {
        return raw_t{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
    }
    // every value rounded to bf16 and widened again: the packed conversion, then the two halves of each word
    static __device__ __forceinline__ void round_all(float (&f)[8]) { widen(narrow(f), f); }
};
template <>
struct Cols<float, 4> {
    typedef f32x4_t raw_t;
    static __device__ __forceinline__ void widen(raw_t r, float (&f)[4]) { f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w; }
    static __device__ __forceinline__ raw_t narrow(const float (&f)[4]) { return raw_t{f[0], f[1], f[2], f[3]}; }
    static __device__ __forceinline__ void round_all(float (&)[4]) {}
};

constexpr int kGateDgradMaxExperts = 16;
constexpr int kGateDgradTokensInFlight = 4;

template <typename T, int V, int EMAX>
__global__ __launch_bounds__(256) void gate_dgrad_kernel(const T* __restrict__ d_logits, const T* __restrict__ w,
                                                         const T* __restrict__ addend, int64_t n_tokens, int E, int64_t hidden,
                                                         T* __restrict__ out) {
    typedef Cols<T, V> C;
    typedef typename C::raw_t raw_t;
    const int lane = threadIdx.x & 63;
    const int64_t col = ((int64_t)blockIdx.y * 256 + threadIdx.x) * V;
    const bool live = col < hidden;  // hidden is a multiple of V: a thread's columns are all inside or all outside
    float wr[EMAX][V];
#pragma unroll
    for (int e = 0; e < EMAX; ++e) {
#pragma unroll
        for (int i = 0; i < V; ++i) wr[e][i] = 0.f;
        if (e < E && live) C::widen(*(const raw_t*)(w + (int64_t)e * hidden + col), wr[e]);
    }
    constexpr int U = kGateDgradTokensInFlight;
    for (int64_t t0 = blockIdx.x; t0 < n_tokens; t0 += (int64_t)gridDim.x * U) {
        raw_t a[U];
        float dl[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t t = t0 + (int64_t)u * gridDim.x;
            dl[u] = 0.f;
            if (t < n_tokens) {  // uniform over the block
                if (lane < E) dl[u] = to_f32<T>(d_logits[t * E + lane]);
                if (addend && live) a[u] = *(const raw_t*)(addend + t * hidden + col);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t t = t0 + (int64_t)u * gridDim.x;
            if (t >= n_tokens) break;
            float acc[V];
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] = 0.f;
#pragma unroll
            for (int e = 0; e < EMAX; ++e) {
                const float d = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(dl[u]), e));  // 0 for e >= E
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] = fmaf(d, wr[e][i], acc[i]);
            }
            if (addend) {
                float av[V];
                if (live) C::widen(a[u], av);
                C::round_all(acc);
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] += live ? av[i] : 0.f;
            }
            if (live) *(raw_t*)(out + t * hidden + col) = C::narrow(acc);
        }
    }
}

template <typename T, int V>
void launch_gate_dgrad(hipStream_t st, const void* d_logits, const void* w, const void* addend, int64_t n_tokens, int E,
                       int64_t hidden, void* out) {
    const int64_t cols_per_block = 256 * V;
    const dim3 grid((unsigned)(n_tokens < 512 ? n_tokens : 512), (unsigned)((hidden + cols_per_block - 1) / cols_per_block));
    if (E <= 8)
        gate_dgrad_kernel<T, V, 8><<<grid, dim3(256), 0, st>>>((const T*)d_logits, (const T*)w, (const T*)addend, n_tokens, E,
                                                               hidden, (T*)out);
    else
        gate_dgrad_kernel<T, V, kGateDgradMaxExperts><<<grid, dim3(256), 0, st>>>((const T*)d_logits, (const T*)w,
                                                                                  (const T*)addend, n_tokens, E, hidden, (T*)out);
}

// The gate's weight gradient d_w[e, :] = sum_t d_logits[t, e] * x[t, :]: E multiply-adds per element of x read, against
// columns the thread owns, so it runs at the rate x can be read -- a GEMM with an E-row output reaches a fifth of that.
// A block's four wavefronts own the same 64 * V columns and every fourth token of the block's share; their sums meet in
// LDS in wave order, the blocks' sums in `partial` [gridDim.x][E][hidden] fp32, which gate_wgrad_reduce_kernel adds in
// block order: no atomics, one fixed order.  (One kernel for d_x and d_w together was measured and dropped: with W and
// the sums both in registers two wavefronts fit a SIMD and the pass ran at 2.8 TB/s, no faster than the two apart.)
constexpr int kGateBwdMaxExperts = 8;
constexpr int kGateWgradTokensInFlight = 4;  // per batch, two batches

template <typename T, int V>
__global__ __launch_bounds__(256) void gate_wgrad_kernel(const T* __restrict__ d_logits, const T* __restrict__ x, int64_t n_tokens,
                                                         int E, int64_t hidden, float* __restrict__ partial) {
    typedef Cols<T, V> C;
    typedef typename C::raw_t raw_t;
    constexpr int EMAX = kGateBwdMaxExperts;
    __shared__ float red[3][EMAX * V][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t col = ((int64_t)blockIdx.y * 64 + lane) * V;
    const bool live = col < hidden;
    float dw[EMAX][V];
#pragma unroll
    for (int e = 0; e < EMAX; ++e)
#pragma unroll
        for (int i = 0; i < V; ++i) dw[e][i] = 0.f;
    // two batches of U tokens: the loads of one are in flight while the other is summed
    constexpr int U = kGateWgradTokensInFlight;
    const int64_t stride = (int64_t)gridDim.x * 4, step = stride * U;
    auto load = [&](raw_t (&xr)[U], float (&dl)[U], int64_t t0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t t = t0 + u * stride;
            dl[u] = 0.f;
            if (t < n_tokens) {  // uniform over the wavefront
                if (lane < E) dl[u] = to_f32<T>(d_logits[t * E + lane]);
                if (live) xr[u] = *(const raw_t*)(x + t * hidden + col);
            }
        }
    };
    auto accumulate = [&](const raw_t (&xr)[U], const float (&dl)[U], int64_t t0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (t0 + u * stride >= n_tokens || !live) break;
            float xv[V];
            C::widen(xr[u], xv);
#pragma unroll
            for (int e = 0; e < EMAX; ++e) {
                const float d = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(dl[u]), e));  // 0 for e >= E
#pragma unroll
                for (int i = 0; i < V; ++i) dw[e][i] = fmaf(d, xv[i], dw[e][i]);
            }
        }
    };
    raw_t xa[U], xb[U];
    float da[U], db[U];
    int64_t t0 = (int64_t)blockIdx.x * 4 + wave;
    if (t0 < n_tokens) load(xa, da, t0);
    while (t0 < n_tokens) {
        if (t0 + step < n_tokens) load(xb, db, t0 + step);
        accumulate(xa, da, t0);
        t0 += step;
        if (t0 >= n_tokens) break;
        if (t0 + step < n_tokens) load(xa, da, t0 + step);
        accumulate(xb, db, t0);
        t0 += step;
    }
    if (wave > 0) {
#pragma unroll
        for (int e = 0; e < EMAX; ++e)
#pragma unroll
            for (int i = 0; i < V; ++i) red[wave - 1][e * V + i][lane] = dw[e][i];
    }
    __syncthreads();
    if (wave == 0 && live) {
#pragma unroll
        for (int e = 0; e < EMAX; ++e) {  // unrolled with a test inside: an index the compiler cannot see would move dw out of the registers
            if (e >= E) break;
            float* dst = partial + ((int64_t)blockIdx.x * E + e) * hidden + col;
#pragma unroll
            for (int i = 0; i < V; i += 4) {
                f32x4_t o;
                o.x = ((dw[e][i] + red[0][e * V + i][lane]) + red[1][e * V + i][lane]) + red[2][e * V + i][lane];
                o.y = ((dw[e][i + 1] + red[0][e * V + i + 1][lane]) + red[1][e * V + i + 1][lane]) + red[2][e * V + i + 1][lane];
                o.z = ((dw[e][i + 2] + red[0][e * V + i + 2][lane]) + red[1][e * V + i + 2][lane]) + red[2][e * V + i + 2][lane];
                o.w = ((dw[e][i + 3] + red[0][e * V + i + 3][lane]) + red[1][e * V + i + 3][lane]) + red[2][e * V + i + 3][lane];
                *(f32x4_t*)(dst + i) = o;
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void gate_wgrad_reduce_kernel(const float* __restrict__ partial, int n_partials, int64_t n,
                                                                T* __restrict__ d_w) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = 0.f;
    int g = 0;
    for (; g + 16 <= n_partials; g += 16) {  // sixteen loads in flight, added in block order
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = partial[(int64_t)(g + j) * n + i];
#pragma unroll
        for (int j = 0; j < 16; ++j) s += v[j];
    }
    for (; g < n_partials; ++g) s += partial[(int64_t)g * n + i];
    d_w[i] = from_f32<T>(s);
}

// token groups (= partial sums of d_w) of a weight-gradient launch: three blocks per CU over the column slabs (what the
// 48 KB of LDS a block takes allows), at least one round of four tokens per block
int gate_bwd_groups(int64_t n_tokens, int64_t hidden, int V) {
    const int64_t slabs = (hidden + 64 * V - 1) / (64 * V);
    int64_t g = 768 / slabs;
    g = g < 8 ? 8 : (g > 96 ? 96 : g);
    const int64_t need = (n_tokens + 3) / 4;
    if (g > need) g = need;
    return (int)(g < 1 ? 1 : g);
}

template <typename T, int V>
void launch_gate_wgrad(hipStream_t st, const void* d_logits, const void* x, int64_t n_tokens, int E, int64_t hidden, void* d_w,
                       float* partial) {
    const int groups = gate_bwd_groups(n_tokens, hidden, V);
    const dim3 grid((unsigned)groups, (unsigned)((hidden + 64 * V - 1) / (64 * V)));
    gate_wgrad_kernel<T, V><<<grid, dim3(256), 0, st>>>((const T*)d_logits, (const T*)x, n_tokens, E, hidden, partial);
    const int64_t n = (int64_t)E * hidden;
    gate_wgrad_reduce_kernel<T><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>(partial, groups, n, (T*)d_w);
}

}  // namespace

extern "C" int picomoe_route_partials(int64_t n_tokens, int num_experts) {
    RouteShape rs;
    if (!route_shape(num_experts, &rs) || n_tokens < 0) return -1;
    const int64_t per_block = kRouteBlock / rs.G;
    int64_t blocks = (n_tokens + per_block - 1) / per_block;
    if (blocks > 1024) blocks = 1024;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

extern "C" int picomoe_route_fwd(const void* logits, int dtype, int64_t n_tokens, int num_experts, int top_k,
                                 const float* expert_bias, int norm_topk, int64_t* topk_idx, void* topk_w, float* probs,
                                 int* counts, float* colsum_partial, void* stream) {
    RouteShape rs;
    PICOMOE_CHECK_ARG(route_shape(num_experts, &rs));
    PICOMOE_CHECK_ARG(dtype == PICOMOE_F32 || dtype == PICOMOE_BF16);
    PICOMOE_CHECK_ARG(top_k >= 1 && top_k <= kMaxTopK && top_k <= num_experts && n_tokens >= 0);
    if (n_tokens == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(logits && topk_idx && topk_w);
    const int blocks = picomoe_route_partials(n_tokens, num_experts);
    hipStream_t st = (hipStream_t)stream;
    const int E = num_experts;
    if (dtype == PICOMOE_F32)
        launch_route_fwd<float>(rs, blocks, st, logits, n_tokens, E, top_k, expert_bias, norm_topk, topk_idx, topk_w, probs,
                                counts, colsum_partial);
    else
        launch_route_fwd<uint16_t>(rs, blocks, st, logits, n_tokens, E, top_k, expert_bias, norm_topk, topk_idx, topk_w,
                                   probs, counts, colsum_partial);
    return picomoe_launch_status();
}

extern "C" int picomoe_route_bwd(const float* probs, const int64_t* topk_idx, const void* d_topk_w, int dtype,
                                 int64_t n_tokens, int num_experts, int top_k, int norm_topk, const float* d_aux,
                                 const int* counts, float aux_coef, void* d_logits, void* stream) {
    RouteShape rs;
    PICOMOE_CHECK_ARG(route_shape(num_experts, &rs));
    PICOMOE_CHECK_ARG(dtype == PICOMOE_F32 || dtype == PICOMOE_BF16);
    PICOMOE_CHECK_ARG(top_k >= 1 && top_k <= kMaxTopK && top_k <= num_experts && n_tokens >= 0);
    if (n_tokens == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(probs && topk_idx && d_logits);
    hipStream_t st = (hipStream_t)stream;
    const int E = num_experts;
    const int64_t per_block = kRouteBlock / rs.G;
    const unsigned blocks = (unsigned)((n_tokens + per_block - 1) / per_block);
    if (dtype == PICOMOE_F32)
        launch_route_bwd<float>(rs, blocks, st, probs, topk_idx, d_topk_w, n_tokens, E, top_k, norm_topk, d_aux, counts,
                                aux_coef, d_logits);
    else
        launch_route_bwd<uint16_t>(rs, blocks, st, probs, topk_idx, d_topk_w, n_tokens, E, top_k, norm_topk, d_aux, counts,
                                   aux_coef, d_logits);
    return picomoe_launch_status();
}

extern "C" int picomoe_balance(const int* counts, const float* colsum_partial, int n_partials, int64_t n_tokens,
                               int num_experts, int top_k, float aux_coef, float bias_rate, float* aux_out,
                               float* expert_bias, void* stream) {
    PICOMOE_CHECK_ARG(counts && num_experts >= 1 && num_experts <= 1024 && n_tokens > 0 && top_k >= 1);
    PICOMOE_CHECK_ARG(!aux_out || (colsum_partial && n_partials >= 1));
    hipLaunchKernelGGL(balance_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, counts, colsum_partial, n_partials,
                       n_tokens, num_experts, top_k, aux_coef, bias_rate, aux_out, expert_bias);
    return picomoe_launch_status();
}

extern "C" int64_t picomoe_gate_bwd_workspace_bytes(int dtype, int64_t n_tokens, int num_experts, int64_t hidden) {
    if ((dtype != PICOMOE_F32 && dtype != PICOMOE_BF16) || n_tokens < 0 || num_experts < 1 || hidden < 1) return -1;
    if (num_experts > kGateBwdMaxExperts) return 0;  // no fused weight gradient for this gate
    return (int64_t)gate_bwd_groups(n_tokens, hidden, dtype == PICOMOE_BF16 ? 8 : 4) * num_experts * hidden * (int64_t)sizeof(float);
}

extern "C" int picomoe_gate_bwd(const void* d_logits, const void* gate_w, const void* addend, const void* tokens, int dtype,
                                int64_t n_tokens, int num_experts, int64_t hidden, void* d_x, void* d_w, void* workspace,
                                int64_t workspace_bytes, void* stream) {
    PICOMOE_CHECK_ARG(dtype == PICOMOE_F32 || dtype == PICOMOE_BF16);
    PICOMOE_CHECK_ARG(n_tokens >= 0 && hidden > 0 && num_experts >= 1);
    PICOMOE_CHECK_ARG(num_experts <= (d_w ? kGateBwdMaxExperts : kGateDgradMaxExperts));
    PICOMOE_CHECK_ARG(hidden % (dtype == PICOMOE_BF16 ? 8 : 4) == 0 && hidden <= (1ll << 22));  // column slabs are the grid's y dimension
    hipStream_t st = (hipStream_t)stream;
    if (n_tokens == 0) {
        if (d_w) {  // the sum over no tokens: the reduction of zero partial sums writes the zeros (a kernel, so that a graph capture holds no memset node)
            const int64_t n = (int64_t)num_experts * hidden;
            if (dtype == PICOMOE_BF16)
                gate_wgrad_reduce_kernel<uint16_t><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>(nullptr, 0, n, (uint16_t*)d_w);
            else
                gate_wgrad_reduce_kernel<float><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>(nullptr, 0, n, (float*)d_w);
            return picomoe_launch_status();
        }
        return PICOMOE_OK;
    }
    PICOMOE_CHECK_ARG(d_logits && (d_x || d_w));
    if (d_x) PICOMOE_CHECK_ARG(gate_w && (uintptr_t)gate_w % 16 == 0 && (uintptr_t)addend % 16 == 0 && (uintptr_t)d_x % 16 == 0);
    if (d_w) {
        PICOMOE_CHECK_ARG(tokens && workspace && (uintptr_t)tokens % 16 == 0 && (uintptr_t)workspace % 16 == 0);
        PICOMOE_CHECK_ARG(workspace_bytes >= picomoe_gate_bwd_workspace_bytes(dtype, n_tokens, num_experts, hidden));
    }
    const bool bf16 = dtype == PICOMOE_BF16;
    if (d_x && bf16) launch_gate_dgrad<uint16_t, 8>(st, d_logits, gate_w, addend, n_tokens, num_experts, hidden, d_x);
    if (d_x && !bf16) launch_gate_dgrad<float, 4>(st, d_logits, gate_w, addend, n_tokens, num_experts, hidden, d_x);
    if (d_w && bf16) launch_gate_wgrad<uint16_t, 8>(st, d_logits, tokens, n_tokens, num_experts, hidden, d_w, (float*)workspace);
    if (d_w && !bf16) launch_gate_wgrad<float, 4>(st, d_logits, tokens, n_tokens, num_experts, hidden, d_w, (float*)workspace);
    return picomoe_launch_status();
}
