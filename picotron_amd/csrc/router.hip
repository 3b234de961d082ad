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
