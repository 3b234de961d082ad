// Token permute / unpermute for gfx950 -- the EP=1 replacement of the dispatch/combine all-to-all.
//
//   plan     stable counting sort of the routed rows by expert: per-block histogram, a scan over
//            blocks and experts, then a scatter whose rank inside an expert is computed from
//            wave ballots (never from the arrival order of atomics), so the permutation is the one
//            a stable argsort yields.  A capacity limit falls out of the same rank.
//   gather   out[i] = src[map[i] / div]   (expand token-major + permute in one pass)
//   combine  out[t] = sum_j w[t,j] * y[inv[t*k+j]]   and its backward
//
// All row movers use one wavefront per row and 16-byte lanes when the row width allows it.
#include <mutex>

#include "common.h"

namespace {

constexpr int kPlanBlock = 256;
constexpr int kPlanRowsPerThread = 4;
constexpr int kPlanChunk = kPlanBlock * kPlanRowsPerThread;  // rows per block
constexpr int kMaxExperts = 1024;
constexpr int kMaxTopK = 16;

// ---- plan -------------------------------------------------------------------------------------
__global__ __launch_bounds__(kPlanBlock) void plan_hist_kernel(const int64_t* __restrict__ expert_idx, int64_t n_rows,
                                                               int E, int* __restrict__ block_hist,
                                                               int* __restrict__ order) {
    extern __shared__ int hist[];
    for (int e = threadIdx.x; e < E; e += kPlanBlock) hist[e] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kPlanChunk;
    for (int i = 0; i < kPlanRowsPerThread; ++i) {
        const int64_t r = base + i * kPlanBlock + threadIdx.x;
        if (r < n_rows) {
            const int64_t e = expert_idx[r];
            if (e >= 0 && e < E) atomicAdd(&hist[(int)e], 1);  // ids outside [0,E) are treated as dropped rows
            order[r] = -1;
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += kPlanBlock) block_hist[(int64_t)blockIdx.x * E + e] = hist[e];
}

// block_hist[b][e] becomes the number of rows of expert e in blocks before b; then experts are laid
// out back to back using the kept (capacity-limited) counts.
// One wave per expert (16 waves take the experts in turn): the per-block counts of an expert are scanned 64 blocks at a
// time with wave shuffles instead of one thread walking all blocks (25 us for 96 blocks x 64 experts, now a few).
constexpr int kScanThreads = 1024;
__global__ __launch_bounds__(kScanThreads) void plan_scan_kernel(int* __restrict__ block_hist, int n_blocks, int E, int64_t capacity,
                                                                 int64_t slot_lo, int64_t* __restrict__ counts,
                                                                 int64_t* __restrict__ kept_counts, int* __restrict__ seg_start) {
    __shared__ int kept[kMaxExperts];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, n_waves = kScanThreads / 64;
    auto wave_scan = [&](int v) {  // inclusive prefix sum over the 64 lanes
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int o = __shfl_up(v, off, 64);
            if (lane >= off) v += o;
        }
        return v;
    };
    for (int e = wave; e < E; e += n_waves) {
        int run = 0;
        for (int b0 = 0; b0 < n_blocks; b0 += 64) {
            const int b = b0 + lane;
            const int c = b < n_blocks ? block_hist[(int64_t)b * E + e] : 0;
            const int incl = wave_scan(c);
            if (b < n_blocks) block_hist[(int64_t)b * E + e] = run + incl - c;
            run += __shfl(incl, 63, 64);
        }
        if (lane == 0) {
            int64_t kc64 = run;  // rows of e whose rank falls in [slot_lo, slot_lo + capacity)
            if (capacity > 0) {
                kc64 = run - slot_lo;
                kc64 = kc64 < 0 ? 0 : (kc64 > capacity ? capacity : kc64);
            }
            kept[e] = (int)kc64;
            counts[e] = run;
            kept_counts[e] = kc64;
        }
    }
    __syncthreads();
    if (wave == 0) {  // experts laid out back to back by their kept counts
        int run = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int k = e < E ? kept[e] : 0;
            const int incl = wave_scan(k);
            if (e < E) seg_start[e] = run + incl - k;
            run += __shfl(incl, 63, 64);
        }
    }
}

__global__ __launch_bounds__(kPlanBlock) void plan_scatter_kernel(const int64_t* __restrict__ expert_idx, int64_t n_rows,
                                                                  int E, int n_bits, int64_t capacity, int64_t slot_lo,
                                                                  const int* __restrict__ block_base,
                                                                  const int* __restrict__ seg_start,
                                                                  int* __restrict__ order, int* __restrict__ inv_order,
                                                                  int* __restrict__ within_out) {
    extern __shared__ int lds[];
    int* wave_hist = lds;            // [4][E] rows of expert e handled by wave w
    int* wave_run = lds + 4 * E;     // [4][E] rows of expert e already ranked by wave w
    for (int i = threadIdx.x; i < 8 * E; i += kPlanBlock) lds[i] = 0;
    __syncthreads();

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // wave w owns rows [base + w*256, base + (w+1)*256): consecutive rows, 64 at a time
    const int64_t wbase = (int64_t)blockIdx.x * kPlanChunk + wave * (kWave * kPlanRowsPerThread);
    int my_e[kPlanRowsPerThread];
#pragma unroll
    for (int i = 0; i < kPlanRowsPerThread; ++i) {
        const int64_t r = wbase + i * kWave + lane;
        int e = -1;
        if (r < n_rows) {
            const int64_t v = expert_idx[r];
            if (v >= 0 && v < E) e = (int)v;
        }
        my_e[i] = e;
        if (e >= 0) atomicAdd(&wave_hist[wave * E + e], 1);
    }
    __syncthreads();

    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int i = 0; i < kPlanRowsPerThread; ++i) {
        const int64_t r = wbase + i * kWave + lane;
        const int e = my_e[i];
        uint64_t peers = __ballot(e >= 0);
        for (int b = 0; b < n_bits; ++b) {
            const uint64_t has = __ballot((e >> b) & 1);
            peers &= ((e >> b) & 1) ? has : ~has;
        }
        if (e >= 0) {
            int before = block_base[(int64_t)blockIdx.x * E + e] + wave_run[wave * E + e];
            for (int w2 = 0; w2 < wave; ++w2) before += wave_hist[w2 * E + e];
            const int within = before + __popcll(peers & lt_mask);
            // the highest peer lane records how many rows of e this step ranked
            if ((peers >> lane) == 1ull) wave_run[wave * E + e] += __popcll(peers);
            if (within_out) within_out[r] = within;
            if (capacity > 0 && (within < slot_lo || within >= slot_lo + capacity)) {
                inv_order[r] = -1;
            } else {
                const int pos = seg_start[e] + within - (int)slot_lo;
                inv_order[r] = pos;
                order[pos] = (int)r;
            }
        } else if (r < n_rows) {
            inv_order[r] = -1;
            if (within_out) within_out[r] = -1;
        }
    }
}

// ---- row movers -------------------------------------------------------------------------------
template <typename T, int V>
struct Vec;
template <>
struct Vec<uint16_t, 8> {
    float v[8];
    typedef u32x4_t raw_t;  // what a load leaves in registers before it is widened to fp32
    static __device__ __forceinline__ raw_t load_raw(const uint16_t* p) { return *(const u32x4_t*)p; }
    __device__ __forceinline__ void load(const uint16_t* p) { set(load_raw(p)); }
    __device__ __forceinline__ void set(raw_t w) {
        const uint32_t a[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(a[i] << 16);
            v[2 * i + 1] = __uint_as_float(a[i] & 0xFFFF0000u);
        }
    }
    __device__ __forceinline__ void store(uint16_t* p) const {
        u32x4_t w;
        w.x = pack_bf16x2(v[0], v[1]);
        w.y = pack_bf16x2(v[2], v[3]);
        w.z = pack_bf16x2(v[4], v[5]);
        w.w = pack_bf16x2(v[6], v[7]);
        *(u32x4_t*)p = w;
    }
};
template <>
struct Vec<uint16_t, 1> {
    float v[1];
    typedef uint16_t raw_t;
    static __device__ __forceinline__ raw_t load_raw(const uint16_t* p) { return *p; }
    __device__ __forceinline__ void set(raw_t w) { v[0] = bf16_bits_to_f32(w); }
    __device__ __forceinline__ void load(const uint16_t* p) { v[0] = bf16_bits_to_f32(*p); }
    __device__ __forceinline__ void store(uint16_t* p) const { *p = (uint16_t)f32_to_bf16_bits(v[0]); }
};
template <>
struct Vec<float, 4> {
    float v[4];
    typedef f32x4_t raw_t;
    static __device__ __forceinline__ raw_t load_raw(const float* p) { return *(const f32x4_t*)p; }
    __device__ __forceinline__ void set(raw_t w) { v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w; }
    __device__ __forceinline__ void load(const float* p) { set(load_raw(p)); }
    __device__ __forceinline__ void store(float* p) const { *(f32x4_t*)p = f32x4_t{v[0], v[1], v[2], v[3]}; }
};
template <>
struct Vec<float, 1> {
    float v[1];
    typedef float raw_t;
    static __device__ __forceinline__ raw_t load_raw(const float* p) { return *p; }
    __device__ __forceinline__ void set(raw_t w) { v[0] = w; }
    __device__ __forceinline__ void load(const float* p) { v[0] = *p; }
    __device__ __forceinline__ void store(float* p) const { *p = v[0]; }
};

// rounding of an intermediate to the tensor dtype (what a torch op on that dtype does)
template <typename T>
__device__ __forceinline__ float round_to(float x);
template <>
__device__ __forceinline__ float round_to<float>(float x) { return x; }
template <>
__device__ __forceinline__ float round_to<uint16_t>(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }

template <typename T, int V>
__global__ __launch_bounds__(256) void gather_rows_kernel(const T* __restrict__ src, const int* __restrict__ row_map,
                                                          int div, int64_t n_out, int64_t hidden, T* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n_out) return;
    const int m = row_map ? row_map[i] : (int)i;
    if (m < 0) return;
    const T* s = src + (int64_t)(m / div) * hidden;
    T* d = out + i * hidden;
    for (int64_t c = (int64_t)(threadIdx.x & 63) * V; c < hidden; c += 64 * V) {
        Vec<T, V> x;
        x.load(s + c);
        x.store(d + c);
    }
}

// out[t] = sum_j w[t,j] * y[inv[t*k+j]].  Each product is rounded to T, the sum is carried in fp32
// and rounded once: what both a reshape-sum over k and a CPU index_add into a zeroed T buffer do.
// Rows with inv < 0 (dropped) add nothing.  w == nullptr means unit weights without the product rounding.
// KMAX: compile-time bound of k (2, 8 or kMaxTopK).  A wave works on one token, so the row positions are wave-uniform
// (kept in scalar registers); per column chunk all of the token's rows are loaded first and summed afterwards, so the
// k loads are in flight together.
template <typename T, int V, int KMAX>
__global__ __launch_bounds__(256) void combine_fwd_kernel(const T* __restrict__ y, const int* __restrict__ inv,
                                                          const T* __restrict__ w, int64_t n_tokens, int k, int64_t hidden,
                                                          T* __restrict__ out) {
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    int pos[KMAX];
    float wj[KMAX];
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
        pos[j] = -1;
        wj[j] = 0.f;
        if (j < k) {
            pos[j] = __builtin_amdgcn_readfirstlane(inv ? inv[t * k + j] : (int)(t * k + j));
            if (w) {
                Vec<T, 1> s;
                s.load(w + t * k + j);
                wj[j] = s.v[0];
            } else {
                wj[j] = 1.f;
            }
        }
    }
    for (int64_t c = (int64_t)(threadIdx.x & 63) * V; c < hidden; c += 64 * V) {
        typename Vec<T, V>::raw_t raw[KMAX];
#pragma unroll
        for (int j = 0; j < KMAX; ++j)
            if (pos[j] >= 0) raw[j] = Vec<T, V>::load_raw(y + (int64_t)pos[j] * hidden + c);
        Vec<T, V> acc;
#pragma unroll
        for (int i = 0; i < V; ++i) acc.v[i] = 0.f;
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
            if (pos[j] >= 0) {
                Vec<T, V> x;
                x.set(raw[j]);
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const float prod = w ? round_to<T>(x.v[i] * wj[j]) : x.v[i];
                    acc.v[i] += prod;
                }
            }
        }
        acc.store(out + t * hidden + c);
    }
}

// d y[inv[t*k+j]] = w[t,j] * d out[t];   d w[t,j] = <d out[t], y[inv[t*k+j]]>
template <typename T, int V, int KMAX>
__global__ __launch_bounds__(256) void combine_bwd_kernel(const T* __restrict__ d_out, const T* __restrict__ y,
                                                          const int* __restrict__ inv, const T* __restrict__ w,
                                                          int64_t n_tokens, int k, int64_t hidden, T* __restrict__ d_y,
                                                          T* __restrict__ d_w) {
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    const int lane = threadIdx.x & 63;
    int pos[KMAX];
    float wj[KMAX], dot[KMAX];
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
        dot[j] = 0.f;
        pos[j] = -1;
        wj[j] = 0.f;
        if (j < k) {
            pos[j] = __builtin_amdgcn_readfirstlane(inv ? inv[t * k + j] : (int)(t * k + j));
            Vec<T, 1> s;
            s.load(w + t * k + j);
            wj[j] = s.v[0];
        }
    }
    for (int64_t c = (int64_t)lane * V; c < hidden; c += 64 * V) {
        Vec<T, V> g;
        g.load(d_out + t * hidden + c);
        typename Vec<T, V>::raw_t raw[KMAX];
#pragma unroll
        for (int j = 0; j < KMAX; ++j)
            if (pos[j] >= 0) raw[j] = Vec<T, V>::load_raw(y + (int64_t)pos[j] * hidden + c);
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
            if (pos[j] >= 0) {
                Vec<T, V> x, o;
                x.set(raw[j]);
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    o.v[i] = g.v[i] * wj[j];
                    dot[j] += g.v[i] * x.v[i];
                }
                o.store(d_y + (int64_t)pos[j] * hidden + c);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
        if (j < k) {
            const float tot = wave_sum(dot[j]);
            if (lane == 0) {
                Vec<T, 1> s;
                s.v[0] = tot;
                s.store(d_w + t * k + j);
            }
        }
    }
}

template <typename T>
constexpr int vec_width() { return sizeof(T) == 2 ? 8 : 4; }

template <typename T>
bool can_vec(int64_t hidden, const void* a, const void* b, const void* c = nullptr) {
    const int v = vec_width<T>();
    return hidden % v == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)b % 16 == 0 && (uintptr_t)c % 16 == 0;
}

}  // namespace

extern "C" int64_t picomoe_permute_workspace_bytes(int64_t n_rows, int num_experts) {
    if (n_rows < 0 || num_experts < 1 || num_experts > kMaxExperts) return -1;
    const int64_t n_blocks = (n_rows + kPlanChunk - 1) / kPlanChunk;
    return (n_blocks * num_experts + num_experts) * (int64_t)sizeof(int);
}

// Scratch of the no-allocation entry point (picomoe_permute_plan_static): file scope, one copy per GPU.
constexpr int64_t kStaticPlanInts = PICOMOE_PLAN_STATIC_BYTES / (int64_t)sizeof(int);
static __device__ __align__(256) int scratch[kStaticPlanInts];

namespace {
// the three launches of a plan; `workspace` holds n_blocks * E block histograms followed by E segment starts (ints).
// Every entry that is read has been written by an earlier launch of the same call: nothing has to start at zero.
int plan_launch(const int64_t* expert_idx, int64_t n_rows, int E, int64_t capacity, int64_t round_index, int32_t* order,
                int32_t* inv_order, int64_t* counts, int64_t* kept_counts, int32_t* within, int* workspace, hipStream_t st) {
    const int n_blocks = (int)((n_rows + kPlanChunk - 1) / kPlanChunk);
    int* block_hist = workspace;
    int* seg_start = block_hist + (int64_t)n_blocks * E;
    if (n_rows > 0) {
        hipLaunchKernelGGL(plan_hist_kernel, dim3(n_blocks), dim3(kPlanBlock), E * sizeof(int), st, expert_idx, n_rows, E,
                           block_hist, order);
    }
    const int64_t slot_lo = capacity > 0 ? round_index * capacity : 0;
    hipLaunchKernelGGL(plan_scan_kernel, dim3(1), dim3(kScanThreads), 0, st, block_hist, n_blocks, E, capacity, slot_lo, counts,
                       kept_counts, seg_start);
    if (n_rows > 0) {
        int n_bits = 0;
        while ((1 << n_bits) < E) ++n_bits;
        hipLaunchKernelGGL(plan_scatter_kernel, dim3(n_blocks), dim3(kPlanBlock), 8 * E * sizeof(int), st, expert_idx, n_rows,
                           E, n_bits, capacity, slot_lo, block_hist, seg_start, order, inv_order, within);
    }
    return picomoe_launch_status();
}

bool plan_args_ok(const int64_t* expert_idx, int64_t n_rows, int num_experts, int64_t capacity, int64_t round_index,
                  const int32_t* order, const int32_t* inv_order, const int64_t* counts, const int64_t* kept_counts) {
    if (!(n_rows >= 0 && n_rows < (1ll << 31) && num_experts >= 1 && num_experts <= kMaxExperts && capacity >= 0 && round_index >= 0))
        return false;
    if (!counts || !kept_counts) return false;
    return n_rows == 0 || (expert_idx && order && inv_order);
}

// ---- the plan without a caller-provided workspace -------------------------------------------------------------
// Scratch of the no-allocation entry point: block histograms + segment starts of one plan, 1 MiB per GPU, held from the
// moment the library is loaded until the process ends.  In host code `scratch` is only a handle for
// hipGetSymbolAddress; kernels get the device address that call returns (each GPU has its own copy of the array).
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
int* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each GPU, looked up on the first call there

// Device address of this GPU's scratch array (looked up once per device, with that device current), or null + *rc.
int* static_scratch(int* rc) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { *rc = PICOMOE_ERR_HIP_BASE + (int)e; return nullptr; }
    if (dev < 0 || dev >= kMaxDevices) { *rc = PICOMOE_ERR_ARG; return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) { *rc = PICOMOE_ERR_HIP_BASE + (int)(e != hipSuccess ? e : hipErrorInvalidSymbol); return nullptr; }
        g_scratch_ptr[dev] = (int*)ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int picomoe_permute_plan(const int64_t* expert_idx, int64_t n_rows, int num_experts, int64_t capacity,
                                    int64_t round_index, int32_t* order, int32_t* inv_order, int64_t* counts, int64_t* kept_counts,
                                    int32_t* within, void* workspace, void* stream) {
    PICOMOE_CHECK_ARG(plan_args_ok(expert_idx, n_rows, num_experts, capacity, round_index, order, inv_order, counts, kept_counts));
    PICOMOE_CHECK_ARG(workspace);
    return plan_launch(expert_idx, n_rows, num_experts, capacity, round_index, order, inv_order, counts, kept_counts, within,
                       (int*)workspace, (hipStream_t)stream);
}

extern "C" int64_t picomoe_permute_plan_static_max_bytes(void) { return PICOMOE_PLAN_STATIC_BYTES; }

extern "C" int picomoe_permute_plan_static_init(void) {
    int rc = PICOMOE_OK;
    return static_scratch(&rc) ? PICOMOE_OK : rc;
}

extern "C" int picomoe_permute_plan_static(const int64_t* expert_idx, int64_t n_rows, int num_experts, int64_t capacity,
                                           int64_t round_index, int32_t* order, int32_t* inv_order, int64_t* counts,
                                           int64_t* kept_counts, int32_t* within, void* stream) {
    PICOMOE_CHECK_ARG(plan_args_ok(expert_idx, n_rows, num_experts, capacity, round_index, order, inv_order, counts, kept_counts));
    const int64_t need = picomoe_permute_workspace_bytes(n_rows, num_experts);
    if (need < 0 || need > PICOMOE_PLAN_STATIC_BYTES) return PICOMOE_ERR_TOO_LARGE;
    int rc = PICOMOE_OK;
    int* ws = static_scratch(&rc);
    if (!ws) return rc;
    return plan_launch(expert_idx, n_rows, num_experts, capacity, round_index, order, inv_order, counts, kept_counts, within, ws,
                       (hipStream_t)stream);
}

extern "C" int picomoe_gather_rows(const void* src, const int32_t* row_map, int div, int64_t n_out, int64_t hidden,
                                   int dtype, void* out, void* stream) {
    PICOMOE_CHECK_ARG(n_out >= 0 && hidden > 0 && div >= 1 && (dtype == PICOMOE_F32 || dtype == PICOMOE_BF16));
    if (n_out == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(src && out);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)((n_out + 3) / 4)), block(256);
    if (dtype == PICOMOE_BF16) {
        if (can_vec<uint16_t>(hidden, src, out))
            hipLaunchKernelGGL((gather_rows_kernel<uint16_t, 8>), grid, block, 0, st, (const uint16_t*)src, row_map, div, n_out, hidden, (uint16_t*)out);
        else
            hipLaunchKernelGGL((gather_rows_kernel<uint16_t, 1>), grid, block, 0, st, (const uint16_t*)src, row_map, div, n_out, hidden, (uint16_t*)out);
    } else {
        if (can_vec<float>(hidden, src, out))
            hipLaunchKernelGGL((gather_rows_kernel<float, 4>), grid, block, 0, st, (const float*)src, row_map, div, n_out, hidden, (float*)out);
        else
            hipLaunchKernelGGL((gather_rows_kernel<float, 1>), grid, block, 0, st, (const float*)src, row_map, div, n_out, hidden, (float*)out);
    }
    return picomoe_launch_status();
}

namespace {
template <typename T>
void launch_combine_fwd(hipStream_t st, const void* y, const int* inv, const void* w, int64_t n_tokens, int k, int64_t hidden,
                        void* out) {
    const dim3 grid((unsigned)((n_tokens + 3) / 4)), block(256);
    constexpr int V = sizeof(T) == 2 ? 8 : 4;
    const bool vec = can_vec<T>(hidden, y, out);
#define PICOMOE_LAUNCH_CF(VV, KK) \
    hipLaunchKernelGGL((combine_fwd_kernel<T, VV, KK>), grid, block, 0, st, (const T*)y, inv, (const T*)w, n_tokens, k, hidden, (T*)out)
    if (vec) {
        if (k <= 2) PICOMOE_LAUNCH_CF(V, 2);
        else if (k <= 8) PICOMOE_LAUNCH_CF(V, 8);
        else PICOMOE_LAUNCH_CF(V, kMaxTopK);
    } else {
        PICOMOE_LAUNCH_CF(1, kMaxTopK);
    }
#undef PICOMOE_LAUNCH_CF
}
template <typename T>
void launch_combine_bwd(hipStream_t st, const void* d_out, const void* y, const int* inv, const void* w, int64_t n_tokens,
                        int k, int64_t hidden, void* d_y, void* d_w) {
    const dim3 grid((unsigned)((n_tokens + 3) / 4)), block(256);
    constexpr int V = sizeof(T) == 2 ? 8 : 4;
#define PICOMOE_LAUNCH_CB(VV, KK) \
    hipLaunchKernelGGL((combine_bwd_kernel<T, VV, KK>), grid, block, 0, st, (const T*)d_out, (const T*)y, inv, (const T*)w, n_tokens, k, hidden, (T*)d_y, (T*)d_w)
    if (can_vec<T>(hidden, d_out, y, d_y)) {
        if (k <= 2) PICOMOE_LAUNCH_CB(V, 2);
        else if (k <= 8) PICOMOE_LAUNCH_CB(V, 8);
        else PICOMOE_LAUNCH_CB(V, kMaxTopK);
    } else {
        PICOMOE_LAUNCH_CB(1, kMaxTopK);
    }
#undef PICOMOE_LAUNCH_CB
}
}  // namespace

extern "C" int picomoe_combine_fwd(const void* y, const int32_t* inv_order, const void* weights, int64_t n_tokens, int top_k,
                                   int64_t hidden, int dtype, void* out, void* stream) {
    PICOMOE_CHECK_ARG(n_tokens >= 0 && hidden > 0 && top_k >= 1 && top_k <= kMaxTopK);
    PICOMOE_CHECK_ARG(dtype == PICOMOE_F32 || dtype == PICOMOE_BF16);
    if (n_tokens == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(y && out);
    if (dtype == PICOMOE_BF16)
        launch_combine_fwd<uint16_t>((hipStream_t)stream, y, inv_order, weights, n_tokens, top_k, hidden, out);
    else
        launch_combine_fwd<float>((hipStream_t)stream, y, inv_order, weights, n_tokens, top_k, hidden, out);
    return picomoe_launch_status();
}

extern "C" int picomoe_combine_bwd(const void* d_out, const void* y, const int32_t* inv_order, const void* weights,
                                   int64_t n_tokens, int top_k, int64_t hidden, int dtype, void* d_y, void* d_weights,
                                   void* stream) {
    PICOMOE_CHECK_ARG(n_tokens >= 0 && hidden > 0 && top_k >= 1 && top_k <= kMaxTopK);
    PICOMOE_CHECK_ARG(dtype == PICOMOE_F32 || dtype == PICOMOE_BF16);
    if (n_tokens == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(d_out && y && weights && d_y && d_weights);
    if (dtype == PICOMOE_BF16)
        launch_combine_bwd<uint16_t>((hipStream_t)stream, d_out, y, inv_order, weights, n_tokens, top_k, hidden, d_y, d_weights);
    else
        launch_combine_bwd<float>((hipStream_t)stream, d_out, y, inv_order, weights, n_tokens, top_k, hidden, d_y, d_weights);
    return picomoe_launch_status();
}
