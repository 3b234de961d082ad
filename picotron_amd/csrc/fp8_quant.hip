// Per-token-scaled FP8 E4M3 quantise / dequantise for gfx950 (HBM-bandwidth bound).
//
// Quantise, bf16 rows: one wavefront owns one row and keeps it in registers (each lane holds
// 16-byte chunks lane, lane+64, ...), so HBM sees exactly one read of the row (2 B/elem) and one
// write of the codes (1 B/elem) plus 4 B/row of scale.  amax is an integer max over the 15-bit
// magnitudes (order-preserving for non-negative floats, and it carries NaN patterns to the top).
//
// The quotient float(x)/scale must be the IEEE-rounded one (the codes have to equal the ones a
// plain fp32 division yields).  A full IEEE division per element would make the kernel ALU bound,
// so each row computes r = RN(1/scale) once and every element uses the two-FMA correction
//     q0 = x*r;  e = fma(-q0, scale, x);  q = fma(e, r, q0)
// which is the correctly rounded quotient whenever r is the correctly rounded reciprocal and
// nothing under/overflows (Markstein); rows whose scale is not finite take the plain division.
#include "common.h"

namespace {

constexpr float kE4M3Max = 448.0f;
constexpr uint32_t kAmaxFloorBf16 = 0x38D2u;  // bf16(1e-4)

__device__ __forceinline__ float clamp448(float v) { return __builtin_amdgcn_fmed3f(v, -kE4M3Max, kE4M3Max); }

// two fp32 -> two E4M3 codes placed in the low (hi_word = false) or high half of `old`
template <bool HI>
__device__ __forceinline__ uint32_t cvt2(float a, float b, uint32_t old) {
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, HI);
}

struct RowScale {
    float s;       // dequant multiplier as fp32
    float r;       // RN(1/s)
    bool finite;   // s is finite and non-NaN
};

__device__ __forceinline__ float quotient(float x, const RowScale& rs) {
    float q0 = x * rs.r;
    float e = __builtin_fmaf(-q0, rs.s, x);
    return __builtin_copysignf(__builtin_fmaf(e, rs.r, q0), x);  // -0.0 / s must stay -0.0
}

// eight bf16 values (one 16-byte chunk) -> eight E4M3 codes
__device__ __forceinline__ u32x2_t quant_chunk(const u32x4_t& vc, const RowScale& rs) {
    const uint32_t w[4] = {vc.x, vc.y, vc.z, vc.w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(w[i] << 16);
        f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
    if (rs.finite) {
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = clamp448(quotient(f[i], rs));
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float t = f[i] / rs.s;
            f[i] = (t != t) ? t : clamp448(t);
        }
    }
    u32x2_t out;
    out.x = cvt2<false>(f[0], f[1], 0u);
    out.x = cvt2<true>(f[2], f[3], out.x);
    out.y = cvt2<false>(f[4], f[5], 0u);
    out.y = cvt2<true>(f[6], f[7], out.y);
    return out;
}

// One row held in the registers of one wavefront: lane l has the 16-byte chunks l, l + 64, ...
// FULL: the row is exactly CHUNKS * 64 chunks long, so no load or store needs a bounds test (and none sits behind a
// branch on the execution mask).
template <int CHUNKS, bool FULL>
__device__ __forceinline__ void load_row(const u32x4_t* xr, int lane, int chunks_per_row, u32x4_t (&v)[CHUNKS]) {
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int idx = c * 64 + lane;
        v[c] = (FULL || idx < chunks_per_row) ? __builtin_nontemporal_load(xr + idx) : u32x4_t{0u, 0u, 0u, 0u};
    }
}

// amax -> scale of the bf16 row a wavefront holds in v
template <int CHUNKS>
__device__ __forceinline__ RowScale row_scale_bf16(const u32x4_t (&v)[CHUNKS]) {
    typedef __attribute__((ext_vector_type(2))) unsigned short u16x2;
    u16x2 m2 = {0, 0};
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u16x2 a = __builtin_bit_cast(u16x2, w[i] & 0x7FFF7FFFu);
            m2 = __builtin_elementwise_max(m2, a);
        }
    }
    uint32_t amax_bits = m2.x > m2.y ? m2.x : m2.y;
    amax_bits = wave_max(amax_bits);
    const bool has_nan = amax_bits > 0x7F80u;
    if (!has_nan && amax_bits < kAmaxFloorBf16) amax_bits = kAmaxFloorBf16;

    RowScale rs;
    rs.s = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(amax_bits) / kE4M3Max));
    rs.r = 1.0f / rs.s;
    rs.finite = amax_bits < 0x7F80u;
    return rs;
}

// amax -> scale -> codes of the row in v; lane 0 writes the scale
template <int CHUNKS, bool FULL>
__device__ __forceinline__ void quant_row(const u32x4_t (&v)[CHUNKS], int lane, int chunks_per_row, u32x2_t* qr, float* scale_out) {
    const RowScale rs = row_scale_bf16<CHUNKS>(v);
    if (lane == 0) *scale_out = rs.s;

#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int idx = c * 64 + lane;
        if (FULL || idx < chunks_per_row) __builtin_nontemporal_store(quant_chunk(v[c], rs), qr + idx);
    }
}

template <int CHUNKS, bool FULL>
__global__ __launch_bounds__(256) void quant_bf16_wave_per_row(const u32x4_t* __restrict__ x, int64_t n_rows,
                                                               int chunks_per_row, u32x2_t* __restrict__ q,
                                                               float* __restrict__ scale) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;  // uniform per wave
    u32x4_t v[CHUNKS];
    load_row<CHUNKS, FULL>(x + row * chunks_per_row, lane, chunks_per_row, v);
    quant_row<CHUNKS, FULL>(v, lane, chunks_per_row, q + row * chunks_per_row, scale + row);
}

// Rows too long for one wavefront's registers (more than 8192 values): one block of 256 threads per row, thread t holding
// chunks t, t + 256, ...; the row maximum goes through LDS.  Same arithmetic, same single read of the row.
template <int CHUNKS>
__global__ __launch_bounds__(256) void quant_bf16_block_per_row(const u32x4_t* __restrict__ x, int chunks_per_row,
                                                                u32x2_t* __restrict__ q, float* __restrict__ scale) {
    __shared__ uint32_t part[4];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const u32x4_t* xr = x + row * chunks_per_row;
    u32x4_t v[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int idx = c * 256 + tid;
        v[c] = idx < chunks_per_row ? __builtin_nontemporal_load(xr + idx) : u32x4_t{0u, 0u, 0u, 0u};
    }
    typedef __attribute__((ext_vector_type(2))) unsigned short u16x2;
    u16x2 m2 = {0, 0};
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(u16x2, w[i] & 0x7FFF7FFFu));
    }
    uint32_t amax_bits = wave_max((uint32_t)(m2.x > m2.y ? m2.x : m2.y));
    if ((tid & 63) == 0) part[tid >> 6] = amax_bits;
    __syncthreads();
    amax_bits = part[0];
#pragma unroll
    for (int i = 1; i < 4; ++i) amax_bits = part[i] > amax_bits ? part[i] : amax_bits;
    const bool has_nan = amax_bits > 0x7F80u;
    if (!has_nan && amax_bits < kAmaxFloorBf16) amax_bits = kAmaxFloorBf16;
    RowScale rs;
    rs.s = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(amax_bits) / kE4M3Max));
    rs.r = 1.0f / rs.s;
    rs.finite = amax_bits < 0x7F80u;
    if (tid == 0) scale[row] = rs.s;
    u32x2_t* qr = q + row * chunks_per_row;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int idx = c * 256 + tid;
        if (idx < chunks_per_row) __builtin_nontemporal_store(quant_chunk(v[c], rs), qr + idx);
    }
}

template <typename T>
__device__ __forceinline__ float load_as_f32(const T* p);
template <>
__device__ __forceinline__ float load_as_f32<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }

// Any dtype / any hidden size: one 256-thread block per row, two passes over the row (the second
// is served by L2).  T = float (fp32 rows) or uint16_t (bf16 bit patterns).
template <typename T>
__global__ __launch_bounds__(256) void quant_generic(const T* __restrict__ x, int64_t hidden, uint8_t* __restrict__ q,
                                                     float* __restrict__ scale) {
    __shared__ uint32_t part[4];
    const int64_t row = blockIdx.x;
    const T* xr = x + row * hidden;
    uint32_t m = 0;  // fp32 magnitude bits (order preserving, NaN on top)
    for (int64_t c = threadIdx.x; c < hidden; c += 256) {
        uint32_t b = __float_as_uint(load_as_f32<T>(xr + c)) & 0x7FFFFFFFu;
        m = b > m ? b : m;
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
    __syncthreads();
    m = part[0];
    for (int i = 1; i < 4; ++i) m = part[i] > m ? part[i] : m;
    const bool has_nan = m > 0x7F800000u;
    float amax = __uint_as_float(m);
    float s;
    if (sizeof(T) == 2) {
        const float floor_v = bf16_bits_to_f32(kAmaxFloorBf16);
        if (!has_nan && amax < floor_v) amax = floor_v;
        s = bf16_bits_to_f32(f32_to_bf16_bits(amax / kE4M3Max));
    } else {
        if (!has_nan && amax < 1e-4f) amax = 1e-4f;
        s = amax / kE4M3Max;
    }
    if (threadIdx.x == 0) scale[row] = s;
    uint8_t* qr = q + row * hidden;
    for (int64_t c = threadIdx.x; c < hidden; c += 256) {
        float t = load_as_f32<T>(xr + c) / s;
        t = (t != t) ? t : clamp448(t);
        qr[c] = (uint8_t)(cvt2<false>(t, t, 0u) & 0xFFu);
    }
}

// ---- dequantise ------------------------------------------------------------------------------
// bf16 out: 8 codes (one u32x2_t) per lane -> 8 bf16 (one u32x4_t).  float(code) * float(bf16(scale))
// is exact in fp32 (4 x 8 significant bits), so one RNE to bf16 gives the reference's product.
__global__ __launch_bounds__(256) void dequant_bf16_vec(const u32x2_t* __restrict__ q, const float* __restrict__ scale,
                                                        int64_t n_rows, int chunks_per_row, u32x4_t* __restrict__ out) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int lane = threadIdx.x & 63;
    const float s = bf16_bits_to_f32(f32_to_bf16_bits(scale[row]));
    const u32x2_t* qr = q + row * chunks_per_row;
    u32x4_t* orow = out + row * chunks_per_row;
    for (int idx = lane; idx < chunks_per_row; idx += 64) {
        const u32x2_t c = __builtin_nontemporal_load(qr + idx);
        typedef __attribute__((ext_vector_type(2))) float f32x2;
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.x, false);
        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.x, true);
        const f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.y, false);
        const f32x2 e = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.y, true);
        u32x4_t o;
        o.x = pack_bf16x2(a.x * s, a.y * s);
        o.y = pack_bf16x2(b.x * s, b.y * s);
        o.z = pack_bf16x2(d.x * s, d.y * s);
        o.w = pack_bf16x2(e.x * s, e.y * s);
        __builtin_nontemporal_store(o, orow + idx);
    }
}

// The same with the row's chunks as a compile-time count: all of a lane's loads are issued before its first store.
template <int CHUNKS>
__global__ __launch_bounds__(256) void dequant_bf16_wave_per_row(const u32x2_t* __restrict__ q, const float* __restrict__ scale,
                                                                 int64_t n_rows, int chunks_per_row, u32x4_t* __restrict__ out) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int lane = threadIdx.x & 63;
    const u32x2_t* qr = q + row * chunks_per_row;
    u32x4_t* orow = out + row * chunks_per_row;
    u32x2_t c[CHUNKS];
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
        const int idx = lane + 64 * k;
        c[k] = idx < chunks_per_row ? __builtin_nontemporal_load(qr + idx) : u32x2_t{0u, 0u};
    }
    const float s = bf16_bits_to_f32(f32_to_bf16_bits(scale[row]));
    typedef __attribute__((ext_vector_type(2))) float f32x2;
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
        const int idx = lane + 64 * k;
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)c[k].x, false);
        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)c[k].x, true);
        const f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8((int)c[k].y, false);
        const f32x2 e = __builtin_amdgcn_cvt_pk_f32_fp8((int)c[k].y, true);
        u32x4_t o;
        o.x = pack_bf16x2(a.x * s, a.y * s);
        o.y = pack_bf16x2(b.x * s, b.y * s);
        o.z = pack_bf16x2(d.x * s, d.y * s);
        o.w = pack_bf16x2(e.x * s, e.y * s);
        if (idx < chunks_per_row) __builtin_nontemporal_store(o, orow + idx);
    }
}

template <bool BF16_OUT>
__global__ __launch_bounds__(256) void dequant_generic(const uint8_t* __restrict__ q, const float* __restrict__ scale,
                                                       int64_t hidden, void* __restrict__ out) {
    const int64_t row = blockIdx.x;
    const float s = BF16_OUT ? bf16_bits_to_f32(f32_to_bf16_bits(scale[row])) : scale[row];
    for (int64_t c = threadIdx.x; c < hidden; c += 256) {
        const float v = __builtin_amdgcn_cvt_f32_fp8((int)q[row * hidden + c], 0) * s;
        if (BF16_OUT)
            ((uint16_t*)out)[row * hidden + c] = (uint16_t)f32_to_bf16_bits(v);
        else
            ((float*)out)[row * hidden + c] = v;
    }
}

// eight E4M3 codes -> eight bf16: float(code) * s is exact in fp32, one rounding to bf16
__device__ __forceinline__ u32x4_t dequant_chunk_bf16(const u32x2_t& c, float s) {
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.x, false);
    const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.x, true);
    const f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.y, false);
    const f32x2 e = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.y, true);
    u32x4_t o;
    o.x = pack_bf16x2(a.x * s, a.y * s);
    o.y = pack_bf16x2(b.x * s, b.y * s);
    o.z = pack_bf16x2(d.x * s, d.y * s);
    o.w = pack_bf16x2(e.x * s, e.y * s);
    return o;
}

// ---- one-pass dispatch -----------------------------------------------------------------------
// One wavefront per token: the row is read once, quantised, dequantised, and the dequantised row (and, when asked for,
// the codes and the scale) written straight to the sorted positions of the token's top_k routed rows.  HBM sees
// hidden * 2 bytes read and top_k * hidden * (2 [+ 1]) bytes written per token: what a quantise pass, a dequantise pass
// and the expand + permute gather(s) move one after the other, without the two intermediate copies.
constexpr int kDispatchMaxTopK = 16;

template <int CHUNKS, bool FULL>
__global__ __launch_bounds__(256) void dispatch_bf16_wave_per_token(const u32x4_t* __restrict__ tokens, int64_t n_tokens,
                                                                    int chunks_per_row, const int32_t* __restrict__ inv_order,
                                                                    int top_k, int64_t n_out, u32x4_t* __restrict__ x_sorted,
                                                                    u32x2_t* __restrict__ q_sorted, float* __restrict__ scale_sorted,
                                                                    u32x2_t* __restrict__ q, float* __restrict__ scale) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tokens) return;  // uniform per wave
    u32x4_t v[CHUNKS];
    load_row<CHUNKS, FULL>(tokens + t * chunks_per_row, lane, chunks_per_row, v);
    // the sorted positions of this token's routed rows: wave-uniform, kept in scalar registers
    int pos[kDispatchMaxTopK];
#pragma unroll
    for (int j = 0; j < kDispatchMaxTopK; ++j) {
        int p = j < top_k ? inv_order[t * top_k + j] : -1;
        if (p >= n_out) p = -1;
        pos[j] = __builtin_amdgcn_readfirstlane(p);
    }
    const RowScale rs = row_scale_bf16<CHUNKS>(v);
    if (lane == 0) {
        if (scale) scale[t] = rs.s;
        if (scale_sorted) {
#pragma unroll
            for (int j = 0; j < kDispatchMaxTopK; ++j)
                if (pos[j] >= 0) scale_sorted[pos[j]] = rs.s;
        }
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int idx = c * 64 + lane;
        if (!FULL && idx >= chunks_per_row) continue;
        const u32x2_t codes = quant_chunk(v[c], rs);
        const u32x4_t deq = dequant_chunk_bf16(codes, rs.s);
        if (q) __builtin_nontemporal_store(codes, q + t * chunks_per_row + idx);
#pragma unroll
        for (int j = 0; j < kDispatchMaxTopK; ++j) {
            if (pos[j] < 0) continue;  // wave-uniform
            __builtin_nontemporal_store(deq, x_sorted + (int64_t)pos[j] * chunks_per_row + idx);
            if (q_sorted) __builtin_nontemporal_store(codes, q_sorted + (int64_t)pos[j] * chunks_per_row + idx);
        }
    }
}

// Any dtype / width: one block per token, the arithmetic of quant_generic and dequant_generic.
template <typename T>
__global__ __launch_bounds__(256) void dispatch_generic(const T* __restrict__ tokens, int64_t hidden,
                                                        const int32_t* __restrict__ inv_order, int top_k, int64_t n_out,
                                                        T* __restrict__ x_sorted, uint8_t* __restrict__ q_sorted,
                                                        float* __restrict__ scale_sorted, uint8_t* __restrict__ q,
                                                        float* __restrict__ scale) {
    __shared__ uint32_t part[4];
    const int64_t t = blockIdx.x;
    const T* xr = tokens + t * hidden;
    uint32_t m = 0;
    for (int64_t c = threadIdx.x; c < hidden; c += 256) {
        uint32_t b = __float_as_uint(load_as_f32<T>(xr + c)) & 0x7FFFFFFFu;
        m = b > m ? b : m;
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
    __syncthreads();
    m = part[0];
    for (int i = 1; i < 4; ++i) m = part[i] > m ? part[i] : m;
    const bool has_nan = m > 0x7F800000u;
    float amax = __uint_as_float(m);
    float s;
    if (sizeof(T) == 2) {
        const float floor_v = bf16_bits_to_f32(kAmaxFloorBf16);
        if (!has_nan && amax < floor_v) amax = floor_v;
        s = bf16_bits_to_f32(f32_to_bf16_bits(amax / kE4M3Max));
    } else {
        if (!has_nan && amax < 1e-4f) amax = 1e-4f;
        s = amax / kE4M3Max;
    }
    if (threadIdx.x == 0 && scale) scale[t] = s;
    for (int j = threadIdx.x; j < top_k; j += 256) {
        const int p = inv_order[t * top_k + j];
        if (p >= 0 && p < n_out && scale_sorted) scale_sorted[p] = s;
    }
    for (int64_t c = threadIdx.x; c < hidden; c += 256) {
        float v = load_as_f32<T>(xr + c) / s;
        v = (v != v) ? v : clamp448(v);
        const uint32_t code = cvt2<false>(v, v, 0u) & 0xFFu;
        const float d = __builtin_amdgcn_cvt_f32_fp8((int)code, 0) * s;
        if (q) q[t * hidden + c] = (uint8_t)code;
        for (int j = 0; j < top_k; ++j) {
            const int p = inv_order[t * top_k + j];
            if (p < 0 || p >= n_out) continue;
            if (sizeof(T) == 2)
                ((uint16_t*)x_sorted)[(int64_t)p * hidden + c] = (uint16_t)f32_to_bf16_bits(d);
            else
                ((float*)x_sorted)[(int64_t)p * hidden + c] = d;
            if (q_sorted) q_sorted[(int64_t)p * hidden + c] = (uint8_t)code;
        }
    }
}

}  // namespace

extern "C" int picomoe_dispatch_fp8(const void* tokens, int dtype, int64_t n_tokens, int64_t hidden, const int32_t* inv_order,
                                    int top_k, int64_t n_out, void* x_sorted, uint8_t* q_sorted, float* scale_sorted,
                                    uint8_t* q, float* scale, void* stream) {
    PICOMOE_CHECK_ARG(n_tokens >= 0 && n_tokens < (1ll << 31) && hidden > 0 && n_out >= 0 && n_out < (1ll << 31));
    PICOMOE_CHECK_ARG((dtype == PICOMOE_F32 || dtype == PICOMOE_BF16) && top_k >= 1 && top_k <= kDispatchMaxTopK);
    PICOMOE_CHECK_ARG((q_sorted == nullptr) == (scale_sorted == nullptr) && (q == nullptr) == (scale == nullptr));
    if (n_tokens == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(tokens && inv_order && (x_sorted || n_out == 0));
    hipStream_t st = (hipStream_t)stream;
    const bool aligned = dtype == PICOMOE_BF16 && hidden % 8 == 0 && hidden <= 8192 && (uintptr_t)tokens % 16 == 0 &&
                         (uintptr_t)x_sorted % 16 == 0 && (uintptr_t)q_sorted % 8 == 0 && (uintptr_t)q % 8 == 0;
    if (aligned) {
        const int cpr = (int)(hidden / 8);
        const int chunks = (cpr + 63) / 64;
        const dim3 grid((unsigned)((n_tokens + 3) / 4)), block(256);
#define PICOMOE_LAUNCH_D(C)                                                                                             \
    if (cpr == C * 64)                                                                                                  \
        hipLaunchKernelGGL((dispatch_bf16_wave_per_token<C, true>), grid, block, 0, st, (const u32x4_t*)tokens, n_tokens, \
                           cpr, inv_order, top_k, n_out, (u32x4_t*)x_sorted, (u32x2_t*)q_sorted, scale_sorted,          \
                           (u32x2_t*)q, scale);                                                                         \
    else                                                                                                                \
        hipLaunchKernelGGL((dispatch_bf16_wave_per_token<C, false>), grid, block, 0, st, (const u32x4_t*)tokens,        \
                           n_tokens, cpr, inv_order, top_k, n_out, (u32x4_t*)x_sorted, (u32x2_t*)q_sorted,              \
                           scale_sorted, (u32x2_t*)q, scale)
        if (chunks <= 1) PICOMOE_LAUNCH_D(1);
        else if (chunks <= 2) PICOMOE_LAUNCH_D(2);
        else if (chunks <= 4) PICOMOE_LAUNCH_D(4);
        else if (chunks <= 8) PICOMOE_LAUNCH_D(8);
        else PICOMOE_LAUNCH_D(16);
#undef PICOMOE_LAUNCH_D
    } else if (dtype == PICOMOE_BF16) {
        hipLaunchKernelGGL(dispatch_generic<uint16_t>, dim3((unsigned)n_tokens), dim3(256), 0, st, (const uint16_t*)tokens,
                           hidden, inv_order, top_k, n_out, (uint16_t*)x_sorted, q_sorted, scale_sorted, q, scale);
    } else {
        hipLaunchKernelGGL(dispatch_generic<float>, dim3((unsigned)n_tokens), dim3(256), 0, st, (const float*)tokens, hidden,
                           inv_order, top_k, n_out, (float*)x_sorted, q_sorted, scale_sorted, q, scale);
    }
    return picomoe_launch_status();
}

extern "C" int picomoe_fp8_quant(const void* x, int dtype, int64_t n_rows, int64_t hidden, uint8_t* q, float* scale,
                                 void* stream) {
    PICOMOE_CHECK_ARG(n_rows >= 0 && hidden > 0 && (dtype == PICOMOE_F32 || dtype == PICOMOE_BF16));
    PICOMOE_CHECK_ARG(n_rows < (1ll << 31));
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(x && q && scale);
    hipStream_t st = (hipStream_t)stream;
    const bool aligned = dtype == PICOMOE_BF16 && hidden % 8 == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)q % 8 == 0);
    const bool vec_ok = aligned && hidden <= 8192;
    if (aligned && hidden > 8192 && hidden <= 32768) {
        const int cpr = (int)(hidden / 8);
        const dim3 grid((unsigned)n_rows), block(256);
        if (cpr <= 8 * 256)
            hipLaunchKernelGGL(quant_bf16_block_per_row<8>, grid, block, 0, st, (const u32x4_t*)x, cpr, (u32x2_t*)q, scale);
        else
            hipLaunchKernelGGL(quant_bf16_block_per_row<16>, grid, block, 0, st, (const u32x4_t*)x, cpr, (u32x2_t*)q, scale);
    } else if (vec_ok) {
        const int cpr = (int)(hidden / 8);
        const int chunks = (cpr + 63) / 64;
        const dim3 grid((unsigned)((n_rows + 3) / 4)), block(256);
        // Rows of 4096 values and more (8 KB in flight per wavefront): 32 KB of LDS per block, which the kernel never
        // touches, holds a CU at five blocks (20 wavefronts) instead of eight.  Measured at 16384 x 4096 with the launches
        // alternating in one run: 72.2-73.8 % of the HBM peak against 71.1-72.5 % with every wave slot filled.
        const unsigned lds = chunks >= 8 ? 32000u : 0u;
#define PICOMOE_LAUNCH_Q(C)                                                                                            \
    if (cpr == C * 64)                                                                                                 \
        hipLaunchKernelGGL((quant_bf16_wave_per_row<C, true>), grid, block, lds, st, (const u32x4_t*)x, n_rows, cpr,   \
                           (u32x2_t*)q, scale);                                                                        \
    else                                                                                                               \
        hipLaunchKernelGGL((quant_bf16_wave_per_row<C, false>), grid, block, lds, st, (const u32x4_t*)x, n_rows, cpr,  \
                           (u32x2_t*)q, scale)
        if (chunks <= 1) PICOMOE_LAUNCH_Q(1);
        else if (chunks <= 2) PICOMOE_LAUNCH_Q(2);
        else if (chunks <= 4) PICOMOE_LAUNCH_Q(4);
        else if (chunks <= 8) PICOMOE_LAUNCH_Q(8);
        else PICOMOE_LAUNCH_Q(16);
#undef PICOMOE_LAUNCH_Q
    } else if (dtype == PICOMOE_BF16) {
        hipLaunchKernelGGL(quant_generic<uint16_t>, dim3((unsigned)n_rows), dim3(256), 0, st, (const uint16_t*)x, hidden,
                           q, scale);
    } else {
        hipLaunchKernelGGL(quant_generic<float>, dim3((unsigned)n_rows), dim3(256), 0, st, (const float*)x, hidden, q,
                           scale);
    }
    return picomoe_launch_status();
}

extern "C" int picomoe_fp8_dequant(const uint8_t* q, const float* scale, int64_t n_rows, int64_t hidden, void* out,
                                   int dtype, void* stream) {
    PICOMOE_CHECK_ARG(n_rows >= 0 && hidden > 0 && (dtype == PICOMOE_F32 || dtype == PICOMOE_BF16));
    PICOMOE_CHECK_ARG(n_rows < (1ll << 31));
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(q && scale && out);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == PICOMOE_BF16 && hidden % 8 == 0 && ((uintptr_t)q % 8 == 0) && ((uintptr_t)out % 16 == 0)) {
        const int cpr = (int)(hidden / 8);
        const dim3 grid((unsigned)((n_rows + 3) / 4)), block(256);
        // rows of up to 8192 values: the kernel that issues all of a lane's loads before its first store (33.9 us against
        // 37.0 us for the loop form at 16384 x 4096); longer rows take the loop
#define PICOMOE_LAUNCH_DQ(C)                                                                                           \
    hipLaunchKernelGGL(dequant_bf16_wave_per_row<C>, grid, block, 0, st, (const u32x2_t*)q, scale, n_rows, cpr, (u32x4_t*)out)
        if (cpr <= 64) PICOMOE_LAUNCH_DQ(1);
        else if (cpr <= 128) PICOMOE_LAUNCH_DQ(2);
        else if (cpr <= 256) PICOMOE_LAUNCH_DQ(4);
        else if (cpr <= 512) PICOMOE_LAUNCH_DQ(8);
        else if (cpr <= 1024) PICOMOE_LAUNCH_DQ(16);
        else
            hipLaunchKernelGGL(dequant_bf16_vec, grid, block, 0, st, (const u32x2_t*)q, scale, n_rows, cpr, (u32x4_t*)out);
#undef PICOMOE_LAUNCH_DQ
    } else if (dtype == PICOMOE_BF16) {
        hipLaunchKernelGGL(dequant_generic<true>, dim3((unsigned)n_rows), dim3(256), 0, st, q, scale, hidden, out);
    } else {
        hipLaunchKernelGGL(dequant_generic<false>, dim3((unsigned)n_rows), dim3(256), 0, st, q, scale, hidden, out);
    }
    return picomoe_launch_status();
}

extern "C" int picomoe_abi_version(void) { return PICOMOE_ABI_VERSION; }

extern "C" const char* picomoe_error_string(int code) {
    if (code == PICOMOE_OK) return "ok";
    if (code == PICOMOE_ERR_ARG) return "picomoe: unsupported shape, dtype, alignment or null pointer";
    if (code == PICOMOE_ERR_TOO_LARGE)
        return "picomoe: too large -- the input exceeds the fixed scratch of a no-allocation entry point (use the variant that "
               "takes a workspace), or an expert-FFN shape has more tiles than the kernels' 32-bit tile numbering holds";
    if (code >= PICOMOE_ERR_HIP_BASE) return hipGetErrorString((hipError_t)(code - PICOMOE_ERR_HIP_BASE));
    return "picomoe: unknown error code";
}
