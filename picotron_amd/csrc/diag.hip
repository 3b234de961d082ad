// Diagnostic launch, not part of the MoE path: a loop of nothing but MFMAs on caller-provided operand data, to measure
// what the matrix pipes of this GPU sustain under its power limit.  Every grouped-GEMM kernel of this library ends up
// clocked down by that limit, so the figure this loop reaches on random data -- not the datasheet peak, which needs the
// full clock -- is the ceiling the GEMM kernels can be compared with on the same box.
//
// One block of 8 wavefronts (two per SIMD) per requested block; every wavefront keeps 8 x 4 independent 16 x 16
// accumulators (or 4 x 2 of 32 x 32) in registers and multiplies the same fragments into them `iters` times, 64 MFMAs
// of 16 x 16 x 32 (or 32 of 32 x 32 x 16: the same FLOP) per iteration.  The operand fragments are read once from
// `operands`, so their bit patterns (random values toggle far more wires than zeros) are the caller's choice.
// With burst_iters > 0 the loop pauses for idle_us after every burst_iters iterations (all wavefronts of a block together):
// the rate inside the bursts then shows how much of a pause the power management gives back as a higher clock -- what a
// phase without MFMAs (an epilogue, a pipeline fill) really costs a GEMM kernel.
#include "common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) int i32x8_t;

constexpr int kDiagThreads = 512;

template <int SHAPE>
__global__ __launch_bounds__(kDiagThreads, 1) void diag_mfma_loop_kernel(const u32x4_t* __restrict__ src, int64_t n_chunks,
                                                                         int64_t n_bursts, int64_t iters, int64_t idle_ticks,
                                                                         float* sink) {
    const int64_t t = (int64_t)blockIdx.x * kDiagThreads + threadIdx.x;
    // between two bursts every wavefront of the block sleeps until idle_ticks of the 100 MHz wall clock have passed
    auto idle = [&]() {
        if (idle_ticks <= 0) return;
        __syncthreads();
        const uint64_t t0 = wall_clock64();
        while ((int64_t)(wall_clock64() - t0) < idle_ticks) __builtin_amdgcn_s_sleep(32);
        __syncthreads();
    };
    auto chunk = [&](int i) { return src[(t * 32 + i) % n_chunks]; };
    float x = 0.f;
    if (SHAPE == PICOMOE_DIAG_BF16_16X16X32 || SHAPE == PICOMOE_DIAG_BF16_32X32X16) {
        bf16x8_t a[2][8], b[2][4];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#pragma unroll
            for (int i = 0; i < 8; ++i) a[s][i] = __builtin_bit_cast(bf16x8_t, chunk(s * 12 + i));
#pragma unroll
            for (int j = 0; j < 4; ++j) b[s][j] = __builtin_bit_cast(bf16x8_t, chunk(s * 12 + 8 + j));
        }
        if (SHAPE == PICOMOE_DIAG_BF16_16X16X32) {
            f32x4_t acc[8][4];
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            for (int64_t bu = 0; bu < n_bursts; ++bu) {
                for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
                    for (int s = 0; s < 2; ++s)
#pragma unroll
                        for (int i = 0; i < 8; ++i)
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
                }
                idle();
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) x += acc[i][j][r];
        } else {
            f32x16_t acc[4][2];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
            for (int64_t bu = 0; bu < n_bursts; ++bu) {
                for (int64_t it = 0; it < iters; ++it) {
                    // four sub-steps of 16 k values, 8 MFMAs of 32 x 32 x 16 each: the FLOP of the 64 narrow MFMAs above
#pragma unroll
                    for (int s = 0; s < 4; ++s)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
#pragma unroll
                            for (int j = 0; j < 2; ++j)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s & 1][2 * (s >> 1) + i], b[s & 1][2 * (s >> 1) + j],
                                                                                    acc[i][j], 0, 0, 0);
                }
                idle();
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) x += acc[i][j][r];
        }
    } else {  // FP8 E4M3 16 x 16 x 128: a fragment is 32 codes per lane
        i32x8_t a[8], b[4];
        auto frag = [&](int i) {
            const u32x4_t lo = chunk(2 * i), hi = chunk(2 * i + 1);
            return i32x8_t{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        };
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = frag(i);
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = frag(8 + j);
        f32x4_t acc[8][4];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        for (int64_t bu = 0; bu < n_bursts; ++bu) {
            for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, 0, 0, 0);
            }
            idle();
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) x += acc[i][j][r];
    }
    // keeps the accumulators alive; the store itself does not happen for any data a caller would pass
    if (x == 12345.678f && sink) sink[0] = x;
}

// FLOP of one wavefront's iteration
int64_t flop_per_wave_iter(int shape) {
    switch (shape) {
        case PICOMOE_DIAG_BF16_16X16X32: return 64ll * 2 * 16 * 16 * 32;
        case PICOMOE_DIAG_BF16_32X32X16: return 32ll * 2 * 32 * 32 * 16;
        case PICOMOE_DIAG_FP8_16X16X128: return 32ll * 2 * 16 * 16 * 128;
        default: return -1;
    }
}

}  // namespace

extern "C" int64_t picomoe_diag_mfma_loop_flop(int shape, int64_t iters, int n_blocks) {
    const int64_t per = flop_per_wave_iter(shape);
    if (per < 0 || iters < 0 || n_blocks < 0) return -1;
    return per * (kDiagThreads / kWave) * iters * n_blocks;
}

extern "C" int picomoe_diag_mfma_loop(const void* operands, int64_t operand_bytes, int shape, int64_t iters, int64_t burst_iters,
                                      int64_t idle_us, int n_blocks, float* sink, void* stream) {
    PICOMOE_CHECK_ARG(operands && (uintptr_t)operands % 16 == 0 && operand_bytes >= 16 && flop_per_wave_iter(shape) > 0);
    PICOMOE_CHECK_ARG(iters >= 0 && iters <= (1ll << 24) && n_blocks >= 1 && n_blocks <= 65536);
    PICOMOE_CHECK_ARG(burst_iters >= 0 && idle_us >= 0 && idle_us <= 1000 && (burst_iters == 0 || iters % burst_iters == 0));
    const int64_t n_chunks = operand_bytes / 16;
    // bursts of burst_iters iterations with idle_us between them (the wall clock of the device counts 100 MHz ticks)
    const int64_t per_burst = burst_iters > 0 ? burst_iters : iters, n_bursts = burst_iters > 0 ? iters / burst_iters : 1;
    const int64_t idle_ticks = burst_iters > 0 ? idle_us * 100 : 0;
    hipStream_t st = (hipStream_t)stream;
    const u32x4_t* src = (const u32x4_t*)operands;
    if (shape == PICOMOE_DIAG_BF16_16X16X32)
        hipLaunchKernelGGL((diag_mfma_loop_kernel<PICOMOE_DIAG_BF16_16X16X32>), dim3(n_blocks), dim3(kDiagThreads), 0, st, src, n_chunks, n_bursts, per_burst, idle_ticks, sink);
    else if (shape == PICOMOE_DIAG_BF16_32X32X16)
        hipLaunchKernelGGL((diag_mfma_loop_kernel<PICOMOE_DIAG_BF16_32X32X16>), dim3(n_blocks), dim3(kDiagThreads), 0, st, src, n_chunks, n_bursts, per_burst, idle_ticks, sink);
    else
        hipLaunchKernelGGL((diag_mfma_loop_kernel<PICOMOE_DIAG_FP8_16X16X128>), dim3(n_blocks), dim3(kDiagThreads), 0, st, src, n_chunks, n_bursts, per_burst, idle_ticks, sink);
    return picomoe_launch_status();
}
