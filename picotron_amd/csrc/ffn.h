// Internal interface between the expert-FFN entry points (ffn_api.hip) and the kernel families:
// the generic tiled kernels (ffn_simple.hip: any shape, fp32 or bf16 storage, fp32 FMA arithmetic),
// the bf16 MFMA kernels (ffn_mfma.hip: aligned shapes) and the fp32 MFMA kernels (ffn_f32_mfma.hip).
#pragma once
#include "common.h"

struct FfnShape {
    const int64_t* counts;  // [E] rows per expert, experts back to back in the row dimension
    int E;
    int64_t n_rows;  // rows allocated (>= sum of counts); only used to bound the grid
    int64_t H, I;
    int dtype;
};

// act[m, n] = swiglu(x[m] . gate_w[e][n], x[m] . up_w[e][n]);  inter13 (optional) = [g | u]
int ffn_simple_gate_up(const FfnShape& s, const void* x, const void* gate_w, const void* up_w, void* act, void* inter13,
                       hipStream_t st);
// y[m, h] = act[m] . down_w[e][h]  (* row_weight[m])
int ffn_simple_down(const FfnShape& s, const void* act, const void* down_w, const void* row_weight, void* y,
                    hipStream_t st);
// da = dy . down_w[e]; d_inter13 = silu_and_mul backward at inter13; act_out (optional) = swiglu(inter13)
int ffn_simple_dgrad_act(const FfnShape& s, const void* dy, const void* down_w, const void* inter13, void* d_inter13,
                         void* act_out, hipStream_t st);
// dx = dg . gate_w[e] + du . up_w[e]
int ffn_simple_dgrad_x(const FfnShape& s, const void* d_inter13, const void* gate_w, const void* up_w, void* dx,
                       hipStream_t st);
// out[e][p, q] = sum_{m in e} lhs[m, p] * rhs[m, q]
int ffn_simple_wgrad(const FfnShape& s, const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, int64_t P,
                     int64_t Q, void* out, hipStream_t st);

// bf16 MFMA family: each returns PICOMOE_ERR_ARG without launching when the shape is not one it handles.
bool ffn_mfma_supported(const FfnShape& s);
bool ffn_mfma_wgrad_supported(int dtype, int64_t P, int64_t Q, int64_t ld_lhs, int64_t ld_rhs, const void* lhs, const void* rhs);
int ffn_mfma_gate_up(const FfnShape& s, const void* x, const void* gate_w, const void* up_w, void* act, void* inter13,
                     void* ws, int64_t ws_bytes, hipStream_t st);
int ffn_mfma_down(const FfnShape& s, const void* act, const void* down_w, const void* row_weight, void* y, void* ws,
                  int64_t ws_bytes, hipStream_t st);
int ffn_mfma_dgrad_act(const FfnShape& s, const void* dy, const void* down_w, const void* inter13, void* d_inter13,
                       void* act_out, void* ws, int64_t ws_bytes, hipStream_t st);
int ffn_mfma_dgrad_x(const FfnShape& s, const void* d_inter13, const void* gate_w, const void* up_w, void* dx, void* ws,
                     int64_t ws_bytes, hipStream_t st);
int64_t ffn_mfma_workspace_bytes();
int ffn_mfma_wgrad(const FfnShape& s, const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, int64_t P, int64_t Q,
                   void* out, hipStream_t st);

// fp32 MFMA family (ffn_f32_mfma.hip: v_mfma_f32_32x32x2_f32, hidden and inter multiples of 4); a call whose tensors are
// not 16-byte aligned falls through to the generic kernel of the same name.
bool ffn_f32_mfma_supported(const FfnShape& s);
bool ffn_f32_mfma_wgrad_supported(int dtype, int64_t P, int64_t Q, int64_t ld_lhs, int64_t ld_rhs, const void* lhs, const void* rhs);
int ffn_f32_mfma_gate_up(const FfnShape& s, const void* x, const void* gate_w, const void* up_w, void* act, void* inter13,
                         hipStream_t st);
int ffn_f32_mfma_down(const FfnShape& s, const void* act, const void* down_w, const void* row_weight, void* y, hipStream_t st);
int ffn_f32_mfma_dgrad_act(const FfnShape& s, const void* dy, const void* down_w, const void* inter13, void* d_inter13,
                           void* act_out, hipStream_t st);
int ffn_f32_mfma_dgrad_x(const FfnShape& s, const void* d_inter13, const void* gate_w, const void* up_w, void* dx, hipStream_t st);
int ffn_f32_mfma_wgrad(const FfnShape& s, const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, int64_t P, int64_t Q,
                       void* out, hipStream_t st);

// FP8 (E4M3) MFMA gate/up and down: codes + one fp32 scale per activation row and per weight row (ffn_fp8.hip)
bool ffn_fp8_supported(const FfnShape& s);
int ffn_fp8_gate_up(const FfnShape& s, const void* xq, const float* x_scale, const void* gq, const void* uq,
                    const float* g_scale, const float* u_scale, void* act, void* inter13, hipStream_t st);

// FP8 MFMA down: act codes + one fp32 scale per row, down_w codes + one scale per output row; y bf16 (* row_weight)
int ffn_fp8_down(const FfnShape& s, const void* actq, const float* act_scale, const void* dq, const float* d_scale,
                 const void* row_weight, void* y, hipStream_t st);

// SwiGLU pieces shared by both families (fp32 arithmetic on values already rounded to the storage type).
__device__ __forceinline__ float sigmoid_f32(float g) { return 1.0f / (1.0f + expf(-g)); }
__device__ __forceinline__ float sigmoid_fast(float g) { return __builtin_amdgcn_rcpf(1.0f + __expf(-g)); }
