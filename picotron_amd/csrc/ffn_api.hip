// extern "C" entry points of the expert FFN (grouped SwiGLU GEMMs, forward + dgrad + wgrad).
// Picks the bf16 or fp32 MFMA kernels when the shape is one they tile, the generic kernels otherwise.
#include "ffn.h"

namespace {
bool fill_shape(FfnShape* s, const int64_t* counts, int E, int64_t n_rows, int64_t H, int64_t I, int dtype) {
    if (!counts || E < 1 || E > 1024 || n_rows < 0 || n_rows >= (1ll << 31) || H < 1 || I < 1) return false;
    if (dtype != PICOMOE_F32 && dtype != PICOMOE_BF16) return false;
    s->counts = counts; s->E = E; s->n_rows = n_rows; s->H = H; s->I = I; s->dtype = dtype;
    return true;
}

// The kernels number their tiles and their launch grids in 32 bits.  An upper bound of the tiles any of the M-grouped launches
// can have (row tiles of 64 rows, the smallest any kernel family uses, plus one tail per expert, times the column tiles of the
// wider output) has to stay below 2^31; so does the grid of the weight gradient.
bool grouped_tiles_fit(const FfnShape& s) {
    const int64_t row_tiles = s.n_rows / 64 + s.E, col_tiles = ((s.H > 2 * s.I ? s.H : 2 * s.I) + 63) / 64;
    return row_tiles <= (int64_t)0x7FFFFFFF / (col_tiles > 0 ? col_tiles : 1) - 4096;
}
bool wgrad_tiles_fit(int E, int64_t P, int64_t Q) {
    const int64_t p_tiles = (P + 63) / 64, q_tiles = (Q + 63) / 64;
    return p_tiles <= (int64_t)0x7FFFFFFF / q_tiles / E - 1;
}
}  // namespace

extern "C" int picomoe_ffn_gate_up(const void* x, const int64_t* counts, int num_experts, int64_t n_rows, int64_t hidden,
                                   int64_t inter, const void* gate_w, const void* up_w, int dtype, void* act, void* inter13,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
    FfnShape s;
    PICOMOE_CHECK_ARG(fill_shape(&s, counts, num_experts, n_rows, hidden, inter, dtype));
    if (!grouped_tiles_fit(s)) return PICOMOE_ERR_TOO_LARGE;
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(x && gate_w && up_w && act);
    if (ffn_mfma_supported(s)) return ffn_mfma_gate_up(s, x, gate_w, up_w, act, inter13, workspace, workspace_bytes, (hipStream_t)stream);
    if (ffn_f32_mfma_supported(s)) return ffn_f32_mfma_gate_up(s, x, gate_w, up_w, act, inter13, (hipStream_t)stream);
    return ffn_simple_gate_up(s, x, gate_w, up_w, act, inter13, (hipStream_t)stream);
}

extern "C" int picomoe_ffn_gate_up_fp8(const void* xq, const float* x_scale, const int64_t* counts, int num_experts,
                                       int64_t n_rows, int64_t hidden, int64_t inter, const void* gate_wq, const void* up_wq,
                                       const float* gate_scale, const float* up_scale, void* act, void* inter13,
                                       void* stream) {
    FfnShape s;
    PICOMOE_CHECK_ARG(fill_shape(&s, counts, num_experts, n_rows, hidden, inter, PICOMOE_BF16));
    if (!grouped_tiles_fit(s)) return PICOMOE_ERR_TOO_LARGE;
    PICOMOE_CHECK_ARG(ffn_fp8_supported(s));
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(xq && x_scale && gate_wq && up_wq && gate_scale && up_scale && act);
    return ffn_fp8_gate_up(s, xq, x_scale, gate_wq, up_wq, gate_scale, up_scale, act, inter13, (hipStream_t)stream);
}

extern "C" int picomoe_ffn_down_fp8(const void* actq, const float* act_scale, const int64_t* counts, int num_experts,
                                    int64_t n_rows, int64_t hidden, int64_t inter, const void* down_wq,
                                    const float* down_scale, const void* row_weight, void* y, void* stream) {
    FfnShape s;
    PICOMOE_CHECK_ARG(fill_shape(&s, counts, num_experts, n_rows, hidden, inter, PICOMOE_BF16));
    if (!grouped_tiles_fit(s)) return PICOMOE_ERR_TOO_LARGE;
    PICOMOE_CHECK_ARG(ffn_fp8_supported(s));
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(actq && act_scale && down_wq && down_scale && y);
    return ffn_fp8_down(s, actq, act_scale, down_wq, down_scale, row_weight, y, (hipStream_t)stream);
}

extern "C" int64_t picomoe_ffn_workspace_bytes(void) { return ffn_mfma_workspace_bytes(); }

extern "C" int picomoe_ffn_kernel_family(int dtype, int64_t hidden, int64_t inter) {
    FfnShape s{};
    s.dtype = dtype; s.H = hidden; s.I = inter;
    if (ffn_mfma_supported(s)) return PICOMOE_FFN_BF16_MFMA;
    if (ffn_f32_mfma_supported(s)) return PICOMOE_FFN_F32_MFMA;
    return PICOMOE_FFN_GENERIC;
}

extern "C" int picomoe_ffn_down(const void* act, const int64_t* counts, int num_experts, int64_t n_rows, int64_t hidden,
                                int64_t inter, const void* down_w, const void* row_weight, int dtype, void* y, void* workspace,
                                int64_t workspace_bytes, void* stream) {
    FfnShape s;
    PICOMOE_CHECK_ARG(fill_shape(&s, counts, num_experts, n_rows, hidden, inter, dtype));
    if (!grouped_tiles_fit(s)) return PICOMOE_ERR_TOO_LARGE;
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(act && down_w && y);
    if (ffn_mfma_supported(s)) return ffn_mfma_down(s, act, down_w, row_weight, y, workspace, workspace_bytes, (hipStream_t)stream);
    if (ffn_f32_mfma_supported(s)) return ffn_f32_mfma_down(s, act, down_w, row_weight, y, (hipStream_t)stream);
    return ffn_simple_down(s, act, down_w, row_weight, y, (hipStream_t)stream);
}

extern "C" int picomoe_ffn_dgrad_act(const void* dy, const int64_t* counts, int num_experts, int64_t n_rows, int64_t hidden,
                                     int64_t inter, const void* down_w, const void* inter13, int dtype, void* d_inter13,
                                     void* act_out, void* workspace, int64_t workspace_bytes, void* stream) {
    FfnShape s;
    PICOMOE_CHECK_ARG(fill_shape(&s, counts, num_experts, n_rows, hidden, inter, dtype));
    if (!grouped_tiles_fit(s)) return PICOMOE_ERR_TOO_LARGE;
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(dy && down_w && inter13 && d_inter13);
    if (ffn_mfma_supported(s)) return ffn_mfma_dgrad_act(s, dy, down_w, inter13, d_inter13, act_out, workspace, workspace_bytes, (hipStream_t)stream);
    if (ffn_f32_mfma_supported(s)) return ffn_f32_mfma_dgrad_act(s, dy, down_w, inter13, d_inter13, act_out, (hipStream_t)stream);
    return ffn_simple_dgrad_act(s, dy, down_w, inter13, d_inter13, act_out, (hipStream_t)stream);
}

extern "C" int picomoe_ffn_dgrad_x(const void* d_inter13, const int64_t* counts, int num_experts, int64_t n_rows,
                                   int64_t hidden, int64_t inter, const void* gate_w, const void* up_w, int dtype, void* dx,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
    FfnShape s;
    PICOMOE_CHECK_ARG(fill_shape(&s, counts, num_experts, n_rows, hidden, inter, dtype));
    if (!grouped_tiles_fit(s)) return PICOMOE_ERR_TOO_LARGE;
    if (n_rows == 0) return PICOMOE_OK;
    PICOMOE_CHECK_ARG(d_inter13 && gate_w && up_w && dx);
    if (ffn_mfma_supported(s)) return ffn_mfma_dgrad_x(s, d_inter13, gate_w, up_w, dx, workspace, workspace_bytes, (hipStream_t)stream);
    if (ffn_f32_mfma_supported(s)) return ffn_f32_mfma_dgrad_x(s, d_inter13, gate_w, up_w, dx, (hipStream_t)stream);
    return ffn_simple_dgrad_x(s, d_inter13, gate_w, up_w, dx, (hipStream_t)stream);
}

extern "C" int picomoe_ffn_wgrad(const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, const int64_t* counts,
                                 int num_experts, int64_t n_rows, int64_t p_dim, int64_t q_dim, int dtype, void* out,
                                 void* stream) {
    FfnShape s;
    PICOMOE_CHECK_ARG(fill_shape(&s, counts, num_experts, n_rows, p_dim, q_dim, dtype));
    if (!wgrad_tiles_fit(num_experts, p_dim, q_dim)) return PICOMOE_ERR_TOO_LARGE;
    PICOMOE_CHECK_ARG(lhs && rhs && out && ld_lhs >= p_dim && ld_rhs >= q_dim);
    // n_rows == 0 still has to zero-fill the output: every expert is empty
    if (ffn_mfma_wgrad_supported(dtype, p_dim, q_dim, ld_lhs, ld_rhs, lhs, rhs))
        return ffn_mfma_wgrad(s, lhs, ld_lhs, rhs, ld_rhs, p_dim, q_dim, out, (hipStream_t)stream);
    if (ffn_f32_mfma_wgrad_supported(dtype, p_dim, q_dim, ld_lhs, ld_rhs, lhs, rhs))
        return ffn_f32_mfma_wgrad(s, lhs, ld_lhs, rhs, ld_rhs, p_dim, q_dim, out, (hipStream_t)stream);
    return ffn_simple_wgrad(s, lhs, ld_lhs, rhs, ld_rhs, p_dim, q_dim, out, (hipStream_t)stream);
}
