// bf16 MFMA expert-FFN kernels (placeholder while the generic kernels carry every shape).
#include "ffn.h"

bool ffn_mfma_supported(const FfnShape&) { return false; }
int ffn_mfma_gate_up(const FfnShape&, const void*, const void*, const void*, void*, void*, hipStream_t) { return PICOMOE_ERR_ARG; }
int ffn_mfma_down(const FfnShape&, const void*, const void*, const void*, void*, hipStream_t) { return PICOMOE_ERR_ARG; }
int ffn_mfma_dgrad_act(const FfnShape&, const void*, const void*, const void*, void*, void*, hipStream_t) { return PICOMOE_ERR_ARG; }
int ffn_mfma_dgrad_x(const FfnShape&, const void*, const void*, const void*, void*, hipStream_t) { return PICOMOE_ERR_ARG; }
int ffn_mfma_wgrad(const FfnShape&, const void*, int64_t, const void*, int64_t, int64_t, int64_t, void*, hipStream_t) { return PICOMOE_ERR_ARG; }
