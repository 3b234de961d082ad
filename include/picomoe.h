/* picomoe -- C ABI of the MI355X (gfx950) kernels for picotron's single-GPU (EP=1) MoE hot path.
 *
 * Conventions (every entry point):
 *   - plain device pointers, explicit sizes, row-major contiguous tensors unless a stride is given;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); work is only enqueued,
 *     nothing synchronises, allocates or keeps a pointer past the call;
 *   - returns 0 on success, PICOMOE_ERR_ARG for a shape / dtype / alignment the kernels do not
 *     accept, or PICOMOE_ERR_HIP_BASE + hipError_t when the launch itself failed;
 *   - `dtype` is PICOMOE_F32 or PICOMOE_BF16 (the dtype of the token features / weights).
 *
 * Each declaration cites the reference code it replaces (paths inside the picotron checkout,
 * `EP/` = picotron/expert_parallel/).
 */
#ifndef PICOMOE_H
#define PICOMOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PICOMOE_OK 0
#define PICOMOE_ERR_ARG 1
#define PICOMOE_ERR_HIP_BASE 1000

#define PICOMOE_F32 0
#define PICOMOE_BF16 1

#define PICOMOE_ABI_VERSION 1

/* ABI version of the loaded library (compare with PICOMOE_ABI_VERSION). */
int picomoe_abi_version(void);

/* Static, human-readable text for a return code of any entry point. */
const char* picomoe_error_string(int code);

/* ---- FP8 E4M3 dispatch quantise / dequantise ---------------------------------------------------
 * Replaces EP/ep_communications.py:63-68 (_per_token_quant_fp8): per row, amax = max|x| floored at
 * 1e-4 and scale = amax/448, both rounded to x's dtype; q = e4m3fn_rne(clamp(float(x)/scale, +-448)).
 * x [n_rows, hidden] (dtype), q [n_rows, hidden] bytes, scale [n_rows] fp32. */
int picomoe_fp8_quant(const void* x, int dtype, int64_t n_rows, int64_t hidden, uint8_t* q, float* scale,
                      void* stream);

/* Replaces EP/ep_communications.py:100: out = dtype(q) * dtype(scale), rounded to dtype. */
int picomoe_fp8_dequant(const uint8_t* q, const float* scale, int64_t n_rows, int64_t hidden, void* out, int dtype,
                        void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PICOMOE_H */
