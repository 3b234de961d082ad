/* CPU oracle, C part.  TEST INFRASTRUCTURE ONLY: loaded by tests/ (via ctypes) to cross-check the
 * numpy/torch restatement in moe_oracle.py and the HIP kernels; never linked into the product.
 *
 * Byte/integer pieces of the reference's MoE hot path, restated in scalar C:
 *   - per-row scaled FP8 E4M3 quantise / dequantise of bf16 rows
 *       (reference: picotron/expert_parallel/ep_communications.py:59-68 and :100)
 *   - stable counting sort of routed rows by expert, and the rank of a row inside its expert
 *       (reference: picotron/expert_parallel/expert_parallel.py:335-339,
 *                   picotron/expert_parallel/capacity_moe.py:44-57)
 *
 * Pinned by: the closed-form E4M3 value table, torch's own float8_e4m3fn cast, and torch.argsort /
 * bincount (tests/test_oracle_fp8.py, tests/test_oracle_permute.py).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bits_to_f32(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }
static float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* round-to-nearest-even fp32 -> bf16, NaN kept quiet */
static uint16_t f32_to_bf16(float f) {
    uint32_t b = f32_to_bits(f);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x40);
    b += 0x7FFFu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

/* value of an E4M3FN code */
float oracle_e4m3_decode(uint8_t code) {
    int e = (code >> 3) & 0xF, m = code & 7;
    float s = (code & 0x80) ? -1.0f : 1.0f;
    if (e == 15 && m == 7) return NAN;
    if (e == 0) return s * ldexpf((float)m / 8.0f, -6);
    return s * ldexpf(1.0f + (float)m / 8.0f, e - 7);
}

/* RNE fp32 -> E4M3FN by searching the value table: nearest code, ties to the even code.
 * Deliberately a different method from the bit-twiddling encoder in moe_oracle.py. */
uint8_t oracle_e4m3_encode(float x) {
    uint8_t sign = (f32_to_bits(x) >> 24) & 0x80;
    float a = fabsf(x);
    if (!(a == a)) return (uint8_t)(sign | 0x7F);
    if (a >= 480.0f) return (uint8_t)(sign | 0x7F); /* past the midpoint above 448 torch yields NaN */
    int best = 0;
    double best_err = 1e300;
    for (int c = 0; c < 0x7F; ++c) {
        double err = fabs((double)oracle_e4m3_decode((uint8_t)c) - (double)a);
        if (err < best_err || (err == best_err && (c & 1) == 0)) { best = c; best_err = err; }
    }
    /* between 448 (0x7E, even) and the phantom 480 the midpoint 464 ties to 448; above it the cast overflows */
    if (a > 464.0f) return (uint8_t)(sign | 0x7F);
    return (uint8_t)(sign | best);
}

/* rows of bf16 -> codes + fp32 scale.  amax and scale are rounded to bf16 like the reference's
 * bf16 tensors; the quotient is an IEEE fp32 division, clamped to +-448, then cast. */
void oracle_quant_rows_bf16(const uint16_t* x, int64_t n_rows, int64_t hidden, uint8_t* q, float* scale) {
    const uint16_t floor_bits = f32_to_bf16(1e-4f);
    for (int64_t r = 0; r < n_rows; ++r) {
        const uint16_t* row = x + r * hidden;
        uint16_t amax_bits = 0;
        int has_nan = 0;
        for (int64_t c = 0; c < hidden; ++c) {
            uint16_t a = row[c] & 0x7FFF;
            if (a > 0x7F80) has_nan = 1;
            if (a > amax_bits) amax_bits = a;
        }
        if (!has_nan && amax_bits < floor_bits) amax_bits = floor_bits;
        float s = bf16_to_f32(f32_to_bf16(bf16_to_f32(amax_bits) / 448.0f));
        scale[r] = s;
        for (int64_t c = 0; c < hidden; ++c) {
            float v = bf16_to_f32(row[c]) / s;
            if (v > 448.0f) v = 448.0f;
            if (v < -448.0f) v = -448.0f;
            q[r * hidden + c] = oracle_e4m3_encode(v);
        }
    }
}

void oracle_dequant_rows_bf16(const uint8_t* q, const float* scale, int64_t n_rows, int64_t hidden, uint16_t* out) {
    for (int64_t r = 0; r < n_rows; ++r) {
        float s = bf16_to_f32(f32_to_bf16(scale[r]));
        for (int64_t c = 0; c < hidden; ++c)
            out[r * hidden + c] = f32_to_bf16(oracle_e4m3_decode(q[r * hidden + c]) * s);
    }
}

/* stable counting sort of rows by expert id */
void oracle_permute_plan(const int64_t* expert_idx, int64_t n, int64_t num_experts,
                         int64_t* order, int64_t* inv_order, int64_t* counts, int64_t* within) {
    for (int64_t e = 0; e < num_experts; ++e) counts[e] = 0;
    for (int64_t r = 0; r < n; ++r) {
        within[r] = counts[expert_idx[r]];
        counts[expert_idx[r]] += 1;
    }
    int64_t start = 0;
    for (int64_t e = 0; e < num_experts; ++e) {
        int64_t c = counts[e];
        counts[e] = start; /* temporarily the segment start */
        start += c;
    }
    for (int64_t r = 0; r < n; ++r) {
        int64_t pos = counts[expert_idx[r]] + within[r];
        order[pos] = r;
        inv_order[r] = pos;
    }
    for (int64_t e = 0; e < num_experts; ++e) {
        int64_t next = (e + 1 < num_experts) ? counts[e + 1] : n;
        counts[e] = next - counts[e];
    }
}
