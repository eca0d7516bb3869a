/* CPU oracle, plain C: the reference's int8 weight-only quantiser restated
 * loop for loop.  TEST INFRASTRUCTURE ONLY -- never linked into the shipped
 * library.  Built by oracle/Makefile into oracle/liboracle.so.
 *
 * Follows 3rdparty/cutlass_kernels/cutlass_preprocessors.cc:581-678
 * (symmetric_quantize, QuantType::INT8_WEIGHT_ONLY branch):
 *   :610      quant_range_scale = 1.f / float(1 << 7)
 *   :619-628  per_col_max[j] = max(per_col_max[j], fabsf(w[i][j]))
 *   :632-635  per_col_max[j] *= quant_range_scale; scale[j] = ComputeType(per_col_max[j])
 *   :643-648  q = int8(max(-128.f, min(127.f, round(w / per_col_max[j]))))
 * std::min(a, b) is (b < a) ? b : a and std::max(a, b) is (a < b) ? b : a;
 * they are spelled out below because the NaN behaviour (0/0 for an all-zero
 * column) depends on that exact form.
 *
 * The weight matrix is passed as fp32; fp16 weights are widened exactly by the
 * caller, and the caller rounds the returned fp32 scale to fp16 (RN-even), as
 * the reference's ComputeType(float) conversion does.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

static float std_min(float a, float b) { return (b < a) ? b : a; }
static float std_max(float a, float b) { return (a < b) ? b : a; }

int oracle_quantize_ref128(const float *w, size_t K, size_t N, int8_t *q, float *scale32)
{
    const float quant_range_scale = 1.f / (float)(1 << 7);
    float *per_col_max = (float *)malloc(sizeof(float) * (N ? N : 1));
    if (!per_col_max)
        return -1;
    for (size_t j = 0; j < N; ++j)
        per_col_max[j] = 0.f;
    for (size_t i = 0; i < K; ++i)
        for (size_t j = 0; j < N; ++j)
            per_col_max[j] = std_max(per_col_max[j], fabsf(w[i * N + j]));
    for (size_t j = 0; j < N; ++j) {
        per_col_max[j] *= quant_range_scale;
        scale32[j] = per_col_max[j];
    }
    for (size_t i = 0; i < K; ++i) {
        for (size_t j = 0; j < N; ++j) {
            const float scaled = roundf(w[i * N + j] / per_col_max[j]);
            q[i * N + j] = (int8_t)std_max(-128.f, std_min(127.f, scaled));
        }
    }
    free(per_col_max);
    return 0;
}
