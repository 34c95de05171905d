/* The saturating part of the quantisers as C's own fmaxf / fminf / rintf / division evaluate it, for
 * tests/test_oracle_attention.py: the clamp is written exactly as in
 * xllm/core/kernels/cuda/fp8_quant_utils.cuh:121-122, fmaxf(-max, fminf(x, max)). */
#include <math.h>

float ref_absmax(const float* x, int n) {
  float m = 0.0f;
  for (int i = 0; i < n; ++i) m = fmaxf(m, fabsf(x[i]));
  return m;
}

/* y = clamp(val / scale) for fp8 (max 448), clamp(rint(val / scale)) for int8 (max 127) */
void ref_scaled_clamp(const float* val, int n, float scale, float max, int round_first, float* out) {
  for (int i = 0; i < n; ++i) {
    float x = val[i] / scale;
    if (round_first) x = rintf(x);
    out[i] = fmaxf(-max, fminf(x, max));
  }
}
