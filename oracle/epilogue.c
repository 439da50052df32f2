/* Float operations of the oracle whose rounding must be fixed exactly.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by oracle/numerics.py, never by the shipped
 * package.  Restates Int8Inference (cumm/gemm/output_op/linear.py:279-360 of
 * the reference) and the float->s8 converter
 * (include/tensorview/gemm/math/numeric_convert.h:171-192, 262-285).
 */
#include <fenv.h>
#include <math.h>
#include <stdint.h>

static float act_apply(float x, int act, float act_alpha) {
  switch (act) {
  case 1: return x > 0.0f ? x : 0.0f;                 /* ReLU: maximum(x, 0) */
  case 2: return 1.0f / (1.0f + expf(-x));            /* Sigmoid */
  case 3: return x >= 0.0f ? x : x * act_alpha;       /* LeakyReLU */
  default: return x;
  }
}

void oracle_int8_epilogue(int8_t *out, const int32_t *acc, const float *scale,
                          const float *bias, const int8_t *src, int64_t rows,
                          int64_t cols, float beta, int act, float act_alpha) {
  fesetround(FE_TONEAREST);
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t c = 0; c < cols; ++c) {
      float t = fmaf(scale[c], (float)acc[r * cols + c], bias[c]);
      if (src) t = fmaf(beta, (float)src[r * cols + c], t);
      t = act_apply(t, act, act_alpha);
      if (t < -128.0f) t = -128.0f;
      if (t > 127.0f) t = 127.0f;
      float q = nearbyintf(t); /* ties to even under FE_TONEAREST */
      if (q != q) q = 0.0f;    /* NaN converts to 0 (cvt.rni.sat) */
      out[r * cols + c] = (int8_t)(int32_t)q;
    }
  }
}

/* LinearCombination (cumm/gemm/output_op/linear.py:108-146 of the reference):
 * x = beta*src (rounded), then alpha*acc + x as one fused multiply-add (the
 * contraction nvcc applies to multiply_add, include/tensorview/gemm/math/functional.h:225-231);
 * with no source: alpha*acc. */
void oracle_linear_combination(float *out, const float *acc, const float *src, int64_t n,
                               float alpha, float beta) {
  for (int64_t i = 0; i < n; ++i) {
    if (src) {
      float x = beta * src[i];
      out[i] = fmaf(alpha, acc[i], x);
    } else {
      out[i] = alpha * acc[i];
    }
  }
}
