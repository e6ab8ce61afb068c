/*
 * fp32 CPU restatement of the EfficientNet squeeze-excite module -- TEST
 * INFRASTRUCTURE ONLY (see oracle.h).  Op order as the reference's own unit test
 * composes it from library ops: avg_pool -> 1x1 conv -> swish -> 1x1 conv ->
 * sigmoid -> combine (cpp/efficientnet/efficientnet_se_module_unittest_binding.cu:123-130;
 * the reference combines with add, the textbook module with mul).
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>

int oracle_se_module_f32(const float *x, const float *w_reduce, const float *b_reduce,
                         const float *w_expand, const float *b_expand, float *y, float *pooled,
                         int C, int HW, int R, int combine) {
  if (!x || !w_reduce || !w_expand || !y || C <= 0 || HW <= 0 || R <= 0) return -1;
  float *p = (float *)malloc(sizeof(float) * (size_t)C);
  float *r = (float *)malloc(sizeof(float) * (size_t)R);
  if (!p || !r) { free(p); free(r); return -3; }
  for (int c = 0; c < C; ++c) {
    double s = 0.0;
    for (int i = 0; i < HW; ++i) s += x[(size_t)c * HW + i];
    p[c] = (float)(s / HW);
    if (pooled) pooled[c] = p[c];
  }
  for (int j = 0; j < R; ++j) {
    float a = b_reduce ? b_reduce[j] : 0.f;
    for (int c = 0; c < C; ++c) a += w_reduce[(size_t)j * C + c] * p[c];
    r[j] = a / (1.0f + expf(-a));          /* swish */
  }
  for (int c = 0; c < C; ++c) {
    float a = b_expand ? b_expand[c] : 0.f;
    for (int j = 0; j < R; ++j) a += w_expand[(size_t)c * R + j] * r[j];
    const float e = 1.0f / (1.0f + expf(-a));
    for (int i = 0; i < HW; ++i) {
      const float v = x[(size_t)c * HW + i];
      y[(size_t)c * HW + i] = combine == ORACLE_SE_ADD ? v + e : v * e;
    }
  }
  free(p); free(r);
  return 0;
}
