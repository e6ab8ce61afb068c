/*
 * fp32 CPU restatement of the EfficientNet MBConv operators -- TEST INFRASTRUCTURE ONLY
 * (see oracle.h).  Each function restates one tensor expression of the reference's
 * python/models/efficientnet/efficientnet.py (NHWC, batch 1) and the block composes them in
 * the order of TVMMBConvBlock.forward (python/models/efficientnet/tvm_efficientnet.py:62-118).
 *
 * The depthwise convolution of the reference is TVM's topi.nn.depthwise_conv2d_nhwc with
 * padding "SAME" (efficientnet.py:173-195; TVM is a dependency that is not vendored in the
 * reference).  Its published padding rule for "SAME" is pad_total = kernel - 1,
 * pad_before = (pad_total + 1) / 2 on both axes whatever the stride, and the output extent is
 * (in + pad_total - kernel) / stride + 1.  The reference hands the stride to the dilation
 * argument as well; the operator restated here is the undilated one that EfficientNet defines.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

static float swishf(float v) { return v / (1.0f + expf(-v)); }

/* Y[p][o] = act((sum_k X[p][k] * gate[k] * W[o][k]) * scale[o] + shift[o]) + shortcut[p][o]
 * (pointwise_conv2d_bn efficientnet.py:41-57, ..._short_cut_add :83-101,
 *  head_conv1x1_bn_swish :502-518; gate = the squeeze-excite factor of
 *  fused_pointwise_conv_bias_add_sigmoid_mul :252-267 applied to the operand). */
int oracle_pointwise_conv_f32(const float *x, const float *w, const float *scale, const float *shift,
                              const float *gate, const float *shortcut, float *y,
                              int pixels, int in_c, int out_c, int act, int num_threads) {
  if (!x || !w || !y || pixels <= 0 || in_c <= 0 || out_c <= 0) return -1;
  (void)num_threads;
#pragma omp parallel for num_threads(num_threads > 0 ? num_threads : 1) schedule(static)
  for (int p = 0; p < pixels; ++p) {
    float *xr = (float *)malloc(sizeof(float) * (size_t)in_c);
    for (int k = 0; k < in_c; ++k) xr[k] = x[(size_t)p * in_c + k] * (gate ? gate[k] : 1.0f);
    for (int o = 0; o < out_c; ++o) {
      float a = 0.f;
      const float *wr = w + (size_t)o * in_c;
      for (int k = 0; k < in_c; ++k) a += xr[k] * wr[k];
      a = a * (scale ? scale[o] : 1.0f) + (shift ? shift[o] : 0.0f);
      if (act == ORACLE_MB_SWISH) a = swishf(a);
      if (shortcut) a += shortcut[(size_t)p * out_c + o];
      y[(size_t)p * out_c + o] = a;
    }
    free(xr);
  }
  return 0;
}

int oracle_depthwise_out_extent(int in, int kernel, int stride) { return (in + (kernel - 1) - kernel) / stride + 1; }

/* Y[ho][wo][c] = swish((sum_ij X[ho*s - pad + i][wo*s - pad + j][c] * W[i][j][c]) * scale[c] + shift[c])
 * (fused_depthwise_conv2d_bn_swish efficientnet.py:173-195). */
int oracle_depthwise_conv_f32(const float *x, const float *w, const float *scale, const float *shift, float *y,
                              int in_h, int in_w, int channels, int kernel, int stride, int act, int num_threads) {
  if (!x || !w || !y || in_h <= 0 || in_w <= 0 || channels <= 0 || kernel <= 0 || stride <= 0) return -1;
  const int pad = (kernel - 1 + 1) / 2;
  const int oh = oracle_depthwise_out_extent(in_h, kernel, stride), ow = oracle_depthwise_out_extent(in_w, kernel, stride);
#pragma omp parallel for num_threads(num_threads > 0 ? num_threads : 1) schedule(static)
  for (int ho = 0; ho < oh; ++ho)
    for (int wo = 0; wo < ow; ++wo)
      for (int c = 0; c < channels; ++c) {
        float a = 0.f;
        for (int i = 0; i < kernel; ++i) {
          const int hi = ho * stride - pad + i;
          if (hi < 0 || hi >= in_h) continue;
          for (int j = 0; j < kernel; ++j) {
            const int wi = wo * stride - pad + j;
            if (wi < 0 || wi >= in_w) continue;
            a += x[((size_t)hi * in_w + wi) * channels + c] * w[((size_t)i * kernel + j) * channels + c];
          }
        }
        a = a * (scale ? scale[c] : 1.0f) + (shift ? shift[c] : 0.0f);
        if (act == ORACLE_MB_SWISH) a = swishf(a);
        y[((size_t)ho * ow + wo) * channels + c] = a;
      }
  return 0;
}

/* w_reduce [squeezed][channels] (output-major), w_expand [squeezed][channels] (input-major, the layout
 * se_module_pointwise_conv declares).
 * gate[c] = sigmoid(b_e[c] + sum_j W_e[j][c] * swish(b_r[j] + sum_c' W_r[j][c'] * mean_p X[p][c']))
 * (reduce_mean efficientnet.py:131-141; se_module_pointwise_conv :270-282 twice, swish between;
 *  fused_pointwise_conv_bias_add_sigmoid :413-424 for the second layer and its sigmoid). */
int oracle_se_gate_f32(const float *x, const float *w_reduce, const float *b_reduce, const float *w_expand,
                       const float *b_expand, float *gate, int pixels, int channels, int squeezed) {
  if (!x || !w_reduce || !w_expand || !gate || pixels <= 0 || channels <= 0 || squeezed <= 0) return -1;
  double *m = (double *)calloc((size_t)channels, sizeof(double));
  float *r = (float *)malloc(sizeof(float) * (size_t)squeezed);
  if (!m || !r) { free(m); free(r); return -3; }
  for (int p = 0; p < pixels; ++p)
    for (int c = 0; c < channels; ++c) m[c] += x[(size_t)p * channels + c];
  for (int j = 0; j < squeezed; ++j) {
    float a = b_reduce ? b_reduce[j] : 0.f;
    for (int c = 0; c < channels; ++c) a += w_reduce[(size_t)j * channels + c] * (float)(m[c] / pixels);
    r[j] = swishf(a);
  }
  for (int c = 0; c < channels; ++c) {
    float a = b_expand ? b_expand[c] : 0.f;
    for (int j = 0; j < squeezed; ++j) a += w_expand[(size_t)j * channels + c] * r[j];
    gate[c] = 1.0f / (1.0f + expf(-a));
  }
  free(m); free(r);
  return 0;
}

/* Nearest fp16 value (round to nearest even), for the "stored as fp16 between operators" variant. */
static float round_half(float v) {
  if (!(fabsf(v) < 65520.0f)) return v;                 /* inf/nan/overflow: leave to the caller's data */
  if (fabsf(v) < 6.103515625e-05f) {                    /* subnormal range of fp16: multiples of 2^-24 */
    return nearbyintf(v * 16777216.0f) / 16777216.0f;
  }
  int e;
  (void)frexpf(v, &e);                                  /* |v| = f * 2^e, f in [0.5, 1) */
  const float ulp = ldexpf(1.0f, e - 11);               /* 11 significant bits */
  return nearbyintf(v / ulp) * ulp;
}

static void round_all(float *p, size_t n) {
  for (size_t i = 0; i < n; ++i) p[i] = round_half(p[i]);
}

/* One MBConv block.  x [in_h*in_w][in_c] -> y [oh*ow][out_c]; dump_e / dump_d (nullable) receive
 * the expanded and the depthwise activations.  round_fp16 != 0 rounds every operator's output
 * tensor to fp16, which is how the fp16 pipeline stores them. */
int oracle_mbconv_block_f32(const oracle_mbconv_block *b, const float *x, float *y, float *dump_e, float *dump_d,
                            int round_fp16, int num_threads) {
  if (!b || !x || !y) return -1;
  const int hw = b->in_h * b->in_w;
  const int oh = oracle_depthwise_out_extent(b->in_h, b->kernel, b->stride);
  const int ow = oracle_depthwise_out_extent(b->in_w, b->kernel, b->stride);
  const int has_expand = b->expand_w != NULL;
  if (!has_expand && b->expand_c != b->in_c) return -1;
  if (b->has_shortcut && (b->stride != 1 || b->in_c != b->out_c)) return -1;
  float *e = NULL, *d = (float *)malloc(sizeof(float) * (size_t)oh * ow * b->expand_c);
  float *gate = (float *)malloc(sizeof(float) * (size_t)b->expand_c);
  int rc = (!d || !gate) ? -3 : 0;
  const float *dw_in = x;
  if (!rc && has_expand) {
    e = (float *)malloc(sizeof(float) * (size_t)hw * b->expand_c);
    if (!e) rc = -3;
    if (!rc) rc = oracle_pointwise_conv_f32(x, b->expand_w, b->expand_scale, b->expand_shift, NULL, NULL, e, hw, b->in_c,
                                            b->expand_c, ORACLE_MB_SWISH, num_threads);
    if (!rc && round_fp16) round_all(e, (size_t)hw * b->expand_c);
    if (!rc && dump_e) memcpy(dump_e, e, sizeof(float) * (size_t)hw * b->expand_c);
    dw_in = e;
  }
  if (!rc) rc = oracle_depthwise_conv_f32(dw_in, b->dw_w, b->dw_scale, b->dw_shift, d, b->in_h, b->in_w, b->expand_c,
                                          b->kernel, b->stride, ORACLE_MB_SWISH, num_threads);
  /* the squeeze-excite statistics are taken from the unrounded activations (the pipeline
   * accumulates them in fp32 while it produces the tensor) */
  if (!rc && b->se_c > 0)
    rc = oracle_se_gate_f32(d, b->se_reduce_w, b->se_reduce_b, b->se_expand_w, b->se_expand_b, gate, oh * ow, b->expand_c,
                            b->se_c);
  if (!rc && round_fp16) round_all(d, (size_t)oh * ow * b->expand_c);
  if (!rc && dump_d) memcpy(dump_d, d, sizeof(float) * (size_t)oh * ow * b->expand_c);
  if (!rc) rc = oracle_pointwise_conv_f32(d, b->project_w, b->project_scale, b->project_shift, b->se_c > 0 ? gate : NULL,
                                          b->has_shortcut ? x : NULL, y, oh * ow, b->expand_c, b->out_c, ORACLE_MB_NONE,
                                          num_threads);
  if (!rc && round_fp16) round_all(y, (size_t)oh * ow * b->out_c);
  free(e); free(d); free(gate);
  return rc;
}
