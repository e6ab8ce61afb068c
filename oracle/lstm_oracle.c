/*
 * fp32 CPU restatement of the stacked LSTM -- TEST INFRASTRUCTURE ONLY (see oracle.h).
 * Cell math: cpp/lstm/lstm_reuse_shared_memory.cu:306-318 (gates, c and h update) and
 * python/models/lstm/tf_lstm.py:59-102 (layer stacking: layer l at step t consumes
 * h of layer l-1 at the same step t).  Weight layout [layer*4+gate][out][in]:
 * cpp/lstm/lstm_reuse_shared_memory.cu:201-222.  The reference kernel's one-step
 * input lag for layer 0 (:324-326) is an artefact and is not reproduced.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

static float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

int oracle_lstm_f32(const oracle_lstm_cfg *c, const float *w_ih, const float *w_hh,
                    const float *bias, const float *x, float *y) {
  if (!c || !w_ih || !w_hh || !x || !y) return -1;
  const int L = c->layers, Hd = c->hidden, T = c->timesteps, B = c->batch;
  if (L <= 0 || Hd <= 0 || T <= 0 || B <= 0) return -2;
  /* slot of each logical gate inside the 4 stored matrices */
  int si, sf, sg, so;
  if (c->gate_order == ORACLE_GATES_IFGO) { si = 0; sf = 1; sg = 2; so = 3; }
  else if (c->gate_order == ORACLE_GATES_IGFO) { si = 0; sg = 1; sf = 2; so = 3; }
  else return -2;
  float *h = (float *)calloc((size_t)L * Hd, sizeof(float));
  float *cs = (float *)calloc((size_t)L * Hd, sizeof(float));
  float *pre = (float *)malloc(sizeof(float) * 4 * (size_t)Hd);
  float *in = (float *)malloc(sizeof(float) * (size_t)Hd);
  if (!h || !cs || !pre || !in) { free(h); free(cs); free(pre); free(in); return -3; }
  for (int b = 0; b < B; ++b) {
    memset(h, 0, sizeof(float) * (size_t)L * Hd);
    memset(cs, 0, sizeof(float) * (size_t)L * Hd);
    for (int t = 0; t < T; ++t) {
      memcpy(in, x + ((size_t)b * T + t) * Hd, sizeof(float) * (size_t)Hd);
      for (int l = 0; l < L; ++l) {
        float *hl = h + (size_t)l * Hd, *cl = cs + (size_t)l * Hd;
        for (int g = 0; g < 4; ++g) {
          const float *wi = w_ih + ((size_t)l * 4 + g) * Hd * Hd;
          const float *wh = w_hh + ((size_t)l * 4 + g) * Hd * Hd;
          for (int r = 0; r < Hd; ++r) {
            float a = bias ? bias[((size_t)l * 4 + g) * Hd + r] : 0.f;
            float s1 = 0.f, s2 = 0.f;
            for (int k = 0; k < Hd; ++k) { s1 += wi[(size_t)r * Hd + k] * in[k]; s2 += wh[(size_t)r * Hd + k] * hl[k]; }
            pre[(size_t)g * Hd + r] = a + s1 + s2;
          }
        }
        for (int r = 0; r < Hd; ++r) {
          const float ig = sigmoidf_(pre[(size_t)si * Hd + r]);
          const float fg = sigmoidf_(pre[(size_t)sf * Hd + r] + c->forget_bias);
          const float gg = tanhf(pre[(size_t)sg * Hd + r]);
          const float og = sigmoidf_(pre[(size_t)so * Hd + r]);
          cl[r] = cl[r] * fg + ig * gg;
          hl[r] = tanhf(cl[r]) * og;
        }
        memcpy(in, hl, sizeof(float) * (size_t)Hd);
      }
      memcpy(y + ((size_t)b * T + t) * Hd, h + (size_t)(L - 1) * Hd, sizeof(float) * (size_t)Hd);
    }
  }
  free(h); free(cs); free(pre); free(in);
  return 0;
}
