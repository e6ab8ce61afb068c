/*
 * fp32 CPU restatement of one BERT encoder layer -- TEST INFRASTRUCTURE ONLY
 * (see oracle.h).  Follows the op order of the reference's fused kernels:
 *   QKV GEMM + bias + head split   cpp/bert/kernels/fused_sqq_bert.cu:2333-2765
 *   scores, scale, (mask), softmax cpp/bert/kernels/fused_sqq_bert.cu:2772-3022,
 *                                  cpp/bert/kernels/softmax.cu:3-44 (max-subtracted form)
 *   context = P.V, heads merged    cpp/bert/kernels/gemm.cu:646-951 (store at :933)
 *   out-proj + residual + LN       cpp/bert/kernels/fused_sqq_bert.cu:3334-3782
 *   FC1 + activation               cpp/bert/kernels/fused_sqq_feedforward.cu:38-362,
 *                                  GELU-tanh: cpp/bert/bert_base_impl.cu:722-734
 *   FC2 + residual + LN            cpp/bert/kernels/fused_sqq_feedforward.cu:368-835
 * and the torch statement of the same layer in
 * cpp/bert/test_souffle_bert_layer.py:78-110.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int clamp_threads(int n) {
#ifdef _OPENMP
  int mx = omp_get_max_threads();
  if (n <= 0 || n > mx) n = mx;
  return n;
#else
  (void)n; return 1;
#endif
}

/* Y[M][N] = X[M][K] . W[K][N] (+ bias[N]) -- cpp/bert/kernels/gemm_three_stages.h:95-131 */
void oracle_gemm_f32(const float *x, const float *w, const float *bias, float *y,
                     int M, int N, int K, int num_threads) {
  int nt = clamp_threads(num_threads);
  (void)nt;
#pragma omp parallel for num_threads(nt) schedule(static)
  for (int m = 0; m < M; ++m) {
    float *yr = y + (size_t)m * N;
    if (bias) memcpy(yr, bias, sizeof(float) * (size_t)N);
    else memset(yr, 0, sizeof(float) * (size_t)N);
    const float *xr = x + (size_t)m * K;
    for (int k = 0; k < K; ++k) {
      const float a = xr[k];
      const float *wr = w + (size_t)k * N;
      for (int n = 0; n < N; ++n) yr[n] += a * wr[n];
    }
  }
}

/* biased variance, eps inside the square root -- cpp/bert/bert_base_impl.cu:762-771 */
void oracle_layernorm_f32(const float *z, const float *g, const float *b, float *y,
                          int rows, int dim, float eps) {
  for (int r = 0; r < rows; ++r) {
    const float *zr = z + (size_t)r * dim;
    float *yr = y + (size_t)r * dim;
    double s = 0.0;
    for (int i = 0; i < dim; ++i) s += zr[i];
    const float mean = (float)(s / dim);
    double v = 0.0;
    for (int i = 0; i < dim; ++i) { double d = zr[i] - mean; v += d * d; }
    const float rstd = 1.0f / sqrtf((float)(v / dim) + eps);
    for (int i = 0; i < dim; ++i) {
      float t = (zr[i] - mean) * rstd;
      yr[i] = t * (g ? g[i] : 1.0f) + (b ? b[i] : 0.0f);
    }
  }
}

/* 0.5 x (1 + tanh(0.79788456 (x + 0.044715 x^3))) -- cpp/bert/bert_base_impl.cu:722-734 */
float oracle_gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}

/* 0.5 x (1 + erf(x / sqrt 2)): the activation of the HuggingFace BERT checkpoints that
   cpp/bert/test_souffle_bert_layer.py:131-143,161 loads ("gelu" = torch.nn.functional.gelu's default form) */
float oracle_gelu_erf(float x) {
  return (float)(0.5 * (double)x * (1.0 + erf((double)x * 0.70710678118654752440)));
}

static void apply_act(float *h, size_t n, int act) {
  if (act == ORACLE_ACT_GELU_TANH) { for (size_t i = 0; i < n; ++i) h[i] = oracle_gelu_tanh(h[i]); }
  else if (act == ORACLE_ACT_GELU_ERF) { for (size_t i = 0; i < n; ++i) h[i] = oracle_gelu_erf(h[i]); }
  else if (act == ORACLE_ACT_RELU) { for (size_t i = 0; i < n; ++i) h[i] = h[i] > 0.f ? h[i] : 0.f; }
}

int oracle_bert_layer_f32(const oracle_bert_cfg *c, const oracle_bert_weights *w,
                          const float *x, const float *mask, float *y,
                          const oracle_bert_dump *dump, int num_threads) {
  if (!c || !w || !x || !y) return -1;
  const int B = c->batch, S = c->seq_len, H = c->hidden, nh = c->heads, F = c->ffn;
  if (B <= 0 || S <= 0 || H <= 0 || nh <= 0 || F <= 0 || H % nh) return -2;
  const int hd = H / nh, M = B * S;
  const int nt = clamp_threads(num_threads);
  float *qkv = (float *)malloc(sizeof(float) * 3 * (size_t)M * H);   /* [3][M][H] token-major */
  float *ctx = (float *)malloc(sizeof(float) * (size_t)M * H);
  float *z = (float *)malloc(sizeof(float) * (size_t)M * H);
  float *y1 = (float *)malloc(sizeof(float) * (size_t)M * H);
  float *h = (float *)malloc(sizeof(float) * (size_t)M * F);
  if (!qkv || !ctx || !z || !y1 || !h) { free(qkv); free(ctx); free(z); free(y1); free(h); return -3; }

  /* 1. Q,K,V = X.W_j + b_j */
  for (int j = 0; j < 3; ++j)
    oracle_gemm_f32(x, w->w_qkv + (size_t)j * H * H, w->b_qkv ? w->b_qkv + (size_t)j * H : NULL,
                    qkv + (size_t)j * M * H, M, H, H, nt);
  if (dump && dump->qkv) { /* head-major [3][B][nh][S][hd] -- fused_sqq_bert.cu:2738-2764 */
    for (int j = 0; j < 3; ++j) for (int b = 0; b < B; ++b) for (int hh = 0; hh < nh; ++hh)
      for (int s = 0; s < S; ++s)
        memcpy(dump->qkv + ((((size_t)j * B + b) * nh + hh) * S + s) * hd,
               qkv + (size_t)j * M * H + ((size_t)b * S + s) * H + (size_t)hh * hd, sizeof(float) * hd);
  }
  const float *Q = qkv, *K = qkv + (size_t)M * H, *V = qkv + 2 * (size_t)M * H;

  /* 2-3. P = softmax(scale * Q.K^T + mask); ctx = P.V with heads merged */
#pragma omp parallel for num_threads(nt) collapse(2) schedule(static)
  for (int b = 0; b < B; ++b) for (int hh = 0; hh < nh; ++hh) {
    float *row = (float *)malloc(sizeof(float) * (size_t)S);
    for (int q = 0; q < S; ++q) {
      const float *qr = Q + ((size_t)b * S + q) * H + (size_t)hh * hd;
      float mx = -INFINITY;
      for (int k = 0; k < S; ++k) {
        const float *kr = K + ((size_t)b * S + k) * H + (size_t)hh * hd;
        float a = 0.f;
        for (int d = 0; d < hd; ++d) a += qr[d] * kr[d];
        a *= c->scale;
        if (mask) a += mask[((size_t)b * S + q) * S + k];
        row[k] = a;
        if (a > mx) mx = a;
      }
      float sum = 0.f;
      for (int k = 0; k < S; ++k) { row[k] = expf(row[k] - mx); sum += row[k]; }
      const float inv = 1.0f / sum;
      for (int k = 0; k < S; ++k) row[k] *= inv;
      if (dump && dump->probs)
        memcpy(dump->probs + ((((size_t)b * nh + hh) * S) + q) * S, row, sizeof(float) * (size_t)S);
      float *cr = ctx + ((size_t)b * S + q) * H + (size_t)hh * hd;
      for (int d = 0; d < hd; ++d) cr[d] = 0.f;
      for (int k = 0; k < S; ++k) {
        const float p = row[k];
        const float *vr = V + ((size_t)b * S + k) * H + (size_t)hh * hd;
        for (int d = 0; d < hd; ++d) cr[d] += p * vr[d];
      }
    }
    free(row);
  }
  if (dump && dump->ctx) memcpy(dump->ctx, ctx, sizeof(float) * (size_t)M * H);

  /* 4. Y1 = LN(ctx.Wo + bo + X) */
  oracle_gemm_f32(ctx, w->w_o, w->b_o, z, M, H, H, nt);
  for (size_t i = 0; i < (size_t)M * H; ++i) z[i] += x[i];
  oracle_layernorm_f32(z, w->ln1_g, w->ln1_b, y1, M, H, c->ln_eps);
  if (dump && dump->ln1) memcpy(dump->ln1, y1, sizeof(float) * (size_t)M * H);

  /* 5. Hh = act(Y1.W1 + b1) */
  oracle_gemm_f32(y1, w->w_fc1, w->b_fc1, h, M, F, H, nt);
  apply_act(h, (size_t)M * F, c->act);
  if (dump && dump->fc1) memcpy(dump->fc1, h, sizeof(float) * (size_t)M * F);

  /* 6. Y = LN(Hh.W2 + b2 + Y1) */
  oracle_gemm_f32(h, w->w_fc2, w->b_fc2, z, M, H, F, nt);
  for (size_t i = 0; i < (size_t)M * H; ++i) z[i] += y1[i];
  oracle_layernorm_f32(z, w->ln2_g, w->ln2_b, y, M, H, c->ln_eps);

  free(qkv); free(ctx); free(z); free(y1); free(h);
  return 0;
}

/* cpp/bert/bert_base_impl.cu:590-678 loops one layer 12 times over a single
 * weight blob; here every layer has its own weights. */
int oracle_bert_encoder_f32(const oracle_bert_cfg *c, const oracle_bert_weights *layers,
                            int num_layers, const float *x, const float *mask, float *y,
                            int num_threads) {
  if (!c || !layers || num_layers <= 0) return -1;
  const size_t n = (size_t)c->batch * c->seq_len * c->hidden;
  float *a = (float *)malloc(sizeof(float) * n), *b = (float *)malloc(sizeof(float) * n);
  if (!a || !b) { free(a); free(b); return -3; }
  memcpy(a, x, sizeof(float) * n);
  int rc = 0;
  for (int l = 0; l < num_layers && rc == 0; ++l) {
    rc = oracle_bert_layer_f32(c, &layers[l], a, mask, b, NULL, num_threads);
    float *t = a; a = b; b = t;
  }
  if (rc == 0) memcpy(y, a, sizeof(float) * n);
  free(a); free(b);
  return rc;
}

/* Embedding stage in front of the encoder: word + position + token-type rows, then LayerNorm.
 * The reference takes this from the HuggingFace module (cpp/bert/test_souffle_bert_layer.py:186-189);
 * positions are 0..S-1 per sequence, token types default to 0. */
int oracle_bert_embed_f32(const int32_t *token_ids, const int32_t *segment_ids, const float *word_emb,
                          const float *pos_emb, const float *type_emb, const float *ln_g, const float *ln_b,
                          float eps, int batch, int seq_len, int hidden, float *out) {
  if (!token_ids || !word_emb || !pos_emb || !out || batch <= 0 || seq_len <= 0 || hidden <= 0) return -1;
  float *row = (float *)malloc(sizeof(float) * (size_t)hidden);
  if (!row) return -2;
  for (int m = 0; m < batch * seq_len; ++m) {
    const float *w = word_emb + (size_t)token_ids[m] * hidden, *p = pos_emb + (size_t)(m % seq_len) * hidden;
    const float *t = type_emb ? type_emb + (size_t)(segment_ids ? segment_ids[m] : 0) * hidden : NULL;
    for (int i = 0; i < hidden; ++i) row[i] = w[i] + p[i] + (t ? t[i] : 0.0f);
    oracle_layernorm_f32(row, ln_g, ln_b, out + (size_t)m * hidden, 1, hidden, eps);
  }
  free(row);
  return 0;
}

/* BERT pooler: tanh(x[b, 0, :] . W + bias), W stored [K][N]. */
int oracle_bert_pooler_f32(const float *x, const float *w, const float *bias, int batch, int seq_len, int hidden, float *out) {
  if (!x || !w || !out || batch <= 0 || seq_len <= 0 || hidden <= 0) return -1;
  for (int b = 0; b < batch; ++b) {
    oracle_gemm_f32(x + (size_t)b * seq_len * hidden, w, bias, out + (size_t)b * hidden, 1, hidden, hidden, 1);
    for (int n = 0; n < hidden; ++n) out[(size_t)b * hidden + n] = tanhf(out[(size_t)b * hidden + n]);
  }
  return 0;
}
