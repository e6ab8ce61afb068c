/*
 * fp32 CPU restatement of a Swin block pair and its index maps -- TEST
 * INFRASTRUCTURE ONLY (see oracle.h).
 * Block structure: python/models/swin_transformer/swin_transformer_main.py:11-61
 * (Part-1..Part-8).  Index maps follow the torch closed forms that the
 * reference's own CPU test asserts equality with
 * (python/models/swin_transformer/test_swin_tensor_transformer_ops.py:27-29 roll,
 * :32-65 window partition, :118-121 roll+partition, :386-390 reverse+roll+add),
 * not the te expressions in swin_self_attention.py, which are only right for
 * square inputs.  qkv column order (q|k|v, head, hd): swin_self_attention.py:739-763.
 * GELU-tanh: python/models/swin_transformer/swin_mlp.py:90-95.  The relative-position
 * bias and the shifted-window mask do not exist in the reference; they follow the
 * published Swin definition.  FFN without bias/activation:
 * cpp/swin_transformer/swin_transformer_binding.cu:154-209.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

static int region_of(int i, int n, int ws, int shift) { /* slices [0,n-ws), [n-ws,n-shift), [n-shift,n) */
  if (i < n - ws) return 0;
  if (i < n - shift) return 1;
  return 2;
}

int oracle_swin_index_maps(int H, int W, int ws, int shift, int32_t *gather_idx,
                           int32_t *scatter_idx, int32_t *relpos_idx, int32_t *region_id) {
  if (H <= 0 || W <= 0 || ws <= 0 || H % ws || W % ws || shift < 0 || shift >= ws) return -2;
  const int nWw = W / ws, N = ws * ws;
  /* rolled[i][j] = x[(i+shift)%H][(j+shift)%W]  (torch.roll by -shift);
   * window = (i/ws)*nWw + j/ws, slot = (i%ws)*ws + j%ws (view+permute partition). */
  for (int i = 0; i < H; ++i) for (int j = 0; j < W; ++j) {
    const int w = (i / ws) * nWw + (j / ws), n = (i % ws) * ws + (j % ws);
    const int src = ((i + shift) % H) * W + ((j + shift) % W);
    if (gather_idx) gather_idx[w * N + n] = src;
    if (scatter_idx) scatter_idx[src] = w * N + n;
    if (region_id) region_id[w * N + n] = shift > 0 ? 3 * region_of(i, H, ws, shift) + region_of(j, W, ws, shift) : 0;
  }
  if (relpos_idx)
    for (int p = 0; p < N; ++p) for (int q = 0; q < N; ++q) {
      const int di = p / ws - q / ws + ws - 1, dj = p % ws - q % ws + ws - 1;
      relpos_idx[p * N + q] = di * (2 * ws - 1) + dj;
    }
  return 0;
}

int oracle_swin_block_f32(const oracle_swin_cfg *c, const oracle_swin_block_w *w,
                          const float *x, float *y, int num_threads) {
  if (!c || !w || !x || !y) return -1;
  const int H = c->height, W = c->width, C = c->channels, nh = c->heads, ws = c->window;
  if (C % nh || H % ws || W % ws || ws * ws > 1024) return -2;
  const int T = H * W, N = ws * ws, nW = T / N, hd = C / nh, F = C * c->mlp_ratio;
  const float qscale = 1.0f / sqrtf((float)hd);
  int32_t *gidx = (int32_t *)malloc(sizeof(int32_t) * (size_t)T);
  int32_t *rel = (int32_t *)malloc(sizeof(int32_t) * (size_t)N * N);
  int32_t *reg = (int32_t *)malloc(sizeof(int32_t) * (size_t)T);
  float *z = (float *)malloc(sizeof(float) * (size_t)T * C);
  float *zw = (float *)malloc(sizeof(float) * (size_t)T * C);
  float *qkv = (float *)malloc(sizeof(float) * (size_t)T * 3 * C);
  float *att = (float *)malloc(sizeof(float) * (size_t)T * C);
  float *x1 = (float *)malloc(sizeof(float) * (size_t)T * C);
  float *hbuf = (float *)malloc(sizeof(float) * (size_t)T * F);
  int rc = oracle_swin_index_maps(H, W, ws, c->shift, gidx, NULL, rel, reg);
  if (rc) goto done;
  /* Part-1: LN1, roll, partition */
  oracle_layernorm_f32(x, w->ln1_g, w->ln1_b, z, T, C, c->ln_eps);
  for (int s = 0; s < T; ++s) memcpy(zw + (size_t)s * C, z + (size_t)gidx[s] * C, sizeof(float) * (size_t)C);
  /* Part-2: qkv */
  oracle_gemm_f32(zw, w->w_qkv, w->b_qkv, qkv, T, 3 * C, C, num_threads);
  /* Part-3/4: per (window, head) attention with relative-position bias (+ shift mask) */
#pragma omp parallel for collapse(2) schedule(static)
  for (int wi = 0; wi < nW; ++wi) for (int hh = 0; hh < nh; ++hh) {
    float row[1024];
    for (int p = 0; p < N; ++p) {
      const float *qr = qkv + ((size_t)wi * N + p) * 3 * C + (size_t)hh * hd;
      float mx = -INFINITY;
      for (int q = 0; q < N; ++q) {
        const float *kr = qkv + ((size_t)wi * N + q) * 3 * C + C + (size_t)hh * hd;
        float a = 0.f;
        for (int d = 0; d < hd; ++d) a += (qr[d] * qscale) * kr[d];
        if (w->rel_table) a += w->rel_table[(size_t)rel[p * N + q] * nh + hh];
        if (c->shift > 0 && c->use_shift_mask && reg[wi * N + p] != reg[wi * N + q]) a += -100.0f;
        row[q] = a; if (a > mx) mx = a;
      }
      float sum = 0.f;
      for (int q = 0; q < N; ++q) { row[q] = expf(row[q] - mx); sum += row[q]; }
      float *o = att + ((size_t)wi * N + p) * C + (size_t)hh * hd;
      for (int d = 0; d < hd; ++d) o[d] = 0.f;
      for (int q = 0; q < N; ++q) {
        const float pq = row[q] / sum;
        const float *vr = qkv + ((size_t)wi * N + q) * 3 * C + 2 * C + (size_t)hh * hd;
        for (int d = 0; d < hd; ++d) o[d] += pq * vr[d];
      }
    }
  }
  /* Part-5: proj ; Part-6: reverse + roll back + shortcut */
  oracle_gemm_f32(att, w->w_proj, w->b_proj, zw, T, C, C, num_threads);
  for (int s = 0; s < T; ++s) {
    const float *src = zw + (size_t)s * C; const size_t tok = (size_t)gidx[s];
    for (int ch = 0; ch < C; ++ch) x1[tok * C + ch] = x[tok * C + ch] + src[ch];
  }
  /* Part-7/8: x1 + FC2(GELU(FC1(LN2(x1)))) */
  oracle_layernorm_f32(x1, w->ln2_g, w->ln2_b, z, T, C, c->ln_eps);
  oracle_gemm_f32(z, w->w_fc1, w->b_fc1, hbuf, T, F, C, num_threads);
  for (size_t i = 0; i < (size_t)T * F; ++i) hbuf[i] = oracle_gelu_tanh(hbuf[i]);
  oracle_gemm_f32(hbuf, w->w_fc2, w->b_fc2, z, T, C, F, num_threads);
  for (size_t i = 0; i < (size_t)T * C; ++i) y[i] = x1[i] + z[i];
done:
  free(gidx); free(rel); free(reg); free(z); free(zw); free(qkv); free(att); free(x1); free(hbuf);
  return rc;
}

int oracle_swin_block_pair_f32(const oracle_swin_cfg *c, const oracle_swin_block_w w[2],
                               const float *x, float *y, int num_threads) {
  if (!c || !w) return -1;
  const size_t n = (size_t)c->height * c->width * c->channels;
  float *mid = (float *)malloc(sizeof(float) * n);
  if (!mid) return -3;
  oracle_swin_cfg c0 = *c; c0.shift = 0;
  int rc = oracle_swin_block_f32(&c0, &w[0], x, mid, num_threads);
  if (rc == 0) rc = oracle_swin_block_f32(c, &w[1], mid, y, num_threads);
  free(mid);
  return rc;
}

int oracle_swin_ffn_f32(const float *x, const float *w1, const float *w2, float *y1, float *y2,
                        int M, int K, int F, int num_threads) {
  if (!x || !w1 || !w2 || !y1 || !y2) return -1;
  oracle_gemm_f32(x, w1, NULL, y1, M, F, K, num_threads);
  oracle_gemm_f32(y1, w2, NULL, y2, M, K, F, num_threads);
  return 0;
}

/* Patch merging (python/models/swin_transformer/swin_patch_merge.py:3-13 and the tensor expression
 * :49-63): merged[m][q*C + c] = x[2i + q%2][2j + q/2][c] with m = i*(W/2) + j, then LayerNorm over
 * the 4C merged channels (:95-144; biased variance, eps inside the root) and the bias-free
 * reduction y = LN(merged) . w, w [4C][2C]. */
int oracle_swin_patch_merge_f32(const float *x, const float *ln_g, const float *ln_b, const float *w, float *y,
                                int height, int width, int channels, float ln_eps, int num_threads) {
  if (!x || !w || !y || height <= 0 || width <= 0 || (height & 1) || (width & 1) || channels <= 0) return -1;
  const int H2 = height / 2, W2 = width / 2, M = H2 * W2, K = 4 * channels, N = 2 * channels;
  float *merged = (float *)malloc(sizeof(float) * (size_t)M * K);
  float *z = (float *)malloc(sizeof(float) * (size_t)M * K);
  if (!merged || !z) { free(merged); free(z); return -3; }
  for (int i = 0; i < H2; ++i)
    for (int j = 0; j < W2; ++j)
      for (int q = 0; q < 4; ++q)
        for (int c = 0; c < channels; ++c)
          merged[((size_t)i * W2 + j) * K + q * channels + c] =
              x[((size_t)(2 * i + q % 2) * width + 2 * j + q / 2) * channels + c];
  oracle_layernorm_f32(merged, ln_g, ln_b, z, M, K, ln_eps);
  oracle_gemm_f32(z, w, NULL, y, M, N, K, num_threads);
  free(merged); free(z);
  return 0;
}
