/*
 * CPU oracle for the fused-encoder hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain C, fp32 arithmetic on caller-supplied (already fp16-rounded) fp32
 * data.  It restates the op sequences of the reference's CUDA bindings so
 * that the HIP kernels can be checked against them.  Only tests, the smoke
 * entry and the benchmark's CPU-baseline leg may load this library; the
 * product library never links or calls it.
 *
 * Pinning status (what independently fixes each function; see tests/):
 *   oracle_bert_layer_f32      torch CPU library ops (matmul, softmax,
 *                              layer_norm, gelu(tanh)/relu) + closed-form
 *                              special cases + committed golden vectors
 *   oracle_lstm_f32            torch.nn.LSTMCell stack + analytic special cases
 *   oracle_swin_index_maps     torch.roll / view+permute window partition,
 *                              brute force on tiny grids, permutation laws
 *   oracle_swin_block_pair_f32 torch CPU library restatement of a Swin block
 *   oracle_swin_patch_merge_f32  the reference's own torch statement (strided slices, cat,
 *                              layer_norm, matmul; swin_patch_merge.py:3-13) in float64 and its
 *                              tensor-expression index formula evaluated by brute force
 *   oracle_se_module_f32       torch avg_pool2d / conv2d / sigmoid composition
 *   oracle_pointwise_conv_f32, oracle_depthwise_conv_f32, oracle_se_gate_f32,
 *   oracle_mbconv_block_f32    torch conv2d (groups / stride / explicit padding), adaptive
 *                              average pooling, sigmoid in float64; brute force on tiny inputs
 *   oracle_bert_embed_f32      torch.nn.functional.embedding + layer_norm (float64)
 *   oracle_bert_pooler_f32     torch matmul + tanh (float64), transposition rule of the
 *                              reference (cpp/bert/test_souffle_bert_layer.py:139-143)
 * No function here is "parity unpinned".
 *
 * Layout rule used everywhere: a weight matrix is stored [K][N] with N
 * contiguous and Y[m][n] = sum_k X[m][k] * W[k][n]
 * (reference: cpp/bert/kernels/gemm_three_stages.h:95-131,292-313;
 *  cpp/bert/test_souffle_bert_layer.py:139-143).
 */
#ifndef SOUFFLE_ORACLE_H
#define SOUFFLE_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { ORACLE_ACT_GELU_TANH = 0, ORACLE_ACT_RELU = 1, ORACLE_ACT_NONE = 2, ORACLE_ACT_GELU_ERF = 3 };

typedef struct {
  int batch, seq_len, hidden, heads, ffn;
  int act;          /* ORACLE_ACT_* */
  float scale;      /* multiplies q.k before softmax */
  float ln_eps;
} oracle_bert_cfg;

/* All pointers are host fp32.  Nullable: every bias, ln gamma/beta (treated as
 * 0 / 1 / 0), mask, and every dump pointer. */
typedef struct {
  const float *w_qkv;  /* [3][H][H]   */
  const float *b_qkv;  /* [3][H]      */
  const float *w_o;    /* [H][H]      */
  const float *b_o;    /* [H]         */
  const float *ln1_g, *ln1_b; /* [H]  */
  const float *w_fc1;  /* [H][F]      */
  const float *b_fc1;  /* [F]         */
  const float *w_fc2;  /* [F][H]      */
  const float *b_fc2;  /* [H]         */
  const float *ln2_g, *ln2_b; /* [H]  */
} oracle_bert_weights;

typedef struct {
  float *qkv;    /* [3][B][heads][S][hd]  (reference output_qkv)          */
  float *probs;  /* [B][heads][S][S]      (reference query_key_output)    */
  float *ctx;    /* [B*S][H]              (reference attn_value_output)   */
  float *ln1;    /* [B*S][H]  post-LN1    (reference attn_fc_output)      */
  float *fc1;    /* [B*S][F]  post-act    (reference feed_forward_fc1_output) */
} oracle_bert_dump;

/* One encoder layer.  mask: additive [B][S][S] or NULL.  y: [B*S][H]. */
int oracle_bert_layer_f32(const oracle_bert_cfg *cfg, const oracle_bert_weights *w,
                          const float *x, const float *mask, float *y,
                          const oracle_bert_dump *dump, int num_threads);
/* num_layers layers applied in sequence (distinct weights per layer). */
int oracle_bert_encoder_f32(const oracle_bert_cfg *cfg, const oracle_bert_weights *layers,
                            int num_layers, const float *x, const float *mask, float *y,
                            int num_threads);

/* Single ops exposed for unit pinning. */
/* Front / back of the encoder (cpp/bert/test_souffle_bert_layer.py:186-189; standard BERT pooler). */
int oracle_bert_embed_f32(const int32_t *token_ids, const int32_t *segment_ids, const float *word_emb,
                          const float *pos_emb, const float *type_emb, const float *ln_g, const float *ln_b,
                          float eps, int batch, int seq_len, int hidden, float *out);
int oracle_bert_pooler_f32(const float *x, const float *w, const float *bias, int batch, int seq_len, int hidden,
                           float *out);

void oracle_gemm_f32(const float *x, const float *w, const float *bias, float *y,
                     int M, int N, int K, int num_threads);
void oracle_layernorm_f32(const float *z, const float *g, const float *b, float *y,
                          int rows, int dim, float eps);
float oracle_gelu_tanh(float x);
float oracle_gelu_erf(float x);

/* ---- stacked LSTM ---- */
enum { ORACLE_GATES_IFGO = 0, ORACLE_GATES_IGFO = 1 };
typedef struct {
  int layers, hidden, timesteps, batch;
  int gate_order;      /* ORACLE_GATES_* : slot meaning of the 4 gate matrices */
  float forget_bias;   /* added to the forget pre-activation */
} oracle_lstm_cfg;
/* w_ih, w_hh: [layers*4][hidden(out)][hidden(in)]; bias: [layers][4][hidden] or NULL;
 * x: [batch][T][hidden]; y: [batch][T][hidden] (top layer h).  Zero initial state. */
int oracle_lstm_f32(const oracle_lstm_cfg *cfg, const float *w_ih, const float *w_hh,
                    const float *bias, const float *x, float *y);

/* ---- Swin ---- */
typedef struct {
  int height, width, channels, heads, window, shift, mlp_ratio;
  int use_shift_mask;  /* apply the -100 region mask in the shifted block */
  float ln_eps;
} oracle_swin_cfg;
typedef struct {
  const float *ln1_g, *ln1_b;
  const float *w_qkv, *b_qkv;   /* [C][3C], [3C] : columns ordered (q|k|v) x head x hd */
  const float *rel_table;       /* [(2ws-1)^2][heads] */
  const float *w_proj, *b_proj; /* [C][C], [C] */
  const float *ln2_g, *ln2_b;
  const float *w_fc1, *b_fc1;   /* [C][rC], [rC] */
  const float *w_fc2, *b_fc2;   /* [rC][C], [C] */
} oracle_swin_block_w;
/* Index maps for one (H,W,window,shift): 
 *  gather_idx[w*N+n]  = flat token h*W+w_ that lands at slot n of window w after roll(-shift)+partition
 *  scatter_idx[token] = w*N+n (the inverse permutation; also what reverse+roll(+shift) reads)
 *  relpos_idx[p*N+q]  = row of the relative-position table
 *  region_id[w*N+n]   = shifted-window region label (0..8); mask(p,q) = region differs ? -100 : 0 */
int oracle_swin_index_maps(int height, int width, int window, int shift,
                           int32_t *gather_idx, int32_t *scatter_idx,
                           int32_t *relpos_idx, int32_t *region_id);
/* One block (shift as given in cfg).  x,y: [H*W][C]. */
int oracle_swin_block_f32(const oracle_swin_cfg *cfg, const oracle_swin_block_w *w,
                          const float *x, float *y, int num_threads);
/* Regular block (shift 0) followed by shifted block (cfg->shift). */
int oracle_swin_block_pair_f32(const oracle_swin_cfg *cfg, const oracle_swin_block_w w[2],
                               const float *x, float *y, int num_threads);
/* Y1 = X.W1 ; Y2 = Y1.W2 (no bias, no activation) -- the reference's fused Swin FFN. */
int oracle_swin_ffn_f32(const float *x, const float *w1, const float *w2, float *y1, float *y2,
                        int M, int K, int F, int num_threads);

/* x [H][W][C] -> y [(H/2)*(W/2)][2C]; ln_g / ln_b [4C] nullable; w [4C][2C]. */
int oracle_swin_patch_merge_f32(const float *x, const float *ln_g, const float *ln_b, const float *w, float *y,
                                int height, int width, int channels, float ln_eps, int num_threads);

/* ---- EfficientNet SE module ---- */
enum { ORACLE_SE_MUL = 0, ORACLE_SE_ADD = 1 };
/* x,y: [C][H*W] (NCHW, batch 1); w_reduce [R][C]; w_expand [C][R]; biases nullable.
 * pooled: [C] mean (nullable out). */
int oracle_se_module_f32(const float *x, const float *w_reduce, const float *b_reduce,
                         const float *w_expand, const float *b_expand, float *y, float *pooled,
                         int C, int HW, int R, int combine);

/* ---- EfficientNet MBConv operators (NHWC, batch 1) ---- */
enum { ORACLE_MB_NONE = 0, ORACLE_MB_SWISH = 1 };
typedef struct {
  int in_h, in_w, in_c, expand_c, out_c, kernel, stride, se_c, has_shortcut;
  const float *expand_w, *expand_scale, *expand_shift;   /* [expand_c][in_c]; NULL = no expansion conv */
  const float *dw_w, *dw_scale, *dw_shift;               /* [kernel][kernel][expand_c] */
  const float *se_reduce_w, *se_reduce_b;                /* [se_c][expand_c], [se_c] */
  const float *se_expand_w, *se_expand_b;                /* [se_c][expand_c] (input-major), [expand_c] */
  const float *project_w, *project_scale, *project_shift;/* [out_c][expand_c] */
} oracle_mbconv_block;
/* x [pixels][in_c], w [out_c][in_c]; scale/shift/gate/shortcut nullable. */
int oracle_pointwise_conv_f32(const float *x, const float *w, const float *scale, const float *shift,
                              const float *gate, const float *shortcut, float *y,
                              int pixels, int in_c, int out_c, int act, int num_threads);
int oracle_depthwise_out_extent(int in, int kernel, int stride);
/* x [in_h][in_w][C], w [kernel][kernel][C] -> y [oh][ow][C]. */
int oracle_depthwise_conv_f32(const float *x, const float *w, const float *scale, const float *shift, float *y,
                              int in_h, int in_w, int channels, int kernel, int stride, int act, int num_threads);
int oracle_se_gate_f32(const float *x, const float *w_reduce, const float *b_reduce, const float *w_expand,
                       const float *b_expand, float *gate, int pixels, int channels, int squeezed);
int oracle_mbconv_block_f32(const oracle_mbconv_block *b, const float *x, float *y, float *dump_e, float *dump_d,
                            int round_fp16, int num_threads);
#ifdef __cplusplus
}
#endif
#endif
