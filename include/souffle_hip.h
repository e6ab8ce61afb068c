/*
 * souffle_hip.h -- C ABI of libsouffle_hip.so: the MI355X (gfx950) implementation of
 * the fused-encoder hot path of summerspringwei/souffle-models.
 *
 * Conventions
 *   - every entry point returns 0 on success or a negative souffle_status; the text
 *     of the last failure on the calling thread is at souffle_last_error();
 *   - no entry point aborts, prints, synchronises the device or allocates device
 *     memory: all buffers (inputs, outputs, workspace) are caller-owned device
 *     pointers, 16-byte aligned, and the work is queued on the given HIP stream
 *     (souffle_stream_t is a hipStream_t; NULL = the default stream);
 *   - a workspace must be zeroed once with souffle_workspace_init() before its
 *     first use (all of it: it holds grid-barrier state, step tags and hand-over
 *     words); it may then be reused by any number of calls of any entry point and
 *     configuration, one at a time.  Calls that share a workspace must not overlap;
 *   - weights are fp16 matrices stored [K][N] with N contiguous, Y = X.W
 *     (reference: cpp/bert/kernels/gemm_three_stages.h:95-131,
 *      cpp/bert/test_souffle_bert_layer.py:139-143); activations are fp16 row-major.
 *
 * Each declaration cites the reference interface it replaces.
 */
#ifndef SOUFFLE_HIP_H
#define SOUFFLE_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef void *souffle_stream_t;

enum souffle_status {
  SOUFFLE_OK = 0,
  SOUFFLE_ERR_NULL = -1,        /* a required pointer is NULL */
  SOUFFLE_ERR_SHAPE = -2,       /* unsupported shape / configuration */
  SOUFFLE_ERR_ALIGN = -3,       /* a pointer is not 16-byte aligned */
  SOUFFLE_ERR_WORKSPACE = -4,   /* workspace missing or too small */
  SOUFFLE_ERR_DEVICE = -5,      /* no usable gfx950 device / query failed */
  SOUFFLE_ERR_LAUNCH = -6,      /* the HIP launch was rejected (text has the HIP error) */
  SOUFFLE_ERR_UNSUPPORTED = -7
};

/* Replaces checkCuda's print+assert (cpp/souffle_utils/cuda_utils.h:10-19). */
const char *souffle_last_error(void);
const char *souffle_version(void);

/* Replaces check_compatability (cpp/souffle_utils/cuda_utils.h:86-98): the device
 * facts the launch geometry and the roofline are derived from. */
typedef struct {
  int num_cus, lds_bytes_per_cu, clock_khz, mem_clock_khz, mem_bus_bits, l2_bytes;
  int cooperative_launch, wavefront_size;
  char arch[64];
} souffle_devinfo;
int souffle_device_info(souffle_devinfo *out);
/* Queues a persistent kernel of `stages` dependent grid-wide stages without arithmetic on an initialised
 * workspace (souffle_workspace_init; 16 KiB are enough).  mode 0: the grid barrier alone; mode 1: 16 bytes
 * written through, the barrier, and a read of what a workgroup of another XCD wrote, per stage.  Timed by
 * the caller it gives the latency floor of a chain of dependent stages on this device, which bounds the
 * skinny shapes (B*S up to about a thousand rows) rather than the HBM or MFMA roofline. */
int souffle_stage_floor_probe(void *workspace, size_t workspace_bytes, int stages, int mode, souffle_stream_t stream);
/* Queues one MFMA-only kernel (4 waves per CU, `iters` x 16 independent fp16 16x16x32 MFMAs per wave, no
 * memory traffic) and reports the flops it performs: timed by the caller, it gives the empirical
 * matrix-core ceiling that the published peak is compared with.  `out` takes 2 KiB per CU of results. */
int souffle_mfma_probe(float *out, size_t out_bytes, int iters, double *flops, souffle_stream_t stream);
/* Queues a kernel in which every workgroup (one per CU) only streams `src` (device memory, 64 KiB..1 GiB,
 * 16-byte aligned; a few MiB stay L2-resident) into LDS with wave-wide 16-byte direct loads, `iters` x 8 KiB
 * per wave, and reports the bytes it moves: timed by the caller, it gives the rate at which the CUs can take
 * operands from the L2s when they do nothing else (the GEMM tiles take theirs in at a third of it).  Like the probes
 * above it has no counterpart in the reference (cpp/souffle_utils/cuda_utils.h:102-136 only times kernels). */
int souffle_l2_stream_probe(const void *src, size_t src_bytes, int iters, double *bytes, souffle_stream_t stream);

/* Zero a workspace, all workspace_bytes of it (stream-ordered fill kernel, no allocation, capturable).
 * Once before the first use, and again after a launch that reported a failed wait.
 * The reference instead zero-allocates its scratch on every call
 * (cpp/bert/bert_binding.cu:32-78). */
int souffle_workspace_init(void *workspace, size_t workspace_bytes, souffle_stream_t stream);

/* In-kernel stage timestamps.  Replaces the profile_clock tensors the reference's fused
 * kernels fill with clock64() per (stage, block, warp) (cpp/bert/bert_binding.cu:67-76,111-114).
 * While a buffer is set, every persistent kernel stamps the 100 MHz wall clock on entry to and
 * exit from each of its grid barriers: uint64 buf[(2*i + {0,1}) * grid + block] for barrier i,
 * i < cap = bytes / (grid * 80); up to 8 marks inside the stage before barrier i follow at
 * buf[(2*cap + 8*i + id) * grid + block].  Pass NULL to switch tracing off (the default). */
int souffle_set_stage_trace(void *device_buf, size_t bytes);

/* How the persistent kernels (those whose workgroups wait for one another: grid barriers, flag hand-overs) are
 * launched.  The reference launches its fused kernels with cudaLaunchCooperativeKernel
 * (cpp/swin_transformer/swin_transformer_binding.cu:95, cpp/efficientnet/efficientnet_se_module_main.cu:62).
 * On MI355X a cooperative launch costs about 13 us more than a plain one (282 against 269 us for the 12-layer
 * encoder at B=1, S=128), so the default (on = 0) is a plain hipLaunchKernel of a grid that the occupancy query has
 * shown to fit the device at once.  Precondition of that default: the device runs nothing else while a fused call
 * runs.  Fused calls must not overlap in time with other kernels on another stream or of another process (two
 * half-resident grids would wait for each other); every wait in the kernels is bounded, so such a call ends, sets
 * the sticky failure flag of its workspace and leaves an invalid output: check souffle_workspace_status (or
 * souffle_bert_static_status) where that cannot be excluded.  on = 1 restores the runtime's guarantee and needs a
 * device that supports cooperative launches.  The environment variable SOUFFLE_COOPERATIVE_LAUNCH=1 sets the
 * initial value. */
int souffle_set_cooperative_launch(int on);

/* The hand-overs between the workgroups of the persistent kernels (flag words of the encoder, grid barriers,
 * row-block and window hand-overs) rest on write-through stores that are acknowledged before the flag is stored and
 * on cache-coherent (sc1) loads behind the poll; on MI355X that is sufficient and costs about 2 us per hand-over.
 * on != 0 adds what the memory model prescribes by the book to every one of them: an agent-scope release fence in
 * front of the flag store and an agent-scope acquire fence behind the poll (an L2 write-back and an L1/L2
 * invalidation each time; about 14 us per hand-over).  Same results, bit for bit.  For a driver, firmware or part
 * whose caches are not known to behave as measured here, and for checking a suspected coherence problem.
 * The environment variable SOUFFLE_STRICT_FENCES=1 sets the initial value.  The reference separates its stages
 * with cooperative-groups grid.sync() (cpp/bert/kernels/fused_sqq_bert.cu), which carries these fences always. */
int souffle_set_strict_fences(int on);

/* Reads (and optionally clears) the sticky failure flags of a workspace after waiting for
 * `stream`: 0 = every launch that used it ran to completion; bit 0 = an LSTM wait, bit 1 = a
 * grid barrier or a hand-over of the encoder gave up (bounded spins; the output of
 * that launch is invalid).  Replaces the reference's abort on a CUDA error after its blocking
 * cudaDeviceSynchronize (cpp/bert/bert_binding.cu:532, cpp/souffle_utils/cuda_utils.h:10-19).
 * This is the one entry point that synchronises. */
int souffle_workspace_status(void *workspace, souffle_stream_t stream, unsigned *flags, int clear);

/* ------------------------------------------------------------------ BERT ---- */
/* GELU_ERF: 0.5 x (1 + erf(x / sqrt 2)), the form that HuggingFace BERT checkpoints (config "gelu") were trained with,
 * which cpp/bert/test_souffle_bert_layer.py:131-143,161 loads; the reference's own kernels compute the tanh form
 * (cpp/bert/bert_base_impl.cu:722-734) or ReLU (cpp/bert/kernels/fused_sqq_feedforward.cu:327-341). */
enum { SOUFFLE_ACT_GELU_TANH = 0, SOUFFLE_ACT_RELU = 1, SOUFFLE_ACT_GELU_ERF = 2 };

typedef struct {
  int batch, seq_len;          /* runtime; seq_len <= 512.  Lengths other than 64/128/256/384/512 run as the next of
                                  these with the surplus keys masked out (rows copied in and out through the
                                  workspace; not with per-stage dump tensors) */
  int hidden, heads, ffn;      /* 768, 12, 3072 (the reference's compile-time family, cpp/bert/kernels/bert.h:8-16) */
  int act;                     /* SOUFFLE_ACT_*; reference fused path uses ReLU, its unfused path tanh-GELU */
  float scale;                 /* multiplies q.k (0.125 = 1/sqrt(64)) */
  float ln_eps;
  int num_layers;              /* used by the encoder entry points */
  int reserved;
} souffle_bert_cfg;

/* fp16 device pointers; every bias and LN vector may be NULL (0 / gamma 1 / beta 0).
 * Roles as in cpp/bert/bert_binding.cu:25-29 (weights) and cpp/bert/bert_base_impl.cu:151-189 (biases, LN). */
typedef struct {
  const void *w_qkv;  /* [3][768][768] */
  const void *b_qkv;  /* [3][768]      */
  const void *w_o;    /* [768][768]    */
  const void *b_o;    /* [768]         */
  const void *ln1_g, *ln1_b;
  const void *w_fc1;  /* [768][3072]   */
  const void *b_fc1;  /* [3072]        */
  const void *w_fc2;  /* [3072][768]   */
  const void *b_fc2;  /* [768]         */
  const void *ln2_g, *ln2_b;
  const void *w_fc2_packed;  /* optional: the copy of w_fc2 that souffle_bert_pack_fc2 makes, or NULL */
} souffle_bert_layer_w;

/* A one-time copy of a layer's w_fc2 ([3072][768], which stays required) in the order the few-rows encoder reads it:
 * 48 slices of 16 output columns, each the 96 k-steps of its MFMA operands, contiguous (souffle_bert_fc2_packed_bytes()
 * = 3072 * 768 * 2 bytes, 16-byte aligned, not overlapping w_fc2).  Make it once when a model is loaded and pass it
 * as w_fc2_packed of the layer.  When EVERY layer of a call has it, and the call runs on the few-rows kernel (up to
 * 1024 rows, and below 1536 where the count is no multiple of 256), a workgroup computes 32 rows x 16 columns of FC2
 * over the whole K = 3072 and finishes them itself (bias, residual, row statistics).  Without it FC2 is cut into four
 * K quarters whose fp32 partial sums are exchanged through memory (the in-block split-K of
 * cpp/bert/kernels/gemm.cu:1260-1330 spread over four workgroups), which costs about 3 us more per layer.
 * Same arithmetic up to the order of the fp32 additions over K.  The reference keeps [K][N] only; it has no
 * counterpart of the packed copy. */
size_t souffle_bert_fc2_packed_bytes(void);
int souffle_bert_pack_fc2(const void *w_fc2, void *packed, souffle_stream_t stream);

/* Optional fp16 device outputs for the per-stage tensors the reference binding returns
 * (cpp/bert/bert_binding.cu:534); any member (or the struct pointer) may be NULL. */
typedef struct {
  void *qkv;    /* [3][B][12][S][64]  output_qkv              */
  void *probs;  /* [B][12][S][S]      query_key_output        */
  void *ctx;    /* [B*S][768]         attn_value_output       */
  void *ln1;    /* [B*S][768]         attn_fc_output (post-LN)*/
  void *fc1;    /* [B*S][3072]        feed_forward_fc1_output */
} souffle_bert_dump;

size_t souffle_bert_workspace_bytes(const souffle_bert_cfg *cfg);

/* One encoder layer as ONE persistent launch (plain by default, see souffle_set_cooperative_launch for the
 * launch mode and its precondition; failed waits are reported by souffle_workspace_status).
 * Replaces souffle_bert_layer<1,12,384,64,3072>(..., opt_level=3|4)
 * (cpp/bert/bert_binding.cu:23-535, fused path :395-528).
 * x,y: [B*S][768] fp16; mask: additive fp16 [B][S][S] or NULL. */
int souffle_bert_layer_fused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *w,
                             const void *x, const void *mask, void *y,
                             const souffle_bert_dump *dump,
                             void *workspace, size_t workspace_bytes, souffle_stream_t stream);
/* The same layer as separate per-op launches: the unfused HIP baseline.
 * Replaces opt_level 1|2 of the same binding (cpp/bert/bert_binding.cu:119-393)
 * and the per-op chain of Bert::Solve (cpp/bert/bert_base_impl.cu:590-678). */
int souffle_bert_layer_unfused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *w,
                               const void *x, const void *mask, void *y,
                               const souffle_bert_dump *dump,
                               void *workspace, size_t workspace_bytes, souffle_stream_t stream);
/* cfg->num_layers layers with distinct weights in one persistent launch (launch mode and precondition as for
 * souffle_bert_layer_fused) / as per-op launches.  Replaces souffle_bert_base() (cpp/bert/bert_base_impl.cu:277-308,590-678). */
int souffle_bert_encoder_fused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                               const void *x, const void *mask, void *y,
                               void *workspace, size_t workspace_bytes, souffle_stream_t stream);
int souffle_bert_encoder_unfused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                                 const void *x, const void *mask, void *y,
                                 void *workspace, size_t workspace_bytes, souffle_stream_t stream);

/* souffle_bert_encoder_fused without a workspace argument and without any allocation: the inter-phase
 * buffers, flag words and control block live in a 48 MiB array in device memory that belongs to the
 * library (one per GPU the library runs on, held until the process ends).  It has no counterpart in the
 * reference; it is for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Same results as souffle_bert_encoder_fused.  A configuration whose
 * workspace (souffle_bert_workspace_bytes) exceeds the array is refused with SOUFFLE_ERR_WORKSPACE
 * (12 layers fit at up to 128 rows, fewer layers at more).  Every call on a GPU uses that GPU's one
 * array: calls that overlap on one GPU (two streams, two threads) race.  Nothing is cleared between calls (the
 * array starts as zeros when the library is loaded; flag values only grow from call to call), so the same work
 * is enqueued whatever was called before.  Under graph capture: make one eager call of the same configuration
 * first (the first call on a device looks the array's address up, and the first call of a kernel variant sets
 * its LDS size and asks the occupancy query, which are not stream work), and replay the graph only while
 * nothing else uses the array.  The sticky failure word of the bounded waits is read with
 * souffle_bert_static_status. */
int souffle_bert_encoder_fused_static(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                                      const void *x, const void *mask, void *y, souffle_stream_t stream);
/* souffle_workspace_status for the array of souffle_bert_encoder_fused_static on the current device (waits for
 * `stream`; allocates nothing).  No counterpart in the reference; for the same callers. */
int souffle_bert_static_status(souffle_stream_t stream, unsigned *flags, int clear);

/* The work split and the hand-over plan of the encoder at few rows (up to 1024, and below 1536 where the count is
 * no multiple of 256), evaluated on the host by the functions the
 * kernel itself uses (no GPU needed; no counterpart in the reference, whose stages are separated by grid barriers):
 * the items of `workgroup` in `phase` (0 QKV, 1 attention, 2 out-projection, 3 FC1, 4 FC2, 6 final LayerNorm) as
 * pairs (m-tile, weight slice) - attention: (block of 16 queries, batch * 12 + head); FC2: slice = 16 output columns
 * when fc2_packed != 0 (every layer brings w_fc2_packed), else 64-column slice * 4 + K quarter - written to items[2 i], items[2 i + 1]
 * (at most max_items pairs; *n_items is their true number), and needs[p] = 1 for every workgroup p of the `grid` whose
 * publication of the phase before the workgroup waits for (phases 1..4; QKV of a later layer and the final LayerNorm
 * wait for FC2: with fc2_packed for the publications of its workgroups, reported here for phases 0 and 6 too, otherwise
 * for the completion words of the twelve FC2 tiles of their m-tile).  items and needs may be NULL. */
int souffle_bert_handover_plan(int batch, int seq_len, int grid, int fc2_packed, int phase, int workgroup, int *items, int max_items,
                               int *n_items, unsigned char *needs);

/* Which copy of its hand-over words each XCD polls in the few-rows encoder, read back from a workspace (a diagnostic;
 * synchronises the stream; no counterpart in the reference).  The words exist in 16 copies of 4 KB, two per XCD and
 * 8 KB apart (their addresses differ in bit 13 only), so that one of the two lies in memory channels on the XCD's side of the package; workgroup x of XCD x
 * times loads of both at the end of each of the first 8 launches on a workspace and the majority decides.
 * votes_cast[x] = votes so far (0..8), copy_block[x] = the 4 KB block XCD x polls in the next launch. */
int souffle_bert_polled_copies(const void *ws, size_t ws_bytes, int *votes_cast, int *copy_block, souffle_stream_t stream);

/* The stage in front of the encoder: out[b*S+s] = LayerNorm(word_emb[token_ids[b*S+s]] +
 * pos_emb[s] + type_emb[segment_ids[b*S+s]]) in fp16, statistics in fp32.  Replaces the
 * HuggingFace embedding module the reference feeds its layer with
 * (cpp/bert/test_souffle_bert_layer.py:186-189; python/models/bert/relay_bert.py:12-13 starts
 * from its [1,384,768] output).  token_ids / segment_ids: int32 device arrays [B*S]
 * (segment_ids and type_emb may be NULL); tables fp16 [rows][768] with vocab_size, max_positions
 * (>= seq_len, else SOUFFLE_ERR_SHAPE) and type_vocab_size rows.  The ids live on the device, so the
 * call cannot refuse them: an id outside its table is clamped into it, never read out of bounds, and
 * counted in the device word *bad_ids (may be NULL; the caller zeroes it and reads it after the stream
 * has finished: a non-zero count means those rows of `out` are wrong). */
int souffle_bert_embed(const int32_t *token_ids, const int32_t *segment_ids,
                       const void *word_emb, int vocab_size, const void *pos_emb, int max_positions,
                       const void *type_emb, int type_vocab_size,
                       const void *ln_g, const void *ln_b, float ln_eps,
                       int batch, int seq_len, int hidden, void *out, uint32_t *bad_ids, souffle_stream_t stream);
/* The stage behind the encoder: out[b] = tanh(x[b*S + 0] . W + bias), W fp16 [768][768] stored
 * [K][N] like every weight here (transposition rule: cpp/bert/test_souffle_bert_layer.py:139-143);
 * out fp16 [B][768].  The reference stops at the last encoder layer. */
int souffle_bert_pooler(const void *x, const void *w, const void *bias,
                        int batch, int seq_len, int hidden, void *out, souffle_stream_t stream);

/* ------------------------------------------------------------------ LSTM ---- */
enum { SOUFFLE_GATES_IFGO = 0, SOUFFLE_GATES_IGFO = 1 };
typedef struct {
  int layers, hidden, timesteps, batch;  /* 10, 256, <=4096, 1 */
  int gate_order;                        /* slot meaning of the four gate matrices */
  float forget_bias;                     /* reference kernel: 1.0 (cpp/lstm/lstm_reuse_shared_memory.cu:314) */
} souffle_lstm_cfg;
size_t souffle_lstm_workspace_bytes(const souffle_lstm_cfg *cfg);
/* Replaces fused_lstm<1,10,256,100> (cpp/lstm/lstm_binding.cu:30-78).
 * w_ih, w_hh: fp16 [layers*4][hidden out][hidden in]; bias: fp32 [layers][4][hidden] or NULL;
 * x: fp32 [T][hidden]; y: fp32 [T][hidden] (top-layer h per step). */
int souffle_lstm_fused(const souffle_lstm_cfg *cfg, const void *w_ih, const void *w_hh,
                       const float *bias, const float *x, float *y,
                       void *workspace, size_t workspace_bytes, souffle_stream_t stream);

/* ------------------------------------------------------------------ Swin ---- */
typedef struct {
  int height, width, channels, heads, window, shift, mlp_ratio;  /* 56,56,128,4,7,3,4 */
  int use_shift_mask;
  float ln_eps;
} souffle_swin_cfg;
typedef struct {   /* fp16 device pointers, biases / LN vectors nullable */
  const void *ln1_g, *ln1_b;
  const void *w_qkv, *b_qkv;    /* [C][3C], [3C]  columns (q|k|v) x head x hd */
  const void *rel_table;        /* [(2w-1)^2][heads] or NULL */
  const void *w_proj, *b_proj;  /* [C][C], [C] */
  const void *ln2_g, *ln2_b;
  const void *w_fc1, *b_fc1;    /* [C][rC] */
  const void *w_fc2, *b_fc2;    /* [rC][C] */
} souffle_swin_block_w;
size_t souffle_swin_workspace_bytes(const souffle_swin_cfg *cfg);
/* How souffle_swin_block_pair_fused spreads a window: on != 0 (default) four workgroups per window (one
 * attention head and a quarter of the MLP each, two hand-overs through memory per block) while there are
 * at most half as many windows as CUs; 0: one workgroup per window.  SOUFFLE_SWIN_SPLIT=0 sets the
 * initial value.  Same arithmetic up to the order of the fp32 additions of FC2. */
int souffle_set_swin_split(int on);
/* Regular + shifted window block in one cooperative launch.  The op list is
 * python/models/swin_transformer/swin_transformer_main.py:11-61 (Part-1..8), which the
 * reference only runs as separate TVM kernels (:196-330).  x,y: fp16 [H*W][C]. */
int souffle_swin_block_pair_fused(const souffle_swin_cfg *cfg, const souffle_swin_block_w w[2],
                                  const void *x, void *y,
                                  void *workspace, size_t workspace_bytes, souffle_stream_t stream);
/* Host-side index maps (bit-exact contract).  Replaces the te index expressions of
 * python/models/swin_transformer/swin_self_attention.py:66-82,101-120,179-204,226-265.
 * gather_idx[w*N+n] = token; scatter_idx[token] = w*N+n; relpos_idx[p*N+q] = table row;
 * region_id[w*N+n] = shifted-window region label.  Any output may be NULL. */
int souffle_swin_index_maps(int height, int width, int window, int shift,
                            int32_t *gather_idx, int32_t *scatter_idx,
                            int32_t *relpos_idx, int32_t *region_id);
/* Y1 = X.W1 ; Y2 = Y1.W2, no bias / activation.
 * Replaces swin_fused_feed_mlp<1,256,512,2048> (cpp/swin_transformer/swin_transformer_binding.cu:154-209). */
int souffle_swin_ffn_fused(const void *x, const void *w1, const void *w2, void *y1, void *y2,
                           int M, int K, int F, void *workspace, size_t workspace_bytes,
                           souffle_stream_t stream);
/* Y = X.W.  Replaces swin_ffn (cpp/swin_transformer/swin_transformer_binding.cu:62-100) and
 * swin_trans_fc2 (cpp/swin_transformer/swin_trans_fc2_binding.cu:19-61). */
int souffle_gemm_f16(const void *x, const void *w, void *y, int M, int N, int K,
                     souffle_stream_t stream);

/* Patch merging between two Swin stages: x [H][W][C] -> y [(H/2)*(W/2)][2C],
 * y = LN(cat(x[0::2,0::2], x[1::2,0::2], x[0::2,1::2], x[1::2,1::2]); gamma, beta, eps) . w, w fp16 [4C][2C],
 * gamma/beta fp16 [4C] nullable.  H, W even, C a multiple of 32.
 * Replaces fused_patch_merging_reshape_reduce_sum, layer_normalization_variance,
 * layer_normalization_normal and the reduction product
 * (python/models/swin_transformer/swin_patch_merge.py:3-13,49-144). */
int souffle_swin_patch_merge(const void *x, const void *ln_g, const void *ln_b, const void *w, void *y,
                             int height, int width, int channels, float ln_eps, souffle_stream_t stream);

/* ----------------------------------------------------- EfficientNet SE ---- */
enum { SOUFFLE_SE_MUL = 0, SOUFFLE_SE_ADD = 1 };
size_t souffle_se_workspace_bytes(int C, int HW, int R);
/* Replaces torch_dispatch_efficientnet_se_module_v2_short_cut_fused
 * (cpp/efficientnet/efficientnet_se_module_binding.cu:164-227).
 * x,y: fp32 [C][H*W] (NCHW, batch 1); w_reduce fp32 [R][C]; w_expand fp32 [C][R];
 * biases nullable; pooled: fp32 [C] out (nullable). */
int souffle_se_module_fused(const float *x, const float *w_reduce, const float *b_reduce,
                            const float *w_expand, const float *b_expand,
                            float *y, float *pooled, int C, int HW, int R, int combine,
                            void *workspace, size_t workspace_bytes, souffle_stream_t stream);

/* ------------------------------------------------- EfficientNet MBConv ---- */
/* NHWC fp16 activations (batch 1), fp16 convolution weights, fp32 folded batch-norm vectors
 * (y = conv * scale + shift) and squeeze-excite biases.  Channel counts are multiples of 8. */
enum { SOUFFLE_MB_NONE = 0, SOUFFLE_MB_SWISH = 1 };
typedef struct {
  int in_h, in_w, in_c, expand_c, out_c;   /* expand_c == in_c and expand_w == NULL: no expansion convolution */
  int kernel, stride;                      /* depthwise: 3 or 5; 1 or 2; padding kernel/2 on every side */
  int se_c;                                /* squeezed channels; 0 = no squeeze-excite module */
  int has_shortcut;                        /* y += x; needs stride 1 and in_c == out_c */
  const void *expand_w;                    /* fp16 [expand_c][in_c] */
  const float *expand_scale, *expand_shift;
  const void *dw_w;                        /* fp16 [kernel][kernel][expand_c] */
  const float *dw_scale, *dw_shift;
  const void *se_reduce_w;                 /* fp16 [se_c][expand_c] */
  const float *se_reduce_b;                /* [se_c], nullable */
  const void *se_expand_w;                 /* fp16 [se_c][expand_c]: input-major, as se_module_pointwise_conv declares it */
  const float *se_expand_b;                /* [expand_c], nullable */
  const void *project_w;                   /* fp16 [out_c][expand_c] */
  const float *project_scale, *project_shift;
} souffle_mbconv_block;
/* 0 (and an error text) when the block list is not valid. */
size_t souffle_mbconv_workspace_bytes(const souffle_mbconv_block *blocks, int num_blocks);
/* A chain of MBConv blocks, x [in_h*in_w][in_c] of block 0 -> y [oh*ow][out_c] of the last block.
 * Replaces the per-block operator sequence of TVMMBConvBlock.forward
 * (python/models/efficientnet/tvm_efficientnet.py:62-118; operators
 * python/models/efficientnet/efficientnet.py:41-57,83-101,131-141,173-195,252-282,502-518).
 * fused != 0: one persistent launch per 16 blocks; fused == 0: one launch per operator group
 * (expansion | depthwise | squeeze-excite + projection), the same arithmetic. */
int souffle_mbconv_stack(const souffle_mbconv_block *blocks, int num_blocks, const void *x, void *y, int fused,
                         void *workspace, size_t workspace_bytes, souffle_stream_t stream);
/* y[p][o] = act((sum_k x[p][k] * gate[k] * w[o][k]) * scale[o] + shift[o]) + shortcut[p][o];
 * scale, shift, gate (fp32 [in_c]) and shortcut (fp16 [pixels][out_c]) nullable.
 * Replaces pointwise_conv2d_bn, pointwise_conv2d_bn_short_cut_add and head_conv1x1_bn_swish
 * (python/models/efficientnet/efficientnet.py:41-57,83-101,502-518). */
int souffle_pointwise_conv2d_bn(const void *x, const void *w, const float *scale, const float *shift,
                                const float *gate, const void *shortcut, void *y,
                                int pixels, int in_c, int out_c, int act, souffle_stream_t stream);
/* x [in_h][in_w][C], w [kernel][kernel][C] -> y [oh][ow][C], o = (in - 1) / stride + 1.
 * Replaces fused_depthwise_conv2d_bn_swish (python/models/efficientnet/efficientnet.py:173-195). */
int souffle_depthwise_conv2d_bn_swish(const void *x, const void *w, const float *scale, const float *shift,
                                      void *y, int in_h, int in_w, int channels, int kernel, int stride,
                                      souffle_stream_t stream);

/* ------------------------------------------------------------- timing ---- */
/* Replaces benchmarkCudaFunc (cpp/souffle_utils/cuda_utils.h:102-136): after `warmup`
 * launches, min over `rounds` of the mean of `repeat` event-timed launches, in us.
 * `fn(arg)` must queue exactly one unit of work on `stream`. */
int souffle_bench_us(int (*fn)(void *), void *arg, souffle_stream_t stream,
                     int warmup, int rounds, int repeat, double *min_of_means_us,
                     double *median_us);
#ifdef __cplusplus
}
#endif
#endif
