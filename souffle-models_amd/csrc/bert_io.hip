// Front and back of the BERT encoder on gfx950: the embedding stage that produces the
// [B*S][768] activations the encoder consumes, and the pooler that follows it.
//
// The reference feeds its layer with the output of the HuggingFace embedding module
// (cpp/bert/test_souffle_bert_layer.py:186-189: word + position + token-type embeddings,
// LayerNorm) and stops at the last encoder layer; the pooler is the standard BERT one
// (dense on the first token of every sequence, tanh).  Both are HBM-bound gathers / a skinny
// GEMV, one launch each.
#include "common.hpp"
#include "host_util.hpp"

namespace souffle {
namespace bert_io {

constexpr int H = 768;

// One wave per token: gather three rows, sum in fp32, two-pass LayerNorm in registers.
// An id outside its table is clamped into it (the row is then wrong, but no address outside the tables is read) and
// counted in *bad_ids.
__global__ void __launch_bounds__(256) k_embed(const int *tok, const int *seg, const half_t *word, int vocab, const half_t *pos,
                                               const half_t *type, int type_vocab, const half_t *gam, const half_t *bet, float eps,
                                               int rows, int S, half_t *out, unsigned *bad_ids) {
  const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= rows) return;
  const int t_raw = tok[m], p = m % S, sg_raw = seg ? seg[m] : 0;
  const int t = min(max(t_raw, 0), vocab - 1), sg = type ? min(max(sg_raw, 0), type_vocab - 1) : 0;
  if (lane == 0 && bad_ids && (t != t_raw || (type && sg != sg_raw))) atomicAdd(bad_ids, 1u);
  f4 v[3];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    const int n = c * 256 + lane * 4;
    const h4 a = *reinterpret_cast<const h4 *>(word + (size_t)t * H + n), b = *reinterpret_cast<const h4 *>(pos + (size_t)p * H + n);
    f4 s = f4{(float)a[0], (float)a[1], (float)a[2], (float)a[3]} + f4{(float)b[0], (float)b[1], (float)b[2], (float)b[3]};
    if (type) {
      const h4 ty = *reinterpret_cast<const h4 *>(type + (size_t)sg * H + n);
      s += f4{(float)ty[0], (float)ty[1], (float)ty[2], (float)ty[3]};
    }
    v[c] = s;
    sum += s[0] + s[1] + s[2] + s[3];
  }
  const float mean = wave_sum(sum) * (1.0f / H);
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < 3; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i) { const float d = v[c][i] - mean; sq += d * d; }
  const float rstd = rsqrtf(wave_sum(sq) * (1.0f / H) + eps);
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    const int n = c * 256 + lane * 4;
    f4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (v[c][i] - mean) * rstd;
    if (gam) {
      const h4 gg = *reinterpret_cast<const h4 *>(gam + n);
      o *= f4{(float)gg[0], (float)gg[1], (float)gg[2], (float)gg[3]};
    }
    if (bet) {
      const h4 bb = *reinterpret_cast<const h4 *>(bet + n);
      o += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
    }
    *reinterpret_cast<u2 *>(out + (size_t)m * H + n) = pack_h4(o);
  }
}

// pooled[b][n] = tanh(sum_k x[b*S][k] W[k][n] + bias[n]).  A workgroup takes 64 output columns of
// one sequence; its four waves split K and meet in LDS.  W is read once per sequence, coalesced
// along n (1.2 MB: the launch is bound by that stream).
__global__ void __launch_bounds__(256) k_pooler(const half_t *x, const half_t *w, const half_t *bias, int S, half_t *out) {
  __shared__ float part[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, b = blockIdx.y, n = blockIdx.x * 64 + lane;
  const half_t *xr = x + (size_t)b * S * H;
  float acc = 0.f;
  for (int k = wave * (H / 4); k < (wave + 1) * (H / 4); ++k) acc += (float)xr[k] * (float)w[(size_t)k * H + n];
  part[wave][lane] = acc;
  __syncthreads();
  if (wave == 0) {
    float s = part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane] + (bias ? (float)bias[n] : 0.f);
    // tanh(s) = 1 - 2 / (exp(2s) + 1); exp overflow gives the correct limit 1
    out[(size_t)b * H + n] = (half_t)(1.0f - 2.0f / (__expf(2.0f * s) + 1.0f));
  }
}

}  // namespace bert_io
}  // namespace souffle

using namespace souffle;

extern "C" int souffle_bert_embed(const int32_t *token_ids, const int32_t *segment_ids, const void *word_emb, int vocab_size,
                                  const void *pos_emb, int max_positions, const void *type_emb, int type_vocab_size,
                                  const void *ln_g, const void *ln_b, float ln_eps, int batch, int seq_len, int hidden,
                                  void *out, uint32_t *bad_ids, souffle_stream_t stream) {
  if (!token_ids || !word_emb || !pos_emb || !out) return fail(SOUFFLE_ERR_NULL, "token_ids, word_emb, pos_emb and out must not be NULL");
  if (hidden != bert_io::H) return fail(SOUFFLE_ERR_SHAPE, "only hidden=768 is built (got %d)", hidden);
  if (batch <= 0 || seq_len <= 0 || (long long)batch * seq_len > (1 << 24)) return fail(SOUFFLE_ERR_SHAPE, "batch and seq_len must be positive");
  if (!(ln_eps >= 0.f)) return fail(SOUFFLE_ERR_SHAPE, "ln_eps must be >= 0");
  if (vocab_size <= 0) return fail(SOUFFLE_ERR_SHAPE, "vocab_size (rows of word_emb) must be positive (got %d)", vocab_size);
  if (max_positions < seq_len) return fail(SOUFFLE_ERR_SHAPE, "pos_emb has %d rows, the sequence length is %d", max_positions, seq_len);
  if (type_emb && type_vocab_size <= 0) return fail(SOUFFLE_ERR_SHAPE, "type_vocab_size (rows of type_emb) must be positive (got %d)", type_vocab_size);
  if (reinterpret_cast<uintptr_t>(bad_ids) & 3u) return fail(SOUFFLE_ERR_ALIGN, "bad_ids must be 4-byte aligned");
  const void *ptrs[6] = {word_emb, pos_emb, type_emb, ln_g, ln_b, out};
  for (const void *q : ptrs)
    if (!aligned16(q)) return fail(SOUFFLE_ERR_ALIGN, "embedding tables, LN vectors and out must be 16-byte aligned");
  const int rows = batch * seq_len;
  hipLaunchKernelGGL(bert_io::k_embed, dim3((rows + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream), token_ids, segment_ids,
                     static_cast<const half_t *>(word_emb), vocab_size, static_cast<const half_t *>(pos_emb),
                     static_cast<const half_t *>(type_emb), type_vocab_size, static_cast<const half_t *>(ln_g),
                     static_cast<const half_t *>(ln_b), ln_eps, rows, seq_len, static_cast<half_t *>(out), bad_ids);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

extern "C" int souffle_bert_pooler(const void *x, const void *w, const void *bias, int batch, int seq_len, int hidden, void *out,
                                   souffle_stream_t stream) {
  if (!x || !w || !out) return fail(SOUFFLE_ERR_NULL, "x, w and out must not be NULL");
  if (hidden != bert_io::H) return fail(SOUFFLE_ERR_SHAPE, "only hidden=768 is built (got %d)", hidden);
  if (batch <= 0 || batch > 65535 || seq_len <= 0) return fail(SOUFFLE_ERR_SHAPE, "batch must be in 1..65535 and seq_len positive");
  if (!aligned16(x) || !aligned16(w) || !aligned16(bias) || !aligned16(out)) return fail(SOUFFLE_ERR_ALIGN, "x, w, bias and out must be 16-byte aligned");
  hipLaunchKernelGGL(bert_io::k_pooler, dim3(bert_io::H / 64, batch), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const half_t *>(x), static_cast<const half_t *>(w), static_cast<const half_t *>(bias), seq_len,
                     static_cast<half_t *>(out));
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}
