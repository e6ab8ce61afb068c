// BERT-base encoder layer(s) on gfx950: one persistent launch for all stages of all layers, and the same
// stages as separate launches (the unfused per-op baseline).  Two paths:
//   few rows (batch * seq_len <= 1024, and up to 1408 where it is no multiple of 256: many_rows()): bert_small.hpp (flag hand-overs between the producers and consumers of a tile);
//   many rows: this file (256-row or 128 x 128 GEMM tiles, hand-overs per 256-row block or grid barriers).
//
// Stage list per layer (reference counterparts in brackets):
//   1 QKV GEMM + bias + head split        [cpp/bert/kernels/fused_sqq_bert.cu:2333-2765]
//   2 scores, scale, mask, softmax, P.V   [fused_sqq_bert.cu:2772-3329]  (P never leaves the CU)
//   3 out-projection                      [fused_sqq_bert.cu:3334-3687]
//   4 bias + residual + LN1               [fused_sqq_bert.cu:3690-3782]
//   5 FC1 + bias + activation             [cpp/bert/kernels/fused_sqq_feedforward.cu:38-362]
//   6 FC2, partial sums over K            [fused_sqq_feedforward.cu:368-835]
//   7 reduce + bias + residual + LN2      [fused_sqq_feedforward.cu:368-835]
// Softmax is max-subtracted fp32 and LayerNorm statistics are fp32 with a fixed summation order (no float
// atomics), so results are run-to-run identical.
#include <mutex>
#include <type_traits>
#include "bert_small.hpp"
#include "gemm_tile.hpp"
#include "gemm_big.hpp"
#include "host_util.hpp"

namespace souffle {
namespace bert {

#ifndef SOUFFLE_ROWBLOCK_LOCAL
#define SOUFFLE_ROWBLOCK_LOCAL 1
#endif
constexpr bool kRowblockLocal = SOUFFLE_ROWBLOCK_LOCAL != 0;   // many rows: hand-overs among the 16 tiles of a row block instead of grid barriers

constexpr int kMaxSplitK = 8;


// Per-launch parameters.  The inter-stage buffers (qkv .. yl) are given per layer
// (`layer_stride` bytes apart) so that inside one launch every address is written by exactly
// one stage of one layer and read only afterwards: readers can then use ordinary cached
// loads (an XCD's L2 never holds an older version of a line) and each XCD fetches a line of
// an activation once instead of every workgroup fetching it from memory.
// The many-rows megakernel (82 MB of such buffers per layer at 4096 rows) rotates through
// `layer_sets` sets instead, which stay in the memory-side cache, and restores the property at
// the hand-over (or barrier) that ends a layer: one wave of every workgroup invalidates its L1 and its
// XCD's L2 (an agent-scope acquire fence) after arriving and before it polls, so the invalidation has
// been performed when the poll returns.  In the last stage of a layer nobody reads a buffer that a later
// layer writes before reading, so no line dropped there can come back in an old version; with
// hand-overs per row block the same holds per row block, whose rows only its own workgroups read.
struct Params {
  int B, S, M, act, num_layers, splitk_o, splitk_f;
  int big;             // rows are a multiple of 256 and many: the 256-row GEMM tiles are used
  float scale, eps;
  const half_t *x, *mask;
  half_t *y;
  half_t *qkv, *ctx, *z1, *y1, *h, *yl, *probs;
  float *part;
  unsigned *ctl;
  unsigned *rbflags;   // many-rows megakernel: 16 hand-over words per 256-row block (see rowblock_ln)
  unsigned long long *trace;
  int trace_cap;
  size_t layer_stride;
  int layer_sets;      // layer l uses buffer set l % layer_sets
  int strict;          // souffle_set_strict_fences
};
struct Args : Params {
  LayerW layers[kMaxLayers];
};

__device__ __forceinline__ Params layer_params(const Params &a, int l) {
  Params p = a;
  const size_t off = (size_t)(l % a.layer_sets) * a.layer_stride;
  auto adv = [&](half_t *q) { return uniform_ptr(reinterpret_cast<half_t *>(reinterpret_cast<char *>(q) + off)); };
  p.qkv = adv(a.qkv); p.ctx = adv(a.ctx); p.z1 = adv(a.z1); p.y1 = adv(a.y1); p.h = adv(a.h); p.yl = adv(a.yl);
  p.part = uniform_ptr(reinterpret_cast<float *>(reinterpret_cast<char *>(a.part) + off));
  return p;
}

// ------------------------------------------------------------------ stages ----
// Stands in for a bias the caller did not give, where a test per result would cost more than adding zeros.
__device__ const half_t g_zero_row[F] = {};
__device__ __forceinline__ f4 add_row4(f4 v, const half_t *row, int n) {
  const h4 bb = ldg<h4>(row + n);
  return v + f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
}
__device__ __forceinline__ f4 add_bias4(f4 v, const half_t *bias, int n) {
  if (bias) {
    const h4 bb = ldg<h4>(bias + n);
    v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
  }
  return v;
}

template <bool COH, class Tile>
__device__ __forceinline__ void stage_qkv(half_t *lds, const Params &a, const LayerW &w, const half_t *xin,
                                          int first, int stride) {
  constexpr int BM = Tile::kBM, BN = Tile::kBN, BK = Tile::kBK;
  const int tiles_n = 3 * H / BN, items = (a.M / BM) * tiles_n;
  for (int item = first; item < items; item += stride) {
    const int tm = item / tiles_n, n0 = (item % tiles_n) * BN, j = n0 / H, nn0 = n0 % H;
    auto aload = [&](int m, int k) { return ld16<false>(xin, (m * H + k) * 2); };
    auto epi = [&](int m, int n, f4 v) {
      if (w.b_qkv) {
        const h4 bb = ldg<h4>(w.b_qkv + j * H + n);
        v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      const int b = m / a.S, s = m % a.S, hh = n / HD, d = n % HD;
      st8<COH>(a.qkv, ((((j * a.B + b) * NH + hh) * a.S + s) * HD + d) * 2, pack_h4(v));
    };
    Tile::run(lds, w.w_qkv + (size_t)j * H * H, H, tm * BM, nn0, 0, H / BK, aload, epi);
  }
}

// Y = act(X.W + b), fp16 out (FC1).
template <bool COH, class Tile>
__device__ __forceinline__ void stage_fc1(half_t *lds, const Params &a, const LayerW &w, int first, int stride) {
  constexpr int BM = Tile::kBM, BN = Tile::kBN, BK = Tile::kBK;
  const int tiles_n = F / BN, items = (a.M / BM) * tiles_n;
  for (int item = first; item < items; item += stride) {
    const int tm = item / tiles_n, n0 = (item % tiles_n) * BN;
    auto aload = [&](int m, int k) { return ld16<false>(a.y1, (m * H + k) * 2); };
    auto epi = [&](int m, int n, f4 v) {
      if (w.b_fc1) {
        const h4 bb = ldg<h4>(w.b_fc1 + n);
        v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      if (a.act == SOUFFLE_ACT_RELU) {            // (one test per group of results, not one per result)
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = fmaxf(v[i], 0.f);
      } else if (a.act == SOUFFLE_ACT_GELU_ERF) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = gelu_erf(v[i]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = gelu_tanh(v[i]);
      }
      st8<COH>(a.h, (m * F + n) * 2, pack_h4(v));
    };
    Tile::run(lds, w.w_fc1, F, tm * BM, n0, 0, H / BK, aload, epi);
  }
}

// fp32 split-K partials of X[M][K].W[K][H]: part[ks][m][n].
template <bool COH, class Tile>
__device__ __forceinline__ void stage_partial(half_t *lds, const Params &a, const half_t *X, int K,
                                              const half_t *W, int splitk, int first, int stride) {
  constexpr int BM = Tile::kBM, BN = Tile::kBN, BK = Tile::kBK;
  const int tiles_n = H / BN, items = (a.M / BM) * tiles_n * splitk, kper = K / splitk;
  for (int item = first; item < items; item += stride) {
    const int ks = item % splitk, t = item / splitk, tm = t / tiles_n, n0 = (t % tiles_n) * BN;
    auto aload = [&](int m, int k) { return ld16<false>(X, (m * K + k) * 2); };
    auto epi = [&](int m, int n, f4 v) {
      st16<COH>(a.part, ((ks * a.M + m) * H + n) * 4, __builtin_bit_cast(u4, v));
    };
    Tile::run(lds, W, H, tm * BM, n0, ks * kper, kper / BK, aload, epi);
  }
}

// out[m] = LN(sum_ks part[ks][m] + bias + resid[m]) * g + b; one wave per row.
template <bool COH, int SPLITK>
__device__ __forceinline__ void stage_ln_t(const Params &a, const half_t *bias, const half_t *resid,
                                         const half_t *gam, const half_t *bet, half_t *out,
                                         int first_row, int row_stride) {
  const int lane = threadIdx.x & 63;
  for (int m = first_row; m < a.M; m += row_stride) {
    f4 v[3];
    u4 raw[3][SPLITK];
    u2 rres[3];
    // every load of the row is issued before the first use
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
#pragma unroll
      for (int ks = 0; ks < SPLITK; ++ks) raw[c][ks] = ld16<COH>(a.part, ((ks * a.M + m) * H + n) * 4);
      rres[c] = ld8<COH>(resid, (m * H + n) * 2);
    }
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
      f4 s = __builtin_bit_cast(f4, raw[c][0]);
#pragma unroll
      for (int ks = 1; ks < SPLITK; ++ks) s += __builtin_bit_cast(f4, raw[c][ks]);
      const h4 r = as_h4(rres[c]);
      s += f4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
      if (bias) {
        const h4 bb = ldg<h4>(bias + n);
        s += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      v[c] = s;
    }
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c) sum += v[c][0] + v[c][1] + v[c][2] + v[c][3];
    const float mean = wave_sum(sum) * (1.0f / H);
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) { const float d = v[c][i] - mean; sq += d * d; }
    const float rstd = rsqrtf(wave_sum(sq) * (1.0f / H) + a.eps);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
      f4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (v[c][i] - mean) * rstd;
      if (gam) {
        const h4 gg = ldg<h4>(gam + n);
        o *= f4{(float)gg[0], (float)gg[1], (float)gg[2], (float)gg[3]};
      }
      if (bet) {
        const h4 bb = ldg<h4>(bet + n);
        o += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      st8<COH>(out, (m * H + n) * 2, pack_h4(o));
    }
  }
}

// ---- many rows (M a multiple of 256): 256 x BN tiles, see gemm_big.hpp ----
// BN is chosen per GEMM so that M = 4096 gives exactly 256 tiles, one per CU: 144 for the
// 2304 QKV columns, 192 for FC1's 3072, 128-row tiles of 96 columns for the 768 of the out-projection; FC2 (K = 3072)
// uses 96 columns and two halves of K, which asks the L2 for 0.6x the operand bytes of 48-column
// tiles over the whole K (a CU takes in operands no faster than it multiplies them): 41 -> 31 us.
// (The same split for the out-projection, K = 768, gains nothing: its tiles are too short.)
// (a ring of four stages: three in flight at the start of a tile cost 1.7 us to queue, four 2.3 us, and the
// loop is no slower: 12 layers at M = 4096 1378 -> 1368 us fused, 1443 -> 1404 us as separate launches)
constexpr int kBigRing = 4;
using BigQkv = GemmBig<144, kBigRing>;
using BigFc1 = GemmBig<192, kBigRing>;
using BigOut = GemmBig<96, kBigRing, 128>;   // (128 x 96: 0.74x the operand bytes of 256 x 48 from the L2)
// FC2: parts of K, each a partial sum of its own.  16 tiles per row block: 4 column tiles of 192 x 4 parts of K
// (the operand reuse of the FC1 tile; 8 column tiles of 96 x 2 parts writes and reads back half the partial
// sums but runs its K loop at a worse ratio of operand bytes to MFMAs: 1434 us against 1417 for the 12
// layers at M = 4096 in the fused kernel, 1430 against 1441 as separate launches).
#ifndef SOUFFLE_FC2_SPLIT
#define SOUFFLE_FC2_SPLIT 4
#endif
constexpr int kFc2Split = SOUFFLE_FC2_SPLIT;
using BigFc2 = GemmBig<H * kFc2Split / 16, kBigRing>;
constexpr int kBigLds = BigFc1::LDS_BYTES;
static_assert(BigQkv::LDS_BYTES <= kBigLds && BigOut::LDS_BYTES <= kBigLds && BigFc2::LDS_BYTES <= kBigLds, "FC1 has the largest ring");

// Workgroup b runs on XCD b % 8.  With a multiple of 8 row tiles an XCD gets an eighth of them and all column
// tiles; otherwise a quarter of the row tiles and half of the column tiles, so that its L2 fetches each operand
// tile it needs once.
__device__ __forceinline__ void big_tile(int it, int m_tiles, int n_tiles, int *tm, int *tn) {
  if ((gridDim.x & 7) == 0 && (m_tiles & 7) == 0) {
    // every tile of a row block on one XCD: what the block's 16 workgroups hand over to each other stays in that
    // XCD's L2 (each XCD then streams all of W instead of half; 12 layers at 4096 rows: 1288 -> 1276 us)
    const int x = it & 7, i = it >> 3, mo = m_tiles >> 3;
    *tm = x * mo + i % mo;
    *tn = i / mo;
  } else
  if ((gridDim.x & 7) == 0 && (m_tiles & 3) == 0 && (n_tiles & 1) == 0) {
    const int x = it & 7, i = it >> 3, mq = m_tiles >> 2;
    *tm = (x & 3) * mq + i % mq;
    *tn = (x >> 2) * (n_tiles >> 1) + i / mq;
  } else {
    *tm = it / n_tiles;
    *tn = it % n_tiles;
  }
}

template <bool COH>
__device__ __forceinline__ void big_qkv(unsigned char *lds, const Params &a, const LayerW &w, const half_t *xin, int first, int stride, const GridBarrier *tb = nullptr) {
  const int m_tiles = a.M / 256, n_tiles = 3 * H / BigQkv::kBN;
  for (int it = first; it < m_tiles * n_tiles; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, n_tiles, &tm, &tn);
    const int n0 = tn * BigQkv::kBN;
    // the three [768][768] matrices are addressed as one [768][2304]
    auto wptr = [&](int k, int col) {
      const int c = n0 + col, j = c / H;
      return w.w_qkv + ((size_t)j * H + k) * H + (c - j * H);
    };
    const half_t *bq = w.b_qkv ? w.b_qkv : g_zero_row;
    const int bq_stride = w.b_qkv ? H : 0;
    auto bias_at = [&](int nr) {
      const int c = n0 + nr, j = c / H, n = c - j * H;
      return ldg<h4>(bq + j * bq_stride + n);
    };
    auto cvt = [&](int, int, f4 v, h4 bb) { return pack_h4(v + f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]}); };
    // (batch and position of a row without a division per store: the tile's first row is divided once, a row of the
    // tile lies at most 256 + S - 1 positions behind the start of that row's sequence)
    const int b0 = (tm * 256) / a.S, s0 = tm * 256 - b0 * a.S;
    auto store16 = [&](int m, int nr, u4 v) {                // 8 columns never straddle a head (64 columns)
      const int c = n0 + nr, j = c / H, n = c - j * H;
      const int rr = m - tm * 256 + s0, kb = sk::idiv_small(rr, a.S);
      const int b = b0 + kb, s = rr - kb * a.S, hh = n / HD, d = n % HD;
      st16<COH>(a.qkv, ((((j * a.B + b) * NH + hh) * a.S + s) * HD + d) * 2, v);
    };
    f4 acc[BigQkv::MI][BigQkv::NT];
    BigQkv::mainloop<H / 32>(lds, xin, H, tm * 256, 0, wptr, acc, tb);
    BigQkv::epilogue_rowvec(lds, tm * 256, acc, bias_at, cvt, store16, tb);
  }
}
template <bool COH>
__device__ __forceinline__ void big_fc1(unsigned char *lds, const Params &a, const LayerW &w, int first, int stride, const GridBarrier *tb = nullptr) {
  const int m_tiles = a.M / 256, n_tiles = F / BigFc1::kBN;
  for (int it = first; it < m_tiles * n_tiles; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, n_tiles, &tm, &tn);
    const int n0 = tn * BigFc1::kBN;
    auto wptr = [&](int k, int col) { return w.w_fc1 + (size_t)k * F + n0 + col; };
    const half_t *b1 = w.b_fc1 ? w.b_fc1 : g_zero_row;
    auto bias_at = [&](int nr) { return ldg<h4>(b1 + n0 + nr); };
    auto cvt_relu = [&](int, int, f4 v, h4 bb) {
      v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = fmaxf(v[i], 0.f);
      return pack_h4(v);
    };
    auto cvt_gelu = [&](int, int, f4 v, h4 bb) {
      v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = gelu_tanh(v[i]);
      return pack_h4(v);
    };
    auto cvt_erf = [&](int, int, f4 v, h4 bb) {
      v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = gelu_erf(v[i]);
      return pack_h4(v);
    };
    auto store16 = [&](int m, int nr, u4 v) { st16<COH>(a.h, (m * F + n0 + nr) * 2, v); };
    f4 acc[BigFc1::MI][BigFc1::NT];
    BigFc1::mainloop<H / 32>(lds, a.y1, H, tm * 256, 0, wptr, acc, tb);
    if (a.act == SOUFFLE_ACT_RELU) BigFc1::epilogue_rowvec(lds, tm * 256, acc, bias_at, cvt_relu, store16, tb);
    else if (a.act == SOUFFLE_ACT_GELU_ERF) BigFc1::epilogue_rowvec(lds, tm * 256, acc, bias_at, cvt_erf, store16, tb);
    else BigFc1::epilogue_rowvec(lds, tm * 256, acc, bias_at, cvt_gelu, store16, tb);
  }
}
// z = X[M][K].W[K][768] + bias, fp16, into a.z1 (the out-projection; no split of K: 256 tiles already
// fill the device).  The residual is added by the LayerNorm that follows, which reads whole rows: read
// here, 8 bytes per lane across 16 rows per instruction, it cost a tile 5 us.
template <bool COH>
__device__ __forceinline__ void big_presum(unsigned char *lds, const Params &a, const half_t *X, int K, const half_t *W,
                                           const half_t *bias, int first, int stride) {
  // 16 tiles per 256-row block as in the other stages, dealt to the same workgroups: tile tn of row
  // block tm is rows [128 (tn & 1), +128) of the block and column tile tn >> 1.
  const int m_tiles = a.M / 256;
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, 16, &tm, &tn);
    const int n0 = (tn >> 1) * BigOut::kBN, m0 = tm * 256 + (tn & 1) * BigOut::kBM;
    auto wptr = [&](int k, int col) { return W + (size_t)k * H + n0 + col; };
    const half_t *bz = bias ? bias : g_zero_row;
    auto bias_at = [&](int nr) { return ldg<h4>(bz + n0 + nr); };
    auto cvt = [&](int, int, f4 v, h4 bb) { return pack_h4(v + f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]}); };
    auto store16 = [&](int m, int nr, u4 v) { st16<COH>(a.z1, (m * H + n0 + nr) * 2, v); };
    f4 acc[BigOut::MI][BigOut::NT];
    BigOut::mainloop<H / 32>(lds, X, H, m0, 0, wptr, acc);      // (K = H: the out-projection)
    BigOut::epilogue_rowvec(lds, m0, acc, bias_at, cvt, store16);
  }
}
// A pre-LayerNorm sum in kFc2Split parts of K: part 0 = X[:, part 0].W[part 0] + bias, part
// p = X[:, part p].W[part p], all fp16, M x H each, one after the other in the (here otherwise
// unused) partials area (not in z1, which the out-projection of the same layer has written); the
// LayerNorm adds them in order, then the residual.
__device__ __forceinline__ half_t *fc2_sums(const Params &a) { return reinterpret_cast<half_t *>(a.part); }
template <bool COH>
__device__ __forceinline__ void big_presum2(unsigned char *lds, const Params &a, const half_t *X, int K, const half_t *W, int first, int stride) {
  // (the bias is added by the LayerNorm that sums the four parts: a tile that added it took 2.4 us longer than the
  // other three of its column group, and the hand-over behind the stage waits for the slowest)
  const int m_tiles = a.M / 256;
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn2;
    big_tile(it, m_tiles, 16, &tm, &tn2);
    const int ks = tn2 % kFc2Split, n0 = (tn2 / kFc2Split) * BigFc2::kBN, k0 = ks * (K / kFc2Split);
    half_t *zp = fc2_sums(a) + (size_t)ks * a.M * H;
    auto wptr = [&](int k, int col) { return W + (size_t)k * H + n0 + col; };
    auto cvt = [&](int, int, f4 v) { return pack_h4(v); };
    auto store16 = [&](int m, int nr, u4 v) { st16<COH>(zp, (m * H + n0 + nr) * 2, v); };
    f4 acc[BigFc2::MI][BigFc2::NT];
    BigFc2::mainloop<F / kFc2Split / 32>(lds, X, F, tm * 256, k0, wptr, acc);      // (K = F: FC2)
    BigFc2::epilogue(lds, tm * 256, acc, cvt, store16);
  }
}
// out[m] = LN(z[0][m] + ... + z[NZ-1][m] + resid[m]) * g + b (z[p] = z + p M H; summed in this order);
// one wave per row, two-pass statistics in fp32 registers.
// NR rows (m0, m0 + mstep, ...) per call: their loads are all issued before the first is used.
template <bool COH, int NR, int NZ>
__device__ __forceinline__ void big_ln_rows(const Params &a, const half_t *z, const half_t *resid, const half_t *bias, const half_t *gam, const half_t *bet, half_t *out, int m0, int mstep) {
  const int lane = opaque_thread_id() & 63;
  u2 raw[NR][NZ + 1][3];
#pragma unroll
  for (int r = 0; r < NR; ++r)
#pragma unroll
    for (int p = 0; p < NZ; ++p)
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        const int m = m0 + r * mstep;
        raw[r][p][c] = ld8<false>(z + (size_t)p * a.M * H, (m * H + c * 256 + lane * 4) * 2);
        if (p == 0) raw[r][NZ][c] = ld8<false>(resid, (m * H + c * 256 + lane * 4) * 2);
      }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int m = m0 + r * mstep;
    f4 v[3];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const h4 q = as_h4(raw[r][0][c]);
      v[c] = f4{(float)q[0], (float)q[1], (float)q[2], (float)q[3]};
#pragma unroll
      for (int p = 1; p <= NZ; ++p) {
        const h4 q2 = as_h4(raw[r][p][c]);
        v[c] += f4{(float)q2[0], (float)q2[1], (float)q2[2], (float)q2[3]};
      }
      if (bias) {                                   // (of the GEMM whose partial sums these are: added once per row here, not per tile there)
        const h4 bb = ldg<h4>(bias + c * 256 + lane * 4);
        v[c] += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      sum += v[c][0] + v[c][1] + v[c][2] + v[c][3];
    }
    const float mean = wave_sum(sum) * (1.0f / H);
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) { const float d = v[c][i] - mean; sq += d * d; }
    const float rstd = rsqrtf(wave_sum(sq) * (1.0f / H) + a.eps);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
      f4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (v[c][i] - mean) * rstd;
      if (gam) {
        const h4 gg = ldg<h4>(gam + n);
        o *= f4{(float)gg[0], (float)gg[1], (float)gg[2], (float)gg[3]};
      }
      if (bet) {
        const h4 bb = ldg<h4>(bet + n);
        o += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      st8<COH>(out, (m * H + n) * 2, pack_h4(o));
    }
  }
}
template <bool COH, int NZ>
__device__ __forceinline__ void big_ln(const Params &a, const half_t *z, const half_t *resid, const half_t *bias, const half_t *gam, const half_t *bet, half_t *out, int first_row, int row_stride) {
  for (int m = first_row; m < a.M; m += row_stride) big_ln_rows<COH, 1, NZ>(a, z, resid, bias, gam, bet, out, m, 0);
}

// The LayerNorm that follows a pre-LayerNorm sum, without a grid barrier in between (rowblock_ln).  A 256-row
// block of the sum is produced by 16 tiles (16 column tiles, or 4 column tiles x 4 parts of K).
// After the hand-over among them (rowblock_sync) tile t normalises rows 16t .. 16t+15 of the block,
// four per wave, by the same routine as the separate LayerNorm kernel: identical results.  The
// hand-over words are cleared by the launch itself (one grid barrier follows) and tags grow within a
// launch.
static_assert((256 / BigOut::kBM) * (H / BigOut::kBN) == 16 && kFc2Split * (H / BigFc2::kBN) == 16, "16 tiles per row block");
// Hand-over among the workgroups of a 256-row block: this workgroup's tiles of the stage are written
// (all of them: nobody waits before that, so the waits end whatever the tile-to-workgroup mapping is):
// publish `tag` in the word of each (row block, tile), run mid(), then wait until the 16 words of every
// row block this workgroup has a tile in have reached `tag`.  Bounded like the grid barrier; a wait that
// gave up ends all waiting of the launch.  With `bar.trace` the entry and exit times are stamped like
// those of a grid barrier.
// `group`: row blocks that hand over together (1, or the 2 or 3 that hold whole sequences of 512 or 384).
template <class Mid>
__device__ __forceinline__ void rowblock_sync(const Params &a, GridBarrier &bar, unsigned tag, int first, int stride, int group, Mid mid) {
  const int m_tiles = a.M / 256;
  const bool tr = bar.trace && bar.trace_idx < bar.trace_cap && threadIdx.x == 0;
  if (tr) bar.trace[(size_t)(2 * bar.trace_idx) * bar.nblk + blockIdx.x] = wall_clock64();
  wait_all_memory();                             // this wave's write-through stores are acknowledged
  strict_release(bar.strict);
  __syncthreads();
  if (threadIdx.x == 0)
    for (int it = first; it < m_tiles * 16; it += stride) {
      int tm, tn;
      big_tile(it, m_tiles, 16, &tm, &tn);
      __hip_atomic_store(a.rbflags + tm * 16 + tn, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  mid();
  if (threadIdx.x < 64 && !bar.failed) {
    for (int it = first; it < m_tiles * 16 && !bar.failed; it += stride) {
      int tm, tn;
      big_tile(it, m_tiles, 16, &tm, &tn);
      const int g0 = tm - tm % group;
      for (int spin = 0; spin < kMaxBarrierSpin; ++spin) {
        bool ok = true;
        if (threadIdx.x < 16 * group)
          ok = (int)(__hip_atomic_load(a.rbflags + g0 * 16 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - tag) >= 0;
        if (__all(ok)) break;
        __builtin_amdgcn_s_sleep(1);
        if (spin == kMaxBarrierSpin - 1) {         // gave up: the launch's output is invalid
          bar.failed = true;
          if (threadIdx.x == 0) (void)__hip_atomic_fetch_or(a.ctl + kCtlErrWord, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }
  if (tr) bar.trace[(size_t)(2 * bar.trace_idx + 1) * bar.nblk + blockIdx.x] = wall_clock64();
  bar.trace_idx++;
  __syncthreads();
  strict_acquire(bar.strict);
  compiler_fence();                              // no load of the other tiles' results is scheduled above the poll
}
template <bool COH, int NZ>
__device__ __forceinline__ void rowblock_ln(const Params &a, GridBarrier &bar, unsigned tag, const half_t *z, const half_t *resid, const half_t *bias,
                                            const half_t *gam, const half_t *bet, half_t *out, int first, int stride) {
  const int m_tiles = a.M / 256, wave = threadIdx.x >> 6;
  rowblock_sync(a, bar, tag, first, stride, 1, []() {});
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, 16, &tm, &tn);
    big_ln_rows<COH, 4, NZ>(a, z, resid, bias, gam, bet, out, tm * 256 + tn * 16 + wave * 4, 1);
  }
}

// One (batch, head, 64-query block) per workgroup pass; each wave owns 16 queries.
// Scores are computed transposed (keys x queries) so that the softmax reduction over
// keys is in-lane plus two cross-lane steps, and the probabilities are already in the
// B-operand layout of the 16x16x16 MFMA used for P.V.  V is staged row-major in LDS
// and read through the transposing LDS load.
// Direct global->LDS load of a [rows][64] fp16 tile (128-byte rows = 8 slots of 16 bytes),
// swizzled for its reader: MODE 0 for b128 operand reads of 16 consecutive rows
// (slot ^= (row >> 1) & 7), MODE 1 for the transposing read of 4 consecutive rows (slot ^= row & 2).
// (The LDS has 64 banks and serves that read half a wave, 8 consecutive rows, per cycle: with row & 2 rows r and r+4
// collide, 196608 conflict cycles per attention stage at 4096 rows.  slot ^= row & 6 removes them all and was
// measured no faster in the fused encoder and 1.8 % slower in the per-op chain at 4096 rows: kept as it was.)
template <bool COH, int MODE>
__device__ __forceinline__ void issue_rows64(unsigned char *lds, const half_t *src, int rows) {
  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int inst = wave; inst < rows / 8; inst += 4) {
    const int sl = inst * 64 + lane, r = sl >> 3, c = (sl & 7) ^ (MODE == 0 ? ((r >> 1) & 7) : (r & 2));
    __builtin_amdgcn_global_load_lds((gptr_t)(src + (size_t)r * HD + c * 8), (lptr_t)(lds + inst * 1024), 16, 0, COH ? kAuxSc1 : 0);
  }
}

// The loads of one attention item (K and V of the head, 64 query rows), through inline assembly so
// that the caller decides what to wait for (see load_lds16); every wave issues kAttnLoads<NKT> of them.
template <int NKT>
constexpr int kAttnLoads = 2 * (NKT * 16 / 32) + 2;
template <int MODE>
__device__ __forceinline__ void issue_rows64_nowait(unsigned lds_addr, const half_t *src, int rows) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int inst = wave; inst < rows / 8; inst += 4) {
    const int sl = inst * 64 + lane, r = sl >> 3, c = (sl & 7) ^ (MODE == 0 ? ((r >> 1) & 7) : (r & 2));
    load_lds16(src + (size_t)r * HD + c * 8, lds_addr + inst * 1024);
  }
}
template <int NKT>
__device__ __forceinline__ void attn_issue(unsigned char *lds, const Params &a, int item) {
  constexpr int S = NKT * 16;
  const int qblocks = S / 64;
  const int qb = item % qblocks, bh = item / qblocks;
  const int head_off = bh * S * HD;                              // halves, within one of q/k/v
  const size_t plane = (size_t)a.B * NH * S * HD;
  const unsigned base = lds_address(lds);
  issue_rows64_nowait<0>(base, a.qkv + plane + head_off, S);
  issue_rows64_nowait<1>(base + S * 128, a.qkv + 2 * plane + head_off, S);
  issue_rows64_nowait<0>(base + 2 * S * 128, a.qkv + head_off + (size_t)qb * 64 * HD, 64);
}
template <int NKT>
constexpr int kAttnItemLds = 2 * NKT * 16 * 128 + 64 * 128;

// PLAIN: no mask and no probabilities to write (tested once per item: a uniform test per key tile
// inside the unrolled loops is not hoisted by the compiler and breaks them into small blocks).
template <bool COH, int NKT, bool PLAIN>
__device__ __forceinline__ void attn_compute_t(unsigned char *lds, const Params &a, int item);
template <bool COH, int NKT>
__device__ __forceinline__ void attn_compute(unsigned char *lds, const Params &a, int item) {
  if (!a.mask && !a.probs) attn_compute_t<COH, NKT, true>(lds, a, item);
  else attn_compute_t<COH, NKT, false>(lds, a, item);
}

template <bool COH, int NKT>
__device__ __forceinline__ void attn_item(half_t *lds_h, const Params &a, int item) {
  unsigned char *lds = reinterpret_cast<unsigned char *>(lds_h);
  __syncthreads();   // LDS reuse
  attn_issue<NKT>(lds, a, item);
  wait_all_memory();
  __syncthreads();
  attn_compute<COH, NKT>(lds, a, item);
}

using TileLarge = GemmTile<128, 128, 64, 2, 2>;
constexpr int kAttnLdsBytes = 2 * 512 * 128 + 64 * 128;
constexpr int kAttnAhead256 = 2 * (2 * 256 * 128 + 64 * 128);   // two items of S = 256 at a time
constexpr int lds_bytes_large() {
  const int t = TileLarge::LDS_BYTES > kBigLds ? TileLarge::LDS_BYTES : kBigLds;
  const int u = t > kAttnLdsBytes ? t : kAttnLdsBytes;
  return u > kAttnAhead256 ? u : kAttnAhead256;
}
constexpr int kMegaLds = lds_bytes_large();

// One work unit after the other with the loads of the next in flight while this one is computed
// (two LDS buffers).  `item_of(it)`: work unit -> item.
template <bool COH, int NKT, class ItemOf>
__device__ __forceinline__ void attn_items_pipelined(unsigned char *lds, const Params &a, int first, int stride, int items, ItemOf item_of) {
  if (first >= items) return;
  __syncthreads();   // LDS reuse
  attn_issue<NKT>(lds, a, item_of(first));
  int cur = 0;
  for (int it = first; it < items; it += stride) {
    if (it + stride < items) {
      attn_issue<NKT>(lds + (cur ^ 1) * kAttnItemLds<NKT>, a, item_of(it + stride));
      wait_vmcnt<kAttnLoads<NKT>>();      // all but the loads just issued (results stored earlier included)
    } else {
      wait_vmcnt<0>();
    }
    __syncthreads();
    attn_compute<COH, NKT>(lds + cur * kAttnItemLds<NKT>, a, item_of(it));
    __syncthreads();   // this buffer is refilled in the next turn
    cur ^= 1;
  }
}

// Three items (base, base + 1, base + 2) with the loads of all three requested at once: an item's operands come from
// the other workgroups of the row block and take some 2 us to arrive, its arithmetic 0.8 us, so that with one item
// requested ahead each item still waited for most of a round trip.  Without mask and probabilities an item's
// arithmetic issues exactly four vector memory instructions per lane (the context stores), which the waits count:
// vector memory instructions of a wave complete in issue order.
template <bool COH, int NKT>
__device__ __forceinline__ void attn_three(unsigned char *lds, const Params &a, int base) {
  constexpr int KL = kAttnLoads<NKT>, ITEM = kAttnItemLds<NKT>, STORES = HD / 16;
  static_assert(3 * ITEM <= kMegaLds && 3 * KL + 2 * STORES < 64, "three buffers; vmcnt is a 6-bit counter");
  __syncthreads();   // LDS reuse
#pragma unroll
  for (int j = 0; j < 3; ++j) attn_issue<NKT>(lds + j * ITEM, a, base + j);
  static_for<0, 3>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    wait_vmcnt<(2 - j) * KL + j * STORES>();
    __syncthreads();
    attn_compute_t<COH, NKT, true>(lds + j * ITEM, a, base + j);
  });
}

template <bool COH, int NKT, bool PLAIN>
__device__ __forceinline__ void attn_compute_t(unsigned char *lds, const Params &a, int item) {
  constexpr int S = NKT * 16;
  unsigned char *ks_ = lds, *vs_ = lds + S * 128, *qs_ = lds + 2 * S * 128;
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const int qblocks = S / 64;
  const int qb = item % qblocks, bh = item / qblocks, b = bh / NH, hh = bh % NH;

  const half_t *kh = reinterpret_cast<const half_t *>(ks_), *vh = reinterpret_cast<const half_t *>(vs_),
               *qh = reinterpret_cast<const half_t *>(qs_);
  const int q0 = qb * 64 + wave * 16, q = q0 + l16;
  h8 qop[2];
  {
    const int r = wave * 16 + l16;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) qop[ks] = *reinterpret_cast<const h8 *>(qh + (r * 8 + ((ks * 4 + g) ^ ((r >> 1) & 7))) * 8);
  }
  f4 sc[NKT];
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    const int r = t * 16 + l16, sw = (r >> 1) & 7;
    const h8 k0 = *reinterpret_cast<const h8 *>(kh + (r * 8 + (g ^ sw)) * 8);
    const h8 k1 = *reinterpret_cast<const h8 *>(kh + (r * 8 + ((4 + g) ^ sw)) * 8);
    f4 c = mfma_16x16x32(k0, qop[0], f4{0.f, 0.f, 0.f, 0.f});
    sc[t] = mfma_16x16x32(k1, qop[1], c);
  }
  // sc[t][v] = score(key = 16t + 4g + v, query = q0 + l16)
  // softmax in base 2: exp(s - max) = exp2(s log2(e) - max'), log2(e) folded into the scale
  constexpr float kLog2e = 1.4426950408889634f;
  const float scale2 = a.scale * kLog2e;
  float mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    f4 sv = sc[t] * scale2;
    if constexpr (!PLAIN) {
      if (a.mask) {
        const h4 mk = ldg<h4>(a.mask + ((size_t)b * S + q) * S + t * 16 + g * 4);
        sv += f4{(float)mk[0], (float)mk[1], (float)mk[2], (float)mk[3]} * kLog2e;
      }
    }
    sc[t] = sv;
    mx = fmaxf(mx, fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));
  }
  mx = fmaxf(mx, wave_xor(mx, 16));
  mx = fmaxf(mx, wave_xor(mx, 32));
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { sc[t][i] = __builtin_amdgcn_exp2f(sc[t][i] - mx); sum += sc[t][i]; }
  }
  sum += wave_xor(sum, 16);
  sum += wave_xor(sum, 32);
  const float inv = __builtin_amdgcn_rcpf(sum);
  h4 p[NKT];
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    const f4 pr = sc[t] * inv;
    p[t] = h4{(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};
    if constexpr (!PLAIN) {
      if (a.probs)
        st8<false>(a.probs, (int)((((size_t)(b * NH + hh) * S + q) * S + t * 16 + g * 4) * 2), as_u2(p[t]));
    }
  }
  f4 o[HD / 16];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    const int kr = t * 16 + g * 4 + (l16 >> 2);
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      const int c = dt * 2 + ((l16 & 3) >> 1);
      const h4 vop = lds_read_tr16(vh + (kr * 8 + (c ^ (kr & 2))) * 8 + (l16 & 1) * 4);
      o[dt] = mfma_16x16x16(vop, p[t], o[dt]);
    }
  }
  // o[dt][v] = ctx(query q, d = 16dt + 4g + v)
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt)
    st8<COH>(a.ctx, ((b * S + q) * H + hh * HD + dt * 16 + g * 4) * 2, pack_h4(o[dt]));
}

// Work unit `it` (units it, it + 8, ... run on one XCD: workgroup b runs on XCD b % 8) -> attention
// item.  The S / 64 query blocks of a head go to the same XCD, next to each other in time, so that
// its L2 fetches the head's K and V once (at S = 128, B = 32: 19 MB instead of 30 MB per layer).
__device__ __forceinline__ int attn_item_of(int it, int qblocks, int items) {
  if ((gridDim.x & 7) != 0 || items % (8 * qblocks) != 0) return it;
  const int x = it & 7, i = it >> 3;
  return ((i / qblocks) * 8 + x) * qblocks + i % qblocks;
}
template <bool COH, int NKT>
__device__ __forceinline__ void stage_attn_t(half_t *lds, const Params &a, int first, int stride) {
  const int items = a.B * NH * (a.S / 64);
  if constexpr (2 * kAttnItemLds<NKT> <= kMegaLds)    // (the megakernel's LDS allocation)
    attn_items_pipelined<COH, NKT>(reinterpret_cast<unsigned char *>(lds), a, first, stride, items,
                                   [&](int it) { return attn_item_of(it, a.S / 64, items); });
  else
    for (int it = first; it < items; it += stride) attn_item<COH, NKT>(lds, a, attn_item_of(it, a.S / 64, items));
}
// The attention items of the sequences of a group of 256-row blocks that holds whole sequences (48 items
// per row block whatever S is), three to each of the group's tiles, for the tiles of this workgroup.
template <bool COH, int NKT>
__device__ __forceinline__ void stage_attn_rowblock(unsigned char *lds, const Params &a, int first, int stride) {
  const int m_tiles = a.M / 256;
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, 16, &tm, &tn);
    const int base = tm * 48 + tn * 3;           // (the tiles of a group are numbered through: 16 tm + tn)
    if constexpr (3 * kAttnItemLds<NKT> <= kMegaLds) {
      if (!a.mask && !a.probs) { attn_three<COH, NKT>(lds, a, base); continue; }
    }
    if constexpr (2 * kAttnItemLds<NKT> <= kMegaLds)
      attn_items_pipelined<COH, NKT>(lds, a, 0, 1, 3, [&](int j) { return base + j; });
    else
      for (int j = 0; j < 3; ++j) attn_item<COH, NKT>(reinterpret_cast<half_t *>(lds), a, base + j);
  }
}
template <bool COH>
__device__ __forceinline__ void stage_attn(half_t *lds, const Params &a, int first, int stride) {
  const int items = a.B * NH * (a.S / 64);
  for (int it = first; it < items; it += stride) {
    const int item = attn_item_of(it, a.S / 64, items);
    switch (a.S) {
      case 64: attn_item<COH, 4>(lds, a, item); break;
      case 128: attn_item<COH, 8>(lds, a, item); break;
      case 256: attn_item<COH, 16>(lds, a, item); break;
      case 384: attn_item<COH, 24>(lds, a, item); break;
      default: attn_item<COH, 32>(lds, a, item); break;   // 512 (validated on the host)
    }
  }
}

constexpr int lds_bytes_small() { return sk::kLdsBytes > sk::attn_lds_bytes(512) ? sk::kLdsBytes : sk::attn_lds_bytes(512); }
static_assert(lds_bytes_small() <= 160 * 1024, "LDS of a CU");

// (the many-rows paths write every pre-LayerNorm sum once: no split of K)
template <bool COH>
__device__ __forceinline__ void stage_ln(const Params &a, const half_t *bias, const half_t *resid, const half_t *gam,
                                         const half_t *bet, half_t *out, int first_row, int row_stride) {
  stage_ln_t<COH, 1>(a, bias, resid, gam, bet, out, first_row, row_stride);
}

// ------------------------------------------------------------ megakernel ----
// Many rows (many_rows(M)).  MODE 1: 128 x 128 tiles; 2: 256-row tiles (M a multiple of 256)
template <int MODE, int NKT>
__global__ void __launch_bounds__(256) k_encoder_mega(Args args) {
  static_assert(MODE == 1 || MODE == 2, "the few-rows path is k_encoder_small");
  constexpr bool BIG = MODE == 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  half_t *lds = reinterpret_cast<half_t *>(lds_raw);
  using Tile = TileLarge;
  GridBarrier bar;
  grid_barrier_begin(bar, args.ctl, args.strict != 0);
  bar.trace = args.trace;
  bar.trace_cap = args.trace_cap;
  const int first = blockIdx.x, stride = gridDim.x;
  const int wave = threadIdx.x >> 6;
  const half_t *xin = args.x;
  if constexpr (BIG) {   // the row-block hand-over words start every launch at 0
    for (int i = first * 256 + threadIdx.x; i < (args.M / 256) * 16; i += stride * 256)
      __hip_atomic_store(args.rbflags + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    grid_sync(bar);
  }
  for (int l = 0; l < args.num_layers; ++l) {
    const LayerW w = args.layers[l];
    const Params a = layer_params(args, l);
    half_t *yout = (l == a.num_layers - 1) ? a.y : a.yl;
    if constexpr (BIG) {
      // Where a 256-row block (S = 64, 128, 256) or a group of 2 (S = 512) or 3 (S = 384) of them holds
      // whole sequences, every stage of a group's tiles reads only what the tiles of the same group
      // wrote in the stage before (attention included: the 48 items per row block go three to a tile),
      // and the tile-to-workgroup mapping is the same in every stage: the 16 row blocks of M = 4096 then
      // run as independent groups of 16 workgroups that hand over among themselves (rowblock_sync).
      // Otherwise (a number of row blocks that is no multiple of the group) the stages are separated by
      // grid barriers.  Hand-over k of layer l carries the tag 7 l + k.
      const int group = a.S <= 256 ? 1 : a.S == 512 ? 2 : 3;
      const bool local = kRowblockLocal && (group * 256) % a.S == 0 && (a.M / 256) % group == 0;
      auto sync = [&](unsigned k) {
        if (local) rowblock_sync(a, bar, 7u * l + k, first, stride, group, []() {});
        else grid_sync(bar);
      };
      big_qkv<true>(lds_raw, a, w, xin, first, stride, &bar);
      sync(1);
      if (local) stage_attn_rowblock<true, NKT>(lds_raw, a, first, stride);
      else stage_attn_t<true, NKT>(lds, a, first, stride);
      sync(2);
      big_presum<true>(lds_raw, a, a.ctx, H, w.w_o, w.b_o, first, stride);
      rowblock_ln<true, 1>(a, bar, 7u * l + 3u, a.z1, xin, nullptr, w.ln1_g, w.ln1_b, a.y1, first, stride);
      sync(4);
      big_fc1<true>(lds_raw, a, w, first, stride, &bar);
      sync(5);
      big_presum2<true>(lds_raw, a, a.h, F, w.w_fc2, first, stride);
      rowblock_ln<true, kFc2Split>(a, bar, 7u * l + 6u, fc2_sums(a), a.y1, w.b_fc2, w.ln2_g, w.ln2_b, yout, first, stride);
      if (l + 1 < a.num_layers) {   // the next layer writes this layer's buffers again: see Params
        auto invalidate = [&]() { if (threadIdx.x < 64) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); };
        if (local) rowblock_sync(a, bar, 7u * l + 7u, first, stride, group, invalidate);
        else grid_sync(bar, invalidate);
      }
    } else {
      stage_qkv<true, Tile>(lds, a, w, xin, first, stride);
      grid_sync(bar);
      stage_attn_t<true, NKT>(lds, a, first, stride);
      grid_sync(bar);
      stage_partial<true, Tile>(lds, a, a.ctx, H, w.w_o, a.splitk_o, first, stride);
      grid_sync(bar);
      stage_ln<true>(a, w.b_o, xin, w.ln1_g, w.ln1_b, a.y1, first * 4 + wave, stride * 4);
      grid_sync(bar);
      stage_fc1<true, Tile>(lds, a, w, first, stride);
      grid_sync(bar);
      stage_partial<true, Tile>(lds, a, a.h, F, w.w_fc2, a.splitk_f, first, stride);
      grid_sync(bar);
      stage_ln<true>(a, w.b_fc2, a.y1, w.ln2_g, w.ln2_b, yout, first * 4 + wave, stride * 4);
    }
    if constexpr (!BIG) {
      if (l + 1 < a.num_layers) grid_sync(bar);
    }
    xin = yout;
  }
  grid_barrier_end(bar);
}

// ------------------------------------------------------ per-op kernels ----
// (many rows; the per-op kernels of the few-rows path are sk::k_small_phase)
template <int MODE>
__global__ void __launch_bounds__(256) k_qkv(Args a, int l, const half_t *xin) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  if constexpr (MODE == 2) big_qkv<false>(lds_raw, a, a.layers[l], xin, blockIdx.x, gridDim.x);
  else stage_qkv<false, TileLarge>(reinterpret_cast<half_t *>(lds_raw), a, a.layers[l], xin, blockIdx.x, gridDim.x);
}
__global__ void __launch_bounds__(256) k_attn(Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  stage_attn<false>(reinterpret_cast<half_t *>(lds_raw), a, blockIdx.x, gridDim.x);
}
__global__ void __launch_bounds__(256) k_partial(Args a, const half_t *X, int K, const half_t *W, int splitk) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  stage_partial<false, TileLarge>(reinterpret_cast<half_t *>(lds_raw), a, X, K, W, splitk, blockIdx.x, gridDim.x);
}
__global__ void __launch_bounds__(256) k_ln(Args a, const half_t *bias, const half_t *resid,
                                            const half_t *gam, const half_t *bet, half_t *out) {
  stage_ln<false>(a, bias, resid, gam, bet, out, blockIdx.x * 4 + (threadIdx.x >> 6), gridDim.x * 4);
}
__global__ void __launch_bounds__(256) k_presum_big(Args a, const half_t *X, int K, const half_t *W, const half_t *bias) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  big_presum<false>(lds_raw, a, X, K, W, bias, blockIdx.x, gridDim.x);
}
__global__ void __launch_bounds__(256) k_presum2_big(Args a, const half_t *X, int K, const half_t *W) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  big_presum2<false>(lds_raw, a, X, K, W, blockIdx.x, gridDim.x);
}
template <int NZ>
__global__ void __launch_bounds__(256) k_ln_big(Args a, const half_t *z, const half_t *resid, const half_t *bias, const half_t *gam, const half_t *bet, half_t *out) {
  big_ln<false, NZ>(a, z, resid, bias, gam, bet, out, blockIdx.x * 4 + (threadIdx.x >> 6), gridDim.x * 4);
}
template <int MODE>
__global__ void __launch_bounds__(256) k_fc1(Args a, int l) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  if constexpr (MODE == 2) big_fc1<false>(lds_raw, a, a.layers[l], blockIdx.x, gridDim.x);
  else stage_fc1<false, TileLarge>(reinterpret_cast<half_t *>(lds_raw), a, a.layers[l], blockIdx.x, gridDim.x);
}

// ---- sequence lengths that are not built: rows copied into / out of a padded layout ----
// xp[b][s][:] = s < S ? x[b][s][:] : 0, 16 bytes per thread.
__global__ void __launch_bounds__(256) k_pad_rows(const half_t *x, half_t *xp, int B, int S, int SP) {
  const int n = B * SP * (H / 8);
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const int g = i % (H / 8), r = i / (H / 8), b = r / SP, sq = r - b * SP;
    u4 v = {0u, 0u, 0u, 0u};
    if (sq < S) v = *reinterpret_cast<const u4 *>(x + ((size_t)(b * S + sq) * H + g * 8));
    *reinterpret_cast<u4 *>(xp + (size_t)i * 8) = v;
  }
}
// y[b][s][:] = yp[b][s][:] for s < S.
__global__ void __launch_bounds__(256) k_unpad_rows(const half_t *yp, half_t *y, int B, int S, int SP) {
  const int n = B * S * (H / 8);
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const int g = i % (H / 8), r = i / (H / 8), b = r / S, sq = r - b * S;
    *reinterpret_cast<u4 *>(y + (size_t)i * 8) = *reinterpret_cast<const u4 *>(yp + ((size_t)(b * SP + sq) * H + g * 8));
  }
}
// mp[b][q][k] = k >= S ? -10000 : (q < S and mask given ? mask[b][q][k] : 0): exp(-10000 - max) is 0 in
// fp32, so the surplus keys take no part in any softmax.
__global__ void __launch_bounds__(256) k_pad_mask(const half_t *mask, half_t *mp, int B, int S, int SP) {
  const int n = B * SP * SP;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const int k = i % SP, r = i / SP, b = r / SP, q = r - b * SP;
    half_t v = (half_t)0.0f;
    if (k >= S) v = (half_t)-10000.0f;
    else if (mask && q < S) v = mask[((size_t)b * S + q) * S + k];
    mp[i] = v;
  }
}

// ------------------------------------------------------------------- host ----
constexpr int kBigSets = 1;     // buffer sets the many-rows megakernel rotates through (1: 1604 us at 4096 rows, 2: 1777, 3: 1787, one per layer: 1808)
struct Plan {
  bool large, big;
  size_t off_ctl, off_flags, off_qkv, off_ctx, off_z1, off_y1, off_h, off_yl, off_part, layer_stride, total;
  size_t off_st1, off_st2, off_z2;        // few rows: row statistics of the pre-LayerNorm sums, the second sum
  int layer_sets;
  size_t off_xpad, off_ypad, off_maskpad;
  size_t off_rbflags;     // 16 words per 256-row block (many-rows megakernel only)
};

// The attention tiles are built for these sequence lengths; any other length up to 512 runs as the
// next one of them with the surplus key positions masked out (rows copied in and out, see run_padded).
static int padded_len(int s) { return s <= 64 ? 64 : s <= 128 ? 128 : s <= 256 ? 256 : s <= 384 ? 384 : 512; }

static int validate(const souffle_bert_cfg *c) {
  if (!c) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  if (c->hidden != H || c->heads != NH || c->ffn != F)
    return fail(SOUFFLE_ERR_SHAPE, "only hidden=768 heads=12 ffn=3072 is built (got %d/%d/%d)", c->hidden, c->heads, c->ffn);
  if (c->batch <= 0 || c->seq_len <= 0) return fail(SOUFFLE_ERR_SHAPE, "batch and seq_len must be positive");
  if (c->seq_len > 512) return fail(SOUFFLE_ERR_SHAPE, "seq_len must be at most 512 (got %d)", c->seq_len);
  const int s = padded_len(c->seq_len);          // other lengths run padded to the next built one
  const long long m = (long long)c->batch * s;
  if (m >= 1536 && m % 128 != 0) return fail(SOUFFLE_ERR_SHAPE, "batch*seq_len >= 1536 must be a multiple of 128 (got %lld)", m);
  if (m > 65536) return fail(SOUFFLE_ERR_SHAPE, "batch*seq_len must be <= 65536 (got %lld)", m);
  if (c->act != SOUFFLE_ACT_GELU_TANH && c->act != SOUFFLE_ACT_RELU && c->act != SOUFFLE_ACT_GELU_ERF) return fail(SOUFFLE_ERR_SHAPE, "unknown activation %d", c->act);
  if (!(c->ln_eps >= 0.f)) return fail(SOUFFLE_ERR_SHAPE, "ln_eps must be >= 0");
  return SOUFFLE_OK;
}

// Which kernel runs a shape.  The few-rows kernel (one weight slice per workgroup and phase, flag hand-overs) is the
// faster one up to 1024 rows (12 layers at 8 x 128: 1042 us against 1209; at 2 x 512: 1101 against 1427) and, where
// the rows are no multiple of 256 and the many-rows kernel has to fall back to its 128 x 128 tiles, up to 1408 rows
// (1152 rows: 1158 against 1436; 1408: 1363 against 1638; at 1280 rows the two are level and at 1536 the 256-row
// tiles win, 1204 against 1451).
static bool many_rows(size_t M) { return M >= 1536 || (M > 1024 && M % 256 == 0); }

static Plan make_plan(const souffle_bert_cfg *c, int num_layers) {
  Plan p{};
  const size_t M = (size_t)c->batch * padded_len(c->seq_len);
  p.large = many_rows(M);
  p.big = p.large && M % 256 == 0;     // (12 layers at M = 1024: 1222 us, with the 128 x 128 tiles 1409 us; at M = 1536: 1225 against 1661)
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += round_up(bytes, 256); return o; };
  p.off_ctl = take(kCtlWords * 4);
  off = round_up(off, 4096);                           // (the 4 KB blocks of the flag copies on 4 KB boundaries of an aligned workspace)
  p.off_flags = take(sk::kFlagRegionWords * 4);        // (at a fixed place, whatever the configuration)
  const size_t first = off;
  p.off_qkv = take(3 * M * H * 2);
  p.off_ctx = take(M * H * 2);
  p.off_z1 = take(M * H * 2);
  p.off_h = take(M * F * 2);
  if (p.large) {
    p.off_y1 = take(M * H * 2);
    // (256-row tiles) FC2's kFc2Split fp16 pre-LayerNorm partial sums, or the fp32 sums of the 128 x 128 tiles
    p.off_part = take(p.big ? (size_t)kFc2Split * M * H * 2 : M * H * 4);
    p.off_yl = take(M * H * 2);
  } else {
    p.off_part = take((size_t)4 * M * H * 4);
    p.off_z2 = take(M * H * 2);
    p.off_st1 = take(M * sk::kNS1 * 8);
    p.off_st2 = take(M * sk::kNS2 * 8);
  }
  p.layer_stride = off - first;                       // one set of inter-stage buffers per layer
  const int nl = num_layers < 1 ? 1 : num_layers;
  p.layer_sets = p.big && nl > kBigSets ? kBigSets : nl;
  p.total = first + p.layer_stride * (size_t)p.layer_sets;
  // (in front of the padding area: the plan of the padded configuration, which lacks that area, must agree)
  p.off_rbflags = 0;
  if (p.big) {
    off = p.total;
    p.off_rbflags = take(M / 256 * 64);
    p.total = off;
  }
  // a sequence length that is not built: padded copies of x and y and the padded additive mask
  p.off_xpad = p.off_ypad = p.off_maskpad = 0;
  if (padded_len(c->seq_len) != c->seq_len) {
    off = p.total;
    p.off_xpad = take(M * H * 2);
    p.off_ypad = take(M * H * 2);
    p.off_maskpad = take(M * (size_t)padded_len(c->seq_len) * 2);
    p.total = off;
  }
  return p;
}

static int check_common(const souffle_bert_layer_w *layers, int nl, const void *x, const void *mask, void *y, void *ws, size_t ws_bytes,
                        const Plan &p) {
  if (!layers || !x || !y) return fail(SOUFFLE_ERR_NULL, "layers, x and y must not be NULL");
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL (need %zu bytes)", p.total);
  if (ws_bytes < p.total) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, p.total);
  if (nl < 1 || nl > kMaxLayers) return fail(SOUFFLE_ERR_SHAPE, "num_layers must be in 1..%d (got %d)", kMaxLayers, nl);
  if (!aligned16(x) || !aligned16(y) || !aligned16(ws) || (mask && !aligned16(mask)))
    return fail(SOUFFLE_ERR_ALIGN, "x, y, mask and workspace must be 16-byte aligned");
  return SOUFFLE_OK;
}
static int fill_layers(LayerW *dst, const souffle_bert_layer_w *layers, int nl) {
  for (int l = 0; l < nl; ++l) {
    const souffle_bert_layer_w &s = layers[l];
    if (!s.w_qkv || !s.w_o || !s.w_fc1 || !s.w_fc2) return fail(SOUFFLE_ERR_NULL, "layer %d: a weight matrix is NULL", l);
    const void *ptrs[12] = {s.w_qkv, s.b_qkv, s.w_o, s.b_o, s.ln1_g, s.ln1_b, s.w_fc1, s.b_fc1, s.w_fc2, s.b_fc2, s.ln2_g, s.ln2_b};
    for (const void *q : ptrs)
      if (!aligned16(q)) return fail(SOUFFLE_ERR_ALIGN, "layer %d: a weight/bias pointer is not 16-byte aligned", l);
    LayerW &d = dst[l];
    d.w_qkv = (const half_t *)s.w_qkv; d.b_qkv = (const half_t *)s.b_qkv; d.w_o = (const half_t *)s.w_o; d.b_o = (const half_t *)s.b_o;
    d.ln1_g = (const half_t *)s.ln1_g; d.ln1_b = (const half_t *)s.ln1_b; d.w_fc1 = (const half_t *)s.w_fc1; d.b_fc1 = (const half_t *)s.b_fc1;
    d.w_fc2 = (const half_t *)s.w_fc2; d.b_fc2 = (const half_t *)s.b_fc2; d.ln2_g = (const half_t *)s.ln2_g; d.ln2_b = (const half_t *)s.ln2_b;
    d.w_fc2p = (const half_t *)s.w_fc2_packed;
    if (!aligned16(s.w_fc2_packed)) return fail(SOUFFLE_ERR_ALIGN, "layer %d: w_fc2_packed is not 16-byte aligned", l);
  }
  return SOUFFLE_OK;
}

static int fill_args(Args &a, const souffle_bert_cfg *c, const souffle_bert_layer_w *layers, int nl,
                     const void *x, const void *mask, void *y, const souffle_bert_dump *dump,
                     void *ws, size_t ws_bytes, const Plan &p) {
  if (int rc = check_common(layers, nl, x, mask, y, ws, ws_bytes, p)) return rc;
  char *base = static_cast<char *>(ws);
  a.B = c->batch; a.S = c->seq_len; a.M = c->batch * c->seq_len; a.act = c->act; a.num_layers = nl;
  a.splitk_o = 1; a.splitk_f = 1; a.scale = c->scale; a.eps = c->ln_eps;
  a.strict = strict_fences_mode();
  a.big = p.big ? 1 : 0;
  a.x = static_cast<const half_t *>(x); a.mask = static_cast<const half_t *>(mask); a.y = static_cast<half_t *>(y);
  a.ctl = reinterpret_cast<unsigned *>(base + p.off_ctl);
  a.rbflags = p.big ? reinterpret_cast<unsigned *>(base + p.off_rbflags) : nullptr;
  a.qkv = reinterpret_cast<half_t *>(base + p.off_qkv);
  a.ctx = reinterpret_cast<half_t *>(base + p.off_ctx);
  a.z1 = reinterpret_cast<half_t *>(base + p.off_z1);
  a.y1 = reinterpret_cast<half_t *>(base + p.off_y1);
  a.h = reinterpret_cast<half_t *>(base + p.off_h);
  a.yl = reinterpret_cast<half_t *>(base + p.off_yl);
  a.layer_stride = p.layer_stride;
  a.layer_sets = p.layer_sets;
  a.part = reinterpret_cast<float *>(base + p.off_part);
  a.probs = nullptr;
  a.trace = nullptr;
  a.trace_cap = 0;
  if (dump) {   // the per-stage tensors are produced in the reference's own layouts: write them in place
    if (dump->qkv) a.qkv = static_cast<half_t *>(dump->qkv);
    if (dump->ctx) a.ctx = static_cast<half_t *>(dump->ctx);
    if (dump->ln1) a.y1 = static_cast<half_t *>(dump->ln1);
    if (dump->fc1) a.h = static_cast<half_t *>(dump->fc1);
    a.probs = static_cast<half_t *>(dump->probs);
    if (!aligned16(a.qkv) || !aligned16(a.ctx) || !aligned16(a.y1) || !aligned16(a.h) || !aligned16(a.probs))
      return fail(SOUFFLE_ERR_ALIGN, "dump pointers must be 16-byte aligned");
  }
  return fill_layers(a.layers, layers, nl);
}
// (few rows)
static int fill_small(sk::Args &a, const souffle_bert_cfg *c, const souffle_bert_layer_w *layers, int nl,
                      const void *x, const void *mask, void *y, const souffle_bert_dump *dump,
                      void *ws, size_t ws_bytes, const Plan &p) {
  if (int rc = check_common(layers, nl, x, mask, y, ws, ws_bytes, p)) return rc;
  char *base = static_cast<char *>(ws);
  a.B = c->batch; a.S = c->seq_len; a.M = c->batch * c->seq_len; a.act = c->act; a.num_layers = nl;
  a.scale = c->scale; a.eps = c->ln_eps;
  a.strict = strict_fences_mode();
  a.x = static_cast<const half_t *>(x); a.mask = static_cast<const half_t *>(mask); a.y = static_cast<half_t *>(y);
  a.ctl = reinterpret_cast<unsigned *>(base + p.off_ctl);
  a.flags = reinterpret_cast<unsigned *>(base + p.off_flags);
  a.qkv = reinterpret_cast<half_t *>(base + p.off_qkv);
  a.ctx = reinterpret_cast<half_t *>(base + p.off_ctx);
  a.z1 = reinterpret_cast<half_t *>(base + p.off_z1);
  a.h = reinterpret_cast<half_t *>(base + p.off_h);
  a.z2 = reinterpret_cast<half_t *>(base + p.off_z2);
  a.st1 = reinterpret_cast<float *>(base + p.off_st1);
  a.st2 = reinterpret_cast<float *>(base + p.off_st2);
  a.part = reinterpret_cast<float *>(base + p.off_part);
  a.layer_stride = p.layer_stride;
  a.probs = nullptr;
  a.ln1_out = nullptr;
  a.fc1_out = nullptr;
  a.trace = nullptr;
  a.trace_cap = 0;
  if (dump) {   // (a single layer: the per-stage tensors are produced in the reference's own layouts, in place)
    if (dump->qkv) a.qkv = static_cast<half_t *>(dump->qkv);
    if (dump->ctx) a.ctx = static_cast<half_t *>(dump->ctx);
    a.fc1_out = static_cast<half_t *>(dump->fc1);      // (moved into a.h below unless h is kept in operand order)
    a.ln1_out = static_cast<half_t *>(dump->ln1);
    a.probs = static_cast<half_t *>(dump->probs);
    if (!aligned16(a.qkv) || !aligned16(a.ctx) || !aligned16(a.ln1_out) || !aligned16(a.fc1_out) || !aligned16(a.probs))
      return fail(SOUFFLE_ERR_ALIGN, "dump pointers must be 16-byte aligned");
  }
  if (int rc = fill_layers(a.layers, layers, nl)) return rc;
  // FC2 runs in its whole-K form when every layer brings the packed copy of its weights (souffle_bert_pack_fc2)
  a.packed = 1;
  for (int l = 0; l < nl; ++l)
    if (!a.layers[l].w_fc2p) a.packed = 0;
  if (!a.packed && a.fc1_out) { a.h = a.fc1_out; a.fc1_out = nullptr; }      // row-major h: written in place
  return SOUFFLE_OK;
}

template <int MODE, int NKT>
static int launch_mega_t(Args &a, int grid, hipStream_t st) {
  const int lds = lds_bytes_large();
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_encoder_mega<MODE, NKT>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    attr_done = true;
  }
  void *args[] = {&a};
  return launch_persistent((const void *)k_encoder_mega<MODE, NKT>, grid, 256, args, lds, st);
}
// one kernel per supported sequence length, so that each carries only its own attention tile
template <int MODE>
static int launch_mega(Args &a, int grid, hipStream_t st) {
  switch (a.S) {
#ifdef SOUFFLE_DEV_ONLY_S128      // development builds: one sequence length, a fifth of the compile time
    case 128: return launch_mega_t<MODE, 8>(a, grid, st);
    default: return fail(SOUFFLE_ERR_SHAPE, "development build: seq_len 128 only");
#else
    case 64: return launch_mega_t<MODE, 4>(a, grid, st);
    case 128: return launch_mega_t<MODE, 8>(a, grid, st);
    case 256: return launch_mega_t<MODE, 16>(a, grid, st);
    case 384: return launch_mega_t<MODE, 24>(a, grid, st);
    default: return launch_mega_t<MODE, 32>(a, grid, st);
#endif
  }
}

template <int NKT, bool MULTI>
static int launch_small_tt(sk::Args &a, int grid, hipStream_t st) {
  const int lds = lds_bytes_small();
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)sk::k_encoder_small<NKT, MULTI>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    attr_done = true;
  }
  void *args[] = {&a};
  return launch_persistent((const void *)sk::k_encoder_small<NKT, MULTI>, grid, 256, args, lds, st);
}
template <int NKT>
static int launch_small_t(sk::Args &a, int grid, hipStream_t st) {
  const sk::Shape sh{a.B, a.S, a.M, a.M / 32, grid, a.packed};
  return sk::single_pass(sh) ? launch_small_tt<NKT, false>(a, grid, st) : launch_small_tt<NKT, true>(a, grid, st);
}
// The few-rows kernels deal weight slices to XCDs by workgroup number modulo 8 and keep one flag word and one row of
// wait masks per workgroup.
static int check_small_grid(int grid) {
  if (grid <= 0 || grid % 8 != 0 || grid > sk::kMaxGrid)
    return fail(SOUFFLE_ERR_DEVICE, "the few-rows encoder needs a grid that is a multiple of 8 in 8..%d workgroups (this device gives %d)", sk::kMaxGrid, grid);
  return SOUFFLE_OK;
}
static int launch_small(sk::Args &a, int grid, hipStream_t st) {
  if (int rc = check_small_grid(grid)) return rc;
  switch (a.S) {
#ifdef SOUFFLE_DEV_ONLY_S128      // development builds: one sequence length, a fifth of the compile time
    case 128: return launch_small_t<8>(a, grid, st);
    default: return fail(SOUFFLE_ERR_SHAPE, "development build: seq_len 128 only");
#else
    case 64: return launch_small_t<4>(a, grid, st);
    case 128: return launch_small_t<8>(a, grid, st);
    case 256: return launch_small_t<16>(a, grid, st);
    case 384: return launch_small_t<24>(a, grid, st);
    default: return launch_small_t<32>(a, grid, st);
#endif
  }
}
// The same phases as separate launches: 6 per layer and one at the end.  Every launch has the grid of the fused
// kernel, so that the items are dealt to the same workgroup numbers and every sum has the same order.
template <int NKT>
static int run_small_unfused_t(sk::Args &a, int grid, hipStream_t st) {
  const int lds = lds_bytes_small();
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)sk::k_small_phase<NKT>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    attr_done = true;
  }
  for (int l = 0; l < a.num_layers; ++l)
    for (int ph = sk::PH_QKV; ph <= sk::PH_FC2; ++ph) {
      const int need = ph == sk::PH_ATT ? sk::attn_lds_bytes(a.S) : sk::kLdsBytes;
      hipLaunchKernelGGL(sk::k_small_phase<NKT>, dim3(grid), dim3(256), need, st, a, l, ph);
    }
  hipLaunchKernelGGL(sk::k_small_phase<NKT>, dim3(grid), dim3(256), 0, st, a, a.num_layers - 1, (int)sk::PH_FIN);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}
static int run_small_unfused(sk::Args &a, int grid, hipStream_t st) {
  if (int rc = check_small_grid(grid)) return rc;
  switch (a.S) {
#ifdef SOUFFLE_DEV_ONLY_S128      // development builds: one sequence length, a fifth of the compile time
    case 128: return run_small_unfused_t<8>(a, grid, st);
    default: return fail(SOUFFLE_ERR_SHAPE, "development build: seq_len 128 only");
#else
    case 64: return run_small_unfused_t<4>(a, grid, st);
    case 128: return run_small_unfused_t<8>(a, grid, st);
    case 256: return run_small_unfused_t<16>(a, grid, st);
    case 384: return run_small_unfused_t<24>(a, grid, st);
    default: return run_small_unfused_t<32>(a, grid, st);
#endif
  }
}

// A sequence length that is not built runs as the next built one: x is copied into a zero-padded
// layout, the additive mask is extended so that the surplus keys drop out of every softmax, and the
// first S rows of every sequence are copied back.  Returns the configuration and pointers the
// kernels see (`before`), and copies the result out (`after`).
struct Padded {
  souffle_bert_cfg cfg;
  const void *x, *mask;
  void *y;
  bool on;
};
static int pad_before(Padded &pd, const souffle_bert_cfg *c, const void *x, const void *mask, void *y, const souffle_bert_dump *dump,
                      void *ws, size_t ws_bytes, const Plan &p, int num_cus, hipStream_t st) {
  pd.cfg = *c; pd.x = x; pd.mask = mask; pd.y = y;
  pd.on = padded_len(c->seq_len) != c->seq_len;
  if (!pd.on) return SOUFFLE_OK;
  if (dump) return fail(SOUFFLE_ERR_SHAPE, "per-stage tensors need seq_len in {64,128,256,384,512} (got %d)", c->seq_len);
  if (!x || !y) return fail(SOUFFLE_ERR_NULL, "layers, x and y must not be NULL");
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL (need %zu bytes)", p.total);
  if (ws_bytes < p.total) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, p.total);
  if (!aligned16(x) || !aligned16(y) || !aligned16(ws))
    return fail(SOUFFLE_ERR_ALIGN, "x, y and workspace must be 16-byte aligned");
  char *base = static_cast<char *>(ws);
  const int SP = padded_len(c->seq_len);
  pd.cfg.seq_len = SP;
  pd.x = base + p.off_xpad; pd.y = base + p.off_ypad; pd.mask = base + p.off_maskpad;
  const int cap = num_cus * 8;
  auto grid_for = [&](long long n) { const long long g = (n + 255) / 256; return (int)(g < cap ? g : cap); };
  hipLaunchKernelGGL(k_pad_rows, dim3(grid_for((long long)c->batch * SP * (H / 8))), dim3(256), 0, st, static_cast<const half_t *>(x),
                     reinterpret_cast<half_t *>(base + p.off_xpad), c->batch, c->seq_len, SP);
  hipLaunchKernelGGL(k_pad_mask, dim3(grid_for((long long)c->batch * SP * SP)), dim3(256), 0, st, static_cast<const half_t *>(mask),
                     reinterpret_cast<half_t *>(base + p.off_maskpad), c->batch, c->seq_len, SP);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}
static int pad_after(const Padded &pd, const souffle_bert_cfg *c, void *y, int num_cus, hipStream_t st) {
  if (!pd.on) return SOUFFLE_OK;
  const long long n = (long long)c->batch * c->seq_len * (H / 8);
  const long long g = (n + 255) / 256;
  hipLaunchKernelGGL(k_unpad_rows, dim3((int)(g < num_cus * 8 ? g : num_cus * 8)), dim3(256), 0, st, static_cast<const half_t *>(pd.y),
                     static_cast<half_t *>(y), c->batch, c->seq_len, pd.cfg.seq_len);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

static int run_fused(const souffle_bert_cfg *c, const souffle_bert_layer_w *layers, int nl, const void *x_in,
                     const void *mask_in, void *y_out, const souffle_bert_dump *dump, void *ws, size_t ws_bytes,
                     souffle_stream_t stream) {
  if (int rc = validate(c)) return rc;
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const Plan p = make_plan(c, nl);      // (cooperative-launch support is asked for by the launch itself, and only in that mode)
  Padded pd;
  if (int rc = pad_before(pd, c, x_in, mask_in, y_out, dump, ws, ws_bytes, p, df.num_cus, static_cast<hipStream_t>(stream))) return rc;
  if (pd.on) {
    const int rc = run_fused(&pd.cfg, layers, nl, pd.x, pd.mask, pd.y, nullptr, ws, ws_bytes, stream);
    return rc ? rc : pad_after(pd, c, y_out, df.num_cus, static_cast<hipStream_t>(stream));
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!p.large) {
    static thread_local sk::Args sa;
    if (int rc = fill_small(sa, c, layers, nl, x_in, mask_in, y_out, dump, ws, ws_bytes, p)) return rc;
    stage_trace(&sa.trace, &sa.trace_cap, df.num_cus & ~7);
    return launch_small(sa, df.num_cus & ~7, st);        // (a multiple of 8: one weight slice per workgroup and phase, see sk::wg_item)
  }
  static thread_local Args a;
  if (int rc = fill_args(a, c, layers, nl, x_in, mask_in, y_out, dump, ws, ws_bytes, p)) return rc;
  stage_trace(&a.trace, &a.trace_cap, df.num_cus);
  return p.big ? launch_mega<2>(a, df.num_cus, st) : launch_mega<1>(a, df.num_cus, st);
}

template <int MODE>
static int run_unfused_t(Args &a, int nl, int num_cus, hipStream_t st) {
  constexpr int GEMM_LDS = lds_bytes_large();
  constexpr int BN = 128, BM = 128;
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_qkv<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    if constexpr (MODE == 2) {
      SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_presum_big, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
      SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_presum2_big, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    }
    else SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_partial, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_fc1<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_attn, hipFuncAttributeMaxDynamicSharedMemorySize, kAttnLdsBytes));
    attr_done = true;
  }
  const int cap = num_cus * 4;
  auto grid_for = [&](int items) { return items < cap ? items : cap; };
  const half_t *xin = a.x;
  for (int l = 0; l < nl; ++l) {
    const LayerW &w = a.layers[l];
    half_t *yout = (l == nl - 1) ? a.y : a.yl;
    hipLaunchKernelGGL(k_qkv<MODE>, dim3(grid_for((a.M / BM) * (3 * H / BN))), dim3(256), GEMM_LDS, st, a, l, xin);
    hipLaunchKernelGGL(k_attn, dim3(grid_for(a.B * NH * (a.S / 64))), dim3(256), 2 * a.S * 128 + 64 * 128, st, a);
    if constexpr (MODE == 2) {
      hipLaunchKernelGGL(k_presum_big, dim3(grid_for((a.M / 256) * 16)), dim3(256), GEMM_LDS, st, a, a.ctx, H, w.w_o, w.b_o);
      hipLaunchKernelGGL(k_ln_big<1>, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, (const half_t *)a.z1, xin, (const half_t *)nullptr, w.ln1_g, w.ln1_b, a.y1);
    } else {
      hipLaunchKernelGGL(k_partial, dim3(grid_for((a.M / BM) * (H / BN))), dim3(256), GEMM_LDS, st, a, a.ctx, H, w.w_o, 1);
      hipLaunchKernelGGL(k_ln, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, w.b_o, xin, w.ln1_g, w.ln1_b, a.y1);
    }
    hipLaunchKernelGGL(k_fc1<MODE>, dim3(grid_for((a.M / BM) * (F / BN))), dim3(256), GEMM_LDS, st, a, l);
    if constexpr (MODE == 2) {
      hipLaunchKernelGGL(k_presum2_big, dim3(grid_for((a.M / 256) * 16)), dim3(256), GEMM_LDS, st, a, a.h, F, w.w_fc2);
      hipLaunchKernelGGL(k_ln_big<kFc2Split>, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, (const half_t *)a.part, (const half_t *)a.y1, w.b_fc2, w.ln2_g, w.ln2_b, yout);
    } else {
      hipLaunchKernelGGL(k_partial, dim3(grid_for((a.M / BM) * (H / BN))), dim3(256), GEMM_LDS, st, a, a.h, F, w.w_fc2, 1);
      hipLaunchKernelGGL(k_ln, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, w.b_fc2, a.y1, w.ln2_g, w.ln2_b, yout);
    }
    xin = yout;
  }
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

static int run_unfused(const souffle_bert_cfg *c, const souffle_bert_layer_w *layers, int nl, const void *x,
                       const void *mask, void *y, const souffle_bert_dump *dump, void *ws, size_t ws_bytes,
                       souffle_stream_t stream) {
  if (int rc = validate(c)) return rc;
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const Plan p = make_plan(c, nl);
  Padded pd;
  if (int rc = pad_before(pd, c, x, mask, y, dump, ws, ws_bytes, p, df.num_cus, static_cast<hipStream_t>(stream))) return rc;
  if (pd.on) {
    const int rc = run_unfused(&pd.cfg, layers, nl, pd.x, pd.mask, pd.y, nullptr, ws, ws_bytes, stream);
    return rc ? rc : pad_after(pd, c, y, df.num_cus, static_cast<hipStream_t>(stream));
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!p.large) {
    static thread_local sk::Args sa;
    if (int rc = fill_small(sa, c, layers, nl, x, mask, y, dump, ws, ws_bytes, p)) return rc;
    return run_small_unfused(sa, df.num_cus & ~7, st);
  }
  static thread_local Args a;
  if (int rc = fill_args(a, c, layers, nl, x, mask, y, dump, ws, ws_bytes, p)) return rc;
  return p.big ? run_unfused_t<2>(a, nl, df.num_cus, st) : run_unfused_t<1>(a, nl, df.num_cus, st);
}

}  // namespace bert
}  // namespace souffle

using namespace souffle;

extern "C" size_t souffle_bert_workspace_bytes(const souffle_bert_cfg *cfg) {
  if (bert::validate(cfg)) return 0;
  const int nl = cfg->num_layers < 1 ? 1 : (cfg->num_layers > bert::kMaxLayers ? bert::kMaxLayers : cfg->num_layers);
  return bert::make_plan(cfg, nl).total;
}
extern "C" int souffle_bert_layer_fused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *w, const void *x,
                                        const void *mask, void *y, const souffle_bert_dump *dump, void *ws,
                                        size_t ws_bytes, souffle_stream_t stream) {
  return bert::run_fused(cfg, w, 1, x, mask, y, dump, ws, ws_bytes, stream);
}
extern "C" int souffle_bert_layer_unfused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *w, const void *x,
                                          const void *mask, void *y, const souffle_bert_dump *dump, void *ws,
                                          size_t ws_bytes, souffle_stream_t stream) {
  return bert::run_unfused(cfg, w, 1, x, mask, y, dump, ws, ws_bytes, stream);
}
extern "C" int souffle_bert_encoder_fused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                                          const void *x, const void *mask, void *y, void *ws, size_t ws_bytes,
                                          souffle_stream_t stream) {
  if (!cfg) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  return bert::run_fused(cfg, layers, cfg->num_layers, x, mask, y, nullptr, ws, ws_bytes, stream);
}
// ---------------------------------------------------------------- the entry point that allocates nothing ----
// The encoder's inter-phase buffers, flag words and control block in device memory that belongs to the library
// instead of a caller's workspace: for callers that cannot allocate (under graph capture, in a serving loop).
namespace souffle {
namespace bert {
constexpr size_t kStaticScratchBytes = (size_t)48 << 20;      // 12 layers at 128 rows need 42.8 MB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device memory of `scratch` on the current device, looked up once per device (each device has its own copy of the
// array at its own address; the array's name in host code is a stand-in, not an address).
static int static_scratch(unsigned char **out) {
  constexpr int kMaxDevices = 64;
  static unsigned char *per_device[kMaxDevices] = {};
  static std::mutex mu;
  int dev = -1;
  SOUFFLE_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(SOUFFLE_ERR_DEVICE, "device index %d is not supported", dev);
  std::lock_guard<std::mutex> lk(mu);
  if (!per_device[dev]) {
    void *p = nullptr;
    SOUFFLE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(SOUFFLE_ERR_DEVICE, "the library's static scratch has no address on device %d", dev);
    per_device[dev] = static_cast<unsigned char *>(p);
  }
  *out = per_device[dev];
  return SOUFFLE_OK;
}
}  // namespace bert
}  // namespace souffle

extern "C" int souffle_bert_encoder_fused_static(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                                                 const void *x, const void *mask, void *y, souffle_stream_t stream) {
  if (!cfg) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  if (int rc = bert::validate(cfg)) return rc;
  const int nl = cfg->num_layers;
  if (nl < 1 || nl > bert::kMaxLayers) return fail(SOUFFLE_ERR_SHAPE, "num_layers must be in 1..%d (got %d)", bert::kMaxLayers, nl);
  const bert::Plan p = bert::make_plan(cfg, nl);
  if (p.total > bert::kStaticScratchBytes)
    return fail(SOUFFLE_ERR_WORKSPACE, "batch %d x seq_len %d x %d layers needs %zu bytes of scratch, the library's static scratch holds %zu: "
                "use souffle_bert_encoder_fused with a workspace", cfg->batch, cfg->seq_len, nl, p.total, bert::kStaticScratchBytes);
  unsigned char *sc = nullptr;
  if (int rc = bert::static_scratch(&sc)) return rc;
  // Nothing is cleared between calls, whatever their configurations: the array starts as zeros when the library is
  // loaded, like a workspace after souffle_workspace_init; from then on the control block and the flag words (the first
  // bytes, at the same place for every configuration) carry over from call to call as they do in a caller's workspace
  // that serves several shapes: sequence numbers only grow, and the kept wait masks are keyed by the shape.  So the same
  // work is enqueued whether or not earlier calls were made: what a graph capture records does not depend on history.
  return bert::run_fused(cfg, layers, nl, x, mask, y, nullptr, sc, bert::kStaticScratchBytes, stream);
}
extern "C" int souffle_bert_static_status(souffle_stream_t stream, unsigned *flags, int clear) {
  unsigned char *sc = nullptr;
  if (int rc = bert::static_scratch(&sc)) return rc;
  return souffle_workspace_status(sc, stream, flags, clear);
}

// w_fc2 [3072][768] -> 48 slices of 16 output columns, each 96 k-steps of 1 KB: lane L of a wave finds the eight
// halves W[32 t + 8 (L / 16) + 0..7][16 s + L % 16] (its A operand of the 16x16x32 MFMA of k-step t) at
// ((s * 96 + t) * 64 + L) * 16 bytes.  One thread per 16 bytes of output.
namespace souffle {
namespace bert {
__global__ void __launch_bounds__(256) k_pack_fc2(const half_t *w, half_t *out) {
  const int idx = blockIdx.x * 256 + threadIdx.x;               // (s * 96 + t) * 64 + L
  if (idx >= 48 * 96 * 64) return;
  const int L = idx & 63, t = (idx >> 6) % 96, s = idx / (96 * 64);
  const half_t *src = w + (size_t)(32 * t + 8 * (L >> 4)) * H + 16 * s + (L & 15);
  h8 v;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = src[(size_t)j * H];
  *reinterpret_cast<h8 *>(out + (size_t)idx * 8) = v;
}
}  // namespace bert
}  // namespace souffle
extern "C" size_t souffle_bert_fc2_packed_bytes(void) { return (size_t)bert::F * bert::H * 2; }
extern "C" int souffle_bert_pack_fc2(const void *w_fc2, void *packed, souffle_stream_t stream) {
  if (!w_fc2 || !packed) return fail(SOUFFLE_ERR_NULL, "w_fc2 and packed must not be NULL");
  if (!aligned16(w_fc2) || !aligned16(packed)) return fail(SOUFFLE_ERR_ALIGN, "w_fc2 and packed must be 16-byte aligned");
  const char *a = static_cast<const char *>(w_fc2), *b = static_cast<const char *>(packed);
  const size_t n = souffle_bert_fc2_packed_bytes();
  if (a < b + n && b < a + n) return fail(SOUFFLE_ERR_SHAPE, "w_fc2 and packed overlap");
  hipLaunchKernelGGL(bert::k_pack_fc2, dim3(48 * 96 * 64 / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const half_t *>(w_fc2), static_cast<half_t *>(packed));
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

// The work split and the hand-over plan of the few-rows encoder, evaluated on the host with the very functions the
// kernel uses: for tests that check the plan against a model of which rows and columns every item reads and writes.
extern "C" int souffle_bert_handover_plan(int batch, int seq_len, int grid, int fc2_packed, int phase, int workgroup, int *items, int max_items,
                                          int *n_items, unsigned char *needs) {
  namespace sk = bert::sk;
  if (!n_items) return fail(SOUFFLE_ERR_NULL, "n_items is NULL");
  if (batch <= 0 || (seq_len != 64 && seq_len != 128 && seq_len != 256 && seq_len != 384 && seq_len != 512) || bert::many_rows((size_t)batch * seq_len))
    return fail(SOUFFLE_ERR_SHAPE, "the few-rows plan exists for seq_len in {64,128,256,384,512} and the row counts that the few-rows kernel runs (got %d x %d)", batch, seq_len);
  if (grid <= 0 || grid > 1024 || workgroup < 0 || workgroup >= grid) return fail(SOUFFLE_ERR_SHAPE, "grid must be in 1..1024 and workgroup below it");
  if (phase < sk::PH_QKV || phase > sk::PH_FIN || phase == sk::PH_RED) return fail(SOUFFLE_ERR_SHAPE, "phase must be 0 (QKV), 1 (ATT), 2 (OUT), 3 (FC1), 4 (FC2) or 6 (FIN)");
  const sk::Shape sh{batch, seq_len, batch * seq_len, batch * seq_len / 32, grid, fc2_packed ? 1 : 0};
  int n = 0;
  sk::It d;
  for (; sk::wg_item(sh, phase, workgroup, n, d); ++n)
    if (items && n < max_items) { items[2 * n] = d.a; items[2 * n + 1] = d.b; }
  *n_items = n;
  if (needs)
    for (int pb = 0; pb < grid; ++pb)
      needs[pb] = (((phase >= sk::PH_ATT && phase <= sk::PH_FC2) || (fc2_packed && (phase == sk::PH_QKV || phase == sk::PH_FIN))) &&
                   sk::wait_needs(sh, phase, workgroup, pb)) ? 1 : 0;
  return SOUFFLE_OK;
}

extern "C" int souffle_bert_polled_copies(const void *ws, size_t ws_bytes, int *votes_cast, int *copy_block, souffle_stream_t stream) {
  namespace sk = bert::sk;
  if (!ws || !votes_cast || !copy_block) return fail(SOUFFLE_ERR_NULL, "ws, votes_cast and copy_block must not be NULL");
  souffle_bert_cfg c{};
  c.batch = 1; c.seq_len = 128;
  const bert::Plan p = bert::make_plan(&c, 1);          // (the flag words lie at the same place in every plan)
  if (ws_bytes < p.off_flags + (size_t)sk::kFlagWords * 4) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small to hold the flag words");
  unsigned words[8];
  hipStream_t st = static_cast<hipStream_t>(stream);
  SOUFFLE_HIP_TRY(hipMemcpyAsync(words, static_cast<const char *>(ws) + p.off_flags + (size_t)sk::kSideWord * 4, sizeof(words), hipMemcpyDeviceToHost, st));
  SOUFFLE_HIP_TRY(hipStreamSynchronize(st));
  for (int x = 0; x < 8; ++x) {
    votes_cast[x] = (int)(words[x] & 0xffffu);
    copy_block[x] = sk::pair_base_of(x) + (((int)words[x] >> 16) < 0 ? 2 : 0);
  }
  return SOUFFLE_OK;
}

extern "C" int souffle_bert_encoder_unfused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                                            const void *x, const void *mask, void *y, void *ws, size_t ws_bytes,
                                            souffle_stream_t stream) {
  if (!cfg) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  return bert::run_unfused(cfg, layers, cfg->num_layers, x, mask, y, nullptr, ws, ws_bytes, stream);
}
