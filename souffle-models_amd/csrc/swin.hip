// Swin-Base stage-1 block pair (regular + shifted window) as one persistent cooperative
// kernel on gfx950, plus the reference's fused two-GEMM Swin FFN and the host index maps.
//
// A block is window-local up to its residual, so one workgroup runs a whole block for one
// 7x7 window without any grid barrier: gather (roll + partition folded into the row index)
// -> LN1 -> QKV -> per-head attention with relative-position bias and shifted-window mask
// -> proj + shortcut -> LN2 -> FC1 + GELU -> FC2 + shortcut -> scatter (reverse + roll back
// folded into the same row index).  Only the hand-over from the regular to the shifted
// block crosses workgroups (one grid barrier).  The 49 tokens of a window are padded to 64
// rows for the 16-row MFMA tiles; every intermediate stays in LDS.
// Op list: python/models/swin_transformer/swin_transformer_main.py:11-61 (Part-1..8); the
// reference runs these as separate TVM kernels (:196-330) and has neither the
// relative-position bias nor the shifted-window mask (published Swin definition used).
#include <algorithm>
#include <type_traits>
#include "gemm_tile.hpp"
#include "host_util.hpp"

namespace souffle {
namespace swin {

constexpr int C = 128, NH = 4, HD = 32, WS = 7, N = 49, NP = 64, F = 512, TAB = (2 * WS - 1) * (2 * WS - 1);
constexpr int ZLD = C + 8, BLD = F + 8;
using Tile = GemmTile<64, 64, 64, 2, 2>;

struct BlockW {
  const half_t *ln1_g, *ln1_b, *w_qkv, *b_qkv, *rel_table, *w_proj, *b_proj, *ln2_g, *ln2_b, *w_fc1, *b_fc1, *w_fc2, *b_fc2;
};
struct Args {
  int Hh, Ww, shift, use_mask;
  float eps;
  const half_t *x;
  half_t *mid, *y;
  unsigned *ctl;
  BlockW w[2];
};

// LDS carve-up (bytes)
constexpr int OFF_GEMM = 0;
constexpr int OFF_ZS = OFF_GEMM + Tile::LDS_BYTES;
constexpr int OFF_BIG = OFF_ZS + NP * ZLD * 2;
constexpr int OFF_X1 = OFF_BIG + NP * BLD * 2;
constexpr int OFF_TAB = OFF_X1 + NP * ZLD * 2;
constexpr int OFF_TOK = OFF_TAB + TAB * NH * 4;
constexpr int OFF_REG = OFF_TOK + NP * 4;
constexpr int LDS_BYTES = OFF_REG + NP * 4;

__device__ __forceinline__ int region_of(int i, int n, int shift) {   // slices [0,n-7), [n-7,n-shift), [n-shift,n)
  return i < n - WS ? 0 : (i < n - shift ? 1 : 2);
}

// rows [16*wave, 16*wave+16) of a [64][C] fp16 source -> LayerNorm -> dst (LDS, ld ZLD)
template <class RowLoad>
__device__ __forceinline__ void layernorm_rows(RowLoad load2, half_t *dst, const half_t *gam, const half_t *bet, float eps) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float g0 = 1.f, g1 = 1.f, b0 = 0.f, b1 = 0.f;
  if (gam) { const h2 t = *reinterpret_cast<const h2 *>(gam + 2 * lane); g0 = (float)t[0]; g1 = (float)t[1]; }
  if (bet) { const h2 t = *reinterpret_cast<const h2 *>(bet + 2 * lane); b0 = (float)t[0]; b1 = (float)t[1]; }
  for (int r = wave * 16; r < wave * 16 + 16; ++r) {
    h2 o = {(half_t)0.f, (half_t)0.f};
    if (r < N) {
      const h2 v = load2(r, 2 * lane);
      const float a = (float)v[0], b = (float)v[1];
      const float mean = wave_sum(a + b) * (1.0f / C);
      const float da = a - mean, db = b - mean;
      const float rstd = rsqrtf(wave_sum(da * da + db * db) * (1.0f / C) + eps);
      o = h2{(half_t)(da * rstd * g0 + b0), (half_t)(db * rstd * g1 + b1)};
    }
    *reinterpret_cast<h2 *>(dst + r * ZLD + 2 * lane) = o;
  }
}

__device__ __forceinline__ f4 add_bias4(f4 v, const half_t *bias, int n) {
  if (bias) {
    const h4 bb = *reinterpret_cast<const h4 *>(bias + n);
    v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
  }
  return v;
}

__device__ void block_for_window(unsigned char *lds, const Args &a, const BlockW &w, int shift, const half_t *xin,
                                 half_t *xout, int win) {
  half_t *gemm_lds = reinterpret_cast<half_t *>(lds + OFF_GEMM);
  half_t *zs = reinterpret_cast<half_t *>(lds + OFF_ZS);
  half_t *big = reinterpret_cast<half_t *>(lds + OFF_BIG);
  half_t *x1s = reinterpret_cast<half_t *>(lds + OFF_X1);
  float *tab = reinterpret_cast<float *>(lds + OFF_TAB);
  int *tok = reinterpret_cast<int *>(lds + OFF_TOK);
  int *reg = reinterpret_cast<int *>(lds + OFF_REG);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const int nww = a.Ww / WS;

  __syncthreads();
  if (tid < NP) {
    int t = -1, rg = 0;
    if (tid < N) {
      // rolled grid position of slot tid of this window, and the token it comes from:
      // roll(-shift) then view+permute partition (torch closed forms)
      const int i = (win / nww) * WS + tid / WS, j = (win % nww) * WS + tid % WS;
      t = ((i + shift) % a.Hh) * a.Ww + (j + shift) % a.Ww;
      if (shift > 0) rg = 3 * region_of(i, a.Hh, shift) + region_of(j, a.Ww, shift);
    }
    tok[tid] = t;
    reg[tid] = rg;
  }
  for (int i = tid; i < TAB * NH; i += 256) tab[i] = w.rel_table ? (float)w.rel_table[i] : 0.f;
  __syncthreads();

  // LN1 of the gathered rows
  layernorm_rows([&](int r, int c) { return __builtin_bit_cast(h2, ld4<true>(xin, (tok[r] * C + c) * 2)); }, zs,
                 w.ln1_g, w.ln1_b, a.eps);
  __syncthreads();

  // QKV = Z.Wqkv + b, q pre-scaled by hd^-0.5; kept in LDS as [64][3C]
  const float qscale = rsqrtf((float)HD);
  for (int nt = 0; nt < 3 * C / 64; ++nt) {
    Tile::run(gemm_lds, w.w_qkv, 3 * C, 0, nt * 64, 0, C / 64,
              [&](int m, int k) { return *reinterpret_cast<const u4 *>(zs + m * ZLD + k); },
              [&](int m, int n, f4 v) {
                v = add_bias4(v, w.b_qkv, n);
                if (n < C) v *= qscale;
                *reinterpret_cast<u2 *>(big + m * BLD + n) = pack_h4(v);
              });
  }
  __syncthreads();

  // attention: wave = head
  {
    const int h = wave;
    for (int qt = 0; qt < NP / 16; ++qt) {
      const int q = qt * 16 + l16;
      const h8 qop = *reinterpret_cast<const h8 *>(big + q * BLD + h * HD + g * 8);
      f4 sc[NP / 16];
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < NP / 16; ++t) {
        const h8 kop = *reinterpret_cast<const h8 *>(big + (t * 16 + l16) * BLD + C + h * HD + g * 8);
        f4 s = mfma_16x16x32(kop, qop, f4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int key = t * 16 + g * 4 + v;
          if (key >= N) s[v] = -INFINITY;
          else if (q < N) {
            const int di = q / WS - key / WS + WS - 1, dj = q % WS - key % WS + WS - 1;
            s[v] += tab[(di * (2 * WS - 1) + dj) * NH + h];
            if (a.use_mask && reg[q] != reg[key]) s[v] += -100.0f;
          }
          mx = fmaxf(mx, s[v]);
        }
        sc[t] = s;
      }
      mx = fmaxf(mx, wave_xor(mx, 16));
      mx = fmaxf(mx, wave_xor(mx, 32));
      float sum = 0.f;
#pragma unroll
      for (int t = 0; t < NP / 16; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) { sc[t][v] = __expf(sc[t][v] - mx); sum += sc[t][v]; }
      sum += wave_xor(sum, 16);
      sum += wave_xor(sum, 32);
      const float inv = 1.0f / sum;
      f4 o[HD / 16];
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < NP / 16; ++t) {
        const f4 pr = sc[t] * inv;
        const h4 p = {(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt) {
          const h4 vop = lds_read_tr16(big + (t * 16 + g * 4 + (l16 >> 2)) * BLD + 2 * C + h * HD + dt * 16 + (l16 & 3) * 4);
          o[dt] = mfma_16x16x16(vop, p, o[dt]);
        }
      }
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt)
        *reinterpret_cast<u2 *>(zs + q * ZLD + h * HD + dt * 16 + g * 4) = pack_h4(o[dt]);
    }
  }
  __syncthreads();

  // x1 = x + ctx.Wproj + b  (kept in LDS)
  for (int nt = 0; nt < C / 64; ++nt) {
    Tile::run(gemm_lds, w.w_proj, C, 0, nt * 64, 0, C / 64,
              [&](int m, int k) { return *reinterpret_cast<const u4 *>(zs + m * ZLD + k); },
              [&](int m, int n, f4 v) {
                v = add_bias4(v, w.b_proj, n);
                if (m < N) {
                  const h4 sh = as_h4(ld8<true>(xin, (tok[m] * C + n) * 2));
                  v += f4{(float)sh[0], (float)sh[1], (float)sh[2], (float)sh[3]};
                } else {
                  v = f4{0.f, 0.f, 0.f, 0.f};
                }
                *reinterpret_cast<u2 *>(x1s + m * ZLD + n) = pack_h4(v);
              });
  }
  __syncthreads();

  layernorm_rows([&](int r, int c) { return *reinterpret_cast<const h2 *>(x1s + r * ZLD + c); }, zs, w.ln2_g, w.ln2_b, a.eps);
  __syncthreads();

  // H = gelu(Z2.W1 + b1) in LDS
  for (int nt = 0; nt < F / 64; ++nt) {
    Tile::run(gemm_lds, w.w_fc1, F, 0, nt * 64, 0, C / 64,
              [&](int m, int k) { return *reinterpret_cast<const u4 *>(zs + m * ZLD + k); },
              [&](int m, int n, f4 v) {
                v = add_bias4(v, w.b_fc1, n);
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = gelu_tanh(v[i]);
                *reinterpret_cast<u2 *>(big + m * BLD + n) = pack_h4(v);
              });
  }
  __syncthreads();

  // out = x1 + H.W2 + b2, scattered back to the token rows
  for (int nt = 0; nt < C / 64; ++nt) {
    Tile::run(gemm_lds, w.w_fc2, C, 0, nt * 64, 0, F / 64,
              [&](int m, int k) { return *reinterpret_cast<const u4 *>(big + m * BLD + k); },
              [&](int m, int n, f4 v) {
                if (m < N) {
                  v = add_bias4(v, w.b_fc2, n);
                  const h4 r = *reinterpret_cast<const h4 *>(x1s + m * ZLD + n);
                  v += f4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
                  st8<true>(xout, (tok[m] * C + n) * 2, pack_h4(v));
                }
              });
  }
}

__global__ void __launch_bounds__(256) k_block_pair(Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl);
  const int nwin = (a.Hh / WS) * (a.Ww / WS);
  for (int win = blockIdx.x; win < nwin; win += gridDim.x) block_for_window(lds, a, a.w[0], 0, a.x, a.mid, win);
  grid_sync(bar);
  for (int win = blockIdx.x; win < nwin; win += gridDim.x) block_for_window(lds, a, a.w[1], a.shift, a.mid, a.y, win);
  grid_barrier_end(bar);
}

// ---- fused two-GEMM FFN: Y1 = X.W1 ; Y2 = Y1.W2 (split-K partials + reduce) ----
struct FfnArgs {
  int M, K, F, splitk;
  const half_t *x, *w1, *w2;
  half_t *y1, *y2;
  float *part;
  unsigned *ctl;
};

__global__ void __launch_bounds__(256) k_ffn(FfnArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  half_t *gl = reinterpret_cast<half_t *>(lds);
  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl);
  {
    const int tn = a.F / 64, items = (a.M / 64) * tn;
    for (int it = blockIdx.x; it < items; it += gridDim.x)
      Tile::run(gl, a.w1, a.F, (it / tn) * 64, (it % tn) * 64, 0, a.K / 64,
                [&](int m, int k) { return *reinterpret_cast<const u4 *>(a.x + (size_t)m * a.K + k); },
                [&](int m, int n, f4 v) { st8<true>(a.y1, (m * a.F + n) * 2, pack_h4(v)); });
  }
  grid_sync(bar);
  {
    const int tn = a.K / 64, items = (a.M / 64) * tn * a.splitk, kper = a.F / a.splitk;
    for (int it = blockIdx.x; it < items; it += gridDim.x) {
      const int ks = it % a.splitk, t = it / a.splitk;
      Tile::run(gl, a.w2, a.K, (t / tn) * 64, (t % tn) * 64, ks * kper, kper / 64,
                [&](int m, int k) { return ld16<true>(a.y1, (m * a.F + k) * 2); },
                [&](int m, int n, f4 v) { st16<true>(a.part, ((ks * a.M + m) * a.K + n) * 4, __builtin_bit_cast(u4, v)); });
    }
  }
  grid_sync(bar);
  for (int i = (blockIdx.x * 256 + threadIdx.x) * 4; i < a.M * a.K; i += gridDim.x * 256 * 4) {
    f4 s = __builtin_bit_cast(f4, ld16<true>(a.part, i * 4));
    for (int ks = 1; ks < a.splitk; ++ks) s += __builtin_bit_cast(f4, ld16<true>(a.part, (ks * a.M * a.K + i) * 4));
    *reinterpret_cast<u2 *>(a.y2 + i) = pack_h4(s);
  }
  grid_barrier_end(bar);
}

static int validate(const souffle_swin_cfg *c) {
  if (!c) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  if (c->channels != C || c->heads != NH || c->window != WS || c->mlp_ratio != 4)
    return fail(SOUFFLE_ERR_SHAPE, "only channels=128 heads=4 window=7 mlp_ratio=4 is built");
  if (c->height <= 0 || c->width <= 0 || c->height % WS || c->width % WS)
    return fail(SOUFFLE_ERR_SHAPE, "height and width must be positive multiples of 7 (got %d x %d)", c->height, c->width);
  if ((long long)c->height * c->width > 1 << 20) return fail(SOUFFLE_ERR_SHAPE, "too many tokens");
  if (c->shift < 0 || c->shift >= WS) return fail(SOUFFLE_ERR_SHAPE, "shift must be in 0..6 (got %d)", c->shift);
  if (!(c->ln_eps >= 0.f)) return fail(SOUFFLE_ERR_SHAPE, "ln_eps must be >= 0");
  return SOUFFLE_OK;
}
static size_t pair_ws_bytes(const souffle_swin_cfg *c) {
  return round_up(kCtlWords * 4, 256) + round_up((size_t)c->height * c->width * C * 2, 256);
}

}  // namespace swin
}  // namespace souffle

using namespace souffle;

extern "C" size_t souffle_swin_workspace_bytes(const souffle_swin_cfg *cfg) {
  if (swin::validate(cfg)) return 0;
  return swin::pair_ws_bytes(cfg);
}

extern "C" int souffle_swin_block_pair_fused(const souffle_swin_cfg *cfg, const souffle_swin_block_w w[2], const void *x,
                                             void *y, void *ws, size_t ws_bytes, souffle_stream_t stream) {
  if (int rc = swin::validate(cfg)) return rc;
  if (!w || !x || !y) return fail(SOUFFLE_ERR_NULL, "w, x and y must not be NULL");
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL (need %zu bytes)", swin::pair_ws_bytes(cfg));
  if (ws_bytes < swin::pair_ws_bytes(cfg)) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, swin::pair_ws_bytes(cfg));
  if (!aligned16(x) || !aligned16(y) || !aligned16(ws)) return fail(SOUFFLE_ERR_ALIGN, "x, y and workspace must be 16-byte aligned");
  swin::Args a;
  a.Hh = cfg->height; a.Ww = cfg->width; a.shift = cfg->shift; a.use_mask = cfg->use_shift_mask && cfg->shift > 0; a.eps = cfg->ln_eps;
  a.x = static_cast<const half_t *>(x); a.y = static_cast<half_t *>(y);
  a.ctl = static_cast<unsigned *>(ws);
  a.mid = reinterpret_cast<half_t *>(static_cast<char *>(ws) + round_up(kCtlWords * 4, 256));
  for (int b = 0; b < 2; ++b) {
    const souffle_swin_block_w &s = w[b];
    if (!s.w_qkv || !s.w_proj || !s.w_fc1 || !s.w_fc2) return fail(SOUFFLE_ERR_NULL, "block %d: a weight matrix is NULL", b);
    const void *ptrs[13] = {s.ln1_g, s.ln1_b, s.w_qkv, s.b_qkv, s.rel_table, s.w_proj, s.b_proj, s.ln2_g, s.ln2_b, s.w_fc1, s.b_fc1, s.w_fc2, s.b_fc2};
    for (const void *q : ptrs)
      if (!aligned16(q)) return fail(SOUFFLE_ERR_ALIGN, "block %d: a weight/bias pointer is not 16-byte aligned", b);
    const half_t **d = reinterpret_cast<const half_t **>(&a.w[b]);
    for (int i = 0; i < 13; ++i) d[i] = static_cast<const half_t *>(ptrs[i]);
  }
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  if (!df.cooperative) return fail(SOUFFLE_ERR_DEVICE, "device does not support cooperative launch");
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)swin::k_block_pair, hipFuncAttributeMaxDynamicSharedMemorySize, swin::LDS_BYTES));
    attr_done = true;
  }
  const int nwin = (cfg->height / swin::WS) * (cfg->width / swin::WS);
  void *args[] = {&a};
  return launch_persistent((const void *)swin::k_block_pair, std::min(nwin, df.num_cus), 256, args, swin::LDS_BYTES,
                           static_cast<hipStream_t>(stream));
}

// Closed forms of torch.roll(-shift) + view/permute window partition, its inverse, the
// relative-position index and the shifted-window region labels.
extern "C" int souffle_swin_index_maps(int height, int width, int window, int shift, int32_t *gather_idx,
                                       int32_t *scatter_idx, int32_t *relpos_idx, int32_t *region_id) {
  if (height <= 0 || width <= 0 || window <= 0 || height % window || width % window)
    return fail(SOUFFLE_ERR_SHAPE, "height and width must be positive multiples of window");
  if (shift < 0 || shift >= window) return fail(SOUFFLE_ERR_SHAPE, "shift must be in 0..window-1");
  const int nww = width / window, n = window * window;
  auto region = [&](int i, int extent) { return i < extent - window ? 0 : (i < extent - shift ? 1 : 2); };
  for (int w = 0; w < (height / window) * nww; ++w)
    for (int s = 0; s < n; ++s) {
      const int i = (w / nww) * window + s / window, j = (w % nww) * window + s % window;
      const int t = ((i + shift) % height) * width + (j + shift) % width;
      if (gather_idx) gather_idx[w * n + s] = t;
      if (scatter_idx) scatter_idx[t] = w * n + s;
      if (region_id) region_id[w * n + s] = shift > 0 ? 3 * region(i, height) + region(j, width) : 0;
    }
  if (relpos_idx)
    for (int p = 0; p < n; ++p)
      for (int q = 0; q < n; ++q)
        relpos_idx[p * n + q] = (p / window - q / window + window - 1) * (2 * window - 1) + (p % window - q % window + window - 1);
  return SOUFFLE_OK;
}

extern "C" int souffle_swin_ffn_fused(const void *x, const void *w1, const void *w2, void *y1, void *y2, int M, int K, int F,
                                      void *ws, size_t ws_bytes, souffle_stream_t stream) {
  if (!x || !w1 || !w2 || !y1 || !y2) return fail(SOUFFLE_ERR_NULL, "x, w1, w2, y1 and y2 must not be NULL");
  if (M <= 0 || K <= 0 || F <= 0 || M % 64 || K % 64 || F % 64 || (long long)M * F > (1 << 28))
    return fail(SOUFFLE_ERR_SHAPE, "M, K and F must be positive multiples of 64 (got %d,%d,%d)", M, K, F);
  if (!aligned16(x) || !aligned16(w1) || !aligned16(w2) || !aligned16(y1) || !aligned16(y2) || !aligned16(ws))
    return fail(SOUFFLE_ERR_ALIGN, "all pointers must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  int splitk = 1;
  while (splitk < 8 && (M / 64) * (K / 64) * splitk * 2 <= df.num_cus && (F / (splitk * 2)) % 64 == 0) splitk *= 2;
  const size_t need = round_up(kCtlWords * 4, 256) + (size_t)splitk * M * K * 4;
  if (!ws || ws_bytes < need) return fail(SOUFFLE_ERR_WORKSPACE, "workspace missing or too small: need %zu bytes", need);
  swin::FfnArgs a{M, K, F, splitk, (const half_t *)x, (const half_t *)w1, (const half_t *)w2, (half_t *)y1, (half_t *)y2,
                  reinterpret_cast<float *>(static_cast<char *>(ws) + round_up(kCtlWords * 4, 256)), static_cast<unsigned *>(ws)};
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)swin::k_ffn, hipFuncAttributeMaxDynamicSharedMemorySize, swin::Tile::LDS_BYTES));
    attr_done = true;
  }
  void *args[] = {&a};
  return launch_persistent((const void *)swin::k_ffn, df.num_cus, 256, args, swin::Tile::LDS_BYTES, static_cast<hipStream_t>(stream));
}
