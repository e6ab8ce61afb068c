// EfficientNet MBConv stack (NHWC, fp16, batch 1) as one persistent kernel on gfx950.
//
// Replaces the operator sequence that the reference times block by block
// (python/models/efficientnet/tvm_efficientnet.py:62-118): head_conv1x1_bn_swish (expansion,
// python/models/efficientnet/efficientnet.py:502-518), fused_depthwise_conv2d_bn_swish
// (:173-195), the squeeze-excite operators (reduce_mean :131-141, se_module_pointwise_conv
// :270-282, fused_pointwise_conv_bias_add_sigmoid_mul :252-267) and pointwise_conv2d_bn
// (:41-57) / pointwise_conv2d_bn_short_cut_add (:83-101).  The reference launches 7 to 9
// kernels per block; here a block is three stages of one launch (four barrier-separated steps:
// the depthwise stage has a barrier of its own in the middle):
//
//   expand   : E = swish(bn(X . We^T))                      one 16x16 MFMA tile per wave
//   depthwise: D = swish(bn(dwconv(E))), and per workgroup the contribution of its pixels or
//              channels to the squeeze layer W_r . sum_p D[p] (R numbers instead of C channel
//              sums); after one more grid barrier workgroup w turns the partials into the
//              squeeze-excite gate of channel group w
//   project  : Y = bn((D * gate) . Wp^T) (+ X), the gate applied to the activation operand on
//              its way into the MFMA
//
// The whole network moves 0.7 GFLOP over ~7 MB of weights and ~12 MB of activations: every
// stage is latency bound, so the design goal is few, short stages with all their loads in flight
// at once, not MFMA utilisation.  The GEMMs therefore take both operands straight from global
// memory/L2 in MFMA operand layout (weights are [out][in], as pointwise_conv2d_bn stores them, so
// a lane's 8 consecutive k-values are one 16-byte load): no LDS staging of operands.
//
// Activations written by one stage and read by the next are stored write-through and read
// with agent-coherent loads: tiles of 16 output channels of neighbouring pixels share cache
// lines, and those lines are written from several XCDs.
#include "common.hpp"
#include "host_util.hpp"

#ifdef SOUFFLE_STAGE_MARKS
#define MB_MARK(tb, id) do { if (tb) { __builtin_amdgcn_s_waitcnt(0); trace_mark(*(tb), (id)); } } while (0)
#else
#define MB_MARK(tb, id) do { } while (0)
#endif

namespace souffle {
namespace mbconv {

constexpr int MAX_BLOCKS = 16;   // per launch (the descriptors travel as kernel arguments)
constexpr int MAX_C = 2048, MAX_R = 64, PART_LD = 64;
#ifndef MBCONV_COH_LOADS
#define MBCONV_COH_LOADS 1
#endif
constexpr bool kCohLoads = MBCONV_COH_LOADS != 0;

struct Block {
  int H, W, Ho, Wo, Cin, Cexp, Cout, k, stride, R, has_expand, has_shortcut;
  const half_t *w_exp, *w_dw, *w_red, *w_se, *w_proj;
  const float *s_exp, *b_exp, *s_dw, *b_dw, *b_red, *b_se, *s_proj, *b_proj;
  const half_t *in;
  half_t *e, *d, *out;
  float *part;                   // [workgroup][PART_LD] partial sums of the squeeze layer
  float *gate;                   // [Cexp] squeeze-excite factors
};

struct Args {
  int nblk, stage_begin, stage_end, trace_cap;
  int strict;                    // souffle_set_strict_fences
  unsigned *ctl;
  unsigned long long *trace;     // optional stage stamps (souffle_set_stage_trace)
  Block blk[MAX_BLOCKS];
};
static_assert(sizeof(Args) <= 4096, "kernel argument segment");

__device__ __forceinline__ float swish(float v) { return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v)); }
__device__ __forceinline__ float sigmoid(float v) { return __builtin_amdgcn_rcpf(1.0f + __expf(-v)); }

// Operands of NS MFMA k-steps (32 k-values each) of one 16 x 16 tile: steps first, first + stride, ...
// of rows xbase / wbase, requested together so that 2*NS 16-byte loads are in flight per wave.
// Steps past K request element 0 and are zeroed.
template <bool COH, int NS>
__device__ __forceinline__ void tile_load(u4 (&xv)[NS], u4 (&wv)[NS], const half_t *X, int xbase, const half_t *__restrict__ Wt,
                                          int wbase, bool wok, int K, int first, int stride, int g) {
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int k0 = (first + i * stride) * 32, kk = k0 + g * 8;
    const bool ok = kk < K;
    const int ks = ok ? kk : 0;
    xv[i] = wv[i] = u4{0u, 0u, 0u, 0u};
    if (k0 < K) {                        // wave-uniform: whole steps past K cost nothing
      xv[i] = ld16<COH && kCohLoads>(X, (xbase + ks) * 2);
      wv[i] = *reinterpret_cast<const u4 *>(Wt + wbase + ks);
      if (!ok) xv[i] = u4{0u, 0u, 0u, 0u};
      if (!ok || !wok) wv[i] = u4{0u, 0u, 0u, 0u};
    }
  }
}
template <bool GATE, int NS>
__device__ __forceinline__ f4 tile_mma(f4 acc, u4 (&xv)[NS], u4 (&wv)[NS], int K, int first, int stride, const float *gate, int g) {
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    if ((first + i * stride) * 32 >= K) break;     // wave-uniform
    if constexpr (GATE) {
      const int kk = (first + i * stride) * 32 + g * 8, ks = kk < K ? kk : 0;
      const f4 g0 = *reinterpret_cast<const f4 *>(gate + ks), g1 = *reinterpret_cast<const f4 *>(gate + ks + 4);
      const h8 x = as_h8(xv[i]);
      xv[i] = as_u4(h8{(half_t)((float)x[0] * g0[0]), (half_t)((float)x[1] * g0[1]), (half_t)((float)x[2] * g0[2]),
                       (half_t)((float)x[3] * g0[3]), (half_t)((float)x[4] * g1[0]), (half_t)((float)x[5] * g1[1]),
                       (half_t)((float)x[6] * g1[2]), (half_t)((float)x[7] * g1[3])});
    }
    acc = mfma_16x16x32(as_h8(wv[i]), as_h8(xv[i]), acc);
  }
  return acc;
}
// All remaining k-steps from `first` on, NS at a time.  The trip count is wave-uniform.
template <bool GATE, bool COH, int NS>
__device__ __forceinline__ f4 tile_dot(f4 acc, const half_t *X, int xbase, const half_t *__restrict__ Wt, int wbase, bool wok, int K,
                                       int first, int stride, const float *gate, int g) {
  for (int s0 = first; s0 * 32 < K; s0 += NS * stride) {
    u4 xv[NS], wv[NS];
    tile_load<COH, NS>(xv, wv, X, xbase, Wt, wbase, wok, K, s0, stride, g);
    acc = tile_mma<GATE, NS>(acc, xv, wv, K, s0, stride, gate, g);
  }
  return acc;
}

// Y[M][N] = act((X[M][K] * gate[K]) . Wt[N][K]^T * scale[N] + shift[N]) (+ shortcut[M][N]) in
// 16 x 16 output tiles.  K and N are multiples of 8, so 16-byte operand granules and 8-byte
// result granules are all-or-nothing at the edges.  With more tiles than workgroups a wave owns
// a tile; otherwise (few pixels, many input channels: the late blocks) a workgroup owns a tile,
// its four waves take every fourth k-step and the partial tiles are summed through `red`.
// mid() is called once by every thread of the workgroup after the operands of the first tile
// have been requested and before they are used: whatever else the stage has to do first (the
// squeeze-excite gate) runs while those loads travel.  It may synchronise the workgroup.
// COH: X and shortcut were written earlier in this launch by other workgroups.
constexpr int kFirstSteps = 12;
template <bool GATE, bool COH, class Mid>
__device__ __forceinline__ void pointwise(const half_t *X, int M, int K, int N, const half_t *__restrict__ Wt,
                                          const float *__restrict__ scale, const float *__restrict__ shift, bool act,
                                          const float *gate, const half_t *shortcut, half_t *Y, float *red, Mid mid) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const int nt_n = (N + 15) >> 4, units = ((M + 15) >> 4) * nt_n;
  const bool split = units <= (int)gridDim.x;
  const int stride = split ? 4 : 1, first = split ? wave : 0;
  auto epilogue = [&](int mt, int nt, f4 acc) {
    const int row = mt * 16 + l16, col = nt * 16 + g * 4;
    if (row < M && col < N) {
      f4 sc = {1.f, 1.f, 1.f, 1.f}, sh = {0.f, 0.f, 0.f, 0.f};
      if (scale) sc = *reinterpret_cast<const f4 *>(scale + col);
      if (shift) sh = *reinterpret_cast<const f4 *>(shift + col);
      f4 v = acc * sc + sh;
      if (act) v = f4{swish(v[0]), swish(v[1]), swish(v[2]), swish(v[3])};
      if (shortcut) {
        const h4 s = as_h4(ld8<COH && kCohLoads>(shortcut, (row * N + col) * 2));
        v += f4{(float)s[0], (float)s[1], (float)s[2], (float)s[3]};
      }
      st8<COH>(Y, (row * N + col) * 2, pack_h4(v));
    }
  };
  int u = split ? (int)blockIdx.x : (int)blockIdx.x * 4 + wave;
  {
    const bool has = u < units;          // workgroup-uniform when split
    const int uu = has ? u : 0, mt = uu / nt_n, nt = uu - mt * nt_n, wrow = nt * 16 + l16;
    const bool wok = wrow < N;
    const int xbase = min(mt * 16 + l16, M - 1) * K, wbase = (wok ? wrow : N - 1) * K;
    u4 xv[kFirstSteps], wv[kFirstSteps];
    if (has) tile_load<COH, kFirstSteps>(xv, wv, X, xbase, Wt, wbase, wok, K, first, stride, g);
    mid();
    if (has) {
      f4 acc = tile_mma<GATE, kFirstSteps>(f4{0.f, 0.f, 0.f, 0.f}, xv, wv, K, first, stride, gate, g);
      acc = tile_dot<GATE, COH, kFirstSteps>(acc, X, xbase, Wt, wbase, wok, K, first + kFirstSteps * stride, stride, gate, g);
      if (split) {
        *reinterpret_cast<f4 *>(red + tid * 4) = acc;
        __syncthreads();
        if (wave == 0) {
#pragma unroll
          for (int w = 1; w < 4; ++w) acc += *reinterpret_cast<const f4 *>(red + (w * 64 + lane) * 4);
          epilogue(mt, nt, acc);
        }
      } else {
        epilogue(mt, nt, acc);
      }
    }
  }
  if (!split) {
    for (u += gridDim.x * 4; u < units; u += gridDim.x * 4) {
      const int mt = u / nt_n, nt = u - mt * nt_n, wrow = nt * 16 + l16;
      const bool wok = wrow < N;
      const f4 acc = tile_dot<GATE, COH, 6>(f4{0.f, 0.f, 0.f, 0.f}, X, min(mt * 16 + l16, M - 1) * K, Wt, (wok ? wrow : N - 1) * K, wok, K,
                                             0, 1, gate, g);
      epilogue(mt, nt, acc);
    }
  }
}

// D[ho][wo][c] = swish(bn(sum_ij X[ho*s - pad + i][wo*s - pad + j][c] * W[i][j][c])), pad = KS/2, for the 8
// channels of group cg at output pixel pix; returns the 8 fp32 results and stores them as fp16.
// All taps and their weights are requested before the first is used (addresses clamped into the
// image, taps outside it masked afterwards): one memory latency per pixel instead of one per tap.
// SLAB: the taps come from an LDS copy of the workgroup's channel groups, laid out
// [input pixel][groups of the workgroup] in 16-byte granules (`slab`, `slab_ld` groups, this thread's `slot`).
template <int KS, bool COH, bool SLAB = false>
__device__ __forceinline__ void dw_pixel(const Block &b, const half_t *src, int pix, int cg, float (&v)[8],
                                         const u4 *slab = nullptr, int slab_ld = 0, int slot = 0) {
  constexpr int pad = KS / 2;
  const int C = b.Cexp, ho = pix / b.Wo, wo = pix - ho * b.Wo;
  u4 xv[KS * KS], wv[KS * KS];
  unsigned inside = 0;
#pragma unroll
  for (int i = 0; i < KS; ++i) {
    const int hi = ho * b.stride - pad + i, hc = min(max(hi, 0), b.H - 1);
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      const int wi = wo * b.stride - pad + j, wc = min(max(wi, 0), b.W - 1);
      if constexpr (SLAB) xv[i * KS + j] = slab[(hc * b.W + wc) * slab_ld + slot];
      else xv[i * KS + j] = ld16<COH && kCohLoads>(src, ((hc * b.W + wc) * C + cg * 8) * 2);
      if (hi == hc && wi == wc) inside |= 1u << (i * KS + j);
    }
  }
#pragma unroll
  for (int t = 0; t < KS * KS; ++t) wv[t] = *reinterpret_cast<const u4 *>(b.w_dw + t * C + cg * 8);
  f4 sc0 = {1.f, 1.f, 1.f, 1.f}, sc1 = sc0, sh0 = {0.f, 0.f, 0.f, 0.f}, sh1 = sh0;
  if (b.s_dw) { sc0 = *reinterpret_cast<const f4 *>(b.s_dw + cg * 8); sc1 = *reinterpret_cast<const f4 *>(b.s_dw + cg * 8 + 4); }
  if (b.b_dw) { sh0 = *reinterpret_cast<const f4 *>(b.b_dw + cg * 8); sh1 = *reinterpret_cast<const f4 *>(b.b_dw + cg * 8 + 4); }
  float acc[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) acc[q] = 0.f;
#pragma unroll
  for (int t = 0; t < KS * KS; ++t) {
    const h8 w = as_h8(wv[t]);
    const h8 x = as_h8((inside >> t) & 1u ? xv[t] : u4{0u, 0u, 0u, 0u});
#pragma unroll
    for (int q = 0; q < 8; ++q) acc[q] += (float)x[q] * (float)w[q];
  }
  h8 o;
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    v[q] = swish(acc[q] * (q < 4 ? sc0[q & 3] : sc1[q & 3]) + (q < 4 ? sh0[q & 3] : sh1[q & 3]));
    o[q] = (half_t)v[q];
  }
  st16<COH>(b.d, (pix * C + cg * 8) * 2, as_u4(o));
}

// How the depthwise stage is dealt to workgroups, and how many of them write a row of squeeze partials.
// Images of at most 256 output pixels: a workgroup owns whole channel groups (all pixels of up to 8
// groups of 8 channels), so its channel sums are complete and its share of the squeeze layer needs
// only its own columns of W_r.  Larger images: a workgroup owns runs of pixels (all channels), so
// that waves read and write contiguous runs of the NHWC tensors.
struct DwPlan {
  bool by_channel;
  int per_wg;        // channel groups per workgroup pass (by_channel) or pixels per pass
  int passes;        // workgroup passes in total
};
__host__ __device__ __forceinline__ DwPlan dw_plan(const Block &b) {
  const int npix = b.Ho * b.Wo, G = b.Cexp >> 3;
  DwPlan p;
  p.by_channel = npix <= 256;
  if (p.by_channel) {
    p.per_wg = 256 / npix < 8 ? 256 / npix : 8;
    p.passes = (G + p.per_wg - 1) / p.per_wg;
  } else {
    p.per_wg = 256 / G;
    p.passes = (npix + p.per_wg - 1) / p.per_wg;
  }
  return p;
}

template <int KS, bool COH>
__device__ __forceinline__ void depthwise(const Block &b, float *red, float *sums, u4 *slab, const GridBarrier *tb = nullptr) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int C = b.Cexp, G = C >> 3, npix = b.Ho * b.Wo;
  const half_t *src = b.has_expand ? b.e : b.in;
  const DwPlan plan = dw_plan(b);
  if ((int)blockIdx.x >= plan.passes) return;
  if (plan.by_channel) {
    const int CGW = plan.per_wg, slot = tid / npix, pix = tid - slot * npix;
    float pj = 0.f;                                  // thread j < R: this workgroup's share of squeeze row j
    for (int set = blockIdx.x; set < plan.passes; set += gridDim.x) {
      const int cg = set * CGW + slot;
      const bool act = slot < CGW && cg < G;
      // thread j requests its row of W_r for the set's channels before anything else
      u4 wr[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const bool ok = tid < b.R && q < CGW && set * CGW + q < G;
        wr[q] = u4{0u, 0u, 0u, 0u};
        if (b.R > 0) {                   // without a squeeze-excite module w_red may be NULL
          wr[q] = *reinterpret_cast<const u4 *>(b.w_red + (ok ? tid * C + (set * CGW + q) * 8 : 0));
          if (!ok) wr[q] = u4{0u, 0u, 0u, 0u};
        }
      }
      // the set's channel groups of every input pixel go to LDS first, [input pixel][CGW] granules of
      // 16 bytes (at most 1024: input pixels <= 4 x output pixels, CGW x output pixels <= 256): the image
      // is fetched once per workgroup in runs of CGW*16 bytes instead of once per tap and lane
      {
        const int ngr = b.H * b.W * CGW;
        u4 sv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int idx = tid + 256 * i, ip = idx / CGW, sl = idx - ip * CGW;
          const bool ok = idx < ngr && set * CGW + sl < G;
          sv[i] = ld16<COH && kCohLoads>(src, ok ? (ip * C + (set * CGW + sl) * 8) * 2 : 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (tid + 256 * i < ngr) slab[tid + 256 * i] = sv[i];
        __syncthreads();
      }
      float v[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] = 0.f;
      MB_MARK(tb, 0);
      if (act) dw_pixel<KS, COH, true>(b, src, pix, cg, v, slab, CGW, slot);
      if (b.R > 0) {
        // channel sums over the pixels: channel ch = slot*8 + q, NP threads per channel take every NP-th pixel
        if (slot < CGW) {
#pragma unroll
          for (int q = 0; q < 8; ++q) red[(slot * 8 + q) * npix + pix] = v[q];        // < 8*CGW*npix <= 2048
        }
        __syncthreads();
        const int nch = CGW * 8, NP = 256 / nch, ch = tid % nch, part = tid / nch;
        MB_MARK(tb, 1);
        if (part < NP) {
          float t = 0.f;
          for (int x = part; x < npix; x += NP) t += red[ch * npix + x];
          sums[part * nch + ch] = t;                                                   // < 256
        }
        __syncthreads();
        if (tid < nch) {
          float t = 0.f;
          for (int x = 0; x < NP; ++x) t += sums[x * nch + tid];
          sums[256 + tid] = t;
        }
        __syncthreads();
        MB_MARK(tb, 2);
        if (tid < b.R) {
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            if (q < CGW) {
              const h8 w = as_h8(wr[q]);
              const f4 s0 = *reinterpret_cast<const f4 *>(sums + 256 + q * 8), s1 = *reinterpret_cast<const f4 *>(sums + 256 + q * 8 + 4);
              pj += (float)w[0] * s0[0] + (float)w[1] * s0[1] + (float)w[2] * s0[2] + (float)w[3] * s0[3] +
                    (float)w[4] * s1[0] + (float)w[5] * s1[1] + (float)w[6] * s1[2] + (float)w[7] * s1[3];
            }
          }
        }
      }
      __syncthreads();               // slab, red and sums are rewritten by the next set
    }
    if (tid < b.R) st4<COH>(b.part, ((int)blockIdx.x * PART_LD + tid) * 4, __float_as_uint(pj));
    MB_MARK(tb, 3);
    return;
  }
  // pixel-major: thread (slot, cg) takes pixel grp*P + slot
  const int P = plan.per_wg, slot = tid / G, cg = tid - slot * G;
  const bool active = slot < P;
  float sum[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) sum[q] = 0.f;
  // rows wave, wave+4, wave+8, wave+12 of W_r are requested now and used after the pixels
  u4 wr[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int j = wave + 4 * a, g8 = lane + 64 * m;
      const bool ok = j < b.R && g8 < G;
      wr[a][m] = u4{0u, 0u, 0u, 0u};
      if (b.R > 0) {                     // without a squeeze-excite module w_red may be NULL
        wr[a][m] = *reinterpret_cast<const u4 *>(b.w_red + (ok ? j * C + g8 * 8 : 0));
        if (!ok) wr[a][m] = u4{0u, 0u, 0u, 0u};
      }
    }
  for (int grp = blockIdx.x; grp < plan.passes; grp += gridDim.x) {
    const int pix = grp * P + slot;
    if (active && pix < npix) {
      float v[8];
      dw_pixel<KS, COH>(b, src, pix, cg, v);
#pragma unroll
      for (int q = 0; q < 8; ++q) sum[q] += v[q];
    }
  }
  if (b.R <= 0) return;
  if (active) {
#pragma unroll
    for (int q = 0; q < 8; ++q) red[slot * C + cg * 8 + q] = sum[q];      // slot*C + ... < P*8G <= 2048
  }
  __syncthreads();
  for (int c = tid; c < C; c += 256) {
    float s = 0.f;
    for (int sl = 0; sl < P; ++sl) s += red[sl * C + c];
    sums[c] = s;
  }
  __syncthreads();
  for (int j0 = wave; j0 < b.R; j0 += 16) {
    if (j0 != wave) {                                // further rows (R > 16): requested here
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const int j = j0 + 4 * a, g8 = lane + 64 * m;
          const bool ok = j < b.R && g8 < G;
          wr[a][m] = *reinterpret_cast<const u4 *>(b.w_red + (ok ? j * C + g8 * 8 : 0));
          if (!ok) wr[a][m] = u4{0u, 0u, 0u, 0u};
        }
    }
    float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int g8 = lane + 64 * m;
      if (g8 < G) {
        const f4 s0 = *reinterpret_cast<const f4 *>(sums + g8 * 8), s1 = *reinterpret_cast<const f4 *>(sums + g8 * 8 + 4);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const h8 w = as_h8(wr[a][m]);
          s[a] += (float)w[0] * s0[0] + (float)w[1] * s0[1] + (float)w[2] * s0[2] + (float)w[3] * s0[3] +
                  (float)w[4] * s1[0] + (float)w[5] * s1[1] + (float)w[6] * s1[2] + (float)w[7] * s1[3];
        }
      }
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const float t = wave_sum(s[a]);
      if (lane == 0 && j0 + 4 * a < b.R) st4<COH>(b.part, ((int)blockIdx.x * PART_LD + j0 + 4 * a) * 4, __float_as_uint(t));
    }
  }
  __syncthreads();                 // red / sums are reused by the next stage
}

// Second half of the depthwise stage of a block with a squeeze-excite module:
// gate[c] = sigmoid(b_e[c] + sum_j W_e[j][c] * swish(b_r[j] + (sum over workgroups of part[.][j]) / pixels)).
// One grid barrier after the partials; then workgroup w evaluates the 8 channels of group w (and
// w + grid, ...): every element of W_e is read once by the whole grid, requested before the barrier.
template <bool COH>
__device__ __forceinline__ void squeeze_gate(const Block &b, GridBarrier &bar, float *red, float *scratch, float *r_s) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int C = b.Cexp, G = C >> 3, npix = b.Ho * b.Wo;
  const bool mine = (int)blockIdx.x < G;
  u4 we = {0u, 0u, 0u, 0u};
  if (mine && tid < b.R) we = *reinterpret_cast<const u4 *>(b.w_se + tid * C + blockIdx.x * 8);
  grid_sync(bar);
  if (!mine) return;
  // the partial rows of all workgroups go through LDS (all loads of a chunk in flight together),
  // thread (quarter, j) sums every fourth row of column j, the quarters are added in a fixed order
  const int nact = min(dw_plan(b).passes, (int)gridDim.x);
  const int R4 = (b.R + 3) >> 2, chunk_rows = 1024 / R4;
  const int j = tid & 63, quarter = tid >> 6;
  float accj = 0.f;
  for (int row0 = 0; row0 < nact; row0 += chunk_rows) {
    const int rows = min(chunk_rows, nact - row0), ngran = rows * R4;
    u4 pv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + 256 * i, r = idx / R4, q = idx - r * R4;
      pv[i] = ld16<COH && kCohLoads>(b.part, idx < ngran ? ((row0 + r) * PART_LD + q * 4) * 4 : 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (tid + 256 * i < ngran) *reinterpret_cast<u4 *>(red + (tid + 256 * i) * 4) = pv[i];
    __syncthreads();
    if (j < b.R)
      for (int r = quarter; r < rows; r += 4) accj += red[r * R4 * 4 + j];
    __syncthreads();
  }
  scratch[quarter * 64 + j] = accj;
  __syncthreads();
  if (tid < 64) {                    // wave 0: lane j holds r[j], then the 8 channel sums over j
    float rj = 0.f;
    if (tid < b.R) {
      const float t = (scratch[tid] + scratch[64 + tid]) + (scratch[128 + tid] + scratch[192 + tid]);
      rj = swish(t / (float)npix + (b.b_red ? b.b_red[tid] : 0.f));
    }
    for (int cg = blockIdx.x; cg < G; cg += gridDim.x) {
      if (cg != (int)blockIdx.x) {
        we = u4{0u, 0u, 0u, 0u};
        if (tid < b.R) we = *reinterpret_cast<const u4 *>(b.w_se + tid * C + cg * 8);
      }
      const h8 w = as_h8(we);
      float mine_q = 0.f;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float t = wave_sum((float)w[q] * rj);
        if (lane == q) mine_q = t;
      }
      if (lane < 8) {
        const int c = cg * 8 + lane;
        st4<COH>(b.gate, c * 4, __float_as_uint(sigmoid(mine_q + (b.b_se ? b.b_se[c] : 0.f))));
      }
    }
  }
  __syncthreads();
}

// Projection with the squeeze-excite gate folded into its activation operand; the gate vector is
// requested together with the operands of the first tile.
template <bool COH>
__device__ __forceinline__ void project(const Block &b, float *gate_s, float *red, const GridBarrier *tb = nullptr) {
  const int tid = threadIdx.x;
  const int npix = b.Ho * b.Wo, C = b.Cexp;
  const half_t *shortcut = b.has_shortcut ? b.in : nullptr;
  if (b.R <= 0) {
    pointwise<false, COH>(b.d, npix, C, b.Cout, b.w_proj, b.s_proj, b.b_proj, false, nullptr, shortcut, b.out, red, []() {});
    return;
  }
  {   // workgroups without a tile of the projection have nothing to do in this stage
    const int units = ((npix + 15) >> 4) * ((b.Cout + 15) >> 4);
    if ((int)blockIdx.x * (units <= (int)gridDim.x ? 1 : 4) >= units) return;
  }
  auto gate = [&]() {
    u4 gv[MAX_C / 1024];
#pragma unroll
    for (int i = 0; i < MAX_C / 1024; ++i) {
      const int idx = tid + 256 * i;
      gv[i] = ld16<COH && kCohLoads>(b.gate, idx * 4 < C ? idx * 16 : 0);
    }
#pragma unroll
    for (int i = 0; i < MAX_C / 1024; ++i)
      if ((tid + 256 * i) * 4 < C) *reinterpret_cast<u4 *>(gate_s + (tid + 256 * i) * 4) = gv[i];
    __syncthreads();
  };
  pointwise<true, COH>(b.d, npix, C, b.Cout, b.w_proj, b.s_proj, b.b_proj, false, gate_s, shortcut, b.out, red, gate);
  MB_MARK(tb, 4);
}

// Stage s of the launch is phase s % 3 (expand, depthwise, project) of block s / 3.
__global__ void __launch_bounds__(256) k_mbconv(const Args a) {
  __shared__ __attribute__((aligned(16))) float red[4096];
  __shared__ __attribute__((aligned(16))) float vec[MAX_C];
  __shared__ u4 slab[1024];
  __shared__ float r_s[MAX_R];
  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl, a.strict != 0);
  bar.trace = a.trace;
  bar.trace_cap = a.trace_cap;
  for (int st = a.stage_begin; st < a.stage_end; ++st) {
    const int bi = st / 3, ph = st - bi * 3;
    const Block &b = a.blk[bi];
    bool ran = true;
    if (ph == 0) {
      if (b.has_expand)
        pointwise<false, true>(b.in, b.H * b.W, b.Cin, b.Cexp, b.w_exp, b.s_exp, b.b_exp, true, nullptr, nullptr, b.e, red, []() {});
      else
        ran = false;
    } else if (ph == 1) {
      if (b.k == 3) depthwise<3, true>(b, red, vec, slab, &bar);
      else depthwise<5, true>(b, red, vec, slab, &bar);
      if (b.R > 0) squeeze_gate<true>(b, bar, red, vec, r_s);
    } else {
      project<true>(b, vec, red, &bar);
    }
    if (ran && st + 1 < a.stage_end) grid_sync(bar);
  }
  grid_barrier_end(bar);
}

// ---- single operators (the reference's operator list as entry points of their own) ----
struct PwArgs {
  const half_t *x, *w, *shortcut;
  const float *scale, *shift, *gate;
  half_t *y;
  int M, K, N, act;
};
__global__ void __launch_bounds__(256) k_pointwise(const PwArgs a) {
  __shared__ __attribute__((aligned(16))) float gate_s[MAX_C];
  __shared__ __attribute__((aligned(16))) float red[1024];
  if (a.gate) {
    for (int c = threadIdx.x; c < a.K; c += 256) gate_s[c] = a.gate[c];
    __syncthreads();
    pointwise<true, false>(a.x, a.M, a.K, a.N, a.w, a.scale, a.shift, a.act != 0, gate_s, a.shortcut, a.y, red, []() {});
  } else {
    pointwise<false, false>(a.x, a.M, a.K, a.N, a.w, a.scale, a.shift, a.act != 0, nullptr, a.shortcut, a.y, red, []() {});
  }
}
__global__ void __launch_bounds__(256) k_depthwise(const Block b) {
  __shared__ __attribute__((aligned(16))) float red[2048];
  __shared__ __attribute__((aligned(16))) float vec[MAX_C];
  __shared__ u4 slab[1024];
  if (b.k == 3) depthwise<3, false>(b, red, vec, slab);
  else depthwise<5, false>(b, red, vec, slab);
}

static int out_extent(int in, int kernel, int stride) { return (in + (kernel - 1) - kernel) / stride + 1; }

static int check_block(const souffle_mbconv_block *s, int i) {
  if (s->in_h <= 0 || s->in_w <= 0) return fail(SOUFFLE_ERR_SHAPE, "block %d: in_h and in_w must be positive", i);
  if (s->in_c <= 0 || s->expand_c <= 0 || s->out_c <= 0 || s->in_c % 8 || s->expand_c % 8 || s->out_c % 8)
    return fail(SOUFFLE_ERR_SHAPE, "block %d: channel counts must be positive multiples of 8 (got %d, %d, %d)", i, s->in_c,
                s->expand_c, s->out_c);
  if (s->expand_c > MAX_C) return fail(SOUFFLE_ERR_SHAPE, "block %d: expand_c <= %d required (got %d)", i, MAX_C, s->expand_c);
  if (s->se_c < 0 || s->se_c > MAX_R) return fail(SOUFFLE_ERR_SHAPE, "block %d: 0 <= se_c <= %d required (got %d)", i, MAX_R, s->se_c);
  if (s->kernel != 3 && s->kernel != 5) return fail(SOUFFLE_ERR_SHAPE, "block %d: kernel must be 3 or 5 (got %d)", i, s->kernel);
  if (s->stride != 1 && s->stride != 2) return fail(SOUFFLE_ERR_SHAPE, "block %d: stride must be 1 or 2 (got %d)", i, s->stride);
  if (!s->expand_w && s->expand_c != s->in_c)
    return fail(SOUFFLE_ERR_SHAPE, "block %d: without an expansion convolution expand_c must equal in_c", i);
  if (s->has_shortcut && (s->stride != 1 || s->in_c != s->out_c))
    return fail(SOUFFLE_ERR_SHAPE, "block %d: the shortcut needs stride 1 and in_c == out_c", i);
  if ((long long)s->in_h * s->in_w * s->expand_c >= (1ll << 29))
    return fail(SOUFFLE_ERR_SHAPE, "block %d: activation of %d x %d x %d elements exceeds the 2^29 limit", i, s->in_h, s->in_w, s->expand_c);
  if (!s->dw_w || !s->project_w) return fail(SOUFFLE_ERR_NULL, "block %d: dw_w and project_w must not be NULL", i);
  if (s->se_c > 0 && (!s->se_reduce_w || !s->se_expand_w))
    return fail(SOUFFLE_ERR_NULL, "block %d: se_reduce_w and se_expand_w must not be NULL when se_c > 0", i);
  if (!aligned16(s->expand_w) || !aligned16(s->dw_w) || !aligned16(s->project_w) || !aligned16(s->expand_scale) ||
      !aligned16(s->expand_shift) || !aligned16(s->project_scale) || !aligned16(s->project_shift))
    return fail(SOUFFLE_ERR_ALIGN, "block %d: weights and folded batch-norm vectors must be 16-byte aligned", i);
  return SOUFFLE_OK;
}

// Workspace: control block, then per block E (if expanded), D, the block output (all blocks but
// the last) and the squeeze partials, each at an address of its own (see the file comment).
struct Plan {
  size_t e[1024], d[1024], out[1024], part[1024], gate[1024], total;
};
static int make_plan(const souffle_mbconv_block *blocks, int n, Plan *p) {
  if (!blocks || n <= 0 || n > 1024) return fail(SOUFFLE_ERR_SHAPE, "need 1..1024 blocks");
  size_t off = round_up(kCtlWords * 4, 256);
  for (int i = 0; i < n; ++i) {
    const souffle_mbconv_block *s = blocks + i;
    if (int rc = check_block(s, i)) return rc;
    const int oh = out_extent(s->in_h, s->kernel, s->stride), ow = out_extent(s->in_w, s->kernel, s->stride);
    if (i + 1 < n && (blocks[i + 1].in_h != oh || blocks[i + 1].in_w != ow || blocks[i + 1].in_c != s->out_c))
      return fail(SOUFFLE_ERR_SHAPE, "block %d does not take what block %d produces (%d x %d x %d)", i + 1, i, oh, ow, s->out_c);
    p->e[i] = off;
    if (s->expand_w) off += round_up((size_t)s->in_h * s->in_w * s->expand_c * 2, 256);
    p->d[i] = off;
    off += round_up((size_t)oh * ow * s->expand_c * 2, 256);
    p->out[i] = off;
    if (i + 1 < n) off += round_up((size_t)oh * ow * s->out_c * 2, 256);
    p->part[i] = off;
    off += round_up((size_t)256 * PART_LD * 4, 256);           // at most 256 workgroups
    p->gate[i] = off;
    off += round_up((size_t)MAX_C * 4, 256);
  }
  p->total = off;
  return SOUFFLE_OK;
}

static void fill_block(Block *b, const souffle_mbconv_block *s) {
  b->H = s->in_h; b->W = s->in_w;
  b->Ho = out_extent(s->in_h, s->kernel, s->stride); b->Wo = out_extent(s->in_w, s->kernel, s->stride);
  b->Cin = s->in_c; b->Cexp = s->expand_c; b->Cout = s->out_c; b->k = s->kernel; b->stride = s->stride; b->R = s->se_c;
  b->has_expand = s->expand_w != nullptr; b->has_shortcut = s->has_shortcut != 0;
  b->w_exp = static_cast<const half_t *>(s->expand_w); b->w_dw = static_cast<const half_t *>(s->dw_w);
  b->w_red = static_cast<const half_t *>(s->se_reduce_w); b->w_se = static_cast<const half_t *>(s->se_expand_w);
  b->w_proj = static_cast<const half_t *>(s->project_w);
  b->s_exp = s->expand_scale; b->b_exp = s->expand_shift; b->s_dw = s->dw_scale; b->b_dw = s->dw_shift;
  b->b_red = s->se_reduce_b; b->b_se = s->se_expand_b; b->s_proj = s->project_scale; b->b_proj = s->project_shift;
}

}  // namespace mbconv
}  // namespace souffle

using namespace souffle;

extern "C" size_t souffle_mbconv_workspace_bytes(const souffle_mbconv_block *blocks, int num_blocks) {
  static thread_local mbconv::Plan p;
  if (mbconv::make_plan(blocks, num_blocks, &p)) return 0;
  return p.total;
}

extern "C" int souffle_mbconv_stack(const souffle_mbconv_block *blocks, int num_blocks, const void *x, void *y, int fused,
                                    void *ws, size_t ws_bytes, souffle_stream_t stream) {
  static thread_local mbconv::Plan p;
  if (int rc = mbconv::make_plan(blocks, num_blocks, &p)) return rc;
  if (!x || !y) return fail(SOUFFLE_ERR_NULL, "x and y must not be NULL");
  if (!aligned16(x) || !aligned16(y)) return fail(SOUFFLE_ERR_ALIGN, "x and y must be 16-byte aligned");
  if (!ws || ws_bytes < p.total) return fail(SOUFFLE_ERR_WORKSPACE, "workspace missing or too small: need %zu bytes", p.total);
  if (!aligned16(ws)) return fail(SOUFFLE_ERR_ALIGN, "workspace must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const int grid = df.num_cus < 256 ? df.num_cus : 256;     // the gate stage reads one partial row per thread
  char *base = static_cast<char *>(ws);
  const hipStream_t st = static_cast<hipStream_t>(stream);
  for (int first = 0; first < num_blocks; first += mbconv::MAX_BLOCKS) {
    const int n = num_blocks - first < mbconv::MAX_BLOCKS ? num_blocks - first : mbconv::MAX_BLOCKS;
    mbconv::Args a;
    a.nblk = n;
    a.ctl = static_cast<unsigned *>(ws);
    a.strict = strict_fences_mode();
    a.trace = nullptr; a.trace_cap = 0;
    if (fused) stage_trace(&a.trace, &a.trace_cap, grid);
    for (int i = 0; i < n; ++i) {
      const int gi = first + i;
      mbconv::Block *b = a.blk + i;
      mbconv::fill_block(b, blocks + gi);
      b->in = gi == 0 ? static_cast<const half_t *>(x) : reinterpret_cast<const half_t *>(base + p.out[gi - 1]);
      b->e = reinterpret_cast<half_t *>(base + p.e[gi]);
      b->d = reinterpret_cast<half_t *>(base + p.d[gi]);
      b->out = gi + 1 == num_blocks ? static_cast<half_t *>(y) : reinterpret_cast<half_t *>(base + p.out[gi]);
      b->part = reinterpret_cast<float *>(base + p.part[gi]);
      b->gate = reinterpret_cast<float *>(base + p.gate[gi]);
    }
    void *args[] = {&a};
    if (fused) {
      a.stage_begin = 0; a.stage_end = 3 * n;
      if (int rc = launch_persistent((const void *)mbconv::k_mbconv, grid, 256, args, 0, st)) return rc;
    } else {
      for (int s = 0; s < 3 * n; ++s) {
        if (s % 3 == 0 && !a.blk[s / 3].has_expand) continue;
        a.stage_begin = s; a.stage_end = s + 1;
        if (int rc = launch_persistent((const void *)mbconv::k_mbconv, grid, 256, args, 0, st)) return rc;
      }
    }
  }
  return SOUFFLE_OK;
}

extern "C" int souffle_pointwise_conv2d_bn(const void *x, const void *w, const float *scale, const float *shift, const float *gate,
                                           const void *shortcut, void *y, int pixels, int in_c, int out_c, int act,
                                           souffle_stream_t stream) {
  if (!x || !w || !y) return fail(SOUFFLE_ERR_NULL, "x, w and y must not be NULL");
  if (pixels <= 0 || in_c <= 0 || out_c <= 0 || in_c % 8 || out_c % 8)
    return fail(SOUFFLE_ERR_SHAPE, "pixels must be positive, in_c and out_c positive multiples of 8 (got %d, %d, %d)", pixels, in_c, out_c);
  if (gate && in_c > mbconv::MAX_C) return fail(SOUFFLE_ERR_SHAPE, "a gated operand needs in_c <= %d (got %d)", mbconv::MAX_C, in_c);
  if ((long long)pixels * in_c >= (1ll << 29) || (long long)pixels * out_c >= (1ll << 29))
    return fail(SOUFFLE_ERR_SHAPE, "tensors of 2^29 elements or more are not supported");
  if (act != SOUFFLE_MB_NONE && act != SOUFFLE_MB_SWISH) return fail(SOUFFLE_ERR_SHAPE, "unknown activation %d", act);
  if (!aligned16(x) || !aligned16(w) || !aligned16(y) || !aligned16(scale) || !aligned16(shift) || !aligned16(shortcut))
    return fail(SOUFFLE_ERR_ALIGN, "tensors must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  mbconv::PwArgs a{static_cast<const half_t *>(x), static_cast<const half_t *>(w), static_cast<const half_t *>(shortcut), scale, shift,
                   gate, static_cast<half_t *>(y), pixels, in_c, out_c, act};
  // few tiles: a workgroup per tile (its waves split K); many: a wave per tile
  const long long units = (long long)((pixels + 15) / 16) * ((out_c + 15) / 16);
  const int grid = units <= df.num_cus ? (int)units : (int)(units / 4 + 1 < df.num_cus * 4 ? units / 4 + 1 : df.num_cus * 4);
  hipLaunchKernelGGL(mbconv::k_pointwise, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

extern "C" int souffle_depthwise_conv2d_bn_swish(const void *x, const void *w, const float *scale, const float *shift, void *y,
                                                 int in_h, int in_w, int channels, int kernel, int stride,
                                                 souffle_stream_t stream) {
  if (!x || !w || !y) return fail(SOUFFLE_ERR_NULL, "x, w and y must not be NULL");
  if (in_h <= 0 || in_w <= 0 || channels <= 0 || channels % 8 || channels > mbconv::MAX_C)
    return fail(SOUFFLE_ERR_SHAPE, "in_h, in_w positive and channels a positive multiple of 8, at most %d (got %d, %d, %d)",
                mbconv::MAX_C, in_h, in_w, channels);
  if (kernel != 3 && kernel != 5) return fail(SOUFFLE_ERR_SHAPE, "kernel must be 3 or 5 (got %d)", kernel);
  if (stride != 1 && stride != 2) return fail(SOUFFLE_ERR_SHAPE, "stride must be 1 or 2 (got %d)", stride);
  if ((long long)in_h * in_w * channels >= (1ll << 29)) return fail(SOUFFLE_ERR_SHAPE, "tensors of 2^29 elements or more are not supported");
  if (!aligned16(x) || !aligned16(w) || !aligned16(y)) return fail(SOUFFLE_ERR_ALIGN, "tensors must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  mbconv::Block b{};
  b.H = in_h; b.W = in_w; b.Ho = mbconv::out_extent(in_h, kernel, stride); b.Wo = mbconv::out_extent(in_w, kernel, stride);
  b.Cin = b.Cexp = channels; b.k = kernel; b.stride = stride; b.R = 0; b.has_expand = 0;
  b.w_dw = static_cast<const half_t *>(w); b.s_dw = scale; b.b_dw = shift;
  b.in = static_cast<const half_t *>(x); b.d = static_cast<half_t *>(y);
  const int passes = mbconv::dw_plan(b).passes;
  const int grid = passes < df.num_cus * 4 ? passes : df.num_cus * 4;
  hipLaunchKernelGGL(mbconv::k_depthwise, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), b);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}
