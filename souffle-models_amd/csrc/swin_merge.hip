// Swin patch merging as one kernel on gfx950: 2x2 neighbourhood gather + LayerNorm over the 4C
// merged channels + the bias-free reduction GEMM (4C -> 2C).
//
// Replaces the operator chain of python/models/swin_transformer/swin_patch_merge.py:
// fused_patch_merging_reshape(_reduce_sum) (:49-92), layer_normalization_variance (:95-118),
// layer_normalization_normal (:121-144) and the dense product that follows.  Merged channel
// c' = q*C + c takes source pixel (2i + q%2, 2j + q/2), i.e. torch.cat([x0, x1, x2, x3], -1) of the
// module's docstring (:3-13).  The gather and the normalisation are applied while the activation
// tile is loaded for the MFMA, so the merged tensor never exists in memory; the row statistics are
// two-pass fp32.
#include "common.hpp"
#include "gemm_tile.hpp"
#include "host_util.hpp"

namespace souffle {
namespace swin_merge {

using Tile = GemmTile<64, 64, 128, 2, 2>;      // K = 4C advances in 4C/128 steps: the kernel is a chain of memory latencies

struct Args {
  int H, W, C, M, K, N;
  float eps;
  const half_t *x, *w, *gamma, *beta;
  half_t *y;
};

__global__ void __launch_bounds__(256) k_patch_merge(const Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  half_t *gl = reinterpret_cast<half_t *>(lds);
  float *stats = reinterpret_cast<float *>(lds + Tile::LDS_BYTES);      // (mean, 1/std) of the tile's 64 rows
  const int tid = threadIdx.x, W2 = a.W >> 1;
  const int tn = a.N / 64, items = ((a.M + 63) / 64) * tn;
  // source of merged element (m, k): k = q*C + c
  auto source = [&](int m, int k) {
    const int q = k / a.C, c = k - q * a.C, i = m / W2, j = m - i * W2;
    return (size_t)((2 * i + (q & 1)) * a.W + 2 * j + (q >> 1)) * a.C + c;
  };
  for (int it = blockIdx.x; it < items; it += gridDim.x) {
    const int m0 = (it / tn) * 64, n0 = (it % tn) * 64;
    {   // four threads per merged row, one source pixel each
      const int row = tid >> 2, q = tid & 3, m = min(m0 + row, a.M - 1);
      const half_t *src = a.x + source(m, q * a.C);
      float s = 0.f;
      for (int c = 0; c < a.C; c += 8) {
        const h8 v = as_h8(*reinterpret_cast<const u4 *>(src + c));
#pragma unroll
        for (int e = 0; e < 8; ++e) s += (float)v[e];
      }
      s += wave_xor(s, 1);
      s += wave_xor(s, 2);
      const float mean = s / (float)a.K;
      float d2 = 0.f;
      for (int c = 0; c < a.C; c += 8) {
        const h8 v = as_h8(*reinterpret_cast<const u4 *>(src + c));
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float d = (float)v[e] - mean; d2 += d * d; }
      }
      d2 += wave_xor(d2, 1);
      d2 += wave_xor(d2, 2);
      if (q == 0) {
        stats[row * 2] = mean;
        stats[row * 2 + 1] = 1.0f / sqrtf(d2 / (float)a.K + a.eps);
      }
    }
    __syncthreads();
    Tile::run(gl, a.w, a.N, m0, n0, 0, a.K / Tile::kBK,
              [&](int m, int k) {
                if (m >= a.M) return u4{0u, 0u, 0u, 0u};
                const h8 v = as_h8(*reinterpret_cast<const u4 *>(a.x + source(m, k)));
                const float mean = stats[(m - m0) * 2], rstd = stats[(m - m0) * 2 + 1];
                h8 g, b;
#pragma unroll
                for (int e = 0; e < 8; ++e) { g[e] = (half_t)1.0f; b[e] = (half_t)0.0f; }
                if (a.gamma) g = as_h8(*reinterpret_cast<const u4 *>(a.gamma + k));
                if (a.beta) b = as_h8(*reinterpret_cast<const u4 *>(a.beta + k));
                h8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (half_t)(((float)v[e] - mean) * rstd * (float)g[e] + (float)b[e]);
                return as_u4(o);
              },
              [&](int m, int n, f4 v) {
                if (m < a.M) *reinterpret_cast<u2 *>(a.y + (size_t)m * a.N + n) = pack_h4(v);
              });
    __syncthreads();
  }
}

}  // namespace swin_merge
}  // namespace souffle

using namespace souffle;

extern "C" int souffle_swin_patch_merge(const void *x, const void *ln_g, const void *ln_b, const void *w, void *y, int height,
                                        int width, int channels, float ln_eps, souffle_stream_t stream) {
  if (!x || !w || !y) return fail(SOUFFLE_ERR_NULL, "x, w and y must not be NULL");
  if (height <= 0 || width <= 0 || (height & 1) || (width & 1))
    return fail(SOUFFLE_ERR_SHAPE, "height and width must be positive and even (got %d x %d)", height, width);
  if (channels <= 0 || channels % 32)
    return fail(SOUFFLE_ERR_SHAPE, "channels must be a positive multiple of 32 (got %d)", channels);
  if ((long long)height * width * channels >= (1ll << 30)) return fail(SOUFFLE_ERR_SHAPE, "tensors of 2^30 elements or more are not supported");
  if (!(ln_eps >= 0.f)) return fail(SOUFFLE_ERR_SHAPE, "ln_eps must be >= 0");
  if (!aligned16(x) || !aligned16(w) || !aligned16(y) || !aligned16(ln_g) || !aligned16(ln_b))
    return fail(SOUFFLE_ERR_ALIGN, "all pointers must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  swin_merge::Args a{height, width, channels, (height / 2) * (width / 2), 4 * channels, 2 * channels, ln_eps,
                     static_cast<const half_t *>(x), static_cast<const half_t *>(w), static_cast<const half_t *>(ln_g),
                     static_cast<const half_t *>(ln_b), static_cast<half_t *>(y)};
  const int items = ((a.M + 63) / 64) * (a.N / 64);
  const int grid = items < df.num_cus * 2 ? items : df.num_cus * 2;
  const size_t lds = swin_merge::Tile::LDS_BYTES + 64 * 2 * sizeof(float);
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)swin_merge::k_patch_merge, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_done = true;
  }
  hipLaunchKernelGGL(swin_merge::k_patch_merge, dim3(grid), dim3(256), lds, static_cast<hipStream_t>(stream), a);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}
