// EfficientNet squeeze-excite module as one persistent cooperative kernel on gfx950.
//
// Replaces torch_dispatch_efficientnet_se_module_v2_short_cut_fused
// (cpp/efficientnet/efficientnet_se_module_binding.cu:164-227) and its kernel
// efficientnet_se_module_v2_short_cut_fused (cpp/efficientnet/kernels/se_module_global_fused.cu:318-444),
// which uses three grid barriers and fixed per-shape launch tables.  Here a WAVE owns a
// (channel, chunk) slice of the input, keeps it in registers from the pooling pass to the
// final combine (x is read from HBM exactly once and y written once), and one grid
// barrier separates the partial sums from the two tiny fully-connected layers, which every
// workgroup evaluates for its own channels.  Any C, H*W, R within the limits below.
#include "common.hpp"
#include "host_util.hpp"

namespace souffle {
namespace se {

constexpr int EPT = 8;        // elements per lane per unit
constexpr int UPW = 2;        // units per wave
constexpr int MAX_C = 2048, MAX_R = 64;

struct Args {
  int C, HW, R, chunks, combine;
  const float *x, *w_reduce, *b_reduce, *w_expand, *b_expand;
  float *y, *pooled, *part;
  unsigned *ctl;
  int strict;        // souffle_set_strict_fences
};

__global__ void __launch_bounds__(256) k_se(Args a) {
  __shared__ __attribute__((aligned(16))) float p_s[MAX_C];
  __shared__ float u_s[4096];
  __shared__ float r_s[MAX_R];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int gw = blockIdx.x * 4 + wave, nw = gridDim.x * 4;
  const int units = a.C * a.chunks, slice = (a.HW + a.chunks - 1) / a.chunks;
  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl, a.strict != 0);

  float v[UPW][EPT];
#pragma unroll
  for (int k = 0; k < UPW; ++k) {
    const int u = gw + k * nw;
    float s = 0.f;
    if (u < units) {
      const int c = u / a.chunks, ch = u % a.chunks;
      const int lo = ch * slice, hi = min(a.HW, lo + slice);
      const float *src = a.x + (size_t)c * a.HW;
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        const int e = lo + lane + 64 * i;
        v[k][i] = e < hi ? src[e] : 0.f;
        s += v[k][i];
      }
      s = wave_sum(s);
      if (lane == 0) st4<true>(a.part, u * 4, __float_as_uint(s));
    }
  }
  grid_sync(bar);

  // pooled mean of every channel (all workgroups need all of it for the reduce layer): the partial sums of all
  // (channel, chunk) units are requested at once, 256 per round, and summed per channel out of LDS
  {
    constexpr int ROUNDS = 4096 / 256;
    unsigned raw[ROUNDS];
#pragma unroll
    for (int i = 0; i < ROUNDS; ++i)
      if (i * 256 < units) raw[i] = ld4<true>(a.part, min(tid + i * 256, units - 1) * 4);
#pragma unroll
    for (int i = 0; i < ROUNDS; ++i)
      if (i * 256 < units && tid + i * 256 < units) u_s[tid + i * 256] = __uint_as_float(raw[i]);
  }
  __syncthreads();
  for (int c = tid; c < a.C; c += 256) {
    float s = 0.f;
    for (int ch = 0; ch < a.chunks; ++ch) s += u_s[c * a.chunks + ch];
    s *= 1.0f / a.HW;
    p_s[c] = s;
    if (blockIdx.x == 0 && a.pooled) a.pooled[c] = s;
  }
  __syncthreads();
  // r = swish(W_r p + b_r): wave w takes outputs w, w + 4, ..., four at a time so that their loads travel together;
  // a lane takes four consecutive channels per load where C allows it
  for (int j0 = wave; j0 < a.R; j0 += 16) {
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if ((a.C & 3) == 0 && (reinterpret_cast<uintptr_t>(a.w_reduce) & 15u) == 0) {
      const int c4n = a.C >> 2;
#pragma unroll 2
      for (int c4 = lane; c4 < c4n; c4 += 64) {
        const f4 pv = *reinterpret_cast<const f4 *>(p_s + 4 * c4);
        f4 wv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          wv[q] = ldg<f4>(reinterpret_cast<const f4 *>(a.w_reduce + (size_t)min(j0 + 4 * q, a.R - 1) * a.C) + c4);
#pragma unroll
        for (int q = 0; q < 4; ++q) s[q] += wv[q][0] * pv[0] + wv[q][1] * pv[1] + wv[q][2] * pv[2] + wv[q][3] * pv[3];
      }
    } else {
#pragma unroll 4
      for (int c = lane; c < a.C; c += 64) {
        const float pv = p_s[c];
#pragma unroll
        for (int q = 0; q < 4; ++q) s[q] += a.w_reduce[(size_t)min(j0 + 4 * q, a.R - 1) * a.C + c] * pv;
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int j = j0 + 4 * q;
      float t = wave_sum(s[q]);
      if (j < a.R) {
        if (a.b_reduce) t += a.b_reduce[j];
        if (lane == 0) r_s[j] = t / (1.0f + __expf(-t));
      }
    }
  }
  __syncthreads();
  // e = sigmoid(W_e r + b_e) for this wave's channels, then combine with the held slice
#pragma unroll
  for (int k = 0; k < UPW; ++k) {
    const int u = gw + k * nw;
    if (u < units) {
      const int c = u / a.chunks, ch = u % a.chunks;
      float s = lane < a.R ? a.w_expand[(size_t)c * a.R + lane] * r_s[lane] : 0.f;
      s = wave_sum(s);
      if (a.b_expand) s += a.b_expand[c];
      const float e = 1.0f / (1.0f + __expf(-s));
      const int lo = ch * slice, hi = min(a.HW, lo + slice);
      float *dst = a.y + (size_t)c * a.HW;
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        const int idx = lo + lane + 64 * i;
        if (idx < hi) dst[idx] = a.combine == SOUFFLE_SE_ADD ? v[k][i] + e : v[k][i] * e;
      }
    }
  }
  grid_barrier_end(bar);
}

static int plan(int C, int HW, int R, int num_cus, int *chunks) {
  if (C <= 0 || HW <= 0 || R <= 0) return fail(SOUFFLE_ERR_SHAPE, "C, HW and R must be positive");
  if (C > MAX_C || R > MAX_R) return fail(SOUFFLE_ERR_SHAPE, "C <= %d and R <= %d required (got %d, %d)", MAX_C, MAX_R, C, R);
  const int waves = num_cus * 4;
  // smallest chunk count whose slices fit a wave's registers, then as many as the waves allow
  int ch = (HW + 64 * EPT - 1) / (64 * EPT);
  while ((long long)C * (ch + 1) <= waves && (HW + ch) / (ch + 1) >= 64) ++ch;
  if ((long long)C * ch > (long long)waves * UPW)
    return fail(SOUFFLE_ERR_SHAPE, "input of %d x %d elements exceeds the register-resident limit of %d", C, HW, waves * UPW * 64 * EPT);
  *chunks = ch;
  return SOUFFLE_OK;
}

}  // namespace se
}  // namespace souffle

using namespace souffle;

extern "C" size_t souffle_se_workspace_bytes(int C, int HW, int R) {
  int chunks = 0;
  if (se::plan(C, HW, R, 256, &chunks)) return 0;
  // sized for any CU count: partial sums of at most 2048 (channel, chunk) units
  return round_up(kCtlWords * 4, 256) + 4 * 4096;
}

extern "C" int souffle_se_module_fused(const float *x, const float *w_reduce, const float *b_reduce, const float *w_expand,
                                       const float *b_expand, float *y, float *pooled, int C, int HW, int R, int combine,
                                       void *ws, size_t ws_bytes, souffle_stream_t stream) {
  if (!x || !w_reduce || !w_expand || !y) return fail(SOUFFLE_ERR_NULL, "x, w_reduce, w_expand and y must not be NULL");
  if (combine != SOUFFLE_SE_MUL && combine != SOUFFLE_SE_ADD) return fail(SOUFFLE_ERR_SHAPE, "unknown combine op %d", combine);
  if (C <= 0 || HW <= 0 || R <= 0 || C > se::MAX_C || R > se::MAX_R)
    return fail(SOUFFLE_ERR_SHAPE, "need 0 < C <= %d, 0 < R <= %d, HW > 0 (got %d, %d, %d)", se::MAX_C, se::MAX_R, C, R, HW);
  const size_t need = round_up(kCtlWords * 4, 256) + 4 * 4096;
  if (!ws || ws_bytes < need) return fail(SOUFFLE_ERR_WORKSPACE, "workspace missing or too small: need %zu bytes", need);
  if (!aligned16(ws)) return fail(SOUFFLE_ERR_ALIGN, "workspace must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  int chunks = 0;
  if (int rc = se::plan(C, HW, R, df.num_cus, &chunks)) return rc;
  if ((long long)C * chunks > 4096) return fail(SOUFFLE_ERR_SHAPE, "too many (channel, chunk) units");
  se::Args a{C, HW, R, chunks, combine, x, w_reduce, b_reduce, w_expand, b_expand, y, pooled,
             reinterpret_cast<float *>(static_cast<char *>(ws) + round_up(kCtlWords * 4, 256)), static_cast<unsigned *>(ws), strict_fences_mode()};
  void *args[] = {&a};
  return launch_persistent((const void *)se::k_se, df.num_cus, 256, args, 0, static_cast<hipStream_t>(stream));
}
