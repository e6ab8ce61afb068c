// Plain C++ caller of the C ABI (no Python, no torch): one fused and one per-operator BERT
// encoder layer at B=1, S=128 on HIP-runtime allocations, checked against the CPU oracle.
// TEST INFRASTRUCTURE: it links oracle/liboracle.so as the checker.  Plays the role of the
// reference's own C++ driver of the layer (cpp/bert/bert_base_impl.cu:277-308), which allocates
// its tensors itself and calls the kernels without a framework.
// Prints one JSON line; exit status 0 when both paths are within max-abs 2e-2 / mean-abs 2e-3.
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>
#include "../../include/souffle_hip.h"
#include "../../oracle/oracle.h"

#define HIP_OK(e) do { hipError_t r_ = (e); if (r_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #e, hipGetErrorString(r_)); return 2; } } while (0)

// fp16 values and their exact fp32 widenings from a 64-bit LCG (uniform in [-a, a))
static void fill(std::vector<_Float16> &h, std::vector<float> &f, size_t n, float a, uint64_t seed) {
  h.resize(n); f.resize(n);
  uint64_t s = seed * 6364136223846793005ull + 1442695040888963407ull;
  for (size_t i = 0; i < n; ++i) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    const float u = (float)((s >> 40) & 0xffffff) / 16777216.0f;
    h[i] = (_Float16)((2.0f * u - 1.0f) * a);
    f[i] = (float)h[i];
  }
}

template <class T>
static int upload(void **dst, const std::vector<T> &src) {
  HIP_OK(hipMalloc(dst, src.size() * sizeof(T)));
  HIP_OK(hipMemcpy(*dst, src.data(), src.size() * sizeof(T), hipMemcpyHostToDevice));
  return 0;
}

int main() {
  const int B = 1, S = 128, H = 768, F = 3072, M = B * S;
  std::vector<_Float16> hx, hqkv, ho, h1, h2, hb1;
  std::vector<float> fx, fqkv, fo, f1, f2, fb1;
  fill(hx, fx, (size_t)M * H, 1.7f, 1);                 // about unit variance
  fill(hqkv, fqkv, (size_t)3 * H * H, 0.035f, 2);       // about N(0, 0.02)
  fill(ho, fo, (size_t)H * H, 0.035f, 3);
  fill(h1, f1, (size_t)H * F, 0.035f, 4);
  fill(h2, f2, (size_t)F * H, 0.035f, 5);
  fill(hb1, fb1, (size_t)F, 0.1f, 6);                   // one bias, to exercise that path

  souffle_bert_cfg cfg = {B, S, H, 12, F, SOUFFLE_ACT_GELU_TANH, 0.125f, 1e-12f, 1, 0};
  const size_t ws_bytes = souffle_bert_workspace_bytes(&cfg);
  if (!ws_bytes) { fprintf(stderr, "workspace: %s\n", souffle_last_error()); return 2; }
  void *dx, *dqkv, *d_o = nullptr, *d1, *d2, *db1, *dy, *ws;
  if (upload(&dx, hx) || upload(&dqkv, hqkv) || upload(&d_o, ho) || upload(&d1, h1) || upload(&d2, h2) || upload(&db1, hb1)) return 2;
  HIP_OK(hipMalloc(&dy, (size_t)M * H * 2));
  HIP_OK(hipMalloc(&ws, ws_bytes));
  HIP_OK(hipMemset(ws, 0, ws_bytes));
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));
  if (souffle_workspace_init(ws, ws_bytes, st)) { fprintf(stderr, "init: %s\n", souffle_last_error()); return 2; }
  souffle_bert_layer_w w = {};
  w.w_qkv = dqkv; w.w_o = d_o; w.w_fc1 = d1; w.w_fc2 = d2; w.b_fc1 = db1;

  oracle_bert_cfg ocfg = {B, S, H, 12, F, ORACLE_ACT_GELU_TANH, 0.125f, 1e-12f};
  oracle_bert_weights ow = {};
  ow.w_qkv = fqkv.data(); ow.w_o = fo.data(); ow.w_fc1 = f1.data(); ow.w_fc2 = f2.data(); ow.b_fc1 = fb1.data();
  std::vector<float> ref((size_t)M * H);
  if (oracle_bert_layer_f32(&ocfg, &ow, fx.data(), nullptr, ref.data(), nullptr, 8)) { fprintf(stderr, "oracle failed\n"); return 2; }

  std::vector<_Float16> got((size_t)M * H);
  double worst_max = 0, worst_mean = 0;
  int bad = 0;
  // four runs: fused and per-op, first with the [K][N] FC2 matrix alone, then with its packed copy as well
  void *d2p = nullptr;
  HIP_OK(hipMalloc(&d2p, souffle_bert_fc2_packed_bytes()));
  if (souffle_bert_pack_fc2(d2, d2p, st)) { fprintf(stderr, "pack: %s\n", souffle_last_error()); return 2; }
  for (int run = 0; run < 4; ++run) {
    const int fused = (run & 1) == 0;
    w.w_fc2_packed = run >= 2 ? d2p : nullptr;
    HIP_OK(hipMemsetAsync(dy, 0xff, (size_t)M * H * 2, st));
    const int rc = fused ? souffle_bert_layer_fused(&cfg, &w, dx, nullptr, dy, nullptr, ws, ws_bytes, st)
                         : souffle_bert_layer_unfused(&cfg, &w, dx, nullptr, dy, nullptr, ws, ws_bytes, st);
    if (rc) { fprintf(stderr, "layer (%s): %d %s\n", fused ? "fused" : "unfused", rc, souffle_last_error()); return 2; }
    unsigned flags = 0;
    if (souffle_workspace_status(ws, st, &flags, 0) || flags) { fprintf(stderr, "status flags %u: %s\n", flags, souffle_last_error()); return 2; }
    HIP_OK(hipMemcpy(got.data(), dy, got.size() * 2, hipMemcpyDeviceToHost));
    double mx = 0, sum = 0;
    for (size_t i = 0; i < got.size(); ++i) {
      const double d = std::fabs((double)(float)got[i] - (double)ref[i]);
      if (!(d == d)) { mx = 1e9; break; }
      mx = d > mx ? d : mx;
      sum += d;
    }
    const double mean = sum / got.size();
    if (!(mx <= 2e-2 && mean <= 2e-3)) bad = 1;
    worst_max = mx > worst_max ? mx : worst_max;
    worst_mean = mean > worst_mean ? mean : worst_mean;
  }
  printf("{\"caller\": \"plain C++ over the C ABI\", \"version\": \"%s\", \"max_abs\": %.6f, \"mean_abs\": %.6f, \"ok\": %s}\n",
         souffle_version(), worst_max, worst_mean, bad ? "false" : "true");
  for (void *p : {dx, dqkv, d_o, d1, d2, d2p, db1, dy, ws}) (void)hipFree(p);
  (void)hipStreamDestroy(st);
  return bad;
}
