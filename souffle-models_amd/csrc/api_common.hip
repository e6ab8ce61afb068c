// Entry points that are not tied to one model family: error text, device facts,
// workspace initialisation, the event-timing helper and the plain GEMM.
#include <algorithm>
#include <cstring>
#include <atomic>
#include <map>
#include <mutex>
#include <cstdlib>
#include <type_traits>
#include <vector>
#include "gemm_tile.hpp"
#include "common.hpp"
#include "host_util.hpp"

namespace souffle {

char *error_buffer() {
  static thread_local char buf[512] = "";
  return buf;
}
int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

int device_facts(DeviceFacts *out) {
  static std::mutex mu;
  static DeviceFacts cached[16] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return fail(SOUFFLE_ERR_DEVICE, "no HIP device is available"); }
  if (dev < 0 || dev >= 16) return fail(SOUFFLE_ERR_DEVICE, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lk(mu);
  if (!cached[dev].ok) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, dev) != hipSuccess) { (void)hipGetLastError(); return fail(SOUFFLE_ERR_DEVICE, "hipGetDeviceProperties failed"); }
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
      return fail(SOUFFLE_ERR_DEVICE, "built for gfx950 only, device is %s", p.gcnArchName);
    // cooperative grids are sized by this number; the grid barrier has 256 arrival flags
    cached[dev].num_cus = p.multiProcessorCount < 256 ? p.multiProcessorCount : 256;
    cached[dev].lds_per_cu = (int)p.maxSharedMemoryPerMultiProcessor;
    cached[dev].cooperative = p.cooperativeLaunch;
    strncpy(cached[dev].arch, p.gcnArchName, 63);
    cached[dev].ok = 1;
  }
  *out = cached[dev];
  return SOUFFLE_OK;
}

static void *g_trace_buf = nullptr;
static size_t g_trace_bytes = 0;
static std::atomic<int> g_swin_split{-1};
int swin_split_mode() {
  int v = g_swin_split.load();
  if (v < 0) {
    const char *e = getenv("SOUFFLE_SWIN_SPLIT");
    v = (e && e[0] == '0') ? 0 : 1;
    g_swin_split.store(v);
  }
  return v;
}
static std::atomic<int> g_strict{-1};
int strict_fences_mode() {
  int v = g_strict.load();
  if (v < 0) {
    const char *e = getenv("SOUFFLE_STRICT_FENCES");
    v = (e && e[0] == '1') ? 1 : 0;
    g_strict.store(v);
  }
  return v;
}
static std::atomic<int> g_cooperative{-1};
static bool cooperative_mode() {
  int v = g_cooperative.load();
  if (v < 0) {
    const char *e = getenv("SOUFFLE_COOPERATIVE_LAUNCH");
    v = (e && e[0] == '1') ? 1 : 0;
    g_cooperative.store(v);
  }
  return v == 1;
}

int launch_persistent(const void *fn, int grid, int block, void **args, size_t lds_bytes, hipStream_t st) {
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  {
    static std::mutex mu;
    static std::map<std::pair<const void *, size_t>, int> per_cu;     // (function, LDS bytes) -> workgroups per CU
    std::lock_guard<std::mutex> lk(mu);
    auto key = std::make_pair(fn, lds_bytes);
    auto it = per_cu.find(key);
    if (it == per_cu.end()) {
      int n = 0;
      SOUFFLE_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, block, lds_bytes));
      it = per_cu.emplace(key, n).first;
    }
    if ((long long)it->second * df.num_cus < grid)
      return fail(SOUFFLE_ERR_DEVICE, "a grid of %d workgroups cannot be resident at once (%d per CU on %d CUs)", grid, it->second, df.num_cus);
  }
  if (cooperative_mode()) {
    if (!df.cooperative) return fail(SOUFFLE_ERR_DEVICE, "device does not support cooperative launches");
    SOUFFLE_HIP_TRY(hipLaunchCooperativeKernel(fn, dim3(grid), dim3(block), args, lds_bytes, st));
  } else {
    SOUFFLE_HIP_TRY(hipLaunchKernel(fn, dim3(grid), dim3(block), args, lds_bytes, st));
  }
  return SOUFFLE_OK;
}

void stage_trace(unsigned long long **buf, int *max_barriers, int nblk) {
  *buf = static_cast<unsigned long long *>(g_trace_buf);
  *max_barriers = g_trace_buf ? (int)(g_trace_bytes / ((size_t)nblk * 80)) : 0;   // 2 stamps + 8 marks per barrier
}

__global__ void k_zero_words(unsigned *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}
// 16 bytes per thread and step, any size (n16 = number of 16-byte units).
__global__ void __launch_bounds__(256) k_zero_bytes(u4 *p, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) p[i] = u4{0u, 0u, 0u, 0u};
}

// Plain Y = X.W (fp16 in/out, fp32 accumulate): one tile per workgroup.
template <class Tile>
__global__ void __launch_bounds__(256) k_gemm(const half_t *X, const half_t *W, half_t *Y, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int tiles_n = N / Tile::kBN, items = (M / Tile::kBM) * tiles_n;
  for (int item = blockIdx.x; item < items; item += gridDim.x) {
    const int tm = item / tiles_n, n0 = (item % tiles_n) * Tile::kBN;
    auto aload = [&](int m, int k) { return *reinterpret_cast<const u4 *>(X + (size_t)m * K + k); };
    auto epi = [&](int m, int n, f4 v) { *reinterpret_cast<u2 *>(Y + (size_t)m * N + n) = pack_h4(v); };
    Tile::run(reinterpret_cast<half_t *>(lds_raw), W, N, tm * Tile::kBM, n0, 0, K / Tile::kBK, aload, epi);
  }
}

template <class Tile>
int launch_gemm(const half_t *x, const half_t *w, half_t *y, int M, int N, int K, int num_cus, hipStream_t st) {
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_gemm<Tile>, hipFuncAttributeMaxDynamicSharedMemorySize, Tile::LDS_BYTES));
    attr_done = true;
  }
  const int items = (M / Tile::kBM) * (N / Tile::kBN);
  hipLaunchKernelGGL(k_gemm<Tile>, dim3(std::min(items, num_cus * 4)), dim3(256), Tile::LDS_BYTES, st, x, w, y, M, N, K);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

}  // namespace souffle

using namespace souffle;

extern "C" const char *souffle_last_error(void) { return error_buffer(); }
extern "C" const char *souffle_version(void) { return "souffle_hip 0.1 (gfx950)"; }

extern "C" int souffle_device_info(souffle_devinfo *out) {
  if (!out) return fail(SOUFFLE_ERR_NULL, "out is NULL");
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return fail(SOUFFLE_ERR_DEVICE, "no HIP device is available"); }
  hipDeviceProp_t p;
  if (hipGetDeviceProperties(&p, dev) != hipSuccess) { (void)hipGetLastError(); return fail(SOUFFLE_ERR_DEVICE, "hipGetDeviceProperties failed"); }
  memset(out, 0, sizeof(*out));
  out->num_cus = p.multiProcessorCount;
  out->lds_bytes_per_cu = (int)p.maxSharedMemoryPerMultiProcessor;
  out->clock_khz = p.clockRate;
  out->mem_clock_khz = p.memoryClockRate;
  out->mem_bus_bits = p.memoryBusWidth;
  out->l2_bytes = p.l2CacheSize;
  out->cooperative_launch = p.cooperativeLaunch;
  out->wavefront_size = p.warpSize;
  strncpy(out->arch, p.gcnArchName, sizeof(out->arch) - 1);
  return SOUFFLE_OK;
}

// MFMA-only loop for the empirical matrix-core ceiling: 16 independent 16x16x32 fp16 accumulator
// tiles per wave, updated in place in AGPRs (the form the GEMM kernels use; the three-address
// builtin issues at 44 instead of 16 cycles per instruction here), no memory traffic in the loop.
namespace souffle {
__global__ void __launch_bounds__(256) k_mfma_probe(float *out, int iters) {
  const int lane = threadIdx.x & 63;
  h8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) { a[i] = (half_t)(0.001f * (lane + i)); b[i] = (half_t)(0.002f * (lane - i)); }
  f4 acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = f4{0.f, 0.f, 0.f, 0.f};
  mfma_pin(acc, true);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) mfma_16x16x32_inplace(acc[j], a, b);
  }
  mfma_pin(acc, false);
  f4 s = acc[0];
#pragma unroll
  for (int j = 1; j < 16; ++j) s += acc[j];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
}
}  // namespace souffle

extern "C" int souffle_mfma_probe(float *out, size_t out_bytes, int iters, double *flops, souffle_stream_t stream) {
  if (!out) return fail(SOUFFLE_ERR_NULL, "out is NULL");
  if (iters <= 0 || iters > (1 << 20)) return fail(SOUFFLE_ERR_SHAPE, "iters must be in 1..2^20 (got %d)", iters);
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const int grid = df.num_cus;                           // one wave per SIMD, as in the GEMM kernels
  if (out_bytes < (size_t)grid * 256 * 4) return fail(SOUFFLE_ERR_WORKSPACE, "out needs %zu bytes", (size_t)grid * 256 * 4);
  hipLaunchKernelGGL(souffle::k_mfma_probe, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), out, iters);
  SOUFFLE_HIP_TRY(hipGetLastError());
  if (flops) *flops = (double)grid * 4 * iters * 16 * (2.0 * 16 * 16 * 32);
  return SOUFFLE_OK;
}

// L2-to-LDS streaming rate: every workgroup does nothing but pull an L2-resident region into LDS with
// wave-wide 16-byte direct loads (1 KB contiguous each, 8 to 12 in flight per wave), the way the GEMM
// kernels take in their operands.  All workgroups walk the same region from different starting points.
namespace souffle {
__global__ void __launch_bounds__(256) k_l2_stream_probe(const unsigned char *src, unsigned span, int iters) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned ring = lds_address(lds);
  unsigned o = ((blockIdx.x % 16u) * 65536u + wave * 1024u + lane * 16u) % span;   // span is a multiple of 4096
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      load_lds16(src + o, ring + (((it & 1) * 8 + u) * 4096) + wave * 1024);
      o += 4096u;
      if (o >= span) o -= span;
    }
    wait_vmcnt<4>();
  }
  wait_vmcnt<0>();
}
}  // namespace souffle

extern "C" int souffle_l2_stream_probe(const void *src, size_t src_bytes, int iters, double *bytes, souffle_stream_t stream) {
  if (!src) return fail(SOUFFLE_ERR_NULL, "src is NULL");
  if (!aligned16(src)) return fail(SOUFFLE_ERR_ALIGN, "src must be 16-byte aligned");
  if (src_bytes < 65536 || src_bytes > ((size_t)1 << 30)) return fail(SOUFFLE_ERR_SHAPE, "src_bytes must be in 64 KiB..1 GiB (got %zu)", src_bytes);
  if (iters <= 0 || iters > (1 << 20)) return fail(SOUFFLE_ERR_SHAPE, "iters must be in 1..2^20 (got %d)", iters);
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const unsigned span = (unsigned)(src_bytes & ~(size_t)4095);
  const unsigned char *p = static_cast<const unsigned char *>(src);
  hipLaunchKernelGGL(souffle::k_l2_stream_probe, dim3(df.num_cus), dim3(256), 0, static_cast<hipStream_t>(stream), p, span, iters);
  SOUFFLE_HIP_TRY(hipGetLastError());
  if (bytes) *bytes = (double)df.num_cus * 4 * iters * 8 * 1024.0;
  return SOUFFLE_OK;
}

// The floor of a chain of dependent grid-wide stages on this device: `n` stages that do nothing but
// hand a value on.  mode 0: the grid barrier alone.  mode 1: every workgroup writes 16 bytes through,
// passes the barrier, and reads the 16 bytes another workgroup (on another XCD) wrote; what it reads
// goes into what it writes next, so each stage costs a store acknowledgement, a barrier and one
// memory round trip, like a real stage with no arithmetic.
namespace souffle {
__global__ void __launch_bounds__(256) k_stage_floor(unsigned *ctl, u4 *buf, int n, int mode, unsigned *out, int strict) {
  GridBarrier bar;
  grid_barrier_begin(bar, ctl, strict != 0);
  const int grid = gridDim.x, peer = (blockIdx.x + 37) % grid;
  u4 v = {blockIdx.x, 1u, 2u, 3u};
  for (int i = 0; i < n; ++i) {
    if (mode && threadIdx.x == 0) st16<true>(buf, ((i & 1) * grid + (int)blockIdx.x) * 16, v);
    grid_sync(bar);
    if (mode) {
      const u4 r = ld16<true>(buf, ((i & 1) * grid + peer) * 16);
      v = u4{v[0] + r[0], v[1] ^ r[1], v[2] + 1u, r[3]};
    }
  }
  if (threadIdx.x == 0) out[blockIdx.x] = v[0] + v[1] + v[2] + v[3];
  grid_barrier_end(bar);
}
}  // namespace souffle

extern "C" int souffle_stage_floor_probe(void *ws, size_t ws_bytes, int stages, int mode, souffle_stream_t stream) {
  if (!ws) return fail(SOUFFLE_ERR_NULL, "workspace is NULL");
  if (stages <= 0 || stages > 100000) return fail(SOUFFLE_ERR_SHAPE, "stages must be in 1..100000 (got %d)", stages);
  if (mode != 0 && mode != 1) return fail(SOUFFLE_ERR_SHAPE, "mode must be 0 or 1");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const size_t ctl_bytes = round_up(kCtlWords * 4, 256), need = ctl_bytes + (size_t)df.num_cus * (2 * 16 + 4);
  if (ws_bytes < need) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: need %zu bytes", need);
  if (!aligned16(ws)) return fail(SOUFFLE_ERR_ALIGN, "workspace must be 16-byte aligned");
  unsigned *ctl = static_cast<unsigned *>(ws);
  u4 *buf = reinterpret_cast<u4 *>(static_cast<char *>(ws) + ctl_bytes);
  unsigned *out = reinterpret_cast<unsigned *>(static_cast<char *>(ws) + ctl_bytes + (size_t)df.num_cus * 32);
  int strict = strict_fences_mode();
  void *args[] = {&ctl, &buf, &stages, &mode, &out, &strict};
  return launch_persistent((const void *)souffle::k_stage_floor, df.num_cus, 256, args, 0, static_cast<hipStream_t>(stream));
}

extern "C" int souffle_set_cooperative_launch(int on) {
  souffle::g_cooperative.store(on ? 1 : 0);
  return SOUFFLE_OK;
}

extern "C" int souffle_set_strict_fences(int on) {
  souffle::g_strict.store(on ? 1 : 0);
  return SOUFFLE_OK;
}
extern "C" int souffle_set_swin_split(int on) {
  souffle::g_swin_split.store(on ? 1 : 0);
  return SOUFFLE_OK;
}

extern "C" int souffle_workspace_status(void *ws, souffle_stream_t stream, unsigned *flags, int clear) {
  if (!ws || !flags) return fail(SOUFFLE_ERR_NULL, "workspace and flags must not be NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned *word = static_cast<unsigned *>(ws) + kCtlErrWord;
  SOUFFLE_HIP_TRY(hipMemcpyAsync(flags, word, sizeof(unsigned), hipMemcpyDeviceToHost, st));
  SOUFFLE_HIP_TRY(hipStreamSynchronize(st));
  if (clear && *flags) {
    hipLaunchKernelGGL(k_zero_words, dim3(1), dim3(64), 0, st, word, 1);
    SOUFFLE_HIP_TRY(hipGetLastError());
  }
  return SOUFFLE_OK;
}

extern "C" int souffle_set_stage_trace(void *device_buf, size_t bytes) {
  if (device_buf && !aligned16(device_buf)) return fail(SOUFFLE_ERR_ALIGN, "trace buffer must be 16-byte aligned");
  g_trace_buf = device_buf;
  g_trace_bytes = device_buf ? bytes : 0;
  return SOUFFLE_OK;
}

extern "C" int souffle_workspace_init(void *ws, size_t bytes, souffle_stream_t stream) {
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL");
  if (!aligned16(ws)) return fail(SOUFFLE_ERR_ALIGN, "workspace must be 16-byte aligned");
  if (bytes < (size_t)kCtlWords * 4) return fail(SOUFFLE_ERR_WORKSPACE, "workspace smaller than its %d-byte control block", kCtlWords * 4);
  // The whole workspace, not only the control block: behind it live step tags (LSTM), hand-over words
  // (Swin) and not-yet-written markers that must not start from whatever the memory held before.
  // A fill kernel rather than a memset node, so that callers may capture this call.
  const size_t n16 = bytes / 16;
  const size_t want = (n16 + 255) / 256;
  hipLaunchKernelGGL(k_zero_bytes, dim3((unsigned)(want < 4096 ? want : 4096)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<u4 *>(ws), n16);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

extern "C" int souffle_gemm_f16(const void *x, const void *w, void *y, int M, int N, int K, souffle_stream_t stream) {
  if (!x || !w || !y) return fail(SOUFFLE_ERR_NULL, "x, w and y must not be NULL");
  if (!aligned16(x) || !aligned16(w) || !aligned16(y)) return fail(SOUFFLE_ERR_ALIGN, "x, w and y must be 16-byte aligned");
  if (M <= 0 || N <= 0 || K <= 0 || M % 64 || N % 64 || K % 64)
    return fail(SOUFFLE_ERR_SHAPE, "M, N and K must be positive multiples of 64 (got %d,%d,%d)", M, N, K);
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool large = M % 128 == 0 && N % 128 == 0 && (long long)(M / 128) * (N / 128) >= df.num_cus;
  if (large) return launch_gemm<GemmTile<128, 128, 64, 2, 2>>((const half_t *)x, (const half_t *)w, (half_t *)y, M, N, K, df.num_cus, st);
  return launch_gemm<GemmTile<64, 64, 64, 2, 2>>((const half_t *)x, (const half_t *)w, (half_t *)y, M, N, K, df.num_cus, st);
}

// Timing rule of the reference's benchmarkCudaFunc (cpp/souffle_utils/cuda_utils.h:102-136):
// warm up, then the minimum over rounds of the mean of `repeat` event-timed launches.
extern "C" int souffle_bench_us(int (*fn)(void *), void *arg, souffle_stream_t stream, int warmup, int rounds,
                                int repeat, double *min_of_means_us, double *median_us) {
  if (!fn) return fail(SOUFFLE_ERR_NULL, "fn is NULL");
  if (rounds <= 0 || repeat <= 0 || warmup < 0) return fail(SOUFFLE_ERR_SHAPE, "rounds and repeat must be positive");
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipEvent_t e0, e1;
  SOUFFLE_HIP_TRY(hipEventCreate(&e0));
  SOUFFLE_HIP_TRY(hipEventCreate(&e1));
  int rc = SOUFFLE_OK;
  for (int i = 0; i < warmup && rc == SOUFFLE_OK; ++i) rc = fn(arg);
  std::vector<double> means;
  for (int r = 0; r < rounds && rc == SOUFFLE_OK; ++r) {
    if (hipEventRecord(e0, st) != hipSuccess) { rc = fail(SOUFFLE_ERR_LAUNCH, "hipEventRecord failed"); break; }
    for (int i = 0; i < repeat && rc == SOUFFLE_OK; ++i) rc = fn(arg);
    if (rc != SOUFFLE_OK) break;
    if (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) { rc = fail(SOUFFLE_ERR_LAUNCH, "event record/sync failed: %s", hipGetErrorString(hipGetLastError())); break; }
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) { rc = fail(SOUFFLE_ERR_LAUNCH, "hipEventElapsedTime failed"); break; }
    means.push_back((double)ms * 1000.0 / repeat);
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != SOUFFLE_OK) return rc;
  std::sort(means.begin(), means.end());
  if (min_of_means_us) *min_of_means_us = means.front();
  if (median_us) *median_us = means[means.size() / 2];
  return SOUFFLE_OK;
}
