// "One-shot" fp16 MFMA GEMM item for skinny problems (few rows, weight-stream bound).
//
// A workgroup of 256 threads computes a BM x 64 tile of Y = X.W over a K slice of KS.
// Both operand slices fit in LDS, so ALL of their loads are queued at once with the direct
// global->LDS instruction (no register staging, ~100 KB in flight per CU): an item costs
// one memory latency instead of one per K step, and the weight slice of the NEXT stage can
// be queued inside a grid barrier and land while the barrier completes.
//
// LDS layouts are unpadded (the direct load writes 64 consecutive 16-byte slots per wave
// instruction) and XOR-swizzled at slot granularity instead:
//   X slice [BM][KS]: slot(r, j) = r*KS/8 + (j ^ (r & 15))   16 rows of one k-granule -> 16 bank groups
//   W slice [KS][64]: slot(k, c) = k*8    + (c ^ (k & 2))    4 rows of a transposing read -> 4 bank groups
//                     (The LDS has 64 banks and serves the transposing read half a wave per cycle, so rows k and
//                     k+8 collide: 384 conflict cycles per item.  XOR with (k & 2) | ((k & 8) >> 1) removes them
//                     and changes nothing measurable: the 12-layer encoder at 128 rows is bound by the latency
//                     of its chain of stages, cold 326.6-327.5 us either way, warm 0.7 % slower.)
// W stays row-major [K][N] as the reference stores it; the k-vector operand comes from the
// transposing LDS read.  The MFMA takes W as operand A and X as operand B so that a lane
// holds 4 consecutive output columns of one row.
//
// The four waves split the tile as WAVES_M row blocks of 32 x WAVES_K slices of K; every
// wave owns all 64 columns (8 independent accumulators, fully unrolled K loop), the K
// slices are summed through a padded fp32 buffer in LDS, and the epilogue then runs with 8
// or 16 consecutive columns of one row per thread.
#pragma once
#include "common.hpp"

namespace souffle {

template <int BM, int KS>
struct GemmOneShot {
  static_assert(KS % 128 == 0, "the X swizzle needs whole groups of 16 slots per row");
  static_assert(BM == 32 || BM == 64, "tile rows");
  static constexpr int kBM = BM, kBN = 64, kKS = KS;
  static constexpr int XGR = KS / 8;                               // 16-byte slots per X row
  static constexpr int X_BYTES = BM * KS * 2, W_BYTES = KS * 64 * 2;
  static constexpr int X_INSTR = X_BYTES / 1024, W_INSTR = W_BYTES / 1024;   // wave-wide loads
  static constexpr int WAVES_M = BM / 32, WAVES_K = 4 / WAVES_M;
  static constexpr int KSTEPS = KS / 32 / WAVES_K;                 // MFMA k-steps per wave
  static_assert((KS / 32) % WAVES_K == 0, "K slice must split evenly over the waves");
  static constexpr int RED_LD = 68;                                // floats per row of the reduction buffer
  static constexpr int RED_BYTES = WAVES_K * BM * RED_LD * 4;
  static_assert(RED_BYTES <= X_BYTES, "the reduction buffer reuses the X region");
  static constexpr int CPT = BM * 64 / 256;                        // output columns per thread in the epilogue

  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;

  // The lane id as a value the optimiser cannot see through: keeps the dozens of per-load
  // addresses from being hoisted out of the layer loop (and spilled) in the megakernel.
  __device__ static __forceinline__ int opaque_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
  }
  // Queue the loads of W[k0 .. k0+KS)[n0 .. n0+64) (plain cached loads: weights are never written).
  // `rot` rotates the order in which the rows are requested: workgroups of one XCD that load
  // the same slice start at different rows, so at any moment they ask their L2 for different
  // lines and everybody but the first requester of a line hits.
  __device__ static __forceinline__ void issue_w(unsigned char *lds_w, const half_t *__restrict__ W, int ldw, int n0, int k0, int rot = 0) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int q0 = 0; q0 < W_INSTR / 4; ++q0) {
      int q = q0 + rot;
      if (q >= W_INSTR / 4) q -= W_INSTR / 4;
      const int inst = q * 4 + wave, s = inst * 64 + lane, k = s >> 3, c = (s & 7) ^ (k & 2);
      __builtin_amdgcn_global_load_lds((gptr_t)(W + (size_t)(k0 + k) * ldw + n0 + c * 8), (lptr_t)(lds_w + inst * 1024), 16, 0, 0);
    }
  }
  // The same slice queued by waves 1..3 only (PREFETCH_INSTR loads each): wave 0 polls the grid
  // barrier, and its polling loads must not queue up behind a weight slice that is still in flight.
  static constexpr int PREFETCH_INSTR = W_INSTR / 3;
  static_assert(W_INSTR % 3 == 0 && PREFETCH_INSTR < 64, "prefetch split over three waves");
  __device__ static __forceinline__ void issue_w_prefetch(unsigned char *lds_w, const half_t *__restrict__ W, int ldw, int n0, int k0, int rot = 0) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    if (wave == 0) return;
#pragma unroll
    for (int q0 = 0; q0 < PREFETCH_INSTR; ++q0) {
      int q = q0 + (rot * 4) / 3;
      if (q >= PREFETCH_INSTR) q -= PREFETCH_INSTR;
      const int inst = q * 3 + wave - 1, s = inst * 64 + lane, k = s >> 3, c = (s & 7) ^ (k & 2);
      __builtin_amdgcn_global_load_lds((gptr_t)(W + (size_t)(k0 + k) * ldw + n0 + c * 8), (lptr_t)(lds_w + inst * 1024), 16, 0, 0);
    }
  }
  // Queue the loads of X[m0 .. m0+BM)[k0 .. k0+KS); COH selects agent-coherent loads.
  template <bool COH>
  __device__ static __forceinline__ void issue_x(unsigned char *lds_x, const half_t *X, int ldx, int m0, int k0) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int q = 0; q < X_INSTR / 4; ++q) {
      const int inst = q * 4 + wave, s = inst * 64 + lane, r = s / XGR, j = (s % XGR) ^ (r & 15);
      __builtin_amdgcn_global_load_lds((gptr_t)(X + (size_t)(m0 + r) * ldx + k0 + j * 8), (lptr_t)(lds_x + inst * 1024), 16, 0,
                                       COH ? kAuxSc1 : 0);
    }
  }
  // All queued loads of this wave have landed, and (after the barrier) everybody's.
  __device__ static __forceinline__ void wait_loads() {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  }

  // MFMA over this wave's share of the slice; then every wave is done reading X and W, the
  // partial tiles are summed through the X region, and epi(m, n, lo, hi) is called with
  // lo[i] = Y[m][n+i], hi[i] = Y[m][n+4+i], i = 0..3 (8 consecutive columns of one row, m and n
  // relative to the tile origin), CPT/8 times per thread.
  // On return the W region is free (new loads may be queued into it).
  template <class Epi>
  __device__ static __forceinline__ void compute(unsigned char *lds_x, const unsigned char *lds_w, Epi epi) {
    const half_t *xs = reinterpret_cast<const half_t *>(lds_x), *ws = reinterpret_cast<const half_t *>(lds_w);
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
    const int wm = wave / WAVES_K, wk = wave % WAVES_K;
    f4 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int ks = wk * KSTEPS + s;
      h8 xop[2], wop[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int r = wm * 32 + i * 16 + l16;
        xop[i] = *reinterpret_cast<const h8 *>(xs + (r * XGR + ((ks * 4 + g) ^ (r & 15))) * 8);
      }
      const int k = ks * 32 + g * 8 + (l16 >> 2);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int c = j * 2 + ((l16 & 3) >> 1);
        const half_t *p = ws + (k * 8 + (c ^ (k & 2))) * 8 + (l16 & 1) * 4;
        const h4 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 4 * 64);
        wop[j] = h8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma_16x16x32(wop[j], xop[i], acc[i][j]);
    }
    __syncthreads();                       // X and W slices are dead from here on
    float *red = reinterpret_cast<float *>(lds_x);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *reinterpret_cast<f4 *>(red + (wk * BM + wm * 32 + i * 16 + l16) * RED_LD + j * 16 + g * 4) = acc[i][j];
    __syncthreads();
    constexpr int TPR = 64 / CPT;           // threads per output row
    const int row = tid / TPR, col0 = (tid % TPR) * CPT;
#pragma unroll
    for (int c = 0; c < CPT / 8; ++c) {
      const float *src = red + row * RED_LD + col0 + c * 8;
      f4 lo = *reinterpret_cast<const f4 *>(src), hi = *reinterpret_cast<const f4 *>(src + 4);
#pragma unroll
      for (int w = 1; w < WAVES_K; ++w) {
        lo += *reinterpret_cast<const f4 *>(src + w * BM * RED_LD);
        hi += *reinterpret_cast<const f4 *>(src + w * BM * RED_LD + 4);
      }
      epi(row, col0 + c * 8, lo, hi);
    }
  }
};

}  // namespace souffle
