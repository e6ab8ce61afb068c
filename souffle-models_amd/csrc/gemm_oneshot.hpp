// "One-shot" fp16 MFMA GEMM item for skinny problems (few rows, weight-stream bound).
//
// A workgroup of 256 threads computes a BM x 64 tile of Y = X.W over a K slice of KS.
// Both operand slices fit in LDS, so ALL of their loads are issued at once with the
// direct global->LDS instruction (no register staging, ~100 KB in flight per CU): the item
// costs one memory latency instead of one per K step.  This matters because at M = 128
// every stage of the encoder is latency bound.
//
// LDS layouts are unpadded (the direct load writes 64 consecutive 16-byte slots per wave
// instruction) and XOR-swizzled at slot granularity instead:
//   X slice [BM][KS]: slot(r, j) = r*KS/8 + (j ^ (r & 15))   16 rows of one k-granule -> 16 banks groups
//   W slice [KS][64]: slot(k, c) = k*8    + (c ^ (k & 2))    4 rows of a transposing read -> 4 bank groups
// W stays row-major [K][N] as the reference stores it; the k-vector operand comes from the
// transposing LDS read.  The MFMA takes W as operand A and X as operand B so that a lane
// holds 4 consecutive output columns of one row.
#pragma once
#include "common.hpp"

namespace souffle {

template <int BM, int KS>
struct GemmOneShot {
  static_assert(KS % 128 == 0, "the X swizzle needs whole groups of 16 slots per row");
  static_assert(BM == 32 || BM == 64 || BM == 128, "tile rows");
  static constexpr int kBM = BM, kBN = 64, kKS = KS;
  static constexpr int XGR = KS / 8;                               // 16-byte slots per X row
  static constexpr int X_BYTES = BM * KS * 2, W_BYTES = KS * 64 * 2;
  static constexpr int LDS_BYTES = X_BYTES + W_BYTES;
  static constexpr int X_INSTR = X_BYTES / 1024, W_INSTR = W_BYTES / 1024;   // wave-wide loads
  static constexpr int WAVES_M = BM == 32 ? 1 : 2, WAVES_N = 4 / WAVES_M;
  static constexpr int WTM = BM / WAVES_M, WTN = 64 / WAVES_N, TM = WTM / 16, TN = WTN / 16;

  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;

  // Queue the loads of W[k0 .. k0+KS)[n0 .. n0+64) (plain cached loads: weights are never written).
  __device__ static __forceinline__ void issue_w(unsigned char *lds_w, const half_t *__restrict__ W, int ldw, int n0, int k0) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int q = 0; q < W_INSTR / 4; ++q) {
      const int inst = q * 4 + wave, s = inst * 64 + lane, k = s >> 3, c = (s & 7) ^ (k & 2);
      __builtin_amdgcn_global_load_lds((gptr_t)(W + (size_t)(k0 + k) * ldw + n0 + c * 8), (lptr_t)(lds_w + inst * 1024), 16, 0, 0);
    }
  }
  // Queue the loads of X[m0 .. m0+BM)[k0 .. k0+KS); COH selects agent-coherent loads.
  template <bool COH>
  __device__ static __forceinline__ void issue_x(unsigned char *lds_x, const half_t *X, int ldx, int m0, int k0) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
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

  // epi(m, n, v): v[i] = sum over the slice of X[m][k] W[k][n+i]; m, n relative to the tile origin.
  template <class Epi>
  __device__ static __forceinline__ void compute(const unsigned char *lds_x, const unsigned char *lds_w, Epi epi) {
    const half_t *xs = reinterpret_cast<const half_t *>(lds_x), *ws = reinterpret_cast<const half_t *>(lds_w);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l16 = lane & 15, g = lane >> 4;
    const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
    f4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int ks = 0; ks < KS / 32; ++ks) {
      h8 xop[TM], wop[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int r = wm0 + i * 16 + l16;
        xop[i] = *reinterpret_cast<const h8 *>(xs + (r * XGR + ((ks * 4 + g) ^ (r & 15))) * 8);
      }
      const int k = ks * 32 + g * 8 + (l16 >> 2);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int c = ((wn0 + j * 16) >> 3) + ((l16 & 3) >> 1);
        const half_t *p = ws + (k * 8 + (c ^ (k & 2))) * 8 + (l16 & 1) * 4;
        const h4 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 4 * 64);
        wop[j] = h8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = mfma_16x16x32(wop[j], xop[i], acc[i][j]);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) epi(wm0 + i * 16 + l16, wn0 + j * 16 + g * 4, acc[i][j]);
  }
};

}  // namespace souffle
