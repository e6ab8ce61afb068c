// LDS-staged, double-buffered fp16 MFMA GEMM tile for gfx950.
//
// One workgroup of 256 threads (4 waves arranged WAVES_M x WAVES_N) computes a
// BM x BN tile of Y = X.W over a K range, X row-major [M][K] (fetched through a
// caller-supplied loader so that LayerNorm-on-load or gathers can be fused), W
// row-major [K][N] exactly as the reference stores it
// (cpp/bert/kernels/gemm_three_stages.h:95-131).
//
// The MFMA is issued with the weight tile as the A operand and the activation tile as
// the B operand, so every lane ends up with 4 consecutive output columns of one output
// row and the epilogue can store 8 bytes of a row-major result per lane.  The weight
// operand (k-vector per column) is produced from the row-major LDS tile by the
// transposing LDS read, so W needs no repacking.
#pragma once
#include "common.hpp"

namespace souffle {

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
struct GemmTile {
  static_assert(WAVES_M * WAVES_N == 4, "256 threads = 4 waves");
  static_assert(BK % 32 == 0 && BM % (16 * WAVES_M) == 0 && BN % (16 * WAVES_N) == 0, "tile shape");
  static constexpr int kBM = BM, kBN = BN, kBK = BK;
  static constexpr int NT = 256;
  static constexpr int XLD = BK + 8;                       // halves per X row in LDS
  static constexpr int WPAD = (BN % 128 == 0) ? 16 : (BN % 64 == 0 ? 8 : 0);
  static constexpr int WLD = BN + WPAD;                    // halves per W row in LDS
  static constexpr int STAGE_HALVES = BM * XLD + BK * WLD;
  static constexpr int LDS_BYTES = 2 * STAGE_HALVES * 2;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 16, TN = WTN / 16;
  static constexpr int XG = BM * BK / 8, WG = BK * BN / 8;  // 16-byte granules per stage
  static constexpr int GX = (XG + NT - 1) / NT, GW = (WG + NT - 1) / NT;

  // aload(m, k)  -> u4 : the 8 halves X[m][k..k+7]
  // epi(m, n, v)       : v[i] = Y[m][n+i], i = 0..3
  template <class ALoad, class Epi>
  __device__ static __forceinline__ void run(half_t *lds, const half_t *__restrict__ W, int ldw,
                                             int m0, int n0, int k0, int nkt, ALoad aload, Epi epi) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;

    f4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

    u4 xr[GX], wr[GW];
    auto gload = [&](int kt) {
      const int kb = k0 + kt * BK;
#pragma unroll
      for (int i = 0; i < GX; ++i) {
        const int id = tid + i * NT;
        if (XG % NT == 0 || id < XG) xr[i] = aload(m0 + id / (BK / 8), kb + (id % (BK / 8)) * 8);
      }
#pragma unroll
      for (int i = 0; i < GW; ++i) {
        const int id = tid + i * NT;
        if (WG % NT == 0 || id < WG)
          wr[i] = *reinterpret_cast<const u4 *>(W + (size_t)(kb + id / (BN / 8)) * ldw + n0 + (id % (BN / 8)) * 8);
      }
    };
    auto sstore = [&](int buf) {
      half_t *xs = lds + buf * STAGE_HALVES, *ws = xs + BM * XLD;
#pragma unroll
      for (int i = 0; i < GX; ++i) {
        const int id = tid + i * NT;
        if (XG % NT == 0 || id < XG)
          *reinterpret_cast<u4 *>(xs + (id / (BK / 8)) * XLD + (id % (BK / 8)) * 8) = xr[i];
      }
#pragma unroll
      for (int i = 0; i < GW; ++i) {
        const int id = tid + i * NT;
        if (WG % NT == 0 || id < WG)
          *reinterpret_cast<u4 *>(ws + (id / (BN / 8)) * WLD + (id % (BN / 8)) * 8) = wr[i];
      }
    };

    gload(0);
    __syncthreads();          // previous user of the LDS stages is done
    sstore(0);
    __syncthreads();
    for (int kt = 0; kt < nkt; ++kt) {
      if (kt + 1 < nkt) gload(kt + 1);
      const half_t *xs = lds + (kt & 1) * STAGE_HALVES, *ws = xs + BM * XLD;
#pragma unroll
      for (int ks = 0; ks < BK / 32; ++ks) {
        h8 xop[TM], wop[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
          xop[i] = *reinterpret_cast<const h8 *>(xs + (wm0 + i * 16 + l16) * XLD + ks * 32 + g * 8);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const half_t *p = ws + (ks * 32 + g * 8 + (l16 >> 2)) * WLD + wn0 + j * 16 + (l16 & 3) * 4;
          const h4 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 4 * WLD);
          wop[j] = h8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = mfma_16x16x32(wop[j], xop[i], acc[i][j]);
      }
      if (kt + 1 < nkt) sstore((kt + 1) & 1);
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        epi(m0 + wm0 + i * 16 + l16, n0 + wn0 + j * 16 + g * 4, acc[i][j]);
  }
};

}  // namespace souffle
