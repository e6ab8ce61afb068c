// fp16 MFMA GEMM tile for many rows (the MFMA-bound shapes) on gfx950.
//
// A workgroup of 256 threads computes a 256 x BN tile of Y = X.W, wave w owning rows
// [64w, 64w+64) and all BN columns (4 x BN/16 accumulator tiles).  K advances in steps of 32
// through a ring of NSTAGE LDS stages that are filled by direct global->LDS loads (no register
// staging) NSTAGE-1 steps ahead, with ONE workgroup barrier per step: with a single wave per
// SIMD nothing else hides the latency of the operand stream.
//
// LDS layouts (16-byte slots; a direct load writes 64 consecutive slots, which global 16 bytes
// each lane fetches is free, so swizzles cost nothing):
//   X stage [256 rows][32 k]: slot(r, s) = 4r + (s ^ ((r >> 1) & 3)); an operand read of 16 rows is
//            one contiguous KB and free of bank conflicts as measured (SQ_LDS_BANK_CONFLICT; a
//            swizzle that also involves bit 3 of r costs one conflict cycle per read cycle);
//   W stage [32 k][BN]:       row k is stored as LDS row wrow_of(k) (bits 2 and 3 of k swapped), slot(k, c)
//            = wrow_of(k)*BN/8 + (c ^ wswz(wrow_of(k))).  The LDS has 64 banks of 4 bytes and serves
//            the transposing read half a wave per cycle.  Half a wave touches 32 bytes of each of the
//            rows k0..k0+3 and k0+8..k0+11, i.e. LDS rows rho0..rho0+7, which must cover the 64 banks
//            once: consecutive LDS rows are 2 (BN = 144) or 6 (BN = 48) 16-byte slots apart modulo 16
//            - eight of them cover everything - or 8 (BN = 192) or 12 (BN = 96), where wswz moves the
//            rows that would coincide apart.  (Measured with SQ_LDS_BANK_CONFLICT: rows k0..k0+3 spread
//            over 32 banks only, as a 32-bank LDS would want it, cost as many conflict cycles as the
//            reads themselves, 192 per K step of a 192-column tile; what is left are the 48 per step
//            of the epilogue's stores.)
// W is row-major [K][N] as the reference stores it (cpp/bert/kernels/gemm_three_stages.h:95-131);
// the MFMA takes W as operand A and X as operand B, so a lane ends up with 4 consecutive output
// columns of one row.
// Tried and dropped, all with the same results: X straight from global memory into registers (a wave's
// 64 rows are its own, and a lane's 16 operand bytes are contiguous in the row-major X), which takes X
// out of LDS altogether: 2 % slower (12 layers at M = 4096: 1421 us against 1393).  X staged two K
// steps at a time ([256][64 k] stages, a ring of three, so that a wave-wide load takes 8 rows x 128
// bytes, whole cache lines, instead of 16 rows x 64 bytes): 2 % slower.  Eight waves of 32 x BN (two
// per SIMD): 3 % less per K step in an isolated loop.  A K step without any X traffic is 16-18 %
// shorter, and the costs of a step add up (MFMAs + X + W) whichever way the operands travel, while the
// same loads alone in a kernel run three times faster than inside the loop: fewer operand bytes per
// MAC is what helps (hence BM).
#pragma once
#include <type_traits>
#include "common.hpp"

namespace souffle {

// f(std::integral_constant<int, I>{}) for I = B .. E-1, in order: a loop whose index is a constant
// expression in the body.
template <int B, int E, class Fn>
__device__ __forceinline__ void static_for(Fn f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

// BM = 256 rows per tile, or 128 (wave w then owns rows [32w, 32w+32)): at N = 768 a 128 x 96 tile asks
// the L2 for (128 + 96) x K x 2 bytes where a 256 x 48 tile of the same area asks for (256 + 48) x K x 2.
template <int BN, int NSTAGE, int BM = 256>
struct GemmBig {
  static_assert(BM == 256 || BM == 128, "four waves of 64 or 32 rows");
  static_assert(BN % 16 == 0 && (BN * 64) % 1024 == 0, "whole MFMA tiles and whole wave-wide loads");
  static_assert(BN == 48 || BN == 96 || BN == 144 || BN == 192, "the W swizzle is worked out for these widths");
  static constexpr int kBM = BM, kBN = BN, kBK = 32;
  static constexpr int RW = BM / 4, MI = RW / 16;           // rows / accumulator row tiles per wave
  static constexpr int NT = BN / 16;                        // accumulator tiles per row block
  static constexpr int WSLOTS = BN / 8;                     // 16-byte slots per W row
  static constexpr int X_STAGE = BM * 32 * 2, W_STAGE = 32 * BN * 2, STAGE = X_STAGE + W_STAGE;
  static constexpr int LDS_BYTES = NSTAGE * STAGE;
  static constexpr int EPITCH = BN * 2 + 16;                // bytes per row of a wave's epilogue slice
  static_assert(4 * RW * EPITCH <= LDS_BYTES, "the epilogue slices fit in the ring");
  static constexpr int XI = X_STAGE / 1024, WI = W_STAGE / 1024;   // wave-wide loads per stage
  // Every wave issues LPW loads per stage: XPW of X and WPW of W.  Where WI is not a multiple of 4
  // some waves fetch a chunk a second time (same bytes to the same place): the loop stays free of
  // wave-dependent branches and every wave can use the same vmcnt.
  static constexpr int XPW = XI / 4, WPW = (WI + 3) / 4, LPW = XPW + WPW;
  static_assert(XI == BM / 16 && XI % 4 == 0, "BM rows x 32 k");
  static_assert(NSTAGE >= 4 && NSTAGE <= 6, "ring depth");
  static_assert((NSTAGE - 2) * LPW < 64, "vmcnt is a 6-bit counter");

  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;

  __device__ static __forceinline__ int wrow_of(int k) { return (k & 0x13) | ((k & 4) << 1) | ((k & 8) >> 1); }   // (its own inverse)
  __device__ static __forceinline__ int wswz(int rho) { return BN == 192 ? (((rho >> 1) & 3) << 1) : (BN == 96 ? ((rho >> 1) & 2) : 0); }

  // Load number L (0 .. LPW-1) of this wave for the stage at LDS address `stage`, K offset kk.
  // wptr(k, col) -> address of W[k][col] (col relative to the tile's first column, multiple of 8)
  template <int L, class WPtr>
  __device__ static __forceinline__ void issue_one(int tid, unsigned stage, const half_t *X, int ldx, int m0, int kk, WPtr wptr) {
    const int lane = tid & 63, wave = tid >> 6;
    if constexpr (L < XPW) {
      const int q = wave + 4 * L, r = q * 16 + (lane >> 2), sl = (lane & 3) ^ ((r >> 1) & 3);
      load_lds16(X + (size_t)(m0 + r) * ldx + kk + sl * 8, stage + q * 1024);
    } else {
      const int q = (wave + 4 * (L - XPW)) % WI, sl = q * 64 + lane, rho = sl / WSLOTS, c = (sl % WSLOTS) ^ wswz(rho);
      load_lds16(wptr(kk + wrow_of(rho), c * 8), stage + X_STAGE + q * 1024);
    }
  }
  template <int L0, int L1, class WPtr>
  __device__ static __forceinline__ void issue_range(int tid, unsigned stage, const half_t *X, int ldx, int m0, int kk, WPtr wptr) {
    if constexpr (L0 < L1) {
      issue_one<L0>(tid, stage, X, ldx, m0, kk, wptr);
      issue_range<L0 + 1, L1>(tid, stage, X, ldx, m0, kk, wptr);
    }
  }

  // All but the loads of the A most recent stages of this wave have landed.
  template <int A>
  __device__ static __forceinline__ void wait_ahead() {
    static_assert(A >= 0 && A * LPW < 64, "vmcnt is a 6-bit counter");
    wait_vmcnt<A * LPW>();
  }

  template <int KM, class Step, class A, class B, class C>
  __device__ static __forceinline__ void template_km(Step &step, int kt, A a, B b, C c) { step(kt, std::integral_constant<int, KM>{}, a, b, c); }

  // LDS read look-ahead, in column tiles: the transposing reads of tile f + D are issued before the
  // MFMAs of tile f (f counts tiles across steps).  D + 1 divides NT, so the rotating operand
  // registers are used identically in every step.
  static constexpr int D = NT % 4 == 0 ? 3 : 2;
  static_assert(NT % (D + 1) == 0, "operand register rotation");
  static constexpr int JB = NT / 2 < NT - D ? NT / 2 : NT - D;   // tile before which the step's barrier sits

  // Y[m0 .. m0+256)[tile columns] over nkt K steps starting at column k0 of X;
  // cvt(m, n, v) -> u2: the four fp16 results for v[i] = (X.W)[m][n + i] (bias, activation, residual
  // are the caller's); store16(m, n, u4): 8 consecutive results of row m from column n on; n is
  // relative to the tile's first column.
  //
  // Step kt multiplies stage kt tile by tile.  Before tile JB it waits for stage kt+1 and passes
  // the workgroup barrier (everybody is then done with stage kt-1); the reads that run ahead into
  // stage kt+1 (its X operand and first D weight tiles) come after the barrier.  The loads that
  // refill the freed buffer with stage kt+NSTAGE-1 are spread over the NT tiles that follow the
  // barrier (into the next step), a load or two per tile: a load takes the vector memory
  // pipeline of the CU 30 cycles or more and stalls the wave meanwhile, which the four MFMAs
  // issued just before it cover.  (Issued as one burst after the barrier, the loads of the four
  // waves queue up behind each other and every SIMD idles: measured 2x the time per step.)
  template <int NKT, class WPtr, class Cvt, class Store16>
  __device__ static __forceinline__ void run(unsigned char *lds, const half_t *X, int ldx, int m0, int k0, WPtr wptr, Cvt cvt, Store16 store16,
                                             const GridBarrier *tb = nullptr) {
    f4 acc[MI][NT];
    mainloop<NKT>(lds, X, ldx, m0, k0, wptr, acc, tb);
    epilogue(lds, m0, acc, cvt, store16, tb);
  }

  // The two halves of run(), for callers whose epilogue depends on a run-time choice (an activation,
  // which half of K): they branch once between two epilogue() calls.  A uniform condition tested inside
  // cvt is not hoisted by the compiler but tested per result, and the tiny basic blocks in between
  // serialise every dependent chain (FC1 with GELU: 12.8 us per tile instead of 5).
  // NKT: K steps of the tile, a compile-time multiple of NSTAGE: the steps between the first and the last NSTAGE-1
  // then run in groups of NSTAGE in which every step knows its ring stage at compile time, so that the LDS addresses
  // of a step's operand reads are a register that does not change plus an immediate.  (With the stage a run-time
  // value a step began with some forty address instructions during which no MFMA was in flight.)
  template <int NKT, class WPtr>
  __device__ static __forceinline__ void mainloop(unsigned char *lds, const half_t *X, int ldx, int m0, int k0, WPtr wptr, f4 (&acc)[MI][NT],
                                                  const GridBarrier *tb = nullptr) {
    static_assert(NKT % NSTAGE == 0 && NKT >= 2 * NSTAGE, "whole groups of steps between the first step and the last NSTAGE-1");
    const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
    STAGE_MARK(tb, 0);
    __syncthreads();                                        // the previous user of the ring is done
    const unsigned ring = lds_address(lds);
#pragma unroll
    for (int s = 0; s < NSTAGE - 1; ++s) issue_range<0, LPW>(tid, ring + s * STAGE, X, ldx, m0, k0 + s * 32, wptr);
    // (the accumulators are cleared while the first stages travel)
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < MI; ++i) mfma_pin(acc[i], true);

    // byte offsets of this lane's operand reads inside a stage
    int xoff[MI];
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const int r = wave * RW + i * 16 + l16;
      xoff[i] = r * 64 + ((g ^ ((r >> 1) & 3)) << 4);
    }
    const int rho = wrow_of(g * 8 + (l16 >> 2));             // LDS row of the first of this lane's two k rows (k, k + 4: LDS rows rho, rho + 8)
    const int wrow = X_STAGE + rho * (BN * 2) + (l16 & 1) * 8, wsw = wswz(rho), wc = (l16 & 3) >> 1;
    // slot of tile j: (2 j + wc) ^ wsw with wsw = 2 h, h < 4, i.e. 2 (j ^ h) + wc = 8 (j >> 2) + 2 ((j & 3) ^ h) + wc:
    // four per-lane offsets (one per j & 3) and a compile-time 128 bytes per j >> 2
    int woff[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) woff[q] = wrow + ((((q * 2 + wc) ^ wsw)) << 4);

    auto read_w = [&](const unsigned char *st, auto jc) {
      constexpr int j = decltype(jc)::value;
      const half_t *p = reinterpret_cast<const half_t *>(st + woff[j & 3] + (j >> 2) * 128);
      const h4 lo = lds_read_tr16(p), hh = lds_read_tr16(p + 8 * BN);
      return h8{lo[0], lo[1], lo[2], lo[3], hh[0], hh[1], hh[2], hh[3]};
    };

    h8 x[MI], xn[MI], w[D + 1];
    wait_ahead<NSTAGE - 2>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    STAGE_MARK(tb, 1);
#pragma unroll
    for (int i = 0; i < MI; ++i) x[i] = as_h8(lds_load16(lds + xoff[i]));
    static_for<0, D>([&](auto jc) { w[decltype(jc)::value] = read_w(lds, jc); });

    // One K step.  LOAD_A: the tiles before the barrier issue the rest of stage kt+NSTAGE-2;
    // LOAD_B: the tiles from the barrier on issue the first part of stage kt+NSTAGE-1;
    // AHEAD: stages requested after stage kt+1 at the time of the wait.  All compile-time so that
    // the body has no branches.
    // kmc: kt % NSTAGE as a constant
    auto step = [&](int kt, auto kmc, auto load_a, auto load_b, auto ahead_c) {
      constexpr bool LOAD_A = decltype(load_a)::value, LOAD_B = decltype(load_b)::value;
      constexpr int AHEAD = decltype(ahead_c)::value, KM = decltype(kmc)::value;
      const unsigned char *st = lds + KM * STAGE, *stn = lds + ((KM + 1) % NSTAGE) * STAGE;
      const unsigned ring_a = ring + ((KM + NSTAGE - 2) % NSTAGE) * STAGE, ring_b = ring + ((KM + NSTAGE - 1) % NSTAGE) * STAGE;
      const int kk_a = k0 + (kt + NSTAGE - 2) * 32, kk_b = kk_a + 32;
      static_for<0, NT>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        if constexpr (j == JB) {
          // stage kt+1 has landed for everybody and everybody has left stage kt-1 (a plain s_barrier:
          // no fence, the loads in flight must stay in flight)
          wait_ahead<AHEAD>();
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
#pragma unroll
          for (int i = 0; i < MI; ++i) xn[i] = as_h8(lds_load16(stn + xoff[i]));
        }
        // (in the last step these read a stale buffer; the values are never used)
        if constexpr (j + D < NT) w[(j + D) % (D + 1)] = read_w(st, std::integral_constant<int, j + D>{});
        else w[(j + D) % (D + 1)] = read_w(stn, std::integral_constant<int, j + D - NT>{});
#pragma unroll
        for (int i = 0; i < MI; ++i) {
          mfma_16x16x32_inplace(acc[i][j], w[j % (D + 1)], x[i]);
        }
        // this tile's share of the refill: slot t counts tiles from the barrier
        constexpr int t = (j - JB + NT) % NT, L0 = t * LPW / NT, L1 = (t + 1) * LPW / NT;
        if constexpr (j >= JB) {
          if constexpr (LOAD_B) issue_range<L0, L1>(tid, ring_b, X, ldx, m0, kk_b, wptr);
        } else {
          if constexpr (LOAD_A) issue_range<L0, L1>(tid, ring_a, X, ldx, m0, kk_a, wptr);
        }
      });
#pragma unroll
      for (int i = 0; i < MI; ++i) x[i] = xn[i];
    };
    using T = std::true_type;
    using F = std::false_type;
    // Stages 0 .. NSTAGE-2 were requested above.
    constexpr int main_end = NKT - (NSTAGE - 1);           // steps 1 .. main_end-1 request on both sides of the barrier
    static_assert((main_end - 1) % NSTAGE == 0, "whole groups");
    template_km<0>(step, 0, F{}, T{}, std::integral_constant<int, NSTAGE - 3>{});
    for (int kt = 1; kt < main_end; kt += NSTAGE)
      static_for<0, NSTAGE>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        template_km<(1 + i) % NSTAGE>(step, kt + i, T{}, T{}, std::integral_constant<int, NSTAGE - 3>{});
      });
    // the last NSTAGE-1 steps: the first still completes stage NKT-1; after stage kt+1 there are
    // NSTAGE-3, ..., 1, 0, 0 stages in flight
    template_km<(main_end + 0) % NSTAGE>(step, main_end + 0, T{}, F{}, std::integral_constant<int, (NSTAGE - 3 > 0 ? NSTAGE - 3 : 0)>{});
    template_km<(main_end + 1) % NSTAGE>(step, main_end + 1, F{}, F{}, std::integral_constant<int, (NSTAGE - 4 > 0 ? NSTAGE - 4 : 0)>{});
    template_km<(main_end + 2) % NSTAGE>(step, main_end + 2, F{}, F{}, std::integral_constant<int, (NSTAGE - 5 > 0 ? NSTAGE - 5 : 0)>{});
    if constexpr (NSTAGE >= 5) template_km<(main_end + 3) % NSTAGE>(step, main_end + 3, F{}, F{}, std::integral_constant<int, (NSTAGE - 6 > 0 ? NSTAGE - 6 : 0)>{});
    if constexpr (NSTAGE >= 6) template_km<(main_end + 4) % NSTAGE>(step, main_end + 4, F{}, F{}, std::integral_constant<int, 0>{});
#pragma unroll
    for (int i = 0; i < MI; ++i) mfma_pin(acc[i], false);
    STAGE_MARK(tb, 2);
  }

  template <class Cvt, class Store16>
  __device__ static __forceinline__ void epilogue(unsigned char *lds, int m0, f4 (&acc)[MI][NT], Cvt cvt, Store16 store16, const GridBarrier *tb = nullptr) {
    epilogue_rowvec(lds, m0, acc, [](int) { return h4{(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f}; },
                    [&](int m, int n, f4 v, h4) { return cvt(m, n, v); }, store16, tb);
  }
  // The same with a per-column vector (a bias) that the conversion adds: vec_at(n) -> the four values for columns
  // n .. n + 3 (relative to the tile's first column), fetched for all of a lane's column groups at once before the first
  // conversion, so that the epilogue waits for memory once and not once per accumulator tile;
  // cvt(m, n, v, vec) -> u2.
  template <class VecAt, class Cvt, class Store16>
  __device__ static __forceinline__ void epilogue_rowvec(unsigned char *lds, int m0, f4 (&acc)[MI][NT], VecAt vec_at, Cvt cvt, Store16 store16,
                                                         const GridBarrier *tb = nullptr) {
    const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
    h4 vec[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) vec[j] = vec_at(j * 16 + g * 4);
    // Epilogue.  A lane holds 4 consecutive columns of 16 rows per accumulator tile; stored
    // directly that would be 8-byte pieces of 32-byte row segments.  The converted tile instead
    // goes through the wave's own slice of the (now idle) ring, and leaves as 16 bytes per lane
    // along whole rows.  It does so in ECH groups of columns: the stores of a group (which the
    // memory system takes at its own pace, 3 us for the 98 KB of an FC1 tile when every workgroup
    // stores at once) drain while the next group is converted.
    __syncthreads();                                        // every wave has left the ring
    unsigned char *mine = lds + wave * (RW * EPITCH);
    constexpr int ECH = (NT % 3 == 0 && BN >= 144) ? 3 : (BN == 96 ? 2 : 1);
    constexpr int TPC = NT / ECH, CPC = TPC * 2;             // accumulator tiles / 16-byte chunks per row and group
    static_for<0, ECH>([&](auto chc) {
      constexpr int ch = decltype(chc)::value;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = ch * TPC; j < (ch + 1) * TPC; ++j)
          lds_store8(mine + (i * 16 + l16) * EPITCH + (j * 16 + g * 4) * 2, cvt(m0 + wave * RW + i * 16 + l16, j * 16 + g * 4, acc[i][j], vec[j]));
      if constexpr (ch == ECH - 1) STAGE_MARK(tb, 3);
      static_assert((RW * CPC) % 64 == 0, "whole wave-wide stores");
#pragma unroll
      for (int t = 0; t < RW * CPC / 64; ++t) {              // RW rows x CPC chunks, 64 per pass
        const int c = t * 64 + lane, row = c / CPC, col8 = ch * CPC + c % CPC;
        const u4 v = lds_load16(mine + row * EPITCH + col8 * 16);
        store16(m0 + wave * RW + row, col8 * 8, v);
      }
    });
    STAGE_MARK(tb, 4);
#ifdef SOUFFLE_STAGE_MARKS
    if (tb && tb->trace) { __builtin_amdgcn_s_waitcnt(0); trace_mark(*tb, 5); }
#endif
  }
};

}  // namespace souffle
