// BERT-base encoder layer(s) on gfx950: a persistent cooperative megakernel (all stages
// of all layers in one launch, grid barriers between stages) and the same stages as
// separate launches (the unfused per-op baseline).
//
// Stage list per layer (reference counterparts in brackets):
//   1 QKV GEMM + bias + head split        [cpp/bert/kernels/fused_sqq_bert.cu:2333-2765]
//   2 scores, scale, mask, softmax, P.V   [fused_sqq_bert.cu:2772-3329]  (P never leaves the CU)
//   3 out-projection, split-K partials    [fused_sqq_bert.cu:3334-3687]
//   4 reduce + bias + residual + LN1      [fused_sqq_bert.cu:3690-3782]
//   5 FC1 + bias + activation             [cpp/bert/kernels/fused_sqq_feedforward.cu:38-362]
//   6 FC2, split-K partials               [fused_sqq_feedforward.cu:368-835]
//   7 reduce + bias + residual + LN2      [fused_sqq_feedforward.cu:368-835]
// Softmax is max-subtracted fp32 and LayerNorm is two-pass fp32 in registers, with a
// fixed summation order (no float atomics), so results are run-to-run identical.
#include <type_traits>
#include "gemm_oneshot.hpp"
#include "gemm_tile.hpp"
#include "gemm_big.hpp"
#include "host_util.hpp"

namespace souffle {
namespace bert {

constexpr int H = 768, NH = 12, HD = 64, F = 3072;
#ifndef SOUFFLE_ROWBLOCK_LOCAL
#define SOUFFLE_ROWBLOCK_LOCAL 1
#endif
constexpr bool kRowblockLocal = SOUFFLE_ROWBLOCK_LOCAL != 0;   // many rows: hand-overs among the 16 tiles of a row block instead of grid barriers

constexpr int kMaxLayers = 24;
constexpr int kMaxSplitK = 8;

struct LayerW {
  const half_t *w_qkv, *b_qkv, *w_o, *b_o, *ln1_g, *ln1_b, *w_fc1, *b_fc1, *w_fc2, *b_fc2, *ln2_g, *ln2_b;
};

// Per-launch parameters.  The inter-stage buffers (qkv .. yl) are given per layer
// (`layer_stride` bytes apart) so that inside one launch every address is written by exactly
// one stage of one layer and read only afterwards: readers can then use ordinary cached
// loads (an XCD's L2 never holds an older version of a line) and each XCD fetches a line of
// an activation once instead of every workgroup fetching it from memory.
// The many-rows megakernel (82 MB of such buffers per layer at 4096 rows) rotates through
// `layer_sets` sets instead, which stay in the memory-side cache, and restores the property at
// the hand-over (or barrier) that ends a layer: one wave of every workgroup invalidates its L1 and its
// XCD's L2 (an agent-scope acquire fence) after arriving and before it polls, so the invalidation has
// been performed when the poll returns.  In the last stage of a layer nobody reads a buffer that a later
// layer writes before reading, so no line dropped there can come back in an old version; with
// hand-overs per row block the same holds per row block, whose rows only its own workgroups read.
struct Params {
  int B, S, M, act, num_layers, splitk_o, splitk_f;
  int big;             // rows are a multiple of 256 and many: the 256-row GEMM tiles are used
  float scale, eps;
  const half_t *x, *mask;
  half_t *y;
  half_t *qkv, *ctx, *z1, *y1, *h, *yl, *probs;
  float *part;
  unsigned *ctl;
  unsigned *rbflags;   // many-rows megakernel: 16 hand-over words per 256-row block (see rowblock_ln)
  unsigned long long *trace;
  int trace_cap;
  size_t layer_stride;
  int layer_sets;      // layer l uses buffer set l % layer_sets
  // dataflow kernel: bytes of one layer's buffers from `qkv` up to (not including) `yl`, and the
  // marker the control block holds while all buffers of this layout are in the unwritten state
  size_t flow_bytes;
  unsigned flow_marker;
};
struct Args : Params {
  LayerW layers[kMaxLayers];
};

__device__ __forceinline__ Params layer_params(const Params &a, int l) {
  Params p = a;
  const size_t off = (size_t)(l % a.layer_sets) * a.layer_stride;
  auto adv = [&](half_t *q) { return uniform_ptr(reinterpret_cast<half_t *>(reinterpret_cast<char *>(q) + off)); };
  p.qkv = adv(a.qkv); p.ctx = adv(a.ctx); p.z1 = adv(a.z1); p.y1 = adv(a.y1); p.h = adv(a.h); p.yl = adv(a.yl);
  p.part = uniform_ptr(reinterpret_cast<float *>(reinterpret_cast<char *>(a.part) + off));
  return p;
}

// ---- dataflow synchronisation (skinny path) ----
// Instead of a grid barrier between stages, a consumer polls the data it needs.  Every
// inter-stage buffer holds the pattern 0xffffffff in each 32-bit word (two fp16 NaNs that no
// conversion from fp32 produces, or an fp32 NaN no arithmetic here produces) until its producer
// has written it; producers write through (sc1), consumers load with sc1 straight from the
// memory side and re-request whatever still shows the pattern.  One load round trip thus both
// detects and fetches the data; there is no arrival counter, no flag and no wait for store
// acknowledgements on the critical path.  Waits are bounded: after kMaxFlowSpin retries the
// workgroup gives up, flags the control block and stops waiting for the rest of the launch.
constexpr int kMaxFlowSpin = 1 << 15;
struct Flow {
  bool failed;
  unsigned long long *trace;   // optional stamps, same layout as the barrier trace: (ready, done) per stage
  int trace_cap, stage;
};
__device__ __forceinline__ void flow_stamp(Flow &fl, int which) {
  if (fl.trace && fl.stage < fl.trace_cap && threadIdx.x == 0)
    fl.trace[(size_t)(2 * fl.stage + which) * gridDim.x + blockIdx.x] = wall_clock64();
}
__device__ __forceinline__ bool has_unwritten(u4 v) {
  return (v[0] == ~0u) | (v[1] == ~0u) | (v[2] == ~0u) | (v[3] == ~0u);
}
__device__ __forceinline__ bool has_unwritten(u2 v) { return (v[0] == ~0u) | (v[1] == ~0u); }

// A wave fetches N direct-to-LDS loads (issue(i): load i, 64 lanes x 16 bytes; slot(i): where this
// lane's 16 bytes of load i land).  Loads in PROBE are repeated until none of their lanes sees
// the pattern; only then are the others requested, and repeated individually while incomplete.
// The probe loads are chosen to touch the last rows of the producers the wave depends on, so
// that waiting costs a few KB per round trip and not the whole operand (polling the whole
// operand from every waiting workgroup saturates the fabric and delays the very stores it waits for).
template <int N, unsigned long long PROBE, class Issue, class Slot>
__device__ __forceinline__ void poll_direct_loads(Issue issue, Slot slot, Flow &fl) {
  static_assert(N >= 1 && N <= 64, "one mask bit per load");
  constexpr unsigned long long ALL = N == 64 ? ~0ull : ((1ull << N) - 1);
  static_assert(PROBE != 0 && (PROBE & ~ALL) == 0, "probe loads are a non-empty subset");
  unsigned long long pending = PROBE;
  bool rest_issued = false;
#pragma unroll
  for (int i = 0; i < N; ++i)
    if ((PROBE >> i) & 1) issue(i);
  for (int spin = 0;; ++spin) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unsigned long long still = 0;
#pragma unroll
    for (int i = 0; i < N; ++i)
      if ((pending >> i) & 1) {
        const u4 v = *reinterpret_cast<const u4 *>(slot(i));
        if (__any(has_unwritten(v))) still |= 1ull << i;
      }
    if (fl.failed || spin >= kMaxFlowSpin) { fl.failed = true; still = 0; }
    if (!still) {
      if (rest_issued || PROBE == ALL) return;
      rest_issued = true;
      still = ALL & ~PROBE;
    }
#pragma unroll
    for (int i = 0; i < N; ++i)
      if ((still >> i) & 1) issue(i);
    pending = still;
  }
}

// The X slice of a one-shot GEMM item, polled (layout as GemmOneShot::issue_x).
template <class G>
__device__ __forceinline__ void poll_x(unsigned char *lds_x, const half_t *X, int ldx, int m0, int k0, Flow &fl) {
  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;
  const int tid = G::opaque_tid(), lane = tid & 63, wave = tid >> 6;
  auto issue = [&](int q) {
    const int inst = q * 4 + wave, sl = inst * 64 + lane, r = sl / G::XGR, j = (sl % G::XGR) ^ (r & 15);
    __builtin_amdgcn_global_load_lds((gptr_t)(X + (size_t)(m0 + r) * ldx + k0 + j * 8), (lptr_t)(lds_x + inst * 1024), 16, 0, kAuxSc1);
  };
  auto slot = [&](int q) { return lds_x + (q * 4 + wave) * 1024 + lane * 16; };
  // Everything is requested at once.  (Waiting on a probe first - this wave's last load, which lies in
  // the last rows of the slice - costs a second memory round trip once the data is there: measured
  // 378 us against 350 us for the 12-layer encoder.)
  constexpr int PER = G::X_INSTR / 4;
  poll_direct_loads<PER, (1ull << PER) - 1>(issue, slot, fl);
}

// ------------------------------------------------------------------ stages ----
// Stands in for a bias the caller did not give, where a test per result would cost more than adding zeros.
__device__ const half_t g_zero_row[F] = {};
__device__ __forceinline__ f4 add_row4(f4 v, const half_t *row, int n) {
  const h4 bb = ldg<h4>(row + n);
  return v + f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
}
__device__ __forceinline__ f4 add_bias4(f4 v, const half_t *bias, int n) {
  if (bias) {
    const h4 bb = ldg<h4>(bias + n);
    v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
  }
  return v;
}

__device__ __forceinline__ void add_bias8(f4 &lo, f4 &hi, const half_t *bias, int n) {
  if (bias) {
    const h8 bb = ldg<h8>(bias + n);
    lo += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
    hi += f4{(float)bb[4], (float)bb[5], (float)bb[6], (float)bb[7]};
  }
}
__device__ __forceinline__ u4 pack_h8(f4 lo, f4 hi) {
  const h8 r = {(half_t)lo[0], (half_t)lo[1], (half_t)lo[2], (half_t)lo[3], (half_t)hi[0], (half_t)hi[1], (half_t)hi[2], (half_t)hi[3]};
  return as_u4(r);
}


template <bool COH, class Tile>
__device__ __forceinline__ void stage_qkv(half_t *lds, const Params &a, const LayerW &w, const half_t *xin,
                                          int first, int stride) {
  constexpr int BM = Tile::kBM, BN = Tile::kBN, BK = Tile::kBK;
  const int tiles_n = 3 * H / BN, items = (a.M / BM) * tiles_n;
  for (int item = first; item < items; item += stride) {
    const int tm = item / tiles_n, n0 = (item % tiles_n) * BN, j = n0 / H, nn0 = n0 % H;
    auto aload = [&](int m, int k) { return ld16<false>(xin, (m * H + k) * 2); };
    auto epi = [&](int m, int n, f4 v) {
      if (w.b_qkv) {
        const h4 bb = ldg<h4>(w.b_qkv + j * H + n);
        v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      const int b = m / a.S, s = m % a.S, hh = n / HD, d = n % HD;
      st8<COH>(a.qkv, ((((j * a.B + b) * NH + hh) * a.S + s) * HD + d) * 2, pack_h4(v));
    };
    Tile::run(lds, w.w_qkv + (size_t)j * H * H, H, tm * BM, nn0, 0, H / BK, aload, epi);
  }
}

// Y = act(X.W + b), fp16 out (FC1).
template <bool COH, class Tile>
__device__ __forceinline__ void stage_fc1(half_t *lds, const Params &a, const LayerW &w, int first, int stride) {
  constexpr int BM = Tile::kBM, BN = Tile::kBN, BK = Tile::kBK;
  const int tiles_n = F / BN, items = (a.M / BM) * tiles_n;
  for (int item = first; item < items; item += stride) {
    const int tm = item / tiles_n, n0 = (item % tiles_n) * BN;
    auto aload = [&](int m, int k) { return ld16<false>(a.y1, (m * H + k) * 2); };
    auto epi = [&](int m, int n, f4 v) {
      if (w.b_fc1) {
        const h4 bb = ldg<h4>(w.b_fc1 + n);
        v += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      if (a.act == SOUFFLE_ACT_RELU) {            // (one test per group of results, not one per result)
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = fmaxf(v[i], 0.f);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = gelu_tanh(v[i]);
      }
      st8<COH>(a.h, (m * F + n) * 2, pack_h4(v));
    };
    Tile::run(lds, w.w_fc1, F, tm * BM, n0, 0, H / BK, aload, epi);
  }
}

// fp32 split-K partials of X[M][K].W[K][H]: part[ks][m][n].
template <bool COH, class Tile>
__device__ __forceinline__ void stage_partial(half_t *lds, const Params &a, const half_t *X, int K,
                                              const half_t *W, int splitk, int first, int stride) {
  constexpr int BM = Tile::kBM, BN = Tile::kBN, BK = Tile::kBK;
  const int tiles_n = H / BN, items = (a.M / BM) * tiles_n * splitk, kper = K / splitk;
  for (int item = first; item < items; item += stride) {
    const int ks = item % splitk, t = item / splitk, tm = t / tiles_n, n0 = (t % tiles_n) * BN;
    auto aload = [&](int m, int k) { return ld16<false>(X, (m * K + k) * 2); };
    auto epi = [&](int m, int n, f4 v) {
      st16<COH>(a.part, ((ks * a.M + m) * H + n) * 4, __builtin_bit_cast(u4, v));
    };
    Tile::run(lds, W, H, tm * BM, n0, ks * kper, kper / BK, aload, epi);
  }
}

// out[m] = LN(sum_ks part[ks][m] + bias + resid[m]) * g + b; one wave per row.
template <bool COH, int SPLITK>
__device__ __forceinline__ void stage_ln_t(const Params &a, const half_t *bias, const half_t *resid,
                                         const half_t *gam, const half_t *bet, half_t *out,
                                         int first_row, int row_stride, Flow *fl = nullptr) {
  const int lane = threadIdx.x & 63;
  for (int m = first_row; m < a.M; m += row_stride) {
    f4 v[3];
    u4 raw[3][SPLITK];
    u2 rres[3];
    // every load of the row is issued before the first use
    if (fl) {   // dataflow kernel: partials and residual come from the memory side and are polled
      for (int spin = 0;; ++spin) {
        asm volatile("" ::: "memory");     // the loads below are repeated, not hoisted
        bool bad = false;
#pragma unroll
        for (int c = 0; c < 3; ++c) {
          const int n = c * 256 + lane * 4;
#pragma unroll
          for (int ks = 0; ks < SPLITK; ++ks) raw[c][ks] = ld16<true>(a.part, ((ks * a.M + m) * H + n) * 4);
          rres[c] = ld8<true>(resid, (m * H + n) * 2);
        }
#pragma unroll
        for (int c = 0; c < 3; ++c) {
#pragma unroll
          for (int ks = 0; ks < SPLITK; ++ks) bad |= has_unwritten(raw[c][ks]);
          bad |= has_unwritten(rres[c]);
        }
        if (!__any(bad)) break;
        if (fl->failed || spin >= kMaxFlowSpin) { fl->failed = true; break; }
      }
    } else {
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
#pragma unroll
      for (int ks = 0; ks < SPLITK; ++ks) raw[c][ks] = ld16<false>(a.part, ((ks * a.M + m) * H + n) * 4);
      rres[c] = ld8<false>(resid, (m * H + n) * 2);
    }
    }
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
      f4 s = __builtin_bit_cast(f4, raw[c][0]);
#pragma unroll
      for (int ks = 1; ks < SPLITK; ++ks) s += __builtin_bit_cast(f4, raw[c][ks]);
      const h4 r = as_h4(rres[c]);
      s += f4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
      if (bias) {
        const h4 bb = ldg<h4>(bias + n);
        s += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      v[c] = s;
    }
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c) sum += v[c][0] + v[c][1] + v[c][2] + v[c][3];
    const float mean = wave_sum(sum) * (1.0f / H);
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) { const float d = v[c][i] - mean; sq += d * d; }
    const float rstd = rsqrtf(wave_sum(sq) * (1.0f / H) + a.eps);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
      f4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (v[c][i] - mean) * rstd;
      if (gam) {
        const h4 gg = ldg<h4>(gam + n);
        o *= f4{(float)gg[0], (float)gg[1], (float)gg[2], (float)gg[3]};
      }
      if (bet) {
        const h4 bb = ldg<h4>(bet + n);
        o += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      st8<COH>(out, (m * H + n) * 2, pack_h4(o));
    }
  }
}

// ---- many rows (M a multiple of 256): 256 x BN tiles, see gemm_big.hpp ----
// BN is chosen per GEMM so that M = 4096 gives exactly 256 tiles, one per CU: 144 for the
// 2304 QKV columns, 192 for FC1's 3072, 128-row tiles of 96 columns for the 768 of the out-projection; FC2 (K = 3072)
// uses 96 columns and two halves of K, which asks the L2 for 0.6x the operand bytes of 48-column
// tiles over the whole K (a CU takes in operands no faster than it multiplies them): 41 -> 31 us.
// (The same split for the out-projection, K = 768, gains nothing: its tiles are too short.)
// (a ring of four stages: three in flight at the start of a tile cost 1.7 us to queue, four 2.3 us, and the
// loop is no slower: 12 layers at M = 4096 1378 -> 1368 us fused, 1443 -> 1404 us as separate launches)
constexpr int kBigRing = 4;
using BigQkv = GemmBig<144, kBigRing>;
using BigFc1 = GemmBig<192, kBigRing>;
using BigOut = GemmBig<96, kBigRing, 128>;   // (128 x 96: 0.74x the operand bytes of 256 x 48 from the L2)
// FC2: parts of K, each a partial sum of its own.  16 tiles per row block: 4 column tiles of 192 x 4 parts of K
// (the operand reuse of the FC1 tile; 8 column tiles of 96 x 2 parts writes and reads back half the partial
// sums but runs its K loop at a worse ratio of operand bytes to MFMAs: 1434 us against 1417 for the 12
// layers at M = 4096 in the fused kernel, 1430 against 1441 as separate launches).
#ifndef SOUFFLE_FC2_SPLIT
#define SOUFFLE_FC2_SPLIT 4
#endif
constexpr int kFc2Split = SOUFFLE_FC2_SPLIT;
using BigFc2 = GemmBig<H * kFc2Split / 16, kBigRing>;
constexpr int kBigLds = BigFc1::LDS_BYTES;
static_assert(BigQkv::LDS_BYTES <= kBigLds && BigOut::LDS_BYTES <= kBigLds && BigFc2::LDS_BYTES <= kBigLds, "FC1 has the largest ring");

// Workgroup b runs on XCD b % 8.  An XCD gets a quarter of the row tiles and half of the
// column tiles, so that its L2 fetches each operand tile it needs once.
__device__ __forceinline__ void big_tile(int it, int m_tiles, int n_tiles, int *tm, int *tn) {
  if ((gridDim.x & 7) == 0 && (m_tiles & 3) == 0 && (n_tiles & 1) == 0) {
    const int x = it & 7, i = it >> 3, mq = m_tiles >> 2;
    *tm = (x & 3) * mq + i % mq;
    *tn = (x >> 2) * (n_tiles >> 1) + i / mq;
  } else {
    *tm = it / n_tiles;
    *tn = it % n_tiles;
  }
}

template <bool COH>
__device__ __forceinline__ void big_qkv(unsigned char *lds, const Params &a, const LayerW &w, const half_t *xin, int first, int stride, const GridBarrier *tb = nullptr) {
  const int m_tiles = a.M / 256, n_tiles = 3 * H / BigQkv::kBN;
  for (int it = first; it < m_tiles * n_tiles; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, n_tiles, &tm, &tn);
    const int n0 = tn * BigQkv::kBN;
    // the three [768][768] matrices are addressed as one [768][2304]
    auto wptr = [&](int k, int col) {
      const int c = n0 + col, j = c / H;
      return w.w_qkv + ((size_t)j * H + k) * H + (c - j * H);
    };
    const half_t *bq = w.b_qkv ? w.b_qkv : g_zero_row;
    const int bq_stride = w.b_qkv ? H : 0;
    auto cvt = [&](int, int nr, f4 v) {
      const int c = n0 + nr, j = c / H, n = c - j * H;
      return pack_h4(add_row4(v, bq + j * bq_stride, n));
    };
    auto store16 = [&](int m, int nr, u4 v) {                // 8 columns never straddle a head (64 columns)
      const int c = n0 + nr, j = c / H, n = c - j * H;
      const int b = m / a.S, s = m % a.S, hh = n / HD, d = n % HD;
      st16<COH>(a.qkv, ((((j * a.B + b) * NH + hh) * a.S + s) * HD + d) * 2, v);
    };
    BigQkv::run(lds, xin, H, tm * 256, 0, H / 32, wptr, cvt, store16, tb);
  }
}
template <bool COH>
__device__ __forceinline__ void big_fc1(unsigned char *lds, const Params &a, const LayerW &w, int first, int stride, const GridBarrier *tb = nullptr) {
  const int m_tiles = a.M / 256, n_tiles = F / BigFc1::kBN;
  for (int it = first; it < m_tiles * n_tiles; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, n_tiles, &tm, &tn);
    const int n0 = tn * BigFc1::kBN;
    auto wptr = [&](int k, int col) { return w.w_fc1 + (size_t)k * F + n0 + col; };
    const half_t *b1 = w.b_fc1 ? w.b_fc1 : g_zero_row;
    auto cvt_relu = [&](int, int nr, f4 v) {
      v = add_row4(v, b1, n0 + nr);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = fmaxf(v[i], 0.f);
      return pack_h4(v);
    };
    auto cvt_gelu = [&](int, int nr, f4 v) {
      v = add_row4(v, b1, n0 + nr);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = gelu_tanh(v[i]);
      return pack_h4(v);
    };
    auto store16 = [&](int m, int nr, u4 v) { st16<COH>(a.h, (m * F + n0 + nr) * 2, v); };
    f4 acc[BigFc1::MI][BigFc1::NT];
    BigFc1::mainloop(lds, a.y1, H, tm * 256, 0, H / 32, wptr, acc, tb);
    if (a.act == SOUFFLE_ACT_RELU) BigFc1::epilogue(lds, tm * 256, acc, cvt_relu, store16, tb);
    else BigFc1::epilogue(lds, tm * 256, acc, cvt_gelu, store16, tb);
  }
}
// z = X[M][K].W[K][768] + bias, fp16, into a.z1 (the out-projection; no split of K: 256 tiles already
// fill the device).  The residual is added by the LayerNorm that follows, which reads whole rows: read
// here, 8 bytes per lane across 16 rows per instruction, it cost a tile 5 us.
template <bool COH>
__device__ __forceinline__ void big_presum(unsigned char *lds, const Params &a, const half_t *X, int K, const half_t *W,
                                           const half_t *bias, int first, int stride) {
  // 16 tiles per 256-row block as in the other stages, dealt to the same workgroups: tile tn of row
  // block tm is rows [128 (tn & 1), +128) of the block and column tile tn >> 1.
  const int m_tiles = a.M / 256;
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, 16, &tm, &tn);
    const int n0 = (tn >> 1) * BigOut::kBN, m0 = tm * 256 + (tn & 1) * BigOut::kBM;
    auto wptr = [&](int k, int col) { return W + (size_t)k * H + n0 + col; };
    const half_t *bz = bias ? bias : g_zero_row;
    auto cvt = [&](int, int nr, f4 v) { return pack_h4(add_row4(v, bz, n0 + nr)); };
    auto store16 = [&](int m, int nr, u4 v) { st16<COH>(a.z1, (m * H + n0 + nr) * 2, v); };
    BigOut::run(lds, X, K, m0, 0, K / 32, wptr, cvt, store16);
  }
}
// A pre-LayerNorm sum in kFc2Split parts of K: part 0 = X[:, part 0].W[part 0] + bias, part
// p = X[:, part p].W[part p], all fp16, M x H each, one after the other in the (here otherwise
// unused) partials area (not in z1, which the out-projection of the same layer has written); the
// LayerNorm adds them in order, then the residual.
__device__ __forceinline__ half_t *fc2_sums(const Params &a) { return reinterpret_cast<half_t *>(a.part); }
template <bool COH>
__device__ __forceinline__ void big_presum2(unsigned char *lds, const Params &a, const half_t *X, int K, const half_t *W,
                                            const half_t *bias, int first, int stride) {
  const int m_tiles = a.M / 256;
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn2;
    big_tile(it, m_tiles, 16, &tm, &tn2);
    const int ks = tn2 % kFc2Split, n0 = (tn2 / kFc2Split) * BigFc2::kBN, k0 = ks * (K / kFc2Split);
    half_t *zp = fc2_sums(a) + (size_t)ks * a.M * H;
    auto wptr = [&](int k, int col) { return W + (size_t)k * H + n0 + col; };
    const half_t *bz = bias ? bias : g_zero_row;
    auto cvt_first = [&](int, int nr, f4 v) { return pack_h4(add_row4(v, bz, n0 + nr)); };
    auto cvt_rest = [&](int, int, f4 v) { return pack_h4(v); };
    auto store16 = [&](int m, int nr, u4 v) { st16<COH>(zp, (m * H + n0 + nr) * 2, v); };
    f4 acc[BigFc2::MI][BigFc2::NT];
    BigFc2::mainloop(lds, X, K, tm * 256, k0, (K / kFc2Split) / 32, wptr, acc);
    if (ks == 0) BigFc2::epilogue(lds, tm * 256, acc, cvt_first, store16);
    else BigFc2::epilogue(lds, tm * 256, acc, cvt_rest, store16);
  }
}
// out[m] = LN(z[0][m] + ... + z[NZ-1][m] + resid[m]) * g + b (z[p] = z + p M H; summed in this order);
// one wave per row, two-pass statistics in fp32 registers.
// NR rows (m0, m0 + mstep, ...) per call: their loads are all issued before the first is used.
template <bool COH, int NR, int NZ>
__device__ __forceinline__ void big_ln_rows(const Params &a, const half_t *z, const half_t *resid, const half_t *gam, const half_t *bet, half_t *out, int m0, int mstep) {
  const int lane = opaque_thread_id() & 63;
  u2 raw[NR][NZ + 1][3];
#pragma unroll
  for (int r = 0; r < NR; ++r)
#pragma unroll
    for (int p = 0; p < NZ; ++p)
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        const int m = m0 + r * mstep;
        raw[r][p][c] = ld8<false>(z + (size_t)p * a.M * H, (m * H + c * 256 + lane * 4) * 2);
        if (p == 0) raw[r][NZ][c] = ld8<false>(resid, (m * H + c * 256 + lane * 4) * 2);
      }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int m = m0 + r * mstep;
    f4 v[3];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const h4 q = as_h4(raw[r][0][c]);
      v[c] = f4{(float)q[0], (float)q[1], (float)q[2], (float)q[3]};
#pragma unroll
      for (int p = 1; p <= NZ; ++p) {
        const h4 q2 = as_h4(raw[r][p][c]);
        v[c] += f4{(float)q2[0], (float)q2[1], (float)q2[2], (float)q2[3]};
      }
      sum += v[c][0] + v[c][1] + v[c][2] + v[c][3];
    }
    const float mean = wave_sum(sum) * (1.0f / H);
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) { const float d = v[c][i] - mean; sq += d * d; }
    const float rstd = rsqrtf(wave_sum(sq) * (1.0f / H) + a.eps);
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      const int n = c * 256 + lane * 4;
      f4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (v[c][i] - mean) * rstd;
      if (gam) {
        const h4 gg = ldg<h4>(gam + n);
        o *= f4{(float)gg[0], (float)gg[1], (float)gg[2], (float)gg[3]};
      }
      if (bet) {
        const h4 bb = ldg<h4>(bet + n);
        o += f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
      }
      st8<COH>(out, (m * H + n) * 2, pack_h4(o));
    }
  }
}
template <bool COH, int NZ>
__device__ __forceinline__ void big_ln(const Params &a, const half_t *z, const half_t *resid, const half_t *gam, const half_t *bet, half_t *out, int first_row, int row_stride) {
  for (int m = first_row; m < a.M; m += row_stride) big_ln_rows<COH, 1, NZ>(a, z, resid, gam, bet, out, m, 0);
}

// The LayerNorm that follows a pre-LayerNorm sum, without a grid barrier in between (rowblock_ln).  A 256-row
// block of the sum is produced by 16 tiles (16 column tiles, or 4 column tiles x 4 parts of K).
// After the hand-over among them (rowblock_sync) tile t normalises rows 16t .. 16t+15 of the block,
// four per wave, by the same routine as the separate LayerNorm kernel: identical results.  The
// hand-over words are cleared by the launch itself (one grid barrier follows) and tags grow within a
// launch.
static_assert((256 / BigOut::kBM) * (H / BigOut::kBN) == 16 && kFc2Split * (H / BigFc2::kBN) == 16, "16 tiles per row block");
// Hand-over among the workgroups of a 256-row block: this workgroup's tiles of the stage are written
// (all of them: nobody waits before that, so the waits end whatever the tile-to-workgroup mapping is):
// publish `tag` in the word of each (row block, tile), run mid(), then wait until the 16 words of every
// row block this workgroup has a tile in have reached `tag`.  Bounded like the grid barrier; a wait that
// gave up ends all waiting of the launch.  With `bar.trace` the entry and exit times are stamped like
// those of a grid barrier.
// `group`: row blocks that hand over together (1, or the 2 or 3 that hold whole sequences of 512 or 384).
template <class Mid>
__device__ __forceinline__ void rowblock_sync(const Params &a, GridBarrier &bar, unsigned tag, int first, int stride, int group, Mid mid) {
  const int m_tiles = a.M / 256;
  const bool tr = bar.trace && bar.trace_idx < bar.trace_cap && threadIdx.x == 0;
  if (tr) bar.trace[(size_t)(2 * bar.trace_idx) * bar.nblk + blockIdx.x] = wall_clock64();
  __builtin_amdgcn_s_waitcnt(0);                 // this wave's write-through stores are acknowledged
  __syncthreads();
  if (threadIdx.x == 0)
    for (int it = first; it < m_tiles * 16; it += stride) {
      int tm, tn;
      big_tile(it, m_tiles, 16, &tm, &tn);
      __hip_atomic_store(a.rbflags + tm * 16 + tn, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  mid();
  if (threadIdx.x < 64 && !bar.failed) {
    for (int it = first; it < m_tiles * 16 && !bar.failed; it += stride) {
      int tm, tn;
      big_tile(it, m_tiles, 16, &tm, &tn);
      const int g0 = tm - tm % group;
      for (int spin = 0; spin < kMaxBarrierSpin; ++spin) {
        bool ok = true;
        if (threadIdx.x < 16 * group)
          ok = (int)(__hip_atomic_load(a.rbflags + g0 * 16 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - tag) >= 0;
        if (__all(ok)) break;
        __builtin_amdgcn_s_sleep(1);
        if (spin == kMaxBarrierSpin - 1) {         // gave up: the launch's output is invalid
          bar.failed = true;
          if (threadIdx.x == 0) (void)__hip_atomic_fetch_or(a.ctl + kCtlErrWord, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }
  if (tr) bar.trace[(size_t)(2 * bar.trace_idx + 1) * bar.nblk + blockIdx.x] = wall_clock64();
  bar.trace_idx++;
  __syncthreads();
}
template <bool COH, int NZ>
__device__ __forceinline__ void rowblock_ln(const Params &a, GridBarrier &bar, unsigned tag, const half_t *z, const half_t *resid, const half_t *gam,
                                            const half_t *bet, half_t *out, int first, int stride) {
  const int m_tiles = a.M / 256, wave = threadIdx.x >> 6;
  rowblock_sync(a, bar, tag, first, stride, 1, []() {});
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, 16, &tm, &tn);
    big_ln_rows<COH, 4, NZ>(a, z, resid, gam, bet, out, tm * 256 + tn * 16 + wave * 4, 1);
  }
}

// ---- skinny (small M) path: one-shot operand loads, see gemm_oneshot.hpp ----
using OsFull = GemmOneShot<32, 768>;    // QKV, out-projection, FC1: whole K in one shot
using OsFc2 = GemmOneShot<32, 768>;     // FC2: 4 K slices as fp32 partials
constexpr int kSplitFc2Small = F / OsFc2::kKS;
constexpr int kXRegion = 49152;         // LDS: [0, 48 KB) X slice / attention tiles / reduction, [48 KB, 144 KB) W slice
static_assert(OsFull::X_BYTES <= kXRegion && OsFc2::X_BYTES <= kXRegion, "X region");
constexpr int kLnParamOff = kXRegion + (OsFull::W_BYTES > OsFc2::W_BYTES ? OsFull::W_BYTES : OsFc2::W_BYTES);   // gamma[768], beta[768]
constexpr int kSmallGemmLds = kLnParamOff + 2 * H * 2;

// One work item of a skinny GEMM stage: output tile origin, weight slice, activation slice.
struct Item {
  int m0, n0;           // output rows / columns of the tile (n0 relative to `W`'s own column space)
  const half_t *W;      // weight matrix the slice comes from
  int ldw, k0;          // its row pitch, first row of the K slice
  int aux;              // stage specific (q/k/v index, K-slice index)
  int rot;              // rotation of the weight-row request order (see GemmOneShot::issue_w)
};

// Workgroup b runs on XCD b % 8 (each XCD has its own L2).  The m-tiles that share one weight
// slice are dealt to workgroups of ONE XCD in the same pass, so the slice crosses the fabric
// once per XCD instead of once per workgroup.  Returns false when `it` names no item.
__device__ __forceinline__ bool xcd_item(int it, int m_tiles, int w_slices, int *mt, int *ws) {
  if ((gridDim.x & 7) != 0) { *mt = it % m_tiles; *ws = it / m_tiles; return it < m_tiles * w_slices; }
  const int xcd = it & 7, j = it >> 3;
  *mt = j % m_tiles;
  *ws = (j / m_tiles) * 8 + xcd;
  return *ws < w_slices;
}
__device__ __forceinline__ int xcd_item_span(int m_tiles, int w_slices) {   // exclusive upper bound of valid `it`
  return (gridDim.x & 7) != 0 ? m_tiles * w_slices : ((w_slices + 7) >> 3) * m_tiles * 8;
}

struct QkvItems {
  const half_t *w_qkv; int M;
  __device__ int span() const { return xcd_item_span(M / OsFull::kBM, 3 * H / 64); }
  __device__ bool at(int it, Item &d) const {
    int mt, ws;
    if (!xcd_item(it, M / OsFull::kBM, 3 * H / 64, &mt, &ws)) return false;
    const int n0 = ws * 64, j = n0 / H;
    d = Item{mt * OsFull::kBM, n0 % H, w_qkv + (size_t)j * H * H, H, 0, j, mt * (OsFull::W_INSTR / 4) / (M / OsFull::kBM)};
    return true;
  }
};
struct OutItems {
  const half_t *w_o; int M;
  __device__ int span() const { return xcd_item_span(M / OsFull::kBM, H / 64); }
  __device__ bool at(int it, Item &d) const {
    int mt, ws;
    if (!xcd_item(it, M / OsFull::kBM, H / 64, &mt, &ws)) return false;
    d = Item{mt * OsFull::kBM, ws * 64, w_o, H, 0, 0, mt * (OsFull::W_INSTR / 4) / (M / OsFull::kBM)};
    return true;
  }
};
struct Fc1Items {
  const half_t *w_fc1; int M;
  __device__ int span() const { return xcd_item_span(M / OsFull::kBM, F / 64); }
  __device__ bool at(int it, Item &d) const {
    int mt, ws;
    if (!xcd_item(it, M / OsFull::kBM, F / 64, &mt, &ws)) return false;
    d = Item{mt * OsFull::kBM, ws * 64, w_fc1, F, 0, 0, mt * (OsFull::W_INSTR / 4) / (M / OsFull::kBM)};
    return true;
  }
};
struct Fc2Items {
  const half_t *w_fc2; int M;
  __device__ int span() const { return xcd_item_span(M / OsFc2::kBM, (H / 64) * kSplitFc2Small); }
  __device__ bool at(int it, Item &d) const {
    int mt, ws;
    if (!xcd_item(it, M / OsFc2::kBM, (H / 64) * kSplitFc2Small, &mt, &ws)) return false;
    const int ks = ws % kSplitFc2Small;
    d = Item{mt * OsFc2::kBM, (ws / kSplitFc2Small) * 64, w_fc2, H, ks * OsFc2::kKS, ks, mt * (OsFc2::W_INSTR / 4) / (M / OsFc2::kBM)};
    return true;
  }
};

// The weight slice of a workgroup's first item of the NEXT stage is queued from inside the grid
// barrier (after the arrival, before the wait), by waves 1..3: it needs nothing from other
// workgroups, and the ~1.3 us its requests take to issue are hidden in the barrier.
constexpr bool kPrefetchAcrossBarrier = true;

// Queue the weight slice of this workgroup's first item of a stage (if it has one).
template <class G, class Items>
__device__ __forceinline__ bool preissue_w(unsigned char *lds, const Items &items) {
  Item d;
  if (!kPrefetchAcrossBarrier || (int)blockIdx.x >= items.span() || !items.at(blockIdx.x, d)) return false;
  G::issue_w_prefetch(lds + kXRegion, d.W, d.ldw, d.n0, d.k0, d.rot);
  return true;
}

// Fine-grained time stamps inside a stage (development builds only: they cost scalar registers).

// Driver of a skinny GEMM stage.  `w_ready`: the weight slice of this workgroup's first item
// was queued earlier (inside the preceding grid barrier, or after the previous stage in the
// dataflow kernel).  `extra()` queues further direct-to-LDS loads
// with the operands, `pre(item)` runs after the operands have
// landed (LayerNorm on load), `epi(item, m, n, lo, hi)` receives 8 consecutive columns of a row.
// With `fl` the X slice is polled (dataflow kernel) unless `x_is_input` (it is then read plainly).
template <class G, bool COH, class Items, class Extra, class Pre, class Epi>
__device__ __forceinline__ void gemm_stage(unsigned char *lds, const Items &items, const half_t *X, int ldx, bool w_ready,
                                           Extra extra, Pre pre, Epi epi, const GridBarrier *tb = nullptr,
                                           Flow *fl = nullptr, bool x_is_input = false) {
  const int span = items.span();
  for (int it = blockIdx.x; it < span; it += gridDim.x) {
    Item d;
    if (!items.at(it, d)) { w_ready = false; continue; }
    __syncthreads();                       // LDS reuse
    STAGE_MARK(tb, 0);
    if (!w_ready) G::issue_w(lds + kXRegion, d.W, d.ldw, d.n0, d.k0, d.rot);
    extra();
    if (fl && !x_is_input) poll_x<G>(lds, X, ldx, d.m0, d.k0, *fl);
    else G::template issue_x<false>(lds, X, ldx, d.m0, d.k0);
    STAGE_MARK(tb, 1);
#ifdef SOUFFLE_STAGE_MARKS
    if (tb && tb->trace) { wait_vmcnt<G::X_INSTR / 4>(); trace_mark(*tb, 2); }
#endif
    G::wait_loads();
    if (fl) flow_stamp(*fl, 0);
    STAGE_MARK(tb, 3);
    pre(d);
    STAGE_MARK(tb, 4);
    G::compute(lds, lds + kXRegion, [&](int mm, int nn, f4 lo, f4 hi) { epi(d, d.m0 + mm, d.n0 + nn, lo, hi); });
    STAGE_MARK(tb, 5);
#ifdef SOUFFLE_STAGE_MARKS
    if (tb && tb->trace) { __builtin_amdgcn_s_waitcnt(0); trace_mark(*tb, 6); }
#endif
    w_ready = false;
  }
}

// LayerNorm of the 32 complete rows of an OsFull X tile, in place in LDS.  Eight lanes
// share a row; slot s of row r holds columns 8*(s ^ (r & 15)) .. +7.  Statistics and the
// normalisation (one FMA per element) are fp32.  When `out` is given the normalised rows are also written to out[m0 + r][:].
// gamma and beta come from LDS (queued with the operands by issue_ln_params), not from global
// memory: a dependent global load after the row statistics would cost another memory latency.
__device__ __forceinline__ void issue_ln_params(unsigned char *lds, const half_t *gam, const half_t *bet) {
  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;
  const int tid = threadIdx.x, wave = tid >> 6;       // 192 slots of 16 bytes: gamma 0..95, beta 96..191
  if (wave < 3) {
    const int s = tid;
    const half_t *src = s < 96 ? (gam ? gam + s * 8 : nullptr) : (bet ? bet + (s - 96) * 8 : nullptr);
    if (src) __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + kLnParamOff + wave * 1024), 16, 0, 0);
  }
}
template <bool COH>
__device__ __forceinline__ void ln_rows_in_lds(unsigned char *lds_x, bool has_gam, bool has_bet, float eps,
                                               half_t *out, int m0) {
  constexpr int XGR = OsFull::XGR, PER = XGR / 8;
  const int tid = threadIdx.x, r = tid >> 3, t8 = tid & 7;
  h8 *row = reinterpret_cast<h8 *>(lds_x) + r * XGR;
  const half_t *gam = has_gam ? reinterpret_cast<const half_t *>(lds_x + kLnParamOff) : nullptr;
  const half_t *bet = has_bet ? reinterpret_cast<const half_t *>(lds_x + kLnParamOff + H * 2) : nullptr;
  // Statistics with the packed dot product (fp16 products are exact in fp32, fp32 accumulation),
  // normalisation with two mixed-precision FMAs per element (fp16 operands, fp32 arithmetic,
  // one rounding at the end): the stage is bound by vector ALU issue, not by LDS.
  h8 x[PER];
  float sum = 0.f, sq = 0.f;
  const h2 ones = {(half_t)1.f, (half_t)1.f};
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    x[i] = row[t8 + 8 * i];
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      const h2 p = {x[i][e], x[i][e + 1]};
      sum = __builtin_amdgcn_fdot2(p, ones, sum, false);
      sq = __builtin_amdgcn_fdot2(p, p, sq, false);
    }
  }
  sum += wave_xor(sum, 1); sum += wave_xor(sum, 2); sum += wave_xor(sum, 4);
  sq += wave_xor(sq, 1); sq += wave_xor(sq, 2); sq += wave_xor(sq, 4);
  // one-pass variance in fp32: the rows are residual sums with |mean| well below the
  // standard deviation, so E[x^2] - mean^2 loses no significant digits
  const float mean = sum * (1.0f / H);
  const float var = fmaxf(sq * (1.0f / H) - mean * mean, 0.f);
  const float rstd = rsqrtf(var + eps), shift = -mean * rstd;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int sl = t8 + 8 * i, k = (sl ^ (r & 15)) * 8;
    h8 o;
    if (gam || bet) {
      h8 g8, b8;
      if (gam) g8 = *reinterpret_cast<const h8 *>(gam + k);     // (LDS copies of the parameters)
      if (bet) b8 = *reinterpret_cast<const h8 *>(bet + k);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float t = __builtin_fmaf((float)x[i][e], rstd, shift);
        o[e] = (half_t)__builtin_fmaf(t, gam ? (float)g8[e] : 1.0f, bet ? (float)b8[e] : 0.0f);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (half_t)__builtin_fmaf((float)x[i][e], rstd, shift);
    }
    row[sl] = o;
    if (out) st16<COH>(out, ((m0 + r) * H + k) * 2, as_u4(o));
  }
  __syncthreads();
}

template <bool COH>
__device__ __forceinline__ void stage_ln(const Params &a, int splitk, const half_t *bias, const half_t *resid,
                                         const half_t *gam, const half_t *bet, half_t *out, int first_row, int row_stride,
                                         Flow *fl = nullptr) {
  if (splitk == 1) stage_ln_t<COH, 1>(a, bias, resid, gam, bet, out, first_row, row_stride, fl);
  else stage_ln_t<COH, kSplitFc2Small>(a, bias, resid, gam, bet, out, first_row, row_stride, fl);
}

// The four skinny GEMM stages (shared by the megakernels and the per-op kernels).  With `fl`
// (dataflow kernel) the activation slice is polled instead of being loaded after a barrier.
template <bool COH>
__device__ __forceinline__ void small_qkv(unsigned char *lds, const Params &a, const LayerW &w, const half_t *xin, bool w_ready,
                                          const GridBarrier *tb = nullptr, Flow *fl = nullptr, bool x_is_input = false) {
  gemm_stage<OsFull, COH>(lds, QkvItems{w.w_qkv, a.M}, xin, H, w_ready, []() {}, [](const Item &) {},
    [&](const Item &d, int m, int n, f4 lo, f4 hi) {
      add_bias8(lo, hi, w.b_qkv ? w.b_qkv + d.aux * H : nullptr, n);
      const int b = m / a.S, s = m % a.S, hh = n / HD, dd = n % HD;
      st16<COH>(a.qkv, ((((d.aux * a.B + b) * NH + hh) * a.S + s) * HD + dd) * 2, pack_h8(lo, hi));
    }, tb, fl, x_is_input);
}
// z1 = ctx.Wo + b_o + x (pre-LayerNorm, fp16).  The residual values of a thread's 8 output
// columns are requested before the MFMAs and used after them.  In the dataflow kernel the rows
// of x are known to be complete (the context rows being there implies it) but may be absent
// from this XCD's L2 or stale in it, hence the memory-side load.
template <bool COH>
__device__ __forceinline__ void small_outproj(unsigned char *lds, const Params &a, const LayerW &w, const half_t *xin, bool w_ready,
                                              const GridBarrier *tb = nullptr, Flow *fl = nullptr, bool x_is_input = false) {
  static_assert(OsFull::CPT == 8, "one epilogue call per thread");
  u4 resid;
  gemm_stage<OsFull, COH>(lds, OutItems{w.w_o, a.M}, a.ctx, H, w_ready, []() {},
    [&](const Item &d) {
      const int tid = threadIdx.x, off = ((d.m0 + tid / 8) * H + d.n0 + (tid % 8) * 8) * 2;
      resid = (fl && !x_is_input) ? ld16<true>(xin, off) : ld16<false>(xin, off);
    },
    [&](const Item &, int m, int n, f4 lo, f4 hi) {
      add_bias8(lo, hi, w.b_o, n);
      const h8 r = as_h8(resid);
      lo += f4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
      hi += f4{(float)r[4], (float)r[5], (float)r[6], (float)r[7]};
      st16<COH>(a.z1, (m * H + n) * 2, pack_h8(lo, hi));
    }, tb, fl);
}
// h = act(LN1(z1).W1 + b1): LayerNorm is applied to the X tile in LDS (every workgroup has
// complete rows); the workgroups of the first n-tile also publish y1 = LN1(z1).
template <bool COH>
__device__ __forceinline__ void small_fc1(unsigned char *lds, const Params &a, const LayerW &w, bool w_ready,
                                          const GridBarrier *tb = nullptr, Flow *fl = nullptr) {
  gemm_stage<OsFull, COH>(lds, Fc1Items{w.w_fc1, a.M}, a.z1, H, w_ready,
    [&]() { issue_ln_params(lds, w.ln1_g, w.ln1_b); },
    [&](const Item &d) { ln_rows_in_lds<COH>(lds, w.ln1_g != nullptr, w.ln1_b != nullptr, a.eps, d.n0 == 0 ? a.y1 : nullptr, d.m0); },
    [&](const Item &, int m, int n, f4 lo, f4 hi) {
      add_bias8(lo, hi, w.b_fc1, n);
      if (a.act == SOUFFLE_ACT_RELU) {            // (one test per group of results, not one per result)
#pragma unroll
        for (int i = 0; i < 4; ++i) { lo[i] = fmaxf(lo[i], 0.f); hi[i] = fmaxf(hi[i], 0.f); }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) { lo[i] = gelu_tanh(lo[i]); hi[i] = gelu_tanh(hi[i]); }
      }
      st16<COH>(a.h, (m * F + n) * 2, pack_h8(lo, hi));
    }, tb, fl);
}
// fp32 partials of h.W2 over 4 K slices
template <bool COH>
__device__ __forceinline__ void small_fc2(unsigned char *lds, const Params &a, const LayerW &w, bool w_ready,
                                          const GridBarrier *tb = nullptr, Flow *fl = nullptr) {
  gemm_stage<OsFc2, COH>(lds, Fc2Items{w.w_fc2, a.M}, a.h, F, w_ready, []() {}, [](const Item &) {},
    [&](const Item &d, int m, int n, f4 lo, f4 hi) {
      st16<COH>(a.part, ((d.aux * a.M + m) * H + n) * 4, __builtin_bit_cast(u4, lo));
      st16<COH>(a.part, ((d.aux * a.M + m) * H + n + 4) * 4, __builtin_bit_cast(u4, hi));
    }, tb, fl);
}

// One (batch, head, 64-query block) per workgroup pass; each wave owns 16 queries.
// Scores are computed transposed (keys x queries) so that the softmax reduction over
// keys is in-lane plus two cross-lane steps, and the probabilities are already in the
// B-operand layout of the 16x16x16 MFMA used for P.V.  V is staged row-major in LDS
// and read through the transposing LDS load.
// Direct global->LDS load of a [rows][64] fp16 tile (128-byte rows = 8 slots of 16 bytes),
// swizzled for its reader: MODE 0 for b128 operand reads of 16 consecutive rows
// (slot ^= (row >> 1) & 7), MODE 1 for the transposing read of 4 consecutive rows (slot ^= row & 2).
// (The LDS has 64 banks and serves that read half a wave, 8 consecutive rows, per cycle: with row & 2 rows r and r+4
// collide, 196608 conflict cycles per attention stage at 4096 rows.  slot ^= row & 6 removes them all and was
// measured no faster in the fused encoder and 1.8 % slower in the per-op chain at 4096 rows: kept as it was.)
template <bool COH, int MODE>
__device__ __forceinline__ void issue_rows64(unsigned char *lds, const half_t *src, int rows) {
  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int inst = wave; inst < rows / 8; inst += 4) {
    const int sl = inst * 64 + lane, r = sl >> 3, c = (sl & 7) ^ (MODE == 0 ? ((r >> 1) & 7) : (r & 2));
    __builtin_amdgcn_global_load_lds((gptr_t)(src + (size_t)r * HD + c * 8), (lptr_t)(lds + inst * 1024), 16, 0, COH ? kAuxSc1 : 0);
  }
}

// The loads of one attention item (K and V of the head, 64 query rows), through inline assembly so
// that the caller decides what to wait for (see load_lds16); every wave issues kAttnLoads<NKT> of them.
template <int NKT>
constexpr int kAttnLoads = 2 * (NKT * 16 / 32) + 2;
template <int MODE>
__device__ __forceinline__ void issue_rows64_nowait(unsigned lds_addr, const half_t *src, int rows) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int inst = wave; inst < rows / 8; inst += 4) {
    const int sl = inst * 64 + lane, r = sl >> 3, c = (sl & 7) ^ (MODE == 0 ? ((r >> 1) & 7) : (r & 2));
    load_lds16(src + (size_t)r * HD + c * 8, lds_addr + inst * 1024);
  }
}
template <int NKT>
__device__ __forceinline__ void attn_issue(unsigned char *lds, const Params &a, int item) {
  constexpr int S = NKT * 16;
  const int qblocks = S / 64;
  const int qb = item % qblocks, bh = item / qblocks;
  const int head_off = bh * S * HD;                              // halves, within one of q/k/v
  const size_t plane = (size_t)a.B * NH * S * HD;
  const unsigned base = lds_address(lds);
  issue_rows64_nowait<0>(base, a.qkv + plane + head_off, S);
  issue_rows64_nowait<1>(base + S * 128, a.qkv + 2 * plane + head_off, S);
  issue_rows64_nowait<0>(base + 2 * S * 128, a.qkv + head_off + (size_t)qb * 64 * HD, 64);
}
template <int NKT>
constexpr int kAttnItemLds = 2 * NKT * 16 * 128 + 64 * 128;

// PLAIN: no mask and no probabilities to write (tested once per item: a uniform test per key tile
// inside the unrolled loops is not hoisted by the compiler and breaks them into small blocks).
template <bool COH, int NKT, bool PLAIN>
__device__ __forceinline__ void attn_compute_t(unsigned char *lds, const Params &a, int item);
template <bool COH, int NKT>
__device__ __forceinline__ void attn_compute(unsigned char *lds, const Params &a, int item) {
  if (!a.mask && !a.probs) attn_compute_t<COH, NKT, true>(lds, a, item);
  else attn_compute_t<COH, NKT, false>(lds, a, item);
}

template <bool COH, int NKT>
__device__ __forceinline__ void attn_item(half_t *lds_h, const Params &a, int item) {
  unsigned char *lds = reinterpret_cast<unsigned char *>(lds_h);
  __syncthreads();   // LDS reuse
  attn_issue<NKT>(lds, a, item);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  attn_compute<COH, NKT>(lds, a, item);
}

// One work unit after the other with the loads of the next in flight while this one is computed
// (two LDS buffers).  `item_of(it)`: work unit -> item.
template <bool COH, int NKT, class ItemOf>
__device__ __forceinline__ void attn_items_pipelined(unsigned char *lds, const Params &a, int first, int stride, int items, ItemOf item_of) {
  if (first >= items) return;
  __syncthreads();   // LDS reuse
  attn_issue<NKT>(lds, a, item_of(first));
  int cur = 0;
  for (int it = first; it < items; it += stride) {
    if (it + stride < items) {
      attn_issue<NKT>(lds + (cur ^ 1) * kAttnItemLds<NKT>, a, item_of(it + stride));
      wait_vmcnt<kAttnLoads<NKT>>();      // all but the loads just issued (results stored earlier included)
    } else {
      wait_vmcnt<0>();
    }
    __syncthreads();
    attn_compute<COH, NKT>(lds + cur * kAttnItemLds<NKT>, a, item_of(it));
    __syncthreads();   // this buffer is refilled in the next turn
    cur ^= 1;
  }
}

template <bool COH, int NKT, bool PLAIN>
__device__ __forceinline__ void attn_compute_t(unsigned char *lds, const Params &a, int item) {
  constexpr int S = NKT * 16;
  unsigned char *ks_ = lds, *vs_ = lds + S * 128, *qs_ = lds + 2 * S * 128;
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const int qblocks = S / 64;
  const int qb = item % qblocks, bh = item / qblocks, b = bh / NH, hh = bh % NH;

  const half_t *kh = reinterpret_cast<const half_t *>(ks_), *vh = reinterpret_cast<const half_t *>(vs_),
               *qh = reinterpret_cast<const half_t *>(qs_);
  const int q0 = qb * 64 + wave * 16, q = q0 + l16;
  h8 qop[2];
  {
    const int r = wave * 16 + l16;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) qop[ks] = *reinterpret_cast<const h8 *>(qh + (r * 8 + ((ks * 4 + g) ^ ((r >> 1) & 7))) * 8);
  }
  f4 sc[NKT];
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    const int r = t * 16 + l16, sw = (r >> 1) & 7;
    const h8 k0 = *reinterpret_cast<const h8 *>(kh + (r * 8 + (g ^ sw)) * 8);
    const h8 k1 = *reinterpret_cast<const h8 *>(kh + (r * 8 + ((4 + g) ^ sw)) * 8);
    f4 c = mfma_16x16x32(k0, qop[0], f4{0.f, 0.f, 0.f, 0.f});
    sc[t] = mfma_16x16x32(k1, qop[1], c);
  }
  // sc[t][v] = score(key = 16t + 4g + v, query = q0 + l16)
  // softmax in base 2: exp(s - max) = exp2(s log2(e) - max'), log2(e) folded into the scale
  constexpr float kLog2e = 1.4426950408889634f;
  const float scale2 = a.scale * kLog2e;
  float mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    f4 sv = sc[t] * scale2;
    if constexpr (!PLAIN) {
      if (a.mask) {
        const h4 mk = ldg<h4>(a.mask + ((size_t)b * S + q) * S + t * 16 + g * 4);
        sv += f4{(float)mk[0], (float)mk[1], (float)mk[2], (float)mk[3]} * kLog2e;
      }
    }
    sc[t] = sv;
    mx = fmaxf(mx, fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));
  }
  mx = fmaxf(mx, wave_xor(mx, 16));
  mx = fmaxf(mx, wave_xor(mx, 32));
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { sc[t][i] = __builtin_amdgcn_exp2f(sc[t][i] - mx); sum += sc[t][i]; }
  }
  sum += wave_xor(sum, 16);
  sum += wave_xor(sum, 32);
  const float inv = __builtin_amdgcn_rcpf(sum);
  h4 p[NKT];
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    const f4 pr = sc[t] * inv;
    p[t] = h4{(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};
    if constexpr (!PLAIN) {
      if (a.probs)
        st8<false>(a.probs, (int)((((size_t)(b * NH + hh) * S + q) * S + t * 16 + g * 4) * 2), as_u2(p[t]));
    }
  }
  f4 o[HD / 16];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < NKT; ++t) {
    const int kr = t * 16 + g * 4 + (l16 >> 2);
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      const int c = dt * 2 + ((l16 & 3) >> 1);
      const h4 vop = lds_read_tr16(vh + (kr * 8 + (c ^ (kr & 2))) * 8 + (l16 & 1) * 4);
      o[dt] = mfma_16x16x16(vop, p[t], o[dt]);
    }
  }
  // o[dt][v] = ctx(query q, d = 16dt + 4g + v)
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt)
    st8<COH>(a.ctx, ((b * S + q) * H + hh * HD + dt * 16 + g * 4) * 2, pack_h4(o[dt]));
}

// ---- attention for the skinny path: one item = one head x 16 queries, keys split over the waves ----
// With few rows the 64-query item above leaves most CUs idle and its per-wave chain
// (scores -> softmax -> P.V over ALL keys) is the stage's critical path.  Here each wave
// handles a quarter of the keys for the same 16 queries and loads exactly the K/V rows it
// multiplies (no workgroup barrier before the MFMAs); the four partial results are merged
// through LDS the flash-attention way (running maximum, rescaled sums).
constexpr int kAttnCombLd = 68;                                   // floats per row of a wave's partial context
constexpr int attn_small_lds_bytes(int S) { return 2 * S * 128 + 4 * 2048 + 4 * 16 * kAttnCombLd * 4 + 512; }

template <int MODE>
__device__ __forceinline__ void issue_rows64_wave(unsigned char *lds_tile, const half_t *src, int row0, int rows) {
  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;
  const int lane = threadIdx.x & 63;
  for (int inst = 0; inst < rows / 8; ++inst) {
    const int r = row0 + inst * 8 + (lane >> 3), c = (lane & 7) ^ (MODE == 0 ? ((r >> 1) & 7) : (r & 2));
    __builtin_amdgcn_global_load_lds((gptr_t)(src + (size_t)r * HD + c * 8), (lptr_t)(lds_tile + (row0 + inst * 8) * 128), 16, 0, 0);
  }
}

// One direct-to-LDS load of 8 rows of a [rows][64] fp16 tile, layout as issue_rows64_wave, memory-side.
template <int MODE>
__device__ __forceinline__ void issue_row8_sc1(unsigned char *lds_tile, const half_t *src, int r0) {
  typedef __attribute__((address_space(1))) const void *gptr_t;
  typedef __attribute__((address_space(3))) void *lptr_t;
  const int lane = threadIdx.x & 63, r = r0 + (lane >> 3), c = (lane & 7) ^ (MODE == 0 ? ((r >> 1) & 7) : (r & 2));
  __builtin_amdgcn_global_load_lds((gptr_t)(src + (size_t)r * HD + c * 8), (lptr_t)(lds_tile + r0 * 128), 16, 0, kAuxSc1);
}

template <bool COH, int NKT>
__device__ __forceinline__ void attn_item_split(unsigned char *lds, const Params &a, int bh, int qb, Flow *fl = nullptr) {
  constexpr int S = NKT * 16, TPW = NKT / 4;                       // key tiles per wave
  static_assert(NKT % 4 == 0, "keys split evenly over four waves");
  unsigned char *ks_ = lds, *vs_ = lds + S * 128, *qs_ = lds + 2 * S * 128;
  float *comb = reinterpret_cast<float *>(lds + 2 * S * 128 + 4 * 2048);
  float *stats = comb + 4 * 16 * kAttnCombLd;                      // [wave][query][max, sum]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const int b = bh / NH, hh = bh % NH;
  const int head_off = ((b * NH + hh) * S) * HD;                   // halves, within one of q/k/v
  const size_t plane = (size_t)a.B * NH * S * HD;
  const half_t *Q = a.qkv + head_off + (size_t)qb * 16 * HD, *K = a.qkv + plane + head_off, *V = a.qkv + 2 * plane + head_off;

  __syncthreads();   // LDS reuse
  if (fl) {
    // 2 loads of queries, then TPW*2 of this wave's keys and as many of its values, each polled
    constexpr int NL = 2 + 4 * TPW;
    const int lane_b = (threadIdx.x & 63) * 16, kr0 = wave * TPW * 16;
    auto issue = [&](int i) {
      if (i < 2) issue_row8_sc1<0>(qs_ + wave * 2048, Q, i * 8);
      else if (i < 2 + 2 * TPW) issue_row8_sc1<0>(ks_, K, kr0 + (i - 2) * 8);
      else issue_row8_sc1<1>(vs_, V, kr0 + (i - 2 - 2 * TPW) * 8);
    };
    auto slot = [&](int i) {
      if (i < 2) return qs_ + wave * 2048 + i * 1024 + lane_b;
      if (i < 2 + 2 * TPW) return ks_ + (kr0 + (i - 2) * 8) * 128 + lane_b;
      return vs_ + (kr0 + (i - 2 - 2 * TPW) * 8) * 128 + lane_b;
    };
    poll_direct_loads<NL, (1ull << NL) - 1>(issue, slot, *fl);
    flow_stamp(*fl, 0);
  } else {
    issue_rows64_wave<0>(qs_ + wave * 2048, Q, 0, 16);             // every wave its own copy of the queries
    issue_rows64_wave<0>(ks_, K, wave * TPW * 16, TPW * 16);
    issue_rows64_wave<1>(vs_, V, wave * TPW * 16, TPW * 16);
    __builtin_amdgcn_s_waitcnt(0);                                 // this wave's rows only: no barrier needed
  }

  const half_t *kh = reinterpret_cast<const half_t *>(ks_), *vh = reinterpret_cast<const half_t *>(vs_),
               *qh = reinterpret_cast<const half_t *>(qs_ + wave * 2048);
  const int q = qb * 16 + l16;
  h8 qop[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) qop[ks] = *reinterpret_cast<const h8 *>(qh + (l16 * 8 + ((ks * 4 + g) ^ ((l16 >> 1) & 7))) * 8);
  f4 sc[TPW];
  float mx = -1e30f;                                               // finite: a fully masked quarter contributes nothing
#pragma unroll
  for (int tt = 0; tt < TPW; ++tt) {
    const int t = wave * TPW + tt, r = t * 16 + l16, sw = (r >> 1) & 7;
    const h8 k0 = *reinterpret_cast<const h8 *>(kh + (r * 8 + (g ^ sw)) * 8);
    const h8 k1 = *reinterpret_cast<const h8 *>(kh + (r * 8 + ((4 + g) ^ sw)) * 8);
    f4 sv = mfma_16x16x32(k1, qop[1], mfma_16x16x32(k0, qop[0], f4{0.f, 0.f, 0.f, 0.f})) * a.scale;
    // sv[v] = score(key = 16t + 4g + v, query = q)
    if (a.mask) {
      const h4 mk = ldg<h4>(a.mask + ((size_t)b * S + q) * S + t * 16 + g * 4);
      sv += f4{(float)mk[0], (float)mk[1], (float)mk[2], (float)mk[3]};
    }
    sc[tt] = sv;
    mx = fmaxf(mx, fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));
  }
  mx = fmaxf(mx, wave_xor(mx, 16));
  mx = fmaxf(mx, wave_xor(mx, 32));
  float sum = 0.f;
  h4 p[TPW];
#pragma unroll
  for (int tt = 0; tt < TPW; ++tt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { sc[tt][i] = __expf(sc[tt][i] - mx); sum += sc[tt][i]; }
    p[tt] = h4{(half_t)sc[tt][0], (half_t)sc[tt][1], (half_t)sc[tt][2], (half_t)sc[tt][3]};
  }
  sum += wave_xor(sum, 16);
  sum += wave_xor(sum, 32);
  f4 o[HD / 16];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int tt = 0; tt < TPW; ++tt) {
    const int kr = (wave * TPW + tt) * 16 + g * 4 + (l16 >> 2);
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      const int c = dt * 2 + ((l16 & 3) >> 1);
      const h4 vop = lds_read_tr16(vh + (kr * 8 + (c ^ (kr & 2))) * 8 + (l16 & 1) * 4);
      o[dt] = mfma_16x16x16(vop, p[tt], o[dt]);
    }
  }
  // o[dt][v] = sum over this wave's keys of exp(score - mx) * V[key][16dt + 4g + v], query q
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt)
    *reinterpret_cast<f4 *>(comb + (wave * 16 + l16) * kAttnCombLd + dt * 16 + g * 4) = o[dt];
  if (g == 0) { stats[(wave * 16 + l16) * 2] = mx; stats[(wave * 16 + l16) * 2 + 1] = sum; }
  __syncthreads();
  float wmx[4], wsum[4];
  auto merged = [&](int qq, float *scale) {                        // scale[w] = exp(mx_w - max) / total
    float m = -1e30f;
#pragma unroll
    for (int w = 0; w < 4; ++w) { wmx[w] = stats[(w * 16 + qq) * 2]; wsum[w] = stats[(w * 16 + qq) * 2 + 1]; m = fmaxf(m, wmx[w]); }
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) { scale[w] = __expf(wmx[w] - m); total += wsum[w] * scale[w]; }
    const float inv = 1.0f / total;
#pragma unroll
    for (int w = 0; w < 4; ++w) scale[w] *= inv;
  };
  {
    const int qq = tid >> 4, d0 = (tid & 15) * 4;
    float scale[4];
    merged(qq, scale);
    f4 r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) r += *reinterpret_cast<const f4 *>(comb + (w * 16 + qq) * kAttnCombLd + d0) * scale[w];
    st8<COH>(a.ctx, ((b * S + qb * 16 + qq) * H + hh * HD + d0) * 2, pack_h4(r));
  }
  if (a.probs) {
    float scale[4];
    merged(l16, scale);
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) {
      const f4 pr = sc[tt] * scale[wave];
      const h4 ph = {(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};
      st8<false>(a.probs, (int)((((size_t)(b * NH + hh) * S + q) * S + (wave * TPW + tt) * 16 + g * 4) * 2), as_u2(ph));
    }
  }
}

// Items are dealt so that the 16-query blocks of one head run on one XCD (they share K and V),
// and, when the grid is large enough, on workgroups 64.. so that the workgroups of the
// out-projection can fetch their weight slice meanwhile.
__device__ __forceinline__ void attn_small_range(const Params &a, int stride, int *off, int *span) {
  *span = xcd_item_span(a.S / 16, a.B * NH);
  *off = (*span + 64 <= stride) ? 64 : 0;
}
template <bool COH, int NKT>
__device__ __forceinline__ void stage_attn_small_t(unsigned char *lds, const Params &a, int first, int stride, Flow *fl = nullptr) {
  int off, span;
  attn_small_range(a, stride, &off, &span);
  for (int it = first - off; it < span; it += stride) {
    int qb, bh;
    if (it >= 0 && xcd_item(it, a.S / 16, a.B * NH, &qb, &bh)) attn_item_split<COH, NKT>(lds, a, bh, qb, fl);
  }
}
// Does this workgroup have an attention item?
__device__ __forceinline__ bool attn_small_busy(const Params &a, int first, int stride) {
  int off, span;
  attn_small_range(a, stride, &off, &span);
  for (int it = first - off; it < span; it += stride) {
    int qb, bh;
    if (it >= 0 && xcd_item(it, a.S / 16, a.B * NH, &qb, &bh)) return true;
  }
  return false;
}
template <bool COH>
__device__ __forceinline__ void stage_attn_small(unsigned char *lds, const Params &a, int first, int stride) {
  switch (a.S) {
    case 64: stage_attn_small_t<COH, 4>(lds, a, first, stride); break;
    case 128: stage_attn_small_t<COH, 8>(lds, a, first, stride); break;
    case 256: stage_attn_small_t<COH, 16>(lds, a, first, stride); break;
    case 384: stage_attn_small_t<COH, 24>(lds, a, first, stride); break;
    default: stage_attn_small_t<COH, 32>(lds, a, first, stride); break;   // 512 (validated on the host)
  }
}

// Work unit `it` (units it, it + 8, ... run on one XCD: workgroup b runs on XCD b % 8) -> attention
// item.  The S / 64 query blocks of a head go to the same XCD, next to each other in time, so that
// its L2 fetches the head's K and V once (at S = 128, B = 32: 19 MB instead of 30 MB per layer).
__device__ __forceinline__ int attn_item_of(int it, int qblocks, int items) {
  if ((gridDim.x & 7) != 0 || items % (8 * qblocks) != 0) return it;
  const int x = it & 7, i = it >> 3;
  return ((i / qblocks) * 8 + x) * qblocks + i % qblocks;
}
template <bool COH, int NKT>
__device__ __forceinline__ void stage_attn_t(half_t *lds, const Params &a, int first, int stride) {
  const int items = a.B * NH * (a.S / 64);
  if constexpr (2 * kAttnItemLds<NKT> <= kBigLds)     // (the megakernel's LDS allocation is at least this)
    attn_items_pipelined<COH, NKT>(reinterpret_cast<unsigned char *>(lds), a, first, stride, items,
                                   [&](int it) { return attn_item_of(it, a.S / 64, items); });
  else
    for (int it = first; it < items; it += stride) attn_item<COH, NKT>(lds, a, attn_item_of(it, a.S / 64, items));
}
// The attention items of the sequences of a group of 256-row blocks that holds whole sequences (48 items
// per row block whatever S is), three to each of the group's tiles, for the tiles of this workgroup.
template <bool COH, int NKT>
__device__ __forceinline__ void stage_attn_rowblock(unsigned char *lds, const Params &a, int first, int stride) {
  const int m_tiles = a.M / 256;
  for (int it = first; it < m_tiles * 16; it += stride) {
    int tm, tn;
    big_tile(it, m_tiles, 16, &tm, &tn);
    const int base = tm * 48 + tn * 3;           // (the tiles of a group are numbered through: 16 tm + tn)
    if constexpr (2 * kAttnItemLds<NKT> <= kBigLds)
      attn_items_pipelined<COH, NKT>(lds, a, 0, 1, 3, [&](int j) { return base + j; });
    else
      for (int j = 0; j < 3; ++j) attn_item<COH, NKT>(reinterpret_cast<half_t *>(lds), a, base + j);
  }
}
template <bool COH>
__device__ __forceinline__ void stage_attn(half_t *lds, const Params &a, int first, int stride) {
  const int items = a.B * NH * (a.S / 64);
  for (int it = first; it < items; it += stride) {
    const int item = attn_item_of(it, a.S / 64, items);
    switch (a.S) {
      case 64: attn_item<COH, 4>(lds, a, item); break;
      case 128: attn_item<COH, 8>(lds, a, item); break;
      case 256: attn_item<COH, 16>(lds, a, item); break;
      case 384: attn_item<COH, 24>(lds, a, item); break;
      default: attn_item<COH, 32>(lds, a, item); break;   // 512 (validated on the host)
    }
  }
}

using TileSmall = GemmTile<64, 64, 64, 2, 2>;
using TileLarge = GemmTile<128, 128, 64, 2, 2>;
constexpr int kAttnLdsBytes = attn_small_lds_bytes(512) > 2 * 512 * 128 + 64 * 128 ? attn_small_lds_bytes(512) : 2 * 512 * 128 + 64 * 128;
constexpr int lds_bytes(bool large) {
  const int t = large ? (TileLarge::LDS_BYTES > kBigLds ? TileLarge::LDS_BYTES : kBigLds) : kSmallGemmLds;
  return t > kAttnLdsBytes ? t : kAttnLdsBytes;
}

// ------------------------------------------------------------ megakernel ----
// MODE 0: skinny path (M < 1024); 1: 128 x 128 tiles; 2: 256-row tiles (M >= 1024, a multiple of 256)
template <int MODE, int NKT>
__global__ void __launch_bounds__(256) k_encoder_mega(Args args) {
  constexpr bool LARGE = MODE != 0, BIG = MODE == 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  half_t *lds = reinterpret_cast<half_t *>(lds_raw);
  using Tile = typename std::conditional<LARGE, TileLarge, TileSmall>::type;
  GridBarrier bar;
  grid_barrier_begin(bar, args.ctl);
  bar.trace = args.trace;
  bar.trace_cap = args.trace_cap;
  const int first = blockIdx.x, stride = gridDim.x;
  const int wave = threadIdx.x >> 6;
  const half_t *xin = args.x;
  bool qkv_ready = false;
  // this kernel leaves data in the workspace buffers: the dataflow kernel must refill them
  if (first == 0 && threadIdx.x == 0) __hip_atomic_store(args.ctl + kCtlFlowWord, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if constexpr (BIG) {   // the row-block hand-over words start every launch at 0
    for (int i = first * 256 + threadIdx.x; i < (args.M / 256) * 16; i += stride * 256)
      __hip_atomic_store(args.rbflags + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    grid_sync(bar);
  }
  for (int l = 0; l < args.num_layers; ++l) {
    const LayerW w = args.layers[l];
    const Params a = layer_params(args, l);
    half_t *yout = (l == a.num_layers - 1) ? a.y : a.yl;
    if constexpr (BIG) {
      // Where a 256-row block (S = 64, 128, 256) or a group of 2 (S = 512) or 3 (S = 384) of them holds
      // whole sequences, every stage of a group's tiles reads only what the tiles of the same group
      // wrote in the stage before (attention included: the 48 items per row block go three to a tile),
      // and the tile-to-workgroup mapping is the same in every stage: the 16 row blocks of M = 4096 then
      // run as independent groups of 16 workgroups that hand over among themselves (rowblock_sync).
      // Otherwise (a number of row blocks that is no multiple of the group) the stages are separated by
      // grid barriers.  Hand-over k of layer l carries the tag 7 l + k.
      const int group = a.S <= 256 ? 1 : a.S == 512 ? 2 : 3;
      const bool local = kRowblockLocal && (group * 256) % a.S == 0 && (a.M / 256) % group == 0;
      auto sync = [&](unsigned k) {
        if (local) rowblock_sync(a, bar, 7u * l + k, first, stride, group, []() {});
        else grid_sync(bar);
      };
      big_qkv<true>(lds_raw, a, w, xin, first, stride, &bar);
      sync(1);
      if (local) stage_attn_rowblock<true, NKT>(lds_raw, a, first, stride);
      else stage_attn_t<true, NKT>(lds, a, first, stride);
      sync(2);
      big_presum<true>(lds_raw, a, a.ctx, H, w.w_o, w.b_o, first, stride);
      rowblock_ln<true, 1>(a, bar, 7u * l + 3u, a.z1, xin, w.ln1_g, w.ln1_b, a.y1, first, stride);
      sync(4);
      big_fc1<true>(lds_raw, a, w, first, stride, &bar);
      sync(5);
      big_presum2<true>(lds_raw, a, a.h, F, w.w_fc2, w.b_fc2, first, stride);
      rowblock_ln<true, kFc2Split>(a, bar, 7u * l + 6u, fc2_sums(a), a.y1, w.ln2_g, w.ln2_b, yout, first, stride);
      if (l + 1 < a.num_layers) {   // the next layer writes this layer's buffers again: see Params
        auto invalidate = [&]() { if (threadIdx.x < 64) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); };
        if (local) rowblock_sync(a, bar, 7u * l + 7u, first, stride, group, invalidate);
        else grid_sync(bar, invalidate);
      }
    } else if constexpr (LARGE) {
      stage_qkv<true, Tile>(lds, a, w, xin, first, stride);
      grid_sync(bar);
      stage_attn_t<true, NKT>(lds, a, first, stride);
      grid_sync(bar);
      stage_partial<true, Tile>(lds, a, a.ctx, H, w.w_o, a.splitk_o, first, stride);
      grid_sync(bar);
      stage_ln<true>(a, a.splitk_o, w.b_o, xin, w.ln1_g, w.ln1_b, a.y1, first * 4 + wave, stride * 4);
      grid_sync(bar);
      stage_fc1<true, Tile>(lds, a, w, first, stride);
      grid_sync(bar);
      stage_partial<true, Tile>(lds, a, a.h, F, w.w_fc2, a.splitk_f, first, stride);
      grid_sync(bar);
      stage_ln<true>(a, a.splitk_f, w.b_fc2, a.y1, w.ln2_g, w.ln2_b, yout, first * 4 + wave, stride * 4);
    } else {
      // Weight slices are queued one stage ahead, from inside the grid barrier that precedes
      // the stage.
      const OutItems out_items{w.w_o, a.M};
      const Fc1Items fc1_items{w.w_fc1, a.M};
      const Fc2Items fc2_items{w.w_fc2, a.M};
      bool out_ready = false, fc1_ready = false, fc2_ready = false;
      small_qkv<true>(lds_raw, a, w, xin, qkv_ready, &bar);
      // (a workgroup that has an attention item would wait for the slice inside attention: it asks later)
      int attn_off, attn_span;
      attn_small_range(a, stride, &attn_off, &attn_span);
      const bool attn_busy = first >= attn_off && first < attn_off + attn_span;
      grid_sync(bar, [&]() { if (!attn_busy) out_ready = preissue_w<OsFull>(lds_raw, out_items); });
      stage_attn_small_t<true, NKT>(lds_raw, a, first, stride);
      grid_sync(bar, [&]() { if (!out_ready) out_ready = preissue_w<OsFull>(lds_raw, out_items); });
      small_outproj<true>(lds_raw, a, w, xin, out_ready, &bar);
      grid_sync(bar, [&]() { fc1_ready = preissue_w<OsFull>(lds_raw, fc1_items); });
      small_fc1<true>(lds_raw, a, w, fc1_ready, &bar);
      grid_sync(bar, [&]() { fc2_ready = preissue_w<OsFc2>(lds_raw, fc2_items); });
      small_fc2<true>(lds_raw, a, w, fc2_ready, &bar);
      grid_sync(bar);
      stage_ln<true>(a, a.splitk_f, w.b_fc2, a.y1, w.ln2_g, w.ln2_b, yout, wave * stride + first, stride * 4);
    }
    qkv_ready = false;
    if (l + 1 < a.num_layers) {
      if constexpr (BIG) {}          // (done above)
      else if constexpr (LARGE) grid_sync(bar);
      else grid_sync(bar, [&]() { qkv_ready = preissue_w<OsFull>(lds_raw, QkvItems{args.layers[l + 1].w_qkv, a.M}); });
    }
    xin = yout;
  }
  grid_barrier_end(bar);
}

// ------------------------------------------------- dataflow megakernel ----
// The skinny path without grid barriers between stages: every consumer polls its input (see
// Flow above).  Buffers are per layer; a layer's buffers are put back into the unwritten state
// by the workgroups that run FC1 items of the NEXT layer, after their own input has arrived:
// a complete row tile of z1(l+1) implies, through the chain of dependencies (context rows <-
// all keys and values <- all rows of the layer input <- every LayerNorm-2 row of layer l <- all
// FC2 partials <- all of h <- all FC1 items <- ...), that every buffer of layer l except its
// output has been read for the last time.  The layer output is still being read by layer l+1
// (queries, residual) and is reset one layer later.  What is left at the end is reset after
// one grid barrier.  Between launches every buffer is therefore in the unwritten state, which
// the control block records as a layout marker; a launch that does not find its marker (first
// use, another layout, an earlier failure, or another kernel having used the workspace) fills
// the buffers first.
__device__ __forceinline__ void fill_unwritten(void *base, size_t bytes, int part, int parts) {
  const size_t n16 = bytes / 16, per = (n16 + parts - 1) / parts;
  const size_t b = per * part, e = b + per < n16 ? b + per : n16;
  const u4 pat = {~0u, ~0u, ~0u, ~0u};
  for (size_t i = b + threadIdx.x; i < e; i += 256)
    st16<true>(base, (int)(i * 16), pat);          // a layer's buffers span far less than 2 GiB
}

template <int NKT>
__global__ void __launch_bounds__(256) k_encoder_flow(Args args) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  GridBarrier bar;
  grid_barrier_begin(bar, args.ctl);
  Flow fl;
  fl.failed = false;
  fl.trace = args.trace;
  fl.trace_cap = args.trace_cap;
  fl.stage = 0;
  const int first = blockIdx.x, stride = gridDim.x, wave = threadIdx.x >> 6;
  const int L = args.num_layers, M = args.M;
  if (__hip_atomic_load(args.ctl + kCtlFlowWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != args.flow_marker) {
    for (int l = 0; l < L; ++l)
      fill_unwritten(reinterpret_cast<char *>(args.qkv) + (size_t)l * args.layer_stride, args.layer_stride, first, stride);
    grid_sync(bar);
  }
  // Weight slice prefetch: at most one slice is in flight or resident (the W region of LDS); it is
  // queued as soon as the region is free, for the next GEMM stage in which this workgroup has an
  // item.  `pf` names that stage (layer * 5 + position; positions 0 QKV, 1 attention, 2 out, 3 FC1, 4 FC2).
  int pf = -1;
  const bool attn_busy = attn_small_busy(args, first, stride);
  auto prefetch_after = [&](int l, int pos) {
    if (pf >= 0) return;
    for (int step = 1; step <= 5; ++step) {
      const int q = pos + step, ll = l + q / 5, pp = q % 5;
      if (ll >= L) return;
      if (pp == 1) { if (attn_busy) return; continue; }
      const LayerW &w = args.layers[ll];
      Item d;
      bool ok = false;
      if (pp == 0) { const QkvItems it{w.w_qkv, M}; ok = first < it.span() && it.at(first, d); }
      else if (pp == 2) { const OutItems it{w.w_o, M}; ok = first < it.span() && it.at(first, d); }
      else if (pp == 3) { const Fc1Items it{w.w_fc1, M}; ok = first < it.span() && it.at(first, d); }
      else { const Fc2Items it{w.w_fc2, M}; ok = first < it.span() && it.at(first, d); }
      if (ok) {
        OsFull::issue_w(lds_raw + kXRegion, d.W, d.ldw, d.n0, d.k0, d.rot);
        pf = ll * 5 + pp;
        return;
      }
    }
  };
  auto take = [&](int l, int pos) { const bool r = pf == l * 5 + pos; if (r) pf = -1; return r; };
  static_assert(std::is_same<OsFull, OsFc2>::value, "one slice shape for every stage");
  // workgroups that reset: those with an FC1 item (all `it` below the span are valid: 48 slices)
  const int fc1_span = Fc1Items{nullptr, M}.span();
  const int resetters = fc1_span < stride ? fc1_span : stride;

  prefetch_after(0, -1);
  const half_t *xin = args.x;
  for (int l = 0; l < L; ++l) {
    const LayerW w = args.layers[l];
    const Params a = layer_params(args, l);
    half_t *yout = (l == L - 1) ? a.y : a.yl;
    const bool in0 = l == 0;                       // the layer input is the caller's tensor: nothing to poll

    small_qkv<true>(lds_raw, a, w, xin, take(l, 0), nullptr, &fl, in0);
    flow_stamp(fl, 1); fl.stage++;
    prefetch_after(l, 0);

    stage_attn_small_t<true, NKT>(lds_raw, a, first, stride, &fl);
    flow_stamp(fl, 1); fl.stage++;
    if (attn_busy) { __syncthreads(); prefetch_after(l, 1); }

    small_outproj<true>(lds_raw, a, w, xin, take(l, 2), nullptr, &fl, in0);
    flow_stamp(fl, 1); fl.stage++;
    prefetch_after(l, 2);

    small_fc1<true>(lds_raw, a, w, take(l, 3), nullptr, &fl);
    flow_stamp(fl, 1); fl.stage++;
    prefetch_after(l, 3);
    if (l >= 1 && first < resetters) {
      fill_unwritten(reinterpret_cast<char *>(args.qkv) + (size_t)(l - 1) * args.layer_stride, args.flow_bytes, first, resetters);
      if (l >= 2) fill_unwritten(reinterpret_cast<char *>(args.yl) + (size_t)(l - 2) * args.layer_stride, (size_t)M * H * 2, first, resetters);
    }

    small_fc2<true>(lds_raw, a, w, take(l, 4), nullptr, &fl);
    flow_stamp(fl, 1); fl.stage++;
    prefetch_after(l, 4);

    stage_ln<true>(a, a.splitk_f, w.b_fc2, a.y1, w.ln2_g, w.ln2_b, yout, wave * stride + first, stride * 4, &fl);
    flow_stamp(fl, 1); fl.stage++;
    xin = yout;
  }
  if (fl.failed && threadIdx.x == 0) (void)__hip_atomic_fetch_or(args.ctl + kCtlErrWord, 4u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  grid_sync(bar);                                  // everything has been consumed
  fill_unwritten(reinterpret_cast<char *>(args.qkv) + (size_t)(L - 1) * args.layer_stride, args.flow_bytes, first, stride);
  if (L >= 2) fill_unwritten(reinterpret_cast<char *>(args.yl) + (size_t)(L - 2) * args.layer_stride, (size_t)M * H * 2, first, stride);
  if (first == 0 && threadIdx.x == 0) {
    const unsigned err = __hip_atomic_load(args.ctl + kCtlErrWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(args.ctl + kCtlFlowWord, err ? 0u : args.flow_marker, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // (the refill is acknowledged before the wave ends: a pattern store still on its way when the next launch
  // writes the same word would put that word back into the "not written" state for good)
  __builtin_amdgcn_s_waitcnt(0);
  grid_barrier_end(bar);
}

// ------------------------------------------------------ per-op kernels ----
template <int MODE>
__global__ void __launch_bounds__(256) k_qkv(Args a, int l, const half_t *xin) {
  constexpr bool LARGE = MODE != 0, BIG = MODE == 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  // the per-op chain leaves data in the workspace buffers: the dataflow kernel must refill them
  if (blockIdx.x == 0 && threadIdx.x == 0) __hip_atomic_store(a.ctl + kCtlFlowWord, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  using Tile = typename std::conditional<LARGE, TileLarge, TileSmall>::type;
  if constexpr (LARGE) {
    if constexpr (BIG) big_qkv<false>(lds_raw, a, a.layers[l], xin, blockIdx.x, gridDim.x);
    else stage_qkv<false, Tile>(reinterpret_cast<half_t *>(lds_raw), a, a.layers[l], xin, blockIdx.x, gridDim.x);
  } else small_qkv<false>(lds_raw, a, a.layers[l], xin, false);
}
__global__ void __launch_bounds__(256) k_attn(Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  stage_attn<false>(reinterpret_cast<half_t *>(lds_raw), a, blockIdx.x, gridDim.x);
}
__global__ void __launch_bounds__(256) k_attn_small(Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  stage_attn_small<false>(lds_raw, a, blockIdx.x, gridDim.x);
}
template <int MODE>
__global__ void __launch_bounds__(256) k_partial(Args a, const half_t *X, int K, const half_t *W, int splitk) {
  constexpr bool LARGE = MODE != 0, BIG = MODE == 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  using Tile = typename std::conditional<LARGE, TileLarge, TileSmall>::type;
  if constexpr (LARGE) {
    static_assert(!BIG, "the 256-row path writes fp16 pre-LayerNorm sums: k_presum_big");
    stage_partial<false, Tile>(reinterpret_cast<half_t *>(lds_raw), a, X, K, W, splitk, blockIdx.x, gridDim.x);
  } else {
    LayerW w{};
    w.w_fc2 = W;
    small_fc2<false>(lds_raw, a, w, false);
  }
}
__global__ void __launch_bounds__(256) k_ln(Args a, int splitk, const half_t *bias, const half_t *resid,
                                            const half_t *gam, const half_t *bet, half_t *out) {
  stage_ln<false>(a, splitk, bias, resid, gam, bet, out, blockIdx.x * 4 + (threadIdx.x >> 6), gridDim.x * 4);
}
__global__ void __launch_bounds__(256) k_presum_big(Args a, const half_t *X, int K, const half_t *W, const half_t *bias) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  big_presum<false>(lds_raw, a, X, K, W, bias, blockIdx.x, gridDim.x);
}
__global__ void __launch_bounds__(256) k_presum2_big(Args a, const half_t *X, int K, const half_t *W, const half_t *bias) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  big_presum2<false>(lds_raw, a, X, K, W, bias, blockIdx.x, gridDim.x);
}
template <int NZ>
__global__ void __launch_bounds__(256) k_ln_big(Args a, const half_t *z, const half_t *resid, const half_t *gam, const half_t *bet, half_t *out) {
  big_ln<false, NZ>(a, z, resid, gam, bet, out, blockIdx.x * 4 + (threadIdx.x >> 6), gridDim.x * 4);
}
template <int MODE>
__global__ void __launch_bounds__(256) k_fc1(Args a, int l) {
  constexpr bool LARGE = MODE != 0, BIG = MODE == 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  using Tile = typename std::conditional<LARGE, TileLarge, TileSmall>::type;
  if constexpr (LARGE) {
    if constexpr (BIG) big_fc1<false>(lds_raw, a, a.layers[l], blockIdx.x, gridDim.x);
    else stage_fc1<false, Tile>(reinterpret_cast<half_t *>(lds_raw), a, a.layers[l], blockIdx.x, gridDim.x);
  } else small_fc1<false>(lds_raw, a, a.layers[l], false);
}
__global__ void __launch_bounds__(256) k_outproj_small(Args a, int l, const half_t *xin) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  small_outproj<false>(lds_raw, a, a.layers[l], xin, false);
}

// ---- sequence lengths that are not built: rows copied into / out of a padded layout ----
// xp[b][s][:] = s < S ? x[b][s][:] : 0, 16 bytes per thread.
__global__ void __launch_bounds__(256) k_pad_rows(const half_t *x, half_t *xp, int B, int S, int SP) {
  const int n = B * SP * (H / 8);
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const int g = i % (H / 8), r = i / (H / 8), b = r / SP, sq = r - b * SP;
    u4 v = {0u, 0u, 0u, 0u};
    if (sq < S) v = *reinterpret_cast<const u4 *>(x + ((size_t)(b * S + sq) * H + g * 8));
    *reinterpret_cast<u4 *>(xp + (size_t)i * 8) = v;
  }
}
// y[b][s][:] = yp[b][s][:] for s < S.
__global__ void __launch_bounds__(256) k_unpad_rows(const half_t *yp, half_t *y, int B, int S, int SP) {
  const int n = B * S * (H / 8);
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const int g = i % (H / 8), r = i / (H / 8), b = r / S, sq = r - b * S;
    *reinterpret_cast<u4 *>(y + (size_t)i * 8) = *reinterpret_cast<const u4 *>(yp + ((size_t)(b * SP + sq) * H + g * 8));
  }
}
// mp[b][q][k] = k >= S ? -10000 : (q < S and mask given ? mask[b][q][k] : 0): exp(-10000 - max) is 0 in
// fp32, so the surplus keys take no part in any softmax.
__global__ void __launch_bounds__(256) k_pad_mask(const half_t *mask, half_t *mp, int B, int S, int SP) {
  const int n = B * SP * SP;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const int k = i % SP, r = i / SP, b = r / SP, q = r - b * SP;
    half_t v = (half_t)0.0f;
    if (k >= S) v = (half_t)-10000.0f;
    else if (mask && q < S) v = mask[((size_t)b * S + q) * S + k];
    mp[i] = v;
  }
}

// ------------------------------------------------------------------- host ----
constexpr int kBigSets = 1;     // buffer sets the many-rows megakernel rotates through (1: 1604 us at 4096 rows, 2: 1777, 3: 1787, one per layer: 1808)
struct Plan {
  bool large, big;
  int splitk_o, splitk_f;
  size_t off_ctl, off_qkv, off_ctx, off_z1, off_y1, off_h, off_yl, off_part, layer_stride, total;
  int layer_sets;
  size_t flow_bytes;      // a layer's buffers without its output (which comes last)
  size_t off_xpad, off_ypad, off_maskpad;
  size_t off_rbflags;     // 16 words per 256-row block (many-rows megakernel only)
  unsigned flow_marker;
};

// The attention tiles are built for these sequence lengths; any other length up to 512 runs as the
// next one of them with the surplus key positions masked out (rows copied in and out, see run_padded).
static int padded_len(int s) { return s <= 64 ? 64 : s <= 128 ? 128 : s <= 256 ? 256 : s <= 384 ? 384 : 512; }

static int validate(const souffle_bert_cfg *c) {
  if (!c) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  if (c->hidden != H || c->heads != NH || c->ffn != F)
    return fail(SOUFFLE_ERR_SHAPE, "only hidden=768 heads=12 ffn=3072 is built (got %d/%d/%d)", c->hidden, c->heads, c->ffn);
  if (c->batch <= 0 || c->seq_len <= 0) return fail(SOUFFLE_ERR_SHAPE, "batch and seq_len must be positive");
  if (c->seq_len > 512) return fail(SOUFFLE_ERR_SHAPE, "seq_len must be at most 512 (got %d)", c->seq_len);
  const int s = padded_len(c->seq_len);          // other lengths run padded to the next built one
  const long long m = (long long)c->batch * s;
  if (m >= 1024 && m % 128 != 0) return fail(SOUFFLE_ERR_SHAPE, "batch*seq_len >= 1024 must be a multiple of 128 (got %lld)", m);
  if (m > 65536) return fail(SOUFFLE_ERR_SHAPE, "batch*seq_len must be <= 65536 (got %lld)", m);
  if (c->act != SOUFFLE_ACT_GELU_TANH && c->act != SOUFFLE_ACT_RELU) return fail(SOUFFLE_ERR_SHAPE, "unknown activation %d", c->act);
  if (!(c->ln_eps >= 0.f)) return fail(SOUFFLE_ERR_SHAPE, "ln_eps must be >= 0");
  return SOUFFLE_OK;
}

static Plan make_plan(const souffle_bert_cfg *c, int num_layers) {
  Plan p;
  const size_t M = (size_t)c->batch * padded_len(c->seq_len);
  p.large = M >= 1024;
  p.big = M >= 1024 && M % 256 == 0;     // (12 layers at M = 1024: 1222 us, with the 128 x 128 tiles 1409 us; at M = 1536: 1225 against 1661)
  p.splitk_o = 1;
  p.splitk_f = p.large ? 1 : kSplitFc2Small;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += round_up(bytes, 256); return o; };
  p.off_ctl = take(kCtlWords * 4);
  const size_t first = off;
  p.off_qkv = take(3 * M * H * 2);
  p.off_ctx = take(M * H * 2);
  p.off_z1 = take(M * H * 2);
  p.off_y1 = take(M * H * 2);
  p.off_h = take(M * F * 2);
  // fp32 split-K partial sums, or (many rows) FC2's kFc2Split fp16 pre-LayerNorm partial sums
  p.off_part = take(p.big ? (size_t)kFc2Split * M * H * 2 : (size_t)(p.splitk_f > p.splitk_o ? p.splitk_f : p.splitk_o) * M * H * 4);
  p.off_yl = take(M * H * 2);
  p.layer_stride = off - first;                       // one set of inter-stage buffers per layer
  p.flow_bytes = p.off_yl - p.off_qkv;
  const int nl = num_layers < 1 ? 1 : num_layers;
  p.layer_sets = p.big && nl > kBigSets ? kBigSets : nl;
  p.total = first + p.layer_stride * (size_t)p.layer_sets;
  // (in front of the padding area: the plan of the padded configuration, which lacks that area, must agree)
  p.off_rbflags = 0;
  if (p.big) {
    off = p.total;
    p.off_rbflags = take(M / 256 * 64);
    p.total = off;
  }
  // a sequence length that is not built: padded copies of x and y and the padded additive mask
  p.off_xpad = p.off_ypad = p.off_maskpad = 0;
  if (padded_len(c->seq_len) != c->seq_len) {
    off = p.total;
    p.off_xpad = take(M * H * 2);
    p.off_ypad = take(M * H * 2);
    p.off_maskpad = take(M * (size_t)padded_len(c->seq_len) * 2);
    p.total = off;
  }
  // names the layout (rows, layers, extent) in the control block; never 0
  p.flow_marker = (unsigned)((M * 2654435761ull) ^ ((size_t)num_layers * 40503ull) ^ (p.total >> 4)) | 0x80000000u;
  return p;
}

static int fill_args(Args &a, const souffle_bert_cfg *c, const souffle_bert_layer_w *layers, int nl,
                     const void *x, const void *mask, void *y, const souffle_bert_dump *dump,
                     void *ws, size_t ws_bytes, const Plan &p) {
  if (!layers || !x || !y) return fail(SOUFFLE_ERR_NULL, "layers, x and y must not be NULL");
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL (need %zu bytes)", p.total);
  if (ws_bytes < p.total) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, p.total);
  if (nl < 1 || nl > kMaxLayers) return fail(SOUFFLE_ERR_SHAPE, "num_layers must be in 1..%d (got %d)", kMaxLayers, nl);
  if (!aligned16(x) || !aligned16(y) || !aligned16(ws) || (mask && !aligned16(mask)))
    return fail(SOUFFLE_ERR_ALIGN, "x, y, mask and workspace must be 16-byte aligned");
  char *base = static_cast<char *>(ws);
  a.B = c->batch; a.S = c->seq_len; a.M = c->batch * c->seq_len; a.act = c->act; a.num_layers = nl;
  a.splitk_o = p.splitk_o; a.splitk_f = p.splitk_f; a.scale = c->scale; a.eps = c->ln_eps;
  a.big = p.big ? 1 : 0;
  a.x = static_cast<const half_t *>(x); a.mask = static_cast<const half_t *>(mask); a.y = static_cast<half_t *>(y);
  a.ctl = reinterpret_cast<unsigned *>(base + p.off_ctl);
  a.rbflags = p.big ? reinterpret_cast<unsigned *>(base + p.off_rbflags) : nullptr;
  a.qkv = reinterpret_cast<half_t *>(base + p.off_qkv);
  a.ctx = reinterpret_cast<half_t *>(base + p.off_ctx);
  a.z1 = reinterpret_cast<half_t *>(base + p.off_z1);
  a.y1 = reinterpret_cast<half_t *>(base + p.off_y1);
  a.h = reinterpret_cast<half_t *>(base + p.off_h);
  a.yl = reinterpret_cast<half_t *>(base + p.off_yl);
  a.layer_stride = p.layer_stride;
  a.layer_sets = p.layer_sets;
  a.flow_bytes = p.flow_bytes;
  a.flow_marker = p.flow_marker;
  a.part = reinterpret_cast<float *>(base + p.off_part);
  a.probs = nullptr;
  a.trace = nullptr;
  a.trace_cap = 0;
  if (dump) {   // the per-stage tensors are produced in the reference's own layouts: write them in place
    if (dump->qkv) a.qkv = static_cast<half_t *>(dump->qkv);
    if (dump->ctx) a.ctx = static_cast<half_t *>(dump->ctx);
    if (dump->ln1) a.y1 = static_cast<half_t *>(dump->ln1);
    if (dump->fc1) a.h = static_cast<half_t *>(dump->fc1);
    a.probs = static_cast<half_t *>(dump->probs);
    if (!aligned16(a.qkv) || !aligned16(a.ctx) || !aligned16(a.y1) || !aligned16(a.h) || !aligned16(a.probs))
      return fail(SOUFFLE_ERR_ALIGN, "dump pointers must be 16-byte aligned");
  }
  for (int l = 0; l < nl; ++l) {
    const souffle_bert_layer_w &s = layers[l];
    if (!s.w_qkv || !s.w_o || !s.w_fc1 || !s.w_fc2) return fail(SOUFFLE_ERR_NULL, "layer %d: a weight matrix is NULL", l);
    const void *ptrs[12] = {s.w_qkv, s.b_qkv, s.w_o, s.b_o, s.ln1_g, s.ln1_b, s.w_fc1, s.b_fc1, s.w_fc2, s.b_fc2, s.ln2_g, s.ln2_b};
    for (const void *q : ptrs)
      if (!aligned16(q)) return fail(SOUFFLE_ERR_ALIGN, "layer %d: a weight/bias pointer is not 16-byte aligned", l);
    LayerW &d = a.layers[l];
    d.w_qkv = (const half_t *)s.w_qkv; d.b_qkv = (const half_t *)s.b_qkv; d.w_o = (const half_t *)s.w_o; d.b_o = (const half_t *)s.b_o;
    d.ln1_g = (const half_t *)s.ln1_g; d.ln1_b = (const half_t *)s.ln1_b; d.w_fc1 = (const half_t *)s.w_fc1; d.b_fc1 = (const half_t *)s.b_fc1;
    d.w_fc2 = (const half_t *)s.w_fc2; d.b_fc2 = (const half_t *)s.b_fc2; d.ln2_g = (const half_t *)s.ln2_g; d.ln2_b = (const half_t *)s.ln2_b;
  }
  return SOUFFLE_OK;
}

template <int MODE, int NKT>
static int launch_mega_t(Args &a, int grid, hipStream_t st) {
  const int lds = lds_bytes(MODE != 0);
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_encoder_mega<MODE, NKT>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    attr_done = true;
  }
  void *args[] = {&a};
  return launch_persistent((const void *)k_encoder_mega<MODE, NKT>, grid, 256, args, lds, st);
}
// one kernel per supported sequence length, so that each carries only its own attention tile
template <int MODE>
static int launch_mega(Args &a, int grid, hipStream_t st) {
  switch (a.S) {
    case 64: return launch_mega_t<MODE, 4>(a, grid, st);
    case 128: return launch_mega_t<MODE, 8>(a, grid, st);
    case 256: return launch_mega_t<MODE, 16>(a, grid, st);
    case 384: return launch_mega_t<MODE, 24>(a, grid, st);
    default: return launch_mega_t<MODE, 32>(a, grid, st);
  }
}

template <int NKT>
static int launch_flow_t(Args &a, int grid, hipStream_t st) {
  const int lds = lds_bytes(false);
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_encoder_flow<NKT>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    attr_done = true;
  }
  void *args[] = {&a};
  return launch_persistent((const void *)k_encoder_flow<NKT>, grid, 256, args, lds, st);
}
static int launch_flow(Args &a, int grid, hipStream_t st) {
  switch (a.S) {
    case 64: return launch_flow_t<4>(a, grid, st);
    case 128: return launch_flow_t<8>(a, grid, st);
    case 256: return launch_flow_t<16>(a, grid, st);
    case 384: return launch_flow_t<24>(a, grid, st);
    default: return launch_flow_t<32>(a, grid, st);
  }
}

// A sequence length that is not built runs as the next built one: x is copied into a zero-padded
// layout, the additive mask is extended so that the surplus keys drop out of every softmax, and the
// first S rows of every sequence are copied back.  Returns the configuration and pointers the
// kernels see (`before`), and copies the result out (`after`).
struct Padded {
  souffle_bert_cfg cfg;
  const void *x, *mask;
  void *y;
  bool on;
};
static int pad_before(Padded &pd, const souffle_bert_cfg *c, const void *x, const void *mask, void *y, const souffle_bert_dump *dump,
                      void *ws, size_t ws_bytes, const Plan &p, int num_cus, hipStream_t st) {
  pd.cfg = *c; pd.x = x; pd.mask = mask; pd.y = y;
  pd.on = padded_len(c->seq_len) != c->seq_len;
  if (!pd.on) return SOUFFLE_OK;
  if (dump) return fail(SOUFFLE_ERR_SHAPE, "per-stage tensors need seq_len in {64,128,256,384,512} (got %d)", c->seq_len);
  if (!x || !y) return fail(SOUFFLE_ERR_NULL, "layers, x and y must not be NULL");
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL (need %zu bytes)", p.total);
  if (ws_bytes < p.total) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, p.total);
  if (!aligned16(x) || !aligned16(y) || !aligned16(ws))
    return fail(SOUFFLE_ERR_ALIGN, "x, y and workspace must be 16-byte aligned");
  char *base = static_cast<char *>(ws);
  const int SP = padded_len(c->seq_len);
  pd.cfg.seq_len = SP;
  pd.x = base + p.off_xpad; pd.y = base + p.off_ypad; pd.mask = base + p.off_maskpad;
  const int cap = num_cus * 8;
  auto grid_for = [&](long long n) { const long long g = (n + 255) / 256; return (int)(g < cap ? g : cap); };
  hipLaunchKernelGGL(k_pad_rows, dim3(grid_for((long long)c->batch * SP * (H / 8))), dim3(256), 0, st, static_cast<const half_t *>(x),
                     reinterpret_cast<half_t *>(base + p.off_xpad), c->batch, c->seq_len, SP);
  hipLaunchKernelGGL(k_pad_mask, dim3(grid_for((long long)c->batch * SP * SP)), dim3(256), 0, st, static_cast<const half_t *>(mask),
                     reinterpret_cast<half_t *>(base + p.off_maskpad), c->batch, c->seq_len, SP);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}
static int pad_after(const Padded &pd, const souffle_bert_cfg *c, void *y, int num_cus, hipStream_t st) {
  if (!pd.on) return SOUFFLE_OK;
  const long long n = (long long)c->batch * c->seq_len * (H / 8);
  const long long g = (n + 255) / 256;
  hipLaunchKernelGGL(k_unpad_rows, dim3((int)(g < num_cus * 8 ? g : num_cus * 8)), dim3(256), 0, st, static_cast<const half_t *>(pd.y),
                     static_cast<half_t *>(y), c->batch, c->seq_len, pd.cfg.seq_len);
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

static int run_fused(const souffle_bert_cfg *c, const souffle_bert_layer_w *layers, int nl, const void *x_in,
                     const void *mask_in, void *y_out, const souffle_bert_dump *dump, void *ws, size_t ws_bytes,
                     souffle_stream_t stream) {
  if (int rc = validate(c)) return rc;
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  if (!df.cooperative) return fail(SOUFFLE_ERR_DEVICE, "device does not support cooperative launch");
  const Plan p = make_plan(c, nl);
  Padded pd;
  if (int rc = pad_before(pd, c, x_in, mask_in, y_out, dump, ws, ws_bytes, p, df.num_cus, static_cast<hipStream_t>(stream))) return rc;
  if (pd.on) {
    const int rc = run_fused(&pd.cfg, layers, nl, pd.x, pd.mask, pd.y, nullptr, ws, ws_bytes, stream);
    return rc ? rc : pad_after(pd, c, y_out, df.num_cus, static_cast<hipStream_t>(stream));
  }
  const void *x = x_in, *mask = mask_in;
  void *y = y_out;
  static thread_local Args a;
  if (int rc = fill_args(a, c, layers, nl, x, mask, y, dump, ws, ws_bytes, p)) return rc;
  stage_trace(&a.trace, &a.trace_cap, df.num_cus);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Skinny shapes run the dataflow kernel unless per-stage tensors are asked for (those are the
  // caller's buffers, which do not start in the unwritten state) or it has been switched off.
  if (!p.large && !dump && bert_sync_mode() == SOUFFLE_SYNC_DATAFLOW) return launch_flow(a, df.num_cus, st);
  return p.big ? launch_mega<2>(a, df.num_cus, st) : p.large ? launch_mega<1>(a, df.num_cus, st) : launch_mega<0>(a, df.num_cus, st);
}

template <int MODE>
static int run_unfused_t(Args &a, int nl, int num_cus, hipStream_t st) {
  constexpr bool LARGE = MODE != 0;
  constexpr int GEMM_LDS = LARGE ? lds_bytes(true) : kSmallGemmLds;
  constexpr int BN = LARGE ? 128 : 64;
  constexpr int BM_QKV = LARGE ? 128 : OsFull::kBM, BM_OUT = LARGE ? 128 : OsFull::kBM, BM_FC2 = LARGE ? 128 : OsFc2::kBM;
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_qkv<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    if constexpr (MODE == 2) {
      SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_presum_big, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
      SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_presum2_big, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    }
    else SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_partial<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_fc1<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS));
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_attn, hipFuncAttributeMaxDynamicSharedMemorySize, kAttnLdsBytes));
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_attn_small, hipFuncAttributeMaxDynamicSharedMemorySize, kAttnLdsBytes));
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)k_outproj_small, hipFuncAttributeMaxDynamicSharedMemorySize, kSmallGemmLds));
    attr_done = true;
  }
  const int cap = num_cus * 4;
  auto grid_for = [&](int items) { return items < cap ? items : cap; };
  const half_t *xin = a.x;
  for (int l = 0; l < nl; ++l) {
    const LayerW &w = a.layers[l];
    half_t *yout = (l == nl - 1) ? a.y : a.yl;
    hipLaunchKernelGGL(k_qkv<MODE>, dim3(grid_for((a.M / BM_QKV) * (3 * H / BN))), dim3(256), GEMM_LDS, st, a, l, xin);
    if (LARGE) hipLaunchKernelGGL(k_attn, dim3(grid_for(a.B * NH * (a.S / 64))), dim3(256), 2 * a.S * 128 + 64 * 128, st, a);
    else hipLaunchKernelGGL(k_attn_small, dim3(grid_for((a.B * NH + 7) / 8 * 8 * (a.S / 16))), dim3(256), attn_small_lds_bytes(a.S), st, a);
    if constexpr (MODE == 2) {
      hipLaunchKernelGGL(k_presum_big, dim3(grid_for((a.M / 256) * 16)), dim3(256), GEMM_LDS, st, a, a.ctx, H, w.w_o, w.b_o);
      hipLaunchKernelGGL(k_ln_big<1>, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, (const half_t *)a.z1, xin, w.ln1_g, w.ln1_b, a.y1);
    } else if constexpr (LARGE) {
      hipLaunchKernelGGL(k_partial<MODE>, dim3(grid_for((a.M / BM_OUT) * (H / BN))), dim3(256), GEMM_LDS, st, a, a.ctx, H, w.w_o, 1);
      hipLaunchKernelGGL(k_ln, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, 1, w.b_o, xin, w.ln1_g, w.ln1_b, a.y1);
    } else {   // small M: LN1 is applied by the FC1 kernel on its LDS-resident rows
      hipLaunchKernelGGL(k_outproj_small, dim3(grid_for((a.M / BM_OUT) * (H / BN))), dim3(256), GEMM_LDS, st, a, l, xin);
    }
    hipLaunchKernelGGL(k_fc1<MODE>, dim3(grid_for((a.M / BM_QKV) * (F / BN))), dim3(256), GEMM_LDS, st, a, l);
    if constexpr (MODE == 2) {
      hipLaunchKernelGGL(k_presum2_big, dim3(grid_for((a.M / 256) * 16)), dim3(256), GEMM_LDS, st, a, a.h, F, w.w_fc2, w.b_fc2);
      hipLaunchKernelGGL(k_ln_big<kFc2Split>, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, (const half_t *)a.part, (const half_t *)a.y1, w.ln2_g, w.ln2_b, yout);
    } else {
      hipLaunchKernelGGL(k_partial<MODE>, dim3(grid_for((a.M / BM_FC2) * (H / BN) * a.splitk_f)), dim3(256), GEMM_LDS, st, a, a.h, F, w.w_fc2, a.splitk_f);
      hipLaunchKernelGGL(k_ln, dim3(grid_for((a.M + 3) / 4)), dim3(256), 0, st, a, a.splitk_f, w.b_fc2, a.y1, w.ln2_g, w.ln2_b, yout);
    }
    xin = yout;
  }
  SOUFFLE_HIP_TRY(hipGetLastError());
  return SOUFFLE_OK;
}

static int run_unfused(const souffle_bert_cfg *c, const souffle_bert_layer_w *layers, int nl, const void *x,
                       const void *mask, void *y, const souffle_bert_dump *dump, void *ws, size_t ws_bytes,
                       souffle_stream_t stream) {
  if (int rc = validate(c)) return rc;
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const Plan p = make_plan(c, nl);
  Padded pd;
  if (int rc = pad_before(pd, c, x, mask, y, dump, ws, ws_bytes, p, df.num_cus, static_cast<hipStream_t>(stream))) return rc;
  if (pd.on) {
    const int rc = run_unfused(&pd.cfg, layers, nl, pd.x, pd.mask, pd.y, nullptr, ws, ws_bytes, stream);
    return rc ? rc : pad_after(pd, c, y, df.num_cus, static_cast<hipStream_t>(stream));
  }
  static thread_local Args a;
  if (int rc = fill_args(a, c, layers, nl, x, mask, y, dump, ws, ws_bytes, p)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return p.big ? run_unfused_t<2>(a, nl, df.num_cus, st) : p.large ? run_unfused_t<1>(a, nl, df.num_cus, st) : run_unfused_t<0>(a, nl, df.num_cus, st);
}

}  // namespace bert
}  // namespace souffle

using namespace souffle;

extern "C" size_t souffle_bert_workspace_bytes(const souffle_bert_cfg *cfg) {
  if (bert::validate(cfg)) return 0;
  const int nl = cfg->num_layers < 1 ? 1 : (cfg->num_layers > bert::kMaxLayers ? bert::kMaxLayers : cfg->num_layers);
  return bert::make_plan(cfg, nl).total;
}
extern "C" int souffle_bert_layer_fused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *w, const void *x,
                                        const void *mask, void *y, const souffle_bert_dump *dump, void *ws,
                                        size_t ws_bytes, souffle_stream_t stream) {
  return bert::run_fused(cfg, w, 1, x, mask, y, dump, ws, ws_bytes, stream);
}
extern "C" int souffle_bert_layer_unfused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *w, const void *x,
                                          const void *mask, void *y, const souffle_bert_dump *dump, void *ws,
                                          size_t ws_bytes, souffle_stream_t stream) {
  return bert::run_unfused(cfg, w, 1, x, mask, y, dump, ws, ws_bytes, stream);
}
extern "C" int souffle_bert_encoder_fused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                                          const void *x, const void *mask, void *y, void *ws, size_t ws_bytes,
                                          souffle_stream_t stream) {
  if (!cfg) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  return bert::run_fused(cfg, layers, cfg->num_layers, x, mask, y, nullptr, ws, ws_bytes, stream);
}
extern "C" int souffle_bert_encoder_unfused(const souffle_bert_cfg *cfg, const souffle_bert_layer_w *layers,
                                            const void *x, const void *mask, void *y, void *ws, size_t ws_bytes,
                                            souffle_stream_t stream) {
  if (!cfg) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  return bert::run_unfused(cfg, layers, cfg->num_layers, x, mask, y, nullptr, ws, ws_bytes, stream);
}
