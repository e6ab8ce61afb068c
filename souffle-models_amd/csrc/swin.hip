// Swin-Base stage-1 block pair (regular + shifted window) as one persistent cooperative
// kernel on gfx950, plus the reference's fused two-GEMM Swin FFN and the host index maps.
//
// A block is window-local up to its residual, so one workgroup runs a whole block for one
// 7x7 window without any grid barrier: gather (roll + partition folded into the row index)
// -> LN1 -> QKV -> per-head attention with relative-position bias and shifted-window mask
// -> proj + shortcut -> LN2 -> FC1 + GELU -> FC2 + shortcut -> scatter (reverse + roll back
// folded into the same row index).  Only the hand-over from the regular to the shifted
// block crosses workgroups (one grid barrier).  The 49 tokens of a window are padded to 64
// rows for the 16-row MFMA tiles; every intermediate stays in LDS.
// Op list: python/models/swin_transformer/swin_transformer_main.py:11-61 (Part-1..8); the
// reference runs these as separate TVM kernels (:196-330) and has neither the
// relative-position bias nor the shifted-window mask (published Swin definition used).
#include <algorithm>
#include <type_traits>
#include "gemm_tile.hpp"
#include "host_util.hpp"

namespace souffle {
namespace swin {

constexpr int C = 128, NH = 4, HD = 32, WS = 7, N = 49, NP = 64, F = 512, TAB = (2 * WS - 1) * (2 * WS - 1);
constexpr int ZLD = C + 8, BLD = F + 8;
using Tile = GemmTile<64, 64, 64, 2, 2>;

struct BlockW {
  const half_t *ln1_g, *ln1_b, *w_qkv, *b_qkv, *rel_table, *w_proj, *b_proj, *ln2_g, *ln2_b, *w_fc1, *b_fc1, *w_fc2, *b_fc2;
};
struct Args {
  int Hh, Ww, shift, use_mask;
  float eps;
  const half_t *x;
  half_t *mid, *y;
  unsigned *ctl;
  unsigned long long *trace;   // optional phase stamps: trace[block * 32 + phase] (development aid)
  half_t *xctx;                // quad kernel: [window][64][C] attention output, a head's columns written by its workgroup
  float *xpart;                // quad kernel: [window][head][64][C] fp32 FC2 partial sums
  unsigned *xflags;            // quad kernel: [window][16] hand-over words (4 used)
  int strict;                  // souffle_set_strict_fences
  BlockW w[2];
};

// Weights reach the CU as a stream of 24 chunks per block, each W[128 k][64 n] (16 KB): 6 of
// QKV, 2 of proj, 8 of FC1, 8 of FC2 (2 column blocks x 4 K blocks).  The stream does not
// depend on any activation, so it runs two chunks ahead of the MFMAs through a ring of three
// LDS buffers filled by direct global->LDS loads, across the LayerNorm / attention phases and
// across the hand-over to the next block: the GEMM phases never wait for a weight load that was
// issued less than a chunk's worth of work earlier.
constexpr int CHUNK_K = 128, CHUNK_N = 64, CHUNK_BYTES = CHUNK_K * CHUNK_N * 2, RING = 3, CHUNKS = 24;
constexpr int CHUNK_LOADS = CHUNK_BYTES / 1024 / 4;      // wave-wide loads per wave per chunk

// LDS carve-up (bytes)
constexpr int OFF_RING = 0;
constexpr int OFF_ZS = OFF_RING + RING * CHUNK_BYTES;
constexpr int OFF_BIG = OFF_ZS + NP * ZLD * 2;
constexpr int OFF_X1 = OFF_BIG + NP * BLD * 2;
constexpr int OFF_TAB = OFF_X1 + NP * ZLD * 2;
constexpr int OFF_TOK = OFF_TAB + TAB * NH * 4;
constexpr int OFF_REG = OFF_TOK + NP * 4;
// biases and LayerNorm vectors of the block, copied once per call (halves): reading them from
// global memory inside the GEMM phases would make the compiler wait for ALL outstanding vector
// memory operations - the prefetched weight chunks included - at every use
constexpr int P_BQKV = 0, P_BPROJ = P_BQKV + 3 * C, P_BFC1 = P_BPROJ + C, P_BFC2 = P_BFC1 + F, P_G1 = P_BFC2 + C,
              P_B1 = P_G1 + C, P_G2 = P_B1 + C, P_B2 = P_G2 + C, P_HALVES = P_B2 + C;
constexpr int OFF_PAR = OFF_REG + NP * 4;
constexpr int LDS_BYTES = OFF_PAR + P_HALVES * 2;
static_assert(LDS_BYTES <= 160 * 1024, "one workgroup per CU");

struct Chunk {
  const half_t *W;
  int ldw, k0, n0;
};
__device__ __forceinline__ Chunk chunk_of(const BlockW &w, int c) {
  if (c < 6) return Chunk{w.w_qkv, 3 * C, 0, c * CHUNK_N};
  if (c < 8) return Chunk{w.w_proj, C, 0, (c - 6) * CHUNK_N};
  if (c < 16) return Chunk{w.w_fc1, F, 0, (c - 8) * CHUNK_N};
  return Chunk{w.w_fc2, C, ((c - 16) & 3) * CHUNK_K, ((c - 16) >> 2) * CHUNK_N};
}

// The weight stream of one workgroup.  `issued` / `used` count chunks over the whole launch.
// Slot swizzles of the weight chunks in LDS (64 banks of 4 bytes; the transposing read is served half a
// wave per cycle: 32 bytes of each of the rows k0..k0+3 and k0+8..k0+11, which must not share banks).
// 128-byte rows: rows of equal parity start in the same bank, bits 1 and 3 of k separate the four of them.
// 64-byte rows: rows k and k+8 start in the same bank, bit 3 separates them (bit 1 is harmless).
__device__ __forceinline__ int wswz8(int k) { return (k & 2) | ((k & 8) >> 1); }
__device__ __forceinline__ int wswz4(int k) { return (k & 2) ^ ((k & 8) >> 2); }
struct WeightRing {
  unsigned char *lds;
  unsigned lds_addr;
  int issued, used;
};
// Queue chunk c of block weights w into the next ring buffer.  Layout as GemmOneShot's W slice:
// slot(k, c8) = 8 k + (c8 ^ wswz8(k)), for the transposing operand read.
__device__ __forceinline__ void ring_issue(WeightRing &r, const BlockW &w, int c) {
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6;
  const Chunk ch = chunk_of(w, c);
  const unsigned base = r.lds_addr + (r.issued % RING) * CHUNK_BYTES;
#pragma unroll
  for (int q = 0; q < CHUNK_LOADS; ++q) {
    const int inst = q * 4 + wave, sl = inst * 64 + lane, k = sl >> 3, c8 = (sl & 7) ^ wswz8(k);
    load_lds16(ch.W + (size_t)(ch.k0 + k) * ch.ldw + ch.n0 + c8 * 8, base + inst * 1024);
  }
  r.issued++;
}
// Wait for the oldest unused chunk and hand out its buffer.  `more`: chunks issued after it
// (0..2).  After the barrier everybody has finished with the chunk before it, whose buffer the
// caller may refill.  Other vector memory operations issued in between only make the wait stricter.
__device__ __forceinline__ const unsigned char *ring_take(WeightRing &r) {
  const int more = r.issued - r.used - 1;
  if (more >= 2) wait_vmcnt<2 * CHUNK_LOADS>();
  else if (more == 1) wait_vmcnt<CHUNK_LOADS>();
  else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  const unsigned char *buf = r.lds + (r.used % RING) * CHUNK_BYTES;
  r.used++;
  return buf;
}
// acc[j] (rows 16 wave .. +15, columns 16 j .. +15 of the chunk) += A[rows][ka .. ka+128) . chunk.
// All 36 operand reads are issued before the first MFMA: with a read-then-multiply order the
// compiler waits for each pair of reads in turn and the chunk costs 16 LDS latencies.
__device__ __forceinline__ void chunk_mma(const unsigned char *buf, const half_t *A, int lda, int ka, f4 (&acc)[4]) {
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const half_t *ws = reinterpret_cast<const half_t *>(buf);
  h8 xop[CHUNK_K / 32], wop[CHUNK_K / 32][4];
#pragma unroll
  for (int ks = 0; ks < CHUNK_K / 32; ++ks) {
    xop[ks] = *reinterpret_cast<const h8 *>(A + (wave * 16 + l16) * lda + ka + ks * 32 + g * 8);
    const int k = ks * 32 + g * 8 + (l16 >> 2);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c8 = j * 2 + ((l16 & 3) >> 1);
      const half_t *p = ws + (k * 8 + (c8 ^ wswz8(k))) * 8 + (l16 & 1) * 4;
      const h4 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 4 * CHUNK_N);
      wop[ks][j] = h8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  }
#pragma unroll
  for (int ks = 0; ks < CHUNK_K / 32; ++ks)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = mfma_16x16x32(wop[ks][j], xop[ks], acc[j]);
}

__device__ __forceinline__ int region_of(int i, int n, int shift) {   // slices [0,n-7), [n-7,n-shift), [n-shift,n)
  return i < n - WS ? 0 : (i < n - shift ? 1 : 2);
}

// LayerNorm of the 64 rows of a [64][C] fp16 source into dst (LDS, ld ZLD): four lanes share a row
// (32 columns each), so all rows are normalised at once; rows >= N become zero.
// load8(r, c) -> the 8 halves [r][c .. c+7]; gam and bet are in LDS.
template <class Load8>
__device__ __forceinline__ void layernorm_rows(Load8 load8, half_t *dst, const half_t *gam, const half_t *bet, float eps) {
  const int tid = opaque_thread_id(), r = tid >> 2, c0 = (tid & 3) * 32;
  h8 x[4];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[i] = r < N ? as_h8(load8(r, c0 + 8 * i)) : h8{};
#pragma unroll
    for (int e = 0; e < 8; ++e) sum += (float)x[i][e];
  }
  sum += wave_xor(sum, 1);
  sum += wave_xor(sum, 2);
  const float mean = sum * (1.0f / C);
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) { const float d = (float)x[i][e] - mean; sq += d * d; }
  sq += wave_xor(sq, 1);
  sq += wave_xor(sq, 2);
  const float rstd = rsqrtf(sq * (1.0f / C) + eps);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h8 o = {};
    if (r < N) {
      const h8 g8 = *reinterpret_cast<const h8 *>(gam + c0 + 8 * i), b8 = *reinterpret_cast<const h8 *>(bet + c0 + 8 * i);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (half_t)(((float)x[i][e] - mean) * rstd * (float)g8[e] + (float)b8[e]);
    }
    *reinterpret_cast<h8 *>(dst + r * ZLD + c0 + 8 * i) = o;
  }
}

__device__ __forceinline__ f4 add_bias4(f4 v, const half_t *bias_lds, int n) {
  const h4 bb = *reinterpret_cast<const h4 *>(bias_lds + n);
  return v + f4{(float)bb[0], (float)bb[1], (float)bb[2], (float)bb[3]};
}

// One block for one window.  `next`: the weights whose first chunks are queued before this call
// returns (the next call of this workgroup), or NULL.
__device__ void block_for_window(unsigned char *lds, WeightRing &ring, const Args &a, const BlockW &w, const BlockW *next,
                                 int shift, const half_t *xin, half_t *xout, int win) {
  half_t *zs = reinterpret_cast<half_t *>(lds + OFF_ZS);
  half_t *big = reinterpret_cast<half_t *>(lds + OFF_BIG);
  half_t *x1s = reinterpret_cast<half_t *>(lds + OFF_X1);
  float *tab = reinterpret_cast<float *>(lds + OFF_TAB);
  int *tok = reinterpret_cast<int *>(lds + OFF_TOK);
  int *reg = reinterpret_cast<int *>(lds + OFF_REG);
  half_t *par = reinterpret_cast<half_t *>(lds + OFF_PAR);
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const int nww = a.Ww / WS;
  const int first_chunk = ring.used;                        // chunk c of this call is ring chunk first_chunk + c
  // keep the stream two chunks ahead: chunk c+2 of this call, or the first chunks of the next
  auto top_up = [&]() {
    const int c = ring.issued - first_chunk;
    if (c < CHUNKS) ring_issue(ring, w, c);
    else if (next && c < CHUNKS + 2) ring_issue(ring, *next, c - CHUNKS);
  };
  // one output column block of a GEMM whose K is one chunk: acc = A[64][128] . chunk
  auto gemm_chunk = [&](const half_t *A, int lda, f4 (&acc)[4]) {
    const unsigned char *buf = ring_take(ring);
    top_up();
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = f4{0.f, 0.f, 0.f, 0.f};
    chunk_mma(buf, A, lda, 0, acc);
  };
  const int row = wave * 16 + l16;                          // the row this lane holds results of
  int mark_id = shift > 0 ? 16 : 0;
  auto mark = [&]() { if (a.trace && tid == 0 && win == (int)blockIdx.x) a.trace[blockIdx.x * 32 + mark_id] = wall_clock64(); ++mark_id; };
  mark();

  __syncthreads();
  while (ring.issued < first_chunk + 2) top_up();           // (already there when the previous call queued them)
  if (tid < NP) {
    int t = -1, rg = 0;
    if (tid < N) {
      // rolled grid position of slot tid of this window, and the token it comes from:
      // roll(-shift) then view+permute partition (torch closed forms)
      const int i = (win / nww) * WS + tid / WS, j = (win % nww) * WS + tid % WS;
      t = ((i + shift) % a.Hh) * a.Ww + (j + shift) % a.Ww;
      if (shift > 0) rg = 3 * region_of(i, a.Hh, shift) + region_of(j, a.Ww, shift);
    }
    tok[tid] = t;
    reg[tid] = rg;
  }
  for (int i = tid; i < TAB * NH; i += 256) tab[i] = w.rel_table ? (float)w.rel_table[i] : 0.f;
  {
    auto copy = [&](int off, const half_t *src, int n, float dflt) {
      for (int i = tid; i < n; i += 256) par[off + i] = src ? src[i] : (half_t)dflt;
    };
    copy(P_BQKV, w.b_qkv, 3 * C, 0.f); copy(P_BPROJ, w.b_proj, C, 0.f); copy(P_BFC1, w.b_fc1, F, 0.f); copy(P_BFC2, w.b_fc2, C, 0.f);
    copy(P_G1, w.ln1_g, C, 1.f); copy(P_B1, w.ln1_b, C, 0.f); copy(P_G2, w.ln2_g, C, 1.f); copy(P_B2, w.ln2_b, C, 0.f);
  }
  __syncthreads();

  mark();
  // LN1 of the gathered rows
  // (the gathered rows are also kept, in x1s, as the shortcut of the projection)
  layernorm_rows([&](int r, int c) {
    const u4 v = ld16<true>(xin, (tok[r] * C + c) * 2);
    *reinterpret_cast<u4 *>(x1s + r * ZLD + c) = v;
    return v;
  }, zs, par + P_G1, par + P_B1, a.eps);
  __syncthreads();

  mark();
  // QKV = Z.Wqkv + b, q pre-scaled by hd^-0.5; kept in LDS as [64][3C]
  const float qscale = rsqrtf((float)HD);
  for (int nt = 0; nt < 3 * C / CHUNK_N; ++nt) {
    f4 acc[4];
    gemm_chunk(zs, ZLD, acc);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = nt * CHUNK_N + j * 16 + g * 4;
      f4 v = add_bias4(acc[j], par + P_BQKV, n);
      if (n < C) v *= qscale;
      *reinterpret_cast<u2 *>(big + row * BLD + n) = pack_h4(v);
    }
  }
  __syncthreads();

  mark();
  // attention: wave = head
  {
    const int h = wave;
    for (int qt = 0; qt < NP / 16; ++qt) {
      const int q = qt * 16 + l16;
      const h8 qop = *reinterpret_cast<const h8 *>(big + q * BLD + h * HD + g * 8);
      f4 sc[NP / 16];
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < NP / 16; ++t) {
        const h8 kop = *reinterpret_cast<const h8 *>(big + (t * 16 + l16) * BLD + C + h * HD + g * 8);
        f4 s = mfma_16x16x32(kop, qop, f4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int key = t * 16 + g * 4 + v;
          if (key >= N) s[v] = -INFINITY;
          else if (q < N) {
            const int di = q / WS - key / WS + WS - 1, dj = q % WS - key % WS + WS - 1;
            s[v] += tab[(di * (2 * WS - 1) + dj) * NH + h];
            if (a.use_mask && reg[q] != reg[key]) s[v] += -100.0f;
          }
          mx = fmaxf(mx, s[v]);
        }
        sc[t] = s;
      }
      mx = fmaxf(mx, wave_xor(mx, 16));
      mx = fmaxf(mx, wave_xor(mx, 32));
      float sum = 0.f;
#pragma unroll
      for (int t = 0; t < NP / 16; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) { sc[t][v] = __expf(sc[t][v] - mx); sum += sc[t][v]; }
      sum += wave_xor(sum, 16);
      sum += wave_xor(sum, 32);
      const float inv = 1.0f / sum;
      f4 o[HD / 16];
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < NP / 16; ++t) {
        const f4 pr = sc[t] * inv;
        const h4 p = {(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};
#pragma unroll
        for (int dt = 0; dt < HD / 16; ++dt) {
          const h4 vop = lds_read_tr16(big + (t * 16 + g * 4 + (l16 >> 2)) * BLD + 2 * C + h * HD + dt * 16 + (l16 & 3) * 4);
          o[dt] = mfma_16x16x16(vop, p, o[dt]);
        }
      }
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt)
        *reinterpret_cast<u2 *>(zs + q * ZLD + h * HD + dt * 16 + g * 4) = pack_h4(o[dt]);
    }
  }
  __syncthreads();

  mark();
  // x1 = x + ctx.Wproj + b  (kept in LDS)
  for (int nt = 0; nt < C / CHUNK_N; ++nt) {
    f4 acc[4];
    gemm_chunk(zs, ZLD, acc);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = nt * CHUNK_N + j * 16 + g * 4;
      f4 v = f4{0.f, 0.f, 0.f, 0.f};
      if (row < N) {
        const h4 sh = *reinterpret_cast<const h4 *>(x1s + row * ZLD + n);
        v = add_bias4(acc[j], par + P_BPROJ, n) + f4{(float)sh[0], (float)sh[1], (float)sh[2], (float)sh[3]};
      }
      *reinterpret_cast<u2 *>(x1s + row * ZLD + n) = pack_h4(v);
    }
  }
  __syncthreads();

  mark();
  layernorm_rows([&](int r, int c) { return *reinterpret_cast<const u4 *>(x1s + r * ZLD + c); }, zs, par + P_G2, par + P_B2, a.eps);
  __syncthreads();
  mark();

  // H = gelu(Z2.W1 + b1) in LDS
  for (int nt = 0; nt < F / CHUNK_N; ++nt) {
    f4 acc[4];
    gemm_chunk(zs, ZLD, acc);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = nt * CHUNK_N + j * 16 + g * 4;
      f4 v = add_bias4(acc[j], par + P_BFC1, n);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = gelu_tanh(v[i]);
      *reinterpret_cast<u2 *>(big + row * BLD + n) = pack_h4(v);
    }
  }
  __syncthreads();

  mark();
  // out = x1 + H.W2 + b2, scattered back to the token rows; K = 512 is four chunks per column block
  for (int nt = 0; nt < C / CHUNK_N; ++nt) {
    f4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = f4{0.f, 0.f, 0.f, 0.f};
    for (int kc = 0; kc < F / CHUNK_K; ++kc) {
      const unsigned char *buf = ring_take(ring);
      top_up();
      chunk_mma(buf, big, BLD, kc * CHUNK_K, acc);
    }
    if (row < N) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = nt * CHUNK_N + j * 16 + g * 4;
        const h4 r = *reinterpret_cast<const h4 *>(x1s + row * ZLD + n);
        const f4 v = add_bias4(acc[j], par + P_BFC2, n) + f4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
        st8<true>(xout, (tok[row] * C + n) * 2, pack_h4(v));
      }
    }
  }
  mark();
}

__global__ void __launch_bounds__(256) k_block_pair(Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl, a.strict != 0);
  WeightRing ring{lds + OFF_RING, lds_address(lds + OFF_RING), 0, 0};
  const int nwin = (a.Hh / WS) * (a.Ww / WS), step = gridDim.x;
  if ((int)blockIdx.x >= nwin) {
    // Fewer windows than CUs: the spare workgroups pull the weights of both blocks into the L2 of
    // their XCD (workgroup b runs on XCD b % 8), so that the weight stream of the working
    // workgroups hits there instead of paying the memory latency for every chunk.
    const int xcd_slots = (step - nwin + 7) / 8, slot = ((int)blockIdx.x - nwin) / 8;
    float sink = 0.f;
    for (int b = 0; b < 2; ++b) {
      const half_t *mats[4] = {a.w[b].w_qkv, a.w[b].w_proj, a.w[b].w_fc1, a.w[b].w_fc2};
      const int halves[4] = {C * 3 * C, C * C, C * F, F * C};
      for (int m = 0; m < 4; ++m)
        for (int i = (slot * 256 + (int)threadIdx.x) * 8; i < halves[m]; i += xcd_slots * 256 * 8)
          sink += __builtin_bit_cast(f4, *reinterpret_cast<const u4 *>(mats[m] + i))[0];
    }
    asm volatile("" ::"v"(sink));
    grid_sync(bar);
    grid_barrier_end(bar);
    return;
  }
  for (int win = blockIdx.x; win < nwin; win += step)
    block_for_window(lds, ring, a, a.w[0], win + step < nwin ? &a.w[0] : &a.w[1], 0, a.x, a.mid, win);
  grid_sync(bar);                                           // (the first weight chunks of the second block are already on their way)
  for (int win = blockIdx.x; win < nwin; win += step)
    block_for_window(lds, ring, a, a.w[1], win + step < nwin ? &a.w[1] : nullptr, a.shift, a.mid, a.y, win);
  grid_barrier_end(bar);
}


// ------------------------------------------------------------------------------------------------
// Four workgroups per window.  A window's block is bound by how fast ONE CU can take in the 393 KB
// of weights (a direct-to-LDS load occupies the CU's load unit ~57 cycles per KB, and the issuing
// wave with it) while three quarters of the CUs idle (64 windows, 256 CUs).  Here workgroup h of a
// window owns attention head h, the h-th quarter of FC1's columns and the matching quarter of FC2's
// K range, so it takes in 120 KB per block:
//   LN1 (all rows, redundantly) -> Q_h, K_h, V_h -> attention of head h (one query tile per wave)
//   -> [hand-over 1: the four heads' context columns, fp16, through memory]
//   -> projection + shortcut (all columns, redundantly: 32 KB of weights) -> LN2
//   -> H_h = gelu(LN2 . W1[:, quarter h]) -> P_h = H_h . W2[quarter h, :] (fp32 partial sums)
//   -> [hand-over 2: partial sums through memory] -> workgroup h adds the four partials, the bias
//      and the shortcut for output columns [32h, 32h+32) in a fixed order and stores them.
// A hand-over is a write-through store of the data, one flag word per workgroup, and a bounded poll
// of the three other flags.  Flag values grow from launch to launch (a launch count kept next to
// them), so nothing is reset.
// The hand-over words sit right behind the control block, at the same place for every image size, so
// that a workspace used for several sizes keeps one consistent set of them.
constexpr int kMaxSplitWindows = 256;
constexpr int QN = 32, QCHUNK_BYTES = CHUNK_K * QN * 2, QCHUNKS = 15, QLOADS = QCHUNK_BYTES / 1024 / 4;
static_assert(F / NH == CHUNK_K && HD == QN, "a head's FC2 share is one chunk deep, its q/k/v slices one chunk wide");

__device__ __forceinline__ Chunk qchunk_of(const BlockW &w, int c, int h) {
  if (c < 3) return Chunk{w.w_qkv, 3 * C, 0, c * C + h * HD};
  if (c < 7) return Chunk{w.w_proj, C, 0, (c - 3) * QN};
  if (c < 11) return Chunk{w.w_fc1, F, 0, h * (F / NH) + (c - 7) * QN};
  return Chunk{w.w_fc2, C, h * (F / NH), (c - 11) * QN};
}
// W[128 k][32 n] chunk: slot(k, c4) = 4 k + (c4 ^ wswz4(k)) (16-byte slots), for the transposing read.
__device__ __forceinline__ void qring_issue(WeightRing &r, const BlockW &w, int c, int h) {
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6;
  const Chunk ch = qchunk_of(w, c, h);
  const unsigned base = r.lds_addr + (r.issued % RING) * QCHUNK_BYTES;
#pragma unroll
  for (int q = 0; q < QLOADS; ++q) {
    const int inst = q * 4 + wave, sl = inst * 64 + lane, k = sl >> 2, c4 = (sl & 3) ^ wswz4(k);
    load_lds16(ch.W + (size_t)(ch.k0 + k) * ch.ldw + ch.n0 + c4 * 8, base + inst * 1024);
  }
  r.issued++;
}
__device__ __forceinline__ const unsigned char *qring_take(WeightRing &r) {
  const int more = r.issued - r.used - 1;
  if (more >= 2) wait_vmcnt<2 * QLOADS>();
  else if (more == 1) wait_vmcnt<QLOADS>();
  else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  const unsigned char *buf = r.lds + (r.used % RING) * QCHUNK_BYTES;
  r.used++;
  return buf;
}
// acc[j] (rows 16 wave .. +15, columns 16 j .. +15 of the chunk) += A[rows][ka .. ka+128) . chunk
__device__ __forceinline__ void qchunk_mma(const unsigned char *buf, const half_t *A, int lda, int ka, f4 (&acc)[2]) {
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const half_t *ws = reinterpret_cast<const half_t *>(buf);
  h8 xop[CHUNK_K / 32], wop[CHUNK_K / 32][2];
#pragma unroll
  for (int ks = 0; ks < CHUNK_K / 32; ++ks) {
    xop[ks] = *reinterpret_cast<const h8 *>(A + (wave * 16 + l16) * lda + ka + ks * 32 + g * 8);
    const int k = ks * 32 + g * 8 + (l16 >> 2);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c4 = j * 2 + ((l16 & 3) >> 1);
      const half_t *p = ws + (k * 4 + (c4 ^ wswz4(k))) * 8 + (l16 & 1) * 4;
      const h4 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 4 * QN);
      wop[ks][j] = h8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  }
#pragma unroll
  for (int ks = 0; ks < CHUNK_K / 32; ++ks)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[j] = mfma_16x16x32(wop[ks][j], xop[ks], acc[j]);
}
// This workgroup's data of a hand-over are written: publish `val` in its flag word, then wait until
// the window's four words have reached it.  Every thread calls it; the wait is bounded.
__device__ __forceinline__ void quad_handover(unsigned *flags, unsigned *ctl, int win, int h, unsigned val, bool strict) {
  wait_all_memory();                             // the write-through stores are acknowledged
  strict_release(strict);
  __syncthreads();
  if (threadIdx.x == 0) __hip_atomic_store(flags + win * 16 + h, val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (threadIdx.x < 64) {
    for (int spin = 0; spin < kMaxBarrierSpin; ++spin) {
      bool ok = true;
      if (threadIdx.x < NH)
        ok = (int)(__hip_atomic_load(flags + win * 16 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - val) >= 0;
      if (__all(ok)) break;
      __builtin_amdgcn_s_sleep(1);
      if (spin == kMaxBarrierSpin - 1 && threadIdx.x == 0)   // gave up: the launch's output is invalid
        (void)__hip_atomic_fetch_or(ctl + kCtlErrWord, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __syncthreads();
  strict_acquire(strict);
  compiler_fence();                              // no load of the other three workgroups' rows is scheduled above the poll
}

// One block for one window, as workgroup h of its four.  fv: the flag value of this block's first hand-over.
__device__ void block_for_window_quad(unsigned char *lds, WeightRing &ring, const Args &a, const BlockW &w, const BlockW *next,
                                      int shift, const half_t *xin, half_t *xout, int win, int h, unsigned fv) {
  half_t *zs = reinterpret_cast<half_t *>(lds + OFF_ZS);
  half_t *big = reinterpret_cast<half_t *>(lds + OFF_BIG);
  half_t *x1s = reinterpret_cast<half_t *>(lds + OFF_X1);
  float *tab = reinterpret_cast<float *>(lds + OFF_TAB);
  int *tok = reinterpret_cast<int *>(lds + OFF_TOK);
  int *reg = reinterpret_cast<int *>(lds + OFF_REG);
  half_t *par = reinterpret_cast<half_t *>(lds + OFF_PAR);
  const int tid = opaque_thread_id(), lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
  const int nww = a.Ww / WS;
  const int first_chunk = ring.used;
  auto top_up = [&]() {
    const int c = ring.issued - first_chunk;
    if (c < QCHUNKS) qring_issue(ring, w, c, h);
    else if (next && c < QCHUNKS + 2) qring_issue(ring, *next, c - QCHUNKS, h);
  };
  auto gemm_chunk = [&](const half_t *A, int lda, int ka, f4 (&acc)[2]) {
    const unsigned char *buf = qring_take(ring);
    top_up();
    acc[0] = acc[1] = f4{0.f, 0.f, 0.f, 0.f};
    qchunk_mma(buf, A, lda, ka, acc);
  };
  const int row = wave * 16 + l16;
  int mark_id = shift > 0 ? 16 : 0;
  auto mark = [&]() { if (a.trace && tid == 0 && win == (int)blockIdx.x / NH) a.trace[blockIdx.x * 32 + mark_id] = wall_clock64(); ++mark_id; };
  mark();

  __syncthreads();
  while (ring.issued < first_chunk + 2) top_up();
  if (tid < NP) {
    int t = -1, rg = 0;
    if (tid < N) {
      const int i = (win / nww) * WS + tid / WS, j = (win % nww) * WS + tid % WS;
      t = ((i + shift) % a.Hh) * a.Ww + (j + shift) % a.Ww;
      if (shift > 0) rg = 3 * region_of(i, a.Hh, shift) + region_of(j, a.Ww, shift);
    }
    tok[tid] = t;
    reg[tid] = rg;
  }
  for (int i = tid; i < TAB * NH; i += 256) tab[i] = w.rel_table ? (float)w.rel_table[i] : 0.f;
  {
    auto copy = [&](int off, const half_t *src, int n, float dflt) {
      for (int i = tid; i < n; i += 256) par[off + i] = src ? src[i] : (half_t)dflt;
    };
    copy(P_BQKV, w.b_qkv, 3 * C, 0.f); copy(P_BPROJ, w.b_proj, C, 0.f); copy(P_BFC1, w.b_fc1, F, 0.f); copy(P_BFC2, w.b_fc2, C, 0.f);
    copy(P_G1, w.ln1_g, C, 1.f); copy(P_B1, w.ln1_b, C, 0.f); copy(P_G2, w.ln2_g, C, 1.f); copy(P_B2, w.ln2_b, C, 0.f);
  }
  __syncthreads();
  mark();

  // LN1 of the gathered rows (kept in x1s as the shortcut of the projection)
  layernorm_rows([&](int r, int c) {
    const u4 v = ld16<true>(xin, (tok[r] * C + c) * 2);
    *reinterpret_cast<u4 *>(x1s + r * ZLD + c) = v;
    return v;
  }, zs, par + P_G1, par + P_B1, a.eps);
  __syncthreads();
  mark();

  // Q_h (pre-scaled), K_h, V_h in big[:, 0..32), [32..64), [64..96)
  const float qscale = rsqrtf((float)HD);
  for (int c = 0; c < 3; ++c) {
    f4 acc[2];
    gemm_chunk(zs, ZLD, 0, acc);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int nl = j * 16 + g * 4;
      f4 v = add_bias4(acc[j], par + P_BQKV, c * C + h * HD + nl);
      if (c == 0) v *= qscale;
      *reinterpret_cast<u2 *>(big + row * BLD + c * HD + nl) = pack_h4(v);
    }
  }
  __syncthreads();
  mark();

  // attention of head h: wave = query tile
  {
    const int q = wave * 16 + l16;
    const h8 qop = *reinterpret_cast<const h8 *>(big + q * BLD + g * 8);
    f4 sc[NP / 16];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < NP / 16; ++t) {
      const h8 kop = *reinterpret_cast<const h8 *>(big + (t * 16 + l16) * BLD + HD + g * 8);
      f4 s = mfma_16x16x32(kop, qop, f4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int key = t * 16 + g * 4 + v;
        if (key >= N) s[v] = -INFINITY;
        else if (q < N) {
          const int di = q / WS - key / WS + WS - 1, dj = q % WS - key % WS + WS - 1;
          s[v] += tab[(di * (2 * WS - 1) + dj) * NH + h];
          if (a.use_mask && reg[q] != reg[key]) s[v] += -100.0f;
        }
        mx = fmaxf(mx, s[v]);
      }
      sc[t] = s;
    }
    mx = fmaxf(mx, wave_xor(mx, 16));
    mx = fmaxf(mx, wave_xor(mx, 32));
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < NP / 16; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) { sc[t][v] = __expf(sc[t][v] - mx); sum += sc[t][v]; }
    sum += wave_xor(sum, 16);
    sum += wave_xor(sum, 32);
    const float inv = 1.0f / sum;
    f4 o[HD / 16];
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < NP / 16; ++t) {
      const f4 pr = sc[t] * inv;
      const h4 p = {(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt) {
        const h4 vop = lds_read_tr16(big + (t * 16 + g * 4 + (l16 >> 2)) * BLD + 2 * HD + dt * 16 + (l16 & 3) * 4);
        o[dt] = mfma_16x16x16(vop, p, o[dt]);
      }
    }
    // this head's context columns: into zs for this workgroup, through memory for the three others
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      const u2 pk = pack_h4(o[dt]);
      *reinterpret_cast<u2 *>(zs + q * ZLD + h * HD + dt * 16 + g * 4) = pk;
      st8<true>(a.xctx, ((win * NP + q) * C + h * HD + dt * 16 + g * 4) * 2, pk);
    }
  }
  mark();
  quad_handover(a.xflags, a.ctl, win, h, fv, a.strict != 0);
  mark();
  for (int idx = tid; idx < NP * (C / 8); idx += 256) {
    const int r = idx / (C / 8), c8 = idx % (C / 8);
    if (c8 / (HD / 8) != h) *reinterpret_cast<u4 *>(zs + r * ZLD + c8 * 8) = ld16<true>(a.xctx, ((win * NP + r) * C + c8 * 8) * 2);
  }
  __syncthreads();
  mark();

  // x1 = x + ctx.Wproj + b (all columns, in every workgroup of the window)
  for (int nt = 0; nt < C / QN; ++nt) {
    f4 acc[2];
    gemm_chunk(zs, ZLD, 0, acc);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = nt * QN + j * 16 + g * 4;
      f4 v = f4{0.f, 0.f, 0.f, 0.f};
      if (row < N) {
        const h4 sh = *reinterpret_cast<const h4 *>(x1s + row * ZLD + n);
        v = add_bias4(acc[j], par + P_BPROJ, n) + f4{(float)sh[0], (float)sh[1], (float)sh[2], (float)sh[3]};
      }
      *reinterpret_cast<u2 *>(x1s + row * ZLD + n) = pack_h4(v);
    }
  }
  __syncthreads();
  mark();
  layernorm_rows([&](int r, int c) { return *reinterpret_cast<const u4 *>(x1s + r * ZLD + c); }, zs, par + P_G2, par + P_B2, a.eps);
  __syncthreads();
  mark();

  // H_h = gelu(Z2 . W1[:, quarter h] + b1) in big[:, 0..128)
  for (int nt = 0; nt < (F / NH) / QN; ++nt) {
    f4 acc[2];
    gemm_chunk(zs, ZLD, 0, acc);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int nl = nt * QN + j * 16 + g * 4;
      f4 v = add_bias4(acc[j], par + P_BFC1, h * (F / NH) + nl);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = gelu_tanh(v[i]);
      *reinterpret_cast<u2 *>(big + row * BLD + nl) = pack_h4(v);
    }
  }
  __syncthreads();
  mark();

  // P_h = H_h . W2[quarter h, :], fp32, through memory
  for (int nt = 0; nt < C / QN; ++nt) {
    f4 acc[2];
    gemm_chunk(big, BLD, 0, acc);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      st16<true>(a.xpart, (((win * NH + h) * NP + row) * C + nt * QN + j * 16 + g * 4) * 4, __builtin_bit_cast(u4, acc[j]));
  }
  mark();
  quad_handover(a.xflags, a.ctl, win, h, fv + 1, a.strict != 0);
  mark();
  // out[:, 32h .. 32h+32) = x1 + b2 + P_0 + P_1 + P_2 + P_3, scattered back to the token rows
  for (int idx = tid; idx < N * (HD / 4); idx += 256) {
    const int r = idx / (HD / 4), col = h * HD + (idx % (HD / 4)) * 4;
    const h4 sh = *reinterpret_cast<const h4 *>(x1s + r * ZLD + col);
    f4 v = add_bias4(f4{(float)sh[0], (float)sh[1], (float)sh[2], (float)sh[3]}, par + P_BFC2, col);
#pragma unroll
    for (int hh = 0; hh < NH; ++hh) v += __builtin_bit_cast(f4, ld16<true>(a.xpart, (((win * NH + hh) * NP + r) * C + col) * 4));
    st8<true>(xout, (tok[r] * C + col) * 2, pack_h4(v));
  }
  mark();
}

__global__ void __launch_bounds__(256) k_block_pair_quad(Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl, a.strict != 0);
  WeightRing ring{lds + OFF_RING, lds_address(lds + OFF_RING), 0, 0};
  const int nwin = (a.Hh / WS) * (a.Ww / WS), quads = gridDim.x / NH;
  // The hand-over words grow from launch to launch: a launch uses four values above those of the one
  // before.  The launch count lives next to the words (behind the last of them), so that clearing the workspace or
  // only its control block cannot set one back without the other.  Everybody reads it here, before the
  // grid barrier below; workgroup 0 advances it after that barrier.
  const unsigned seq = __hip_atomic_load(a.xflags + kMaxSplitWindows * 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned fv = seq * 4u + 1u;
  const int quad = blockIdx.x / NH, h = blockIdx.x % NH;
  for (int win = quad; win < nwin; win += quads)
    block_for_window_quad(lds, ring, a, a.w[0], win + quads < nwin ? &a.w[0] : &a.w[1], 0, a.x, a.mid, win, h, fv);
  grid_sync(bar);
  for (int win = quad; win < nwin; win += quads)
    block_for_window_quad(lds, ring, a, a.w[1], win + quads < nwin ? &a.w[1] : nullptr, a.shift, a.mid, a.y, win, h, fv + 2);
  if (blockIdx.x == 0 && threadIdx.x == 0)
    __hip_atomic_store(a.xflags + kMaxSplitWindows * 16, seq + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  grid_barrier_end(bar);
}

// ---- fused two-GEMM FFN: Y1 = X.W1 ; Y2 = Y1.W2 (split-K partials + reduce) ----
struct FfnArgs {
  int M, K, F, splitk;
  const half_t *x, *w1, *w2;
  half_t *y1, *y2;
  float *part;
  unsigned *ctl;
  int strict;
};

__global__ void __launch_bounds__(256) k_ffn(FfnArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  half_t *gl = reinterpret_cast<half_t *>(lds);
  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl, a.strict != 0);
  {
    const int tn = a.F / 64, items = (a.M / 64) * tn;
    for (int it = blockIdx.x; it < items; it += gridDim.x)
      Tile::run(gl, a.w1, a.F, (it / tn) * 64, (it % tn) * 64, 0, a.K / 64,
                [&](int m, int k) { return *reinterpret_cast<const u4 *>(a.x + (size_t)m * a.K + k); },
                [&](int m, int n, f4 v) { st8<true>(a.y1, (m * a.F + n) * 2, pack_h4(v)); });
  }
  grid_sync(bar);
  {
    const int tn = a.K / 64, items = (a.M / 64) * tn * a.splitk, kper = a.F / a.splitk;
    for (int it = blockIdx.x; it < items; it += gridDim.x) {
      const int ks = it % a.splitk, t = it / a.splitk;
      Tile::run(gl, a.w2, a.K, (t / tn) * 64, (t % tn) * 64, ks * kper, kper / 64,
                [&](int m, int k) { return ld16<true>(a.y1, (m * a.F + k) * 2); },
                [&](int m, int n, f4 v) { st16<true>(a.part, ((ks * a.M + m) * a.K + n) * 4, __builtin_bit_cast(u4, v)); });
    }
  }
  grid_sync(bar);
  for (int i = (blockIdx.x * 256 + threadIdx.x) * 4; i < a.M * a.K; i += gridDim.x * 256 * 4) {
    f4 s = __builtin_bit_cast(f4, ld16<true>(a.part, i * 4));
    for (int ks = 1; ks < a.splitk; ++ks) s += __builtin_bit_cast(f4, ld16<true>(a.part, (ks * a.M * a.K + i) * 4));
    *reinterpret_cast<u2 *>(a.y2 + i) = pack_h4(s);
  }
  grid_barrier_end(bar);
}

static int validate(const souffle_swin_cfg *c) {
  if (!c) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  if (c->channels != C || c->heads != NH || c->window != WS || c->mlp_ratio != 4)
    return fail(SOUFFLE_ERR_SHAPE, "only channels=128 heads=4 window=7 mlp_ratio=4 is built");
  if (c->height <= 0 || c->width <= 0 || c->height % WS || c->width % WS)
    return fail(SOUFFLE_ERR_SHAPE, "height and width must be positive multiples of 7 (got %d x %d)", c->height, c->width);
  if ((long long)c->height * c->width > 1 << 20) return fail(SOUFFLE_ERR_SHAPE, "too many tokens");
  if (c->shift < 0 || c->shift >= WS) return fail(SOUFFLE_ERR_SHAPE, "shift must be in 0..6 (got %d)", c->shift);
  if (!(c->ln_eps >= 0.f)) return fail(SOUFFLE_ERR_SHAPE, "ln_eps must be >= 0");
  return SOUFFLE_OK;
}
struct PairWs { size_t mid, xctx, xpart, xflags, total; };
static PairWs pair_ws(const souffle_swin_cfg *c) {
  const size_t nwin = (size_t)(c->height / WS) * (c->width / WS);
  PairWs p;
  p.xflags = round_up(kCtlWords * 4, 256);
  p.mid = p.xflags + round_up((kMaxSplitWindows * 16 + 1) * 4, 256);      // hand-over words + the launch count
  p.xctx = p.mid + round_up((size_t)c->height * c->width * C * 2, 256);
  p.xpart = p.xctx + round_up(nwin * NP * C * 2, 256);
  p.total = p.xpart + round_up(nwin * NH * NP * C * 4, 256);
  return p;
}
static size_t pair_ws_bytes(const souffle_swin_cfg *c) { return pair_ws(c).total; }

}  // namespace swin
}  // namespace souffle

using namespace souffle;

extern "C" size_t souffle_swin_workspace_bytes(const souffle_swin_cfg *cfg) {
  if (swin::validate(cfg)) return 0;
  return swin::pair_ws_bytes(cfg);
}

extern "C" int souffle_swin_block_pair_fused(const souffle_swin_cfg *cfg, const souffle_swin_block_w w[2], const void *x,
                                             void *y, void *ws, size_t ws_bytes, souffle_stream_t stream) {
  if (int rc = swin::validate(cfg)) return rc;
  if (!w || !x || !y) return fail(SOUFFLE_ERR_NULL, "w, x and y must not be NULL");
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL (need %zu bytes)", swin::pair_ws_bytes(cfg));
  if (ws_bytes < swin::pair_ws_bytes(cfg)) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, swin::pair_ws_bytes(cfg));
  if (!aligned16(x) || !aligned16(y) || !aligned16(ws)) return fail(SOUFFLE_ERR_ALIGN, "x, y and workspace must be 16-byte aligned");
  swin::Args a;
  a.Hh = cfg->height; a.Ww = cfg->width; a.shift = cfg->shift; a.use_mask = cfg->use_shift_mask && cfg->shift > 0; a.eps = cfg->ln_eps;
  a.x = static_cast<const half_t *>(x); a.y = static_cast<half_t *>(y);
  a.ctl = static_cast<unsigned *>(ws);
  a.strict = strict_fences_mode();
  const swin::PairWs pw = swin::pair_ws(cfg);
  a.mid = reinterpret_cast<half_t *>(static_cast<char *>(ws) + pw.mid);
  a.xctx = reinterpret_cast<half_t *>(static_cast<char *>(ws) + pw.xctx);
  a.xpart = reinterpret_cast<float *>(static_cast<char *>(ws) + pw.xpart);
  a.xflags = reinterpret_cast<unsigned *>(static_cast<char *>(ws) + pw.xflags);
  {
    int cap = 0;
    stage_trace(&a.trace, &cap, 256);
    if (cap < 1) a.trace = nullptr;
  }
  for (int b = 0; b < 2; ++b) {
    const souffle_swin_block_w &s = w[b];
    if (!s.w_qkv || !s.w_proj || !s.w_fc1 || !s.w_fc2) return fail(SOUFFLE_ERR_NULL, "block %d: a weight matrix is NULL", b);
    const void *ptrs[13] = {s.ln1_g, s.ln1_b, s.w_qkv, s.b_qkv, s.rel_table, s.w_proj, s.b_proj, s.ln2_g, s.ln2_b, s.w_fc1, s.b_fc1, s.w_fc2, s.b_fc2};
    for (const void *q : ptrs)
      if (!aligned16(q)) return fail(SOUFFLE_ERR_ALIGN, "block %d: a weight/bias pointer is not 16-byte aligned", b);
    const half_t **d = reinterpret_cast<const half_t **>(&a.w[b]);
    for (int i = 0; i < 13; ++i) d[i] = static_cast<const half_t *>(ptrs[i]);
  }
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)swin::k_block_pair, hipFuncAttributeMaxDynamicSharedMemorySize, swin::LDS_BYTES));
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)swin::k_block_pair_quad, hipFuncAttributeMaxDynamicSharedMemorySize, swin::LDS_BYTES));
    attr_done = true;
  }
  const int nwin = (cfg->height / swin::WS) * (cfg->width / swin::WS);
  void *args[] = {&a};
  // four workgroups per window (unless switched off) while that gives a window at most two turns per quad
  if (swin_split_mode() && df.num_cus >= 4 && nwin <= swin::kMaxSplitWindows && (long long)nwin * swin::NH <= 2ll * df.num_cus)
    return launch_persistent((const void *)swin::k_block_pair_quad, (df.num_cus / 4) * 4 < nwin * swin::NH ? (df.num_cus / 4) * 4 : nwin * swin::NH,
                             256, args, swin::LDS_BYTES, static_cast<hipStream_t>(stream));
  return launch_persistent((const void *)swin::k_block_pair, df.num_cus, 256, args, swin::LDS_BYTES,
                           static_cast<hipStream_t>(stream));
}

// Closed forms of torch.roll(-shift) + view/permute window partition, its inverse, the
// relative-position index and the shifted-window region labels.
extern "C" int souffle_swin_index_maps(int height, int width, int window, int shift, int32_t *gather_idx,
                                       int32_t *scatter_idx, int32_t *relpos_idx, int32_t *region_id) {
  if (height <= 0 || width <= 0 || window <= 0 || height % window || width % window)
    return fail(SOUFFLE_ERR_SHAPE, "height and width must be positive multiples of window");
  if (shift < 0 || shift >= window) return fail(SOUFFLE_ERR_SHAPE, "shift must be in 0..window-1");
  const int nww = width / window, n = window * window;
  auto region = [&](int i, int extent) { return i < extent - window ? 0 : (i < extent - shift ? 1 : 2); };
  for (int w = 0; w < (height / window) * nww; ++w)
    for (int s = 0; s < n; ++s) {
      const int i = (w / nww) * window + s / window, j = (w % nww) * window + s % window;
      const int t = ((i + shift) % height) * width + (j + shift) % width;
      if (gather_idx) gather_idx[w * n + s] = t;
      if (scatter_idx) scatter_idx[t] = w * n + s;
      if (region_id) region_id[w * n + s] = shift > 0 ? 3 * region(i, height) + region(j, width) : 0;
    }
  if (relpos_idx)
    for (int p = 0; p < n; ++p)
      for (int q = 0; q < n; ++q)
        relpos_idx[p * n + q] = (p / window - q / window + window - 1) * (2 * window - 1) + (p % window - q % window + window - 1);
  return SOUFFLE_OK;
}

extern "C" int souffle_swin_ffn_fused(const void *x, const void *w1, const void *w2, void *y1, void *y2, int M, int K, int F,
                                      void *ws, size_t ws_bytes, souffle_stream_t stream) {
  if (!x || !w1 || !w2 || !y1 || !y2) return fail(SOUFFLE_ERR_NULL, "x, w1, w2, y1 and y2 must not be NULL");
  if (M <= 0 || K <= 0 || F <= 0 || M % 64 || K % 64 || F % 64 || (long long)M * F > (1 << 28))
    return fail(SOUFFLE_ERR_SHAPE, "M, K and F must be positive multiples of 64 (got %d,%d,%d)", M, K, F);
  if (!aligned16(x) || !aligned16(w1) || !aligned16(w2) || !aligned16(y1) || !aligned16(y2) || !aligned16(ws))
    return fail(SOUFFLE_ERR_ALIGN, "all pointers must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  int splitk = 1;
  while (splitk < 8 && (M / 64) * (K / 64) * splitk * 2 <= df.num_cus && (F / (splitk * 2)) % 64 == 0) splitk *= 2;
  const size_t need = round_up(kCtlWords * 4, 256) + (size_t)splitk * M * K * 4;
  if (!ws || ws_bytes < need) return fail(SOUFFLE_ERR_WORKSPACE, "workspace missing or too small: need %zu bytes", need);
  swin::FfnArgs a{M, K, F, splitk, (const half_t *)x, (const half_t *)w1, (const half_t *)w2, (half_t *)y1, (half_t *)y2,
                  reinterpret_cast<float *>(static_cast<char *>(ws) + round_up(kCtlWords * 4, 256)), static_cast<unsigned *>(ws), strict_fences_mode()};
  static bool attr_done = false;
  if (!attr_done) {
    SOUFFLE_HIP_TRY(hipFuncSetAttribute((const void *)swin::k_ffn, hipFuncAttributeMaxDynamicSharedMemorySize, swin::Tile::LDS_BYTES));
    attr_done = true;
  }
  void *args[] = {&a};
  return launch_persistent((const void *)swin::k_ffn, df.num_cus, 256, args, swin::Tile::LDS_BYTES, static_cast<hipStream_t>(stream));
}
