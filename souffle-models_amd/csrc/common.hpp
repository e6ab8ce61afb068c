// Shared device-side building blocks for gfx950 (CDNA4, wave64): vector types, MFMA
// wrappers, agent-coherent loads/stores, wave reductions and the grid barrier used by
// the persistent cooperative kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace souffle {

typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned u2 __attribute__((ext_vector_type(2)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// ---------------------------------------------------------------- MFMA ----
// v_mfma_f32_16x16x32_f16: D[i][j] += sum_k A[i][k] B[k][j]
//   A: lane l holds row i = l%16, k = 8*(l/16) .. +7
//   B: lane l holds col j = l%16, k = 8*(l/16) .. +7
//   D: lane l holds col j = l%16, rows i = 4*(l/16) + v, v = 0..3
__device__ __forceinline__ f4 mfma_16x16x32(h8 a, h8 b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
// v_mfma_f32_16x16x16_f16: same layouts with k = 4*(l/16) .. +3
__device__ __forceinline__ f4 mfma_16x16x16(h4 a, h4 b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
}

// ds_read_b64_tr_b16: within each group of 16 lanes the 16 x 4 halves addressed by the
// lanes form 4 rows of 16 (lanes 4r..4r+3 supply row r, 4 consecutive halves each);
// lane i of the group receives column i: (row0[i], row1[i], row2[i], row3[i]).
// With a row-major [k][n] tile in LDS this yields the k-vector of column n.
__device__ __forceinline__ h4 lds_read_tr16(const half_t *p) {
  typedef short s4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) s4 lds_s4;
  const s4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4 *)(__attribute__((address_space(3))) void *)const_cast<half_t *>(p));
  return __builtin_bit_cast(h4, r);
}

// ------------------------------------------- agent-coherent global access ----
// Data handed from one workgroup to another inside a persistent kernel is written
// through (sc1) and read with sc1 so that it is coherent across the eight XCD L2s
// without L2 write-back / invalidate fences.  Buffer instructions carry the cache
// bits; the base pointer must be wave-uniform, the offset is in bytes (< 2 GiB).
typedef __attribute__((address_space(8))) void *buf_rsrc_t;
__device__ __forceinline__ auto make_rsrc(const void *base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0x7fffffff, 0x00027000);
}
constexpr int kAuxSc1 = 16;

template <bool COH>
__device__ __forceinline__ u4 ld16(const void *base, int byte_off) {
  if constexpr (COH) return __builtin_amdgcn_raw_buffer_load_b128(make_rsrc(base), byte_off, 0, kAuxSc1);
  else return *reinterpret_cast<const u4 *>(reinterpret_cast<const char *>(base) + byte_off);
}
template <bool COH>
__device__ __forceinline__ u2 ld8(const void *base, int byte_off) {
  if constexpr (COH) return __builtin_amdgcn_raw_buffer_load_b64(make_rsrc(base), byte_off, 0, kAuxSc1);
  else return *reinterpret_cast<const u2 *>(reinterpret_cast<const char *>(base) + byte_off);
}
// 8-byte relaxed agent-scope atomics: a (value, tag) pair that is published and polled
// as one unit.  Being atomic operations, polling loads are re-issued on every spin.
__device__ __forceinline__ u2 ld8_atomic(const void *p) {
  const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p), __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
  return u2{(unsigned)v, (unsigned)(v >> 32)};
}
__device__ __forceinline__ void st8_atomic(void *p, u2 v) {
  __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), (unsigned long long)v[0] | ((unsigned long long)v[1] << 32),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool COH>
__device__ __forceinline__ unsigned ld4(const void *base, int byte_off) {
  if constexpr (COH) return __builtin_amdgcn_raw_buffer_load_b32(make_rsrc(base), byte_off, 0, kAuxSc1);
  else return *reinterpret_cast<const unsigned *>(reinterpret_cast<const char *>(base) + byte_off);
}
template <bool COH>
__device__ __forceinline__ void st16(void *base, int byte_off, u4 v) {
  if constexpr (COH) __builtin_amdgcn_raw_buffer_store_b128(v, make_rsrc(base), byte_off, 0, kAuxSc1);
  else *reinterpret_cast<u4 *>(reinterpret_cast<char *>(base) + byte_off) = v;
}
template <bool COH>
__device__ __forceinline__ void st8(void *base, int byte_off, u2 v) {
  if constexpr (COH) __builtin_amdgcn_raw_buffer_store_b64(v, make_rsrc(base), byte_off, 0, kAuxSc1);
  else *reinterpret_cast<u2 *>(reinterpret_cast<char *>(base) + byte_off) = v;
}
template <bool COH>
__device__ __forceinline__ void st4(void *base, int byte_off, unsigned v) {
  if constexpr (COH) __builtin_amdgcn_raw_buffer_store_b32(v, make_rsrc(base), byte_off, 0, kAuxSc1);
  else *reinterpret_cast<unsigned *>(reinterpret_cast<char *>(base) + byte_off) = v;
}

__device__ __forceinline__ h8 as_h8(u4 v) { return __builtin_bit_cast(h8, v); }
__device__ __forceinline__ u4 as_u4(h8 v) { return __builtin_bit_cast(u4, v); }
__device__ __forceinline__ h4 as_h4(u2 v) { return __builtin_bit_cast(h4, v); }
__device__ __forceinline__ u2 as_u2(h4 v) { return __builtin_bit_cast(u2, v); }
__device__ __forceinline__ u2 pack_h4(f4 v) {
  h4 r = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
  return as_u2(r);
}

// ------------------------------------------------------ wave reductions ----
__device__ __forceinline__ float wave_xor(float v, int mask) { return __shfl_xor(v, mask, kWave); }
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += wave_xor(v, m);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, wave_xor(v, m));
  return v;
}

// ---------------------------------------------------------- activations ----
// 0.5 x (1 + tanh(0.79788456 (x + 0.044715 x^3)))  (cpp/bert/bert_base_impl.cu:722-734)
__device__ __forceinline__ float gelu_tanh(float x) {
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  // tanh(u) = 1 - 2 / (exp(2u) + 1); exp overflow gives the correct limit 1.
  const float t = 1.0f - 2.0f / (__expf(2.0f * u) + 1.0f);
  return 0.5f * x * (1.0f + t);
}

// -------------------------------------------------------- grid barrier ----
// Two-level arrival tree on relaxed agent-scope atomics plus a monotonic generation
// word.  Control block (uint32 words, zeroed once before first use):
//   [0]            root arrival count
//   [32]           generation (monotonic; its start value is irrelevant)
//   [64 + 32*g]    arrival count of group g, g < 64
// Arrival counts run up on even barriers of a launch and down on odd ones, so no
// count is ever reset (nothing to order against the release of the generation word).
// grid_barrier_end() leaves every count at zero for the next launch.
// All data exchanged across a barrier must be written with st*<true> and read with
// ld*<true>; the barrier itself carries no cache write-back or invalidate.
constexpr int kBarGroup = 16;
constexpr int kCtlWords = 64 + 32 * 64;

struct GridBarrier {
  unsigned *ctl;
  unsigned gen;    // meaningful in thread 0 only
  unsigned nblk;
  int down;        // 0: counts run up on the next barrier, 1: down
  // optional stage trace: thread 0 stamps the 100 MHz wall clock on entry to and exit from
  // every barrier: trace[(2*i + {0,1}) * nblk + block] for the i-th barrier of the launch
  unsigned long long *trace;
  int trace_idx, trace_cap;
};

__device__ __forceinline__ void grid_barrier_begin(GridBarrier &b, unsigned *ctl) {
  b.ctl = ctl;
  b.nblk = gridDim.x;
  b.down = 0;
  b.trace = nullptr;
  b.trace_idx = 0;
  b.trace_cap = 0;
  // Read before this workgroup's first arrival: the generation cannot advance until
  // every workgroup has arrived, so all workgroups read the same value.
  b.gen = __hip_atomic_load(ctl + 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Thread 0 only.  Returns true when this arrival completed the whole grid.
__device__ __forceinline__ bool grid_arrive(GridBarrier &b) {
  const unsigned grp = blockIdx.x / kBarGroup;
  const unsigned ngrp = (b.nblk + kBarGroup - 1) / kBarGroup;
  const unsigned gsz = min((unsigned)kBarGroup, b.nblk - grp * kBarGroup);
  unsigned *gc = b.ctl + 64 + 32 * grp;
  const unsigned inc = b.down ? 0xffffffffu : 1u;
  const unsigned prev = __hip_atomic_fetch_add(gc, inc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (prev != (b.down ? 1u : gsz - 1)) return false;
  const unsigned prev2 = __hip_atomic_fetch_add(b.ctl, inc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return prev2 == (b.down ? 1u : ngrp - 1);
}

__device__ __forceinline__ void grid_sync(GridBarrier &b) {
  const bool tr = b.trace && b.trace_idx < b.trace_cap && threadIdx.x == 0;
  if (tr) b.trace[(size_t)(2 * b.trace_idx) * b.nblk + blockIdx.x] = wall_clock64();
  __builtin_amdgcn_s_waitcnt(0);   // this wave's write-through stores are acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    b.gen++;
    if (grid_arrive(b)) {
      __hip_atomic_store(b.ctl + 32, b.gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      while ((int)(__hip_atomic_load(b.ctl + 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - b.gen) < 0)
        __builtin_amdgcn_s_sleep(1);
    }
  }
  b.down ^= 1;
  if (tr) b.trace[(size_t)(2 * b.trace_idx + 1) * b.nblk + blockIdx.x] = wall_clock64();
  b.trace_idx++;
  __syncthreads();
}

// Call once by every workgroup before the kernel returns.
__device__ __forceinline__ void grid_barrier_end(GridBarrier &b) {
  if (b.down) {            // odd number of barriers so far: run the counts back to zero
    __syncthreads();
    if (threadIdx.x == 0) (void)grid_arrive(b);
  }
}

}  // namespace souffle
