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

// The thread id as a value the optimiser cannot see through.  Inside a persistent kernel that
// loops over layers and stages, every address computed from the plain thread id is loop-invariant
// and gets hoisted to the top of the kernel, where dozens of such values stay live across the
// register-hungry GEMM loops and are spilled there.  Stages take their thread id from here.
__device__ __forceinline__ int opaque_thread_id() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// ---------------------------------------------------------------- MFMA ----
// v_mfma_f32_16x16x32_f16: D[i][j] += sum_k A[i][k] B[k][j]
//   A: lane l holds row i = l%16, k = 8*(l/16) .. +7
//   B: lane l holds col j = l%16, k = 8*(l/16) .. +7
//   D: lane l holds col j = l%16, rows i = 4*(l/16) + v, v = 0..3
__device__ __forceinline__ f4 mfma_16x16x32(h8 a, h8 b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
// The same instruction with the accumulator tied to AGPRs and updated in place.  With many live
// accumulators the register allocator otherwise gives the three-address form different
// source and destination registers and copies dozens of accumulators per loop iteration.
// The compiler does not see inside, so the wait states that its hazard recognizer would insert
// between a VALU write of an accumulator and the first MFMA, and between the last MFMA and a
// VALU read, are supplied by hand: mfma_pin() after the accumulators are initialised and again
// before they are read.  All of these are volatile, so they keep their program order.
__device__ __forceinline__ void mfma_16x16x32_inplace(f4 &c, h8 a, h8 b) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
// `n` accumulators exist in AGPRs here (not rematerialised later, not read earlier), with
// 32 wait states in between.
template <int N>
__device__ __forceinline__ void mfma_pin(f4 (&acc)[N], bool before) {
  if (!before) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+a"(acc[i]));
  if (before) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
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

// LDS accesses through an explicit address-space cast: they stay DS instructions also where the
// compiler cannot infer that a generic pointer points into LDS (inside functions that are not
// inlined), instead of becoming flat accesses that count on both memory counters.
__device__ __forceinline__ u4 lds_load16(const unsigned char *p) {
  return *reinterpret_cast<const __attribute__((address_space(3))) u4 *>((const __attribute__((address_space(3))) unsigned char *)p);
}
__device__ __forceinline__ void lds_store8(unsigned char *p, u2 v) {
  *reinterpret_cast<__attribute__((address_space(3))) u2 *>((__attribute__((address_space(3))) unsigned char *)p) = v;
}

// One wave-wide direct global->LDS load: lane L's 16 bytes at `src` land at LDS byte address
// lds_addr + 16 L.  Issued through inline assembly on purpose: for the builtin the compiler
// tracks the LDS write and makes every later LDS read wait for ALL outstanding loads (vmcnt 0),
// which serialises any scheme that keeps loads in flight across LDS reads; with this form the
// waits are the explicit wait_vmcnt<N>() of the caller.
__device__ __forceinline__ void load_lds16(const void *src, unsigned lds_addr) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(src) : "memory", "m0");
#pragma clang diagnostic pop
}
__device__ __forceinline__ unsigned lds_address(const unsigned char *p) {
  return (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char *)p;
}

// ------------------------------------------- agent-coherent global access ----
// Data handed from one workgroup to another inside a persistent kernel is written
// through (sc1) and read with sc1 so that it is coherent across the eight XCD L2s
// without L2 write-back / invalidate fences.  Buffer instructions carry the cache
// bits; the base pointer must be wave-uniform, the offset is in bytes (< 2 GiB).
// A pointer that is the same in every lane, told to the compiler: computed with vector instructions
// (a 64-bit multiply of a layer number by a stride is), a pointer sits in vector registers, and a
// buffer access whose descriptor comes from there is wrapped in a loop over the distinct values
// (four readfirstlanes, two compares, an exec-mask dance and a branch around every store).
template <class T>
__device__ __forceinline__ T *uniform_ptr(T *p) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return reinterpret_cast<T *>(((unsigned long long)hi << 32) | lo);
}
typedef __attribute__((address_space(8))) void *buf_rsrc_t;
__device__ __forceinline__ auto make_rsrc(const void *base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(uniform_ptr(base)), 0, 0x7fffffff, 0x00027000);
}
constexpr int kAuxSc1 = 16;

// A load the compiler knows to come from global memory.  Where it cannot infer the address space of
// a pointer it emits a flat load, which may alias LDS: such a load is not moved across the LDS
// accesses around it and each is waited for before the next LDS store (an epilogue that reads a
// bias or a residual per result group then pays one memory latency per group).
template <class T>
__device__ __forceinline__ T ldg(const void *p) {
  return *(const __attribute__((address_space(1))) T *)p;
}
template <bool COH>
__device__ __forceinline__ u4 ld16(const void *base, int byte_off) {
  if constexpr (COH) return __builtin_amdgcn_raw_buffer_load_b128(make_rsrc(base), byte_off, 0, kAuxSc1);
  else return ldg<u4>(reinterpret_cast<const char *>(base) + byte_off);
}
template <bool COH>
__device__ __forceinline__ u2 ld8(const void *base, int byte_off) {
  if constexpr (COH) return __builtin_amdgcn_raw_buffer_load_b64(make_rsrc(base), byte_off, 0, kAuxSc1);
  else return ldg<u2>(reinterpret_cast<const char *>(base) + byte_off);
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
  else return ldg<unsigned>(reinterpret_cast<const char *>(base) + byte_off);
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
  // 0.5 (1 + tanh(u)) = 1 - 1 / (exp(2u) + 1) with u = 0.79788456 (x + 0.044715 x^3), and
  // exp(2u) = exp2(x (K1 + K2 x^2)): five full-rate operations and two quarter-rate ones (the bare
  // v_exp_f32 and v_rcp_f32, 1 ulp each; the library exp and an IEEE division cost some 20 more
  // instructions, which at 192 results per lane made the FC1 epilogue at 4096 rows 12.8 us long).
  // exp2 overflow gives the limit x, underflow the limit 0.
  constexpr float K1 = 2.0f * 0.7978845608028654f * 1.4426950408889634f, K2 = K1 * 0.044715f;
  const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(x * x, K2, K1));
  return x - x * __builtin_amdgcn_rcpf(e + 1.0f);
}

// 0.5 x (1 + erf(x / sqrt 2)): the exact form (library erff; some 30 instructions per value).
__device__ __forceinline__ float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f)); }

// -------------------------------------------------------- grid barrier ----
// Two kinds of words, never mixed on one cache line:
//  * arrival counter x (x = workgroup % 8, the XCD the workgroup runs on): incremented with an
//    atomic whose result IS awaited, and read by nobody else.  The line therefore stays with
//    the L2 of that XCD and the increments of its workgroups do not compete with pollers for it
//    (with polled counters every poll from another XCD pulls the line away between two
//    increments, and a barrier after a balanced stage takes 4 us instead of 1.5);
//  * done flag x: the workgroup whose increment completes the count of XCD x stores the barrier
//    number there once (write-through), and every workgroup polls the eight flags with one
//    8-lane load until all have reached that number.
// Counters and barrier numbers only grow (across launches too) and are compared as signed
// differences, so a fast workgroup arriving at the next barrier never disturbs a slow one.
// Control block (uint32 words, zeroed once before first use); x = workgroup index % 8, the XCD it runs on:
//   [kCtlArrive + 32 x]  arrival counter x        [kCtlDone + 32 x]  done flag x (number of the last barrier completed)
//   [kCtlCarry + 32 x]   the value counter x holds between launches, [kCtlEpoch] the barrier number between launches:
//                        rewritten by grid_barrier_end() (all workgroups read them before their first arrival,
//                        nobody writes them before the last barrier of the launch has completed)
//   [kCtlErrWord]        sticky error flag for kernels with bounded spin loops (bit 0: LSTM wait,
//                        bit 1: grid barrier or hand-over of the encoder)
// Every word has a place of its own (the assertions below): a done flag that shared its word with a carried counter
// value would read as "completed" to every waiter, since counter values are far larger than barrier numbers.
// Data exchanged across a barrier must be written with st*<true> (write-through); the barrier
// itself carries no cache write-back or invalidate.
constexpr int kCtlArrive = 0, kCtlDone = 256, kCtlCarry = 16, kCtlEpoch = 24;
constexpr int kCtlWords = 512;
constexpr int kCtlErrWord = 400;
constexpr bool ctl_words_distinct() {
  for (int x = 0; x < 8; ++x) {
    const int w[3] = {kCtlArrive + 32 * x, kCtlDone + 32 * x, kCtlCarry + 32 * x};
    for (int y = 0; y < 8; ++y) {
      const int v[3] = {kCtlArrive + 32 * y, kCtlDone + 32 * y, kCtlCarry + 32 * y};
      for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j)
          if ((x != y || i != j) && w[i] == v[j]) return false;
    }
    for (int i = 0; i < 3; ++i)
      if (w[i] == kCtlEpoch || w[i] == kCtlErrWord || w[i] < 0 || w[i] >= 512) return false;
  }
  return kCtlEpoch != kCtlErrWord;
}
static_assert(ctl_words_distinct(), "two words of the control block share a place");
constexpr int kMaxBarrierSpin = 1 << 20;       // about a second of polling; a barrier normally completes in microseconds

// The hand-overs of this library rest on write-through (sc1) stores that are acknowledged before a flag is stored, and
// on sc1 loads behind the poll (served by the L2, never by a stale L1 line).  The memory model's own form is an
// agent-scope release fence in front of the flag store and an agent-scope acquire fence behind the poll (an L2
// write-back and an L1/L2 invalidation per hand-over: measured at 14 us each, against 2).  `strict` switches them on
// in every hand-over (souffle_set_strict_fences): for a driver or part whose caches might behave differently, and
// for the test that requires both forms to give the same bits.
__device__ __forceinline__ void strict_release(bool strict) {
  if (strict) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
}
__device__ __forceinline__ void strict_acquire(bool strict) {
  if (strict) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

struct GridBarrier {
  unsigned *ctl;
  bool strict;       // release / acquire fences of the memory model around every hand-over (see strict_release)
  unsigned target;   // value this workgroup's arrival counter holds once its XCD is complete
  unsigned gsz;      // workgroups that share this workgroup's counter
  unsigned epoch;    // number of the last barrier passed
  unsigned nblk;
  int count;         // barriers passed in this launch
  bool failed;       // a wait of this launch gave up: later barriers are not waited for either
  // optional stage trace: thread 0 stamps the 100 MHz wall clock on entry to and exit from
  // every barrier: trace[(2*i + {0,1}) * nblk + block] for the i-th barrier of the launch,
  // plus up to 8 free-form marks inside the stage that precedes barrier i:
  // trace[(2*cap + 8*i + id) * nblk + block]
  unsigned long long *trace;
  int trace_idx, trace_cap;
};

__device__ __forceinline__ void trace_mark(const GridBarrier &b, int id) {
  if (b.trace && b.trace_idx < b.trace_cap && threadIdx.x == 0)
    b.trace[(size_t)(2 * b.trace_cap + 8 * b.trace_idx + id) * b.nblk + blockIdx.x] = wall_clock64();
}

// Development marks inside a stage (compiled in only with SOUFFLE_STAGE_MARKS).
#ifdef SOUFFLE_STAGE_MARKS
#define STAGE_MARK(tb, id) do { if (tb) trace_mark(*(tb), (id)); } while (0)
#else
#define STAGE_MARK(tb, id) do { (void)(tb); } while (0)
#endif

__device__ __forceinline__ void grid_barrier_begin(GridBarrier &b, unsigned *ctl, bool strict = false) {
  b.ctl = ctl;
  b.strict = strict;
  b.nblk = gridDim.x;
  b.count = 0;
  b.failed = false;
  b.trace = nullptr;
  b.trace_idx = 0;
  b.trace_cap = 0;
  const unsigned x = blockIdx.x & 7;
  b.gsz = (b.nblk + 7 - x) >> 3;
  b.target = __hip_atomic_load(ctl + kCtlCarry + 32 * x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  b.epoch = __hip_atomic_load(ctl + kCtlEpoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// s_waitcnt with only the vector-memory counter: all but the youngest N vector memory
// instructions of this wave have completed (they complete in issue order).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  // No memory access of the program may cross the wait in either direction: a load hoisted above it
  // would be one of the N youngest, and one of the loads the caller waits for could still be in flight.
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}

// Every memory operation this wave has issued is complete (write-through stores acknowledged, loads returned,
// LDS and scalar traffic done), and the compiler moves no memory access across the wait in either direction:
// the release half of a hand-over to other workgroups, in front of the barrier that precedes the flag store.
__device__ __forceinline__ void wait_all_memory() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }
// The compiler moves no memory access across this point (the hardware is not involved): behind the poll of a
// hand-over, so that no load of what other workgroups published is scheduled in front of the poll.
__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

// `mid()` is called by every wave after the workgroup has arrived and before it starts to wait:
// the place to queue loads that do not depend on other workgroups (the next stage's weight
// slice), so that they travel while the barrier completes.  Wave 0 polls; its polling loads
// return in issue order, so it must not queue anything slow in mid() itself.
template <class Mid>
__device__ __forceinline__ void grid_sync(GridBarrier &b, Mid mid) {
  const bool tr = b.trace && b.trace_idx < b.trace_cap && threadIdx.x == 0;
  if (tr) b.trace[(size_t)(2 * b.trace_idx) * b.nblk + blockIdx.x] = wall_clock64();
  wait_all_memory();                       // write-through stores are acknowledged
  strict_release(b.strict);
  __builtin_amdgcn_s_barrier();
  compiler_fence();
#ifdef SOUFFLE_STAGE_MARKS
  trace_mark(b, 7);
#endif
  b.target += b.gsz;
  b.epoch += 1;
  if (threadIdx.x == 0) {
    const unsigned x = blockIdx.x & 7;
    const unsigned old = __hip_atomic_fetch_add(b.ctl + kCtlArrive + 32 * x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old + 1 == b.target) __hip_atomic_store(b.ctl + kCtlDone + 32 * x, b.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_barrier();            // the arrival (and the done flag) precede whatever mid() queues
  mid();
  if (threadIdx.x < 64 && !b.failed) {
    for (int spin = 0; spin < kMaxBarrierSpin; ++spin) {
      bool ok = true;
      if (threadIdx.x < 8 && threadIdx.x < b.nblk)
        ok = (int)(__hip_atomic_load(b.ctl + kCtlDone + 32 * threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - b.epoch) >= 0;
      if (__all(ok)) break;
      __builtin_amdgcn_s_sleep(1);
      if (spin == kMaxBarrierSpin - 1) {   // gave up: the launch's output is invalid, and it ends without further waits
        b.failed = true;
        if (threadIdx.x == 0) (void)__hip_atomic_fetch_or(b.ctl + kCtlErrWord, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  b.count++;
  if (tr) b.trace[(size_t)(2 * b.trace_idx + 1) * b.nblk + blockIdx.x] = wall_clock64();
  b.trace_idx++;
  __builtin_amdgcn_s_barrier();            // no memory wait here: loads queued by mid() may still be in flight
  strict_acquire(b.strict);
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  compiler_fence();                        // no load of what the other workgroups wrote is scheduled above the poll
}
__device__ __forceinline__ void grid_sync(GridBarrier &b) { grid_sync(b, []() {}); }

// Call once by every workgroup before the kernel returns.
__device__ __forceinline__ void grid_barrier_end(GridBarrier &b) {
  if (b.count > 0 && blockIdx.x < 8 && threadIdx.x == 0) {
    __hip_atomic_store(b.ctl + kCtlCarry + 32 * blockIdx.x, b.target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (blockIdx.x == 0) __hip_atomic_store(b.ctl + kCtlEpoch, b.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The next launch on this control block reads these words first thing.  The wave does not end
    // before they are acknowledged, so that their arrival does not rest on what the end of a kernel
    // waits for when the runtime queues two launches without a cache release in between.
    wait_all_memory();
  }
}

}  // namespace souffle
