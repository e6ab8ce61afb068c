// Stacked LSTM (10 x 256, batch 1) as one persistent cooperative kernel on gfx950.
//
// Replaces fused_lstm<1,10,256,100> (cpp/lstm/lstm_binding.cu:30-78) and its wavefront
// kernel (cpp/lstm/lstm_reuse_shared_memory.cu:179-337).  Differences by design:
//   - every layer's W_ih|W_hh slice lives in REGISTERS for the whole sequence (64 VGPRs of
//     packed fp16 per lane; the reference splits it over shared memory and registers);
//   - there is no grid barrier per step: a cell (layer l, step t) starts as soon as
//     h(l-1, t) and h(l, t-1) have arrived.  Each published h value carries its step tag in
//     the same 8-byte write-through store, so consumers poll the data itself (one round
//     trip, no flags, no atomics) and the layers run as a true wavefront;
//   - layer 0 consumes x_t (not the reference kernel's one-step-late x_{t-1}, :324-326),
//     state and accumulation are fp32, weights fp16.
//   - (tried: the 16 workgroups of a layer on one XCD with L2-scope polls for the recurrent
//     hand-over; 258 us against 223 us, the write-through stores are not seen sooner through the L2);
// Workgroup (l, g) owns hidden units [16g, 16g+16) of layer l: 64 gate rows x 512 inputs.
// Lane layout inside a wave: unit = lane/16, gate = (lane/4)%4, column phase = lane%4, so
// the four gates of a unit meet through three lane shuffles.
#include "common.hpp"
#include "host_util.hpp"

namespace souffle {
namespace lstm {

constexpr int HID = 256, WG_PER_LAYER = 16, UNITS_PER_WG = 16;
constexpr int kMaxSpin = 1 << 22;

struct Args {
  int layers, timesteps, gate_order;
  float forget_bias;
  const half_t *w_ih, *w_hh;
  const float *bias, *x;
  float *y;
  u2 *hbuf;          // [layers][timesteps][256] of (value bits, step tag)
  unsigned *ctl;     // grid-barrier control block; word kCtlErrWord = sticky error flag
  int strict;        // souffle_set_strict_fences (the grid barrier at the end; the step tags travel with their values)
};

__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + __expf(-v)); }
__device__ __forceinline__ float tanhf_(float v) { return 1.0f - 2.0f / (__expf(2.0f * v) + 1.0f); }

__global__ void __launch_bounds__(256) k_lstm(Args a) {
  __shared__ __attribute__((aligned(16))) float in_s[2][2 * HID];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l = blockIdx.x / WG_PER_LAYER, g = blockIdx.x % WG_PER_LAYER;
  const int ul = lane >> 4, k = (lane >> 2) & 3, c = lane & 3;
  const int unit = g * UNITS_PER_WG + wave * 4 + ul;
  // logical gate k (0 i, 1 f, 2 g, 3 o) -> stored slot
  const int slot = a.gate_order == SOUFFLE_GATES_IFGO ? k : (k == 1 ? 2 : (k == 2 ? 1 : k));

  GridBarrier bar;
  grid_barrier_begin(bar, a.ctl, a.strict != 0);

  // weights of this lane: row (l, slot, unit), columns 32j + 8c .. +7 of [W_ih | W_hh]
  u4 w[16];
  {
    const size_t row = ((size_t)(l * 4 + slot) * HID + unit) * HID;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      w[j] = *reinterpret_cast<const u4 *>(a.w_ih + row + 32 * j + 8 * c);
      w[8 + j] = *reinterpret_cast<const u4 *>(a.w_hh + row + 32 * j + 8 * c);
    }
  }
  const float bias = a.bias ? a.bias[(size_t)(l * 4 + slot) * HID + unit] : 0.f;
  float cstate = 0.f;
  bool failed = false;
  const u2 *below = a.hbuf + (size_t)(l > 0 ? l - 1 : 0) * a.timesteps * HID;
  u2 *own = a.hbuf + (size_t)l * a.timesteps * HID;

  for (int t = 0; t < a.timesteps; ++t) {
    float *in = in_s[t & 1];
    // gather the 512 inputs: thread tid fetches element tid of each half.  h(l-1, t) and h(l, t-1)
    // were produced in the same wavefront step, so both are polled together: one memory round
    // trip when both are there, not one after the other.  (Keeping several polls in flight per
    // thread to see the value sooner was tried: the extra traffic made a step 45 % slower.)
    float v0 = 0.f, v1 = 0.f;
    {
      const bool need0 = l > 0, need1 = t > 0;
      if (!need0) v0 = a.x[(size_t)t * HID + tid];
      const u2 *p0 = below + (size_t)t * HID + tid, *p1 = own + (size_t)(t > 0 ? t - 1 : 0) * HID + tid;
      bool ok0 = !need0, ok1 = !need1;
      // once a wait has given up, later steps do not wait again: the launch is flagged as failed and ends quickly
      for (int spin = 0; !(ok0 && ok1) && !failed; ++spin) {
        if (spin >= kMaxSpin) { failed = true; break; }
        // (a slot that is already in is polled again: harmless, and the loop stays branch-free)
        const u2 q0 = ld8_atomic(p0), q1 = ld8_atomic(p1);
        if (!ok0 && q0[1] == (unsigned)(t + 1)) { v0 = __uint_as_float(q0[0]); ok0 = true; }
        if (!ok1 && q1[1] == (unsigned)t) { v1 = __uint_as_float(q1[0]); ok1 = true; }
      }
    }
    in[tid] = v0;
    in[HID + tid] = v1;
    __syncthreads();

    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const f4 x0 = *reinterpret_cast<const f4 *>(in + 32 * j + 8 * c);
      const f4 x1 = *reinterpret_cast<const f4 *>(in + 32 * j + 8 * c + 4);
      const h8 wv = as_h8(w[j]);
      acc += (float)wv[0] * x0[0] + (float)wv[1] * x0[1] + (float)wv[2] * x0[2] + (float)wv[3] * x0[3];
      acc += (float)wv[4] * x1[0] + (float)wv[5] * x1[1] + (float)wv[6] * x1[2] + (float)wv[7] * x1[3];
    }
    acc += wave_xor(acc, 1);
    acc += wave_xor(acc, 2);
    acc += bias;
    // bring the four gate pre-activations of this unit to its lane with k == 0, c == 0
    const int base = lane & ~15;
    const float pi = __shfl(acc, base + 0, kWave), pf = __shfl(acc, base + 4, kWave);
    const float pg = __shfl(acc, base + 8, kWave), po = __shfl(acc, base + 12, kWave);
    if ((lane & 15) == 0) {
      // c' = c sigma(f + fb) + sigma(i) tanh(g); h = tanh(c') sigma(o)
      // (cpp/lstm/lstm_reuse_shared_memory.cu:309-318)
      cstate = cstate * sigmoidf_(pf + a.forget_bias) + sigmoidf_(pi) * tanhf_(pg);
      const float h = tanhf_(cstate) * sigmoidf_(po);
      st8_atomic(own + (size_t)t * HID + unit, u2{__float_as_uint(h), (unsigned)(t + 1)});
      if (l == a.layers - 1) a.y[(size_t)t * HID + unit] = h;
    }
  }
  if (failed) atomicOr(a.ctl + kCtlErrWord, 1u);
  // everything has been consumed once every workgroup is here: clear this workgroup's
  // published slots so that the next launch (or a graph replay) starts from empty tags
  grid_sync(bar);
  for (int i = tid; i < a.timesteps * UNITS_PER_WG; i += 256) {
    const int t = i / UNITS_PER_WG, u = g * UNITS_PER_WG + i % UNITS_PER_WG;
    st8_atomic(own + (size_t)t * HID + u, u2{0u, 0u});
  }
  // (acknowledged before the wave ends: a clearing store that were still on its way when the next
  // launch publishes into the same slot would wipe that value out)
  wait_all_memory();
  grid_barrier_end(bar);
}

static size_t ws_bytes(const souffle_lstm_cfg *c) {
  return round_up(kCtlWords * 4, 256) + (size_t)c->layers * c->timesteps * HID * 8;
}

static int validate(const souffle_lstm_cfg *c) {
  if (!c) return fail(SOUFFLE_ERR_NULL, "cfg is NULL");
  if (c->hidden != HID) return fail(SOUFFLE_ERR_SHAPE, "only hidden=256 is built (got %d)", c->hidden);
  if (c->batch != 1) return fail(SOUFFLE_ERR_SHAPE, "only batch=1 is built (got %d)", c->batch);
  if (c->layers < 1 || c->layers > 16) return fail(SOUFFLE_ERR_SHAPE, "layers must be in 1..16 (got %d)", c->layers);
  if (c->timesteps < 1 || c->timesteps > 4096) return fail(SOUFFLE_ERR_SHAPE, "timesteps must be in 1..4096 (got %d)", c->timesteps);
  if (c->gate_order != SOUFFLE_GATES_IFGO && c->gate_order != SOUFFLE_GATES_IGFO)
    return fail(SOUFFLE_ERR_SHAPE, "unknown gate order %d", c->gate_order);
  return SOUFFLE_OK;
}

}  // namespace lstm
}  // namespace souffle

using namespace souffle;

extern "C" size_t souffle_lstm_workspace_bytes(const souffle_lstm_cfg *cfg) {
  if (lstm::validate(cfg)) return 0;
  return lstm::ws_bytes(cfg);
}

extern "C" int souffle_lstm_fused(const souffle_lstm_cfg *cfg, const void *w_ih, const void *w_hh, const float *bias,
                                  const float *x, float *y, void *ws, size_t ws_bytes, souffle_stream_t stream) {
  if (int rc = lstm::validate(cfg)) return rc;
  if (!w_ih || !w_hh || !x || !y) return fail(SOUFFLE_ERR_NULL, "w_ih, w_hh, x and y must not be NULL");
  if (!ws) return fail(SOUFFLE_ERR_WORKSPACE, "workspace is NULL (need %zu bytes)", lstm::ws_bytes(cfg));
  if (ws_bytes < lstm::ws_bytes(cfg)) return fail(SOUFFLE_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, lstm::ws_bytes(cfg));
  if (!aligned16(w_ih) || !aligned16(w_hh) || !aligned16(x) || !aligned16(y) || !aligned16(ws) || (bias && !aligned16(bias)))
    return fail(SOUFFLE_ERR_ALIGN, "all pointers must be 16-byte aligned");
  DeviceFacts df;
  if (int rc = device_facts(&df)) return rc;
  const int grid = cfg->layers * lstm::WG_PER_LAYER;
  if (grid > df.num_cus)
    return fail(SOUFFLE_ERR_DEVICE, "needs %d workgroups resident at once, device has %d CUs", grid, df.num_cus);
  lstm::Args a;
  a.layers = cfg->layers; a.timesteps = cfg->timesteps; a.gate_order = cfg->gate_order; a.forget_bias = cfg->forget_bias;
  a.w_ih = static_cast<const half_t *>(w_ih); a.w_hh = static_cast<const half_t *>(w_hh);
  a.bias = bias; a.x = x; a.y = y;
  a.ctl = static_cast<unsigned *>(ws);
  a.strict = strict_fences_mode();
  a.hbuf = reinterpret_cast<u2 *>(static_cast<char *>(ws) + round_up(kCtlWords * 4, 256));
  void *args[] = {&a};
  return launch_persistent((const void *)lstm::k_lstm, grid, 256, args, 0, static_cast<hipStream_t>(stream));
}
