// Definitions shared by the two BERT encoder paths (few rows: bert_small.hpp; many rows: bert.hip).
#pragma once
#include "common.hpp"
#include "../../include/souffle_hip.h"

namespace souffle {
namespace bert {

constexpr int H = 768, NH = 12, HD = 64, F = 3072;
constexpr int kMaxLayers = 24;

struct LayerW {
  const half_t *w_qkv, *b_qkv, *w_o, *b_o, *ln1_g, *ln1_b, *w_fc1, *b_fc1, *w_fc2, *b_fc2, *ln2_g, *ln2_b;
  const half_t *w_fc2p;      // w_fc2 in the layout of souffle_bert_pack_fc2, or null
};

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

}  // namespace bert
}  // namespace souffle
