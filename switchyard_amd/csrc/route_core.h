// One wavefront routes one token: fp32 softmax over E logits and the k best experts.
//
// Lane l holds logit l (and l + 64 when E > 64), so for 64 experts every lane owns exactly one
// logit. Max and sum are wave all-reduces; the k picks are k rounds of a wave arg-max over
// the key (logit descending, expert id ascending). The key is the logit itself: exp is
// monotone, so this is the order of the softmax probabilities, and it is exact. For f16
// logits the pair packs into one integer (the logit's bits made monotone above, 127 - id
// below), so a round is a single integer max over the wavefront (3.0 us for a launch of 8
// tokens against 5.4 us with a compare of pairs); f32 logits compare the pair. Lane r keeps
// pick r: on return lanes 0..k-1 hold (expert, weight) of the token's k choices.
//
// Follows route_kernel of the reference (switchyard/csrc/moe_kernels.cu:23-71).
#pragma once

#include "common.h"

namespace route_core {

constexpr int NO_EXPERT = 0x7fffffff;

struct Cand {
  float v;
  int e;
};

__device__ __forceinline__ Cand better(Cand a, Cand b) {
  // b replaces a if a is empty, or b is a real candidate with a larger logit, or an equal
  // logit and a lower expert id.
  bool take = b.e != NO_EXPERT && (a.e == NO_EXPERT || b.v > a.v || (b.v == a.v && b.e < a.e));
  return take ? b : a;
}

template <int N>
__device__ __forceinline__ Cand cand_row_ror(Cand c) {
  return Cand{dpp_row_ror<N>(c.v), dpp_row_ror<N>(c.e)};
}
__device__ __forceinline__ Cand cand_lane(Cand c, int lane) { return Cand{read_lane(c.v, lane), read_lane(c.e, lane)}; }

// The best candidate of the wavefront, wave-uniform: DPP inside the rows of 16 lanes, then the
// four row winners meet in scalar registers.
__device__ __forceinline__ Cand wave_best(Cand c) {
  c = better(c, cand_row_ror<8>(c));
  c = better(c, cand_row_ror<4>(c));
  c = better(c, cand_row_ror<2>(c));
  c = better(c, cand_row_ror<1>(c));
  return better(better(cand_lane(c, 0), cand_lane(c, 16)), better(cand_lane(c, 32), cand_lane(c, 48)));
}

// Must be called by all 64 lanes of a wavefront. `row` points at the token's E logits.
template <typename T, int PER_LANE>
__device__ __forceinline__ void route_token(const T* row, int E, int k, int norm, int& my_e, float& my_w) {
  const int lane = threadIdx.x & 63;
  float v[PER_LANE], p[PER_LANE];
  bool open[PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < PER_LANE; ++j) {
    const int e = lane + WAVE * j;
    open[j] = e < E;
    v[j] = open[j] ? (float)row[e] : -INFINITY;
    mx = fmaxf(mx, v[j]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < PER_LANE; ++j) {
    p[j] = open[j] ? expf(v[j] - mx) : 0.f;
    sum += p[j];
  }
  sum = wave_sum(sum);

  my_e = 0;
  float my_p = 0.f, total = 0.f;
  if (sizeof(T) == 2) {
    // f16 logits: (logit, id) packs into one unsigned key that orders like the pair, the
    // logit's bits made monotone in the upper half (with -0 as +0, which compare equal) and
    // 127 - id below them, so a pick is one wave-wide integer max.
    unsigned key[PER_LANE];
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
      const half_t hv = (half_t)v[j];
      unsigned bits = v[j] == 0.f ? 0u : (unsigned)__builtin_bit_cast(unsigned short, hv);
      bits = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
      key[j] = open[j] ? (bits << 7) | (unsigned)(127 - (lane + WAVE * j)) : 0u;  // 0 is below every real key
    }
    for (int r = 0; r < k; ++r) {
      int best = (int)key[0];  // 23 bits
#pragma unroll
      for (int j = 1; j < PER_LANE; ++j) best = best > (int)key[j] ? best : (int)key[j];
      best = wave_allreduce(best, [](int a, int b) { return a > b ? a : b; });
      const int e = 127 - (best & 127);
      float pw = read_lane(p[0], e & 63);
#pragma unroll
      for (int j = 1; j < PER_LANE; ++j) pw = (e >= WAVE * j) ? read_lane(p[j], e & 63) : pw;
#pragma unroll
      for (int j = 0; j < PER_LANE; ++j)
        if (lane + WAVE * j == e) key[j] = 0u;
      const float picked = pw / sum;
      total += picked;
      if (lane == r) {
        my_e = e;
        my_p = picked;
      }
    }
    my_w = norm ? my_p / total : my_p;
    return;
  }
  for (int r = 0; r < k; ++r) {
    Cand c{0.f, NO_EXPERT};
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j)
      if (open[j]) c = better(c, Cand{v[j], lane + WAVE * j});
    c = wave_best(c);
    // the winner's probability lives in lane c.e % 64, register c.e / 64
    float pw = read_lane(p[0], c.e & 63);
#pragma unroll
    for (int j = 1; j < PER_LANE; ++j) pw = (c.e >= WAVE * j) ? read_lane(p[j], c.e & 63) : pw;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j)
      if (lane + WAVE * j == c.e) open[j] = false;
    const float picked = pw / sum;
    total += picked;
    if (lane == r) {
      my_e = c.e;
      my_p = picked;
    }
  }
  my_w = norm ? my_p / total : my_p;
}

}  // namespace route_core
