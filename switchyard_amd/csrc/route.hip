// route: router logits -> fp32 softmax -> top-k expert ids and weights.
//
// One wavefront (64 lanes) per token; lane l holds logit l (and l+64 when E > 64), so for
// OLMoE's 64 experts every lane owns exactly one logit. Max and sum are wave all-reduces;
// the k picks are k rounds of a wave arg-max over the key (logit descending, expert id
// ascending). The key is the logit itself: exp is monotone, so this is the order of the
// softmax probabilities, and it is exact. Lane r keeps pick r and writes it.
//
// Replaces route() / route_kernel of the reference (switchyard/csrc/moe_kernels.cu:20-89).
#include "common.h"

namespace {

constexpr int ROUTE_THREADS = 256;
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
__device__ __forceinline__ Cand cand_xor(Cand c, int o) {
  return Cand{__shfl_xor(c.v, o, WAVE), __shfl_xor(c.e, o, WAVE)};
}

template <typename T, int PER_LANE>
__global__ void __launch_bounds__(ROUTE_THREADS)
route_kernel(const T* __restrict__ logits, int N, int E, int k, int norm, int* __restrict__ idx, T* __restrict__ w) {
  const int token = (blockIdx.x * ROUTE_THREADS + threadIdx.x) >> 6, lane = threadIdx.x & 63;
  if (token >= N) return;  // whole wavefronts leave together
  const T* row = logits + (size_t)token * E;

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

  int my_e = 0;
  float my_p = 0.f, total = 0.f;
  for (int r = 0; r < k; ++r) {
    Cand c{0.f, NO_EXPERT};
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j)
      if (open[j]) c = better(c, Cand{v[j], lane + WAVE * j});
    c = better(c, cand_row_ror<8>(c));
    c = better(c, cand_row_ror<4>(c));
    c = better(c, cand_row_ror<2>(c));
    c = better(c, cand_row_ror<1>(c));
    c = better(c, cand_xor(c, 16));
    c = better(c, cand_xor(c, 32));
    // the winner's probability lives in lane c.e % 64, register c.e / 64
    float pw = p[0];
#pragma unroll
    for (int j = 1; j < PER_LANE; ++j) pw = (c.e >= WAVE * j) ? p[j] : pw;
    pw = __shfl(pw, c.e & 63, WAVE);
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
  if (lane < k) {
    idx[(size_t)token * k + lane] = my_e;
    w[(size_t)token * k + lane] = (T)(norm ? my_p / total : my_p);
  }
}

template <typename T>
int launch_route(const void* logits, int N, int E, int k, int norm, int32_t* idx, void* w, hipStream_t stream) {
  const int blocks = (int)(((size_t)N * WAVE + ROUTE_THREADS - 1) / ROUTE_THREADS);
  if (E <= 64)
    route_kernel<T, 1><<<blocks, ROUTE_THREADS, 0, stream>>>((const T*)logits, N, E, k, norm, idx, (T*)w);
  else
    route_kernel<T, 2><<<blocks, ROUTE_THREADS, 0, stream>>>((const T*)logits, N, E, k, norm, idx, (T*)w);
  return sy_check_launch("route");
}

}  // namespace

extern "C" SY_API int sy_route(const void* logits, int dtype, int N, int E, int k, int norm, int32_t* idx, void* w,
                        void* stream) {
  SY_REQUIRE(N >= 0, "route: N = %d is negative", N);
  SY_REQUIRE(E >= 1 && E <= 128 && k >= 1 && k <= 8 && k <= E,
             "route: at most 128 experts and top-8 (got E = %d, k = %d)", E, k);
  SY_REQUIRE(dtype == SY_DTYPE_F16 || dtype == SY_DTYPE_F32, "route: logits must be f16 or f32 (dtype %d)", dtype);
  if (N == 0) return SY_OK;
  SY_REQUIRE(logits && idx && w, "route: null pointer");
  if (dtype == SY_DTYPE_F16) return launch_route<half_t>(logits, N, E, k, norm, idx, w, (hipStream_t)stream);
  return launch_route<float>(logits, N, E, k, norm, idx, w, (hipStream_t)stream);
}
