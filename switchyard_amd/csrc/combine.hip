// combine: each token's k expert outputs summed in fp32, in ascending expert id, rounded to
// f16 once.
//
// One workgroup per token. The first wavefront loads the token's k ids and rows together, ranks
// the choices by (expert id, slot) with lane reads and leaves the k source rows in LDS in that
// order; then every thread owns 16-byte columns of the output and adds the k rows in order, so
// the result does not depend on the launch shape.
//
// Replaces combine_kernel / combine of the reference (switchyard/csrc/moe_kernels.cu:417-444).
#include "common.h"

namespace {

constexpr int COMBINE_THREADS = 256;
constexpr int MAX_K = 64;

// WEIGHTED: y holds the down projection before the router weight, and each row is multiplied by
// its choice's weight here, rounded to f16 as the projection's own epilogue rounds it, before it
// is added: the same bits as combining rows that were scaled where they were computed.
template <bool WEIGHTED>
__global__ void __launch_bounds__(COMBINE_THREADS)
combine_kernel(const half_t* __restrict__ y, const int* __restrict__ pos_of, const int* __restrict__ idx,
               const half_t* __restrict__ w, int k, int H, half_t* __restrict__ out) {
  __shared__ int rows[MAX_K];
  __shared__ float weights[MAX_K];
  const int t = blockIdx.x, tid = threadIdx.x;
  if (tid < WAVE) {
    const int mine = tid < k ? idx[(size_t)t * k + tid] : 0x7fffffff;
    const int row = tid < k ? pos_of[(size_t)t * k + tid] : 0;
    int rank = 0;
    for (int j = 0; j < k; ++j) {
      const int other = read_lane(mine, j);
      rank += (other < mine) || (other == mine && j < tid);
    }
    if (tid < k) {
      rows[rank] = row;
      if (WEIGHTED) weights[rank] = (float)w[(size_t)t * k + tid];
    }
  }
  __syncthreads();
  for (int c = tid * 8; c < H; c += COMBINE_THREADS * 8) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const half8_t v = *reinterpret_cast<const half8_t*>(y + (size_t)rows[j] * H + c);
      const float wt = WEIGHTED ? weights[j] : 1.f;
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] += WEIGHTED ? (float)(half_t)((float)v[q] * wt) : (float)v[q];
    }
    half8_t o;
#pragma unroll
    for (int q = 0; q < 8; ++q) o[q] = (half_t)acc[q];
    *reinterpret_cast<half8_t*>(out + (size_t)t * H + c) = o;
  }
}

}  // namespace

extern "C" SY_API int sy_combine(const void* y, const int32_t* pos_of, const int32_t* idx, int N, int k, int H, void* out,
                          void* stream) {
  SY_REQUIRE(N >= 0, "combine: N = %d is negative", N);
  SY_REQUIRE(k >= 1 && k <= MAX_K, "combine: 1 <= k <= %d (got %d)", MAX_K, k);
  SY_REQUIRE(H >= 8 && H % 8 == 0, "combine: H must be a positive multiple of 8 (got %d)", H);
  if (N == 0) return SY_OK;
  SY_REQUIRE(y && pos_of && idx && out, "combine: null pointer");
  combine_kernel<false><<<N, COMBINE_THREADS, 0, (hipStream_t)stream>>>((const half_t*)y, pos_of, idx, nullptr, k, H, (half_t*)out);
  return sy_check_launch("combine");
}

// combine of rows that the down projection left unscaled: w f16 [N, k] are the router weights of
// the choices in routing order (route's output). Used by sy_moe_experts, whose down projection
// then needs no scales: fetching them costs its epilogue more than the multiply costs here.
int sy_combine_weighted(const void* y, const int32_t* pos_of, const int32_t* idx, const void* w, int N, int k, int H, void* out,
                        void* stream) {
  SY_REQUIRE(N >= 0 && k >= 1 && k <= MAX_K && H >= 8 && H % 8 == 0, "combine: N = %d, k = %d, H = %d", N, k, H);
  if (N == 0) return SY_OK;
  SY_REQUIRE(y && pos_of && idx && w && out, "combine: null pointer");
  combine_kernel<true><<<N, COMBINE_THREADS, 0, (hipStream_t)stream>>>((const half_t*)y, pos_of, idx, (const half_t*)w, k, H,
                                                                     (half_t*)out);
  return sy_check_launch("combine");
}
