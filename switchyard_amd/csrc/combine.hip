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

__global__ void __launch_bounds__(COMBINE_THREADS)
combine_kernel(const half_t* __restrict__ y, const int* __restrict__ pos_of, const int* __restrict__ idx, int k, int H,
               half_t* __restrict__ out) {
  __shared__ int rows[MAX_K];
  const int t = blockIdx.x, tid = threadIdx.x;
  if (tid < WAVE) {
    const int mine = tid < k ? idx[(size_t)t * k + tid] : 0x7fffffff;
    const int row = tid < k ? pos_of[(size_t)t * k + tid] : 0;
    int rank = 0;
    for (int j = 0; j < k; ++j) {
      const int other = read_lane(mine, j);
      rank += (other < mine) || (other == mine && j < tid);
    }
    if (tid < k) rows[rank] = row;
  }
  __syncthreads();
  for (int c = tid * 8; c < H; c += COMBINE_THREADS * 8) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const half8_t v = *reinterpret_cast<const half8_t*>(y + (size_t)rows[j] * H + c);
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] += (float)v[q];
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
  combine_kernel<<<N, COMBINE_THREADS, 0, (hipStream_t)stream>>>((const half_t*)y, pos_of, idx, k, H, (half_t*)out);
  return sy_check_launch("combine");
}
