// route: router logits -> fp32 softmax -> top-k expert ids and weights.
//
// One wavefront (64 lanes) per token; the per-token work is route_core.h.
//
// Replaces route() / route_kernel of the reference (switchyard/csrc/moe_kernels.cu:20-89).
#include "route_core.h"

namespace {

constexpr int ROUTE_THREADS = 256;

template <typename T, int PER_LANE>
__global__ void __launch_bounds__(ROUTE_THREADS)
route_kernel(const T* __restrict__ logits, int N, int E, int k, int norm, int* __restrict__ idx, T* __restrict__ w) {
  const int token = (blockIdx.x * ROUTE_THREADS + threadIdx.x) >> 6, lane = threadIdx.x & 63;
  if (token >= N) return;  // whole wavefronts leave together
  int my_e;
  float my_w;
  route_core::route_token<T, PER_LANE>(logits + (size_t)token * E, E, k, norm, my_e, my_w);
  if (lane < k) {
    idx[(size_t)token * k + lane] = my_e;
    w[(size_t)token * k + lane] = (T)my_w;
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
