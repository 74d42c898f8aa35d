// route_sort: route and sort of a decode step in one launch.
//
// At a handful of tokens each step is a few microseconds of launch and memory latency around
// almost no work, next to two projections that take about 90 microseconds. One workgroup
// routes every token (one wavefront per token, the code of route.hip), keeps ids and weights
// in LDS, and sorts them with the single-workgroup code of sort.hip. The outputs are exactly
// those of route followed by sort_by_expert.
//
// Fuses route() and sort_by_expert() of the reference
// (switchyard/csrc/moe_kernels.cu:73-89,142-157; called back to back in switchyard/kernels.py:91-93,84).
#include "route_core.h"
#include "sort_core.h"

namespace {

using namespace sort_core;

constexpr int FRONT_THREADS = SORT_THREADS;  // 1024: the sort wants 16 wavefronts
constexpr int FRONT_MAX_TOKENS = 256;
constexpr int FRONT_MAX_K = 8;

template <int PER_LANE>
__global__ void __launch_bounds__(FRONT_THREADS)
front_kernel(const half_t* __restrict__ logits, int N, int E, int k, int norm, int nbits, int* __restrict__ idx,
             half_t* __restrict__ w, int* __restrict__ counts, int* __restrict__ offsets, int* __restrict__ token,
             half_t* __restrict__ wsorted, int* __restrict__ pos_of) {
  extern __shared__ int lds[];  // sort scratch, then idx [N*k] and w [N*k]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;

  // ---- route: one wavefront per token; ids and weights go to HBM and stay in LDS for the sort
  const int M = N * k;
  int* sidx = lds + small_sort_lds_ints(E);
  half_t* sw = reinterpret_cast<half_t*>(sidx + M);
  for (int t = wave; t < N; t += (int)(blockDim.x >> 6)) {
    int my_e;
    float my_w;
    route_core::route_token<half_t, PER_LANE>(logits + (size_t)t * E, E, k, norm, my_e, my_w);
    if (lane < k) {
      const half_t wh = (half_t)my_w;
      idx[t * k + lane] = my_e;
      w[t * k + lane] = wh;
      sidx[t * k + lane] = my_e;
      sw[t * k + lane] = wh;
    }
  }
  __syncthreads();

  // ---- sort: at most one choice per lane of one wavefront, or the workgroup's counting sort
  if (M <= WAVE) {
    if (wave == 0)
      sort_one_wave<uint16_t>(sidx, reinterpret_cast<const uint16_t*>(sw), M, k, E, nbits, counts, offsets, token,
                              reinterpret_cast<uint16_t*>(wsorted), pos_of, lds);
    return;
  }
  sort_small_block<uint16_t>(sidx, reinterpret_cast<const uint16_t*>(sw), M, k, E, nbits, counts, offsets, token,
                             reinterpret_cast<uint16_t*>(wsorted), pos_of, lds);
}

}  // namespace

extern "C" SY_API int sy_route_sort(const void* logits, int N, int E, int k, int norm, int32_t* idx, void* w,
                                    int32_t* counts, int32_t* offsets, int32_t* token, void* wsorted, int32_t* pos_of,
                                    void* stream) {
  SY_REQUIRE(N >= 1 && N <= FRONT_MAX_TOKENS, "route_sort: 1 <= N <= %d (got %d)", FRONT_MAX_TOKENS, N);
  SY_REQUIRE(E >= 1 && E <= 128 && k >= 1 && k <= FRONT_MAX_K && k <= E,
             "route_sort: at most 128 experts and top-8 (got E = %d, k = %d)", E, k);
  SY_REQUIRE(logits && idx && w && counts && offsets && token && wsorted && pos_of, "route_sort: null pointer");
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const int M = N * k;
  const size_t lds = sizeof(int) * (small_sort_lds_ints(E) + M) + sizeof(half_t) * M;
  hipStream_t st = (hipStream_t)stream;
  // one wavefront per token is all that the route needs when one wavefront sorts
  // (the route loop strides by the wavefronts present, so fewer wavefronts than tokens is fine)
  const int threads = M <= WAVE && N * WAVE <= FRONT_THREADS ? N * WAVE : FRONT_THREADS;
  if (E <= 64)
    front_kernel<1><<<1, threads, lds, st>>>((const half_t*)logits, N, E, k, norm, nbits, idx, (half_t*)w, counts,
                                                  offsets, token, (half_t*)wsorted, pos_of);
  else
    front_kernel<2><<<1, threads, lds, st>>>((const half_t*)logits, N, E, k, norm, nbits, idx, (half_t*)w, counts,
                                                  offsets, token, (half_t*)wsorted, pos_of);
  return sy_check_launch("route_sort");
}
