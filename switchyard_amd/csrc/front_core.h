// The tail that turns a launch with one workgroup per token, each holding its token's router
// logits in LDS, into the whole front of the layer: every workgroup routes its own token, and the
// workgroup that finishes last sorts all the choices.
//
// The order of arrival is a ticket: after its token's ids and weights are in memory a workgroup
// takes the next number of a counter (behind a release fence of device scope), and the one that
// draws N - 1 knows that every other workgroup's choices were written before (acquire fence). Nobody waits for anybody:
// a workgroup that is not last simply ends. The last one puts the counter back to zero, so the
// next launch that uses it finds it as this one did.
//
// The counters are a pool in device memory that the library owns; consecutive launches take
// consecutive slots of one half of the pool (launches recorded by a stream capture of the other
// half, because they keep their slot for every replay), so two launches share a slot only if
// FRONT_TICKETS / 2 launches of their kind were enqueued between them, and then only matter to
// each other if they run at the same time on different streams.
//
// Outputs are those of route followed by sort_by_expert of the reference
// (switchyard/csrc/moe_kernels.cu:73-89,142-157).
#pragma once

#include "route_core.h"
#include "sort_core.h"

namespace front_core {

constexpr int FRONT_TICKETS = 1024;
constexpr int TAIL_MAX_TOKENS = 256;  // the last workgroup sorts alone
constexpr int TAIL_MAX_K = 8;

struct Outputs {
  int* idx;            // [N, k]
  half_t* w;           // [N, k]
  int* counts;         // [E]
  int* offsets;        // [E + 1]
  int* token;          // [N * k]
  half_t* wsorted;     // [N * k]
  int* pos_of;         // [N * k]
  unsigned* ticket;    // this launch's counter, zero on entry and on exit
  int k, norm, nbits;
};

// Bytes of LDS the tail needs behind the caller's own: the token's logits, the sort's scratch
// and every choice's id and weight.
__host__ __device__ constexpr size_t tail_lds_bytes(int N, int E, int k) {
  return sizeof(half_t) * ((size_t)(E + 7) / 8 * 8) + sizeof(int) * (sort_core::small_sort_lds_ints(E) + (size_t)N * k) +
         sizeof(half_t) * (size_t)N * k;
}

// The route alone, for a caller whose next launch sorts for itself (the weight stream of a decode
// step of at most 64 choices does): the workgroup's first wavefront routes token t from the
// logits at `lds`; nothing is counted and nobody sorts. Only idx and w of `o` are used.
template <int PER_LANE>
__device__ __forceinline__ void route_own(int t, int E, const Outputs& o, const unsigned char* lds) {
  if ((threadIdx.x >> 6) != 0) return;
  const int lane = threadIdx.x & 63;
  int my_e;
  float my_w;
  route_core::route_token<half_t, PER_LANE>(reinterpret_cast<const half_t*>(lds), E, o.k, o.norm, my_e, my_w);
  if (lane < o.k) {
    o.idx[t * o.k + lane] = my_e;
    o.w[t * o.k + lane] = (half_t)my_w;
  }
}

// Called by every thread of a workgroup of SORT_THREADS threads whose token is t of N, after a
// barrier behind which `lg` (the first E halves of `lds`) holds the token's logits.
template <int PER_LANE>
__device__ __forceinline__ void route_own_sort_last(int t, int N, int E, const Outputs& o, unsigned char* lds) {
  using namespace sort_core;
  __shared__ int s_last;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int k = o.k, M = N * k;
  const half_t* lg = reinterpret_cast<const half_t*>(lds);
  int* scratch = reinterpret_cast<int*>(lds + sizeof(half_t) * ((size_t)(E + 7) / 8 * 8));
  int* sidx = scratch + small_sort_lds_ints(E);
  half_t* sw = reinterpret_cast<half_t*>(sidx + M);

  bool last = false;
  if (wave == 0) {
    int my_e;
    float my_w;
    route_core::route_token<half_t, PER_LANE>(lg, E, k, o.norm, my_e, my_w);
    if (lane < k) {
      o.idx[t * k + lane] = my_e;
      o.w[t * k + lane] = (half_t)my_w;
    }
    // every lane's stores are released before lane 0 draws (the fence is the wavefront's)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    unsigned drawn = 0;
    if (lane == 0) drawn = __hip_atomic_fetch_add(o.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = __builtin_amdgcn_readfirstlane(drawn) == (unsigned)(N - 1);
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (lane == 0) {
      s_last = last;
      if (last) __hip_atomic_store(o.ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (M <= WAVE) {
    // one choice per lane: the wavefront that routed sorts, nobody else has anything to do
    if (wave != 0 || !last) return;
    sort_one_wave<uint16_t>(o.idx, reinterpret_cast<const uint16_t*>(o.w), M, k, E, o.nbits, o.counts, o.offsets, o.token,
                            reinterpret_cast<uint16_t*>(o.wsorted), o.pos_of, scratch);
    return;
  }
  __syncthreads();
  if (!s_last) return;
  // the barrier carried wavefront 0's acquire to the others
  for (int i = threadIdx.x; i < M; i += (int)blockDim.x) {
    sidx[i] = o.idx[i];
    sw[i] = o.w[i];
  }
  __syncthreads();
  sort_small_block<uint16_t>(sidx, reinterpret_cast<const uint16_t*>(sw), M, k, E, o.nbits, o.counts, o.offsets, o.token,
                             reinterpret_cast<uint16_t*>(o.wsorted), o.pos_of, scratch);
}

}  // namespace front_core
