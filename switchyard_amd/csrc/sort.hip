// sort_by_expert: stable counting sort of the N*k routing choices by expert id, without
// atomics, so a run is deterministic.
//
// The flat choices i = t*k + s are cut into consecutive pieces, one per wavefront. A
// wavefront walks its piece 64 choices at a time. For one group of 64 it finds, for every
// lane, the set of lanes holding the same expert (a "match" built from one ballot per bit of
// the expert id); the number of matching lanes below a lane is that choice's rank inside the
// group, and the highest matching lane adds the group's count to the wavefront's running
// per-expert counter in LDS (one writer per expert, so no atomic is needed).
//
//   pass 1  per-wavefront histograms
//   scan    per expert: exclusive prefix over wavefronts (stability across pieces) and the
//           total; then an exclusive scan over experts gives `offsets`
//   pass 2  the same walk again; row = offsets[e] + prefix[wavefront][e] + running + rank
//
// Up to SMALL_M choices the three steps run in one launch of one workgroup (decode: one
// launch instead of the reference's two kernels and three library calls). Above that, pass 1
// is a launch over many workgroups that leaves its histograms in the workspace, and the
// second launch does the scan redundantly in every workgroup before its pass 2.
//
// Replaces count_kernel / assign_kernel / sort_by_expert of the reference
// (switchyard/csrc/moe_kernels.cu:91-157).
#include <mutex>

#include "sort_core.h"

namespace {

using namespace sort_core;

// Workspace of sy_sort_by_expert_static: the per-wavefront histograms of the launches over many
// workgroups, for callers that cannot allocate. Every GPU the library runs on holds its own
// copy of this array until the process ends. In host code the array's name is only a handle
// for hipGetSymbolAddress, never a device address: launches take static_scratch()'s pointer.
static __device__ __align__(256) unsigned char scratch[SY_SORT_STATIC_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES] = {nullptr};

// Address of `scratch` on the current device, resolved once per device.
int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
    return sy_fail(SY_ERR_LAUNCH, "sort_by_expert_static: no current device below %d", MAX_DEVICES);
  std::lock_guard<std::mutex> hold(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* p = nullptr;
    const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !p)
      return sy_fail(SY_ERR_LAUNCH, "sort_by_expert_static: hipGetSymbolAddress: %s", hipGetErrorString(err));
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return SY_OK;
}

// ---------------------------------------------------------------- one workgroup does it all
template <typename W>
__global__ void __launch_bounds__(SORT_THREADS)
sort_small_kernel(const int* __restrict__ idx, const W* __restrict__ w, int M, int k, int E, int nbits,
                  int* __restrict__ counts, int* __restrict__ offsets, int* __restrict__ token,
                  W* __restrict__ wsorted, int* __restrict__ pos_of) {
  extern __shared__ int lds[];
  sort_small_block<W>(idx, w, M, k, E, nbits, counts, offsets, token, wsorted, pos_of, lds);
}

// ---------------------------------------------------------------- many workgroups
// Launch 1: virtual wavefront v = blockIdx.x * SORT_WAVES + wave owns choices
// [v*piece, (v+1)*piece) and writes its histogram to ws[v][0..E).
__global__ void __launch_bounds__(SORT_THREADS)
sort_count_kernel(const int* __restrict__ idx, int M, int E, int nbits, int piece, int* __restrict__ ws) {
  extern __shared__ int lds[];  // [SORT_WAVES][E]
  const int t = threadIdx.x, wv = t >> 6;
  for (int j = t; j < SORT_WAVES * E; j += SORT_THREADS) lds[j] = 0;
  __syncthreads();
  const int v = blockIdx.x * SORT_WAVES + wv;
  const long lo64 = (long)v * piece;
  const int lo = (int)(lo64 < M ? lo64 : M), hi = min(lo + piece, M);
  count_piece(idx, lo, hi, E, nbits, lds + wv * E);
  __syncthreads();
  int* out = ws + (size_t)blockIdx.x * SORT_WAVES * E;
  for (int j = t; j < SORT_WAVES * E; j += SORT_THREADS) out[j] = lds[j];
}

// Launch 2: every workgroup sums the histograms of all virtual wavefronts before its own
// (and of all of them, for the totals), scans, and assigns its pieces.
template <typename W>
__global__ void __launch_bounds__(SORT_THREADS)
sort_assign_kernel(const int* __restrict__ idx, const W* __restrict__ w, int M, int k, int E, int nbits, int piece,
                   const int* __restrict__ ws, int nvirtual, int* __restrict__ counts, int* __restrict__ offsets,
                   int* __restrict__ token, W* __restrict__ wsorted, int* __restrict__ pos_of) {
  extern __shared__ int lds[];
  int* base = lds;                         // [SORT_WAVES][E]
  int* part_before = base + SORT_WAVES * E;  // [parts][E]
  int* part_total = part_before + SORT_THREADS;
  int* total = part_total + SORT_THREADS;  // [E]
  int* before = total + E;                 // [E]
  int* offs = before + E;                  // [E+1]
  int* tmp = offs + E + 1;                 // [SORT_WAVES]
  const int t = threadIdx.x, wv = t >> 6;
  const int v0 = blockIdx.x * SORT_WAVES;
  const long lo64 = (long)(v0 + wv) * piece;
  const int lo = (int)(lo64 < M ? lo64 : M), hi = min(lo + piece, M);

  // Everything this workgroup reads that does not depend on the scan is asked for first: its
  // own wavefronts' histograms, and (pieces of two groups) the keys and weights it will
  // scatter. The kernel is a chain of memory round trips around little work; this makes it one.
  const bool loaded = piece == 2 * WAVE;
  int keys[2] = {-1, -1};
  W weights[2] = {0, 0};
  if (loaded) {
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const int i = lo + g * WAVE + (t & 63);
      if (i < hi) {
        keys[g] = idx[i];
        weights[g] = w[i];
      }
    }
  }
  int own[SORT_WAVES];
  if (t < E) {
#pragma unroll
    for (int j = 0; j < SORT_WAVES; ++j) own[j] = v0 + j < nvirtual ? ws[(size_t)(v0 + j) * E + t] : 0;
  }

  // thread (part, e): sums ws[v][e] over v = part, part + parts, ...
  const int parts = SORT_THREADS / E;  // >= 1 because E <= 1024
  const int e = t % E, part = t / E;
  int sb = 0, st = 0;
  if (part < parts) {
    for (int v = part; v < nvirtual; v += parts) {
      const int c = ws[(size_t)v * E + e];
      st += c;
      if (v < v0) sb += c;
    }
    part_before[part * E + e] = sb;
    part_total[part * E + e] = st;
  }
  __syncthreads();
  if (t < E) {
    int b = 0, s = 0;
    for (int j = 0; j < parts; ++j) {
      b += part_before[j * E + t];
      s += part_total[j * E + t];
    }
    before[t] = b;
    total[t] = s;
    if (blockIdx.x == 0) counts[t] = s;
  }
  __syncthreads();
  scan_experts(total, E, offs, tmp);
  if (blockIdx.x == 0)
    for (int j = t; j <= E; j += SORT_THREADS) offsets[j] = offs[j];
  if (t < E) {
    int run = offs[t] + before[t];
#pragma unroll
    for (int j = 0; j < SORT_WAVES; ++j) {
      base[j * E + t] = run;
      run += own[j];
    }
  }
  __syncthreads();
  if (loaded) assign_loaded(keys, weights, lo, k, E, nbits, base + wv * E, token, wsorted, pos_of);
  else assign_piece(idx, w, lo, hi, k, E, nbits, base + wv * E, token, wsorted, pos_of);
}

int bits_for(int E) {
  int b = 0;
  while ((1 << b) < E) ++b;
  return b;
}

template <typename W>
int launch_sort(const int32_t* idx, const void* w, int M, int k, int E, int32_t* counts, int32_t* offsets,
                int32_t* token, void* wsorted, int32_t* pos_of, void* workspace, hipStream_t stream, bool counted = false) {
  const int nbits = bits_for(E);
  if (M <= SMALL_M) {
    const size_t lds = sizeof(int) * small_sort_lds_ints(E);
    sort_small_kernel<W><<<1, SORT_THREADS, lds, stream>>>(idx, (const W*)w, M, k, E, nbits, counts, offsets, token,
                                                           (W*)wsorted, pos_of);
    return sy_check_launch("sort_by_expert");
  }
  const int blocks = large_blocks(M), nvirtual = blocks * SORT_WAVES;
  const int piece = piece_for(M);
  if (!counted) {
    sort_count_kernel<<<blocks, SORT_THREADS, sizeof(int) * SORT_WAVES * E, stream>>>(idx, M, E, nbits, piece, (int*)workspace);
    if (int rc = sy_check_launch("sort_by_expert (count)")) return rc;
  }
  const size_t lds = sizeof(int) * ((size_t)SORT_WAVES * E + 2 * SORT_THREADS + 3 * E + 1 + SORT_WAVES);
  sort_assign_kernel<W><<<blocks, SORT_THREADS, lds, stream>>>(idx, (const W*)w, M, k, E, nbits, piece, (const int*)workspace,
                                                               nvirtual, counts, offsets, token, (W*)wsorted, pos_of);
  return sy_check_launch("sort_by_expert (assign)");
}

}  // namespace

// The second launch alone, for a caller whose own kernel has left the per-piece histograms in the
// workspace (the router + route launch of front.hip). Weights of 2 bytes; N*k above SMALL_M.
int sy_sort_assign_counted(const int32_t* idx, const void* w, int N, int k, int E, int32_t* counts, int32_t* offsets,
                           int32_t* token, void* wsorted, int32_t* pos_of, void* workspace, void* stream) {
  return launch_sort<uint16_t>(idx, w, N * k, k, E, counts, offsets, token, wsorted, pos_of, workspace, (hipStream_t)stream, true);
}

extern "C" SY_API size_t sy_sort_workspace_bytes(int N, int k, int E) {
  const long M = (long)N * k;
  if (N <= 0 || k <= 0 || E <= 0 || M <= SMALL_M) return 0;
  return sizeof(int) * (size_t)large_blocks(M) * SORT_WAVES * E;
}

extern "C" SY_API int sy_sort_by_expert(const int32_t* idx, const void* w, int w_bytes, int N, int k, int E, int32_t* counts,
                                 int32_t* offsets, int32_t* token, void* wsorted, int32_t* pos_of, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  SY_REQUIRE(N >= 0 && k >= 1, "sort_by_expert: N = %d, k = %d", N, k);
  SY_REQUIRE(E >= 1 && E <= MAX_E, "sort_by_expert: 1 <= E <= %d (got %d)", MAX_E, E);
  SY_REQUIRE(w_bytes == 2 || w_bytes == 4, "sort_by_expert: weights of 2 or 4 bytes (got %d)", w_bytes);
  SY_REQUIRE((long)N * k < (1l << 31) - SORT_THREADS * PIECE, "sort_by_expert: N*k too large");
  SY_REQUIRE(counts && offsets, "sort_by_expert: null counts/offsets");
  const int M = N * k;
  SY_REQUIRE(M == 0 || (idx && w && token && wsorted && pos_of), "sort_by_expert: null pointer");
  const size_t need = sy_sort_workspace_bytes(N, k, E);
  SY_REQUIRE(need == 0 || (workspace && workspace_bytes >= need),
             "sort_by_expert: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  if (w_bytes == 2)
    return launch_sort<uint16_t>(idx, w, M, k, E, counts, offsets, token, wsorted, pos_of, workspace,
                                 (hipStream_t)stream);
  return launch_sort<uint32_t>(idx, w, M, k, E, counts, offsets, token, wsorted, pos_of, workspace,
                               (hipStream_t)stream);
}

// The same sort with the histograms in the library's own static device array instead of a
// workspace argument. The first launch overwrites every word of the array that the second one
// reads, so nothing has to be cleared between calls.
extern "C" SY_API int sy_sort_by_expert_static(const int32_t* idx, const void* w, int w_bytes, int N, int k, int E,
                                               int32_t* counts, int32_t* offsets, int32_t* token, void* wsorted,
                                               int32_t* pos_of, void* stream) {
  SY_REQUIRE(N >= 0 && k >= 1 && E >= 1, "sort_by_expert_static: N = %d, k = %d, E = %d", N, k, E);
  const size_t need = sy_sort_workspace_bytes(N, k, E);
  SY_REQUIRE(need <= (size_t)SY_SORT_STATIC_BYTES,
             "sort_by_expert_static: N*k = %ld choices over %d experts need %zu bytes of histograms, the static "
             "array holds %d; use sy_sort_by_expert with a workspace",
             (long)N * k, E, need, SY_SORT_STATIC_BYTES);
  void* ws = nullptr;
  if (need)
    if (int rc = static_scratch(&ws)) return rc;
  return sy_sort_by_expert(idx, w, w_bytes, N, k, E, counts, offsets, token, wsorted, pos_of, ws, need, stream);
}
