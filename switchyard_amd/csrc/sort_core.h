// Device pieces of the stable counting sort by expert (see sort.hip for the algorithm).
#pragma once

#include "common.h"

namespace sort_core {

constexpr int SORT_THREADS = 1024;
constexpr int SORT_WAVES = SORT_THREADS / WAVE;  // 16
constexpr int SMALL_M = 2048;                    // one workgroup sorts up to this many choices
constexpr int PIECE = 512;                       // choices per wavefront in the large path
constexpr int MAX_E = 512;                     // keeps every launch under 64 KB of LDS

// Choices per wavefront in the launches over many workgroups. A wavefront walks its piece 64
// choices at a time and every step is a chain of a load, ballots and scattered stores, so
// short pieces on many CUs finish sooner (32 768 choices: 23 us with pieces of 512 on 4 CUs);
// long inputs take longer pieces so that the table of histograms, which every workgroup of the
// second launch reads in full, stays small.
inline int piece_for(long M) { return M <= 65536 ? 128 : M <= 262144 ? 256 : PIECE; }

inline int large_blocks(long M) {
  const long per_block = (long)piece_for(M) * SORT_WAVES;
  return (int)((M + per_block - 1) / per_block);
}

// Lanes of this wavefront whose key equals mine (restricted to `valid` lanes).
__device__ __forceinline__ uint64_t match_lanes(int key, bool valid, int nbits) {
  uint64_t m = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (key >> b) & 1;
    const uint64_t bal = __ballot(bit);
    m &= bit ? bal : ~bal;
  }
  return m;
}

// Pass 1 for one wavefront: hist[e] += number of choices in [lo, hi) equal to e.
__device__ __forceinline__ void count_piece(const int* __restrict__ idx, int lo, int hi, int E, int nbits, int* hist) {
  const int lane = threadIdx.x & 63;
  for (int base = lo; base < hi; base += WAVE) {
    const int i = base + lane;
    int key = i < hi ? idx[i] : -1;
    const bool valid = (unsigned)key < (unsigned)E;  // ids outside [0, E) are ignored
    key = valid ? key : 0;
    const uint64_t m = match_lanes(key, valid, nbits);
    const int rank = __popcll(m & lanemask_lt()), cnt = __popcll(m);
    if (valid && rank == cnt - 1) hist[key] += cnt;  // one lane per expert
  }
}

// Pass 2 for one wavefront: base[e] is the row of this wavefront's first choice of expert e.
template <typename W>
__device__ __forceinline__ void assign_piece(const int* __restrict__ idx, const W* __restrict__ w, int lo, int hi, int k,
                                             int E, int nbits, int* base, int* __restrict__ token, W* __restrict__ wsorted,
                                             int* __restrict__ pos_of) {
  const int lane = threadIdx.x & 63;
  for (int at = lo; at < hi; at += WAVE) {
    const int i = at + lane;
    int key = i < hi ? idx[i] : -1;
    const bool valid = (unsigned)key < (unsigned)E;
    key = valid ? key : 0;
    const uint64_t m = match_lanes(key, valid, nbits);
    const int rank = __popcll(m & lanemask_lt()), cnt = __popcll(m);
    int row = 0;
    if (valid) row = base[key] + rank;
    // every lane has read base[] before the one writer per expert updates it
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      token[row] = i / k;
      wsorted[row] = w[i];
      pos_of[i] = row;
      if (rank == cnt - 1) base[key] += cnt;
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// Exclusive scan over experts of total[0..E) into offs[0..E], E <= 1024, by the whole
// workgroup (SORT_THREADS threads). tmp holds SORT_WAVES ints.
__device__ __forceinline__ void scan_experts(const int* total, int E, int* offs, int* tmp) {
  const int t = threadIdx.x, lane = t & 63, wv = t >> 6;
  const int v = t < E ? total[t] : 0;
  int inc = v;
  for (int o = 1; o < WAVE; o <<= 1) {
    const int up = __shfl_up(inc, o, WAVE);
    if (lane >= o) inc += up;
  }
  if (lane == WAVE - 1) tmp[wv] = inc;
  __syncthreads();
  int before = 0;
  for (int j = 0; j < wv; ++j) before += tmp[j];
  if (t < E) offs[t] = before + inc - v;
  if (t == E - 1) offs[E] = before + inc;
  __syncthreads();
}

// The whole sort by one workgroup of SORT_THREADS threads (up to SMALL_M choices); `lds` holds
// small_sort_lds_ints(E) ints. idx and w may live in global memory or in LDS.
__host__ __device__ constexpr size_t small_sort_lds_ints(int E) { return (size_t)SORT_WAVES * E + 2 * E + 1 + SORT_WAVES; }

// The same for a piece of two groups of 64 whose keys and weights the caller has already loaded
// (key -1 where the piece has no choice): the loads were issued before the histograms were
// summed, so nothing here waits for memory before it scatters.
template <typename W>
__device__ __forceinline__ void assign_loaded(const int (&keys)[2], const W (&weights)[2], int lo, int k, int E, int nbits,
                                              int* base, int* __restrict__ token, W* __restrict__ wsorted,
                                              int* __restrict__ pos_of) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const int i = lo + g * WAVE + lane;
    int key = keys[g];
    const bool valid = (unsigned)key < (unsigned)E;
    key = valid ? key : 0;
    const uint64_t m = match_lanes(key, valid, nbits);
    const int rank = __popcll(m & lanemask_lt()), cnt = __popcll(m);
    int row = 0;
    if (valid) row = base[key] + rank;
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      token[row] = i / k;
      wsorted[row] = weights[g];
      pos_of[i] = row;
      if (rank == cnt - 1) base[key] += cnt;
    }
    __builtin_amdgcn_wave_barrier();
  }
}

template <typename W>
__device__ __forceinline__ void sort_small_block(const int* idx, const W* w, int M, int k, int E, int nbits,
                                                 int* __restrict__ counts, int* __restrict__ offsets,
                                                 int* __restrict__ token, W* __restrict__ wsorted,
                                                 int* __restrict__ pos_of, int* lds) {
  int* hist = lds;                     // [SORT_WAVES][E]
  int* total = hist + SORT_WAVES * E;  // [E]
  int* offs = total + E;               // [E+1]
  int* tmp = offs + E + 1;             // [SORT_WAVES]
  const int t = threadIdx.x, wv = t >> 6;
  for (int j = t; j < SORT_WAVES * E; j += SORT_THREADS) hist[j] = 0;
  __syncthreads();

  const int piece = ((M + SORT_WAVES - 1) / SORT_WAVES + WAVE - 1) / WAVE * WAVE;
  const int lo = min(wv * piece, M), hi = min(lo + piece, M);
  count_piece(idx, lo, hi, E, nbits, hist + wv * E);
  __syncthreads();

  if (t < E) {
    int run = 0;
    for (int j = 0; j < SORT_WAVES; ++j) {
      const int c = hist[j * E + t];
      hist[j * E + t] = run;
      run += c;
    }
    total[t] = run;
    counts[t] = run;
  }
  __syncthreads();
  scan_experts(total, E, offs, tmp);
  for (int j = t; j <= E; j += SORT_THREADS) offsets[j] = offs[j];
  for (int j = t; j < SORT_WAVES * E; j += SORT_THREADS) hist[j] += offs[j % E];
  __syncthreads();

  assign_piece(idx, w, lo, hi, k, E, nbits, hist + wv * E, token, wsorted, pos_of);
}

// The whole sort by one wavefront when there are at most 64 choices (a decode step of 8 tokens):
// one choice per lane, no workgroup barrier. `lds` holds 2 * E + 1 ints; E <= 128.
template <typename W>
__device__ __forceinline__ void sort_one_wave(const int* idx, const W* w, int M, int k, int E, int nbits,
                                              int* __restrict__ counts, int* __restrict__ offsets,
                                              int* __restrict__ token, W* __restrict__ wsorted,
                                              int* __restrict__ pos_of, int* lds) {
  int* total = lds;      // [E]
  int* offs = lds + E;   // [E + 1]
  const int lane = threadIdx.x & 63;
  for (int x = lane; x < E; x += WAVE) total[x] = 0;
  int key = lane < M ? idx[lane] : -1;
  const bool valid = (unsigned)key < (unsigned)E;
  key = valid ? key : 0;
  const uint64_t m = match_lanes(key, valid, nbits);
  const int rank = __popcll(m & lanemask_lt()), cnt = __popcll(m);
  __builtin_amdgcn_wave_barrier();
  if (valid && rank == cnt - 1) total[key] = cnt;  // one lane per expert
  __builtin_amdgcn_wave_barrier();
  int run = 0;
  for (int x0 = 0; x0 < E; x0 += WAVE) {
    const int x = x0 + lane;
    const int c = x < E ? total[x] : 0;
    int inc = c;
    for (int o = 1; o < WAVE; o <<= 1) {
      const int up = __shfl_up(inc, o, WAVE);
      if (lane >= o) inc += up;
    }
    if (x < E) {
      counts[x] = c;
      offsets[x] = run + inc - c;
      offs[x] = run + inc - c;
    }
    run += __shfl(inc, WAVE - 1, WAVE);
  }
  if (lane == 0) offsets[E] = run;
  __builtin_amdgcn_wave_barrier();
  if (valid) {
    const int row = offs[key] + rank;
    token[row] = lane / k;
    wsorted[row] = w[lane];
    pos_of[lane] = row;
  }
}

}  // namespace sort_core
