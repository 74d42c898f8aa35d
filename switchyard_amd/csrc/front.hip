// The front of the layer in fewer launches. Two entry points:
//   sy_route_sort    a decode step's route and sort in one launch (below);
//   sy_router_route  for more tokens, the router GEMM and route in one launch, which inside
//                    sy_moe_experts is also the first pass of the sort (further down).
// (The decode step's router GEMM, route and sort in one launch, sy_router_route_sort, is the
// row kernel of decode.hip with front_core.h's tail: one workgroup per token, not one in all.)
//
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


// ---------------------------------------------------------------------------------------------
// router_route: the router's logits, route and, when asked, the first pass of the sort, in one
// launch, for more tokens than the decode path's kernels are for.
//
// At hundreds to thousands of tokens the library's GEMM for [N, H] x [E, H]^T (64 output
// columns) takes about 14 us, the route launch 6 and the sort's counting launch 5, in front of
// two projections; each is a launch's latency around very little work. Here a workgroup takes
// 16 tokens: its wavefronts (16, or 4 where H is not a multiple of 2048 or there are more than
// 64 experts) each multiply their share of H on v_mfma_f32_16x16x32_f16 (the tokens as the 16
// rows, 16 experts per block as the columns, operands straight from memory: 16 bytes per lane,
// 64 contiguous bytes of a row per instruction), the partial sums meet in LDS and are added in
// a fixed order, rounded to f16 once (the logits, also written out), and the wavefronts then
// route a token each from LDS with the code of route.hip. Everything here is latency, so the
// workgroup is as wide as the shape allows: 21 us with 4 wavefronts at 4096 tokens. With `hist` the
// workgroup is one piece of the sort (sort.hip): it owns piece / k tokens, 16 at a time, and
// leaves the histogram of its choices where the sort's second launch expects it.
//
// Fuses F.linear(h, router) + route() of the reference (switchyard/kernels.py:30-32,
// switchyard/csrc/moe_kernels.cu:23-89) and count_kernel (:91-104).
constexpr int RR_TOKENS = 16, RR_KSTEP = 32;

typedef float float4v_t __attribute__((ext_vector_type(4)));

template <int PER_LANE, int RR_WAVES>
__global__ void __launch_bounds__(RR_WAVES * WAVE)
router_route_kernel(const half_t* __restrict__ h, const half_t* __restrict__ router, int N, int H, int E, int k, int norm,
                    int nbits, int groups, half_t* __restrict__ logits, int* __restrict__ idx, half_t* __restrict__ w,
                    int* __restrict__ hist_out) {
  constexpr int EB = 4 * PER_LANE;             // blocks of 16 experts
  constexpr int RR_THREADS = RR_WAVES * WAVE;
  constexpr int EP = 16 * EB;                  // experts, padded
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  float* part = reinterpret_cast<float*>(lds_raw);                      // [RR_WAVES][RR_TOKENS][EP]
  half_t* lg = reinterpret_cast<half_t*>(part + RR_WAVES * RR_TOKENS * EP);  // [RR_TOKENS][EP]
  int* sidx = reinterpret_cast<int*>(lg + RR_TOKENS * EP);              // [groups * RR_TOKENS * k]
  int* hist = sidx + groups * RR_TOKENS * k;                           // [E]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int row = lane & 15, kq = (lane >> 4) * 8;   // the operand row of this lane and its 8 halves of a K step
  const int kwave = H / RR_WAVES, steps = kwave / RR_KSTEP;   // a multiple of 4 steps per wavefront
  const __amdgpu_buffer_rsrc_t hrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(h), 0, (int)((size_t)N * H * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(router), 0, (int)((size_t)E * H * 2), 0x00020000);

  for (int g = 0; g < groups; ++g) {
    const int t0 = (blockIdx.x * groups + g) * RR_TOKENS;
    if (t0 < N) {
      // ---- this wavefront's share of the dot products. Loads go through buffer descriptors: a
      // token past N or an expert past E is out of range and reads as 0
      const unsigned aoff = ((unsigned)(t0 + row) * (unsigned)H + (unsigned)(wave * kwave + kq)) * 2u;
      const unsigned boff = ((unsigned)row * (unsigned)H + (unsigned)(wave * kwave + kq)) * 2u;
      float4v_t acc[EB];
#pragma unroll
      for (int b = 0; b < EB; ++b) acc[b] = float4v_t{0.f, 0.f, 0.f, 0.f};
      half8_t a0[2], a1[2], b0[2][EB], b1[2][EB];
      auto load = [&](half8_t (&a)[2], half8_t (&bb)[2][EB], int s) {
        // two steps are the two halves of a 128-byte line of each row: asked for one after the other
#pragma unroll
        for (int u = 0; u < 2; ++u)
          a[u] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(hrsrc, aoff, (s + u) * RR_KSTEP * 2, 0));
#pragma unroll
        for (int b = 0; b < EB; ++b)
#pragma unroll
          for (int u = 0; u < 2; ++u)
            bb[u][b] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rrsrc, boff + (unsigned)(16 * b) * (unsigned)H * 2u,
                                                                                        (s + u) * RR_KSTEP * 2, 0));
      };
      auto multiply = [&](const half8_t (&a)[2], const half8_t (&bb)[2][EB]) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int b = 0; b < EB; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u], bb[u][b], acc[b], 0, 0, 0);
      };
      load(a0, b0, 0);
      for (int s = 0; s < steps; s += 4) {
        load(a1, b1, s + 2);
        multiply(a0, b0);
        if (s + 4 < steps) load(a0, b0, s + 4);
        multiply(a1, b1);
      }
      // lane holds tokens 4 * (lane / 16) + r, expert 16 b + lane % 16
#pragma unroll
      for (int b = 0; b < EB; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) part[(wave * RR_TOKENS + 4 * (lane >> 4) + r) * EP + 16 * b + row] = acc[b][r];
    }
    __syncthreads();
    if (t0 < N) {
      for (int o = tid; o < RR_TOKENS * EP; o += RR_THREADS) {
        const int tok = o / EP, e = o - tok * EP;
        float v = part[o];
#pragma unroll
        for (int q = 1; q < RR_WAVES; ++q) v += part[q * RR_TOKENS * EP + o];
        const half_t hv = (half_t)v;
        lg[o] = hv;
        if (t0 + tok < N && e < E) logits[(size_t)(t0 + tok) * E + e] = hv;
      }
    }
    __syncthreads();
    // ---- route: one wavefront per token
    for (int tok = wave; tok < RR_TOKENS; tok += RR_WAVES) {
      const int t = t0 + tok;
      int my_e = -1;
      if (t < N) {
        float my_w;
        route_core::route_token<half_t, PER_LANE>(lg + tok * EP, E, k, norm, my_e, my_w);
        if (lane < k) {
          idx[(size_t)t * k + lane] = my_e;
          w[(size_t)t * k + lane] = (half_t)my_w;
        }
      }
      if (lane < k) sidx[(g * RR_TOKENS + tok) * k + lane] = my_e;
    }
  }
  if (!hist_out) return;
  __syncthreads();
  // ---- the workgroup's choices are one piece of the sort: their histogram
  if (wave == 0) {
    for (int e = lane; e < E; e += WAVE) hist[e] = 0;
    count_piece(sidx, 0, groups * RR_TOKENS * k, E, nbits, hist);
    for (int e = lane; e < E; e += WAVE) hist_out[(size_t)blockIdx.x * E + e] = hist[e];
  }
}

// ---------------------------------------------------------------------------------------------
// The same launch with the operands staged through LDS, for up to 64 experts. What the kernel
// above waits for is its compute unit's L1: every workgroup pulls the whole router through it, and
// an MFMA operand load takes a 64-byte piece of each of 16 rows, which costs the L1 what a whole
// line costs. Here the router's rows and the workgroup's 16 token rows come in K slices of 64
// (128 bytes of a row: whole lines, 8 rows per instruction) by buffer loads that write LDS
// directly, fourteen slices deep, so 130 KB of loads are in flight while one slice is multiplied
// (with eight slices the loop waited for data in every iteration: 11.0 us a launch against 9);
// a slice's 16-byte chunks are XOR-swizzled by row so that the operand reads spread over the
// banks. Ten wavefronts issue one load per slice each (eight the router's rows, two the
// tokens'), eight multiply (expert block x half of the slice's K), all sixteen route. The waits
// for the loads are counted by hand: the compiler is not told about them.
constexpr int RS_WAVES = 16, RS_THREADS = RS_WAVES * WAVE, RS_DEPTH = 14;   // 140 of the 160 KB of LDS are slices
constexpr int RS_ROWS = 64 + RR_TOKENS, RS_STAGE = RS_ROWS * 128, RS_LOADS = RS_ROWS / 8;
constexpr int RS_BK = 64;

typedef int int4v_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int4v_t raw_descriptor(const void* base, unsigned bytes) {
  const uint64_t a = (uint64_t)base;
  int4v_t d;
  d[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)a);
  d[1] = __builtin_amdgcn_readfirstlane((int)((unsigned)(a >> 32) & 0xffffu));
  d[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  d[3] = 0x00020000;
  return d;
}

// 16 bytes per lane from buffer offset voffset + soffset to LDS address lds_addr + 16 * lane;
// only voffset is checked against the size of the buffer. The LDS address travels in m0.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void buffer_to_lds(int4v_t rsrc, unsigned voffset, unsigned soffset, unsigned lds_addr) {
#pragma unroll
  for (int c = 0; c < 4; ++c) rsrc[c] = __builtin_amdgcn_readfirstlane(rsrc[c]);
  soffset = __builtin_amdgcn_readfirstlane(soffset);
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
      : "memory", "m0");
}
#pragma clang diagnostic pop

__global__ void __launch_bounds__(RS_THREADS)
router_route_staged_kernel(const half_t* __restrict__ h, const half_t* __restrict__ router, int N, int H, int E, int k,
                           int norm, int nbits, int groups, half_t* __restrict__ logits, int* __restrict__ idx,
                           half_t* __restrict__ w, int* __restrict__ hist_out) {
  constexpr int EP = 64;
  constexpr unsigned OUT_OF_RANGE = 0x80000000u;
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  float* part = reinterpret_cast<float*>(lds_raw + RS_DEPTH * RS_STAGE);   // [2][RR_TOKENS][EP]
  half_t* lg = reinterpret_cast<half_t*>(part + 2 * RR_TOKENS * EP);      // [RR_TOKENS][EP]
  int* sidx = reinterpret_cast<int*>(lg + RR_TOKENS * EP);                // [groups * RR_TOKENS * k]
  int* hist = sidx + groups * RR_TOKENS * k;                             // [E]
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int nk = H / RS_BK;
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds_raw;
  const int4v_t rrsrc = raw_descriptor(router, (unsigned)((size_t)E * H * 2));
  const int4v_t hrsrc = raw_descriptor(h, (unsigned)((size_t)N * H * 2));
  const bool loads = wave < RS_LOADS, multiplies = wave < 8;
  // a multiplying wavefront: expert block and which half of a slice's K
  const int block = wave & 3, khalf = (wave >> 2) & 1;
  const int orow = lane & 15, ochunk = 4 * khalf + (lane >> 4);
  const int arow = 64 + orow, brow = 16 * block + orow;
  const unsigned aread = arow * 128 + ((ochunk ^ ((arow >> 1) & 7)) * 16), bread = brow * 128 + ((ochunk ^ ((brow >> 1) & 7)) * 16);

  for (int g = 0; g < groups; ++g) {
    const int t0 = (blockIdx.x * groups + g) * RR_TOKENS;
    if (t0 < N) {
      // the row of the stage that this lane fetches a chunk of (rows 0..63 the router's, 64..79 the tokens')
      const int srow = 8 * wave + (lane >> 3);
      const unsigned chunk = (unsigned)((lane & 7) ^ ((srow >> 1) & 7));
      unsigned voff = OUT_OF_RANGE;
      if (wave < 8) {
        if (srow < E) voff = ((unsigned)srow * (unsigned)H + chunk * 8u) * 2u;
      } else if (loads) {
        const int t = t0 + srow - 64;
        if (t < N) voff = ((unsigned)t * (unsigned)H + chunk * 8u) * 2u;
      }
      // slices past the end are asked for too, out of range: they keep the count of loads in flight
      // the same in every iteration and bring nothing
      auto issue = [&](int s, int stage) {
        if (loads)
          buffer_to_lds(wave < 8 ? rrsrc : hrsrc, s < nk ? voff : OUT_OF_RANGE, (unsigned)s * (RS_BK * 2),
                        lds_base + (unsigned)stage * RS_STAGE + (unsigned)wave * 1024u);
      };
      for (int s = 0; s < RS_DEPTH - 2; ++s) issue(s, s);
      float4v_t acc = {0.f, 0.f, 0.f, 0.f};
      int at = 0, fill = RS_DEPTH - 2;   // the buffer of slice s, and the one the next load fills
      // two slices to a barrier (the number of slices is even: H is a multiple of 512)
      for (int s = 0; s < nk; s += 2) {
        // this wavefront's loads of slices s and s + 1 have landed when only the RS_DEPTH - 4 after them are in flight
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RS_DEPTH - 4) : "memory");
        __syncthreads();   // everybody's have; and everybody has read slices s - 2 and s - 1, whose buffers the next loads fill
        const int at1 = at + 1, fill1 = fill + 1 == RS_DEPTH ? 0 : fill + 1;
        issue(s + RS_DEPTH - 2, fill);
        issue(s + RS_DEPTH - 1, fill1);
        if (multiplies) {
          const char* stage = lds_raw + at * RS_STAGE;
          const half8_t a0 = *reinterpret_cast<const half8_t*>(stage + aread);
          const half8_t b0 = *reinterpret_cast<const half8_t*>(stage + bread);
          const half8_t a1 = *reinterpret_cast<const half8_t*>(stage + RS_STAGE + aread);
          const half8_t b1 = *reinterpret_cast<const half8_t*>(stage + RS_STAGE + bread);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, acc, 0, 0, 0);
        }
        fill = at;   // slices s and s + 1 sit in buffers at, at + 1 (RS_DEPTH is even: pairs never wrap inside)
        at = at1 + 1 == RS_DEPTH ? 0 : at1 + 1;
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      // lane holds tokens 4 * (lane / 16) + r, expert 16 * block + lane % 16, for its half of every slice
      if (multiplies) {
#pragma unroll
        for (int r = 0; r < 4; ++r) part[(khalf * RR_TOKENS + 4 * (lane >> 4) + r) * EP + 16 * block + orow] = acc[r];
      }
    }
    __syncthreads();
    if (t0 < N) {
      const int o = tid, tok = o / EP, e = o - tok * EP;   // RS_THREADS == RR_TOKENS * EP
      const half_t hv = (half_t)(part[o] + part[RR_TOKENS * EP + o]);
      lg[o] = hv;
      if (t0 + tok < N && e < E) logits[(size_t)(t0 + tok) * E + e] = hv;
    }
    __syncthreads();
    // ---- route: one wavefront per token
    {
      const int tok = wave, t = t0 + tok;
      int my_e = -1;
      if (t < N) {
        float my_w;
        route_core::route_token<half_t, 1>(lg + tok * EP, E, k, norm, my_e, my_w);
        if (lane < k) {
          idx[(size_t)t * k + lane] = my_e;
          w[(size_t)t * k + lane] = (half_t)my_w;
        }
      }
      if (lane < k) sidx[(g * RR_TOKENS + tok) * k + lane] = my_e;
    }
  }
  if (!hist_out) return;
  __syncthreads();
  if (wave == 0) {
    for (int e = lane; e < E; e += WAVE) hist[e] = 0;
    count_piece(sidx, 0, groups * RR_TOKENS * k, E, nbits, hist);
    for (int e = lane; e < E; e += WAVE) hist_out[(size_t)blockIdx.x * E + e] = hist[e];
  }
}
static_assert(RS_THREADS == RR_TOKENS * 64, "one thread per logit of the workgroup");
static_assert(RS_WAVES == RR_TOKENS, "one wavefront per token routes");
static_assert(RS_DEPTH % 2 == 0, "pairs of slices never wrap inside the ring");

bool router_route_shape_ok(int N, int H, int E, int k) {
  return N >= 1 && H >= 512 && H % 512 == 0 && E >= 1 && E <= 128 && k >= 1 && k <= FRONT_MAX_K && k <= E &&
         (long)N * H * 2 < (1l << 31);
}

int launch_router_route(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits,
                        int32_t* idx, void* w, void* hist, hipStream_t st) {
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const long M = (long)N * k;
  int groups = 1, grid = (N + RR_TOKENS - 1) / RR_TOKENS;
  if (hist) {   // one workgroup per piece of the sort, and as many pieces as its second launch reads
    groups = piece_for(M) / (RR_TOKENS * k);
    grid = large_blocks(M) * SORT_WAVES;
  }
  if (E <= 64 && H / RS_BK >= RS_DEPTH) {   // staged through LDS (H is a multiple of 512: at least 1024 here)
    const size_t lds = (size_t)RS_DEPTH * RS_STAGE + sizeof(float) * 2 * RR_TOKENS * 64 + sizeof(half_t) * RR_TOKENS * 64 +
                       sizeof(int) * ((size_t)groups * RR_TOKENS * k + E);
    if (hipFuncSetAttribute((const void*)router_route_staged_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return sy_fail(SY_ERR_LAUNCH, "router_route: cannot reserve %zu bytes of LDS", lds);
    router_route_staged_kernel<<<grid, RS_THREADS, lds, st>>>((const half_t*)h, (const half_t*)router, N, H, E, k, norm, nbits,
                                                             groups, (half_t*)logits, idx, (half_t*)w, (int*)hist);
    return sy_check_launch("router_route");
  }
  const int EP = E <= 64 ? 64 : 128;
  const bool wide = E <= 64 && H % 2048 == 0;   // 16 wavefronts: four K steps each at H = 2048
  const int waves = wide ? 16 : 4;
  const size_t lds = sizeof(float) * waves * RR_TOKENS * EP + sizeof(half_t) * RR_TOKENS * EP +
                     sizeof(int) * ((size_t)groups * RR_TOKENS * k + E);
  void (*kern)(const half_t*, const half_t*, int, int, int, int, int, int, int, half_t*, int*, half_t*, int*) =
      wide ? router_route_kernel<1, 16> : E <= 64 ? router_route_kernel<1, 4> : router_route_kernel<2, 4>;
  if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return sy_fail(SY_ERR_LAUNCH, "router_route: cannot reserve %zu bytes of LDS", lds);
  kern<<<grid, waves * WAVE, lds, st>>>((const half_t*)h, (const half_t*)router, N, H, E, k, norm, nbits, groups,
                                        (half_t*)logits, idx, (half_t*)w, (int*)hist);
  return sy_check_launch("router_route");
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

// Whether the router + route launch can also be the sort's first pass: the sort runs over many
// workgroups (above the one-workgroup limit) and a piece is whole groups of 16 tokens.
bool sy_router_route_shape_ok(int N, int H, int E, int k) { return router_route_shape_ok(N, H, E, k); }

bool sy_router_route_counts(int N, int k) {
  const long M = (long)N * k;
  return M > SMALL_M && piece_for(M) % (RR_TOKENS * k) == 0;
}

int sy_router_route_counting(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits,
                             int32_t* idx, void* w, void* hist, void* stream) {
  SY_REQUIRE(router_route_shape_ok(N, H, E, k),
             "router_route: H a multiple of 512, at most 128 experts and top-8 (got N = %d, H = %d, E = %d, k = %d)", N, H, E, k);
  SY_REQUIRE(h && router && logits && idx && w, "router_route: null pointer");
  SY_REQUIRE(!hist || sy_router_route_counts(N, k), "router_route: no histograms for N = %d, k = %d", N, k);
  return launch_router_route(h, router, N, H, E, k, norm, logits, idx, w, hist, (hipStream_t)stream);
}

extern "C" SY_API int sy_router_route(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits,
                                      int32_t* idx, void* w, void* stream) {
  if (N == 0) return SY_OK;
  // a decode step: one workgroup per row (the kernels above take 16 rows to a workgroup)
  if (N <= 64) return sy_router_route_rows(h, router, N, H, E, k, norm, logits, idx, w, stream);
  return sy_router_route_counting(h, router, N, H, E, k, norm, logits, idx, w, nullptr, stream);
}
