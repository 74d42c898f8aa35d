// The attention side of one decode step, for the caller of the MoE hook: what sits between two
// MoE layers when every sequence of the batch advances by one token. In the reference this is
// a few dozen PyTorch launches per layer (switchyard/model.py:14-17 rmsnorm, :61-84
// _attention, :117-121 attention_block); at decode each of them is a launch that moves a few
// kilobytes, so the step is bound by launches, not by the 34 MB of attention weights and the
// KV cache it has to read. A few kernels replace them (the projections themselves go through
// the weight-stream kernel with a single "expert"):
//
//   row_kernel            one token per workgroup: x += delta; h = w * f16(x * rsqrt(mean(x^2) + eps)).
//                         x may be an embedding lookup (embed_rmsnorm), delta may be the combine
//                         of the MoE layer's rows (combine_add_rmsnorm, which also applies
//                         the router weights to rows that were left unscaled), and the router's
//                         logits of h may come out of the same launch (add_rmsnorm_logits); with
//                         them route and the sort as well (add_rmsnorm_route_sort, and
//                         router_route_sort for rows that need no norm: front_core.h), the whole
//                         front of the MoE layer in the launch that the step needs anyway
//   qk_norm_rope_cache    q/k RMS norm over the whole projection, clamp, rotary embedding, and
//                         the new keys and values written into the cache from `slot` on (one
//                         token per sequence at decode, the whole prompt at prefill)
//   decode_attention      one query per (sequence, head) against the cache: a single pass over
//                         the keys and values with a running softmax, HBM-bound; its _qkv form
//                         does the work of qk_norm_rope_cache in its own prologue
//   greedy_advance        arg-max of the logits, the token appended to the output, rotary
//                         positions and cache slot advanced
//
// Everything a replayed HIP graph must not bake in (the cache slot, the rotary positions, the
// output column) is read from device memory, so the same launches serve every step.
//
// Rounding follows the PyTorch graph on fp16 tensors where it is cheap to do so: the norm is
// taken in fp32, rounded to fp16 and then scaled in fp16; rotary products and their sum are
// each rounded to fp16. Attention scores and the softmax stay in fp32 (the reference rounds
// the scores to fp16 first), which is the more exact of the two.
#include <mutex>

#include "common.h"
#include "front_core.h"
#include "../../include/switchyard_decode.h"

namespace {

constexpr int ROW_THREADS = 256;
constexpr int MAX_CHUNKS = 4;  // 8-half chunks per thread: rows of up to 8192 halves

__device__ __forceinline__ float block_sum(float v, float* lds, int slot_base) {
  // sum over the wavefronts of the workgroup (at most 16); every thread gets the total
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  if ((threadIdx.x & 63) == 0) lds[slot_base + wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += lds[slot_base + w];
  return total;
}

constexpr int ROW_MAX_K = 64;  // choices per token the combining variant ranks in one wavefront

// One workgroup per token (row). The residual `delta` is either a tensor, or (COMBINE) the
// token's k expert outputs summed in fp32 in ascending expert id and rounded to f16 once,
// exactly as the combine kernel leaves it (`delta` then holds the router weights [N, k] of rows
// that the down projection left unscaled, or is null); then x_out = f16(x + delta) and h = the RMS norm
// of x_out. With LOGITS the normalised row stays in LDS and the four wavefronts also take its
// dot products with the E rows of the router (fp32 sums, one rounding to f16), so that the
// router needs no launch of its own; that variant runs 16 wavefronts, each with the loads of
// four experts in flight at once, because the router's rows come from L2 one round trip at a
// time and the trips, not the bytes, are what it waits for.
// With FRONT (and LOGITS) the workgroup then routes its token from the logits in LDS; with FRONT
// == FRONT_SORT the last workgroup of the launch to get there also sorts every token's choices
// (front_core.h): the layer's router GEMM, route and sort in one launch.
constexpr int FRONT_ROUTE = 1, FRONT_SORT = 2;
template <bool COMBINE, bool LOGITS, int FRONT = 0>
__global__ void __launch_bounds__(LOGITS ? 1024 : ROW_THREADS)
row_kernel(const half_t* x, const half_t* __restrict__ delta, const half_t* __restrict__ y,
           const int* __restrict__ pos_of, const int* __restrict__ idx, int k, const half_t* __restrict__ weight,
           float eps, const half_t* __restrict__ router, int E, int H, half_t* x_out, half_t* __restrict__ h_out,
           half_t* __restrict__ logits, const int64_t* __restrict__ gather, int src_rows,
           front_core::Outputs front = front_core::Outputs{}) {  // x_out may be x
  extern __shared__ __attribute__((aligned(16))) half_t hs[];  // LOGITS: the normalised row [H]; FRONT: the tail's LDS behind it
  __shared__ float part[16];
  __shared__ int rows[ROW_MAX_K];
  __shared__ float wts[ROW_MAX_K];   // COMBINE: the router weight of each row, 1 where y is already scaled
  const int t = blockIdx.x, tid = threadIdx.x, nthreads = blockDim.x;
  const size_t row = (size_t)t * H;
  const int chunks = H >> 3;
  // the input row: row t of x, or (an embedding lookup) the row of x that gather[t] names
  const half_t* xrow = x + row;
  if (gather) {
    long g = (long)gather[t];
    g = g < 0 ? 0 : g >= src_rows ? src_rows - 1 : g;
    xrow = x + (size_t)g * H;
  }
  if (COMBINE) {
    // rank the k choices by (expert id, slot); rows[] lists their rows of y in that order
    if (tid < WAVE) {
      const int mine = tid < k ? idx[(size_t)t * k + tid] : 0x7fffffff;
      const int src = tid < k ? pos_of[(size_t)t * k + tid] : 0;
      int rank = 0;
      for (int j = 0; j < k; ++j) {
        const int other = read_lane(mine, j);
        rank += (other < mine) || (other == mine && j < tid);
      }
      if (tid < k) {
        rows[rank] = src;
        wts[rank] = delta ? (float)delta[(size_t)t * k + tid] : 1.f;
      }
    }
    __syncthreads();
  }
  half8_t v[MAX_CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAX_CHUNKS; ++i) {
    const int c = tid + i * nthreads;
    if (c < chunks) {
      v[i] = *reinterpret_cast<const half8_t*>(xrow + c * 8);
      if (COMBINE) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < k; ++j) {
          const half8_t e = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(y + (size_t)rows[j] * H + c * 8));   // read once
          const float wt = wts[j];
          // the rounding of the down projection's scaled epilogue (times 1 it changes nothing)
#pragma unroll
          for (int q = 0; q < 8; ++q) acc[q] += (float)(half_t)((float)e[q] * wt);
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) v[i][q] = (half_t)((float)v[i][q] + (float)(half_t)acc[q]);
      } else if (delta) {
        const half8_t d = *reinterpret_cast<const half8_t*>(delta + row + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = (half_t)((float)v[i][j] + (float)d[j]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (float)v[i][j] * (float)v[i][j];
    }
  }
  if (LOGITS && !weight) {
    // no norm asked for: the logits of the rows as they are (the router GEMM alone)
#pragma unroll
    for (int i = 0; i < MAX_CHUNKS; ++i) {
      const int c = tid + i * nthreads;
      if (c < chunks) *reinterpret_cast<half8_t*>(hs + c * 8) = v[i];
    }
  } else {
    const float rs = rsqrtf(block_sum(ss, part, 0) / (float)H + eps);
#pragma unroll
    for (int i = 0; i < MAX_CHUNKS; ++i) {
      const int c = tid + i * nthreads;
      if (c < chunks) {
        const half8_t w = *reinterpret_cast<const half8_t*>(weight + c * 8);
        half8_t h;
#pragma unroll
        for (int j = 0; j < 8; ++j) h[j] = (half_t)((float)w[j] * (float)(half_t)((float)v[i][j] * rs));
        if (x_out) *reinterpret_cast<half8_t*>(x_out + row + c * 8) = v[i];
        *reinterpret_cast<half8_t*>(h_out + row + c * 8) = h;
        if (LOGITS) *reinterpret_cast<half8_t*>(hs + c * 8) = h;
      }
    }
  }
  if (!LOGITS) return;
  __syncthreads();
  // wavefront w takes experts w, w + nwaves, ...: four at a time with every load issued before
  // the first is used (rows of 2048: 16 loads of 16 bytes per lane)
  const int wave = tid >> 6, lane = tid & 63, nwaves = nthreads >> 6;
  for (int e0 = wave; e0 < E; e0 += 4 * nwaves) {
    const half_t* r[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = e0 + nwaves * u;
      r[u] = router + (size_t)(e < E ? e : e0) * H;
    }
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (chunks == 4 * WAVE) {
      half8_t rv[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int u = 0; u < 4; ++u) rv[u][i] = *reinterpret_cast<const half8_t*>(r[u] + (lane + WAVE * i) * 8);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const half8_t hv = *reinterpret_cast<const half8_t*>(hs + (lane + WAVE * i) * 8);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[u] += (float)hv[j] * (float)rv[u][i][j];
      }
    } else {
      for (int c = lane; c < chunks; c += WAVE) {
        const half8_t hv = *reinterpret_cast<const half8_t*>(hs + c * 8);
        half8_t rv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) rv[u] = *reinterpret_cast<const half8_t*>(r[u] + c * 8);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[u] += (float)hv[j] * (float)rv[u][j];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float total = wave_sum(acc[u]);
      const int e = e0 + nwaves * u;
      if (lane == 0 && e < E) {
        logits[(size_t)t * E + e] = (half_t)total;
        if (FRONT) hs[H + e] = (half_t)total;
      }
    }
  }
  if (FRONT) {
    __syncthreads();
    unsigned char* tail = reinterpret_cast<unsigned char*>(hs + H);
    if (FRONT == FRONT_ROUTE) {
      if (E <= 64) front_core::route_own<1>(t, E, front, tail);
      else front_core::route_own<2>(t, E, front, tail);
    } else if (E <= 64) {
      front_core::route_own_sort_last<1>(t, (int)gridDim.x, E, front, tail);
    } else {
      front_core::route_own_sort_last<2>(t, (int)gridDim.x, E, front, tail);
    }
  }
}

__device__ __forceinline__ half_t clamp_f16(half_t v, float clip) {
  if (clip > 0.f) {
    const float f = (float)v;
    return (half_t)(f < -clip ? -clip : f > clip ? clip : f);
  }
  return v;
}

// out = f16(f16(y * cos) + f16(rot * sin)): three roundings, as three PyTorch operators on
// fp16 tensors make them. Contraction is switched off here, or the compiler narrows the
// arithmetic to fp16 and fuses product and sum into one fma with a single rounding.
__device__ __forceinline__ half_t rotary_f16(half_t y, half_t rot, half_t cos_v, half_t sin_v) {
#pragma clang fp contract(off)
  const half_t t1 = (half_t)((float)y * (float)cos_v);
  const half_t t2 = (half_t)((float)rot * (float)sin_v);
  return (half_t)((float)t1 + (float)t2);
}

// One workgroup per token. qkv row = [q (heads*D) | k (kv_heads*D) | v (kv_heads*D)].
__global__ void __launch_bounds__(ROW_THREADS)
qk_norm_rope_cache_kernel(const half_t* __restrict__ qkv, const half_t* __restrict__ q_norm,
                          const half_t* __restrict__ k_norm, float eps, float clip, const half_t* __restrict__ cos_t,
                          const half_t* __restrict__ sin_t, int max_positions, const int64_t* __restrict__ positions,
                          const int64_t* __restrict__ slot_ptr, int T, int heads, int kv_heads, int D, int capacity,
                          half_t* __restrict__ q_out, half_t* __restrict__ kcache, half_t* __restrict__ vcache) {
  extern __shared__ __attribute__((aligned(16))) half_t normed[];  // [qd + kvd] after norm and clamp
  __shared__ float part[32];
  // row r of qkv is token t = r % T of sequence b = r / T; it goes to cache position slot + t
  const int r = blockIdx.x, b = r / T;
  const int qd = heads * D, kvd = kv_heads * D;
  const half_t* row = qkv + (size_t)r * (qd + 2 * kvd);
  const int qchunks = qd >> 3, kchunks = kvd >> 3;
  const long slot = (long)*slot_ptr + (r - b * T);
  long pos = (long)positions[r];
  pos = pos < 0 ? 0 : pos >= max_positions ? max_positions - 1 : pos;
  const bool slot_ok = slot >= 0 && slot < capacity;

  half8_t q[MAX_CHUNKS], k[MAX_CHUNKS];
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int i = 0; i < MAX_CHUNKS; ++i) {
    const int c = threadIdx.x + i * ROW_THREADS;
    if (c < qchunks) {
      q[i] = *reinterpret_cast<const half8_t*>(row + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) sq += (float)q[i][j] * (float)q[i][j];
    }
    if (c < kchunks) {
      k[i] = *reinterpret_cast<const half8_t*>(row + qd + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) sk += (float)k[i][j] * (float)k[i][j];
    }
  }
  const float rq = rsqrtf(block_sum(sq, part, 0) / (float)qd + eps);
  const float rk = rsqrtf(block_sum(sk, part, 16) / (float)kvd + eps);
#pragma unroll
  for (int i = 0; i < MAX_CHUNKS; ++i) {
    const int c = threadIdx.x + i * ROW_THREADS;
    if (c < qchunks) {
      const half8_t w = *reinterpret_cast<const half8_t*>(q_norm + c * 8);
      half8_t o;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        o[j] = clamp_f16((half_t)((float)w[j] * (float)(half_t)((float)q[i][j] * rq)), clip);
      *reinterpret_cast<half8_t*>(normed + c * 8) = o;
    }
    if (c < kchunks) {
      const half8_t w = *reinterpret_cast<const half8_t*>(k_norm + c * 8);
      half8_t o;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        o[j] = clamp_f16((half_t)((float)w[j] * (float)(half_t)((float)k[i][j] * rk)), clip);
      *reinterpret_cast<half8_t*>(normed + qd + c * 8) = o;
    }
  }
  __syncthreads();

  // rotary embedding: out[d] = f16(y[d] * cos[d]) + f16(rot[d] * sin[d]), rot = [-y[D/2:], y[:D/2]]
  const int half_d = D >> 1;
  const half_t* cs = cos_t + (size_t)pos * D;
  const half_t* sn = sin_t + (size_t)pos * D;
  const int all = qchunks + kchunks;
  for (int c = threadIdx.x; c < all; c += ROW_THREADS) {
    const int d0 = (c * 8) % D;  // qd is a multiple of D, so this also holds in the k part
    const half8_t y = *reinterpret_cast<const half8_t*>(normed + c * 8);
    const bool low = d0 < half_d;
    const half8_t other = *reinterpret_cast<const half8_t*>(normed + c * 8 + (low ? half_d : -half_d));
    const half8_t cc = *reinterpret_cast<const half8_t*>(cs + d0);
    const half8_t ssn = *reinterpret_cast<const half8_t*>(sn + d0);
    half8_t o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      o[j] = rotary_f16(y[j], low ? -other[j] : other[j], cc[j], ssn[j]);
    }
    if (c < qchunks) {
      *reinterpret_cast<half8_t*>(q_out + (size_t)r * qd + c * 8) = o;
    } else if (slot_ok) {
      const int e = (c - qchunks) * 8, h = e / D;
      *reinterpret_cast<half8_t*>(kcache + (((size_t)b * kv_heads + h) * capacity + slot) * D + (e - h * D)) = o;
    }
  }
  if (slot_ok) {
    for (int c = threadIdx.x; c < kchunks; c += ROW_THREADS) {
      half8_t v = *reinterpret_cast<const half8_t*>(row + qd + kvd + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = clamp_f16(v[j], clip);
      const int e = c * 8, h = e / D;
      *reinterpret_cast<half8_t*>(vcache + (((size_t)b * kv_heads + h) * capacity + slot) * D + (e - h * D)) = v;
    }
  }
}

// Sum over the LPK lanes that share a key (LPK = 16: one DPP row; 8: half a row).
template <int LPK>
__device__ __forceinline__ float key_sum(float v) {
  if (LPK == 16) return row_allreduce(v, [](float a, float b) { return a + b; });
  v += __shfl_xor(v, 4, WAVE);
  v += __shfl_xor(v, 2, WAVE);
  v += __shfl_xor(v, 1, WAVE);
  return v;
}

constexpr float MASKED = -1.0e30f;   // running maximum before any key was seen

// One workgroup per (sequence, query head), NW wavefronts. A load instruction covers KPL =
// 64 / LPK consecutive keys (LPK = D / 8 lanes per key, 16 bytes per lane: whole 256-byte rows
// for D = 128), so the cache is read as long contiguous runs. Each group of LPK lanes keeps its
// own running softmax (maximum, sum, 8 output dimensions per lane) over the keys it meets, so
// the key loop has no cross-lane traffic except the score's sum; the KPL x NW partial results
// are merged once at the end.
// What the fused variant needs beyond the plain one: the projections' output and what
// qk_norm_rope_cache takes.
struct NewToken {
  const half_t* qkv;      // [B, (heads + 2 kv_heads) D]
  const half_t* q_norm;   // [heads D]
  const half_t* k_norm;   // [kv_heads D]
  const half_t* cos_t;    // [max_positions, D]
  const half_t* sin_t;
  const int64_t* positions;
  half_t* kcache_w;       // the caches again, writable
  half_t* vcache_w;
  uint8_t* real_w;        // the mask again, writable: the new token's position becomes real
  float eps, clip;
  int max_positions;
};

// A head's 16-byte chunk c of a projection, loaded with everything its norm and rotary
// embedding need, so that the loads are in flight before the norm's scale is known.
template <int LPK>
struct HeadChunk {
  half8_t mine, other, wm, wo;
  __device__ __forceinline__ void load(const half_t* head, const half_t* norm_w, int c) {
    const int partner = c ^ (LPK / 2);
    mine = *reinterpret_cast<const half8_t*>(head + c * 8);
    other = *reinterpret_cast<const half8_t*>(head + partner * 8);
    wm = *reinterpret_cast<const half8_t*>(norm_w + c * 8);
    wo = *reinterpret_cast<const half8_t*>(norm_w + partner * 8);
  }
  // RMS norm (scale rs), clamp and rotary embedding, with the roundings of qk_norm_rope_cache
  __device__ __forceinline__ half8_t finish(float rs, float clip, half8_t cc, half8_t ss, int c) const {
    const bool low = c < LPK / 2;
    half8_t o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half_t a = clamp_f16((half_t)((float)wm[j] * (float)(half_t)((float)mine[j] * rs)), clip);
      const half_t r = clamp_f16((half_t)((float)wo[j] * (float)(half_t)((float)other[j] * rs)), clip);
      o[j] = rotary_f16(a, low ? -r : r, cc[j], ss[j]);
    }
    return o;
  }
};

// A batch of UNROLL key groups of one wavefront: 16 bytes of key and of value per lane each.
template <int UNROLL>
struct KeyBatch {
  half8_t kk[UNROLL], vv[UNROLL];
  bool ok[UNROLL];
};

// FUSED: the query is taken from the projections' output (norm over the whole q and k rows of
// the sequence, clamp, rotary embedding: the work of qk_norm_rope_cache, redone by every
// workgroup for its own head, which costs two 4 KB reads from L2), the new key and value are
// used from registers as the last key, and the first query head of each kv head writes them
// into the cache; the loop then covers the cached keys before `slot` only.
// The first batch of keys and values is requested before any of that. (Requesting each further
// batch while the previous one is multiplied costs registers, hence resident wavefronts, and
// with them bandwidth: 67.5 us against 55.3 us at 64 sequences x 16 heads x 536 keys.)
// NW wavefronts per workgroup, each with a batch of UNROLL key groups in flight: 16 wavefronts
// when there are few (sequence, head) pairs, so that the cache is still read by many, 4 when
// the pairs fill the chip.
template <int LPK, bool FUSED, int NW, int UNROLL>
__global__ void __launch_bounds__(NW * WAVE)
decode_attention_kernel(const half_t* __restrict__ q, const half_t* kcache, const half_t* vcache,
                                        const uint8_t* __restrict__ real, const int64_t* __restrict__ slot_ptr,
                                        int heads, int kv_heads, int capacity, float scale_log2e,
                                        half_t* __restrict__ out, NewToken nt) {
  constexpr int D = LPK * 8, KPL = WAVE / LPK;
  extern __shared__ float merge[];  // [NW][D + 2]: accumulators, maximum, sum
  __shared__ float part[32];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int sub = lane / LPK, c = lane % LPK;
  const int b = blockIdx.x / heads, qh = blockIdx.x % heads;
  const int group = heads / kv_heads, kvh = qh / group;
  const long slot = (long)*slot_ptr;
  long n = FUSED ? slot : slot + 1;   // cached keys the loop visits
  n = n < 0 ? 0 : n > capacity ? capacity : n;
  const size_t base = ((size_t)b * kv_heads + kvh) * (size_t)capacity * D + c * 8;
  const uint8_t* rl = real + (size_t)b * capacity;
  const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int groups = ((int)n + KPL - 1) / KPL, stride = NW * UNROLL;

  auto fetch = [&](KeyBatch<UNROLL>& kb, int g0) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int key = (g0 + u * NW) * KPL + sub;
      kb.ok[u] = key < n;
      kb.kk[u] = zero8;
      kb.vv[u] = zero8;
      if (kb.ok[u]) {
        kb.kk[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(kcache + base + (size_t)key * D));   // the cache is
        kb.vv[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(vcache + base + (size_t)key * D));   // read once a step
        kb.ok[u] = rl[key] != 0;
      }
    }
  };
  KeyBatch<UNROLL> ka;
  fetch(ka, wave);   // requested before the prologue, so that the two waits overlap

  float qf[8];
  half8_t knew = zero8, vnew = zero8;
  if (FUSED) {
    const int qd = heads * D, kvd = kv_heads * D;
    const half_t* row = nt.qkv + (size_t)b * (qd + 2 * kvd);
    long pos = (long)nt.positions[b];
    pos = pos < 0 ? 0 : pos >= nt.max_positions ? nt.max_positions - 1 : pos;
    HeadChunk<LPK> hq, hk;
    hq.load(row + qh * D, nt.q_norm + qh * D, c);
    hk.load(row + qd + kvh * D, nt.k_norm + kvh * D, c);
    vnew = *reinterpret_cast<const half8_t*>(row + qd + kvd + kvh * D + c * 8);
    const half8_t cc = *reinterpret_cast<const half8_t*>(nt.cos_t + (size_t)pos * D + c * 8);
    const half8_t ss = *reinterpret_cast<const half8_t*>(nt.sin_t + (size_t)pos * D + c * 8);
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < (qd >> 3); i += blockDim.x) {
      const half8_t v = *reinterpret_cast<const half8_t*>(row + i * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) sq += (float)v[j] * (float)v[j];
    }
    for (int i = threadIdx.x; i < (kvd >> 3); i += blockDim.x) {
      const half8_t v = *reinterpret_cast<const half8_t*>(row + qd + i * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) sk += (float)v[j] * (float)v[j];
    }
    // both sums through one barrier
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if (lane == 0) {
      part[wave] = sq;
      part[16 + wave] = sk;
    }
    __syncthreads();
    sq = sk = 0.f;
    for (int w = 0; w < NW; ++w) {
      sq += part[w];
      sk += part[16 + w];
    }
    const float rq = rsqrtf(sq / (float)qd + nt.eps), rk = rsqrtf(sk / (float)kvd + nt.eps);
    const half8_t qv = hq.finish(rq, nt.clip, cc, ss, c);
#pragma unroll
    for (int j = 0; j < 8; ++j) qf[j] = (float)qv[j] * scale_log2e;
    knew = hk.finish(rk, nt.clip, cc, ss, c);
#pragma unroll
    for (int j = 0; j < 8; ++j) vnew[j] = clamp_f16(vnew[j], nt.clip);
    if (slot >= 0 && slot < capacity && qh % group == 0 && wave == 0 && sub == 0) {
      const size_t at = (((size_t)b * kv_heads + kvh) * capacity + slot) * D + c * 8;
      *reinterpret_cast<half8_t*>(nt.kcache_w + at) = knew;
      *reinterpret_cast<half8_t*>(nt.vcache_w + at) = vnew;
      // no workgroup of this launch reads the mask at `slot`: the loop stops before it
      if (qh == 0 && c == 0) nt.real_w[(size_t)b * capacity + slot] = 1;
    }
  } else {
    const half8_t qv = *reinterpret_cast<const half8_t*>(q + ((size_t)b * heads + qh) * D + c * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) qf[j] = (float)qv[j] * scale_log2e;
  }

  float m = MASKED, l = 0.f, acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;

  auto consume = [&](const KeyBatch<UNROLL>& kb) {
    float s[UNROLL], mx = m;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      float d = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) d += qf[j] * (float)kb.kk[u][j];
      s[u] = key_sum<LPK>(d);
      if (kb.ok[u]) mx = fmaxf(mx, s[u]);
    }
    const float alpha = __builtin_amdgcn_exp2f(m - mx);
    m = mx;
    l *= alpha;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] *= alpha;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const float p = kb.ok[u] ? __builtin_amdgcn_exp2f(s[u] - mx) : 0.f;
      l += p;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] += p * (float)kb.vv[u][j];
    }
  };
  for (int g0 = wave; g0 < groups; g0 += stride) {
    if (g0 != wave) fetch(ka, g0);
    consume(ka);
  }

  if (FUSED && wave == 0 && slot >= 0 && slot < capacity) {
    // the new token's own key and value, from registers: one more key for the first key group
    float d = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) d += qf[j] * (float)knew[j];
    const float sc = key_sum<LPK>(d);
    const bool ok = sub == 0;   // the new token is real
    const float mx = ok ? fmaxf(m, sc) : m;
    const float alpha = __builtin_amdgcn_exp2f(m - mx);
    const float p = ok ? __builtin_amdgcn_exp2f(sc - mx) : 0.f;
    m = mx;
    l = l * alpha + p;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = acc[j] * alpha + p * (float)vnew[j];
  }

  // ---- merge the KPL key groups of the wavefront (lanes with equal c)
  float mw = m;
#pragma unroll
  for (int off = LPK; off < WAVE; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, WAVE));
  const float a = __builtin_amdgcn_exp2f(m - mw);
  l *= a;
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] *= a;
#pragma unroll
  for (int off = LPK; off < WAVE; off <<= 1) {
    l += __shfl_xor(l, off, WAVE);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] += __shfl_xor(acc[j], off, WAVE);
  }
  float* mine = merge + wave * (D + 2);
  if (sub == 0) {
#pragma unroll
    for (int j = 0; j < 8; ++j) mine[c * 8 + j] = acc[j];
    if (c == 0) {
      mine[D] = mw;
      mine[D + 1] = l;
    }
  }
  __syncthreads();
  // ---- merge the wavefronts: thread d < D finishes output dimension d
  if (threadIdx.x < D) {
    float M = MASKED;
    for (int w = 0; w < NW; ++w) M = fmaxf(M, merge[w * (D + 2) + D]);
    float num = 0.f, den = 0.f;
    for (int w = 0; w < NW; ++w) {
      const float f = __builtin_amdgcn_exp2f(merge[w * (D + 2) + D] - M);
      num += f * merge[w * (D + 2) + threadIdx.x];
      den += f * merge[w * (D + 2) + D + 1];
    }
    out[((size_t)b * heads + qh) * D + threadIdx.x] = (half_t)(den > 0.f ? num / den : 0.f);
  }
}

// One workgroup per sequence: the arg-max of its logits (the lowest index among equal maxima)
// becomes its next token, is appended to its output row, and its rotary position advances;
// the first workgroup also advances the cache slot, which nothing in this launch reads.
constexpr int PICK_THREADS = 1024;

__global__ void __launch_bounds__(PICK_THREADS)
greedy_advance_kernel(const half_t* __restrict__ logits, int V, int64_t* __restrict__ tok, int64_t* __restrict__ out,
                      int out_stride, const int64_t* __restrict__ base_position, int64_t* __restrict__ next_position,
                      int64_t* __restrict__ slot) {
  __shared__ float best_v[PICK_THREADS / WAVE];
  __shared__ int best_i[PICK_THREADS / WAVE];
  const int b = blockIdx.x, tid = threadIdx.x;
  const half_t* row = logits + (size_t)b * V;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  const int chunks = V % 8 == 0 ? V >> 3 : 0;   // 16-byte loads need rows that start on 16 bytes
  for (int c = tid; c < chunks; c += PICK_THREADS) {
    const half8_t v = *reinterpret_cast<const half8_t*>(row + c * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float f = (float)v[j];
      if (f > bv) {           // ascending indices per thread: the first of equal values is kept
        bv = f;
        bi = c * 8 + j;
      }
    }
  }
  for (int i = chunks * 8 + tid; i < V; i += PICK_THREADS) {
    const float f = (float)row[i];
    if (f > bv) {
      bv = f;
      bi = i;
    }
  }
  // wavefront, then workgroup: larger value wins, equal values go to the lower index
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, WAVE);
    const int oi = __shfl_xor(bi, off, WAVE);
    if (ov > bv || (ov == bv && oi < bi)) {
      bv = ov;
      bi = oi;
    }
  }
  if ((tid & 63) == 0) {
    best_v[tid >> 6] = bv;
    best_i[tid >> 6] = bi;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < PICK_THREADS / WAVE; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
        bv = best_v[w];
        bi = best_i[w];
      }
    if (bi == 0x7fffffff) bi = 0;   // a row of NaNs or -inf: token 0
    tok[b] = bi;
    const long col = (long)(next_position[b] - base_position[b]);
    if (col >= 0 && col < out_stride) out[(size_t)b * out_stride + col] = bi;
    next_position[b] += 1;
    if (b == 0) *slot += 1;
  }
}

}  // namespace

#define ROW_LIMITS(what)                                                                          \
  SY_REQUIRE(N >= 0 && H >= 8 && H % 8 == 0 && H <= 8 * ROW_THREADS * MAX_CHUNKS,                \
             what ": N = %d, H = %d (a multiple of 8 up to %d)", N, H, 8 * ROW_THREADS * MAX_CHUNKS)

extern "C" SY_API int sy_add_rmsnorm(const void* x, const void* delta, const void* weight, float eps, int N, int H,
                                     void* x_out, void* h_out, void* stream) {
  ROW_LIMITS("add_rmsnorm");
  if (N == 0) return SY_OK;
  SY_REQUIRE(x && weight && h_out, "add_rmsnorm: null pointer");
  row_kernel<false, false><<<N, ROW_THREADS, 0, (hipStream_t)stream>>>(
      (const half_t*)x, (const half_t*)delta, nullptr, nullptr, nullptr, 0, (const half_t*)weight, eps, nullptr, 0, H,
      (half_t*)x_out, (half_t*)h_out, nullptr, nullptr, 0);
  return sy_check_launch("add_rmsnorm");
}

extern "C" SY_API int sy_embed_rmsnorm(const int64_t* tokens, const void* embed, int vocab, const void* weight, float eps,
                                       int N, int H, void* x_out, void* h_out, void* stream) {
  ROW_LIMITS("embed_rmsnorm");
  SY_REQUIRE(vocab >= 1, "embed_rmsnorm: vocab = %d", vocab);
  if (N == 0) return SY_OK;
  SY_REQUIRE(tokens && embed && weight && x_out && h_out, "embed_rmsnorm: null pointer");
  row_kernel<false, false><<<N, ROW_THREADS, 0, (hipStream_t)stream>>>(
      (const half_t*)embed, nullptr, nullptr, nullptr, nullptr, 0, (const half_t*)weight, eps, nullptr, 0, H,
      (half_t*)x_out, (half_t*)h_out, nullptr, tokens, vocab);
  return sy_check_launch("embed_rmsnorm");
}

extern "C" SY_API int sy_add_rmsnorm_logits(const void* x, const void* delta, const void* weight, float eps,
                                            const void* router, int E, int N, int H, void* x_out, void* h_out,
                                            void* logits, void* stream) {
  ROW_LIMITS("add_rmsnorm_logits");
  SY_REQUIRE(E >= 1 && E <= 1024, "add_rmsnorm_logits: 1 <= E <= 1024 (got %d)", E);
  if (N == 0) return SY_OK;
  SY_REQUIRE(x && weight && h_out && router && logits, "add_rmsnorm_logits: null pointer");
  row_kernel<false, true><<<N, 1024, (size_t)H * sizeof(half_t), (hipStream_t)stream>>>(
      (const half_t*)x, (const half_t*)delta, nullptr, nullptr, nullptr, 0, (const half_t*)weight, eps,
      (const half_t*)router, E, H, (half_t*)x_out, (half_t*)h_out, (half_t*)logits, nullptr, 0);
  return sy_check_launch("add_rmsnorm_logits");
}

extern "C" SY_API int sy_router_logits(const void* h, const void* router, int N, int H, int E, void* logits, void* stream) {
  ROW_LIMITS("router_logits");
  SY_REQUIRE(E >= 1 && E <= 1024, "router_logits: 1 <= E <= 1024 (got %d)", E);
  if (N == 0) return SY_OK;
  SY_REQUIRE(h && router && logits, "router_logits: null pointer");
  row_kernel<false, true><<<N, 1024, (size_t)H * sizeof(half_t), (hipStream_t)stream>>>(
      (const half_t*)h, nullptr, nullptr, nullptr, nullptr, 0, nullptr, 0.f, (const half_t*)router, E, H, nullptr, nullptr,
      (half_t*)logits, nullptr, 0);
  return sy_check_launch("router_logits");
}

// The counters of the launches that end in front_core's tail. Every GPU the library runs on
// holds its own copy, all zero when the module is loaded and again after every launch. In host
// code the array's name is only a handle for hipGetSymbolAddress: launches take next_ticket()'s
// pointer.
static __device__ unsigned front_tickets[front_core::FRONT_TICKETS];

namespace {
constexpr int TICKET_DEVICES = 64;
std::mutex ticket_mutex;
unsigned* ticket_base[TICKET_DEVICES] = {nullptr};
unsigned ticket_next[TICKET_DEVICES][2] = {{0, 0}};

// The counter for the next launch on the current device. Slots are handed out in turn, the
// lower half of the pool to launches that run now and the upper half to launches that a stream
// capture records: a captured launch keeps its slot for every replay of its graph, so no launch
// outside a capture may ever be given it, and two captured launches share a slot only if half
// the pool's size in launches was captured between them.
int next_ticket(unsigned** out, hipStream_t stream) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= TICKET_DEVICES)
    return sy_fail(SY_ERR_LAUNCH, "router_route_sort: no current device below %d", TICKET_DEVICES);
  std::lock_guard<std::mutex> hold(ticket_mutex);
  if (!ticket_base[dev]) {
    void* p = nullptr;
    const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(front_tickets));
    if (err != hipSuccess || !p)
      return sy_fail(SY_ERR_LAUNCH, "router_route_sort: hipGetSymbolAddress: %s", hipGetErrorString(err));
    ticket_base[dev] = static_cast<unsigned*>(p);
  }
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    status = hipStreamCaptureStatusNone;
  }
  constexpr unsigned HALF = front_core::FRONT_TICKETS / 2;
  const int captured = status == hipStreamCaptureStatusActive ? 1 : 0;
  *out = ticket_base[dev] + captured * HALF + ticket_next[dev][captured]++ % HALF;
  return SY_OK;
}

int front_outputs(const char* what, int N, int E, int k, int norm, int32_t* idx, void* w, int32_t* counts, int32_t* offsets,
                  int32_t* token, void* wsorted, int32_t* pos_of, hipStream_t stream, front_core::Outputs* out) {
  SY_REQUIRE(N <= front_core::TAIL_MAX_TOKENS, "%s: at most %d tokens (got %d)", what, front_core::TAIL_MAX_TOKENS, N);
  SY_REQUIRE(E <= 128 && k >= 1 && k <= front_core::TAIL_MAX_K && k <= E, "%s: at most 128 experts and top-8 (got E = %d, k = %d)",
             what, E, k);
  SY_REQUIRE(idx && w && counts && offsets && token && wsorted && pos_of, "%s: null pointer", what);
  unsigned* ticket = nullptr;
  const int rc = next_ticket(&ticket, stream);
  if (rc) return rc;
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  *out = front_core::Outputs{idx, (half_t*)w, counts, offsets, token, (half_t*)wsorted, pos_of, ticket, k, norm, nbits};
  return SY_OK;
}
}  // namespace

extern "C" SY_API int sy_router_route_sort(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits,
                                           int32_t* idx, void* w, int32_t* counts, int32_t* offsets, int32_t* token,
                                           void* wsorted, int32_t* pos_of, void* stream) {
  ROW_LIMITS("router_route_sort");
  SY_REQUIRE(E >= 1, "router_route_sort: E = %d", E);
  if (N == 0) return SY_OK;
  SY_REQUIRE(h && router && logits, "router_route_sort: null pointer");
  front_core::Outputs front;
  const int rc = front_outputs("router_route_sort", N, E, k, norm, idx, w, counts, offsets, token, wsorted, pos_of, (hipStream_t)stream, &front);
  if (rc) return rc;
  const size_t lds = (size_t)H * sizeof(half_t) + front_core::tail_lds_bytes(N, E, k);
  row_kernel<false, true, FRONT_SORT><<<N, 1024, lds, (hipStream_t)stream>>>(
      (const half_t*)h, nullptr, nullptr, nullptr, nullptr, 0, nullptr, 0.f, (const half_t*)router, E, H, nullptr, nullptr,
      (half_t*)logits, nullptr, 0, front);
  return sy_check_launch("router_route_sort");
}

// The router GEMM and route for a few rows, one workgroup per row and no sort: what
// sy_router_route does for a decode step (front.hip hands such calls over).
int sy_router_route_rows(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits, int32_t* idx,
                         void* w, void* stream) {
  ROW_LIMITS("router_route");
  SY_REQUIRE(E >= 1 && E <= 128 && k >= 1 && k <= front_core::TAIL_MAX_K && k <= E,
             "router_route: at most 128 experts and top-8 (got E = %d, k = %d)", E, k);
  if (N == 0) return SY_OK;
  SY_REQUIRE(h && router && logits && idx && w, "router_route: null pointer");
  front_core::Outputs front{idx, (half_t*)w, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, k, norm, 0};
  const size_t lds = (size_t)H * sizeof(half_t) + sizeof(half_t) * ((size_t)(E + 7) / 8 * 8);
  row_kernel<false, true, FRONT_ROUTE><<<N, 1024, lds, (hipStream_t)stream>>>(
      (const half_t*)h, nullptr, nullptr, nullptr, nullptr, 0, nullptr, 0.f, (const half_t*)router, E, H, nullptr, nullptr,
      (half_t*)logits, nullptr, 0, front);
  return sy_check_launch("router_route");
}

extern "C" SY_API int sy_add_rmsnorm_route_sort(const void* x, const void* delta, const void* weight, float eps,
                                                const void* router, int E, int N, int H, int k, int norm, void* x_out,
                                                void* h_out, void* logits, int32_t* idx, void* w, int32_t* counts,
                                                int32_t* offsets, int32_t* token, void* wsorted, int32_t* pos_of,
                                                void* stream) {
  ROW_LIMITS("add_rmsnorm_route_sort");
  SY_REQUIRE(E >= 1, "add_rmsnorm_route_sort: E = %d", E);
  if (N == 0) return SY_OK;
  SY_REQUIRE(x && weight && h_out && router && logits, "add_rmsnorm_route_sort: null pointer");
  front_core::Outputs front;
  const int rc = front_outputs("add_rmsnorm_route_sort", N, E, k, norm, idx, w, counts, offsets, token, wsorted, pos_of, (hipStream_t)stream, &front);
  if (rc) return rc;
  const size_t lds = (size_t)H * sizeof(half_t) + front_core::tail_lds_bytes(N, E, k);
  row_kernel<false, true, FRONT_SORT><<<N, 1024, lds, (hipStream_t)stream>>>(
      (const half_t*)x, (const half_t*)delta, nullptr, nullptr, nullptr, 0, (const half_t*)weight, eps,
      (const half_t*)router, E, H, (half_t*)x_out, (half_t*)h_out, (half_t*)logits, nullptr, 0, front);
  return sy_check_launch("add_rmsnorm_route_sort");
}

extern "C" SY_API int sy_combine_add_rmsnorm(const void* y, const int32_t* pos_of, const int32_t* idx, const void* w, int k,
                                             const void* x, const void* weight, float eps, int N, int H, void* x_out,
                                             void* h_out, void* stream) {
  ROW_LIMITS("combine_add_rmsnorm");
  SY_REQUIRE(k >= 1 && k <= ROW_MAX_K, "combine_add_rmsnorm: 1 <= k <= %d (got %d)", ROW_MAX_K, k);
  if (N == 0) return SY_OK;
  SY_REQUIRE(y && pos_of && idx && x && weight && h_out, "combine_add_rmsnorm: null pointer");
  row_kernel<true, false><<<N, ROW_THREADS, 0, (hipStream_t)stream>>>(
      (const half_t*)x, (const half_t*)w, (const half_t*)y, pos_of, idx, k, (const half_t*)weight, eps, nullptr, 0, H,
      (half_t*)x_out, (half_t*)h_out, nullptr, nullptr, 0);
  return sy_check_launch("combine_add_rmsnorm");
}

extern "C" SY_API int sy_qk_norm_rope_cache(const void* qkv, const void* q_norm, const void* k_norm, float eps, float clip,
                                            const void* cos_table, const void* sin_table, int max_positions,
                                            const int64_t* positions, const int64_t* slot, int B, int T, int heads,
                                            int kv_heads, int D, int capacity, void* q_out, void* kcache, void* vcache,
                                            void* stream) {
  SY_REQUIRE(B >= 0 && T >= 1 && (long)B * T < (1l << 31) && heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0,
             "qk_norm_rope_cache: B = %d, T = %d, heads = %d, kv_heads = %d", B, T, heads, kv_heads);
  SY_REQUIRE(D >= 16 && D % 16 == 0 && (long)heads * D <= 8 * ROW_THREADS * MAX_CHUNKS,
             "qk_norm_rope_cache: head_dim = %d must be a multiple of 16 and heads * head_dim at most %d", D,
             8 * ROW_THREADS * MAX_CHUNKS);
  SY_REQUIRE(capacity >= 1 && max_positions >= 1, "qk_norm_rope_cache: capacity = %d, max_positions = %d", capacity,
             max_positions);
  if (B == 0) return SY_OK;
  SY_REQUIRE(qkv && q_norm && k_norm && cos_table && sin_table && positions && slot && q_out && kcache && vcache,
             "qk_norm_rope_cache: null pointer");
  const size_t lds = (size_t)(heads + kv_heads) * D * sizeof(half_t);
  qk_norm_rope_cache_kernel<<<B * T, ROW_THREADS, lds, (hipStream_t)stream>>>(
      (const half_t*)qkv, (const half_t*)q_norm, (const half_t*)k_norm, eps, clip, (const half_t*)cos_table,
      (const half_t*)sin_table, max_positions, positions, slot, T, heads, kv_heads, D, capacity, (half_t*)q_out,
      (half_t*)kcache, (half_t*)vcache);
  return sy_check_launch("qk_norm_rope_cache");
}

extern "C" SY_API int sy_decode_attention(const void* q, const void* kcache, const void* vcache, const uint8_t* real,
                                          const int64_t* slot, int B, int heads, int kv_heads, int D, int capacity,
                                          void* out, void* stream) {
  SY_REQUIRE(B >= 0 && heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0,
             "decode_attention: B = %d, heads = %d, kv_heads = %d", B, heads, kv_heads);
  SY_REQUIRE(D == 64 || D == 128, "decode_attention: head_dim must be 64 or 128 (got %d)", D);
  SY_REQUIRE(capacity >= 1, "decode_attention: capacity = %d", capacity);
  if (B == 0) return SY_OK;
  SY_REQUIRE(q && kcache && vcache && real && slot && out, "decode_attention: null pointer");
  // few (sequence, head) pairs: 16 wavefronts each, so that the cache is still read by many
  const long pairs = (long)B * heads;
  const int waves = pairs >= 2l * sy_compute_units() ? 4 : 16;
  const size_t lds = (size_t)waves * (D + 2) * sizeof(float);
  const float scale_log2e = 1.4426950408889634f / sqrtf((float)D);
  auto kern = D == 128 ? (waves == 4 ? decode_attention_kernel<16, false, 4, 4> : decode_attention_kernel<16, false, 16, 4>)
                       : (waves == 4 ? decode_attention_kernel<8, false, 4, 4> : decode_attention_kernel<8, false, 16, 4>);
  kern<<<(unsigned)pairs, waves * WAVE, lds, (hipStream_t)stream>>>((const half_t*)q, (const half_t*)kcache,
                                                                   (const half_t*)vcache, real, slot, heads, kv_heads,
                                                                   capacity, scale_log2e, (half_t*)out, NewToken{});
  return sy_check_launch("decode_attention");
}

extern "C" SY_API int sy_decode_attention_qkv(const void* qkv, const void* q_norm, const void* k_norm, float eps, float clip,
                                              const void* cos_table, const void* sin_table, int max_positions,
                                              const int64_t* positions, const int64_t* slot, uint8_t* real, int B,
                                              int heads, int kv_heads, int D, int capacity, void* kcache, void* vcache,
                                              void* out, void* stream) {
  SY_REQUIRE(B >= 0 && heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0,
             "decode_attention_qkv: B = %d, heads = %d, kv_heads = %d", B, heads, kv_heads);
  SY_REQUIRE(D == 64 || D == 128, "decode_attention_qkv: head_dim must be 64 or 128 (got %d)", D);
  SY_REQUIRE(capacity >= 1 && max_positions >= 1, "decode_attention_qkv: capacity = %d, max_positions = %d", capacity,
             max_positions);
  if (B == 0) return SY_OK;
  SY_REQUIRE(qkv && q_norm && k_norm && cos_table && sin_table && positions && slot && real && kcache && vcache && out,
             "decode_attention_qkv: null pointer");
  const long pairs = (long)B * heads;
  const int waves = pairs >= 2l * sy_compute_units() ? 4 : 16;
  const size_t lds = (size_t)waves * (D + 2) * sizeof(float);
  const float scale_log2e = 1.4426950408889634f / sqrtf((float)D);
  NewToken nt{(const half_t*)qkv, (const half_t*)q_norm, (const half_t*)k_norm, (const half_t*)cos_table,
              (const half_t*)sin_table, positions, (half_t*)kcache, (half_t*)vcache, real, eps, clip, max_positions};
  auto kern = D == 128 ? (waves == 4 ? decode_attention_kernel<16, true, 4, 4> : decode_attention_kernel<16, true, 16, 4>)
                       : (waves == 4 ? decode_attention_kernel<8, true, 4, 4> : decode_attention_kernel<8, true, 16, 4>);
  kern<<<(unsigned)pairs, waves * WAVE, lds, (hipStream_t)stream>>>(nullptr, (const half_t*)kcache, (const half_t*)vcache,
                                                                   real, slot, heads, kv_heads, capacity, scale_log2e,
                                                                   (half_t*)out, nt);
  return sy_check_launch("decode_attention_qkv");
}

extern "C" SY_API int sy_greedy_advance(const void* logits, int B, int V, int64_t* tok, int64_t* out, int out_stride,
                                        const int64_t* base_position, int64_t* next_position, int64_t* slot,
                                        void* stream) {
  SY_REQUIRE(B >= 0 && V >= 1 && out_stride >= 0, "greedy_advance: B = %d, V = %d, out_stride = %d", B, V, out_stride);
  if (B == 0) return SY_OK;
  SY_REQUIRE(logits && tok && out && base_position && next_position && slot, "greedy_advance: null pointer");
  greedy_advance_kernel<<<B, PICK_THREADS, 0, (hipStream_t)stream>>>((const half_t*)logits, V, tok, out, out_stride,
                                                                    base_position, next_position, slot);
  return sy_check_launch("greedy_advance");
}
