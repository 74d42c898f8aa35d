// grouped_gemv: the decode path. With a handful of rows per expert the layer is a stream over
// the used experts' weights, so the kernel is built around how HBM likes to be read.
//
// Access pattern. A wavefront streams 4 consecutive weight rows (output columns) at a time,
// sweeping along K. One 128-bit load instruction covers 4 rows x 256 contiguous bytes: lane
// l = 4*b + i reads the 8 halves k = 8*b .. 8*b+7 (plus 128 per step) of row i. That footprint
// (whole cache lines, four sequential streams) reads HBM about 25% faster than the 16 rows x
// 64 bytes a 16x16 MFMA operand would ask for, and it is exactly the operand layout of
// v_mfma_f32_4x4x4_16B_f16: 16 independent 4x4x4 products, block b of lanes 4b..4b+3. With
// the weights as the 4 M rows and 4 of the expert's rows (tokens) as the N columns, block b
// accumulates the partial dot products of its own slice of K; the loaded registers feed the
// MFMA directly, the low and the high 4 halves in two instructions. At the end of K the 16
// blocks are summed across lanes (a fixed tree, so results are deterministic) and lanes 0..3
// hold 4 consecutive output columns of one row each. With SwiGLU a unit of work is the 4 gate
// rows and then the 4 up rows of the same columns; the reduced gate values wait in registers.
//
// Balance. What a CU can pull from HBM is capped by the cache lines it may have in flight,
// so the stream is only as fast as its slowest CU: every CU must be busy until the end. The
// launch is therefore persistent, a fixed number of workgroups per CU, and the units of the
// experts that received rows (found from `offsets` by every workgroup itself) are dealt to
// the workgroups in equal contiguous shares. Experts without rows cost nothing.
//
// Rows. The expert's rows (up to `row_cap` <= 16 per pass, in quads of 4) are staged in LDS,
// padded so that the 128-bit operand reads are bank-conflict free, and shared by the
// workgroup's 4 wavefronts, which split the units of the current expert between them and
// otherwise run independently. Loads are issued one chunk (4 or 8 steps) ahead of the MFMAs that
// consume them, through a buffer descriptor whose range check masks ragged edges without
// branches. An expert with more rows than `row_cap` takes further passes over its weights.
//
// Replaces grouped_gemv_kernel / grouped_gemv of the reference
// (switchyard/csrc/moe_kernels.cu:301-415); epilogue rounding points as :373-378.
#include "sort_core.h"

namespace {

constexpr int GEMV_WAVES = 4;   // wavefronts per workgroup (they share the staged rows)
constexpr int GEMV_THREADS = GEMV_WAVES * WAVE;
constexpr int UNIT_COLS = 4;    // output columns per unit (MFMA M)
constexpr int QUAD = 4;         // rows of the expert per MFMA (MFMA N)
constexpr int MAX_QUADS = 4;    // up to 16 rows per pass
constexpr int STEP_K = 128;     // K covered by one load instruction (16 blocks x 8 halves)
constexpr int CH_SHORT = 4, CH_LONG = 8;  // load steps per chunk (a template parameter: see launch_gemv)
constexpr int ROW_PAD = 32;     // halves of padding per staged row (64 bytes)
constexpr int MAX_E = 1024;     // experts whose ids fit the LDS list

// 128-bit streaming load through a buffer descriptor: lane offset in bytes (out of range
// reads return 0), wave-uniform offset in an SGPR.
__device__ __forceinline__ half8_t load_stream(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_off, unsigned uniform_off) {
  return __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off, uniform_off, /*nt*/ 2));
}
constexpr unsigned OUT_OF_RANGE = 0x80000000u;

__device__ __forceinline__ half4_t lo4(half8_t v) { return __builtin_shufflevector(v, v, 0, 1, 2, 3); }
__device__ __forceinline__ half4_t hi4(half8_t v) { return __builtin_shufflevector(v, v, 4, 5, 6, 7); }

// Sum over the 16 blocks (lanes with equal lane % 4); lanes 0..3 end with the total.
__device__ __forceinline__ float sum_blocks(float v) {
  v += dpp_row_ror<4>(v);
  v += dpp_row_ror<8>(v);   // every lane: the sum over its row of 16 lanes (4 blocks)
  v += __shfl_down(v, 32, WAVE);
  v += __shfl_down(v, 16, WAVE);
  return v;
}

template <int CH>
struct Chunk {
  half8_t w[CH];
};

struct Pass {
  const half_t* xs;             // staged rows
  __amdgpu_buffer_rsrc_t rsrc;  // the expert's weight matrix
  const half_t* scale;
  half_t* C;
  int Nout, K, RS, r0, nr, unit0, nunits, nchunks;
};

// One wavefront streams units [unit0, unit0 + nunits) of one expert against NQ staged quads.
// EXACT: K is a multiple of a chunk (512) and Nout of a unit (4), so nothing needs masking.
template <bool SWIGLU, bool SCALE, bool EXACT, int CH, int NQ>
__device__ __forceinline__ void run_pass(const Pass& p) {
  const int lane = threadIdx.x & 63, blk = lane >> 2, sub = lane & 3;
  const int klane = blk * 8;
  constexpr int PARTS = SWIGLU ? 2 : 1;  // a unit is streamed as its gate rows, then its up rows
  const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // Units start at different steps of K and wrap around: wavefronts that run in step would
  // otherwise all ask for the same stretch of their rows at the same time, and rows a multiple
  // of 4 KB apart then meet on the same few memory channels.
  const int nsteps = p.nchunks * CH;
  const int rot0 = (p.unit0 * 5) % nsteps;

  // ---- issue side: part `ipt` of unit `iun`, chunk `ich` (counted from the unit's start `irot`)
  // is the next to load
  int iun = 0, ipt = 0, ich = 0, irot = rot0;
  auto issue = [&](Chunk<CH>& c) {
    const int col = (p.unit0 + iun) * UNIT_COLS + sub;
    const int wr = ipt ? p.Nout + col : col;
    unsigned lane_off = ((unsigned)wr * (unsigned)p.K + (unsigned)klane) * 2u;
    if (!EXACT && col >= p.Nout) lane_off = OUT_OF_RANGE;
#pragma unroll
    for (int s = 0; s < CH; ++s) {
      const int at = ich * CH + s + irot;
      const int kk = (at - (at >= nsteps ? nsteps : 0)) * STEP_K;
      unsigned off = lane_off;
      if (!EXACT && kk + klane >= p.K) off = OUT_OF_RANGE;
      c.w[s] = load_stream(p.rsrc, off, (unsigned)kk * 2u);
    }
    if (++ich == p.nchunks) {
      ich = 0;
      if (++ipt == PARTS) {
        ipt = 0;
        ++iun;
        irot = (irot + 5) % nsteps;
      }
    }
  };

  // ---- compute side
  int cun = 0, cpt = 0, cch = 0, crot = rot0;
  float4_t acc[NQ], gate[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) acc[q] = gate[q] = float4_t{0.f, 0.f, 0.f, 0.f};
  const half_t* xlane = p.xs + sub * p.RS + klane;  // row `sub` of quad 0 at this lane's K offset

  auto compute = [&](const Chunk<CH>& c) {
#pragma unroll
    for (int s = 0; s < CH; ++s) {
      const int at = cch * CH + s + crot;
      const int kk = (at - (at >= nsteps ? nsteps : 0)) * STEP_K;
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        half8_t x = *reinterpret_cast<const half8_t*>(xlane + q * QUAD * p.RS + kk);
        if (!EXACT && kk + klane >= p.K) x = zero8;  // the weights are 0 there; keep stale LDS out
        acc[q] = __builtin_amdgcn_mfma_f32_4x4x4f16(lo4(c.w[s]), lo4(x), acc[q], 0, 0, 0);
        acc[q] = __builtin_amdgcn_mfma_f32_4x4x4f16(hi4(c.w[s]), hi4(x), acc[q], 0, 0, 0);
      }
    }
    if (++cch < p.nchunks) return;
    cch = 0;
    // part done: sum the 16 K-slices; lane j < 4 then holds columns c0..c0+3 of row 4q + j
    const bool is_gate = SWIGLU && cpt == 0;
    const int c0 = (p.unit0 + cun) * UNIT_COLS;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      float4_t v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = sum_blocks(acc[q][i]);
      acc[q] = float4_t{0.f, 0.f, 0.f, 0.f};
      if (is_gate) {
        gate[q] = v;
        continue;
      }
      const int r = q * QUAD + lane;
      if (lane < QUAD && r < p.nr) {
        const float row_scale = SCALE ? (float)p.scale[p.r0 + r] : 1.f;
        half4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (SWIGLU) o[i] = swiglu_f16(gate[q][i], v[i]);
          else if (SCALE) o[i] = (half_t)((float)(half_t)v[i] * row_scale);
          else o[i] = (half_t)v[i];
        }
        half_t* dst = p.C + (size_t)(p.r0 + r) * p.Nout + c0;
        if (EXACT || (c0 + 3 < p.Nout && (p.Nout & 3) == 0)) {
          *reinterpret_cast<half4_t*>(dst) = o;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (c0 + i < p.Nout) dst[i] = o[i];
        }
      }
    }
    if (++cpt == PARTS) {
      cpt = 0;
      ++cun;
      crot = (crot + 5) % nsteps;
    }
  };

  // chunk q+1 is in flight while chunk q is multiplied
  const int total = p.nunits * PARTS * p.nchunks;
  if (total <= 0) return;
  Chunk<CH> c0, c1;
  issue(c0);
  int q = 0;
  for (; q + 3 <= total; q += 2) {
    issue(c1);
    compute(c0);
    issue(c0);
    compute(c1);
  }
  if (total - q == 2) {
    issue(c1);
    compute(c0);
    compute(c1);
  } else {
    compute(c0);
  }
}

// What a launch that sorts for itself reads and leaves behind: the routing of at most 64 choices
// (a decode step of 8 tokens) in, the five results of sort_by_expert out.
struct SortHere {
  const int* idx;        // [N, k]
  const half_t* w;       // [N, k]
  int M, k, nbits;
  int* counts;           // [E]
  int* offsets;          // [E + 1]
  int* token;            // [M]
  half_t* wsorted;       // [M]
  int* pos_of;           // [M]
};
constexpr int SORT_HERE_MAX = WAVE;   // choices that one wavefront sorts with one per lane
__host__ __device__ constexpr size_t sort_here_ints(int E) {
  return (size_t)E + (E + 1) + 2 * SORT_HERE_MAX + SORT_HERE_MAX / 2 + (2 * E + 1);
}

// With SORT the launch has no sorted rows to start from, only the routing: every workgroup
// sorts the (at most 64) choices itself, one wavefront with a choice per lane, into LDS, and
// the first workgroup also writes the results out for the launches that follow. In front of a
// weight stream of tens of microseconds that costs each workgroup a few hundred cycles where
// its scan of `offsets` stood, and the launch before it need not gather every token's choices
// in one place.
template <bool SWIGLU, bool SCALE, bool EXACT, int CH, bool SORT = false>
__global__ void __launch_bounds__(GEMV_THREADS)
gemv_kernel(const half_t* __restrict__ A, const int* __restrict__ a_rows, const half_t* __restrict__ B,
            const int* __restrict__ offsets, int E, int Nout, int K, const half_t* __restrict__ scale,
            half_t* __restrict__ C, int row_cap, SortHere sort = SortHere{}) {
  extern __shared__ __attribute__((aligned(16))) half_t xs[];  // [row_cap][K + ROW_PAD], then the used experts
  // the wavefront's number is the same in all its lanes, and said so: every unit, K offset and
  // buffer descriptor below derives from it, and what the compiler cannot prove uniform it wraps
  // in a loop over the lanes' values, around every load of the stream
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int RS = K + ROW_PAD;
  int* used = reinterpret_cast<int*>(xs + (size_t)row_cap * RS);  // [E] ids of experts with rows, [E] = how many
  const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // SORT: the sort's results in LDS, behind the list of used experts
  int* s_counts = used + E + 1;
  int* s_offsets = s_counts + E;
  int* s_token = s_offsets + E + 1;
  int* s_pos = s_token + SORT_HERE_MAX;
  uint16_t* s_wsorted = reinterpret_cast<uint16_t*>(s_pos + SORT_HERE_MAX);
  if (SORT) {
    if (wave == 0)
      sort_core::sort_one_wave<uint16_t>(sort.idx, reinterpret_cast<const uint16_t*>(sort.w), sort.M, sort.k, E, sort.nbits,
                                         s_counts, s_offsets, s_token, s_wsorted, s_pos,
                                         reinterpret_cast<int*>(s_wsorted + SORT_HERE_MAX));
    __syncthreads();
    if (blockIdx.x == 0) {
      for (int i = threadIdx.x; i <= E; i += GEMV_THREADS) {
        sort.offsets[i] = s_offsets[i];
        if (i < E) sort.counts[i] = s_counts[i];
      }
      for (int i = threadIdx.x; i < sort.M; i += GEMV_THREADS) {
        sort.token[i] = s_token[i];
        sort.pos_of[i] = s_pos[i];
        reinterpret_cast<uint16_t*>(sort.wsorted)[i] = s_wsorted[i];
      }
    }
  }

  // ---- the experts that received rows, in order (one wavefront, 64 experts per step)
  if (wave == 0) {
    int n = 0;
    for (int e0 = 0; e0 < E; e0 += WAVE) {
      const int e = e0 + lane;
      const bool has = e < E && (SORT ? s_offsets[e + 1] > s_offsets[e] : offsets[e + 1] > offsets[e]);
      const uint64_t m = __ballot(has);
      if (has) used[n + __popcll(m & lanemask_lt())] = e;
      n += __popcll(m);
    }
    if (lane == 0) used[E] = n;
  }
  __syncthreads();
  const int nused = used[E];
  const int units_per_expert = (Nout + UNIT_COLS - 1) / UNIT_COLS;

  // ---- this workgroup's equal share of all units, a contiguous range [lo, hi)
  const long total_units = (long)nused * units_per_expert;
  const int lo = (int)(total_units * blockIdx.x / gridDim.x), hi = (int)(total_units * (blockIdx.x + 1) / gridDim.x);

  Pass p;
  p.xs = xs;
  p.Nout = Nout;
  p.K = K;
  p.RS = RS;
  p.scale = scale;
  p.C = C;
  p.nchunks = ((K + STEP_K - 1) / STEP_K + CH - 1) / CH;
  const int Nfull = SWIGLU ? 2 * Nout : Nout;
  bool staged = false;

  for (int at = lo; at < hi;) {
    // the part of the range that falls into one expert
    const int u = at / units_per_expert, first = at - u * units_per_expert;
    const int count = min(hi - at, units_per_expert - first);
    // the same in every lane, and said so: the weights' buffer descriptor is built from it, and a
    // descriptor that the compiler cannot prove uniform costs every load a loop over its lanes
    const int e = __builtin_amdgcn_readfirstlane(used[u]);
    const int start = __builtin_amdgcn_readfirstlane(SORT ? s_offsets[e] : offsets[e]);
    const int end = __builtin_amdgcn_readfirstlane(SORT ? s_offsets[e + 1] : offsets[e + 1]);
    p.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(B + (size_t)e * Nfull * K), 0,
                                               (int)((size_t)Nfull * K * 2), 0x00020000);
    // wavefront w takes a contiguous quarter of the units
    p.unit0 = first + (int)((long)count * wave / GEMV_WAVES);
    p.nunits = first + (int)((long)count * (wave + 1) / GEMV_WAVES) - p.unit0;

    for (int r0 = start; r0 < end; r0 += row_cap) {
      const int nr = min(row_cap, end - r0);
      const int nq = (nr + QUAD - 1) / QUAD;
      // ---- stage the pass's rows: wavefront w copies rows w, w+4, ...; missing rows of the last quad are zero
      if (staged) __syncthreads();
      for (int r = wave; r < nq * QUAD; r += GEMV_WAVES) {
        const half_t* src = r < nr ? A + (size_t)(SORT ? s_token[r0 + r] : a_rows ? a_rows[r0 + r] : r0 + r) * K : nullptr;
        for (int kk = lane * 8; kk < K; kk += WAVE * 8)
          *reinterpret_cast<half8_t*>(xs + r * RS + kk) = src ? *reinterpret_cast<const half8_t*>(src + kk) : zero8;
      }
      __syncthreads();
      staged = true;
      p.r0 = r0;
      p.nr = nr;
      switch (nq) {
        case 1: run_pass<SWIGLU, SCALE, EXACT, CH, 1>(p); break;
        case 2: run_pass<SWIGLU, SCALE, EXACT, CH, 2>(p); break;
        case 3: run_pass<SWIGLU, SCALE, EXACT, CH, 3>(p); break;
        default: run_pass<SWIGLU, SCALE, EXACT, CH, 4>(p); break;
      }
    }
    at += count;
  }
}

int launch_gemv(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets, int E, int rows,
                int max_rows_hint, int Nout, int K, int swiglu, const void* scale, void* C, hipStream_t stream,
                const SortHere* sort = nullptr) {
  // rows staged per pass: no expert has more rows than there are rows in all; a caller that
  // knows a tighter bound (the number of tokens) saves LDS and gains occupancy
  const int bound = max_rows_hint > 0 && max_rows_hint < rows ? max_rows_hint : rows;
  int row_cap = (bound + QUAD - 1) / QUAD * QUAD;
  row_cap = row_cap > MAX_QUADS * QUAD ? MAX_QUADS * QUAD : row_cap;
  const size_t lds = (size_t)row_cap * (K + ROW_PAD) * sizeof(half_t) + (size_t)(E + 1) * sizeof(int) +
                     (sort ? sort_here_ints(E) * sizeof(int) : 0);
  // Loads in flight per wavefront: a chunk of 4 KB, or of 8 KB where a unit is long enough to be
  // cut into such chunks (gate and up rows of 2048 at 8 tokens: 56.6 us against 57.5; for rows of
  // 1024 the longer chunk is one per unit and loses: 34.8 us against 30.6).
  const bool long_chunks = swiglu && K % (CH_LONG * STEP_K) == 0 && K >= 2 * CH_LONG * STEP_K;
  const bool exact = K % (CH_SHORT * STEP_K) == 0 && Nout % UNIT_COLS == 0;
  // persistent: a fixed number of workgroups per CU, but no more than there are units. Two per
  // CU stream best when a unit is 32 KB of weights (gate and up rows of 2048: 57.8 us against
  // 59.0 and 63.4 with three and four), four when it is 8 KB (rows of 1024: 31.8 us against
  // 32.2 and 33.4 with three and two); all of them must be resident at once.
  const long unit_bytes = (long)UNIT_COLS * K * 2 * (swiglu ? 2 : 1);
  long per_cu = unit_bytes >= 32768 ? 2 : unit_bytes >= 16384 ? 3 : 4;
  if (!exact && per_cu > 3) per_cu = 3;                       // the masked variants need more registers
  const long fit = (160 * 1024) / (long)(lds ? lds : 1);      // by LDS
  per_cu = per_cu > fit ? (fit > 0 ? fit : 1) : per_cu;
  const long max_units = (long)(E < rows ? E : rows) * ((Nout + UNIT_COLS - 1) / UNIT_COLS);
  long grid = (long)sy_compute_units() * per_cu;
  grid = grid > max_units ? max_units : grid;
  const half_t* a = (const half_t*)A;
  const half_t* b = (const half_t*)B;
  const half_t* s = (const half_t*)scale;
  half_t* c = (half_t*)C;
  void (*kern)(const half_t*, const int*, const half_t*, const int*, int, int, int, const half_t*, half_t*, int, SortHere);
  if (sort && long_chunks && exact) kern = gemv_kernel<true, false, true, CH_LONG, true>;
  else if (sort) kern = exact ? gemv_kernel<true, false, true, CH_SHORT, true> : gemv_kernel<true, false, false, CH_SHORT, true>;
  else if (swiglu && long_chunks && exact) kern = gemv_kernel<true, false, true, CH_LONG>;
  else if (swiglu) kern = exact ? gemv_kernel<true, false, true, CH_SHORT> : gemv_kernel<true, false, false, CH_SHORT>;
  else if (s) kern = exact ? gemv_kernel<false, true, true, CH_SHORT> : gemv_kernel<false, true, false, CH_SHORT>;
  else kern = exact ? gemv_kernel<false, false, true, CH_SHORT> : gemv_kernel<false, false, false, CH_SHORT>;
  hipError_t attr = hipSuccess;
  if (lds > 48 * 1024) attr = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return sy_fail(SY_ERR_LAUNCH, "grouped_gemv: cannot reserve %zu bytes of LDS", lds);
  kern<<<(unsigned)grid, GEMV_THREADS, lds, stream>>>(a, a_rows, b, offsets, E, Nout, K, swiglu ? nullptr : s, c, row_cap,
                                                      sort ? *sort : SortHere{});
  return sy_check_launch("grouped_gemv");
}

// ---------------------------------------------------------------------------------------------
// The down projection and combine of a decode step in one launch, for at most 32 sorted rows of
// at most 4 tokens.
//
// With a handful of tokens the combine is a launch's latency around a microsecond of work, and
// the rows it adds up were written a moment earlier by the launch before it. Here the work is
// cut by output column instead of by expert: a unit of 4 columns is streamed for every expert
// that has rows, in ascending expert order, so whoever owns the unit sees all of a token's k
// rows and can add them up itself, in the order combine adds them, and `y` never exists. Every
// unit costs the same, so the shares are equal by construction. A workgroup of eight wavefronts
// takes two units; the four wavefronts of a unit take the experts in turn and leave each row's
// scaled, rounded values in LDS; after a
// barrier the rows of every token are added in row order (rows are sorted by expert, so that
// is ascending expert id, and then by slot, as in combine_kernel). All sorted rows are staged
// in LDS once, straight from memory, behind the first loads of weights.
//
// Measured against the two launches (down projection, then combine; OLMoE shape): 1 token 10.5
// against 13.9 us, 4 tokens 23 against 26.4; at 8 tokens it loses, 37.0 against 35.2 (every
// workgroup stages all 64 rows, and a launch cut by column streams at 4.7 TB/s where the one cut
// by expert reaches 5.7), so it takes up to 4 tokens. Four wavefronts per compute unit with 8, 16
// or 32 KB in flight each took 41 to 43 us at 8 tokens whatever the depth, and as long with the
// MFMAs taken out: more wavefronts, not more loads per wavefront, is what a compute unit needs.
//
// The roundings are those of the two launches it replaces (gemv_kernel without scales, then
// combine_kernel<true>): the fp32 dot product in the same K order (a unit starts at the same
// step of K) rounded to f16, times the router weight rounded to f16, added in fp32.
constexpr int DC_WAVES = 8, DC_THREADS = DC_WAVES * WAVE;
constexpr int DC_UNITS = 2;        // units per workgroup; DC_WAVES / DC_UNITS wavefronts share the experts of one
constexpr int DC_DEPTH = 2;        // chunks of weights (4 KB) a wavefront asks for ahead
constexpr int DC_MAX_ROWS = 32, DC_MAX_TOKENS = 4, DC_MAX_E = 128;

__host__ __device__ constexpr size_t dc_rows(int M) { return (size_t)(M + 3) / 4 * 4 + 8; }   // staged rows, zero rows behind the last
__host__ __device__ constexpr size_t dc_lds_bytes(int M, int K, int E) {
  return dc_rows(M) * (K + ROW_PAD) * sizeof(half_t) + sizeof(float) * 4 * DC_UNITS * DC_MAX_ROWS +
         sizeof(int) * ((E + 1) + 2 * (DC_MAX_ROWS + 1) + 2 * DC_MAX_ROWS);
}

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // m0 carries the LDS address of the staging loads
template <int NQ>
__global__ void __launch_bounds__(DC_THREADS)
gemv_down_combine_kernel(const half_t* __restrict__ act, const half_t* __restrict__ B, const int* __restrict__ offsets,
                         const int* __restrict__ token, const half_t* __restrict__ wsorted, int E, int Nout, int K, int N,
                         int M, half_t* __restrict__ out) {
  constexpr int CH = CH_SHORT;
  extern __shared__ __attribute__((aligned(16))) half_t xs[];   // [dc_rows(M)][K + ROW_PAD]
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int RS = K + ROW_PAD;
  const int nrows_lds = (int)dc_rows(M);
  float* sval = reinterpret_cast<float*>(xs + (size_t)nrows_lds * RS);   // [DC_UNITS][DC_MAX_ROWS][4]
  int* offs = reinterpret_cast<int*>(sval + 4 * DC_UNITS * DC_MAX_ROWS);   // [E + 1]
  int* item_e = offs + E + 1;             // [items + 1]: expert of a pass; [DC_MAX_ROWS] = how many
  int* item_r = item_e + DC_MAX_ROWS + 1;   // first row of the pass
  int* tok = item_r + DC_MAX_ROWS + 1;    // [M]
  float* wt = reinterpret_cast<float*>(tok + DC_MAX_ROWS);   // [M]

  // ---- the passes: per expert with rows, ceil(rows / (4 NQ)) of them (one, unless an id repeats)
  for (int i = tid; i <= E; i += DC_THREADS) offs[i] = offsets[i];
  for (int i = tid; i < M; i += DC_THREADS) {
    tok[i] = token[i];
    wt[i] = (float)wsorted[i];
  }
  __syncthreads();
  if (wave == 0) {
    int run = 0;
    for (int e0 = 0; e0 < E; e0 += WAVE) {
      const int e = e0 + lane;
      const int n = e < E ? offs[e + 1] - offs[e] : 0;
      const int mine = (n + 4 * NQ - 1) / (4 * NQ);
      int inc = mine;
      for (int o = 1; o < WAVE; o <<= 1) {
        const int up = __shfl_up(inc, o, WAVE);
        if (lane >= o) inc += up;
      }
      for (int j = 0; j < mine; ++j) {
        const int at = run + inc - mine + j;
        if (at < DC_MAX_ROWS) {
          item_e[at] = e;
          item_r[at] = offs[e] + j * 4 * NQ;
        }
      }
      run += __shfl(inc, WAVE - 1, WAVE);
    }
    if (lane == 0) item_e[DC_MAX_ROWS] = run < DC_MAX_ROWS ? run : DC_MAX_ROWS;
  }
  __syncthreads();
  const int nitems = item_e[DC_MAX_ROWS];
  const int rows_end = offs[E];

  const int blk = lane >> 2, sub = lane & 3, klane = blk * 8;
  const int nchunks = K / (CH * STEP_K), nsteps = nchunks * CH;
  const int units = Nout / UNIT_COLS;
  constexpr int SHARE = DC_WAVES / DC_UNITS;   // wavefronts per unit
  const int us = wave / SHARE, part = wave % SHARE;
  const int mine_items = nitems > part ? (nitems - part + SHARE - 1) / SHARE : 0;
  const int total = mine_items * nchunks;
  const size_t bstride = (size_t)Nout * K;
  // ---- stages every sorted row, straight into LDS (1 KB per instruction: half a row of 1024)
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)xs;
  auto stage_rows = [&]() {
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(act), 0, (int)((size_t)M * K * 2), 0x00020000);
    const int pieces = K / 512;   // 1 KB pieces per row
    for (int j = wave; j < M * pieces; j += DC_WAVES) {
      const int r = j / pieces, c = j - r * pieces;
      const unsigned src = ((unsigned)r * (unsigned)K + (unsigned)c * 512u) * 2u;
      const unsigned dst = __builtin_amdgcn_readfirstlane(lds_base + (unsigned)(r * RS + c * 512) * 2u);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                   :: "s"(dst), "v"(src + (unsigned)lane * 16u), "s"(arsrc), "s"(0u) : "memory", "m0");
    }
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int j = tid; j < (nrows_lds - M) * (K / 8); j += DC_THREADS)
      *reinterpret_cast<half8_t*>(xs + (size_t)(M + j / (K / 8)) * RS + (j % (K / 8)) * 8) = zero8;
  };
  bool staged = false;

  for (int ub = blockIdx.x; ub * DC_UNITS < units; ub += gridDim.x) {
    const int u = ub * DC_UNITS + us;
    const bool live = u < units;
    const int rot = (u * 5) % nsteps;
    const unsigned lane_off = (((unsigned)(u * UNIT_COLS + sub)) * (unsigned)K + (unsigned)klane) * 2u;
    Chunk<CH> buf[DC_DEPTH];
    auto issue = [&](Chunk<CH>& c, int i) {
      const int it = i / nchunks, ch = i - it * nchunks;
      const int e = __builtin_amdgcn_readfirstlane(item_e[part + it * SHARE]);
      const __amdgpu_buffer_rsrc_t rsrc =
          __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(B + (size_t)e * bstride), 0, (int)(bstride * 2), 0x00020000);
#pragma unroll
      for (int s = 0; s < CH; ++s) {
        const int at = ch * CH + s + rot;
        const int kk = (at - (at >= nsteps ? nsteps : 0)) * STEP_K;
        c.w[s] = load_stream(rsrc, lane_off, (unsigned)kk * 2u);
      }
    };
    float4_t acc[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) acc[q] = float4_t{0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const Chunk<CH>& c, int i) {
      const int it = i / nchunks, ch = i - it * nchunks;
      const int r0 = __builtin_amdgcn_readfirstlane(item_r[part + it * SHARE]);
      const half_t* xlane = xs + (size_t)(r0 + sub) * RS + klane;
#pragma unroll
      for (int s = 0; s < CH; ++s) {
        const int at = ch * CH + s + rot;
        const int kk = (at - (at >= nsteps ? nsteps : 0)) * STEP_K;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const half8_t x = *reinterpret_cast<const half8_t*>(xlane + q * QUAD * RS + kk);
          acc[q] = __builtin_amdgcn_mfma_f32_4x4x4f16(lo4(c.w[s]), lo4(x), acc[q], 0, 0, 0);
          acc[q] = __builtin_amdgcn_mfma_f32_4x4x4f16(hi4(c.w[s]), hi4(x), acc[q], 0, 0, 0);
        }
      }
      if (ch != nchunks - 1) return;
      // the pass is through K: sum the 16 K-slices; lane j < 4 then holds the unit's 4 columns of row r0 + 4q + j
      const int e = __builtin_amdgcn_readfirstlane(item_e[part + it * SHARE]);
      const int last = min(__builtin_amdgcn_readfirstlane(offs[e + 1]), r0 + 4 * NQ);
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        float4_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = sum_blocks(acc[q][j]);
        acc[q] = float4_t{0.f, 0.f, 0.f, 0.f};
        const int r = r0 + q * QUAD + lane;
        if (lane < QUAD && r < last) {
          const float scale = wt[r];
          float4_t o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = (float)(half_t)((float)(half_t)v[j] * scale);
          *reinterpret_cast<float4_t*>(sval + ((size_t)us * DC_MAX_ROWS + r) * 4) = o;
        }
      }
    };
    if (live) {
#pragma unroll
      for (int b = 0; b < DC_DEPTH; ++b)
        if (b < total) issue(buf[b], b);
    }
    if (!staged) {
      // The sorted rows go into LDS behind the first loads of weights, so that the two latencies
      // overlap; vmcnt(0) because the compiler does not know of these loads (the weights asked
      // for above are older and have landed by then too).
      stage_rows();
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      staged = true;
    }
    if (live) {
      for (int i0 = 0; i0 < total; i0 += DC_DEPTH) {
#pragma unroll
        for (int b = 0; b < DC_DEPTH; ++b) {
          const int i = i0 + b;
          if (i < total) {
            compute(buf[b], i);
            if (i + DC_DEPTH < total) issue(buf[b], i + DC_DEPTH);
          }
        }
      }
    }
    __syncthreads();
    // ---- combine: thread (unit, token, column) adds the token's rows in row order
    if (tid < DC_UNITS * N * 4) {
      const int cu = tid / (N * 4), t = (tid / 4) % N, j = tid & 3;
      const int col = (ub * DC_UNITS + cu) * UNIT_COLS + j;
      float sum = 0.f;
      for (int r = 0; r < rows_end; ++r)
        if (tok[r] == t) sum += sval[((size_t)cu * DC_MAX_ROWS + r) * 4 + j];
      if (col < Nout) out[(size_t)t * Nout + col] = (half_t)sum;
    }
    __syncthreads();
  }
}
#pragma clang diagnostic pop

}  // namespace

// The gate/up projection (SwiGLU) of a decode step straight from the routing: sort_by_expert of
// at most 64 choices happens inside the launch, whose first workgroup also writes the sort's
// five results for the launches behind it. Same `act` as sy_sort_by_expert followed by
// sy_grouped_gemv, bit for bit.
extern "C" SY_API int sy_grouped_gemv_sorting(const void* h, const int32_t* idx, const void* w, int N, int k, const void* gate_up,
                                              int E, int I, int H, int32_t* counts, int32_t* offsets, int32_t* token,
                                              void* wsorted, int32_t* pos_of, void* act, void* stream) {
  SY_REQUIRE(sy_gemv_sorts(N, k, E, H), "grouped_gemv_sorting: N = %d, k = %d, E = %d, H = %d", N, k, E, H);
  SY_REQUIRE((long)2 * I * H * 2 < (1l << 31) && I >= 1, "grouped_gemv_sorting: an expert's matrix must stay under 2 GiB");
  SY_REQUIRE(h && idx && w && gate_up && counts && offsets && token && wsorted && pos_of && act, "grouped_gemv_sorting: null pointer");
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const SortHere sort{idx, (const half_t*)w, N * k, k, nbits, counts, offsets, token, (half_t*)wsorted, pos_of};
  return launch_gemv(h, nullptr, gate_up, nullptr, E, N * k, N, I, H, 1, nullptr, act, (hipStream_t)stream, &sort);
}

// Whether sy_gemv_down_combine takes this shape.
bool sy_gemv_combines(int N, int k, int E, int H, int I) {
  const long M = (long)N * k;
  return N >= 1 && N <= DC_MAX_TOKENS && k >= 1 && M <= DC_MAX_ROWS && E >= 1 && E <= DC_MAX_E && I % (CH_SHORT * STEP_K) == 0 &&
         I >= CH_SHORT * STEP_K && H % UNIT_COLS == 0 && H >= UNIT_COLS && dc_lds_bytes((int)M, I, E) <= 160 * 1024 &&
         (long)H * I * 2 < (1l << 31);
}

// The down projection and combine of a decode step in one launch: act f16 [M, I] sorted rows,
// down f16 [E, H, I], the sort's offsets / token / wsorted -> out f16 [N, H], with the bits of
// sy_grouped_gemv (no scale) followed by the combine that applies the router weights.
int sy_gemv_down_combine(const void* act, const void* down, const int32_t* offsets, const int32_t* token, const void* wsorted,
                         int N, int k, int E, int H, int I, void* out, void* stream) {
  SY_REQUIRE(sy_gemv_combines(N, k, E, H, I), "gemv_down_combine: N = %d, k = %d, E = %d, H = %d, I = %d", N, k, E, H, I);
  SY_REQUIRE(act && down && offsets && token && wsorted && out, "gemv_down_combine: null pointer");
  const int M = N * k;
  const size_t lds = dc_lds_bytes(M, I, E);
  const int units = H / UNIT_COLS;
  int grid = (units + DC_UNITS - 1) / DC_UNITS;
  const int cus = sy_compute_units();
  grid = grid > cus ? cus : grid;
  void (*kern)(const half_t*, const half_t*, const int*, const int*, const half_t*, int, int, int, int, int, half_t*) =
      gemv_down_combine_kernel<1>;   // at most 4 tokens: one quad of rows per expert (more only if an id repeats)
  if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return sy_fail(SY_ERR_LAUNCH, "gemv_down_combine: cannot reserve %zu bytes of LDS", lds);
  kern<<<grid, DC_THREADS, lds, (hipStream_t)stream>>>((const half_t*)act, (const half_t*)down, offsets, token,
                                                      (const half_t*)wsorted, E, H, I, N, M, (half_t*)out);
  return sy_check_launch("gemv_down_combine");
}

// Whether sy_grouped_gemv_sorting takes this shape: one choice per lane of a wavefront.
bool sy_gemv_sorts(int N, int k, int E, int H) {
  return N >= 1 && k >= 1 && (long)N * k <= SORT_HERE_MAX && E >= 1 && E <= 128 && k <= E && H >= 8 && H % 8 == 0 && H <= 4096;
}

extern "C" SY_API int sy_grouped_gemv(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets,
                                      int E, int rows, int max_rows_hint, int Nout, int K, int swiglu,
                                      const void* scale, void* C, void* stream) {
  SY_REQUIRE(rows >= 0 && E >= 1 && E <= MAX_E && Nout >= 1, "grouped_gemv: rows = %d, E = %d (at most %d), Nout = %d",
             rows, E, MAX_E, Nout);
  SY_REQUIRE(K >= 8 && K % 8 == 0 && K <= 4096, "grouped_gemv: K must be a multiple of 8 up to 4096 (got %d)", K);
  SY_REQUIRE((long)Nout * K * (swiglu ? 4 : 2) < (1l << 31), "grouped_gemv: an expert's matrix must stay under 2 GiB");
  SY_REQUIRE(!(swiglu && scale), "grouped_gemv: swiglu and scale are not combined");
  if (rows == 0) return SY_OK;
  SY_REQUIRE(A && B && offsets && C, "grouped_gemv: null pointer");
  return launch_gemv(A, a_rows, B, offsets, E, rows, max_rows_hint, Nout, K, swiglu, scale, C, (hipStream_t)stream);
}
