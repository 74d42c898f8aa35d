// grouped_gemm: the prefill path. Every expert's slice of the sorted rows goes through that
// expert's weights on fp16 MFMA tiles, all experts in one launch.
//
// Tile: 64*MI rows x 256 weight rows (MI = 1 or 2), K in slices of 64, 4 wavefronts, each computing
// all of the tile's rows x 64 weight rows as (2*MI) x 2 v_mfma_f32_32x32x16_f16 blocks with fp32
// accumulators. With SwiGLU the 256 weight rows are 128 gate rows and the 128 up rows of the
// same output columns, and a wavefront holds gate and up of the same 32 columns, so the
// activation is applied in registers. Every wavefront sees every row of the tile, so 32-row
// blocks past the end of the expert are skipped by all four: a ragged last tile costs what its
// live blocks cost. Weights are the MFMA M operand and rows the N operand: a lane ends
// up with runs of 4 consecutive output columns of one row and stores them as 8 bytes.
//
// Rows are gathered from the unsorted input inside the kernel (a_rows). A K-slice is 64 wide
// so that every row contributes a whole 128-byte cache line per slice. While the MFMAs
// consume slice i from LDS, the global loads of slice i+1 are in flight into registers; they
// are written to LDS between two barriers, and the second workgroup resident on the CU
// computes meanwhile. LDS rows are padded to 144 bytes so that the 128-bit operand reads of
// 16 consecutive lanes fall in distinct banks.
//
// The row tiles of all experts are laid end to end. The map from a tile to (expert, first
// row) is rebuilt by every workgroup from `offsets` with one wavefront scan, so the host
// needs neither the reference's tile_offsets tensor nor a device-to-host read; the grid is
// sized for the worst case and surplus workgroups leave at once. Workgroups are renumbered
// so that consecutive tiles, which share rows or weights, run on the same XCD and meet in
// its L2.
//
// Replaces grouped_gemm_kernel / grouped_gemm of the reference
// (switchyard/csrc/moe_kernels.cu:159-298); epilogue rounding points as :253-259.
#include <type_traits>

#include "common.h"

namespace {

constexpr int BW = 256;          // weight rows per tile
constexpr int BK = 64;           // K per slice
constexpr int LDS_LD = BK + 8;   // halves per LDS row (144 bytes)
constexpr int GEMM_THREADS = 256;
constexpr int XCDS = 8;

__device__ __forceinline__ half_t swiglu_f16(float gate, float up) {
  const float g = (float)(half_t)gate, u = (float)(half_t)up;
  const float s = (float)(half_t)(g / (1.f + expf(-g)));
  return (half_t)(s * u);
}

template <int MI, bool SWIGLU, bool SCALE>
__global__ void __launch_bounds__(GEMM_THREADS, 2)
gemm_kernel(const half_t* __restrict__ A, const int* __restrict__ a_rows, const half_t* __restrict__ B,
            const int* __restrict__ offsets, int E, int Nout, int K, const half_t* __restrict__ scale,
            half_t* __restrict__ C, int ncol_tiles, int per_xcd) {
  constexpr int BM = 64 * MI;  // rows per tile
  __shared__ __attribute__((aligned(16))) half_t lds[(BM + BW) * LDS_LD];
  __shared__ int s_tile[3];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;

  // consecutive logical tiles on one XCD (workgroups are dealt round-robin to the XCDs)
  const int logical = (blockIdx.x % XCDS) * per_xcd + blockIdx.x / XCDS;
  const int row_tile = logical / ncol_tiles, col_tile = logical % ncol_tiles;

  if (tid == 0) s_tile[0] = -1;
  __syncthreads();
  if (wave == 0) {
    int run = 0;
    for (int e0 = 0; e0 < E; e0 += WAVE) {
      const int e = e0 + lane;
      const int first = e < E ? offsets[e] : 0, last = e < E ? offsets[e + 1] : 0;
      const int tiles = (last - first + BM - 1) / BM;
      int inc = tiles;
      for (int o = 1; o < WAVE; o <<= 1) {
        const int up = __shfl_up(inc, o, WAVE);
        if (lane >= o) inc += up;
      }
      const int lo = run + inc - tiles;
      if (row_tile >= lo && row_tile < lo + tiles) {
        s_tile[0] = e;
        s_tile[1] = first + (row_tile - lo) * BM;
        s_tile[2] = last;
      }
      run += __shfl(inc, WAVE - 1, WAVE);
    }
  }
  __syncthreads();
  const int e = s_tile[0];
  if (e < 0) return;
  const int row0 = s_tile[1], row_end = s_tile[2];
  const int nrows = min(BM, row_end - row0);

  constexpr int COLS = SWIGLU ? BW / 2 : BW;  // output columns per tile
  const int n0 = col_tile * COLS;
  const int Nfull = SWIGLU ? 2 * Nout : Nout;
  const half_t* Be = B + (size_t)e * Nfull * K;

  // ---- loader: thread t moves 16-byte chunk (t & 7) of rows (t >> 3) + 32*q through buffer
  // descriptors: a row that does not exist (past the expert's end, past Nout) or a chunk past K
  // gets an out-of-range offset and reads as 0, so the loop has no branches
  const int lrow = tid >> 3, lch = (tid & 7) * 8;
  constexpr int NA = BM / 32, NB = BW / 32;
  constexpr unsigned OUT_OF_RANGE = 0x80000000u;
  const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(A), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t brsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(Be), 0, (int)((size_t)Nfull * K * 2), 0x00020000);
  unsigned oa[NA], ob[NB];
#pragma unroll
  for (int q = 0; q < NA; ++q) {
    const int r = lrow + 32 * q;
    const int src = r < nrows ? (a_rows ? a_rows[row0 + r] : row0 + r) : 0;
    oa[q] = r < nrows ? ((unsigned)src * (unsigned)K + (unsigned)lch) * 2u : OUT_OF_RANGE;
  }
#pragma unroll
  for (int q = 0; q < NB; ++q) {
    const int br = lrow + 32 * q;
    int wr, col;
    if (SWIGLU) {
      col = n0 + (br & (COLS - 1));
      wr = br < COLS ? col : Nout + col;
    } else {
      col = n0 + br;
      wr = col;
    }
    ob[q] = col < Nout ? ((unsigned)wr * (unsigned)K + (unsigned)lch) * 2u : OUT_OF_RANGE;
  }
  half8_t ra[NA], rb[NB];
  auto fetch = [&](int k0) {
    const bool kok = k0 + lch < K;  // K may end in the middle of the last slice
#pragma unroll
    for (int q = 0; q < NA; ++q)
      ra[q] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(arsrc, kok ? oa[q] : OUT_OF_RANGE, k0 * 2, 0));
#pragma unroll
    for (int q = 0; q < NB; ++q)
      rb[q] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(brsrc, kok ? ob[q] : OUT_OF_RANGE, k0 * 2, 0));
  };
  auto stash = [&]() {
    half_t* as = lds;
    half_t* bs = as + BM * LDS_LD;
#pragma unroll
    for (int q = 0; q < NA; ++q) *reinterpret_cast<half8_t*>(as + (lrow + 32 * q) * LDS_LD + lch) = ra[q];
#pragma unroll
    for (int q = 0; q < NB; ++q) *reinterpret_cast<half8_t*>(bs + (lrow + 32 * q) * LDS_LD + lch) = rb[q];
  };

  // ---- wavefront tile: all of the tile's rows x 64 weight rows (wavefront w owns weight rows
  // brow[0], brow[1]); row blocks past the expert's end are skipped, so a tile costs what its
  // 32-row blocks cost and not what a full tile costs
  const int l32 = lane & 31, lk = (lane >> 5) * 8;
  constexpr int RB = BM / 32;  // 32-row blocks per tile
  int brow[2];
  brow[0] = SWIGLU ? wave * 32 : wave * 64;
  brow[1] = SWIGLU ? COLS + wave * 32 : wave * 64 + 32;

  float16_t acc[RB][2];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = (K + BK - 1) / BK;
  const half_t* as = lds + l32 * LDS_LD + lk;
  const half_t* bs = lds + (BM + l32) * LDS_LD + lk;
  // the K loop for LIVE live row blocks (a compile-time count: the loop body stays branch-free)
  auto k_loop = [&](auto live_blocks) {
    constexpr int LIVE = decltype(live_blocks)::value;
    fetch(0);
    for (int kt = 0; kt < nk; ++kt) {
      if (kt) __syncthreads();  // every wavefront is done reading the previous slice
      stash();
      if (kt + 1 < nk) fetch((kt + 1) * BK);  // in flight during this slice's MFMAs
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < BK; kk += 16) {
        half8_t xf[LIVE], wf[2];
#pragma unroll
        for (int i = 0; i < LIVE; ++i) xf[i] = *reinterpret_cast<const half8_t*>(as + i * 32 * LDS_LD + kk);
#pragma unroll
        for (int j = 0; j < 2; ++j) wf[j] = *reinterpret_cast<const half8_t*>(bs + brow[j] * LDS_LD + kk);
#pragma unroll
        for (int i = 0; i < LIVE; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[j], xf[i], acc[i][j], 0, 0, 0);
      }
    }
  };
  const int live = (nrows + 31) / 32;
  if (RB == 4 && live == 4) k_loop(std::integral_constant<int, RB>{});
  else if (RB == 4 && live == 3) k_loop(std::integral_constant<int, (RB > 3 ? 3 : RB)>{});
  else if (live >= 2) k_loop(std::integral_constant<int, 2>{});
  else k_loop(std::integral_constant<int, 1>{});

  // ---- epilogue: acc element 4*q + r of block (i, j) is row i*32 + l32, column 8*q + 4*(lane/32) + r
  const int chalf = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int row = row0 + i * 32 + l32;
    if (row >= row_end) continue;
    const float sc_row = SCALE ? (float)scale[row] : 1.f;
    half_t* crow = C + (size_t)row * Nout;
    constexpr int NJ = SWIGLU ? 1 : 2;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int cbase = n0 + (SWIGLU ? wave * 32 : wave * 64 + j * 32) + chalf;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int c0 = cbase + 8 * q;
        half4_t o;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float v = acc[i][j][4 * q + r];
          if (SWIGLU) o[r] = swiglu_f16(v, acc[i][1][4 * q + r]);
          else if (SCALE) o[r] = (half_t)((float)(half_t)v * sc_row);
          else o[r] = (half_t)v;
        }
        if (c0 + 3 < Nout && (Nout & 3) == 0) {
          *reinterpret_cast<half4_t*>(crow + c0) = o;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (c0 + r < Nout) crow[c0 + r] = o[r];
        }
      }
    }
  }
}

template <int MI>
int launch_gemm(const half_t* a, const int32_t* a_rows, const half_t* b, const int32_t* offsets, int E, int rows,
                int Nout, int K, int swiglu, const half_t* s, half_t* c, hipStream_t st) {
  constexpr int BM = 64 * MI;
  const int cols = swiglu ? BW / 2 : BW;
  const int ncol_tiles = (Nout + cols - 1) / cols;
  // sum over experts of ceil(count / BM) <= rows / BM + (experts with rows) <= rows / BM + min(E, rows)
  const long max_row_tiles = rows / BM + (E < rows ? E : rows);
  const long total = max_row_tiles * ncol_tiles;
  if (total >= (1l << 31) - XCDS) return sy_fail(SY_ERR_ARG, "grouped_gemm: too many tiles");
  const int per_xcd = (int)((total + XCDS - 1) / XCDS);
  const int grid = per_xcd * XCDS;
  if (swiglu)
    gemm_kernel<MI, true, false><<<grid, GEMM_THREADS, 0, st>>>(a, a_rows, b, offsets, E, Nout, K, nullptr, c, ncol_tiles, per_xcd);
  else if (s)
    gemm_kernel<MI, false, true><<<grid, GEMM_THREADS, 0, st>>>(a, a_rows, b, offsets, E, Nout, K, s, c, ncol_tiles, per_xcd);
  else
    gemm_kernel<MI, false, false><<<grid, GEMM_THREADS, 0, st>>>(a, a_rows, b, offsets, E, Nout, K, nullptr, c, ncol_tiles, per_xcd);
  return sy_check_launch("grouped_gemm");
}

}  // namespace

extern "C" SY_API int sy_grouped_gemm(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets, int E,
                               int rows, int Nout, int K, int swiglu, const void* scale, void* C, void* stream) {
  SY_REQUIRE(rows >= 0 && E >= 1 && Nout >= 1, "grouped_gemm: rows = %d, E = %d, Nout = %d", rows, E, Nout);
  SY_REQUIRE(K >= 32 && K % 32 == 0, "grouped_gemm: K must be a multiple of 32 (got %d)", K);
  SY_REQUIRE(!(swiglu && scale), "grouped_gemm: swiglu and scale are not combined");
  SY_REQUIRE((long)Nout * K * (swiglu ? 4 : 2) < (1l << 31), "grouped_gemm: an expert's matrix must stay under 2 GiB");
  if (rows == 0) return SY_OK;
  SY_REQUIRE(A && B && offsets && C, "grouped_gemm: null pointer");
  // rows per tile: 64 while the typical expert fits in one such tile (the launch is then a
  // stream over the weights and the smaller tile halves the padded MFMA work), else 128. Under
  // near-uniform routing an expert's rows scatter around the mean by about its square root.
  const int mean = (rows + E - 1) / E;
  int typical = mean;
  while ((typical - mean) * (typical - mean) < 4 * mean) ++typical;
  const half_t* a = (const half_t*)A;
  const half_t* b = (const half_t*)B;
  const half_t* s = (const half_t*)scale;
  half_t* c = (half_t*)C;
  if (typical <= 64) return launch_gemm<1>(a, a_rows, b, offsets, E, rows, Nout, K, swiglu, s, c, (hipStream_t)stream);
  return launch_gemm<2>(a, a_rows, b, offsets, E, rows, Nout, K, swiglu, s, c, (hipStream_t)stream);
}
