// grouped_gemm: the prefill path. Every expert's slice of the sorted rows goes through that
// expert's weights on fp16 MFMA tiles, all experts in one launch. Three tiles, chosen by the
// host from the mean rows per expert: 64 or 128 rows (gemm_kernel, below) while the launch is
// mostly a stream over the weights, 256 rows (gemm_stream_kernel, further down) once it is
// bound by the MFMAs and by what a compute unit can pull through its L1.
//
// gemm_kernel. Tile: 64*MI rows x 256 weight rows (MI = 1 or 2), K in slices of 64, 4 wavefronts, each computing
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
// computes meanwhile. The weights are loaded non-temporal: in this regime a launch is a stream
// over them (at most a few row tiles share a column tile's weights, and those run side by
// side), and without the hint the same loads run 10 to 13 % slower at 24 to 768 tokens (gate/up
// 90.2 -> 80.8 us at 64 tokens, which is 6.6 TB/s; down 48.7 -> 42.6). The rows, which every
// column tile of an expert reads again, stay cached. LDS rows are padded to 144 bytes so that the 128-bit operand reads of
// 16 consecutive lanes fall in distinct banks.
//
// The map from a workgroup to its tile is rebuilt on the device from `offsets` (find_tile), so
// the host needs neither the reference's tile_offsets tensor nor a device-to-host read.
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

// Inclusive prefix sum over the lanes of a wavefront, on DPP: shifts inside each row of 16 lanes,
// then lane 15 of a row broadcast into the next row and lane 31 into the upper half. Six adds and
// no trip through the LDS crossbar (a scan of shuffles is six dependent ds_bpermute, about 700
// cycles, and the tile list of the stream kernel scans once per tile height).
__device__ __forceinline__ int wave_inclusive_scan(int v, int /*lane*/) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
  return v;
}

// Which tile this workgroup computes. An expert with n rows gets ceil(n / BM) row tiles of equal
// height (a multiple of 32, the last one takes what is left): a short remainder tile would
// stream the expert's weights again for a handful of rows, equal tiles all carry enough MFMA
// work to cover their loads, and no 32-row block is computed that a BM-high tiling would not
// compute. The row tiles of all experts are laid end to end, each followed by its column
// tiles, and the list is cut into 8 equal runs, one per XCD (workgroups are dealt round-robin
// to the XCDs), so that neighbours, which share rows or weights, meet in one L2 and every XCD
// gets the same share whatever the routing. The first wavefront rebuilds the list from
// `offsets` with two scans; the grid is sized for the worst case and surplus workgroups leave
// at once.
// Returns false for a surplus workgroup, else the expert, the tile's first row and the row
// after its last; must be called by every thread of the workgroup.
template <int BM>
__device__ __forceinline__ bool find_tile(const int* __restrict__ offsets, int E, int ncol_tiles, int* s_tile,
                                          int& e, int& row0, int& row_end, int& col_tile) {
  const int tid = threadIdx.x, lane = tid & 63;
  if (tid == 0) s_tile[0] = -1;
  __syncthreads();
  if (tid < WAVE) {
    int row_tiles = 0;
    for (int e0 = 0; e0 < E; e0 += WAVE) {
      const int x = e0 + lane;
      const int n = x < E ? offsets[x + 1] - offsets[x] : 0;
      row_tiles += (n + BM - 1) / BM;
    }
    row_tiles = __builtin_amdgcn_readlane(wave_inclusive_scan(row_tiles, lane), WAVE - 1);
    const long total = (long)row_tiles * ncol_tiles;
    const long per_xcd = (total + XCDS - 1) / XCDS;
    const long slot = blockIdx.x / XCDS;
    const long logical = (blockIdx.x % XCDS) * per_xcd + slot;
    if (slot < per_xcd && logical < total) {
      const int want = (int)(logical / ncol_tiles);
      int run = 0;
      for (int e0 = 0; e0 < E; e0 += WAVE) {
        const int x = e0 + lane;
        const int first = x < E ? offsets[x] : 0, last = x < E ? offsets[x + 1] : 0;
        const int mine = (last - first + BM - 1) / BM;
        const int inc = wave_inclusive_scan(mine, lane);
        const int lo = run + inc - mine;
        if (want >= lo && want < lo + mine) {
          const int height = ((last - first + mine - 1) / mine + 31) & ~31;
          // inside an expert the row tiles of one column tile follow each other: they stream the
          // same weights, are equally high, and so start and finish together and meet in L2
          const int within = (int)(logical - (long)lo * ncol_tiles);
          const int col = BM == 256 ? within / mine : (int)(logical % ncol_tiles);
          const int rt = BM == 256 ? within - col * mine : want - lo;
          const int begin = first + rt * height;
          s_tile[0] = x;
          s_tile[1] = begin;
          s_tile[2] = min(begin + height, last);
          s_tile[3] = col;
        }
        run += __builtin_amdgcn_readlane(inc, WAVE - 1);
      }
    }
  }
  __syncthreads();
  e = __builtin_amdgcn_readfirstlane(s_tile[0]);
  if (e < 0) return false;
  row0 = __builtin_amdgcn_readfirstlane(s_tile[1]);
  row_end = __builtin_amdgcn_readfirstlane(s_tile[2]);
  col_tile = __builtin_amdgcn_readfirstlane(s_tile[3]);
  return true;
}

template <int MI, bool SWIGLU, bool SCALE>
__global__ void __launch_bounds__(GEMM_THREADS, 2)
gemm_kernel(const half_t* __restrict__ A, const int* __restrict__ a_rows, const half_t* __restrict__ B,
            const int* __restrict__ offsets, int E, int Nout, int K, const half_t* __restrict__ scale,
            half_t* __restrict__ C, int ncol_tiles) {
  constexpr int BM = 64 * MI;  // rows per tile
  __shared__ __attribute__((aligned(16))) half_t lds[(BM + BW) * LDS_LD];
  __shared__ int s_tile[4];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  int e, row0, row_end, col_tile;
  if (!find_tile<BM>(offsets, E, ncol_tiles, s_tile, e, row0, row_end, col_tile)) return;
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
      rb[q] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(brsrc, kok ? ob[q] : OUT_OF_RANGE, k0 * 2, /*nt*/ 2));
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
  // Tiles run through K in step, and weight rows a multiple of 4 KB apart put a whole launch's
  // requests on the same few memory channels at any one time (4.6 against 5.8 TB/s in a
  // streaming probe): then every expert starts at a slice of its own and wraps around. All
  // tiles of an expert share the start, so a row's sum does not depend on the tile it falls
  // in, and tiles that share rows or weights still ask for them at the same time. (With rows
  // 2 KB apart the rotation gains nothing and was measured to cost a little.)
  const int rot = K % 2048 == 0 ? (e * 5) % nk : 0;
  const half_t* as = lds + l32 * LDS_LD + lk;
  const half_t* bs = lds + (BM + l32) * LDS_LD + lk;
  // the K loop for LIVE live row blocks (a compile-time count: the loop body stays branch-free)
  auto k_loop = [&](auto live_blocks) {
    constexpr int LIVE = decltype(live_blocks)::value;
    int next = rot;  // the slice to fetch
    fetch(next * BK);
    for (int kt = 0; kt < nk; ++kt) {
      if (kt) __syncthreads();  // every wavefront is done reading the previous slice
      stash();
      next = next + 1 == nk ? 0 : next + 1;
      if (kt + 1 < nk) fetch(next * BK);  // in flight during this slice's MFMAs
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

// ---------------------------------------------------------------------------------------------
// The tile for many rows per expert: 256 rows x 256 weight rows, 8 wavefronts (2 x 4, each 128
// rows x 64 weight rows), one workgroup per CU, and that workgroup stays: it walks its share of
// the tile list as one stream.
//
// A 128-row tile asks the CU for 48 KB of operands per 1024 MFMA cycles, more than the path
// from L2 delivers, and moving them through registers into LDS costs more LDS write cycles than
// the MFMAs take. This tile halves the bytes per flop and lets the memory pipeline write LDS
// itself (buffer loads with the LDS modifier): no staging registers and no ds_write. Even so a
// full tile's 2 MB of operands take a CU about as long to pull in as its MFMAs take (a loop of
// the loads alone runs at 25 B per clock and CU: 85 thousand cycles against 65 thousand of
// MFMAs), so nothing else may stand in front of either.
//
// All 160 KB of LDS are operand slices of 32 KB: two of the rows, three of the weight rows.
// The rows of a tile are shared by all its column tiles and mostly hit in L2; the weights are
// read from HBM by the first of the few row tiles that share them, and such a load is away for
// longer than the MFMAs of a slice take, so weights are fetched two slices ahead and rows one.
// A slice is four K-steps; the one barrier per slice sits before the last step, where that
// step's operands are already in registers: it publishes slice i + 1 and says that every
// wavefront has read all of slice i, so the MFMAs of the last step run while the first
// operands of slice i + 1 are read and the loads of rows i + 2 and weights i + 3 go out, one
// at a time between the MFMAs, into the buffers that slice i has just left.
//
// The slices of a workgroup's tiles form one sequence: in a tile's last iterations the loads
// that run ahead already belong to the next tile, so its first slices are in LDS when the
// epilogue of this one is done. What a tile launched as a workgroup of its own pays in front of
// an idle MFMA pipe (the lookup in the tile list, the row numbers, the latency of the first
// loads, the launch of the workgroup: 6 to 9 of 55 microseconds) is paid once per launch here.
// A tile's row numbers are read through the scalar cache, whose counter the vector loads in
// flight do not share: those are counted by hand (below) and must never be waited for by a
// load the compiler knows about.
//
// Which tiles a workgroup takes is fixed by its number (no queue, no atomics): the list is
// ordered tallest tile first and dealt back and forth, consecutive places to workgroups of one
// XCD, and when the tiles do not divide evenly the workgroups with one tile fewer get the
// tallest ones (see the kernel).
//
// One such load writes the 64 lanes' 16 bytes to 1 KB of consecutive LDS: 8 unpadded rows of
// 128 bytes. Which 16 bytes of its row a lane fetches is therefore chosen so that the operand
// reads stay free of bank conflicts: chunk c of row r sits at position c ^ ((r >> 1) & 7).
// The compiler is not told about these loads (it would wait for all of them before every LDS
// read), so the waits are written by hand.
constexpr int BIG_BM = 256;
constexpr int BIG_BK = 64;                                        // K per slice
constexpr int BIG_STEPS = BIG_BK / 32;                            // MFMA K-steps per slice
constexpr int BIG_ROW_BYTES = BIG_BK * 2;                         // 128
constexpr int BIG_A_BYTES = BIG_BM * BIG_ROW_BYTES;               // 32 KB: a slice of the rows
constexpr int BIG_B_BYTES = BW * BIG_ROW_BYTES;                   // 32 KB: a slice of the weight rows
constexpr int BIG_A_STAGES = 2, BIG_B_STAGES = 3;                 // all 160 KB of LDS

typedef int int4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int4_t buffer_descriptor(const void* base, unsigned bytes) {
  const uint64_t a = (uint64_t)base;
  int4_t d;
  d[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)a);
  d[1] = __builtin_amdgcn_readfirstlane((int)((unsigned)(a >> 32) & 0xffffu));
  d[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  d[3] = 0x00020000;
  return d;
}

// 16 bytes per lane from buffer offset voffset + soffset to LDS address lds_addr + 16 * lane.
// Only voffset is checked against the size of the buffer. The LDS address travels in m0, which
// the statement declares as clobbered; the compiler reserves m0 and warns about that on principle.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// NT: the load is marked non-temporal (data that the launch reads once).
template <bool NT = false>
__device__ __forceinline__ void load_to_lds(int4_t rsrc, unsigned voffset, unsigned soffset, unsigned lds_addr) {
  // the descriptor, the slice offset and the LDS address are the same in every lane; say so
#pragma unroll
  for (int c = 0; c < 4; ++c) rsrc[c] = __builtin_amdgcn_readfirstlane(rsrc[c]);
  soffset = __builtin_amdgcn_readfirstlane(soffset);
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  if (NT)
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen nt lds"
        :
        : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
        : "memory", "m0");
  else
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen lds"
        :
        : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
        : "memory", "m0");
}
#pragma clang diagnostic pop

typedef int int8v_t __attribute__((ext_vector_type(8)));

// Four runs of 8 consecutive ints through the scalar cache, waited for here.
__device__ __forceinline__ void scalar_load_4x8(const int* p0, const int* p1, const int* p2, const int* p3, int8v_t& a,
                                                int8v_t& b, int8v_t& c, int8v_t& d) {
  asm volatile(
      "s_load_dwordx8 %0, %4, 0x0\n\t"
      "s_load_dwordx8 %1, %5, 0x0\n\t"
      "s_load_dwordx8 %2, %6, 0x0\n\t"
      "s_load_dwordx8 %3, %7, 0x0\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(a), "=&s"(b), "=&s"(c), "=&s"(d)
      : "s"(p0), "s"(p1), "s"(p2), "s"(p3));
}

typedef int int16v_t __attribute__((ext_vector_type(16)));
// scale[first + l] and scale[first + 16 + l] for l = 0..15 (first is the same in the whole
// wavefront): 17 dwords from the dword at or below scale + first through the scalar cache, waited
// for here; a lane picks its two halves. The run is moved up where it would pass the end of the M
// scales (M >= 34); lanes whose row is past the end get whatever is there.
__device__ __forceinline__ void scales_of_rows(const half_t* scale, int M, int first, int l, half_t& lo16, half_t& hi16) {
  const uint64_t want = (uint64_t)(scale + first), end = ((uint64_t)(scale + M) + 3) & ~(uint64_t)3;
  uint64_t from = want & ~(uint64_t)3;
  from = from < end - 68 ? from : end - 68;
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)from), hi = __builtin_amdgcn_readfirstlane((unsigned)(from >> 32));
  from = ((uint64_t)hi << 32) | lo;
  int16v_t words;
  int last;
  asm volatile(
      "s_load_dwordx16 %0, %2, 0x0\n\t"
      "s_load_dword %1, %2, 0x40\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(words), "=&s"(last)
      : "s"((const unsigned*)from));
  auto pick = [&](int h) {
    int word = last;
#pragma unroll
    for (int d = 0; d < 16; ++d) word = (h >> 1) == d ? words[d] : word;
    return __builtin_bit_cast(half_t, (unsigned short)((h & 1) ? (unsigned)word >> 16 : (unsigned)word));
  };
  const int h = (int)((want - from) >> 1) + l;
  lo16 = pick(h);
  hi16 = pick(h + 16);
}

template <int EPL>
struct ExpertTable {
  int first[EPL], count[EPL], tiles[EPL], lo[EPL];  // lane x holds experts x, x + 64, ...
};

struct StreamTile {
  int e, row0, row_end, n0;
  unsigned b_lo, b_hi;   // address of the expert's matrix
  int rot;
  bool valid;
};

// STREAMED: an expert's weights are read by one row tile only (at most 256 rows per expert on
// average), so their loads are marked non-temporal: 1024 tokens 108.8 -> 104.7 us (gate/up) and
// 61.7 -> 54.1 (down), 2048 tokens 157.8 -> 154.6 and 90.5 -> 86.0. With two row tiles per
// column tile (4096 tokens) the second one finds the weights in L2, and the hint costs 3 to 7 %.
template <bool SWIGLU, bool SCALE, int EPL, bool STREAMED>
__global__ void __launch_bounds__(512, 1)
gemm_stream_kernel(const half_t* __restrict__ A, const int* __restrict__ a_rows, const half_t* __restrict__ B,
                   const int* __restrict__ offsets, int E, int M, int Nout, int K, const half_t* __restrict__ scale,
                   half_t* __restrict__ C, int ncol_tiles) {
  constexpr int BM = BIG_BM, WN = 4;
  constexpr int WAVES = 2 * WN, THREADS = WAVES * WAVE;
  constexpr int WB = BW / (16 * WN);   // blocks of 16 weight rows per wavefront
  constexpr int LOADS = BIG_A_BYTES / (THREADS * 16);
  __shared__ __attribute__((aligned(1024))) char lds[BIG_A_STAGES * BIG_A_BYTES + BIG_B_STAGES * BIG_B_BYTES];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  constexpr int COLS = SWIGLU ? BW / 2 : BW;
  const int Nfull = SWIGLU ? 2 * Nout : Nout;
  constexpr unsigned OUT_OF_RANGE = 0x80000000u;
  const int nk = K / BIG_BK;

  // ---- the tile list: per expert ceil(n / 256) row tiles of equal height, each with its column
  // tiles (the row tiles of one column tile adjacent); every wavefront keeps the table in registers
  ExpertTable<EPL> tb;
  int cls[EPL];   // 32-row blocks in one of the expert's tiles: what a tile costs
#pragma unroll
  for (int s = 0; s < EPL; ++s) {
    const int x = s * WAVE + lane;
    const int f = x < E ? offsets[x] : 0, l = x < E ? offsets[x + 1] : 0;
    tb.first[s] = f;
    tb.count[s] = l - f;
    tb.tiles[s] = (l - f + BM - 1) / BM;
    cls[s] = tb.tiles[s] ? (((l - f + tb.tiles[s] - 1) / tb.tiles[s] + 31) >> 5) : 0;
    tb.lo[s] = 0;
  }
  // The list is ordered by tile height, tallest first (experts of one height in their own order),
  // and dealt to the workgroups back and forth, so that a workgroup with one tile fewer than its
  // neighbour has the taller ones.
  int run = 0;
  for (int c = BM / 32; c >= 1; --c) {
    bool present = false;
#pragma unroll
    for (int s = 0; s < EPL; ++s) present |= __ballot(cls[s] == c) != 0;
    if (!present) continue;
#pragma unroll
    for (int s = 0; s < EPL; ++s) {
      const int mine = cls[s] == c ? tb.tiles[s] * ncol_tiles : 0;
      const int inc = wave_inclusive_scan(mine, lane);
      if (cls[s] == c) tb.lo[s] = run + inc - mine;
      run += __builtin_amdgcn_readlane(inc, WAVE - 1);
    }
  }
  const int total = __builtin_amdgcn_readfirstlane(run);
  // consecutive places of the list go to workgroups of one XCD (workgroups are dealt round-robin
  // to the XCDs): neighbours share rows or weights and meet in that XCD's L2
  const int G = gridDim.x;
  const int place = (blockIdx.x % XCDS) * (G / XCDS) + blockIdx.x / XCDS;
  // With T tiles for G workgroups, T = q * G + rem, rem workgroups must take q + 1 tiles and the
  // other G - rem take q. The latter get the tallest q * (G - rem) tiles of the list, so that four
  // tall tiles stand against five lower ones; inside each group the tiles are dealt back and
  // forth over full rounds, which evens out what is left of the difference in height.
  const int q_tiles = total / G, rem = total - q_tiles * G;
  const int n_short = rem ? G - rem : 0;                 // workgroups with q tiles
  const bool is_short = place < n_short;
  const int group = is_short ? n_short : G - n_short, seat = is_short ? place : place - n_short;
  const int group_first = is_short ? 0 : q_tiles * n_short, group_rounds = is_short || !rem ? q_tiles : q_tiles + 1;
  auto logical_of = [&](int r) {
    return r < group_rounds ? group_first + r * group + ((r & 1) ? group - 1 - seat : seat) : total;
  };
  const int list_end = total;
  const int4_t arsrc = buffer_descriptor(A, 0x7fffffffu);

  // per-lane offsets of the tile being loaded; the tile being computed keeps what its epilogue needs
  auto lookup = [&](int logical, StreamTile& t, unsigned (&oa)[LOADS], unsigned (&ob)[LOADS]) {
    t.valid = logical < list_end;
    int e = 0, first = 0, count = 0, tiles = 1, lo = 0;
    if (t.valid) {
#pragma unroll
      for (int s = 0; s < EPL; ++s) {
        const uint64_t hit = __ballot(logical >= tb.lo[s] && logical < tb.lo[s] + tb.tiles[s] * ncol_tiles);
        if (hit) {
          const int src = __builtin_ctzll(hit);
          e = s * WAVE + src;
          first = __builtin_amdgcn_readlane(tb.first[s], src);
          count = __builtin_amdgcn_readlane(tb.count[s], src);
          tiles = __builtin_amdgcn_readlane(tb.tiles[s], src);
          lo = __builtin_amdgcn_readlane(tb.lo[s], src);
        }
      }
    }
    const int within = logical - lo;
    const int col = within / tiles, rt = within - col * tiles;
    const int height = ((count + tiles - 1) / tiles + 31) & ~31;
    t.e = e;
    t.row0 = first + rt * height;
    t.row_end = t.valid ? min(t.row0 + height, first + count) : t.row0;
    t.n0 = col * COLS;
    const uint64_t be = (uint64_t)(B + (size_t)e * Nfull * K);
    t.b_lo = (unsigned)be;
    t.b_hi = (unsigned)(be >> 32) & 0xffffu;
    t.rot = K % 2048 == 0 ? (e * 5) % nk : 0;
    const int nrows = t.row_end - t.row0;
    // Row numbers come through the scalar path (its own counter: the vector loads in flight are
    // counted by hand and must not be waited for here), the 8 rows of a load in one request and
    // the tile's four requests in flight together. At the very end of the list the 8 are taken
    // from further up and a lane picks its own from there.
    int8v_t numbers[LOADS];
    int mine[LOADS];
    if (a_rows) {
      static_assert(LOADS == 4, "one request per load of the tile");
      const int* from[LOADS];
#pragma unroll
      for (int q = 0; q < LOADS; ++q) {
        const int want = t.row0 + 8 * (WAVES * q + wave);
        const int first = __builtin_amdgcn_readfirstlane(max(0, min(want, M - 8)));
        from[q] = a_rows + first;
        mine[q] = (lane >> 3) + (want - first);
      }
      scalar_load_4x8(from[0], from[1], from[2], from[3], numbers[0], numbers[1], numbers[2], numbers[3]);
    }
#pragma unroll
    for (int q = 0; q < LOADS; ++q) {
      const int rbase = 8 * (WAVES * q + wave);     // the 8 rows this load brings
      const int r = rbase + (lane >> 3);
      const unsigned chunk = (unsigned)((lane & 7) ^ ((r >> 1) & 7));
      int src = t.row0 + r;
      if (a_rows) {
        int picked = 0;
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) picked = mine[q] == jj ? numbers[q][jj] : picked;
        src = picked;
      }
      oa[q] = r < nrows ? ((unsigned)src * (unsigned)K + chunk * 8u) * 2u : OUT_OF_RANGE;
      int wr, colw;
      if (SWIGLU) {
        colw = t.n0 + (r & (COLS - 1));
        wr = r < COLS ? colw : Nout + colw;
      } else {
        colw = t.n0 + r;
        wr = colw;
      }
      ob[q] = (t.valid && colw < Nout) ? ((unsigned)wr * (unsigned)K + chunk * 8u) * 2u : OUT_OF_RANGE;
    }
  };

  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds;
  const unsigned wave_base = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);
  const unsigned b_bytes = (unsigned)((size_t)Nfull * K * 2);

  StreamTile cur, nxt;
  unsigned oa_c[LOADS], ob_c[LOADS], oa_n[LOADS], ob_n[LOADS];
  lookup(logical_of(0), cur, oa_c, ob_c);
  if (!cur.valid) return;
  nxt = cur;   // until the second tile is known, nothing of the stream refers to it
#pragma unroll
  for (int q = 0; q < LOADS; ++q) {
    oa_n[q] = oa_c[q];
    ob_n[q] = ob_c[q];
  }
  int round = 1;

  // load q of stream slice p (counted from the current tile's first slice; p >= nk is the next tile's)
  auto issue_rows = [&](int p, int stage, int q) {
    const bool later = p >= nk;
    const int rot_c = cur.rot, rot_n = nxt.rot;
    int at = later ? p - nk + rot_n : p + rot_c;
    at = at >= nk ? at - nk : at;
    const unsigned vc = oa_c[q], vn = oa_n[q];
    load_to_lds(arsrc, later ? vn : vc, (unsigned)at * (BIG_BK * 2), wave_base + stage * BIG_A_BYTES + q * (WAVES * 1024));
  };
  auto issue_weights = [&](int p, int stage, int q) {
    const bool later = p >= nk;
    const int rot_c = cur.rot, rot_n = nxt.rot;
    int at = later ? p - nk + rot_n : p + rot_c;
    at = at >= nk ? at - nk : at;
    const unsigned vc = ob_c[q], vn = ob_n[q];
    const unsigned lo_c = cur.b_lo, lo_n = nxt.b_lo, hi_c = cur.b_hi, hi_n = nxt.b_hi;
    int4_t rsrc;
    rsrc[0] = (int)(later ? lo_n : lo_c);
    rsrc[1] = (int)(later ? hi_n : hi_c);
    rsrc[2] = (int)b_bytes;
    rsrc[3] = 0x00020000;
    load_to_lds<STREAMED>(rsrc, later ? vn : vc, (unsigned)at * (BIG_BK * 2),
                          wave_base + BIG_A_STAGES * BIG_A_BYTES + stage * BIG_B_BYTES + q * (WAVES * 1024));
  };

  const int wm = wave / WN, wn = wave % WN;
  // v_mfma_f32_16x16x32_f16: a lane gives 8 consecutive K of row (lane & 15), the four groups of
  // 16 lanes cover the 32 K of a step, and ends with 4 consecutive weight rows (output columns),
  // 4 * (lane >> 4) + 0..3, of row (lane & 15). A wavefront's 128 rows x 64 weight rows are 8 x 4
  // such blocks. (On random operands this shape sustains 16 % more flops than 32x32x16 under the
  // chip's power management: 2.0 against 1.72 Pflop/s in a loop of MFMAs alone.)
  const int l16 = lane & 15, lg = lane >> 4;
  int brow[WB];
#pragma unroll
  for (int j = 0; j < WB; ++j)
    brow[j] = SWIGLU ? (j < WB / 2 ? 0 : COLS) + wn * (WB / 2 * 16) + (j % (WB / 2)) * 16 : wn * (WB * 16) + j * 16;
  int koff[BIG_STEPS];
#pragma unroll
  for (int s = 0; s < BIG_STEPS; ++s) koff[s] = (((4 * s + lg) ^ (l16 >> 1)) * 16);
  const char* as = lds + (wm * 32 + l16) * BIG_ROW_BYTES;
  const char* bs = lds + BIG_A_STAGES * BIG_A_BYTES + l16 * BIG_ROW_BYTES;

  // ---- fill the pipe for the first tile: rows 0, weights 0 | rows 1, weights 1 (the first
  // iteration asks for weights 2)
#pragma unroll
  for (int p = 0; p < 2; ++p) {
#pragma unroll
    for (int q = 0; q < LOADS; ++q) issue_rows(p, p, q);
#pragma unroll
    for (int q = 0; q < LOADS; ++q) issue_weights(p, p, q);
  }
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LOADS) : "memory");
  __syncthreads();
  int a_stage = 0, b_stage = 0;  // where the current tile's slice 0 is

  float4_t acc[8][WB];   // [16-row unit ib: rows (2 (ib / 2) + wm) * 32 + (ib % 2) * 16 ..][16 weight rows jb]
  for (;;) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < WB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    // On entry slice 0 of the current tile has landed and every wavefront knows it.
    //
    // A slice is two K-steps of 2 * LIVE units; a unit is the 4 MFMAs of one 16-row block against
    // the wavefront's 4 blocks of weight rows, and a quarter of a slice is LIVE units. The weight
    // operands of a K-step live in registers for the whole step (two sets: the second step's are
    // read in the slice's first quarter, the next slice's first step's in its last, behind the
    // barrier: 249.7 -> 246.6 us against reading them a quarter later). The row operands go through a ring: the read
    // for the unit one quarter ahead goes into the slot that a unit of this quarter has just left
    // (LIVE >= 3; with fewer units the ring has two quarters, so that a read is not issued only
    // one unit before its use). Reads never run more than a quarter ahead, because the barrier
    // before the last quarter is what publishes the next slice and frees this one's buffers.
    // (Skipping 16-row blocks past the tile's end as well, not only 32-row ones, gains 0.4 % at
    // 4096 tokens and loses 4 us on the down projection at 1024: not the MFMAs' time to win.)
    auto k_loop = [&](auto live_blocks) {
      constexpr int LIVE = decltype(live_blocks)::value;
      constexpr int QU = LIVE, NU = 2 * LIVE;          // units per quarter, per K-step
      constexpr int R = LIVE >= 3 ? LIVE : 2 * LIVE;   // slots of the ring
      half8_t xr[R > 0 ? R : 1], wf[2][WB];
      auto read_x = [&](int sa, int g) {   // unit g of a slice (0 .. 4 LIVE - 1) into its slot
        const int s = (g / (NU > 0 ? NU : 1)) & 1, ib = g % (NU > 0 ? NU : 1);
        xr[g % (R > 0 ? R : 1)] =
            *reinterpret_cast<const half8_t*>(as + sa + ((ib >> 1) * 64 + (ib & 1) * 16) * BIG_ROW_BYTES + koff[s]);
      };
      auto read_w = [&](int sb, int s, int j) {
        wf[s][j] = *reinterpret_cast<const half8_t*>(bs + sb + brow[j] * BIG_ROW_BYTES + koff[s]);
      };
      auto mfma = [&](int g, int j) {
        const int s = (g / (NU > 0 ? NU : 1)) & 1, ib = g % (NU > 0 ? NU : 1);
        acc[ib][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[s][j], xr[g % (R > 0 ? R : 1)], acc[ib][j], 0, 0, 0);
      };
      if constexpr (LIVE > 0) {
#pragma unroll
        for (int j = 0; j < WB; ++j) read_w(b_stage * BIG_B_BYTES, 0, j);
#pragma unroll
        for (int u = 0; u < QU; ++u) read_x(a_stage * BIG_A_BYTES, u);
      }
      for (int kt = 0; kt < nk; ++kt) {
        const int a_next = a_stage ^ 1, b_next = b_stage == BIG_B_STAGES - 1 ? 0 : b_stage + 1;
        const int b_free = b_stage == 0 ? BIG_B_STAGES - 1 : b_stage - 1;   // the buffer slice kt - 1 has left
        const int sa = a_stage * BIG_A_BYTES, sb = b_stage * BIG_B_BYTES;
        // A compute unit takes a load of this kind every 25 to 40 cycles, and a wavefront whose
        // load is not taken issues no MFMA either: the eight loads of an iteration are spread over
        // it, the weights (slice kt + 2) one or two after each of the first three quarters, the
        // rows after the barrier, instead of all 64 of the workgroup at once.
#pragma unroll
        for (int q = 0; q < 3; ++q) {
          if constexpr (LIVE > 0) {
#pragma unroll
            for (int u = 0; u < QU; ++u) {
              if (q == 0) {   // the second K-step's weight operands, as early as their registers are free
#pragma unroll
                for (int j = 0; j < WB; ++j)
                  if (j * QU / WB == u) {
                    read_w(sb, 1, j);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                  }
              }
#pragma unroll
              for (int j = 0; j < WB; ++j) mfma(q * QU + u, j);
              read_x(sa, (q + 1) * QU + u);
              if (R == LIVE) {
                __builtin_amdgcn_sched_group_barrier(0x008, WB, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
              } else {
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, WB, 0);
              }
            }
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int l = 0; l < LOADS; ++l)
            if (l * 3 / LOADS == q) issue_weights(kt + 2, b_free, l);
          __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LOADS) : "memory");
        __syncthreads();
        // the last quarter, in LOADS parts with a load of rows (slice kt + 2) behind each; it reads
        // the first operands of the next slice
#pragma unroll
        for (int part = 0; part < LOADS; ++part) {
          if constexpr (LIVE > 0) {
#pragma unroll
            for (int j = 0; j < WB; ++j)
              if (j * LOADS / WB / 2 == part) read_w(b_next * BIG_B_BYTES, 0, j);
            if (R != LIVE) {
#pragma unroll
              for (int u = 0; u < QU; ++u)
                if (4 * u / QU == part) read_x(a_next * BIG_A_BYTES, u);
            }
#pragma unroll
            for (int m = 0; m < QU * WB; ++m)
              if (m * LOADS / (QU * WB) == part) mfma(3 * QU + m / WB, m % WB);
            if (R == LIVE) {
#pragma unroll
              for (int u = 0; u < QU; ++u)
                if ((WB * u + WB - 1) * LOADS / (QU * WB) == part) read_x(a_next * BIG_A_BYTES, u);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          issue_rows(kt + 2, a_stage, part);
          __builtin_amdgcn_sched_barrier(0);
        }
        a_stage = a_next;
        b_stage = b_next;
        // The tile after this one is looked up here, where the MFMAs of the other wavefront of the
        // SIMD cover it; its offsets are first needed two iterations before this tile ends.
        if (kt == 0) lookup(logical_of(round++), nxt, oa_n, ob_n);
      }
    };
    const int nrows = cur.row_end - cur.row0;
    const int live = ((nrows + 31) / 32 + 1 - wm) / 2;
    switch (live) {
      case 4: k_loop(std::integral_constant<int, 4>{}); break;
      case 3: k_loop(std::integral_constant<int, 3>{}); break;
      case 2: k_loop(std::integral_constant<int, 2>{}); break;
      case 1: k_loop(std::integral_constant<int, 1>{}); break;
      default: k_loop(std::integral_constant<int, 0>{}); break;
    }
    // ---- epilogue. A lane holds 4 consecutive columns (8 bytes as f16) of its row in each of the
    // wavefront's blocks of 16 columns, and the lane 16 further on the next 4. Two neighbouring
    // blocks swap halves between those lanes (v_permlane16_swap), after which every lane holds 16
    // consecutive bytes and a store instruction writes 64 consecutive bytes of each of 16 rows.
    // No LDS is involved, so the stream's loads run on into the next tile meanwhile.
    {
      const int cofs = (lg & 1) * 16 + (lg >> 1) * 8;   // where a lane's 8 columns start after the swap
      auto swap_halves = [&](half4_t a, half4_t b) -> half8_t {
        typedef unsigned u2_t __attribute__((ext_vector_type(2)));
        const u2_t ua = __builtin_bit_cast(u2_t, a), ub = __builtin_bit_cast(u2_t, b);
        const auto lo = __builtin_amdgcn_permlane16_swap(ua[0], ub[0], false, false);
        const auto hi = __builtin_amdgcn_permlane16_swap(ua[1], ub[1], false, false);
        // lane group 0: a of groups 0 and 1 (columns 0..7 of the first block); group 1: b of groups
        // 0 and 1 (columns 0..7 of the second block); groups 2 and 3 the same for columns 8..15
        typedef unsigned u4_t __attribute__((ext_vector_type(4)));
        const u4_t v = {lo[0], hi[0], lo[1], hi[1]};
        return __builtin_bit_cast(half8_t, v);
      };
      auto blocks = [&](auto whole_columns) {
        constexpr bool WHOLE = decltype(whole_columns)::value;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int rblock = cur.row0 + (2 * i + wm) * 32;
          if (rblock >= cur.row_end) continue;   // the same for the whole wavefront
          // the block's 32 scales come through the scalar cache: a vector load here would have to be
          // waited for, and with it every load of the stream that is in flight and every store so far
          half_t sc[2] = {(half_t)1.f, (half_t)1.f};
          if (SCALE) scales_of_rows(scale, M, rblock, l16, sc[0], sc[1]);
#pragma unroll
          for (int hb = 0; hb < 2; ++hb) {
            const int ib = 2 * i + hb, row = rblock + hb * 16 + l16;
            if (rblock + hb * 16 >= cur.row_end) continue;
            if constexpr (SWIGLU) {
              const half8_t v = swap_halves(swiglu_f16x4(acc[ib][0], acc[ib][2]), swiglu_f16x4(acc[ib][1], acc[ib][3]));
              const int c0 = cur.n0 + wn * 32 + cofs;
              if (row < cur.row_end) {
                half_t* dst = C + (size_t)row * Nout + c0;
                if (WHOLE) {
                  *reinterpret_cast<half8_t*>(dst) = v;
                } else {
#pragma unroll
                  for (int r = 0; r < 8; ++r)
                    if (c0 + r < Nout) dst[r] = v[r];
                }
              }
            } else {
              // The wavefront's 64 columns of a row are one 128-byte line, held as two 16-byte pieces
              // in each of four lanes. Rows n and n + 8 of the unit trade halves (a rotation by 8
              // inside each row of 16 lanes), so that 8 lanes hold a whole line and a store
              // instruction writes 8 whole lines: rows 0..7 of the unit, then rows 8..15.
              half4_t o[WB];
#pragma unroll
              for (int j = 0; j < WB; ++j) {
                o[j] = __builtin_convertvector(acc[ib][j], half4_t);   // two packed conversions
                if (SCALE) {
                  // the product of two fp16 numbers is exact in fp32, so the fp16 multiply rounds as
                  // (half)((float)o * (float)scale) does
                  const half4_t sc4 = {sc[hb], sc[hb], sc[hb], sc[hb]};
                  o[j] = o[j] * sc4;
                }
              }
              typedef int i4_t __attribute__((ext_vector_type(4)));
              const i4_t v0 = __builtin_bit_cast(i4_t, swap_halves(o[0], o[1]));   // columns 0..31
              const i4_t v1 = __builtin_bit_cast(i4_t, swap_halves(o[2], o[3]));   // columns 32..63
              const bool low = l16 < 8;
              i4_t got;
#pragma unroll
              for (int d = 0; d < 4; ++d) got[d] = dpp_row_ror<8>(low ? v1[d] : v0[d]);
              const int c0 = cur.n0 + wn * 64 + (low ? 0 : 32) + cofs;
#pragma unroll
              for (int half = 0; half < 2; ++half) {
                i4_t vi;
#pragma unroll
                for (int d = 0; d < 4; ++d) vi[d] = half == 0 ? (low ? v0[d] : got[d]) : (low ? got[d] : v1[d]);
                const half8_t v = __builtin_bit_cast(half8_t, vi);
                const int r = rblock + hb * 16 + half * 8 + (l16 & 7);
                if (r < cur.row_end) {
                  half_t* dst = C + (size_t)r * Nout + c0;
                  if (WHOLE) {
                    // whole lines, stored the plain way: the combine behind this launch reads them,
                    // and finds some still cached (down 148.0 -> 146.7 us and combine 28.8 -> 27.0
                    // at 4096 tokens against non-temporal stores)
                    *reinterpret_cast<half8_t*>(dst) = v;
                  } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                      if (c0 + e < Nout) dst[e] = v[e];
                  }
                }
              }
            }
          }
        }
      };
      if ((Nout & 7) == 0 && cur.n0 + COLS <= Nout) blocks(std::true_type{});
      else blocks(std::false_type{});
    }
    if (!nxt.valid) break;
    cur = nxt;
#pragma unroll
    for (int q = 0; q < LOADS; ++q) {
      oa_c[q] = oa_n[q];
      ob_c[q] = ob_n[q];
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS after this workgroup has given it back
}

template <int EPL>
int launch_gemm_stream(const half_t* a, const int32_t* a_rows, const half_t* b, const int32_t* offsets, int E, int rows,
                       int Nout, int K, int swiglu, const half_t* s, half_t* c, hipStream_t st) {
  const int cols = swiglu ? BW / 2 : BW;
  const int ncol_tiles = (Nout + cols - 1) / cols;
  const int grid = sy_compute_units() / XCDS * XCDS;
  const bool streamed = (long)rows <= 256l * E;   // one row tile per expert, mostly
#define SY_STREAM_LAUNCH(SW, SC, ST) \
  gemm_stream_kernel<SW, SC, EPL, ST><<<grid, 512, 0, st>>>(a, a_rows, b, offsets, E, rows, Nout, K, SC ? s : nullptr, c, ncol_tiles)
  if (swiglu) { if (streamed) SY_STREAM_LAUNCH(true, false, true); else SY_STREAM_LAUNCH(true, false, false); }
  else if (s) { if (streamed) SY_STREAM_LAUNCH(false, true, true); else SY_STREAM_LAUNCH(false, true, false); }
  else { if (streamed) SY_STREAM_LAUNCH(false, false, true); else SY_STREAM_LAUNCH(false, false, false); }
#undef SY_STREAM_LAUNCH
  return sy_check_launch("grouped_gemm");
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
    gemm_kernel<MI, true, false><<<grid, GEMM_THREADS, 0, st>>>(a, a_rows, b, offsets, E, Nout, K, nullptr, c, ncol_tiles);
  else if (s)
    gemm_kernel<MI, false, true><<<grid, GEMM_THREADS, 0, st>>>(a, a_rows, b, offsets, E, Nout, K, s, c, ncol_tiles);
  else
    gemm_kernel<MI, false, false><<<grid, GEMM_THREADS, 0, st>>>(a, a_rows, b, offsets, E, Nout, K, nullptr, c, ncol_tiles);
  return sy_check_launch("grouped_gemm");
}

}  // namespace

// Rows per tile: 64 while the typical expert fits in one such tile (the launch is then a stream
// over the weights and the smaller tile halves the padded MFMA work), 128 up to that many, else
// 256. Under near-uniform routing an expert's rows scatter around the mean by about its square
// root. Measured on 64 experts, 2048 x 1024: the 256-row tile wins from about 128 rows per
// expert on. Its loads run three slices ahead, into the next tile, so it wants four slices of
// K; its tile table is one or two experts per lane.
int sy_gemm_rows_per_tile(int rows, int E, int K) {
  const int mean = (rows + E - 1) / E;
  int typical = mean;
  while ((typical - mean) * (typical - mean) < 4 * mean) ++typical;
  const bool stream_ok = K % BIG_BK == 0 && K / BIG_BK >= 4 && E <= 2 * WAVE;
  return typical <= 64 ? 64 : (typical <= 128 || !stream_ok) ? 128 : 256;
}

extern "C" SY_API int sy_grouped_gemm(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets, int E,
                               int rows, int Nout, int K, int swiglu, const void* scale, void* C, void* stream) {
  SY_REQUIRE(rows >= 0 && E >= 1 && Nout >= 1, "grouped_gemm: rows = %d, E = %d, Nout = %d", rows, E, Nout);
  SY_REQUIRE(K >= 32 && K % 32 == 0, "grouped_gemm: K must be a multiple of 32 (got %d)", K);
  SY_REQUIRE(!(swiglu && scale), "grouped_gemm: swiglu and scale are not combined");
  SY_REQUIRE((long)Nout * K * (swiglu ? 4 : 2) < (1l << 31), "grouped_gemm: an expert's matrix must stay under 2 GiB");
  SY_REQUIRE(a_rows || (long)rows * K * 2 < (1l << 31), "grouped_gemm: A must stay under 2 GiB (%d rows of %d)", rows, K);
  if (rows == 0) return SY_OK;
  SY_REQUIRE(A && B && offsets && C, "grouped_gemm: null pointer");
  const half_t* a = (const half_t*)A;
  const half_t* b = (const half_t*)B;
  const half_t* s = (const half_t*)scale;
  half_t* c = (half_t*)C;
  const int tile = sy_gemm_rows_per_tile(rows, E, K);
  if (tile == 256 && E <= WAVE) return launch_gemm_stream<1>(a, a_rows, b, offsets, E, rows, Nout, K, swiglu, s, c, (hipStream_t)stream);
  if (tile == 256) return launch_gemm_stream<2>(a, a_rows, b, offsets, E, rows, Nout, K, swiglu, s, c, (hipStream_t)stream);
  if (tile == 64) return launch_gemm<1>(a, a_rows, b, offsets, E, rows, Nout, K, swiglu, s, c, (hipStream_t)stream);
  return launch_gemm<2>(a, a_rows, b, offsets, E, rows, Nout, K, swiglu, s, c, (hipStream_t)stream);
}
