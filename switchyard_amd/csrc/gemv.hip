// grouped_gemv: the decode path. With a handful of rows per expert the layer is a stream over
// the used experts' weights, so the kernel is built around that stream.
//
// A workgroup of 4 wavefronts owns one expert and a run of 16-column groups of its weight
// matrix. For a column group, lane (n = lane % 16, g = lane / 16) reads 16-byte pieces of
// weight row col0 + n: the wavefronts split K between them in interleaved 32-wide steps, so
// the workgroup as a whole reads 16 consecutive weight rows (one contiguous region of
// 16*K*2 bytes) exactly once, every load 128 bits wide, and the pieces go from the load
// straight into the MFMA operand registers (no LDS staging of weights).
//
// The expert's rows (up to 16 at a time) are the other MFMA operand: lane (n, g) holds row n
// at the same K positions, loaded once per workgroup and kept in registers across all of its
// column groups. v_mfma_f32_16x16x32_f16 then does the 16 rows x 16 columns of dot products
// with fp32 accumulation: weights are the M operand and rows the N operand, so a lane ends
// up with 4 consecutive output columns of one row. The 4 wavefronts' partial sums meet in
// LDS (fixed order: deterministic) and wavefront 0 applies the epilogue and stores.
//
// Experts without rows leave at once; an expert with more than 16 rows takes further passes.
//
// Replaces grouped_gemv_kernel / grouped_gemv of the reference
// (switchyard/csrc/moe_kernels.cu:301-415); epilogue rounding points as :373-378.
#include "common.h"

namespace {

constexpr int GEMV_WAVES = 4;
constexpr int GEMV_THREADS = GEMV_WAVES * WAVE;
constexpr int GEMV_ROWS = 16;   // rows per pass (MFMA N)
constexpr int GEMV_COLS = 16;   // columns per group (MFMA M)
constexpr int GEMV_MAX_KS = 16; // 32-wide K steps a wavefront keeps in registers

__device__ __forceinline__ half8_t load_stream(const half_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(p));
}

__device__ __forceinline__ half_t swiglu_f16(float gate, float up) {
  // the rounding points of the fp16 torch graph: gate and up to f16, silu in fp32 to f16, product to f16
  const float g = (float)(half_t)gate, u = (float)(half_t)up;
  const float s = (float)(half_t)(g / (1.f + expf(-g)));
  return (half_t)(s * u);
}

template <int KS, bool SWIGLU, bool SCALE>
__global__ void __launch_bounds__(GEMV_THREADS)
gemv_kernel(const half_t* __restrict__ A, const int* __restrict__ a_rows, const half_t* __restrict__ B,
            const int* __restrict__ offsets, int Nout, int K, const half_t* __restrict__ scale,
            half_t* __restrict__ C, int groups_per_block) {
  const int e = blockIdx.y;
  const int start = offsets[e], end = offsets[e + 1];
  if (start >= end) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int Nfull = SWIGLU ? 2 * Nout : Nout;
  const half_t* Be = B + (size_t)e * Nfull * K;
  constexpr int NACC = SWIGLU ? 2 : 1;
  __shared__ float4_t part[2][GEMV_WAVES][NACC][WAVE];

  const int ngroups = (Nout + GEMV_COLS - 1) / GEMV_COLS;
  const int cg0 = blockIdx.x * groups_per_block, cg1 = min(cg0 + groups_per_block, ngroups);
  constexpr int SUPER = GEMV_WAVES * KS * 32;  // K covered by one register-resident set of steps
  const int nsuper = (K + SUPER - 1) / SUPER;
  const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  int flip = 0;

  for (int r0 = start; r0 < end; r0 += GEMV_ROWS) {
    const int nr = min(GEMV_ROWS, end - r0);
    const half_t* xrow = nullptr;
    if (n < nr) xrow = A + (size_t)(a_rows ? a_rows[r0 + n] : r0 + n) * K;
    half8_t xf[KS];
    auto load_rows = [&](int sc) {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int kk = sc * SUPER + (s * GEMV_WAVES + wave) * 32 + g * 8;
        xf[s] = (xrow && kk < K) ? *reinterpret_cast<const half8_t*>(xrow + kk) : zero8;
      }
    };
    if (nsuper == 1) load_rows(0);

    for (int cg = cg0; cg < cg1; ++cg) {
      const int col = cg * GEMV_COLS + n;
      const bool colok = col < Nout;
      const half_t* wrow = Be + (size_t)col * K;
      const half_t* urow = Be + (size_t)(Nout + col) * K;
      float4_t accg = {0.f, 0.f, 0.f, 0.f}, accu = {0.f, 0.f, 0.f, 0.f};
      for (int sc = 0; sc < nsuper; ++sc) {
        if (nsuper > 1) load_rows(sc);
        half8_t wg[KS], wu[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const int kk = sc * SUPER + (s * GEMV_WAVES + wave) * 32 + g * 8;
          const bool ok = colok && kk < K;
          wg[s] = ok ? load_stream(wrow + kk) : zero8;
          if (SWIGLU) wu[s] = ok ? load_stream(urow + kk) : zero8;
        }
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          accg = __builtin_amdgcn_mfma_f32_16x16x32_f16(wg[s], xf[s], accg, 0, 0, 0);
          if (SWIGLU) accu = __builtin_amdgcn_mfma_f32_16x16x32_f16(wu[s], xf[s], accu, 0, 0, 0);
        }
      }
      part[flip][wave][0][lane] = accg;
      if (SWIGLU) part[flip][wave][NACC - 1][lane] = accu;
      __syncthreads();
      if (wave == 0 && n < nr) {
        float4_t sg = part[flip][0][0][lane], su = {0.f, 0.f, 0.f, 0.f};
        if (SWIGLU) su = part[flip][0][NACC - 1][lane];
#pragma unroll
        for (int wv = 1; wv < GEMV_WAVES; ++wv) {
          sg += part[flip][wv][0][lane];
          if (SWIGLU) su += part[flip][wv][NACC - 1][lane];
        }
        const int row = r0 + n, c0 = cg * GEMV_COLS + 4 * g;
        const float sc_row = SCALE ? (float)scale[row] : 1.f;
        half4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (SWIGLU) o[i] = swiglu_f16(sg[i], su[i]);
          else if (SCALE) o[i] = (half_t)((float)(half_t)sg[i] * sc_row);
          else o[i] = (half_t)sg[i];
        }
        half_t* dst = C + (size_t)row * Nout + c0;
        if (c0 + 3 < Nout && (Nout & 3) == 0) {
          *reinterpret_cast<half4_t*>(dst) = o;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (c0 + i < Nout) dst[i] = o[i];
        }
      }
      flip ^= 1;
    }
  }
}

template <int KS>
int launch_gemv(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets, int E, int Nout, int K,
                int swiglu, const void* scale, void* C, hipStream_t stream) {
  const int ngroups = (Nout + GEMV_COLS - 1) / GEMV_COLS;
  // about 128 KB of weights per workgroup
  const long group_bytes = (long)GEMV_COLS * K * 2 * (swiglu ? 2 : 1);
  int gpb = (int)((128 * 1024 + group_bytes - 1) / group_bytes);
  gpb = gpb < 1 ? 1 : (gpb > ngroups ? ngroups : gpb);
  const dim3 grid((ngroups + gpb - 1) / gpb, E);
  const half_t* a = (const half_t*)A;
  const half_t* b = (const half_t*)B;
  const half_t* s = (const half_t*)scale;
  half_t* c = (half_t*)C;
  if (swiglu)
    gemv_kernel<KS, true, false><<<grid, GEMV_THREADS, 0, stream>>>(a, a_rows, b, offsets, Nout, K, nullptr, c, gpb);
  else if (s)
    gemv_kernel<KS, false, true><<<grid, GEMV_THREADS, 0, stream>>>(a, a_rows, b, offsets, Nout, K, s, c, gpb);
  else
    gemv_kernel<KS, false, false><<<grid, GEMV_THREADS, 0, stream>>>(a, a_rows, b, offsets, Nout, K, nullptr, c, gpb);
  return sy_check_launch("grouped_gemv");
}

}  // namespace

extern "C" SY_API int sy_grouped_gemv(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets, int E,
                               int rows, int Nout, int K, int swiglu, const void* scale, void* C, void* stream) {
  SY_REQUIRE(rows >= 0 && E >= 1 && E <= 65535 && Nout >= 1, "grouped_gemv: rows = %d, E = %d, Nout = %d", rows, E, Nout);
  SY_REQUIRE(K >= 8 && K % 8 == 0 && K <= 8192, "grouped_gemv: K must be a multiple of 8 up to 8192 (got %d)", K);
  SY_REQUIRE(!(swiglu && scale), "grouped_gemv: swiglu and scale are not combined");
  if (rows == 0) return SY_OK;
  SY_REQUIRE(A && B && offsets && C, "grouped_gemv: null pointer");
  const int per_wave = ((K + 31) / 32 + GEMV_WAVES - 1) / GEMV_WAVES;
  hipStream_t st = (hipStream_t)stream;
  if (per_wave <= 1) return launch_gemv<1>(A, a_rows, B, offsets, E, Nout, K, swiglu, scale, C, st);
  if (per_wave <= 2) return launch_gemv<2>(A, a_rows, B, offsets, E, Nout, K, swiglu, scale, C, st);
  if (per_wave <= 4) return launch_gemv<4>(A, a_rows, B, offsets, E, Nout, K, swiglu, scale, C, st);
  if (per_wave <= 8) return launch_gemv<8>(A, a_rows, B, offsets, E, Nout, K, swiglu, scale, C, st);
  return launch_gemv<GEMV_MAX_KS>(A, a_rows, B, offsets, E, Nout, K, swiglu, scale, C, st);
}
