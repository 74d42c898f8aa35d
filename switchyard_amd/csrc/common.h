// Shared device helpers for the gfx950 MoE kernels: 16-bit float vectors, wavefront-64
// reductions (DPP inside a row of 16 lanes, cross-lane shuffles above that) and the
// error plumbing of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/switchyard_moe.h"

typedef _Float16 half_t;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int WAVE = 64;

// Records a message for sy_last_error() and returns `code`.
int sy_fail(int code, const char* fmt, ...);
// Returns SY_OK, or records the pending HIP launch error and returns SY_ERR_LAUNCH.
int sy_check_launch(const char* what);

// Compute units of the current device (cached per device).
int sy_compute_units();
// sort.hip: the second launch of the sort over many workgroups, for a caller that has left the
// per-piece histograms in the workspace itself (f16 weights, N*k above the one-workgroup limit)
int sy_sort_assign_counted(const int32_t* idx, const void* w, int N, int k, int E, int32_t* counts, int32_t* offsets,
                           int32_t* token, void* wsorted, int32_t* pos_of, void* workspace, void* stream);
// front.hip: router logits + route in one launch; with `hist` also the sort's per-piece histograms
int sy_router_route_counting(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits,
                             int32_t* idx, void* w, void* hist, void* stream);
bool sy_router_route_counts(int N, int k);
// front.hip: whether that launch takes the shape (H a multiple of 512, at most 128 experts, top-8)
bool sy_router_route_shape_ok(int N, int H, int E, int k);
// gemm.hip: rows of the tile that sy_grouped_gemm picks for `rows` sorted rows over E experts (64, 128 or 256)
int sy_gemm_rows_per_tile(int rows, int E, int K);
// decode.hip: router GEMM + route for a few rows (one workgroup per row)
int sy_router_route_rows(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits, int32_t* idx,
                         void* w, void* stream);
// gemv.hip: the gate/up projection of a decode step that sorts its (at most 64) choices itself
bool sy_gemv_sorts(int N, int k, int E, int H);
// gemv.hip: the down projection and combine of a decode step (at most 8 tokens, 64 rows) in one launch
bool sy_gemv_combines(int N, int k, int E, int H, int I);
int sy_gemv_down_combine(const void* act, const void* down, const int32_t* offsets, const int32_t* token, const void* wsorted,
                         int N, int k, int E, int H, int I, void* out, void* stream);
// combine.hip: combine of rows that were left unscaled, times the router weights w [N, k]
int sy_combine_weighted(const void* y, const int32_t* pos_of, const int32_t* idx, const void* w, int N, int k, int H, void* out,
                        void* stream);

#define SY_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return sy_fail(SY_ERR_ARG, __VA_ARGS__); \
  } while (0)

// ---- DPP: rotate right by N inside each row of 16 lanes (row_ror:N = 0x120 + N).
template <int N>
__device__ __forceinline__ int dpp_row_ror(int v) {
  return __builtin_amdgcn_update_dpp(0, v, 0x120 + N, 0xf, 0xf, false);
}
template <int N>
__device__ __forceinline__ float dpp_row_ror(float v) {
  return __int_as_float(dpp_row_ror<N>(__float_as_int(v)));
}

// All-reduce inside each row of 16 lanes with DPP rotations: every lane of a row ends with the
// same bits, because each step combines two values that are identical across partner lanes.
template <typename T, typename Op>
__device__ __forceinline__ T row_allreduce(T v, Op op) {
  v = op(v, dpp_row_ror<8>(v));
  v = op(v, dpp_row_ror<4>(v));
  v = op(v, dpp_row_ror<2>(v));
  v = op(v, dpp_row_ror<1>(v));
  return v;
}

__device__ __forceinline__ float read_lane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ int read_lane(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }

// All-reduce over the 64 lanes of a wavefront: DPP inside the four rows, then the four row
// results are read into scalar registers and combined in a fixed order, so the result is
// wave-uniform and needs no trip through the LDS crossbar.
template <typename T, typename Op>
__device__ __forceinline__ T wave_allreduce(T v, Op op) {
  v = row_allreduce(v, op);
  return op(op(read_lane(v, 0), read_lane(v, 16)), op(read_lane(v, 32), read_lane(v, 48)));
}

__device__ __forceinline__ float wave_max(float v) {
  return wave_allreduce(v, [](float a, float b) { return fmaxf(a, b); });
}
__device__ __forceinline__ float wave_sum(float v) {
  return wave_allreduce(v, [](float a, float b) { return a + b; });
}

// SwiGLU with the reference's rounding points: gate and up are rounded to fp16, silu(gate) is
// rounded to fp16, and so is the product (F.silu(gate) * up on fp16 tensors). The sigmoid uses
// the hardware's exp2 and reciprocal (about 1 ulp each in fp32, far below the fp16 rounding);
// exp2 overflows to +inf for very negative gates and the result is then -0, the right limit.
__device__ __forceinline__ half_t swiglu_f16(float gate, float up) {
  const float g = (float)(half_t)gate, u = (float)(half_t)up;
  const float sig = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
  const float s = (float)(half_t)(g * sig);
  return (half_t)(s * u);
}

// The same for four outputs at a time: the roundings to fp16 pack two values per instruction, and
// the last product is an fp16 multiply (the product of two fp16 numbers is exact in fp32, so it
// rounds as the fp32 product rounded to fp16 does).
__device__ __forceinline__ half4_t swiglu_f16x4(float4_t gate, float4_t up) {
  const half4_t gh = __builtin_convertvector(gate, half4_t), uh = __builtin_convertvector(up, half4_t);
  const float4_t g = __builtin_convertvector(gh, float4_t);
  float4_t s;
#pragma unroll
  for (int r = 0; r < 4; ++r) s[r] = g[r] * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g[r] * -1.4426950408889634f));
  return __builtin_convertvector(s, half4_t) * uh;
}

__device__ __forceinline__ uint64_t lanemask_lt() {
  return (1ull << (threadIdx.x & 63)) - 1ull;
}
