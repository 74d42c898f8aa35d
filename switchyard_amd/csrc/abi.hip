// Error plumbing and version of the C ABI (include/switchyard_moe.h).
#include <stdarg.h>
#include <stdio.h>

#include "common.h"
#include "../../include/switchyard_decode.h"

namespace {
thread_local char g_error[512] = "";
}

int sy_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int sy_check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return SY_OK;
  return sy_fail(SY_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(err));
}

// Compute units of the current device (cached per device id; read-only after the first call).
int sy_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

extern "C" SY_API int sy_version(void) { return 200; }  // 0.2.0: the decode-step entry points

extern "C" SY_API const char* sy_last_error(void) { return g_error; }

// The experts of one layer in one call: (the router's logits,) route and sort, the two
// projections and combine, enqueued back to back. Nothing here that the separate entry points do not do; it exists
// because a host binding pays several microseconds per call, and in front of the first
// projection the GPU waits for exactly those (a layer of 8 tokens called once: 132 us with
// five calls, the kernels themselves 102).
extern "C" SY_API int sy_moe_experts(const void* h, const void* router, void* logits, int N, int E, int k, int norm, const void* gate_up,
                                     const void* down, int H, int I, int mfma_tiles, int one_launch_front, int32_t* idx,
                                     void* w, int32_t* counts, int32_t* offsets, int32_t* token, void* wsorted,
                                     int32_t* pos_of, void* act, void* y, void* out, void* sort_workspace,
                                     size_t sort_workspace_bytes, void* stream) {
  SY_REQUIRE(N >= 0 && H >= 8 && I >= 8, "moe_experts: N = %d, H = %d, I = %d", N, H, I);
  if (N == 0) return SY_OK;
  SY_REQUIRE(h && logits && act && y && out, "moe_experts: null pointer");
  // the projections address the gathered rows of h with 32-bit byte offsets
  SY_REQUIRE((long)N * H * 2 < (1l << 31), "moe_experts: h must stay under 2 GiB (%d rows of %d)", N, H);
  int rc;
  if (router && N > 64 && !sy_router_route_shape_ok(N, H, E, k)) {
    // a width the MFMA front does not take (H not a multiple of 512): the row kernel makes the
    // logits, a workgroup per token, and route and sort are their own launches
    rc = sy_router_logits(h, router, N, H, E, logits, stream);
    if (rc) return rc;
    rc = sy_route(logits, SY_DTYPE_F16, N, E, k, norm, idx, w, stream);
    if (rc) return rc;
    rc = sy_sort_by_expert(idx, w, 2, N, k, E, counts, offsets, token, wsorted, pos_of, sort_workspace, sort_workspace_bytes,
                           stream);
  } else if (router && N > 64) {
    // beyond the decode kernels' range: one launch for the logits and route, which is also the
    // sort's first pass where the sort runs over many workgroups
    SY_REQUIRE(!one_launch_front, "moe_experts: one_launch_front with a router is for at most 64 tokens");
    const bool counted = sy_router_route_counts(N, k) && sort_workspace && sort_workspace_bytes >= sy_sort_workspace_bytes(N, k, E);
    rc = sy_router_route_counting(h, router, N, H, E, k, norm, logits, idx, w, counted ? sort_workspace : nullptr, stream);
    if (rc) return rc;
    rc = counted ? sy_sort_assign_counted(idx, w, N, k, E, counts, offsets, token, wsorted, pos_of, sort_workspace, stream)
                 : sy_sort_by_expert(idx, w, 2, N, k, E, counts, offsets, token, wsorted, pos_of, sort_workspace,
                                     sort_workspace_bytes, stream);
  } else if (router && !mfma_tiles && sy_gemv_sorts(N, k, E, H)) {
    // a decode step of at most 64 choices: logits and route in one launch, and the first
    // projection sorts for itself
    rc = sy_router_route_rows(h, router, N, H, E, k, norm, logits, idx, w, stream);
    if (rc) return rc;
    return sy_experts_routed(h, N, E, k, gate_up, down, H, I, 0, idx, w, counts, offsets, token, wsorted, pos_of, act, y, out,
                             sort_workspace, sort_workspace_bytes, stream);
  } else if (router && E <= 128 && k >= 1 && k <= 8 && k <= E) {
    // a decode step: logits, route and sort in one launch
    rc = sy_router_route_sort(h, router, N, H, E, k, norm, logits, idx, w, counts, offsets, token, wsorted, pos_of, stream);
  } else {
    if (router) {   // the router GEMM too: logits is then an output
      rc = sy_router_logits(h, router, N, H, E, logits, stream);
      if (rc) return rc;
    }
    if (one_launch_front) {
      rc = sy_route_sort(logits, N, E, k, norm, idx, w, counts, offsets, token, wsorted, pos_of, stream);
    } else {
      rc = sy_route(logits, SY_DTYPE_F16, N, E, k, norm, idx, w, stream);
      if (rc) return rc;
      rc = sy_sort_by_expert(idx, w, 2, N, k, E, counts, offsets, token, wsorted, pos_of, sort_workspace,
                             sort_workspace_bytes, stream);
    }
  }
  if (rc) return rc;
  return sy_experts_sorted(h, N, E, k, gate_up, down, H, I, mfma_tiles, idx, w, offsets, token, wsorted, pos_of, act, y, out,
                           stream);
}

// moe_layer() of the reference in one call with one scratch buffer: the layout of the
// intermediate results is the library's business here.
namespace {
struct LayerScratch {
  size_t idx, w, counts, offsets, token, wsorted, pos_of, act, y, sort_ws, logits, end, sort_bytes;
};
LayerScratch layer_scratch(int N, int E, int k, int H, int I) {
  LayerScratch s;
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t here = at;
    at += (bytes + 255) / 256 * 256;
    return here;
  };
  const size_t M = (size_t)N * k;
  s.idx = take(M * 4);
  s.w = take(M * 2);
  s.counts = take((size_t)E * 4);
  s.offsets = take((size_t)(E + 1) * 4);
  s.token = take(M * 4);
  s.wsorted = take(M * 2);
  s.pos_of = take(M * 4);
  s.act = take(M * I * 2);
  s.y = take(M * H * 2);
  s.sort_bytes = sy_sort_workspace_bytes(N, k, E);
  s.sort_ws = take(s.sort_bytes);
  s.logits = take((size_t)N * E * 2);
  s.end = at;
  return s;
}
}  // namespace

extern "C" SY_API size_t sy_moe_layer_scratch_bytes(int N, int E, int k, int H, int I) {
  if (N <= 0 || E <= 0 || k <= 0 || H <= 0 || I <= 0) return 0;
  return layer_scratch(N, E, k, H, I).end;
}

extern "C" SY_API int sy_moe_layer(const SyMoeLayer* L, const void* h, void* out, void* stream) {
  SY_REQUIRE(L, "moe_layer: null layer");
  SY_REQUIRE(L->N >= 0 && L->E >= 1 && L->k >= 1 && L->H >= 8 && L->I >= 8, "moe_layer: N = %d, E = %d, k = %d, H = %d, I = %d",
             L->N, L->E, L->k, L->H, L->I);
  if (L->N == 0) return SY_OK;
  SY_REQUIRE(L->router && L->gate_up && L->down && h && out, "moe_layer: null pointer");
  const LayerScratch s = layer_scratch(L->N, L->E, L->k, L->H, L->I);
  SY_REQUIRE(L->scratch && L->scratch_bytes >= s.end && ((uintptr_t)L->scratch & 255) == 0,
             "moe_layer: scratch of %zu bytes, 256-byte aligned, needed (%zu given)", s.end, L->scratch_bytes);
  char* b = (char*)L->scratch;
  return sy_moe_experts(h, L->router, b + s.logits, L->N, L->E, L->k, L->norm, L->gate_up, L->down, L->H, L->I, L->mfma_tiles, 0,
                        (int32_t*)(b + s.idx), b + s.w, (int32_t*)(b + s.counts), (int32_t*)(b + s.offsets),
                        (int32_t*)(b + s.token), b + s.wsorted, (int32_t*)(b + s.pos_of), b + s.act, b + s.y, out,
                        s.sort_bytes ? b + s.sort_ws : nullptr, s.sort_bytes, stream);
}

// experts() of the reference in one call: sort, the two projections, combine, from the routing.
extern "C" SY_API int sy_experts_routed(const void* h, int N, int E, int k, const void* gate_up, const void* down, int H, int I,
                                        int mfma_tiles, const int32_t* idx, const void* w, int32_t* counts, int32_t* offsets,
                                        int32_t* token, void* wsorted, int32_t* pos_of, void* act, void* y, void* out,
                                        void* sort_workspace, size_t sort_workspace_bytes, void* stream) {
  SY_REQUIRE(N >= 0 && H >= 8 && I >= 8 && k >= 1, "experts_routed: N = %d, H = %d, I = %d, k = %d", N, H, I, k);
  if (N == 0) return SY_OK;
  SY_REQUIRE(h && idx && w && act && y && out, "experts_routed: null pointer");
  int rc;
  if (!mfma_tiles && sy_gemv_sorts(N, k, E, H)) {
    // at most 64 choices: the gate/up stream sorts them in its own prologue
    rc = sy_grouped_gemv_sorting(h, idx, w, N, k, gate_up, E, I, H, counts, offsets, token, wsorted, pos_of, act, stream);
    if (rc) return rc;
    // up to 4 tokens the down projection adds a token's rows up itself: no combine launch, no y
    if (sy_gemv_combines(N, k, E, H, I)) return sy_gemv_down_combine(act, down, offsets, token, wsorted, N, k, E, H, I, out, stream);
    rc = sy_grouped_gemv(act, nullptr, down, offsets, E, N * k, N, H, I, 0, nullptr, y, stream);
    if (rc) return rc;
    return sy_combine_weighted(y, pos_of, idx, w, N, k, H, out, stream);
  }
  rc = sy_sort_by_expert(idx, w, 2, N, k, E, counts, offsets, token, wsorted, pos_of, sort_workspace, sort_workspace_bytes,
                         stream);
  if (rc) return rc;
  return sy_experts_sorted(h, N, E, k, gate_up, down, H, I, mfma_tiles, idx, w, offsets, token, wsorted, pos_of, act, y, out,
                           stream);
}

// What follows the sort in sy_moe_experts, for a caller that has enqueued the front itself.
extern "C" SY_API int sy_experts_sorted(const void* h, int N, int E, int k, const void* gate_up, const void* down, int H, int I,
                                        int mfma_tiles, const int32_t* idx, const void* w, const int32_t* offsets,
                                        const int32_t* token, const void* wsorted, const int32_t* pos_of, void* act,
                                        void* y, void* out, void* stream) {
  SY_REQUIRE(N >= 0 && H >= 8 && I >= 8, "experts_sorted: N = %d, H = %d, I = %d", N, H, I);
  if (N == 0) return SY_OK;
  SY_REQUIRE(h && act && y && out, "experts_sorted: null pointer");
  // the projections address the gathered rows of h with 32-bit byte offsets
  SY_REQUIRE((long)N * H * 2 < (1l << 31), "experts_sorted: h must stay under 2 GiB (%d rows of %d)", N, H);
  int rc;
  const int M = N * k;
  // Where it pays, the down projection runs without its row scales: y then holds its rows before
  // the router weight, and the combine multiplies, with the same roundings in the same order.
  // Fetching the scales costs the weight-stream kernel and the 256-row MFMA tile more than the
  // multiply costs the combine (8 tokens: 0.7 us against 0.1; 4096: 3 to 9 us against 0.7); the
  // smaller MFMA tiles gain nothing, so there the projection scales. `out` has the same bits
  // either way.
  const bool combine_scales = !mfma_tiles || sy_gemm_rows_per_tile(M, E, I) == 256;
  const void* scale = combine_scales ? nullptr : wsorted;
  if (mfma_tiles) {
    rc = sy_grouped_gemm(h, token, gate_up, offsets, E, M, I, H, 1, nullptr, act, stream);
    if (rc) return rc;
    rc = sy_grouped_gemm(act, nullptr, down, offsets, E, M, H, I, 0, scale, y, stream);
  } else {
    rc = sy_grouped_gemv(h, token, gate_up, offsets, E, M, N, I, H, 1, nullptr, act, stream);
    if (rc) return rc;
    rc = sy_grouped_gemv(act, nullptr, down, offsets, E, M, N, H, I, 0, scale, y, stream);
  }
  if (rc) return rc;
  return combine_scales ? sy_combine_weighted(y, pos_of, idx, w, N, k, H, out, stream)
                        : sy_combine(y, pos_of, idx, N, k, H, out, stream);
}
