/* switchyard_moe.h: C ABI of libswitchyard_moe.so, the MI355X (gfx950) kernels of the OLMoE
 * mixture-of-experts layer.
 *
 * Every entry point replaces one function of the reference's native module
 * (switchyard/csrc/moe_kernels.cu, pybind surface at :491-500) and is what a binding for that
 * path would call. Conventions:
 *   - all pointers are device pointers on the current HIP device, borrowed for the call;
 *     outputs (and workspaces) are allocated by the caller; nothing is allocated or freed here;
 *   - `stream` is a hipStream_t passed as void*; work is enqueued on it and the call returns
 *     without waiting;
 *   - "f16" is IEEE binary16; every matrix is row-major and contiguous;
 *   - the return value is 0 on success, otherwise an SY_ERR_* code, and sy_last_error()
 *     returns a message for the calling thread;
 *   - calls are re-entrant and the library keeps no state between calls (the exceptions say so:
 *     sy_sort_by_expert_static's workspace, and the launch counters of sy_router_route_sort and
 *     sy_add_rmsnorm_route_sort in switchyard_decode.h).
 */
#ifndef SWITCHYARD_MOE_H
#define SWITCHYARD_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SY_API __attribute__((visibility("default")))

#define SY_OK 0
#define SY_ERR_ARG 1     /* an argument is out of the supported range */
#define SY_ERR_LAUNCH 2  /* the HIP runtime refused a launch */

#define SY_DTYPE_F16 0
#define SY_DTYPE_F32 1

/* Library version, major*10000 + minor*100 + patch. */
SY_API int sy_version(void);

/* Message of the last error on this thread ("" if none). */
SY_API const char* sy_last_error(void);

/* Replaces route() (moe_kernels.cu:73-89, kernel :23-71).
 * logits [N,E] of `dtype` (SY_DTYPE_F16 or SY_DTYPE_F32) -> idx int32 [N,k], w [N,k] of the
 * same dtype. Softmax in fp32; the k largest ordered by (logit descending, expert id
 * ascending); w = p, or p / sum of the chosen k when norm != 0.
 * Limits: 1 <= E <= 128, 1 <= k <= 8, k <= E (the reference's, :77). N == 0 is a no-op. */
SY_API int sy_route(const void* logits, int dtype, int N, int E, int k, int norm, int32_t* idx, void* w, void* stream);

/* Bytes of workspace sy_sort_by_expert needs for N*k choices (may be 0). */
SY_API size_t sy_sort_workspace_bytes(int N, int k, int E);

/* Replaces sort_by_expert() (moe_kernels.cu:142-157, kernels :112-139, plus the ATen
 * cumsum/zeros/copy_ at :148-149, folded into the kernels).
 * Stable counting sort of the flat choices i = t*k + s by idx[i], without atomics.
 * idx int32 [N,k] with values in [0,E); w [N,k] of w_bytes (2 or 4) per element ->
 * counts int32 [E], offsets int32 [E+1], token int32 [M], wsorted [M], pos_of int32 [M],
 * M = N*k. `workspace` holds sy_sort_workspace_bytes() bytes. Choices whose id is outside
 * [0,E) are ignored (they get no row). Limits: 1 <= E <= 512. */
SY_API int sy_sort_by_expert(const int32_t* idx, const void* w, int w_bytes, int N, int k, int E, int32_t* counts,
                      int32_t* offsets, int32_t* token, void* wsorted, int32_t* pos_of, void* workspace,
                      size_t workspace_bytes, void* stream);

/* sy_sort_by_expert for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference: it
 * exists for those callers only. Same arguments and results
 * as sy_sort_by_expert without the workspace: the per-wavefront histograms live in a static
 * device array of SY_SORT_STATIC_BYTES inside the library (one copy per GPU, held until the
 * process ends). Calls whose sy_sort_workspace_bytes() exceeds that return SY_ERR_ARG (with 64
 * experts the array covers about two million choices). Every call on a GPU uses that GPU's one
 * array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do
 * not. The array's address is looked up on the first call on each device; make that call
 * outside a graph capture. */
#define SY_SORT_STATIC_BYTES (1 << 20)
SY_API int sy_sort_by_expert_static(const int32_t* idx, const void* w, int w_bytes, int N, int k, int E,
                                    int32_t* counts, int32_t* offsets, int32_t* token, void* wsorted,
                                    int32_t* pos_of, void* stream);

/* The router GEMM and route() in ONE launch.
 * Fuses F.linear(h, router) + route() (switchyard/kernels.py:30-32; kernel moe_kernels.cu:23-71):
 * h f16 [N,H]; router f16 [E,H] -> logits f16 [N,E] (fp32 sums in a fixed order, rounded once),
 * and from those logits exactly the outputs of sy_route (idx, w in f16). Up to 64 tokens a
 * workgroup per token computes the logits as sy_router_logits does (the same bits) and routes it;
 * above, 16 tokens to a workgroup on MFMA.
 * Limits: E <= 128, k <= 8; up to 64 tokens H a multiple of 8 up to 8192, above H a multiple of
 * 512 and N*H*2 < 2 GiB. N == 0 is a no-op. */
SY_API int sy_router_route(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits,
                           int32_t* idx, void* w, void* stream);

/* Route and sort of a decode step in ONE launch (one workgroup).
 * Fuses route() (moe_kernels.cu:73-89) and sort_by_expert() (moe_kernels.cu:142-157), which the
 * reference's layer calls back to back (switchyard/kernels.py:91-93,84).
 * logits f16 [N,E] -> exactly the outputs of sy_route (idx, w in f16) and of sy_sort_by_expert.
 * Limits: 1 <= N <= 256, E <= 128, k <= 8. */
SY_API int sy_route_sort(const void* logits, int N, int E, int k, int norm, int32_t* idx, void* w, int32_t* counts,
                         int32_t* offsets, int32_t* token, void* wsorted, int32_t* pos_of, void* stream);

/* Replaces grouped_gemv() (moe_kernels.cu:385-415, kernel :308-383): the decode weight stream.
 * For every expert e and row r in offsets[e]..offsets[e+1]:
 *   C[r,:] = epilogue(A[a_rows ? a_rows[r] : r, :] @ B[e]^T)
 * A f16 [*,K]; a_rows int32 [rows] or NULL; B f16 [E,Nfull,K] (nn.Linear layout),
 * Nfull = 2*Nout when swiglu (gate rows first) else Nout; offsets int32 [E+1];
 * scale f16 [rows] or NULL; C f16 [rows,Nout].
 * swiglu: C = f16(f16(silu(f16(gate))) * f16(up)); scale: C = f16(f16(acc) * scale[r]).
 * max_rows_hint: an upper bound on the rows of any one expert if the caller knows one (the
 * number of tokens, when a token picks an expert at most once), else 0. It only sizes the
 * kernel's row staging; results do not depend on it, and it need not hold.
 * Limits: K % 8 == 0, K <= 4096. rows == 0 is a no-op. */
SY_API int sy_grouped_gemv(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets, int E, int rows,
                           int max_rows_hint, int Nout, int K, int swiglu, const void* scale, void* C, void* stream);

/* sort_by_expert() and the gate/up grouped_gemv() of a decode step in ONE launch: replaces the two
 * calls as experts() makes them (switchyard/kernels.py:84,67; moe_kernels.cu:142-157,385-415) for
 * at most 64 choices. Every workgroup of the weight stream sorts the choices itself (one per lane
 * of a wavefront) where it would otherwise read `offsets`, and the first one also writes the
 * sort's five results for the launches behind it. h f16 [N,H]; idx int32 [N,k]; w f16 [N,k];
 * gate_up f16 [E,2I,H] -> counts, offsets, token, wsorted, pos_of as sy_sort_by_expert leaves
 * them and act f16 [N*k, I] as sy_grouped_gemv (swiglu) does, bit for bit. This is the gate/up
 * launch of sy_moe_experts / sy_experts_routed at decode.
 * Limits: N*k <= 64, E <= 128, k <= E, H % 8 == 0, H <= 4096. */
SY_API int sy_grouped_gemv_sorting(const void* h, const int32_t* idx, const void* w, int N, int k, const void* gate_up,
                                   int E, int I, int H, int32_t* counts, int32_t* offsets, int32_t* token,
                                   void* wsorted, int32_t* pos_of, void* act, void* stream);

/* Replaces grouped_gemm() (moe_kernels.cu:264-298, kernel :167-261): the same function on
 * MFMA tiles for many rows per expert. The row tiles of every expert are derived from
 * `offsets` inside the kernel, so the reference's tile_offsets / total_tiles arguments (and
 * the host read behind them, kernels.py:61) have no counterpart here.
 * Limits: K % 32 == 0; A under 2 GiB (its rows are addressed with 32-bit byte offsets; with
 * a_rows the library cannot see A's size and the caller must keep to this). rows == 0 is a no-op. */
SY_API int sy_grouped_gemm(const void* A, const int32_t* a_rows, const void* B, const int32_t* offsets, int E, int rows,
                    int Nout, int K, int swiglu, const void* scale, void* C, void* stream);

/* Replaces combine() (moe_kernels.cu:435-444, kernel :419-433).
 * out[t,:] = f16(sum over t's k choices, in ascending expert id, of y[pos_of[t*k+j],:]) with
 * the sum in fp32. y f16 [M,H]; pos_of int32 [N*k]; idx int32 [N,k]; out f16 [N,H].
 * Limits: H % 8 == 0, 1 <= k <= 64. N == 0 is a no-op. */
SY_API int sy_combine(const void* y, const int32_t* pos_of, const int32_t* idx, int N, int k, int H, void* out,
               void* stream);

/* Replaces moe_layer() (switchyard/kernels.py:91-93: route() with its router GEMM, :30-32, then
 * experts(), :76-88: sort -> pick -> ffn -> combine) in ONE call: the router's logits
 * (when `router` is given: up to 64 tokens sy_router_route_sort, which is the whole front in one
 * launch, or, with the weight-stream kernels and at most 64 choices, sy_router_route and a
 * gate/up projection that sorts for itself; above that sy_router_route, which routes in the same launch and is also the first pass
 * of the sort; with router NULL `logits` is an input), route and sort (sy_route_sort when one_launch_front is nonzero, else sy_route and
 * sy_sort_by_expert with the given workspace), the gate/up projection (SwiGLU, rows of h gathered through `token`), the
 * down projection (x router weight) and sy_combine are enqueued back to back, exactly as the
 * separate calls would be.
 * h f16 [N,H]; router f16 [E,H] or NULL; logits f16 [N,E]; gate_up f16 [E,2I,H]; down f16
 * [E,H,I]; mfma_tiles 0 runs sy_grouped_gemv twice, nonzero sy_grouped_gemm. Outputs as the
 * separate calls' (idx, w, counts, offsets, token, wsorted, pos_of), plus act f16 [N*k, I],
 * y f16 [N*k, H] (scratch: the down projection's rows, before or after the router weight; with
 * the weight-stream kernels and with the 256-row MFMA tile this call applies the weight in its
 * combine instead, with the roundings of the separate calls, so `out` has their bits) and
 * out f16 [N,H], all caller-allocated. Limits: those of the entry points it
 * calls. */
SY_API int sy_moe_experts(const void* h, const void* router, void* logits, int N, int E, int k, int norm,
                          const void* gate_up, const void* down, int H, int I, int mfma_tiles, int one_launch_front,
                          int32_t* idx, void* w, int32_t* counts, int32_t* offsets, int32_t* token, void* wsorted,
                          int32_t* pos_of, void* act, void* y, void* out, void* sort_workspace,
                          size_t sort_workspace_bytes, void* stream);

/* Replaces moe_layer() (switchyard/kernels.py:91-93) in ONE call that takes one description of
 * the layer and one scratch buffer: sy_moe_experts with the router given, the intermediate
 * results (ids, weights, the sort's outputs, act, y, the sort's workspace, the logits) laid out by
 * the library in `scratch`. A binding fills a SyMoeLayer once per (shape, weights) and then
 * passes only h, out and the stream per call, which is what a call that is waited for wants:
 * the host's time in front of the first launch is GPU idle time (switchyard/kernels.py:91-93 is
 * two Python-level calls and a library GEMM in the reference).
 * h f16 [N,H]; router f16 [E,H]; gate_up f16 [E,2I,H]; down f16 [E,H,I]; mfma_tiles 0 runs the
 * weight-stream kernels, nonzero the MFMA tiles; scratch holds sy_moe_layer_scratch_bytes(N, E,
 * k, H, I) bytes, 256-byte aligned, and is free again when the call's launches have run;
 * out f16 [N,H]. Limits: those of sy_moe_experts with a router (E <= 128, k <= 8, H % 8 == 0 and
 * H <= 8192, N*H*2 < 2 GiB). N == 0 is a no-op. */
typedef struct SyMoeLayer {
  int32_t N, E, k, norm, H, I, mfma_tiles, reserved;
  const void* router;
  const void* gate_up;
  const void* down;
  void* scratch;
  size_t scratch_bytes;
} SyMoeLayer;
SY_API size_t sy_moe_layer_scratch_bytes(int N, int E, int k, int H, int I);
SY_API int sy_moe_layer(const SyMoeLayer* layer, const void* h, void* out, void* stream);

/* Replaces experts() (switchyard/kernels.py:76-88: sort -> pick -> ffn -> combine, for routing
 * computed elsewhere) in ONE call. idx int32 [N,k] and w f16 [N,k] are inputs; counts ... pos_of
 * are the sort's outputs as sy_sort_by_expert leaves them, act / y / out as in sy_moe_experts.
 * With the weight-stream kernels (mfma_tiles 0) and at most 64 choices (N*k <= 64, E <= 128,
 * H <= 4096) there is no sort launch: the gate/up projection sorts in its own prologue and its
 * first workgroup writes the sort's outputs; otherwise sy_sort_by_expert runs with the given
 * workspace (sy_sort_workspace_bytes). `out` has the bits of the separate calls. */
SY_API int sy_experts_routed(const void* h, int N, int E, int k, const void* gate_up, const void* down, int H, int I,
                             int mfma_tiles, const int32_t* idx, const void* w, int32_t* counts, int32_t* offsets,
                             int32_t* token, void* wsorted, int32_t* pos_of, void* act, void* y, void* out,
                             void* sort_workspace, size_t sort_workspace_bytes, void* stream);

/* The part of sy_moe_experts behind the sort, for a caller that has enqueued the front of the
 * layer on the same stream itself (sy_router_route_sort, or sy_route and sy_sort_by_expert):
 * replaces pick() / ffn() / combine() as experts() calls them (switchyard/kernels.py:85-88).
 * Inputs idx int32 [N,k], w f16 [N,k], offsets int32 [E+1], token int32 [N*k], wsorted f16
 * [N*k], pos_of int32 [N*k] as the front leaves them; act, y and out as in sy_moe_experts. */
SY_API int sy_experts_sorted(const void* h, int N, int E, int k, const void* gate_up, const void* down, int H, int I,
                             int mfma_tiles, const int32_t* idx, const void* w, const int32_t* offsets,
                             const int32_t* token, const void* wsorted, const int32_t* pos_of, void* act, void* y,
                             void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SWITCHYARD_MOE_H */
