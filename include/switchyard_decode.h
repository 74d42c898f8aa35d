/* switchyard_decode.h: C ABI of the decode-step kernels in libswitchyard_moe.so that sit around
 * the MoE layer: the attention side of one step of the decoder that calls the MoE hook, when
 * every sequence of the batch advances by one token. They replace the PyTorch operator
 * sequences of the reference's switchyard/model.py named at each entry point; the projections
 * between them (wq/wk/wv stacked, wo, lm_head) go through sy_grouped_gemv / sy_grouped_gemm of
 * switchyard_moe.h with one "expert". Conventions as in switchyard_moe.h: device pointers
 * borrowed for the call, caller-allocated outputs, `stream` a hipStream_t, f16 row-major
 * tensors, 0 or an SY_ERR_* code returned, no state kept, nothing allocated.
 * The cache slot and the rotary positions are read from device memory, so a captured HIP
 * graph of these launches can be replayed for every step.
 */
#ifndef SWITCHYARD_DECODE_H
#define SWITCHYARD_DECODE_H

#include "switchyard_moe.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Residual add and RMS norm in one pass; replaces `x = x + delta` followed by rmsnorm()
 * (switchyard/model.py:14-17 as used at :119-121,142 and :130).
 * x, delta f16 [N,H] (delta may be NULL: no add); weight f16 [H] ->
 * x_out f16 [N,H] = f16(x + delta) (may be x itself, or NULL to skip the store),
 * h_out f16 [N,H] = weight * f16(x_out * rsqrt(mean(x_out^2) + eps)), the mean in fp32.
 * Limits: H % 8 == 0, H <= 8192. N == 0 is a no-op. */
SY_API int sy_add_rmsnorm(const void* x, const void* delta, const void* weight, float eps, int N, int H, void* x_out,
                          void* h_out, void* stream);

/* The embedding lookup and the first RMS norm of a step in one launch; replaces F.embedding
 * (switchyard/model.py:111) followed by rmsnorm() (:119).
 * tokens int64 [N] (values outside [0, vocab) are clamped); embed f16 [vocab, H]; weight f16 [H]
 * -> x_out f16 [N,H] = embed[tokens], h_out f16 [N,H] = its RMS norm as sy_add_rmsnorm.
 * Limits: as sy_add_rmsnorm. */
SY_API int sy_embed_rmsnorm(const int64_t* tokens, const void* embed, int vocab, const void* weight, float eps, int N,
                            int H, void* x_out, void* h_out, void* stream);

/* sy_add_rmsnorm that also takes the router's logits of the normalised rows, so that the router
 * GEMM of the MoE layer (`F.linear(h, router)`, switchyard/kernels.py:30-32 after
 * switchyard/model.py:121) needs no launch of its own at decode.
 * router f16 [E,H] -> logits f16 [N,E] = f16(h_out @ router^T), fp32 sums; the other arguments
 * and results as sy_add_rmsnorm. Limits: as sy_add_rmsnorm, 1 <= E <= 1024. */
SY_API int sy_add_rmsnorm_logits(const void* x, const void* delta, const void* weight, float eps, const void* router,
                                 int E, int N, int H, void* x_out, void* h_out, void* logits, void* stream);

/* sy_add_rmsnorm_logits with the front of the MoE layer in the same launch: every token's
 * workgroup also routes it, and the last one to finish sorts (as sy_router_route_sort below,
 * whose limits and note on the launch counter apply): replaces the residual add, the RMS norm,
 * the router GEMM, route() and sort_by_expert() of a decode step (switchyard/model.py:119-121,
 * switchyard/kernels.py:30-32,84). Outputs are bit for bit those of sy_add_rmsnorm_logits
 * followed by sy_route and sy_sort_by_expert. */
SY_API int sy_add_rmsnorm_route_sort(const void* x, const void* delta, const void* weight, float eps, const void* router,
                                     int E, int N, int H, int k, int norm, void* x_out, void* h_out, void* logits,
                                     int32_t* idx, void* w, int32_t* counts, int32_t* offsets, int32_t* token,
                                     void* wsorted, int32_t* pos_of, void* stream);

/* The router GEMM alone, for a few rows (a decode step): replaces `F.linear(h, router)`
 * (switchyard/kernels.py:30-32). h f16 [N,H]; router f16 [E,H] -> logits f16 [N,E], fp32 sums
 * rounded once. One workgroup per row reads the whole router from L2, so this is for tens of
 * rows, not thousands (the library GEMM takes over there). Limits: as sy_add_rmsnorm_logits. */
SY_API int sy_router_logits(const void* h, const void* router, int N, int H, int E, void* logits, void* stream);

/* sy_router_logits, sy_route and sy_sort_by_expert in ONE launch, for a decode step: replaces
 * `F.linear(h, router)` + route() + sort_by_expert() (switchyard/kernels.py:30-32,84;
 * switchyard/csrc/moe_kernels.cu:73-89,142-157). One workgroup per token computes its logits as
 * sy_router_logits does, routes it, and the workgroup that finishes last sorts every token's
 * choices; outputs (logits included) are bit for bit those of the three separate calls.
 * Limits: those of sy_router_logits, 1 <= N <= 256, E <= 128, 1 <= k <= min(8, E). N == 0 is a
 * no-op. The launch counts its workgroups in a counter of a pool of 1024 that the library keeps
 * in device memory. Launches that run at once take the lower 512 counters in turn, so launches
 * on DIFFERENT streams may only disturb each other if one is still waiting to run when the 512th
 * after it is issued. A launch that a stream capture records takes one of the upper 512 in turn
 * and keeps it for every replay of its graph: no launch outside a capture is ever given that
 * counter, and two captured launches share one only if 512 launches were captured between them;
 * graphs that old must not be replayed at the same time as newer ones on another stream.
 * The first call on a device looks the pool's address up (hipGetSymbolAddress): make one call
 * outside stream capture before capturing one. */
SY_API int sy_router_route_sort(const void* h, const void* router, int N, int H, int E, int k, int norm, void* logits,
                                int32_t* idx, void* w, int32_t* counts, int32_t* offsets, int32_t* token, void* wsorted,
                                int32_t* pos_of, void* stream);

/* sy_combine folded into the residual add and the next RMS norm: replaces combine()
 * (switchyard/csrc/moe_kernels.cu:435-444) followed by `x = x + moe(i, h)` and the rmsnorm of
 * the next block (switchyard/model.py:142,119 or :130).
 * y f16 [M,H], pos_of int32 [N*k], idx int32 [N,k] as sy_combine takes them; x f16 [N,H] ->
 * x_out = f16(x + d) with d the f16 result sy_combine would give (the same bits), and
 * h_out = the RMS norm of x_out as sy_add_rmsnorm. w is NULL, or the router weights f16 [N,k]
 * (route's output) when y holds the down projection's rows BEFORE the router weight (scale NULL
 * in sy_grouped_gemv / sy_grouped_gemm): each row is then multiplied and rounded to f16 here as
 * the projection's epilogue would have, so the results have the same bits either way, and the
 * projection does not fetch a scale per row. Limits: as sy_add_rmsnorm, 1 <= k <= 64. */
SY_API int sy_combine_add_rmsnorm(const void* y, const int32_t* pos_of, const int32_t* idx, const void* w, int k,
                                  const void* x, const void* weight, float eps, int N, int H, void* x_out, void* h_out,
                                  void* stream);

/* What follows the q/k/v projections of T new tokens per sequence (T = 1 at decode, the prompt
 * length at prefill); replaces the rmsnorm of q and k, the clamp, the rotary embedding and the
 * cache write of _attention() (switchyard/model.py:64-77).
 * qkv f16 [B*T, (heads + 2*kv_heads)*D]: row b*T + t holds q, then k, then v of token t of
 * sequence b; q_norm f16 [heads*D], k_norm f16 [kv_heads*D] (the norm runs over the whole
 * projection, not per head); clip > 0 clamps q, k and v to [-clip, clip]; cos_table, sin_table
 * f16 [max_positions, D] (both halves of a row equal, as cat([freqs, freqs])); positions int64
 * [B*T] rotary position of each token; slot int64 [1] cache position of token 0 (the same for
 * every sequence of a left-padded batch) ->
 * q_out f16 [B*T, heads*D]; kcache, vcache f16 [B, kv_heads, capacity, D] get the new keys and
 * values at [:, :, slot + t, :]. A position outside [0, capacity) is not written.
 * Limits: D % 16 == 0, heads*D <= 8192, heads % kv_heads == 0. B == 0 is a no-op. */
SY_API int sy_qk_norm_rope_cache(const void* qkv, const void* q_norm, const void* k_norm, float eps, float clip,
                                 const void* cos_table, const void* sin_table, int max_positions,
                                 const int64_t* positions, const int64_t* slot, int B, int T, int heads, int kv_heads,
                                 int D, int capacity, void* q_out, void* kcache, void* vcache, void* stream);

/* One query per (sequence, head) against the KV cache; replaces the scores / mask / softmax /
 * value product of _attention() (switchyard/model.py:78-84) with T = 1.
 * q f16 [B, heads*D]; kcache, vcache f16 [B, kv_heads, capacity, D]; real uint8 [B, capacity]
 * (0 where the cache position holds left padding); slot int64 [1]: keys 0..slot are visible ->
 * out f16 [B, heads*D] = softmax(q.k / sqrt(D)) v over the visible real keys (fp32 inside);
 * zeros if a sequence has none. Query head h reads kv head h / (heads / kv_heads).
 * Limits: D is 64 or 128. B == 0 is a no-op. */
SY_API int sy_decode_attention(const void* q, const void* kcache, const void* vcache, const uint8_t* real,
                               const int64_t* slot, int B, int heads, int kv_heads, int D, int capacity, void* out,
                               void* stream);

/* sy_qk_norm_rope_cache and sy_decode_attention in one launch (switchyard/model.py:64-84 with
 * T = 1): every workgroup norms, clamps and rotates its own head of q and of the new key from
 * `qkv`, attends to the cached keys before `slot` and to the new key and value from registers,
 * and the first query head of each kv head writes them into the cache at `slot`. Arguments as
 * for the two entry points; q is not materialised. The new token is a real one by definition:
 * `real` is read for the positions before `slot` and real[:, slot] is SET to 1 (the
 * `cache.valid[:, start:start+T] = valid` of switchyard/model.py:98 for T = 1), so `real` is
 * in/out here. Results equal the two entry points' (with real[:, slot] = 1) up to the order of
 * the fp32 softmax sums. */
SY_API int sy_decode_attention_qkv(const void* qkv, const void* q_norm, const void* k_norm, float eps, float clip,
                                   const void* cos_table, const void* sin_table, int max_positions,
                                   const int64_t* positions, const int64_t* slot, uint8_t* real, int B, int heads,
                                   int kv_heads, int D, int capacity, void* kcache, void* vcache, void* out,
                                   void* stream);

/* The end of a greedy decode step in one launch; replaces `logits.argmax(-1)`, the append to
 * the output and the cache counters' increments of generate() / finish()
 * (switchyard/model.py:154-157,123-124) for T = 1.
 * logits f16 [B,V] -> tok int64 [B] = arg-max of each row (the lowest index among equal
 * maxima); out int64 [B, out_stride]: out[b, next_position[b] - base_position[b]] = tok[b] when
 * that column exists; next_position int64 [B] += 1; slot int64 [1] += 1.
 * base_position int64 [B] is what next_position held when column 0 was due. */
SY_API int sy_greedy_advance(const void* logits, int B, int V, int64_t* tok, int64_t* out, int out_stride,
                             const int64_t* base_position, int64_t* next_position, int64_t* slot, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SWITCHYARD_DECODE_H */
