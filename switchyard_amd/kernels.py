"""The MoE layer assembled from the gfx950 kernels: the same entry points, argument order and
defaults as the reference's switchyard/kernels.py (:12-93), so `from switchyard_amd import
kernels` stands in for `from switchyard import kernels`.

Differences that follow from the hardware, none visible in the results:
  - the native library is prebuilt C ABI + ctypes, not a JIT-built pybind module (`ext()`);
  - "auto" never reads the per-expert counts back from the GPU (the reference waits on
    `int(counts.max())`, kernels.py:86): it decides from the number of tokens, so a layer
    enqueues its launches and returns;
  - the grouped GEMM finds its row tiles on the device, so `tile_offsets` is kept only as a
    helper with the reference's meaning and nothing here waits on `int(toff[-1])` (:61);
  - `pick` never answers "cublas": the MFMA kernel covers that regime. The mode string
    "cublas" is still accepted and runs the MFMA kernel.
"""

import torch
import torch.nn.functional as F

from . import _abi

_EXT = None


def ext():
    global _EXT
    if _EXT is None:
        _EXT = _abi.Ext()
    return _EXT


def tile_offsets(counts, block=64):
    tiles = (counts + block - 1) // block
    off = torch.zeros(counts.numel() + 1, dtype=torch.int32, device=counts.device)
    off[1:] = torch.cumsum(tiles, 0)
    return off


# From this many tokens on the router GEMM and route are one launch of this library (the
# library GEMM for 64 output columns takes about 14 us at any of these sizes, the route launch 6).
ROUTER_ROUTE_MIN_TOKENS = 65


def route(h, router, top_k, norm_topk_prob):
    """Returns (indices int32 [N, k], weights in h's dtype [N, k]); ties go to the lower expert id."""
    N, H = h.shape
    if (N >= ROUTER_ROUTE_MIN_TOKENS and h.dtype == torch.float16 and router.dtype == torch.float16
            and _abi.Ext.router_route_ok(N, H, router.shape[0], top_k)):
        idx, w, _ = ext().router_route(h.contiguous(), router.contiguous(), top_k, norm_topk_prob)
        return idx, w
    return ext().route(F.linear(h, router).contiguous(), top_k, norm_topk_prob)


# Measured on an MI355X with OLMoE's shapes (bench.py --sweep, ms for the experts of one layer,
# weight stream vs MFMA tiles): 8 tokens 0.147 vs 0.160, 16 tokens 0.174 vs 0.174, 24 tokens
# 0.190 vs 0.191, 32 tokens (busiest expert 9 rows) 0.201 vs 0.194, 64 tokens 0.231 vs 0.209,
# 96 tokens 0.305 vs 0.203. The weight-stream kernel wins while the busiest expert has at most
# 8 rows. The reference's third regime (a library GEMM per expert above 48 rows) does not
# exist on this hardware.
GEMV_MAX_ROWS = 8
GEMM_MAX_ROWS = 1 << 30


def pick(max_rows):
    if max_rows <= GEMV_MAX_ROWS:
        return "gemv"
    return "gemm"


# Above this many tokens "auto" never takes the weight-stream kernel. Up to GEMV_MAX_ROWS tokens
# no expert can have more rows than that, whatever the routing, and the weight stream wins (8
# tokens: 88.7 us for the two projections against 95.8 on the MFMA tiles, whose one workgroup
# per tile leaves a third of the CUs' slots empty with 41 used experts). Above, the MFMA tiles
# with their weights loaded non-temporal stream faster than the weight-stream kernel does (12
# tokens 102.4 against 107.2 us, 16 tokens 106.3 against 113.0, 32 tokens 119.8 against 133.4:
# 6.5 to 6.6 TB/s against 6.0 to 6.2), and they do not slow down when a popular expert collects
# many rows (Zipf routing cost the weight stream 20 to 30 % at 17 to 32 tokens).
GEMV_MAX_TOKENS = 8


def _auto(n_tokens, n_choices, n_experts):
    """Mode for "auto" without a device read: the weight stream while no expert can have more
    than GEMV_MAX_ROWS rows (at most that many tokens), else the MFMA tiles. Both kernels are
    correct for any routing."""
    if n_tokens <= min(GEMV_MAX_ROWS, GEMV_MAX_TOKENS):
        return "gemv"
    return "gemm"


def ffn(x, a_rows, offsets, counts, wsorted, gate_up, down, rows, mode, host_counts=None):
    """Both projections of the experts for `rows` sorted rows -> y [rows, H], router weight
    already applied (wsorted None: not applied, for a combine that multiplies). offsets [E + 1]
    cuts the sorted rows into one run per expert; sorted row i reads x[a_rows[i]] (x[i] if
    a_rows is None), so the unsorted activations are never copied. mode is "gemv" or "gemm"
    ("cublas" means "gemm" here). `counts` and `host_counts` only keep the reference's argument
    list (kernels.py:48): no launch here depends on a value read back from the GPU."""
    E = ext()
    if rows == 0:
        return torch.empty(0, down.shape[1], dtype=x.dtype, device=x.device)
    if mode == "gemv":
        # a token picks an expert at most once, so no expert has more rows than x has tokens
        bound = x.shape[0] if a_rows is not None else 0
        act = E.grouped_gemv(x.contiguous(), a_rows, gate_up, offsets, rows, True, None, bound)
        return E.grouped_gemv(act, None, down, offsets, rows, False, wsorted, bound)
    if mode in ("gemm", "cublas"):
        act = E.grouped_gemm(x.contiguous(), a_rows, gate_up, offsets, None, 0, rows, True, None)
        return E.grouped_gemm(act, None, down, offsets, None, 0, rows, False, wsorted)
    raise ValueError(f"unknown mode {mode!r}")


def experts(h, idx, w, gate_up, down, mode="auto"):
    """Everything of the layer after routing: h [N, H], idx int32 [N, k] (expert ids
    0..E-1), w [N, k] -> out [N, H] = sum over each token's k choices of
    w * expert(h[token]). Four launches and no host read: counting sort, gate/up projection with
    SwiGLU, down projection times w, fp32 combine in expert order. "auto" picks the weight-stream
    kernel or the MFMA tiles from the token count (see _auto); "gemv" / "gemm" force one."""
    E = ext()
    N = h.shape[0]
    idx = idx.contiguous()
    if mode == "auto":
        mode = _auto(N, idx.numel(), gate_up.shape[0])
    if mode not in ("gemv", "gemm", "cublas"):
        raise ValueError(f"unknown mode {mode!r}")
    if (N > 0 and h.dtype == torch.float16 and w.dtype == torch.float16 and gate_up.shape[0] <= 512
            and idx.shape[1] <= 64 and N * h.shape[1] * 2 < 2 ** 31):
        # one call of the library: the host pays per call what the GPU needs for a small kernel
        return E.experts_routed(h.contiguous(), idx, w.contiguous(), gate_up, down, mfma_tiles=mode != "gemv")
    counts, offsets, token, wsorted, pos_of = E.sort_by_expert(idx, w.contiguous(), gate_up.shape[0])
    y = ffn(h, token, offsets, counts, wsorted, gate_up, down, idx.numel(), mode)
    return E.combine(y, pos_of, idx, N)


_ONE_EXPERT = {}


def dense(x, weight):
    """x [rows, K] @ weight [Nout, K]^T for the projections around the MoE layer at decode
    (q/k/v, output, lm_head), which are weight streams like the experts are. Up to 16 rows the
    weight-stream kernel runs with a single expert that owns every row (one pass over the
    matrix; measured in a replayed graph at 8 rows: 9.7 us for [6144, 2048], 6.8 us for
    [2048, 2048], 36.9 us for [50304, 2048], against 12.4, 8.8 and 52.9 us for the library
    GEMM). Above that a plain GEMM is the library's job (12.5 us at 64 rows where the kernel's
    four passes take 33.6 us)."""
    rows = x.shape[0]
    if rows > 16 or weight.shape[1] > 4096 or weight.shape[1] % 8:
        return F.linear(x, weight)
    key = (rows, x.device)
    if key not in _ONE_EXPERT:
        _ONE_EXPERT[key] = torch.tensor([0, rows], dtype=torch.int32, device=x.device)
    return ext().grouped_gemv(x, None, weight[None], _ONE_EXPERT[key], rows, False, None, rows)


# Up to this many tokens route and sort run as one launch of one workgroup (a decode step is
# launch- and latency-bound in front of its two projections). Measured in a replayed graph, one
# launch against route + sort_by_expert: 8 tokens 3.7 against 6.5 us, 16 tokens 6.5 against 6.6,
# 32 tokens 9.2 against 6.8, 64 tokens 14.6 against 6.9 (one compute unit routes every token).
FUSED_FRONT_MAX_TOKENS = 16


def experts_rows(h, logits, gate_up, down, top_k, norm_topk_prob, mode="auto", router=None):
    """The MoE layer from its router logits [N, E] up to, not including, combine: returns
    (y [N*k, H] expert outputs scaled by the router weights, pos_of, idx), which `combine`
    or a kernel that folds it into what follows takes. Route and sort are one launch up to
    FUSED_FRONT_MAX_TOKENS tokens. With logits None the router [E, H] is given instead and
    `route` computes them (for a prompt: the router GEMM and route in one launch)."""
    E = ext()
    N, n_experts = h.shape[0], gate_up.shape[0]
    if logits is None:
        idx, w = route(h, router, top_k, norm_topk_prob)
        counts, offsets, token, wsorted, pos_of = E.sort_by_expert(idx, w, n_experts)
    elif 0 < N <= FUSED_FRONT_MAX_TOKENS and n_experts <= 128 and top_k <= 8 and logits.dtype == torch.float16:
        idx, w, counts, offsets, token, wsorted, pos_of = E.route_sort(logits, top_k, norm_topk_prob)
    else:
        idx, w = E.route(logits, top_k, norm_topk_prob)
        counts, offsets, token, wsorted, pos_of = E.sort_by_expert(idx, w, n_experts)
    if mode == "auto":
        mode = _auto(N, idx.numel(), n_experts)
    return ffn(h, token, offsets, counts, wsorted, gate_up, down, idx.numel(), mode), pos_of, idx


# Up to this many tokens the router's logits come from the library's own kernel, inside the same
# call as everything else: it takes the GPU as long as the library GEMM (a layer of 8 tokens in
# a stream of layers 102.0 us either way; the logits come out bit-equal), and the host does not
# spend 18 us on a separate GEMM call (a layer called once: 116 us against 130). One workgroup
# per token reads the whole router, so it is for tens of tokens.
OWN_ROUTER_MAX_TOKENS = 64


def moe_layer(h, router, gate_up, down, top_k, norm_topk_prob, mode="auto"):
    N, n_experts = h.shape[0], gate_up.shape[0]
    if N > 0 and n_experts <= 128 and top_k <= 8 and h.dtype == torch.float16:
        if mode == "auto":
            mode = _auto(N, N * top_k, n_experts)
        if mode not in ("gemv", "gemm", "cublas"):
            raise ValueError(f"unknown mode {mode!r}")
        H = h.shape[1]
        if (router.dtype == torch.float16 and H % 8 == 0 and H <= 8192 and N * H * 2 < 2 ** 31 and h.is_contiguous()
                and router.is_contiguous()
                and (N <= OWN_ROUTER_MAX_TOKENS or _abi.Ext.router_route_ok(N, H, n_experts, top_k))):
            # one call of the library for the whole layer, the router's logits included: the host
            # pays for a call what the GPU needs for a small kernel, and a layer that is waited
            # for pays the host's time in front of its first launch in full
            return ext().moe_layer(h, router, gate_up, down, top_k, norm_topk_prob, mode != "gemv")
        # other shapes (a width the one-launch router does not take at more than 64 tokens, another
        # dtype of the router): the library GEMM makes the logits, as in the reference (kernels.py:30-32)
        if N <= OWN_ROUTER_MAX_TOKENS:
            own = H % 8 == 0 and H <= 8192
        else:   # the router GEMM, route and the sort's first pass in one launch
            own = router.dtype == torch.float16 and _abi.Ext.router_route_ok(N, H, n_experts, top_k)
        return ext().moe_experts(h.contiguous(), None if own else F.linear(h, router).contiguous(), gate_up, down, top_k,
                                 norm_topk_prob, mfma_tiles=mode != "gemv", one_launch_front=N <= FUSED_FRONT_MAX_TOKENS,
                                 router=router.contiguous() if own else None)
    idx, w = route(h, router, top_k, norm_topk_prob)
    return experts(h, idx, w, gate_up, down, mode)
