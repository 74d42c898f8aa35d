"""ctypes binding of libswitchyard_moe.so (C ABI in include/switchyard_moe.h and, for the
decode-step kernels around the MoE layer, include/switchyard_decode.h).

`Ext` offers the functions of the reference's pybind module `switchyard_moe`
(switchyard/csrc/moe_kernels.cu:491-500) with the same names, argument order and results,
so code written against `kernels.ext()` keeps working. Outputs are allocated here with
torch.empty on the current stream; the library itself never allocates. ctypes releases the
GIL around every call, as the reference's call guards do.

There is no fallback: if the library is missing and cannot be built, loading raises."""

import collections
import ctypes
import threading
import os
import weakref

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libswitchyard_moe.so")

_c_int, _c_void_p, _c_size_t, _c_float = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float


class SyMoeLayer(ctypes.Structure):
    """struct SyMoeLayer of include/switchyard_moe.h: one layer's shape, weights and scratch."""
    _fields_ = [("N", ctypes.c_int32), ("E", ctypes.c_int32), ("k", ctypes.c_int32), ("norm", ctypes.c_int32),
                ("H", ctypes.c_int32), ("I", ctypes.c_int32), ("mfma_tiles", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("router", _c_void_p), ("gate_up", _c_void_p), ("down", _c_void_p), ("scratch", _c_void_p),
                ("scratch_bytes", _c_size_t)]


# name -> (restype, argtypes); mirrors include/switchyard_moe.h and include/switchyard_decode.h
SIGNATURES = {
    "sy_version": (_c_int, []),
    "sy_last_error": (ctypes.c_char_p, []),
    "sy_route": (_c_int, [_c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p]),
    "sy_sort_workspace_bytes": (_c_size_t, [_c_int, _c_int, _c_int]),
    "sy_sort_by_expert": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                                   _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_size_t, _c_void_p]),
    "sy_sort_by_expert_static": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                                          _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "sy_route_sort": (_c_int, [_c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                               _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "sy_grouped_gemv": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_int, _c_void_p, _c_void_p, _c_void_p]),
    "sy_grouped_gemv_sorting": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_int]
                                + [_c_void_p] * 7),
    "sy_grouped_gemm": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_void_p, _c_void_p, _c_void_p]),
    "sy_combine": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p]),
    "sy_moe_experts": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                                _c_int, _c_int, _c_int, _c_int] + [_c_void_p] * 11 + [_c_size_t, _c_void_p]),
    "sy_moe_layer_scratch_bytes": (_c_size_t, [_c_int, _c_int, _c_int, _c_int, _c_int]),
    "sy_moe_layer": (_c_int, [ctypes.POINTER(SyMoeLayer), _c_void_p, _c_void_p, _c_void_p]),
    "sy_router_logits": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p]),
    "sy_router_route_sort": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int] + [_c_void_p] * 9),
    "sy_experts_sorted": (_c_int, [_c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int]
                          + [_c_void_p] * 10),
    "sy_experts_routed": (_c_int, [_c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_int]
                          + [_c_void_p] * 11 + [_c_size_t, _c_void_p]),
    "sy_router_route": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                                 _c_void_p, _c_void_p]),
    "sy_add_rmsnorm": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_int, _c_int, _c_void_p, _c_void_p,
                                _c_void_p]),
    "sy_embed_rmsnorm": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_float, _c_int, _c_int, _c_void_p, _c_void_p,
                                  _c_void_p]),
    "sy_greedy_advance": (_c_int, [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                                   _c_void_p, _c_void_p]),
    "sy_add_rmsnorm_logits": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_int,
                                       _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "sy_add_rmsnorm_route_sort": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_int, _c_int, _c_int,
                                           _c_int, _c_int] + [_c_void_p] * 11),
    "sy_combine_add_rmsnorm": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_float, _c_int,
                                        _c_int, _c_void_p, _c_void_p, _c_void_p]),
    "sy_qk_norm_rope_cache": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_float, _c_void_p, _c_void_p, _c_int,
                                       _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p,
                                       _c_void_p, _c_void_p, _c_void_p]),
    "sy_decode_attention_qkv": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_float, _c_void_p, _c_void_p, _c_int,
                                         _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                         _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "sy_decode_attention": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                     _c_int, _c_int, _c_void_p, _c_void_p]),
}


def load_library(path=LIB_PATH):
    """dlopen the library and declare every entry point; builds it first if it is absent."""
    if not os.path.exists(path):
        from . import build

        try:
            build.build()
        except Exception as exc:  # no hipcc, or the compile failed
            raise RuntimeError(f"switchyard_amd: {path} is missing and could not be built: {exc}") from exc
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype, fn.argtypes = restype, argtypes
    return lib


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """Raw handle of the current stream of the current device. torch.cuda.current_stream() builds
    a Stream object on every call (2.8 us of host time per launch measured); the accessor torch
    itself uses underneath returns the same handle in a fraction of that."""
    if _raw_stream is not None and _device_index is not None:
        return _raw_stream(_device_index())
    return torch.cuda.current_stream().cuda_stream


def _check(t, name, dtype=None):
    if not (t.is_cuda and t.is_contiguous()):
        raise RuntimeError(f"{name} must be a contiguous GPU tensor")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")


_DTYPE_CODE = {torch.float16: 0, torch.float32: 1}


class Ext:
    """The native module: route, sort_by_expert, grouped_gemv, grouped_gemm, combine."""

    PLAN_BYTES_MAX = 32 << 20   # moe_experts keeps the scratch of calls up to this size ...
    PLANS_MAX = 16              # ... for this many (shape, stream) pairs, least recently used first out

    def __init__(self, lib=None):
        self.lib = lib or load_library()
        self._plans = collections.OrderedDict()   # (shape, stream) -> plan; evicted least recently used first
        self._captured = {}                       # plans that a stream capture has seen: never evicted
        self._plans_lock = threading.Lock()
        self._layers = {}                         # (N, ids of the weights, k, norm, tiles, stream) -> a prepared SyMoeLayer
        self._scratch = collections.OrderedDict() # (bytes, device, stream) -> [alive, pinned, tensor] of moe_layer
        self._scratch_pinned = []                 # scratch that a stream capture has seen: kept for good

    def _call(self, fn, *args):
        rc = fn(*args)
        if rc:
            raise RuntimeError(self.lib.sy_last_error().decode())

    def version(self):
        return self.lib.sy_version()

    def route(self, logits, k, norm):
        """logits [N, E] f16 (or f32) -> [idx int32 [N, k], w [N, k] in logits' dtype]."""
        _check(logits, "logits")
        if logits.dtype not in _DTYPE_CODE:
            raise RuntimeError("route: fp16 logits")
        N, E = logits.shape
        idx = torch.empty((N, k), dtype=torch.int32, device=logits.device)
        w = torch.empty((N, k), dtype=logits.dtype, device=logits.device)
        self._call(self.lib.sy_route, logits.data_ptr(), _DTYPE_CODE[logits.dtype], N, E, int(k), int(bool(norm)),
                   idx.data_ptr(), w.data_ptr(), _stream())
        return [idx, w]

    def sort_by_expert(self, idx, w, E):
        """idx int32 [N, k], w [N, k] -> [counts [E], offsets [E+1], token [M], wsorted [M], pos_of [M]]."""
        _check(idx, "idx", torch.int32)
        _check(w, "w")
        N, k = idx.shape
        M, dev = N * k, idx.device
        counts = torch.empty(E, dtype=torch.int32, device=dev)
        offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
        token = torch.empty(M, dtype=torch.int32, device=dev)
        wsorted = torch.empty(M, dtype=w.dtype, device=dev)
        pos_of = torch.empty(M, dtype=torch.int32, device=dev)
        need = self.lib.sy_sort_workspace_bytes(N, k, E)
        ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
        self._call(self.lib.sy_sort_by_expert, idx.data_ptr(), w.data_ptr(), w.element_size(), N, k, int(E),
                   counts.data_ptr(), offsets.data_ptr(), token.data_ptr(), wsorted.data_ptr(), pos_of.data_ptr(),
                   ws.data_ptr() if need else None, need, _stream())
        return [counts, offsets, token, wsorted, pos_of]

    def route_sort(self, logits, k, norm, n_experts=None):
        """route then sort_by_expert in one launch (decode). logits [N, E] f16 ->
        [idx [N, k], w [N, k], counts [E], offsets [E+1], token [M], wsorted [M], pos_of [M]]."""
        _check(logits, "logits", torch.float16)
        N, E = logits.shape
        dev, M = logits.device, N * k
        i32 = dict(dtype=torch.int32, device=dev)
        idx, w = torch.empty((N, k), **i32), torch.empty((N, k), dtype=torch.float16, device=dev)
        counts, offsets = torch.empty(E, **i32), torch.empty(E + 1, **i32)
        token, pos_of = torch.empty(M, **i32), torch.empty(M, **i32)
        wsorted = torch.empty(M, dtype=torch.float16, device=dev)
        self._call(self.lib.sy_route_sort, logits.data_ptr(), N, E, int(k), int(bool(norm)), idx.data_ptr(),
                   w.data_ptr(), counts.data_ptr(), offsets.data_ptr(), token.data_ptr(), wsorted.data_ptr(),
                   pos_of.data_ptr(), _stream())
        return [idx, w, counts, offsets, token, wsorted, pos_of]

    def _grouped(self, fn, A, a_rows, B, offsets, rows, swiglu, scale, hint=None):
        _check(A, "A", torch.float16)
        _check(B, "B", torch.float16)
        _check(offsets, "offsets", torch.int32)
        if a_rows is not None:
            _check(a_rows, "a_rows", torch.int32)
        if scale is not None:
            _check(scale, "scale", torch.float16)
        E, Nfull, K = B.shape
        if A.shape[1] != K:
            raise RuntimeError("grouped: K must match")
        if offsets.numel() != E + 1:
            raise RuntimeError("grouped: offsets must have E + 1 entries")
        if a_rows is not None and a_rows.numel() < rows or scale is not None and scale.numel() < rows:
            raise RuntimeError("grouped: a_rows / scale shorter than rows")
        if a_rows is None and A.shape[0] < rows:
            raise RuntimeError("grouped: A has fewer rows than `rows`")
        if a_rows is not None and A.numel() * 2 >= 2 ** 31:
            raise RuntimeError("grouped: a gathered A must stay under 2 GiB (32-bit row offsets)")
        Nout = Nfull // 2 if swiglu else Nfull
        C = torch.empty((rows, Nout), dtype=A.dtype, device=A.device)
        extra = () if hint is None else (int(hint),)
        self._call(fn, A.data_ptr(), a_rows.data_ptr() if a_rows is not None else None, B.data_ptr(),
                   offsets.data_ptr(), E, int(rows), *extra, Nout, K, int(bool(swiglu)),
                   scale.data_ptr() if scale is not None else None, C.data_ptr(), _stream())
        return C

    def grouped_gemv(self, A, a_rows, B, offsets, rows, swiglu, scale, max_rows=0):
        """max_rows: an upper bound on the rows of one expert if known (0: unknown); a sizing
        hint with no effect on the result."""
        return self._grouped(self.lib.sy_grouped_gemv, A, a_rows, B, offsets, rows, swiglu, scale, hint=max_rows)

    def grouped_gemv_sorting(self, h, idx, w, gate_up):
        """sort_by_expert and the gate/up weight stream of a decode step in one launch (at most 64
        choices): h [N, H], idx int32 [N, k], w f16 [N, k], gate_up [E, 2I, H] ->
        [counts, offsets, token, wsorted, pos_of, act [N*k, I]]."""
        for t, name, dt in ((h, "h", torch.float16), (idx, "idx", torch.int32), (w, "w", torch.float16),
                            (gate_up, "gate_up", torch.float16)):
            _check(t, name, dt)
        (N, H), k, E = h.shape, idx.shape[1], gate_up.shape[0]
        I, M, dev = gate_up.shape[1] // 2, N * k, h.device
        if tuple(idx.shape) != (N, k) or tuple(w.shape) != (N, k) or gate_up.shape[2] != H:
            raise RuntimeError("grouped_gemv_sorting: idx and w must be [N, k], gate_up [E, 2I, H]")
        i32 = dict(dtype=torch.int32, device=dev)
        counts, offsets = torch.empty(E, **i32), torch.empty(E + 1, **i32)
        token, pos_of = torch.empty(M, **i32), torch.empty(M, **i32)
        wsorted = torch.empty(M, dtype=torch.float16, device=dev)
        act = torch.empty((M, I), dtype=torch.float16, device=dev)
        self._call(self.lib.sy_grouped_gemv_sorting, h.data_ptr(), idx.data_ptr(), w.data_ptr(), N, k, gate_up.data_ptr(),
                   E, I, H, counts.data_ptr(), offsets.data_ptr(), token.data_ptr(), wsorted.data_ptr(), pos_of.data_ptr(),
                   act.data_ptr(), _stream())
        return [counts, offsets, token, wsorted, pos_of, act]

    def grouped_gemm(self, A, a_rows, B, offsets, tile_offsets, total_tiles, rows, swiglu, scale):
        """tile_offsets / total_tiles are accepted for the reference's call shape and unused:
        the kernel derives its row tiles from `offsets`."""
        return self._grouped(self.lib.sy_grouped_gemm, A, a_rows, B, offsets, rows, swiglu, scale)

    def combine(self, y, pos_of, idx, n_tokens):
        _check(y, "y", torch.float16)
        _check(pos_of, "pos_of", torch.int32)
        _check(idx, "idx", torch.int32)
        H, k = y.shape[1], idx.shape[1]
        if pos_of.numel() < n_tokens * k or idx.shape[0] < n_tokens:
            raise RuntimeError("combine: pos_of / idx shorter than n_tokens * k")
        out = torch.empty((n_tokens, H), dtype=y.dtype, device=y.device)
        self._call(self.lib.sy_combine, y.data_ptr(), pos_of.data_ptr(), idx.data_ptr(), int(n_tokens), k, H,
                   out.data_ptr(), _stream())
        return out

    def moe_experts(self, h, logits, gate_up, down, k, norm, mfma_tiles=False, one_launch_front=True, router=None):
        """(The router's logits,) route and sort, the two projections and combine in one call of
        the library (at most 128 experts, top-8; one_launch_front needs at most 256 tokens).
        h [N, H] and either logits [N, E] f16 or router [E, H] f16 (then logits is None and the
        library's own router kernel computes them: for tens of tokens) -> out [N, H]. The
        intermediate results live in one scratch allocation and are not returned."""
        # Only what the front of the layer reads is checked here: a call that is waited for is
        # timed with the host time in front of its first launch, so the weights of the experts
        # are checked behind that launch (_enqueue_experts), before anything reads them.
        _check(h, "h", torch.float16)
        N, H = h.shape
        if (logits is None) == (router is None):
            raise RuntimeError("moe_experts: give the logits or the router")
        if logits is not None:
            _check(logits, "logits", torch.float16)
            E = logits.shape[1]
            if logits.shape[0] != N:
                raise RuntimeError("moe_experts: logits must be [N, E]")
        else:
            _check(router, "router", torch.float16)
            E = router.shape[0]
            if router.shape[1] != H:
                raise RuntimeError("moe_experts: router must be [E, H]")
        if down.dim() != 3:
            raise RuntimeError("moe_experts: down must be [E, H, I]")
        I, k, norm = down.shape[2], int(k), int(bool(norm))
        stream = _stream()
        # The intermediate results of small calls (a decode step's) live in an allocation that is
        # kept per shape and stream: calls on one stream run in order, so they may share it. A HIP
        # graph that is captured through this call keeps the allocation's address for as long as it
        # can be replayed, so a plan that a capture has seen is never evicted; the others leave
        # least recently used first. (The reference allocates per call, moe_kernels.cu:146-152,272,
        # 391,438, which costs a call that is waited for the allocator's time in front of its
        # first launch.)
        key = (N, E, k, H, I, norm, logits is None, bool(one_launch_front), h.device.index, stream)
        with self._plans_lock:
            plan = self._captured.get(key)
            if plan is None:
                capturing = torch.cuda.is_current_stream_capturing()
                plan = self._plans.get(key)
                if plan is None:
                    plan = self._new_plan(N, E, k, H, I, logits is None, bool(one_launch_front), h.device)
                    if plan[3] is not None:
                        if capturing:
                            self._captured[key] = plan
                        else:
                            if len(self._plans) >= self.PLANS_MAX:
                                self._plans.popitem(last=False)
                            self._plans[key] = plan
                elif capturing:
                    self._captured[key] = self._plans.pop(key)
                else:
                    self._plans.move_to_end(key)
            starts, at, need, scratch, where = plan
            if scratch is not None:
                # kept scratch: two threads enqueueing the same shape on one stream must not
                # interleave their launches (ctypes releases the GIL inside the calls)
                return self._enqueue_experts(h, router, logits, gate_up, down, N, H, E, I, k, norm, mfma_tiles,
                                             one_launch_front, scratch, where, need, stream)
        scratch = torch.empty(at, dtype=torch.uint8, device=h.device)
        return self._enqueue_experts(h, router, logits, gate_up, down, N, H, E, I, k, norm, mfma_tiles, one_launch_front,
                                     scratch, self._addresses(scratch, starts), need, stream)

    def _new_plan(self, N, E, k, H, I, own_logits, one_launch_front, device):
        """(offsets of the intermediate results, bytes, bytes of the sort's workspace, the kept
        allocation or None for a call too large to keep one, its addresses)."""
        M = N * k
        need = 0 if one_launch_front else self.lib.sy_sort_workspace_bytes(N, k, E)
        # idx w counts offsets token wsorted pos_of act y, then the sort's workspace and the logits
        sizes = [M * 4, M * 2, E * 4, (E + 1) * 4, M * 4, M * 2, M * 4, M * I * 2, M * H * 2, need,
                 N * E * 2 if own_logits else 0]
        starts, at = [], 0
        for size in sizes:
            starts.append(at)
            at += (size + 255) // 256 * 256
        if at > self.PLAN_BYTES_MAX:
            return (starts, at, need, None, None)
        scratch = torch.empty(at, dtype=torch.uint8, device=device)
        return (starts, at, need, scratch, self._addresses(scratch, starts))

    LAYERS_MAX = 1024   # prepared layer descriptions kept (a few hundred bytes each)

    def moe_layer(self, h, router, gate_up, down, k, norm, mfma_tiles=False):
        """moe_layer() of the reference in one call of the library (sy_moe_layer): h [N, H],
        router [E, H], gate_up [E, 2I, H], down [E, H, I], all f16 -> out [N, H]. The description of
        the layer (shape, weights, scratch) is prepared once per (token count, weights, stream)
        and kept, so a call is a lookup, the allocation of `out` and one call with four arguments:
        the host's time in front of the first launch is what a call that is waited for pays on
        top of its kernels. The scratch is kept per (size, stream) up to PLAN_BYTES_MAX, with the
        rules of moe_experts: calls on one stream share it, the least recently used of PLANS_MAX
        goes first, and one that a stream capture has seen is never freed. Above that size the
        scratch is allocated per call."""
        if not (h.is_cuda and h.is_contiguous() and h.dtype == torch.float16 and h.dim() == 2):
            raise RuntimeError("moe_layer: h must be a contiguous f16 GPU tensor [N, H]")
        N = h.shape[0]
        stream = _stream()
        key = (N, id(router), id(gate_up), id(down), k, norm, mfma_tiles, stream)
        with self._plans_lock:
            entry = self._layers.get(key)
            if entry is not None:
                desc, plan, refs, ptrs = entry
                if not (plan[0] and refs[0]() is router and refs[1]() is gate_up and refs[2]() is down and
                        ptrs == (router.data_ptr(), gate_up.data_ptr(), down.data_ptr()) and desc.H == h.shape[1]):
                    entry = None      # the scratch was evicted, or other tensors live at these ids now
                elif not plan[1] and torch.cuda.is_current_stream_capturing():
                    self._pin(plan)
            if entry is None:
                desc, plan = self._prepare_layer(h, router, gate_up, down, int(k), int(bool(norm)), bool(mfma_tiles), stream)
                if plan[0]:      # kept scratch: keep the description with it
                    if len(self._layers) >= self.LAYERS_MAX:
                        self._layers.clear()
                    self._layers[key] = (desc, plan, (weakref.ref(router), weakref.ref(gate_up), weakref.ref(down)),
                                         (router.data_ptr(), gate_up.data_ptr(), down.data_ptr()))
            out = torch.empty_like(h)
            rc = self.lib.sy_moe_layer(desc, h.data_ptr(), out.data_ptr(), stream)
        if rc:
            raise RuntimeError(self.lib.sy_last_error().decode())
        return out

    def _pin(self, plan):
        """A stream capture has seen this scratch: it leaves the least-recently-used list for good."""
        plan[1] = True
        for key, other in list(self._scratch.items()):
            if other is plan:
                del self._scratch[key]
                self._scratch_pinned.append(plan)

    def _prepare_layer(self, h, router, gate_up, down, k, norm, mfma_tiles, stream):
        for t, name in ((router, "router"), (gate_up, "gate_up"), (down, "down")):
            _check(t, name, torch.float16)
        N, H = h.shape
        E = router.shape[0]
        if down.dim() != 3 or router.dim() != 2:
            raise RuntimeError("moe_layer: router must be [E, H] and down [E, H, I]")
        I = down.shape[2]
        if tuple(router.shape) != (E, H) or tuple(gate_up.shape) != (E, 2 * I, H) or tuple(down.shape) != (E, H, I):
            raise RuntimeError("moe_layer: shapes of h / router / gate_up / down do not match")
        need = self.lib.sy_moe_layer_scratch_bytes(N, E, k, H, I)
        if need > self.PLAN_BYTES_MAX:
            # a large call: its scratch is this call's own (the allocator hands it on in stream order,
            # and a capture keeps it in the graph's pool); nothing is kept, nothing can be evicted
            scratch = torch.empty(need, dtype=torch.uint8, device=h.device)
            desc = SyMoeLayer(N, E, k, norm, H, I, int(mfma_tiles), 0, router.data_ptr(), gate_up.data_ptr(),
                              down.data_ptr(), scratch.data_ptr(), need)
            return desc, [False, False, scratch]
        skey = (need, h.device.index, stream)
        plan = self._scratch.get(skey)          # [alive, pinned, tensor]
        capturing = torch.cuda.is_current_stream_capturing()
        if plan is None:
            plan = [True, capturing, torch.empty(max(need, 256), dtype=torch.uint8, device=h.device)]
            if capturing:
                self._scratch_pinned.append(plan)
            else:
                if len(self._scratch) >= self.PLANS_MAX:
                    _, old = self._scratch.popitem(last=False)
                    old[0] = False              # descriptions that point at it are rebuilt on their next use
                    old[2] = None               # ... and must not keep its memory meanwhile (what is queued on
                                                # the stream it was allocated on runs before the memory is reused)
                self._scratch[skey] = plan
        else:
            self._scratch.move_to_end(skey)
            if capturing and not plan[1]:
                self._pin(plan)
        desc = SyMoeLayer(N, E, k, norm, H, I, int(mfma_tiles), 0, router.data_ptr(), gate_up.data_ptr(), down.data_ptr(),
                          plan[2].data_ptr(), plan[2].numel())
        return desc, plan

    def experts_routed(self, h, idx, w, gate_up, down, mfma_tiles=False):
        """experts() of the reference in one call of the library: h [N, H], idx int32 [N, k],
        w f16 [N, k] -> out [N, H] (sort, the two projections, combine). The intermediate
        results are allocated here and not returned."""
        for t, name, dt in ((h, "h", torch.float16), (idx, "idx", torch.int32), (w, "w", torch.float16),
                            (gate_up, "gate_up", torch.float16), (down, "down", torch.float16)):
            _check(t, name, dt)
        N, H = h.shape
        k, E, I = idx.shape[1], gate_up.shape[0], down.shape[2]
        if tuple(idx.shape) != (N, k) or tuple(w.shape) != (N, k):
            raise RuntimeError("experts_routed: idx and w must be [N, k]")
        if tuple(gate_up.shape) != (E, 2 * I, H) or tuple(down.shape) != (E, H, I):
            raise RuntimeError("experts_routed: shapes of h / gate_up / down do not match")
        M = N * k
        need = self.lib.sy_sort_workspace_bytes(N, k, E)
        # idx-independent scratch: counts offsets token wsorted pos_of act y, then the sort's workspace
        sizes = [E * 4, (E + 1) * 4, M * 4, M * 2, M * 4, M * I * 2, M * H * 2, need]
        starts, at = [], 0
        for size in sizes:
            starts.append(at)
            at += (size + 255) // 256 * 256
        scratch = torch.empty(max(at, 1), dtype=torch.uint8, device=h.device)
        where = self._addresses(scratch, starts)
        out = torch.empty((N, H), dtype=torch.float16, device=h.device)
        self._call(self.lib.sy_experts_routed, h.data_ptr(), N, E, k, gate_up.data_ptr(), down.data_ptr(), H, I,
                   int(bool(mfma_tiles)), idx.data_ptr(), w.data_ptr(), *where[:7], out.data_ptr(),
                   where[7] if need else None, need, _stream())
        return out

    @staticmethod
    def _addresses(scratch, starts):
        base = scratch.data_ptr()
        return tuple(base + s for s in starts)

    def _enqueue_experts(self, h, router, logits, gate_up, down, N, H, E, I, k, norm, mfma_tiles, one_launch_front, scratch,
                         where, need, stream):
        lib = self.lib
        front_done = router is not None and N <= 64 and E <= 128 and 1 <= k <= 8 and k <= E
        # at most 64 choices on the weight-stream kernels: the front only routes, and the first
        # projection sorts for itself (sy_experts_routed)
        routed_only = front_done and not mfma_tiles and N * k <= 64 and H <= 4096
        if front_done:
            # the front of the layer (logits and route, or logits, route and sort: one launch) is
            # enqueued at once: the GPU works on it while the host checks the weights, allocates
            # the result and marshals the long call (a call that is waited for starts its first
            # kernel sooner; in a stream of calls nothing changes)
            if routed_only:
                rc = lib.sy_router_route(h.data_ptr(), router.data_ptr(), N, H, E, k, norm, where[10], where[0], where[1],
                                         stream)
            else:
                rc = lib.sy_router_route_sort(h.data_ptr(), router.data_ptr(), N, H, E, k, norm, where[10], *where[:7],
                                              stream)
            if rc:
                raise RuntimeError(lib.sy_last_error().decode())
        _check(gate_up, "gate_up", torch.float16)
        _check(down, "down", torch.float16)
        if tuple(gate_up.shape) != (E, 2 * I, H) or tuple(down.shape) != (E, H, I):
            raise RuntimeError("moe_experts: shapes of h / gate_up / down do not match")
        out = torch.empty((N, H), dtype=torch.float16, device=h.device)
        if routed_only:
            self._call(lib.sy_experts_routed, h.data_ptr(), N, E, k, gate_up.data_ptr(), down.data_ptr(), H, I, 0,
                       *where[:9], out.data_ptr(), None, 0, stream)
            return out
        if front_done:
            self._call(lib.sy_experts_sorted, h.data_ptr(), N, E, k, gate_up.data_ptr(), down.data_ptr(), H, I,
                       int(bool(mfma_tiles)), where[0], where[1], where[3], where[4], where[5], where[6], where[7], where[8],
                       out.data_ptr(), stream)
            return out
        router_ptr = router.data_ptr() if router is not None else None
        if router is not None and N <= 64:
            self._call(lib.sy_router_logits, h.data_ptr(), router_ptr, N, H, E, where[10], stream)
            router_ptr = None
        self._call(lib.sy_moe_experts, h.data_ptr(), router_ptr, logits.data_ptr() if logits is not None else where[10],
                   N, E, k, norm, gate_up.data_ptr(), down.data_ptr(), H, I, int(bool(mfma_tiles)),
                   int(bool(one_launch_front)), *where[:9], out.data_ptr(), where[9] if need else None, need, stream)
        return out

    @staticmethod
    def router_route_ok(N, H, E, k):
        """Whether router_route (and moe_experts with a router, above 64 tokens) takes this shape."""
        return N >= 1 and H >= 512 and H % 512 == 0 and E <= 128 and 1 <= k <= 8 and k <= E and N * H * 2 < 2 ** 31

    def router_route(self, h, router, k, norm):
        """h [N, H], router [E, H] -> (idx int32 [N, k], w f16 [N, k], logits f16 [N, E]): the
        router GEMM and route in one launch (H a multiple of 512, at most 128 experts, top-8)."""
        _check(h, "h", torch.float16)
        _check(router, "router", torch.float16)
        N, H = h.shape
        E = router.shape[0]
        if router.shape[1] != H:
            raise RuntimeError("router_route: h and router must have the same width")
        logits = torch.empty((N, E), dtype=torch.float16, device=h.device)
        idx = torch.empty((N, int(k)), dtype=torch.int32, device=h.device)
        w = torch.empty((N, int(k)), dtype=torch.float16, device=h.device)
        self._call(self.lib.sy_router_route, h.data_ptr(), router.data_ptr(), N, H, E, int(k), int(bool(norm)),
                   logits.data_ptr(), idx.data_ptr(), w.data_ptr(), _stream())
        return idx, w, logits

    def router_route_sort(self, h, router, k, norm):
        """h [N, H], router [E, H] -> [logits f16 [N, E], idx [N, k], w [N, k], counts [E], offsets
        [E+1], token [M], wsorted [M], pos_of [M]]: router_logits, route and sort_by_expert in one
        launch, for a decode step (at most 256 tokens, 128 experts, top-8)."""
        _check(h, "h", torch.float16)
        _check(router, "router", torch.float16)
        N, H = h.shape
        E, k = router.shape[0], int(k)
        if router.shape[1] != H:
            raise RuntimeError("router_route_sort: h and router must have the same width")
        dev, M = h.device, N * k
        i32 = dict(dtype=torch.int32, device=dev)
        f16 = dict(dtype=torch.float16, device=dev)
        logits, idx, w = torch.empty((N, E), **f16), torch.empty((N, k), **i32), torch.empty((N, k), **f16)
        counts, offsets = torch.empty(E, **i32), torch.empty(E + 1, **i32)
        token, wsorted, pos_of = torch.empty(M, **i32), torch.empty(M, **f16), torch.empty(M, **i32)
        self._call(self.lib.sy_router_route_sort, h.data_ptr(), router.data_ptr(), N, H, E, k, int(bool(norm)),
                   logits.data_ptr(), idx.data_ptr(), w.data_ptr(), counts.data_ptr(), offsets.data_ptr(),
                   token.data_ptr(), wsorted.data_ptr(), pos_of.data_ptr(), _stream())
        return [logits, idx, w, counts, offsets, token, wsorted, pos_of]

    def router_logits(self, h, router):
        """h [N, H] @ router [E, H]^T -> logits [N, E] f16 by the library's own kernel (tens of rows)."""
        _check(h, "h", torch.float16)
        _check(router, "router", torch.float16)
        if h.shape[1] != router.shape[1]:
            raise RuntimeError("router_logits: h and router must have the same width")
        logits = torch.empty((h.shape[0], router.shape[0]), dtype=torch.float16, device=h.device)
        self._call(self.lib.sy_router_logits, h.data_ptr(), router.data_ptr(), h.shape[0], h.shape[1], router.shape[0],
                   logits.data_ptr(), _stream())
        return logits

    # ---- the decode-step kernels around the MoE layer (include/switchyard_decode.h)
    def add_rmsnorm(self, x, delta, weight, eps, x_out=None, router=None, front=None):
        """x [N, H] (+ delta [N, H] or None) -> (x + delta, weight * rmsnorm(x + delta)).
        With delta None the first result is x itself; x_out may be x for an update in place.
        With `router` [E, H] a third result is the logits [N, E] of the normalised rows; with
        front = (top_k, norm_topk_prob) as well (at most 256 rows, 128 experts, top-8) the launch
        also routes and sorts, and route_sort's seven results follow the logits."""
        _check(x, "x", torch.float16)
        _check(weight, "weight", torch.float16)
        N, H = x.shape
        if weight.numel() != H:
            raise RuntimeError("add_rmsnorm: weight must have H entries")
        if delta is not None:
            _check(delta, "delta", torch.float16)
            if delta.shape != x.shape:
                raise RuntimeError("add_rmsnorm: delta must have x's shape")
            if x_out is None:
                x_out = torch.empty_like(x)
            _check(x_out, "x_out", torch.float16)
            if x_out.shape != x.shape:
                raise RuntimeError("add_rmsnorm: x_out must have x's shape")
        h = torch.empty_like(x)
        d_ptr = delta.data_ptr() if delta is not None else None
        o_ptr = x_out.data_ptr() if delta is not None else None
        first = x_out if delta is not None else x
        if router is None:
            self._call(self.lib.sy_add_rmsnorm, x.data_ptr(), d_ptr, weight.data_ptr(), float(eps), N, H, o_ptr,
                       h.data_ptr(), _stream())
            return first, h
        _check(router, "router", torch.float16)
        if router.dim() != 2 or router.shape[1] != H:
            raise RuntimeError("add_rmsnorm: router must be [E, H]")
        logits = torch.empty((N, router.shape[0]), dtype=torch.float16, device=x.device)
        if front is not None:
            E, k, dev = router.shape[0], int(front[0]), x.device
            M = N * k
            i32 = dict(dtype=torch.int32, device=dev)
            idx, w = torch.empty((N, k), **i32), torch.empty((N, k), dtype=torch.float16, device=dev)
            counts, offsets = torch.empty(E, **i32), torch.empty(E + 1, **i32)
            token, pos_of = torch.empty(M, **i32), torch.empty(M, **i32)
            wsorted = torch.empty(M, dtype=torch.float16, device=dev)
            self._call(self.lib.sy_add_rmsnorm_route_sort, x.data_ptr(), d_ptr, weight.data_ptr(), float(eps),
                       router.data_ptr(), E, N, H, k, int(bool(front[1])), o_ptr, h.data_ptr(), logits.data_ptr(),
                       idx.data_ptr(), w.data_ptr(), counts.data_ptr(), offsets.data_ptr(), token.data_ptr(),
                       wsorted.data_ptr(), pos_of.data_ptr(), _stream())
            return first, h, logits, idx, w, counts, offsets, token, wsorted, pos_of
        self._call(self.lib.sy_add_rmsnorm_logits, x.data_ptr(), d_ptr, weight.data_ptr(), float(eps), router.data_ptr(),
                   router.shape[0], N, H, o_ptr, h.data_ptr(), logits.data_ptr(), _stream())
        return first, h, logits

    def embed_rmsnorm(self, tokens, embed, weight, eps):
        """tokens int64 [N] -> (embed[tokens], weight * rmsnorm(embed[tokens])) in one launch."""
        _check(tokens, "tokens", torch.int64)
        _check(embed, "embed", torch.float16)
        _check(weight, "weight", torch.float16)
        N, (vocab, H) = tokens.numel(), embed.shape
        if weight.numel() != H:
            raise RuntimeError("embed_rmsnorm: weight must have H entries")
        x = torch.empty((N, H), dtype=torch.float16, device=embed.device)
        h = torch.empty_like(x)
        self._call(self.lib.sy_embed_rmsnorm, tokens.data_ptr(), embed.data_ptr(), vocab, weight.data_ptr(), float(eps), N,
                   H, x.data_ptr(), h.data_ptr(), _stream())
        return x, h

    def greedy_advance(self, logits, tok, out, base_position, next_position, slot):
        """The end of a greedy step, in place: tok[b] = argmax(logits[b]) (lowest index among equal
        maxima), out[b, next_position[b] - base_position[b]] = tok[b], next_position += 1, slot += 1."""
        _check(logits, "logits", torch.float16)
        for t, name in ((tok, "tok"), (out, "out"), (base_position, "base_position"), (next_position, "next_position"),
                        (slot, "slot")):
            _check(t, name, torch.int64)
        B, V = logits.shape
        if tok.numel() != B or out.dim() != 2 or out.shape[0] != B or base_position.numel() != B or \
                next_position.numel() != B or slot.numel() != 1:
            raise RuntimeError("greedy_advance: tok / out / positions must have one entry (row) per row of logits")
        self._call(self.lib.sy_greedy_advance, logits.data_ptr(), B, V, tok.data_ptr(), out.data_ptr(), out.shape[1],
                   base_position.data_ptr(), next_position.data_ptr(), slot.data_ptr(), _stream())

    def combine_add_rmsnorm(self, y, pos_of, idx, x, weight, eps, x_out=None, w=None):
        """combine(y, pos_of, idx) added to x [N, H] and normalised in one launch ->
        (x + combine, weight * rmsnorm(x + combine)); x_out may be x. With w [N, k] (route's
        weights) y holds the down projection's rows before the router weight, which is applied
        here: the same bits as rows scaled where they were computed."""
        _check(y, "y", torch.float16)
        _check(pos_of, "pos_of", torch.int32)
        _check(idx, "idx", torch.int32)
        _check(x, "x", torch.float16)
        _check(weight, "weight", torch.float16)
        N, H = x.shape
        k = idx.shape[1]
        if y.shape[1] != H or weight.numel() != H or pos_of.numel() < N * k or idx.shape[0] < N:
            raise RuntimeError("combine_add_rmsnorm: shapes of y / pos_of / idx / weight do not match x")
        if x_out is None:
            x_out = torch.empty_like(x)
        _check(x_out, "x_out", torch.float16)
        h = torch.empty_like(x)
        if w is not None:
            _check(w, "w", torch.float16)
            if w.numel() < N * k:
                raise RuntimeError("combine_add_rmsnorm: w shorter than N * k")
        self._call(self.lib.sy_combine_add_rmsnorm, y.data_ptr(), pos_of.data_ptr(), idx.data_ptr(),
                   w.data_ptr() if w is not None else None, k, x.data_ptr(),
                   weight.data_ptr(), float(eps), N, H, x_out.data_ptr(), h.data_ptr(), _stream())
        return x_out, h

    def qk_norm_rope_cache(self, qkv, q_norm, k_norm, eps, clip, cos, sin, positions, slot, heads, kv_heads, head_dim,
                           kcache, vcache):
        """qkv [B*T, (heads + 2 kv_heads) D] (T tokens per sequence, T = rows / batch of the caches)
        -> q [B*T, heads D] normed and rotated; the new keys and values go into kcache / vcache
        [B, kv_heads, capacity, D] from the device-held `slot` on."""
        for t, name in ((qkv, "qkv"), (q_norm, "q_norm"), (k_norm, "k_norm"), (cos, "cos"), (sin, "sin"),
                        (kcache, "kcache"), (vcache, "vcache")):
            _check(t, name, torch.float16)
        _check(positions, "positions", torch.int64)
        _check(slot, "slot", torch.int64)
        rows, D = qkv.shape[0], int(head_dim)
        if qkv.shape[1] != (heads + 2 * kv_heads) * D or q_norm.numel() != heads * D or k_norm.numel() != kv_heads * D:
            raise RuntimeError("qk_norm_rope_cache: qkv / q_norm / k_norm do not match heads, kv_heads and head_dim")
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != D:
            raise RuntimeError("qk_norm_rope_cache: cos and sin must be [max_positions, head_dim]")
        if kcache.shape != vcache.shape or kcache.dim() != 4 or kcache.shape[1] != kv_heads or kcache.shape[3] != D:
            raise RuntimeError("qk_norm_rope_cache: caches must be [B, kv_heads, capacity, head_dim]")
        B = kcache.shape[0]
        if B == 0 or rows % B or positions.numel() != rows or slot.numel() != 1:
            raise RuntimeError("qk_norm_rope_cache: qkv needs T rows per sequence of the caches, positions one entry "
                               "per row, slot one entry")
        q = torch.empty((rows, heads * D), dtype=torch.float16, device=qkv.device)
        self._call(self.lib.sy_qk_norm_rope_cache, qkv.data_ptr(), q_norm.data_ptr(), k_norm.data_ptr(), float(eps),
                   float(clip or 0.0), cos.data_ptr(), sin.data_ptr(), cos.shape[0], positions.data_ptr(),
                   slot.data_ptr(), B, rows // B, int(heads), int(kv_heads), D, kcache.shape[2], q.data_ptr(),
                   kcache.data_ptr(), vcache.data_ptr(), _stream())
        return q

    def decode_attention(self, q, kcache, vcache, real, slot, heads):
        """q [B, heads D] against kcache / vcache [B, kv_heads, capacity, D], keys 0..slot that
        `real` [B, capacity] (bool) marks -> [B, heads D]."""
        _check(q, "q", torch.float16)
        _check(kcache, "kcache", torch.float16)
        _check(vcache, "vcache", torch.float16)
        _check(real, "real", torch.bool)
        _check(slot, "slot", torch.int64)
        B, kv_heads, capacity, D = kcache.shape
        if vcache.shape != kcache.shape or tuple(q.shape) != (B, heads * D) or tuple(real.shape) != (B, capacity) or \
                slot.numel() != 1:
            raise RuntimeError("decode_attention: shapes of q / caches / real / slot do not match")
        out = torch.empty_like(q)
        self._call(self.lib.sy_decode_attention, q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), real.data_ptr(),
                   slot.data_ptr(), B, int(heads), kv_heads, D, capacity, out.data_ptr(), _stream())
        return out

    def decode_attention_qkv(self, qkv, q_norm, k_norm, eps, clip, cos, sin, positions, slot, real, heads, kv_heads,
                             head_dim, kcache, vcache):
        """qk_norm_rope_cache and decode_attention in one launch: qkv [B, (heads + 2 kv_heads) D]
        -> attention output [B, heads D]; the new key and value are written at `slot`, and
        real[:, slot] is set (the new token is a real one)."""
        for t, name in ((qkv, "qkv"), (q_norm, "q_norm"), (k_norm, "k_norm"), (cos, "cos"), (sin, "sin"),
                        (kcache, "kcache"), (vcache, "vcache")):
            _check(t, name, torch.float16)
        _check(positions, "positions", torch.int64)
        _check(slot, "slot", torch.int64)
        _check(real, "real", torch.bool)
        B, D = qkv.shape[0], int(head_dim)
        if qkv.shape[1] != (heads + 2 * kv_heads) * D or q_norm.numel() != heads * D or k_norm.numel() != kv_heads * D:
            raise RuntimeError("decode_attention_qkv: qkv / q_norm / k_norm do not match heads, kv_heads and head_dim")
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != D:
            raise RuntimeError("decode_attention_qkv: cos and sin must be [max_positions, head_dim]")
        if kcache.shape != vcache.shape or kcache.dim() != 4 or tuple(kcache.shape[:2]) != (B, kv_heads) or \
                kcache.shape[3] != D:
            raise RuntimeError("decode_attention_qkv: caches must be [B, kv_heads, capacity, head_dim]")
        capacity = kcache.shape[2]
        if positions.numel() != B or slot.numel() != 1 or tuple(real.shape) != (B, capacity):
            raise RuntimeError("decode_attention_qkv: positions [B], slot [1], real [B, capacity]")
        out = torch.empty((B, heads * D), dtype=torch.float16, device=qkv.device)
        self._call(self.lib.sy_decode_attention_qkv, qkv.data_ptr(), q_norm.data_ptr(), k_norm.data_ptr(), float(eps),
                   float(clip or 0.0), cos.data_ptr(), sin.data_ptr(), cos.shape[0], positions.data_ptr(),
                   slot.data_ptr(), real.data_ptr(), B, int(heads), int(kv_heads), D, capacity, kcache.data_ptr(),
                   vcache.data_ptr(), out.data_ptr(), _stream())
        return out
